"""GPU parity for the integer side of the verify step and for the rollback caches:
acceptance length, commit bookkeeping, conv-window rebuild, KV append, and a full
arm -> forward -> record -> rollback cycle against the oracle's state machine.
Integer results are bit-exact; copied bytes are bit-exact; the replayed state is
held to rtol 1e-4."""

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

STATE_TOL = dict(rtol=1e-4, atol=1e-6)


def dev(a, dt=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dt)


def host(t):
    return t.detach().float().cpu().numpy()


def test_match_acceptance_length_bit_exact(gpu_lib):
    from swiftlm_amd import DFlashRuntime as R

    # the reference's documented example (DFlashRuntime.swift:130-132)
    got = R.match_acceptance_length(torch.tensor([1, 2, 3], device="cuda"), torch.tensor([1, 2, 5], device="cuda"))
    assert got.dtype == torch.int32 and int(got) == 2
    assert int(R.match_acceptance_length(torch.empty(0, dtype=torch.int64, device="cuda"),
                                         torch.empty(0, dtype=torch.int64, device="cuda"))) == 0
    rng = np.random.default_rng(0)
    for n in [1, 2, 15, 16, 63, 64, 65, 200]:
        for _ in range(6):
            a = rng.integers(0, 3, n)
            b = a.copy()
            if rng.random() < 0.8:
                b[rng.integers(0, n):] = rng.integers(0, 3)
            got = int(R.match_acceptance_length(torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()))
            assert got == O.match_acceptance_length(a, b)
    # token ids above 2^31 compare as 32-bit patterns
    big = torch.tensor([4000000000, 7], device="cuda")
    assert int(R.match_acceptance_length(big, big.clone())) == 2


def test_accept_commit_bit_exact(gpu_lib):
    from swiftlm_amd import DFlashRuntime as R

    rng = np.random.default_rng(1)
    for _ in range(60):
        V = int(rng.integers(1, 17))
        staged = int(rng.integers(0, 50000))
        drafted = rng.integers(0, 3, V - 1)
        posterior = rng.integers(0, 3, V)
        if V > 1 and rng.random() < 0.5:
            posterior[: V - 1] = drafted                      # fully accepted
        start = int(rng.integers(0, 100000))
        verify_ids = torch.tensor([staged] + list(drafted), device="cuda")
        r = R.accept_commit(verify_ids, torch.from_numpy(posterior).cuda(), start)
        w = O.accept_commit(staged, drafted, posterior, start)
        assert (r.acceptance_len, r.commit_count, r.staged_first_next, r.start) == (
            w["acceptance_len"], w["commit_count"], w["staged_next"], w["start"])


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
def test_rebuild_conv_state_bit_exact(gpu_lib, dt):
    import ctypes as C

    from swiftlm_amd import _lib

    B, keep, T, Cc = 2, 3, 16, 8192                           # Qwen3-Next conv width 2*Hk*Dk + Hv*Dv
    rng = np.random.default_rng(2)
    snap = dev(rng.standard_normal((B, keep, Cc)).astype(np.float32), dt)
    qkv = dev(rng.standard_normal((B, T, Cc)).astype(np.float32), dt)
    lib = _lib.load()
    for steps in [1, 2, 3, 4, 9, 16]:
        out = torch.full((B, keep, Cc), 9.0, dtype=dt, device="cuda")
        rc = lib.dflash_rebuild_conv_state(None, C.c_void_p(snap.data_ptr()), C.c_void_p(qkv.data_ptr()),
                                           C.c_void_p(out.data_ptr()), B, keep, T, Cc, snap.element_size(), steps, None)
        assert rc == 0, _lib.last_error()
        want = O.rebuild_conv_state(host(snap), host(qkv), steps, keep)
        assert np.array_equal(host(out), want), steps
    # missing snapshot counts as zeros; step count read on the device
    sd = torch.tensor([2], dtype=torch.int32, device="cuda")
    out = torch.full((B, keep, Cc), 9.0, dtype=dt, device="cuda")
    rc = lib.dflash_rebuild_conv_state(None, None, C.c_void_p(qkv.data_ptr()), C.c_void_p(out.data_ptr()), B, keep, T,
                                       Cc, snap.element_size(), 0, C.c_void_p(sd.data_ptr()))
    assert rc == 0
    assert np.array_equal(host(out), O.rebuild_conv_state(None, host(qkv), 2, keep))


def test_kv_append_bit_exact(gpu_lib):
    import ctypes as C

    from swiftlm_amd import _lib

    B, Hk, M, D, cap = 2, 2, 16, 256, 300
    g = torch.Generator(device="cuda").manual_seed(3)
    kc = torch.randn(B, Hk, cap, D, generator=g, device="cuda").bfloat16()
    vc = torch.randn(B, Hk, cap, D, generator=g, device="cuda").bfloat16()
    kn = torch.randn(B, Hk, M, D, generator=g, device="cuda").bfloat16()
    vn = torch.randn(B, Hk, M, D, generator=g, device="cuda").bfloat16()
    k0, v0 = kc.clone(), vc.clone()
    lib = _lib.load()
    p = lambda t: C.c_void_p(t.data_ptr())
    assert lib.dflash_kv_append(None, p(kc), p(vc), p(kn), p(vn), B, Hk, M, D, 2, Hk * cap * D, cap * D, 100, None,
                                cap, None) == 0
    k0[:, :, 100:116] = kn
    v0[:, :, 100:116] = vn
    assert torch.equal(kc, k0) and torch.equal(vc, v0)
    # offset on the device
    od = torch.tensor([250], dtype=torch.int32, device="cuda")
    nl = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.dflash_kv_append(None, p(kc), p(vc), p(kn), p(vn), B, Hk, M, D, 2, Hk * cap * D, cap * D, 0, p(od),
                                cap, p(nl)) == 0
    k0[:, :, 250:266] = kn
    assert torch.equal(kc, k0) and int(nl) == 266
    # rows outside the capacity are refused on the host
    assert lib.dflash_kv_append(None, p(kc), p(vc), p(kn), p(vn), B, Hk, M, D, 2, Hk * cap * D, cap * D, 290, None,
                                cap, None) == _lib.INVALID


def _forward_into_cache(cache, d, qkv, K):
    q, k, v, g, beta = (dev(d[n], torch.bfloat16) for n in ("q", "k", "v", "g", "beta"))
    y, s_new, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, cache[1])
    cache[1] = s_new                                           # post-verify state: a new buffer
    cache[0] = qkv[:, -3:].clone()                             # post-verify conv window: its own buffer (for B = 1
                                                               # .contiguous() would hand back a view of qkv)
    cache.record_tape(tape, k, g, qkv)
    return tape


@pytest.mark.parametrize("n_accepted", [0, 3, 14])
def test_recurrent_rollback_cache_cycle(gpu_lib, n_accepted):
    from swiftlm_amd import DFlashKernels as K, RecurrentRollbackCache

    B, T, Hk, Hv, Dk, Dv, Cc = 1, 16, 16, 32, 128, 128, 8192
    d = O.make_gdn_inputs(50, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
    rng = np.random.default_rng(5)
    conv0 = O.round_to_bf16(rng.standard_normal((B, 3, Cc)).astype(np.float32))
    qkv = O.round_to_bf16(rng.standard_normal((B, T, Cc)).astype(np.float32))

    cache = RecurrentRollbackCache()
    cache[0] = dev(conv0, torch.bfloat16)
    cache[1] = dev(d["state"])
    cache.arm_rollback(prefix_len=100)
    assert cache.is_armed
    tape = _forward_into_cache(cache, d, dev(qkv, torch.bfloat16), K)
    cache.rollback(n_accepted)
    torch.cuda.synchronize()
    assert not cache.is_armed

    oc = O.RecurrentRollbackCacheOracle()
    oc.slots = [conv0, d["state"]]
    oc.arm_rollback(100)
    oc.slots = [qkv[:, -3:], None]
    oc.record_tape(host(tape), d["k"], d["g"], qkv)
    oc.slots[1] = d["state"]                                   # any non-nil state; rollback restores the snapshot first
    oc.rollback(n_accepted, dtype=np.float64)
    np.testing.assert_allclose(host(cache[1]), oc.slots[1], **STATE_TOL)
    assert np.array_equal(host(cache[0]), oc.slots[0])         # conv window: bit-exact copy


def test_rollback_refuses_a_conv_window_that_is_a_view_of_qkv(gpu_lib):
    """The rebuilt window is written in place while qkv is read: a window that shares memory with qkv
    is rejected instead of racing."""
    from swiftlm_amd import DFlashKernels as K, DFlashError, RecurrentRollbackCache

    B, T, Hk, Hv, Dk, Dv, Cc = 1, 16, 2, 4, 64, 32, 512
    d = O.make_gdn_inputs(51, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
    cache = RecurrentRollbackCache()
    cache[0] = torch.zeros(B, 3, Cc, dtype=torch.bfloat16, device="cuda")
    cache[1] = dev(d["state"])
    cache.arm_rollback(prefix_len=0)
    qkv = torch.randn(B, T, Cc, device="cuda").bfloat16()
    q, k, v, g, beta = (dev(d[n], torch.bfloat16) for n in ("q", "k", "v", "g", "beta"))
    y, s_new, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, cache[1])
    cache[1] = s_new
    cache[0] = qkv[:, -3:]                                     # a view of the tape's qkv
    cache.record_tape(tape, k, g, qkv)
    with pytest.raises(DFlashError):
        cache.rollback(3)


def test_restore_target_cache_hybrid_stack(gpu_lib):
    """A 4-layer hybrid stack (3 GDN + 1 attention) through HybridGDNEngine: partial
    acceptance replays all tape caches in one launch; full acceptance replays nothing."""
    from swiftlm_amd import (DFlashKernels as K, HybridGDNEngine, KVCacheSimple, MambaCache,
                             RecurrentRollbackCache)

    B, T, Hk, Hv, Dk, Dv, Cc = 1, 16, 16, 32, 128, 128, 8192
    rng = np.random.default_rng(6)
    engine = HybridGDNEngine()
    for acceptance_len in (4, 15):
        caches, ds, qkvs, tapes, conv0s = [], [], [], [], []
        for layer in range(3):
            d = O.make_gdn_inputs(60 + layer, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
            c = RecurrentRollbackCache()
            conv0 = O.round_to_bf16(rng.standard_normal((B, 3, Cc)).astype(np.float32))
            c[0] = dev(conv0, torch.bfloat16)
            c[1] = dev(d["state"])
            caches.append(c); ds.append(d); conv0s.append(conv0)
        kv = KVCacheSimple(); kv.offset = 1000 + T
        plain = MambaCache(); plain.offset = 0
        stack = caches + [kv, plain]
        engine.arm_rollback(stack, prefix_len=1000)
        post_states = []
        for c, d in zip(caches, ds):
            qkv = O.round_to_bf16(rng.standard_normal((B, T, Cc)).astype(np.float32))
            tapes.append(_forward_into_cache(c, d, dev(qkv, torch.bfloat16), K)); qkvs.append(qkv)
            post_states.append(c[1].clone())
        target_len = 1000 + 1 + acceptance_len
        ns = engine.rollback(stack, target_len=target_len, acceptance_length=acceptance_len, drafted_tokens=T - 1)
        torch.cuda.synchronize()
        assert ns >= 0
        assert kv.offset == target_len and plain.offset == target_len
        for c, d, qkv, tape, conv0, post in zip(caches, ds, qkvs, tapes, conv0s, post_states):
            assert not c.is_armed
            if acceptance_len == T - 1:                        # fully accepted: keep the forward's state
                assert torch.equal(c[1], post)
                assert np.array_equal(host(c[0]), qkv[:, -3:])
            else:
                steps = acceptance_len + 1
                want = O.tape_replay_ops(host(tape)[:, :steps], d["k"][:, :steps], d["g"][:, :steps], d["state"],
                                         dtype=np.float64)
                np.testing.assert_allclose(host(c[1]), want, **STATE_TOL)
                assert np.array_equal(host(c[0]), O.rebuild_conv_state(conv0, qkv, steps, 3))


def test_snapshot_cache_restores_pre_verify_state(gpu_lib):
    from swiftlm_amd import MambaSnapshotCache

    c = MambaSnapshotCache()
    conv, state = torch.ones(1, 3, 64, device="cuda"), torch.ones(1, 4, 8, 64, device="cuda")
    c[0], c[1] = conv, state
    c.arm_rollback(0)
    c[0], c[1] = conv * 2, state * 2
    c.rollback(5)
    assert c[0] is conv and c[1] is state and not c.is_armed


# ---- greedy tokens + fused acceptance (DFlashRuntime.swift:118-128, :513-547) ----

@pytest.mark.parametrize("dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("V", [151936, 8192, 1000, 37])
def test_greedy_tokens_with_mask_matches_oracle(gpu_lib, dt, V):
    import torch
    from swiftlm_amd import DFlashRuntime
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}[dt]
    T = 16
    g = torch.Generator(device="cuda").manual_seed(V)
    logits = (4 * torch.randn(T, V, generator=g, device="cuda")).to(tdt)
    ids = [0, 5, V - 1, V + 3, -2] + list(range(10, min(V, 30)))
    # make the unmasked winner of some rows a suppressed token, and plant exact ties
    logits[0, 5] = 100.0
    logits[1, V - 1] = 100.0
    logits[2, 7] = 90.0
    logits[2, V // 2] = 90.0
    logits[3, :] = 1.0
    host_logits = logits.float().cpu().numpy()
    for ids_case in (None, ids):
        mask_o = O.build_suppress_token_mask(V, ids_case)
        mask_d = DFlashRuntime.build_suppress_token_mask(V, ids_case)
        assert (mask_o is None) == (mask_d is None)
        got = DFlashRuntime.greedy_tokens_with_mask(logits, mask_d)
        torch.cuda.synchronize()
        want = O.greedy_tokens_with_mask(host_logits, mask_o, dtype=dt)
        np.testing.assert_array_equal(got.cpu().numpy().astype(np.uint32), want)


def test_greedy_accept_commit_equals_two_steps(gpu_lib):
    """One call = greedyTokensWithMask + matchAcceptanceLength + the commit bookkeeping; repeated
    calls reuse the workspace."""
    import torch
    from swiftlm_amd import DFlashRuntime
    T, V = 16, 151936
    g = torch.Generator(device="cuda").manual_seed(1)
    mask = DFlashRuntime.build_suppress_token_mask(V, [1, 2, 3])
    start = 1000
    for acc in (0, 3, 15, 7):
        logits = torch.randn(T, V, generator=g, device="cuda").bfloat16()
        post = O.greedy_tokens_with_mask(logits.float().cpu().numpy(), O.build_suppress_token_mask(V, [1, 2, 3]), dtype="bf16")
        verify = np.empty(T, np.int64)
        verify[0] = 42
        verify[1:] = post[:-1]
        if acc < T - 1:
            verify[1 + acc] = (int(post[acc]) + 1) % V          # first mismatch at draft position acc
        res, post_d = DFlashRuntime.greedy_accept_commit(logits, mask, torch.from_numpy(verify).cuda(), start)
        want = O.accept_commit(int(verify[0]), verify[1:], post, start)
        np.testing.assert_array_equal(post_d.cpu().numpy().astype(np.uint32), post)
        assert (res.acceptance_len, res.commit_count, res.staged_first_next, res.start) == (
            want["acceptance_len"], want["commit_count"], want["staged_next"], want["start"])
        assert res.acceptance_len == acc
        start = res.start


def test_plain_c_client_of_the_abi(gpu_lib):
    """tests/cabi_c/cabi_check.c, built with gcc as C99 against include/dflash_hip.h: tape replay against
    the recurrence computed on the host in C, the acceptance bookkeeping, and an unsupported shape."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "swiftlm_amd", "lib", "cabi_check")
    assert os.path.exists(exe), "build it with `make -C swiftlm_amd/csrc`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "C ABI check passed" in r.stdout


def test_plain_c_host_drives_whole_verify_steps_through_a_captured_graph(gpu_lib):
    """tests/cabi_c/step_check.c: a 3 GatedDelta + 1 attention stack stepped four times by a C99 host through
    include/dflash_hip.h only -- two steps captured with hipStreamBeginCapture on a fresh stream and launched twice,
    then the same steps eagerly -- with graph == eager byte for byte and states, offsets, accept words, appended rows
    and the attention output checked against values computed on the host in C."""
    import os
    import subprocess
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "swiftlm_amd", "lib", "step_check")
    assert os.path.exists(exe), "build it with `make -C swiftlm_amd/csrc`"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "verify-step check passed" in r.stdout


# ---- the verify-step driver (what bench.py times): fused and unfused acceptance agree, both match the oracle ----

def test_verify_stack_steps_match_oracle_and_fused_accept(gpu_lib):
    import torch
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    cfg = StackConfig(n_layers=8, attn_every=4, block=16, Hk=2, Hv=4, Dk=128, Dv=32, Hq=4, Hkv=2, D=128,
                      context=150, max_steps=6)
    stacks = [HybridVerifyStack(cfg, seed=3), HybridVerifyStack(cfg, seed=3)]
    stacks[0].fuse_accept, stacks[1].fuse_accept = True, False
    commits = [3, 16, 1, 9]
    offset = cfg.context
    for step, cc in enumerate(commits):
        pre = None
        for st in stacks:
            ph = st.phase
            st.set_acceptance(ph, cc, seed=step)
            if pre is None:
                pre = [dict(state=host(l["state"][ph])) for l in st.gdn]
            st.enqueue_step()
        torch.cuda.synchronize()
        offset += cc
        a, b = stacks
        assert a.accept.tolist() == b.accept.tolist() == [cc - 1, cc, int(a.posterior[1 - a.phase][cc - 1]), offset]
        assert int(a.offset) == int(b.offset) == offset
        for la, lb, p0 in zip(a.gdn, b.gdn, pre):
            post = 1 - (1 - a.phase)          # the buffer the step wrote = the new pre-verify state = state[a.phase]
            assert torch.equal(la["state"][a.phase], lb["state"][b.phase])
            assert torch.equal(la["tape"], lb["tape"]) and torch.equal(la["y"], lb["y"])
            # oracle: forward on the block, then (unless everything was accepted) replay of cc steps
            yw, sw, tw = O.gated_delta_ops_with_tape(host(la["q"]), host(la["k"]), host(la["v"]), host(la["g"]),
                                                      host(la["beta"]), p0["state"])
            want = sw if cc == cfg.block else O.tape_replay_ops(tw[:, :cc].astype(np.float32), host(la["k"])[:, :cc],
                                                                host(la["g"])[:, :cc], p0["state"])
            np.testing.assert_allclose(host(la["state"][a.phase]), want, **STATE_TOL)
        for la, lb in zip(a.attn, b.attn):
            assert torch.equal(la["out"], lb["out"])
            n_keys = offset - cc + cfg.block
            ow, _ = O.sdpa_block_causal(host(la["q"]), host(la["k_cache"])[:, :, :n_keys], host(la["v_cache"])[:, :, :n_keys],
                                        a.scale)
            np.testing.assert_allclose(host(la["out"]), ow, rtol=2e-2, atol=2e-2)


def test_verify_stack_without_post_block_state_commits_the_same_states(gpu_lib):
    """The variant in which no forward stores the state after the whole block and the rollback replays the tape also
    for a block accepted whole: bookkeeping and attention identical; tapes, y and committed states identical bit for
    bit until a block is accepted whole (the same replay from the same tape), and to the state's bar from then on (that
    block's state is a replay of 16 steps instead of the forward's own state, and the later steps start from it)."""
    import torch
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    cfg = StackConfig(n_layers=8, attn_every=4, block=16, Hk=2, Hv=4, Dk=128, Dv=32, Hq=4, Hkv=2, D=128,
                      context=150, max_steps=6)
    for fuse in (True, False):
        a, b = HybridVerifyStack(cfg, seed=3), HybridVerifyStack(cfg, seed=3)
        a.fuse_accept = b.fuse_accept = fuse
        b.post_block_state = False
        same_bits = True
        for step, cc in enumerate([3, 16, 1, 16, 9]):
            for st in (a, b):
                st.set_acceptance(st.phase, cc, seed=step)
                if st is b:                                  # nothing may rely on what the buffer held before
                    for l in st.gdn:
                        l["state"][1 - st.phase].fill_(float("nan"))
                st.enqueue_step()
            torch.cuda.synchronize()
            assert a.accept.tolist() == b.accept.tolist() and int(a.offset) == int(b.offset)
            for la, lb in zip(a.gdn, b.gdn):
                sa, sb = la["state"][a.phase], lb["state"][b.phase]
                assert bool(torch.isfinite(sb).all())
                if same_bits:
                    assert torch.equal(la["tape"], lb["tape"]) and torch.equal(la["y"], lb["y"])
                    if cc < cfg.block:
                        assert torch.equal(sa, sb)
                np.testing.assert_allclose(host(lb["tape"]), host(la["tape"]), rtol=1e-4, atol=1e-5)
                np.testing.assert_allclose(host(lb["y"]), host(la["y"]), rtol=2e-2, atol=2e-2)
                np.testing.assert_allclose(host(sb), host(sa), rtol=1e-4, atol=1e-5)
            same_bits = same_bits and cc < cfg.block
            for la, lb in zip(a.attn, b.attn):
                assert torch.equal(la["out"], lb["out"]) and torch.equal(la["lse"], lb["lse"])


def test_verify_stack_paged_equals_dense(gpu_lib):
    """The verify-step driver with paged K/V pools gives the bytes of the dense driver, step after step,
    and the appended rows sit in the pages the table names."""
    import torch
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    kw = dict(n_layers=8, attn_every=4, block=16, Hk=2, Hv=4, Dk=128, Dv=32, Hq=4, Hkv=2, D=128, context=150, max_steps=6)
    dense = HybridVerifyStack(StackConfig(**kw), seed=3)
    paged = HybridVerifyStack(StackConfig(page_size=32, **kw), seed=3)
    offset = kw["context"]
    for step, cc in enumerate([3, 16, 1, 9, 5]):
        for st in (dense, paged):
            st.set_acceptance(st.phase, cc, seed=step)
            st.enqueue_step()
        torch.cuda.synchronize()
        offset += cc
        assert int(dense.offset) == int(paged.offset) == offset
        assert dense.accept.tolist() == paged.accept.tolist()
        for ld, lp in zip(dense.attn, paged.attn):
            assert torch.equal(ld["out"], lp["out"]) and torch.equal(ld["lse"], lp["lse"])
            n_keys = offset - cc + 16                       # rows the step left in the cache (commit or not, all 16 were stored)
            tb = lp["page_table"][0].cpu().numpy()
            gathered = O.gather_pages(host(lp["k_pool"]), tb[None], n_keys)
            assert np.array_equal(gathered, host(ld["k_cache"])[:, :, :n_keys])
        for ld, lp in zip(dense.gdn, paged.gdn):
            assert torch.equal(ld["state"][dense.phase], lp["state"][paged.phase])



def test_device_status_word_reports_out_of_contract_device_lengths(gpu_lib):
    """Lengths read from device memory cannot be checked by the host.  Out of contract they are clamped (or the
    write is skipped) and the registered status word receives a bit per kind; in contract it stays 0."""
    from swiftlm_amd import DFlashKernels as K, _lib
    from swiftlm_amd.dflash_kernels import _ptr, _stream

    lib = _lib.load()
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.dflash_set_status_word(_ptr(status)) == 0
    try:
        B, Hq, Hk, D, cap = 1, 4, 2, 128, 96
        g = torch.Generator(device="cuda").manual_seed(3)
        q = torch.randn(B, Hq, 16, D, generator=g, device="cuda").bfloat16()
        kc = torch.randn(B, Hk, cap, D, generator=g, device="cuda").bfloat16()
        vc = torch.randn(B, Hk, cap, D, generator=g, device="cuda").bfloat16()
        kn = torch.randn(B, Hk, 16, D, generator=g, device="cuda").bfloat16()
        vn = torch.randn(B, Hk, 16, D, generator=g, device="cuda").bfloat16()
        # in contract: 40 cached rows + 16 <= n_keys = 64
        good = torch.tensor([40], dtype=torch.int32, device="cuda")
        K.batched_sdpa_2pass_append(q, kc.clone(), vc.clone(), kn, vn, D ** -0.5, 64, cache_len=good)
        torch.cuda.synchronize()
        assert int(status) == 0
        # out of contract: 60 cached rows + 16 > 64 -> clamped to 64 keys, flagged; rows beyond the bound stay untouched
        bad = torch.tensor([60], dtype=torch.int32, device="cuda")
        kc2, vc2 = kc.clone(), vc.clone()
        out = K.batched_sdpa_2pass_append(q, kc2, vc2, kn, vn, D ** -0.5, 64, cache_len=bad)
        torch.cuda.synchronize()
        assert int(status) == _lib.STATUS_SDPA_LEN
        assert torch.isfinite(out.float()).all()
        assert torch.equal(kc2[:, :, 64:], kc[:, :, 64:]) and torch.equal(vc2[:, :, 64:], vc[:, :, 64:])
        # kv_append past the capacity: nothing written, flagged
        status.zero_()
        off = torch.tensor([cap - 8], dtype=torch.int32, device="cuda")
        kc3 = kc.clone()
        rc = lib.dflash_kv_append(_stream(), _ptr(kc3), _ptr(vc.clone()), _ptr(kn), _ptr(vn), B, Hk, 16, D, 2,
                                  kc3.stride(0), kc3.stride(1), 0, _ptr(off), cap, None)
        assert rc == 0
        torch.cuda.synchronize()
        assert int(status) == _lib.STATUS_APPEND_RANGE and torch.equal(kc3, kc)
        # conv rebuild with a step count beyond the tape
        status.zero_()
        keep, T, C = 3, 4, 64
        snap = torch.randn(B, keep, C, generator=g, device="cuda").bfloat16()
        qkv = torch.randn(B, T, C, generator=g, device="cuda").bfloat16()
        dst = torch.zeros(B, keep, C, dtype=torch.bfloat16, device="cuda")
        steps = torch.tensor([T + 3], dtype=torch.int32, device="cuda")
        assert lib.dflash_rebuild_conv_state(_stream(), _ptr(snap), _ptr(qkv), _ptr(dst), B, keep, T, C, 2, 0, _ptr(steps)) == 0
        torch.cuda.synchronize()
        assert int(status) == _lib.STATUS_CONV_STEPS
    finally:
        lib.dflash_set_status_word(None)
