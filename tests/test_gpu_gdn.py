"""GPU parity: GatedDelta forward-with-tape and tape replay (HIP, through the C ABI)
against the CPU oracle on the same seeded inputs.

Bars: fp32 recurrent state rtol 1e-4 (atol 1e-6 for entries
near zero); bf16/f16 outputs 2e-2 abs/rel; the fp32 tape is held to the state's bar.
"""

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

TORCH_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}
STATE_TOL = dict(rtol=1e-4, atol=1e-6)
LOWP_TOL = dict(rtol=2e-2, atol=2e-2)


def dev(a, dt="f32"):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", TORCH_DT[dt])


def host(t):
    return t.detach().float().cpu().numpy()


def make_mask(seed, B, T):
    rng = np.random.default_rng(seed)
    m = (rng.random((B, T)) < 0.6).astype(np.float32)
    m[:, 0] = 1.0
    return m


def run_forward(K, d, in_dt, state_dt, mask=None, mask_dt="f32"):
    args = [dev(d[n], in_dt) for n in ("q", "k", "v", "g", "beta")]
    state = dev(d["state"], state_dt)
    m = None if mask is None else (torch.from_numpy(mask).to("cuda").to(torch.uint8) if mask_dt == "u8"
                                   else dev(mask, mask_dt))
    y, s, tape = K.gated_delta_kernel_with_tape(*args, state, m)
    torch.cuda.synchronize()
    return y, s, tape


# (name, B, T, Hk, Hv, Dk, Dv)
SHAPES = [
    ("cfg0", 1, 8, 4, 8, 64, 64),
    ("cfg1", 1, 16, 16, 32, 128, 128),
    ("ragged_dv", 2, 5, 2, 6, 128, 40),
    ("dk32", 1, 7, 2, 4, 32, 24),
    ("dk256", 1, 6, 1, 2, 256, 64),
    ("dk96", 1, 9, 2, 4, 96, 40),        # DK/4 = 24 threads per row does not divide the workgroup
    ("dk160", 2, 5, 1, 3, 160, 16),
    ("dk192", 1, 18, 2, 2, 192, 48),
    ("dk224", 1, 4, 1, 2, 224, 24),
    ("long_T", 1, 40, 2, 4, 64, 32),
]


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
@pytest.mark.parametrize("in_dt", ["f32", "bf16"])
def test_forward_matches_oracle(gpu_lib, shape, vec, in_dt):
    from swiftlm_amd import DFlashKernels as K

    name, B, T, Hk, Hv, Dk, Dv = shape
    d = O.make_gdn_inputs(100 + len(name), B, T, Hk, Hv, Dk, Dv, in_dtype=in_dt, vec_gate=vec)
    y, s, tape = run_forward(K, d, in_dt, "f32")
    yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], dtype=np.float64)
    assert y.dtype == TORCH_DT[in_dt] and s.dtype == torch.float32 and tape.dtype == torch.float32
    np.testing.assert_allclose(host(s), sw, **STATE_TOL)
    np.testing.assert_allclose(host(tape), tw, rtol=1e-4, atol=1e-5)
    if in_dt == "f32":
        np.testing.assert_allclose(host(y), yw, rtol=1e-4, atol=1e-5)
    else:
        np.testing.assert_allclose(host(y), yw, **LOWP_TOL)


@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
@pytest.mark.parametrize("mask_dt", ["f32", "bf16", "u8"])
def test_forward_masked(gpu_lib, vec, mask_dt):
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 2, 12, 2, 4, 128, 48
    d = O.make_gdn_inputs(7, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16", vec_gate=vec)
    mask = make_mask(8, B, T)
    y, s, tape = run_forward(K, d, "bf16", "f32", mask, mask_dt)
    yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask,
                                             dtype=np.float64)
    np.testing.assert_allclose(host(s), sw, **STATE_TOL)
    np.testing.assert_allclose(host(tape), tw, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(host(y), yw, **LOWP_TOL)
    off = mask < 0.5
    assert np.all(host(y)[off] == 0) and np.all(host(tape)[off] == 0)     # exact zeros on masked steps


@pytest.mark.parametrize("dt", ["bf16", "f16"])
def test_forward_low_precision_state_requantises_each_step(gpu_lib, dt):
    """State stored in the input type: rounded after every step like the Metal kernel
    (DFlashKernels.swift:183-186)."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 8, 2, 4, 128, 32
    d = O.make_gdn_inputs(9, B, T, Hk, Hv, Dk, Dv, in_dtype=dt)
    d["state"] = O.quantize(d["state"], dt)
    y, s, tape = run_forward(K, d, dt, dt)
    assert s.dtype == TORCH_DT[dt]
    yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], requant=dt)
    np.testing.assert_allclose(host(s), sw, **LOWP_TOL)
    np.testing.assert_allclose(host(y), yw, **LOWP_TOL)
    np.testing.assert_allclose(host(tape), tw, **LOWP_TOL)


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
def test_replay_matches_oracle_for_every_prefix(gpu_lib, shape, vec):
    from swiftlm_amd import DFlashKernels as K

    name, B, T, Hk, Hv, Dk, Dv = shape
    in_dt = "f32" if name == "cfg0" else "bf16"
    d = O.make_gdn_inputs(200 + len(name), B, T, Hk, Hv, Dk, Dv, in_dtype=in_dt, vec_gate=vec)
    rng = np.random.default_rng(3)
    tape = rng.standard_normal((B, T, Hv, Dv)).astype(np.float32)
    tape_d, k_d, g_d, s_d = dev(tape), dev(d["k"], in_dt), dev(d["g"], in_dt), dev(d["state"])
    steps = sorted(set([1, 2, T // 2, T - 1, T]) - {0})
    for n in steps:                                    # the caller slices the accepted prefix
        out = K.tape_replay_kernel(tape_d[:, :n], k_d[:, :n], g_d[:, :n], s_d)
        torch.cuda.synchronize()
        want = O.tape_replay_ops(tape[:, :n], d["k"][:, :n], d["g"][:, :n], d["state"], dtype=np.float64)
        np.testing.assert_allclose(host(out), want, **STATE_TOL, err_msg=f"n={n}")
    # T == 0 returns the input state
    out = K.tape_replay_kernel(tape_d[:, :0], k_d[:, :0], g_d[:, :0], s_d)
    assert torch.equal(out, s_d)


def test_replay_masked_and_bf16_tape(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 2, 16, 8, 16, 128, 128        # the reference bench's shape (DFlashKernelBench/main.swift:107)
    d = O.make_gdn_inputs(11, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
    tape = O.round_to_bf16(np.random.default_rng(4).uniform(-0.1, 0.1, (B, T, Hv, Dv)).astype(np.float32))
    mask = make_mask(12, B, T)
    out = K.tape_replay_kernel(dev(tape, "bf16"), dev(d["k"], "bf16"), dev(d["g"], "bf16"), dev(d["state"]),
                               dev(mask, "bf16"))
    want = O.tape_replay_ops(tape, d["k"], d["g"], d["state"], mask, dtype=np.float64)
    np.testing.assert_allclose(host(out), want, **STATE_TOL)
    # all-zero mask: state untouched bit for bit
    out = K.tape_replay_kernel(dev(tape, "bf16"), dev(d["k"], "bf16"), dev(d["g"], "bf16"), dev(d["state"]),
                               dev(np.zeros_like(mask)))
    assert np.array_equal(host(out), d["state"])


def test_replay_low_precision_state(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 8, 8, 16, 128, 128
    rng = np.random.default_rng(5)
    u = lambda *s: O.round_to_bf16(rng.uniform(-0.1, 0.1, s).astype(np.float32))   # DFlashKernelBench inputs (main.swift:28-30)
    tape, k, g, state = u(B, T, Hv, Dv), u(B, T, Hk, Dk), u(B, T, Hv), u(B, Hv, Dv, Dk)
    out = K.tape_replay_kernel(dev(tape, "bf16"), dev(k, "bf16"), dev(g, "bf16"), dev(state, "bf16"))
    assert out.dtype == torch.bfloat16
    want = O.tape_replay_ops(tape, k, g, state, requant="bf16")
    # the reference's own consistency bar for this kernel (tests/DFlash/DFlashProfiler.swift:239)
    a, b = host(out).ravel(), want.ravel()
    assert np.abs(a - b).max() < 0.01
    assert a @ b / (np.linalg.norm(a) * np.linalg.norm(b)) > 0.999
    np.testing.assert_allclose(a, b, **LOWP_TOL)


def test_forward_tape_replays_to_forward_state_at_full_size(gpu_lib):
    """Size-independent property at the Qwen3-Next shape: replaying the recorded tape
    for n steps from the pre-verify state gives the state of a forward over n tokens."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 16, 16, 32, 128, 128
    rng = np.random.default_rng(6)
    for layer in range(4):
        d = O.make_gdn_inputs(1000 + layer, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
        q, k, v, g, beta = (dev(d[n], "bf16") for n in ("q", "k", "v", "g", "beta"))
        s0 = dev(d["state"])
        y, s_full, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
        n = O.draw_accepted(rng, T, "geometric")
        _, s_n, _ = K.gated_delta_kernel_with_tape(q[:, :n].contiguous(), k[:, :n].contiguous(),
                                                   v[:, :n].contiguous(), g[:, :n].contiguous(),
                                                   beta[:, :n].contiguous(), s0)
        rep = K.tape_replay_kernel(tape[:, :n], k[:, :n], g[:, :n], s0)
        np.testing.assert_allclose(host(rep), host(s_n), **STATE_TOL)
        rep_full = K.tape_replay_kernel(tape, k, g, s0)
        np.testing.assert_allclose(host(rep_full), host(s_full), **STATE_TOL)
        assert torch.equal(s0, dev(d["state"]))             # inputs are never written


def test_batched_replay_equals_per_layer_replay(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv, L = 1, 16, 16, 32, 128, 128, 36
    rng = np.random.default_rng(7)
    tapes, ks, gs, sin = [], [], [], []
    for layer in range(L):
        d = O.make_gdn_inputs(2000 + layer, B, T, Hk, Hv, Dk, Dv, in_dtype="bf16")
        tapes.append(dev(rng.standard_normal((B, T, Hv, Dv)).astype(np.float32)))
        ks.append(dev(d["k"], "bf16")); gs.append(dev(d["g"], "bf16")); sin.append(dev(d["state"]))
    for n in (1, 4, 16):
        sout = [torch.full_like(s, float("nan")) for s in sin]
        K.tape_replay_batched(tapes, ks, gs, sin, sout, steps=n)
        torch.cuda.synchronize()
        for layer in (0, 17, 35):
            one = K.tape_replay_kernel(tapes[layer][:, :n], ks[layer][:, :n], gs[layer][:, :n], sin[layer])
            assert torch.equal(sout[layer], one), f"layer {layer} n={n}"
        want = O.tape_replay_ops(host(tapes[5])[:, :n], host(ks[5])[:, :n], host(gs[5])[:, :n], host(sin[5]),
                                 dtype=np.float64)
        np.testing.assert_allclose(host(sout[5]), want, **STATE_TOL)
    # step count read on the device; a fully accepted block leaves state_out alone
    steps_dev = torch.tensor([3], dtype=torch.int32, device="cuda")
    sout = [torch.zeros_like(s) for s in sin]
    K.tape_replay_batched(tapes, ks, gs, sin, sout, steps=0, steps_dev=steps_dev, skip_if_full=True)
    assert torch.equal(sout[9], K.tape_replay_kernel(tapes[9][:, :3], ks[9][:, :3], gs[9][:, :3], sin[9]))
    steps_dev.fill_(T)
    marker = [torch.full_like(s, 7.0) for s in sin]
    K.tape_replay_batched(tapes, ks, gs, sin, marker, steps=0, steps_dev=steps_dev, skip_if_full=True)
    torch.cuda.synchronize()
    assert all(bool((m == 7.0).all()) for m in marker)


@pytest.mark.parametrize("shape", [("cfg1", 1, 16, 16, 32, 128, 128), ("cfg0", 1, 8, 4, 8, 64, 64), ("dk256", 1, 6, 1, 2, 256, 64),
                                   ("long_T", 1, 40, 2, 4, 64, 32)], ids=lambda s: s[0])
@pytest.mark.parametrize("in_dt", ["f32", "bf16"])
def test_forward_without_post_block_state(gpu_lib, shape, in_dt):
    """state_out = NULL: y and the tape are the bits of the ordinary call, no state is written anywhere, and replaying
    the whole tape from the same start gives the state the ordinary call returns (to the state's bar)."""
    from swiftlm_amd import DFlashKernels as K, DFlashUnsupported

    _, B, T, Hk, Hv, Dk, Dv = shape
    d = O.make_gdn_inputs(77, B, T, Hk, Hv, Dk, Dv, in_dtype=in_dt)
    q, k, v, g, beta = (dev(d[n], in_dt) for n in ("q", "k", "v", "g", "beta"))
    s0 = dev(d["state"])
    keep = s0.clone()
    y1, s1, t1 = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
    y2, s2, t2 = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0, want_state=False)
    torch.cuda.synchronize()
    assert s2 is None
    assert torch.equal(y1, y2) and torch.equal(t1, t2)
    assert torch.equal(s0, keep)
    rep = K.tape_replay_kernel(t2, k, g, s0)
    np.testing.assert_allclose(host(rep), host(s1), **STATE_TOL)
    # the step-by-step kernel (per-channel gate, low-precision state) always stores its state
    dv = O.make_gdn_inputs(78, 1, 4, 2, 4, 64, 16, vec_gate=True)
    with pytest.raises(DFlashUnsupported):
        K.gated_delta_kernel_with_tape(*(dev(dv[n]) for n in ("q", "k", "v", "g", "beta")), dev(dv["state"]), want_state=False)


def test_unsupported_and_invalid_arguments(gpu_lib):
    from swiftlm_amd import DFlashKernels as K, DFlashError, DFlashUnsupported

    d = O.make_gdn_inputs(1, 1, 4, 2, 4, 48, 16)           # Dk = 48: the reference takes its ops path (:271-273)
    with pytest.raises(DFlashUnsupported):
        K.tape_replay_kernel(dev(d["v"][..., :16]), dev(d["k"]), dev(d["g"]), dev(d["state"]))
    d = O.make_gdn_inputs(1, 1, 4, 3, 4, 64, 16)           # Hv % Hk != 0
    with pytest.raises(DFlashError):
        K.gated_delta_kernel_with_tape(*(dev(d[n]) for n in ("q", "k", "v", "g", "beta")), dev(d["state"]))
    with pytest.raises(DFlashError):                        # CPU tensors: there is no CPU path
        K.tape_replay_kernel(torch.zeros(1, 1, 4, 16), torch.zeros(1, 1, 2, 64), torch.zeros(1, 1, 4),
                             torch.zeros(1, 4, 16, 64))


# ---- pre-ops: conv + SiLU, q/k normalisation, gates (KimiLinearDFlash.swift:274-293, :362-363, :390-391) ----

def _prep_inputs(seed, B, T, Hk, Hv, Dk, Dv, K, vec):
    rng = np.random.default_rng(seed)
    C = 2 * Hk * Dk + Hv * Dv
    return dict(
        x=rng.standard_normal((B, T, C)).astype(np.float32),
        state=rng.standard_normal((B, K - 1, C)).astype(np.float32),
        w=(rng.standard_normal((C, K)) * 0.5).astype(np.float32),
        a=(rng.standard_normal((B, T, Hv, Dk) if vec else (B, T, Hv)) * 2).astype(np.float32),
        b=(rng.standard_normal((B, T, Hv)) * 2).astype(np.float32),
        a_log=(rng.standard_normal(Hv) * 0.5).astype(np.float32),
        dt_bias=rng.standard_normal((Hv, Dk) if vec else Hv).astype(np.float32),
    )


@pytest.mark.parametrize("cfg", [(1, 16, 16, 32, 128, 128, 4), (2, 5, 2, 4, 64, 96, 4), (1, 2, 1, 2, 32, 32, 4),
                                 (1, 7, 2, 2, 128, 128, 2)],
                         ids=["qwen3next_block", "ragged_dims", "T_shorter_than_window", "K2"])
@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
@pytest.mark.parametrize("in_dt", ["f32", "bf16"])
def test_gdn_prepare_matches_oracle(gpu_lib, cfg, vec, in_dt):
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv, Kc = cfg
    if vec and Hk != Hv and False:
        pytest.skip()
    d = _prep_inputs(B * 100 + T, B, T, Hk, Hv, Dk, Dv, Kc, vec)
    # the oracle sees exactly the values the device sees
    rd = (lambda a: O.round_to_bf16(a)) if in_dt == "bf16" else (lambda a: a)
    dd = {k: (rd(v) if k not in ("a_log", "dt_bias") else v) for k, v in d.items()}
    want = O.gdn_prepare(dd["x"], dd["state"], dd["w"], dd["a"], dd["b"], dd["a_log"], dd["dt_bias"], Hk, Hv, Dk, Dv,
                         q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    got = K.gdn_prepare(dev(dd["x"], in_dt), dev(dd["state"], in_dt), dev(dd["w"], in_dt), dev(dd["a"], in_dt),
                        dev(dd["b"], in_dt), dev(d["a_log"]), dev(d["dt_bias"]), Hk, Hv, Dk, Dv,
                        q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    torch.cuda.synchronize()
    tol = dict(rtol=2e-5, atol=2e-6) if in_dt == "f32" else LOWP_TOL
    for name, g in zip(("q", "k", "v", "g", "beta"), got[:5]):
        np.testing.assert_allclose(host(g), want[name], err_msg=name, **tol)
    np.testing.assert_array_equal(host(got[5]), want["conv_state"].astype(np.float32))      # copied rows: bit-exact
    # no carried window = zeros
    got0 = K.gdn_prepare(dev(dd["x"], in_dt), None, dev(dd["w"], in_dt), dev(dd["a"], in_dt), dev(dd["b"], in_dt),
                         dev(d["a_log"]), dev(d["dt_bias"]), Hk, Hv, Dk, Dv, q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    want0 = O.gdn_prepare(dd["x"], None, dd["w"], dd["a"], dd["b"], dd["a_log"], dd["dt_bias"], Hk, Hv, Dk, Dv,
                          q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    np.testing.assert_allclose(host(got0[2]), want0["v"], **tol)


def test_gdn_prepare_feeds_the_forward_and_the_rollback_window(gpu_lib):
    """pre-ops -> forward with tape -> conv-window rebuild after n accepted steps: the window equals
    what the pre-ops leave after the first n tokens (RecurrentRollbackCache.swift:139-158)."""
    from swiftlm_amd import DFlashKernels as K, _lib
    from swiftlm_amd.dflash_kernels import _ptr, _stream

    B, T, Hk, Hv, Dk, Dv, Kc = 1, 16, 4, 8, 128, 128, 4
    d = _prep_inputs(9, B, T, Hk, Hv, Dk, Dv, Kc, False)
    bf = lambda a: dev(O.round_to_bf16(a), "bf16")
    x, st, w = bf(d["x"]), bf(d["state"]), bf(d["w"])
    q, k, v, g, beta, new_state = K.gdn_prepare(x, st, w, bf(d["a"]), bf(d["b"]), dev(d["a_log"]), dev(d["dt_bias"]),
                                                Hk, Hv, Dk, Dv, q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    s0 = 0.1 * torch.randn(B, Hv, Dv, Dk, device="cuda")
    y, s1, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
    yw, sw, tw = O.gated_delta_ops_with_tape(host(q), host(k), host(v), host(g), host(beta), host(s0))
    np.testing.assert_allclose(host(s1), sw, **STATE_TOL)
    np.testing.assert_allclose(host(y), yw, **LOWP_TOL)
    lib = _lib.load()
    C = x.shape[-1]
    for n in (1, 5, 16):
        out = torch.empty(B, Kc - 1, C, dtype=torch.bfloat16, device="cuda")
        _lib.check(lib.dflash_rebuild_conv_state(_stream(), _ptr(st), _ptr(x), _ptr(out), B, Kc - 1, T, C, 2, n, None),
                   "rebuild")
        again = K.gdn_prepare(x[:, :n], st, w, bf(d["a"])[:, :n], bf(d["b"])[:, :n], dev(d["a_log"]), dev(d["dt_bias"]),
                              Hk, Hv, Dk, Dv, q_scale=1.0 / Dk, k_scale=Dk ** -0.5)[5]
        torch.cuda.synchronize()
        assert torch.equal(out, again)


@pytest.mark.parametrize("kind", ["sigmoid", "silu"])
@pytest.mark.parametrize("in_dt", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("shape", [(1, 16, 32, 128), (2, 3, 5, 40), (1, 2, 2, 200)], ids=["block", "odd", "wide"])
def test_gdn_finish_matches_oracle(gpu_lib, shape, in_dt, kind):
    from swiftlm_amd import DFlashKernels as K

    rng = np.random.default_rng(sum(shape))
    rd = {"f32": lambda a: a, "bf16": O.round_to_bf16, "f16": lambda a: a.astype(np.float16).astype(np.float32)}[in_dt]
    y = rd(rng.standard_normal(shape).astype(np.float32))
    z = rd((rng.standard_normal(shape) * 2).astype(np.float32))
    w = rd((1 + 0.1 * rng.standard_normal(shape[-1])).astype(np.float32))
    got = K.gdn_finish(dev(y, in_dt), dev(z, in_dt), dev(w, in_dt), 1e-6, kind)
    torch.cuda.synchronize()
    tol = dict(rtol=2e-5, atol=2e-6) if in_dt == "f32" else LOWP_TOL
    np.testing.assert_allclose(host(got), O.gdn_finish(y, z, w, 1e-6, kind), **tol)


# ---- one-launch layer: pre-ops inside the forward kernel (KimiLinearDFlash.swift:351-378) ----

@pytest.mark.parametrize("cfg", [(1, 16, 16, 32, 128, 128), (2, 5, 2, 4, 64, 48), (1, 2, 1, 2, 256, 32),
                                 (1, 1, 2, 2, 128, 16), (1, 16, 4, 8, 64, 64), (2, 7, 2, 6, 128, 32)],
                         ids=["qwen3next_block", "short_block_b2", "T_shorter_than_window_dk256", "single_step", "dk64",
                              "three_value_heads_per_key_head_b2"])
@pytest.mark.parametrize("in_dt", ["bf16", "f32", "f16"])
@pytest.mark.parametrize("carry", [True, False], ids=["conv_state", "no_conv_state"])
def test_gdn_layer_equals_prepare_forward_finish_bitwise(gpu_lib, cfg, in_dt, carry):
    """dflash_gdn_layer against the three calls it replaces: every output bit for bit, and the three-call
    result against the oracle (so the equality is not two wrong answers agreeing)."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = cfg
    Kc = 4
    d = _prep_inputs(B * 1000 + T * 10 + Dk, B, T, Hk, Hv, Dk, Dv, Kc, False)
    rd = {"f32": lambda a: a, "bf16": O.round_to_bf16, "f16": lambda a: a.astype(np.float16).astype(np.float32)}[in_dt]
    x, st, w, a, bl = (dev(rd(d[n]), in_dt) for n in ("x", "state", "w", "a", "b"))
    if not carry:
        st = None
    rng = np.random.default_rng(5)
    s0 = dev(0.1 * rng.standard_normal((B, Hv, Dv, Dk)).astype(np.float32))
    z = dev(rd((rng.standard_normal((B, T, Hv, Dv)) * 2).astype(np.float32)), in_dt)
    nw = dev(rd((1 + 0.1 * rng.standard_normal(Dv)).astype(np.float32)), in_dt)
    sc = dict(q_scale=1.0 / Dk, k_scale=Dk ** -0.5)

    q, k, v, g, beta, conv1 = K.gdn_prepare(x, st, w, a, bl, dev(d["a_log"]), dev(d["dt_bias"]), Hk, Hv, Dk, Dv, **sc)
    y, s1, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
    out = K.gdn_finish(y, z, nw, 1e-6, "silu")
    # the gated norm inside the launch (twice with one counter array: the call must leave it zeroed), and as a
    # second launch
    arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
    layer_args = (x, st, w, a, bl, dev(d["a_log"]), dev(d["dt_bias"]), s0, Hk, Hv, Dk, Dv)
    layer_kw = dict(**sc, gate=z, norm_weight=nw, norm_eps=1e-6, gate_kind="silu", want_intermediates=True)
    runs = [K.gdn_layer(*layer_args, **layer_kw, arrivals=arrivals), K.gdn_layer(*layer_args, **layer_kw, arrivals=arrivals),
            K.gdn_layer(*layer_args, **layer_kw, one_launch=False)]
    torch.cuda.synchronize()
    assert not arrivals.any()
    for r in runs:
        for name, want in (("q", q), ("k", k), ("v", v), ("g", g), ("beta", beta), ("conv_state", conv1), ("y", y),
                           ("state", s1), ("tape", tape), ("out", out)):
            assert torch.equal(r[name], want), name
    r = runs[0]
    # without the optional outputs and without a gate: same recurrence results
    r2 = K.gdn_layer(x, st, w, a, bl, dev(d["a_log"]), dev(d["dt_bias"]), s0, Hk, Hv, Dk, Dv, **sc)
    torch.cuda.synchronize()
    assert r2["out"] is None
    for name in ("y", "state", "tape", "k", "g", "conv_state"):
        assert torch.equal(r2[name], r[name]), name
    # and the three calls against the oracle
    want = O.gdn_prepare(host(x), None if st is None else host(st), host(w), host(a), host(bl), d["a_log"], d["dt_bias"],
                         Hk, Hv, Dk, Dv, **sc)
    tol = dict(rtol=2e-5, atol=2e-6) if in_dt == "f32" else LOWP_TOL
    for name in ("q", "k", "v", "g", "beta"):
        np.testing.assert_allclose(host(r[name]), want[name], err_msg=name, **tol)
    yw, sw, tw = O.gated_delta_ops_with_tape(host(q), host(k), host(v), host(g), host(beta), host(s0), dtype=np.float64)
    np.testing.assert_allclose(host(r["state"]), sw, **STATE_TOL)
    np.testing.assert_allclose(host(r["tape"]), tw, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(host(r["y"]), yw, **(dict(rtol=1e-4, atol=1e-5) if in_dt == "f32" else LOWP_TOL))
    np.testing.assert_allclose(host(r["out"]), O.gdn_finish(host(y), host(z), host(nw), 1e-6, "silu"), **tol)


def test_gdn_layer_reports_unsupported_outside_the_verify_block(gpu_lib):
    from swiftlm_amd import DFlashKernels as K
    from swiftlm_amd.dflash_kernels import DFlashUnsupported

    B, Hk, Hv, Dk, Dv = 1, 2, 2, 128, 32
    for T, Kc in ((17, 4), (8, 3)):
        d = _prep_inputs(3, B, T, Hk, Hv, Dk, Dv, Kc, False)
        args = [dev(d[n], "bf16") for n in ("x", "state", "w", "a", "b")] + [dev(d["a_log"]), dev(d["dt_bias"])]
        with pytest.raises(DFlashUnsupported):
            K.gdn_layer(*args, torch.zeros(B, Hv, Dv, Dk, device="cuda"), Hk, Hv, Dk, Dv, q_scale=1.0, k_scale=1.0)


def _layer_case(seed, B, T, Hk, Hv, Dk, Dv, in_dt="bf16"):
    """Device inputs of one layer call plus the three-call result they must reproduce."""
    from swiftlm_amd import DFlashKernels as K

    d = _prep_inputs(seed, B, T, Hk, Hv, Dk, Dv, 4, False)
    rd = {"f32": lambda a: a, "bf16": O.round_to_bf16, "f16": lambda a: a.astype(np.float16).astype(np.float32)}[in_dt]
    x, st, w, a, bl = (dev(rd(d[n]), in_dt) for n in ("x", "state", "w", "a", "b"))
    rng = np.random.default_rng(seed + 1)
    s0 = dev(0.1 * rng.standard_normal((B, Hv, Dv, Dk)).astype(np.float32))
    z = dev(rd((rng.standard_normal((B, T, Hv, Dv)) * 2).astype(np.float32)), in_dt)
    nw = dev(rd((1 + 0.1 * rng.standard_normal(Dv)).astype(np.float32)), in_dt)
    sc = dict(q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    args = (x, st, w, a, bl, dev(d["a_log"]), dev(d["dt_bias"]), s0, Hk, Hv, Dk, Dv)
    kw = dict(**sc, gate=z, norm_weight=nw, norm_eps=1e-6, gate_kind="silu")
    q, k, v, g, beta, conv1 = K.gdn_prepare(x, st, w, a, bl, dev(d["a_log"]), dev(d["dt_bias"]), Hk, Hv, Dk, Dv, **sc)
    y, s1, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
    out = K.gdn_finish(y, z, nw, 1e-6, "silu")
    want = dict(out=out, y=y, state=s1, tape=tape, k=k, g=g, conv_state=conv1)
    return args, kw, want


def _assert_layer_equals(r, want, what=""):
    for name, w in want.items():
        assert torch.equal(r[name], w), f"{name} {what}"


@pytest.mark.parametrize("cfg", [(1, 16, 2, 4, 128, 256), (1, 16, 2, 2, 128, 272), (1, 8, 1, 2, 64, 512), (2, 16, 16, 32, 128, 128)],
                         ids=["dv256_widest_in_launch_norm", "dv272_second_launch", "dv512_second_launch", "64_heads"])
def test_gdn_layer_widest_norm_fallback_and_many_heads(gpu_lib, cfg):
    """The in-launch gated norm at the widest head it is unrolled for (Dv = 256: 16 row tiles per head), the
    automatic second launch beyond that, and 64 heads counting into ONE arrivals array over six back-to-back calls."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = cfg
    args, kw, want = _layer_case(77 + Dv, B, T, Hk, Hv, Dk, Dv)
    arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
    runs = [K.gdn_layer(*args, **kw, arrivals=arrivals) for _ in range(6)]
    torch.cuda.synchronize()
    assert not arrivals.any()
    for i, r in enumerate(runs):
        _assert_layer_equals(r, want, f"(call {i})")
    pre = K.gdn_prepare(*args[:7], Hk, Hv, Dk, Dv, q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    yw, sw, tw = O.gated_delta_ops_with_tape(*(host(t) for t in pre[:5]), host(args[7]), dtype=np.float64)
    np.testing.assert_allclose(host(runs[0]["state"]), sw, **STATE_TOL)     # the equality is not two wrong answers agreeing


def test_gdn_layer_out_aliasing_gate_or_misaligned_takes_the_second_launch(gpu_lib):
    """While the launch runs, `out` carries partial sums; a caller that norms in place (out is gate) or hands a
    2-byte-aligned `out` must still get the three-call bits (the library then runs the norm as a second launch)."""
    from swiftlm_amd import DFlashKernels as K, DFlashError

    B, T, Hk, Hv, Dk, Dv = 1, 16, 4, 8, 128, 128
    args, kw, want = _layer_case(5, B, T, Hk, Hv, Dk, Dv)
    arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
    gate_copy = kw["gate"].clone()
    kw_alias = dict(kw, gate=gate_copy)
    r = K.gdn_layer(*args, **kw_alias, arrivals=arrivals, out=gate_copy)          # in place
    torch.cuda.synchronize()
    assert r["out"].data_ptr() == gate_copy.data_ptr()
    _assert_layer_equals(r, want, "(out is gate)")
    odd = torch.empty(B * T * Hv * Dv + 1, dtype=torch.bfloat16, device="cuda")[1:].view(B, T, Hv, Dv)
    assert odd.data_ptr() % 4 == 2
    r = K.gdn_layer(*args, **kw, arrivals=arrivals, out=odd)
    torch.cuda.synchronize()
    _assert_layer_equals(r, want, "(out 2-byte aligned)")
    assert not arrivals.any()
    # out overlapping y_out cannot be served by either form; the mirror allocates y itself, so go through the C ABI
    from swiftlm_amd import _lib
    from swiftlm_amd.dflash_kernels import _ptr, _stream
    x, st, w, a, bl, al, db, s0 = args[:8]
    C = x.shape[-1]
    y = torch.empty(B, T, Hv, Dv, dtype=torch.bfloat16, device="cuda")
    rc = _lib.load().dflash_gdn_layer(
        _stream(), _ptr(x), _ptr(st), _ptr(w), _ptr(a), _ptr(bl), _ptr(al), _ptr(db), _lib.BF16, 1.0 / Dk, Dk ** -0.5, 1e-6,
        _ptr(s0), _ptr(torch.empty_like(s0)), None, None, _ptr(torch.empty(B, T, Hv, Dv, device="cuda")),
        _ptr(torch.empty(B, 3, C, dtype=torch.bfloat16, device="cuda")), _ptr(y), _ptr(kw["gate"]), _ptr(kw["norm_weight"]), 1e-6, 1,
        _ptr(y.view(-1)[8:]), _ptr(arrivals), None, None, None, B, T, Hk, Hv, Dk, Dv, 4)
    assert rc == _lib.INVALID and "overlaps y_out" in _lib.last_error()


def test_gdn_layer_flags_an_arrivals_array_that_was_not_zero(gpu_lib):
    from swiftlm_amd import DFlashKernels as K, _lib
    from swiftlm_amd.dflash_kernels import _ptr

    B, T, Hk, Hv, Dk, Dv = 1, 16, 2, 4, 128, 64
    args, kw, want = _layer_case(6, B, T, Hk, Hv, Dk, Dv)
    lib = _lib.load()
    status = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.dflash_set_status_word(_ptr(status)) == 0
    try:
        arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
        _assert_layer_equals(K.gdn_layer(*args, **kw, arrivals=arrivals), want)
        torch.cuda.synchronize()
        assert int(status) == 0                                  # in contract: no flag
        garbage = torch.full((B * Hv,), 1000, dtype=torch.int32, device="cuda")
        r = K.gdn_layer(*args, **kw, arrivals=garbage)
        torch.cuda.synchronize()
        assert int(status) == _lib.STATUS_LAYER_ARRIVALS
        for name in ("y", "state", "tape", "k", "g", "conv_state"):      # everything but the gated norm is unaffected
            assert torch.equal(r[name], want[name]), name
    finally:
        lib.dflash_set_status_word(None)


def test_gdn_layer_inside_a_capture_needs_its_counters_from_outside(gpu_lib):
    """On a stream the module has not served yet, a capture cannot create the counters (their zero-fill would only
    be recorded): the mirror refuses; with a caller-provided array the captured call replays to the eager bits."""
    from swiftlm_amd import DFlashKernels as K, DFlashError

    B, T, Hk, Hv, Dk, Dv = 1, 16, 2, 4, 128, 64
    args, kw, want = _layer_case(8, B, T, Hk, Hv, Dk, Dv)
    fresh = torch.cuda.Stream()
    fresh.wait_stream(torch.cuda.current_stream())
    arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=fresh):
        with pytest.raises(DFlashError, match="inside a graph capture"):
            K.gdn_layer(*args, **kw)
        r = K.gdn_layer(*args, **kw, arrivals=arrivals)
    for i in range(3):
        for t in r.values():
            if t is not None:
                t.zero_()
        g.replay()
        torch.cuda.synchronize()
        _assert_layer_equals(r, want, f"(replay {i})")
        assert not arrivals.any()


def test_gdn_layer_hand_over_holds_over_many_graph_launches(gpu_lib):
    """The Qwen3-Next block through the one-launch layer 320 times inside captured graphs (8 graphs x 40 layer
    launches, each followed by other kernels: a fill of the previous result and a tape replay that dirties the L2s),
    compared bit for bit with the three-call result; stops at the first mismatch."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 16, 16, 32, 128, 128
    cases = [_layer_case(900 + i, B, T, Hk, Hv, Dk, Dv) for i in range(4)]
    arrivals = torch.zeros(B * Hv, dtype=torch.int32, device="cuda")
    for args, kw, _ in cases:                                    # code objects loaded, attributes set: nothing to set up inside a capture
        K.gdn_layer(*args, **kw, arrivals=arrivals)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    side.wait_stream(torch.cuda.current_stream())
    per_graph = 40
    g = torch.cuda.CUDAGraph()
    scratch_state = torch.empty(B, Hv, Dv, Dk, device="cuda")
    with torch.cuda.graph(g, stream=side):
        results = []
        for i in range(per_graph):
            args, kw, want = cases[i % len(cases)]
            r = K.gdn_layer(*args, **kw, arrivals=arrivals)
            results.append((r, want))
            # other work between the layer launches: a replay over the fresh tape (reads what the layer wrote,
            # writes 2 MB elsewhere) and a fill
            K.tape_replay_batched([r["tape"]], [r["k"]], [r["g"]], [args[7]], [scratch_state], 3)
            scratch_state.mul_(0.5)
    torch.cuda.current_stream().wait_stream(side)
    launches = 0
    for rep in range(8):
        for r, _ in results:
            r["out"].fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        for i, (r, want) in enumerate(results):
            launches += 1
            for name, w in want.items():
                if not torch.equal(r[name], w):
                    bad = (r[name].float() - w.float()).abs()
                    pytest.fail(f"replay {rep}, layer launch {i}: {name} differs from the three calls "
                                f"({int((bad > 0).sum())} elements, max abs {float(bad.max()):.3e})")
        assert not arrivals.any()
    assert launches == 320
