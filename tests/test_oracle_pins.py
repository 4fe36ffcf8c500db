"""Pins the CPU oracle against what the mathematics fixes.

The reference ships no golden vectors for this path, so every oracle function
is checked against an independent formulation (closed forms, matrix form of the
delta rule, library softmax/logsumexp, brute force), chosen so that a dropped
term, a wrong sign or index, or a transposed operand fails at least one test.
"""

import numpy as np
import pytest
from scipy.special import logsumexp, softmax

from oracle import dflash_oracle as O

F64 = np.float64


def _gdn(seed, B=2, T=6, Hk=2, Hv=4, Dk=8, Dv=5, vec=False):
    d = O.make_gdn_inputs(seed, B, T, Hk, Hv, Dk, Dv, vec_gate=vec)
    rng = np.random.default_rng(seed + 1000)
    d["tape"] = rng.standard_normal((B, T, Hv, Dv)).astype(np.float32)
    return d


# ------------------------------------------------------------------ replay --


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_replay_scalar_gate_closed_form(seed):
    d = _gdn(seed)
    B, T, Hv, Dv = d["tape"].shape
    Hk, Dk = d["k"].shape[2:]
    got = O.tape_replay_ops(d["tape"], d["k"], d["g"], d["state"], dtype=F64)
    g = d["g"].astype(F64)                                  # [B,T,Hv]
    # suffix products  c_t = prod_{s>t} g_s
    c = np.ones((B, T, Hv))
    for t in range(T - 2, -1, -1):
        c[:, t] = c[:, t + 1] * g[:, t + 1]
    total = g.prod(axis=1)                                  # [B,Hv]
    k_rep = np.repeat(d["k"].astype(F64), Hv // Hk, axis=2)  # [B,T,Hv,Dk]
    want = total[:, :, None, None] * d["state"].astype(F64) + np.einsum(
        "bth,bthv,bthk->bhvk", c, d["tape"].astype(F64), k_rep)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-14)


def test_replay_vector_gate_closed_form():
    d = _gdn(3, vec=True)
    B, T, Hv, Dv = d["tape"].shape
    Hk, Dk = d["k"].shape[2:]
    got = O.tape_replay_ops(d["tape"], d["k"], d["g"], d["state"], dtype=F64)
    g = d["g"].astype(F64)                                  # [B,T,Hv,Dk]
    c = np.ones_like(g)
    for t in range(T - 2, -1, -1):
        c[:, t] = c[:, t + 1] * g[:, t + 1]
    k_rep = np.repeat(d["k"].astype(F64), Hv // Hk, axis=2)
    want = g.prod(axis=1)[:, :, None, :] * d["state"].astype(F64) + np.einsum(
        "bthk,bthv,bthk->bhvk", c, d["tape"].astype(F64), k_rep)
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-14)


def test_replay_identities():
    d = _gdn(4)
    S0 = d["state"]
    # zero steps
    out = O.tape_replay_ops(d["tape"][:, :0], d["k"][:, :0], d["g"][:, :0], S0)
    np.testing.assert_array_equal(out, S0)
    # all-zero mask: untouched, not even decayed (DFlashKernels.swift:30-34)
    mask = np.zeros(d["tape"].shape[:2], np.float32)
    np.testing.assert_array_equal(O.tape_replay_ops(d["tape"], d["k"], d["g"], S0, mask), S0)
    # delta = 0, g = 1
    out = O.tape_replay_ops(np.zeros_like(d["tape"]), d["k"], np.ones_like(d["g"]), S0)
    np.testing.assert_array_equal(out, S0)
    # g = 0 on the last step: only the last outer product survives
    g = d["g"].copy()
    g[:, -1] = 0
    out = O.tape_replay_ops(d["tape"], d["k"], g, S0, dtype=F64)
    k_rep = np.repeat(d["k"], 2, axis=2).astype(F64)
    want = d["tape"][:, -1, :, :, None].astype(F64) * k_rep[:, -1, :, None, :]
    np.testing.assert_allclose(out, want, rtol=0, atol=1e-15)


def test_replay_is_not_symmetric_in_dv_dk():
    # state is [.., Dv, Dk]: delta indexes rows, k indexes columns.
    d = _gdn(5, B=1, T=1, Hk=1, Hv=1, Dk=3, Dv=2)
    tape = np.array([[[[1.0, 2.0]]]], np.float32)
    k = np.array([[[[10.0, 20.0, 30.0]]]], np.float32)
    out = O.tape_replay_ops(tape, k, np.zeros((1, 1, 1), np.float32), d["state"])
    np.testing.assert_array_equal(out[0, 0], [[10, 20, 30], [20, 40, 60]])


def test_replay_gqa_head_mapping_is_consecutive_repeat():
    # value head hv reads key head hv // (Hv/Hk): heads 0,1 -> key head 0; 2,3 -> key head 1.
    B, T, Hk, Hv, Dk, Dv = 1, 1, 2, 4, 4, 3
    k = np.zeros((B, T, Hk, Dk), np.float32)
    k[0, 0, 1] = 1.0                                     # only key head 1 is non-zero
    tape = np.ones((B, T, Hv, Dv), np.float32)
    out = O.tape_replay_ops(tape, k, np.ones((B, T, Hv), np.float32),
                            np.zeros((B, Hv, Dv, Dk), np.float32))
    assert np.all(out[0, :2] == 0) and np.all(out[0, 2:] == 1)


@pytest.mark.parametrize("vec", [False, True])
def test_replay_prefix_composition(vec):
    d = _gdn(6, vec=vec)
    full = O.tape_replay_ops(d["tape"], d["k"], d["g"], d["state"], dtype=F64)
    for m in range(0, 7):
        head = O.tape_replay_ops(d["tape"][:, :m], d["k"][:, :m], d["g"][:, :m], d["state"], dtype=F64)
        both = O.tape_replay_ops(d["tape"][:, m:], d["k"][:, m:], d["g"][:, m:], head, dtype=F64)
        np.testing.assert_allclose(both, full, rtol=1e-13, atol=1e-15)


def test_replay_masked_equals_subsequence():
    d = _gdn(7, B=1)
    mask = np.array([[1, 0, 1, 1, 0, 1]], np.float32)
    keep = mask[0] > 0.5
    got = O.tape_replay_ops(d["tape"], d["k"], d["g"], d["state"], mask)
    want = O.tape_replay_ops(d["tape"][:, keep], d["k"][:, keep], d["g"][:, keep], d["state"])
    np.testing.assert_array_equal(got, want)


def test_replay_requant_rounds_each_step():
    d = _gdn(8, T=3)
    out = O.tape_replay_ops(d["tape"], d["k"], d["g"], O.round_to_bf16(d["state"]), requant="bf16")
    np.testing.assert_array_equal(out, O.round_to_bf16(out))
    loose = O.tape_replay_ops(d["tape"], d["k"], d["g"], O.round_to_bf16(d["state"]))
    assert not np.array_equal(out, loose)
    np.testing.assert_allclose(out, loose, rtol=3e-2, atol=3e-2)


# ------------------------------------------------------------- gated delta --


def _matrix_form(q, k, v, g, beta, S0):
    """Independent statement: S <- S diag(g) (I - b k k^T) + b v k^T per head, y = S q."""
    B, T, Hk, Dk = q.shape
    Hv, Dv = v.shape[2:]
    rf = Hv // Hk
    S = S0.astype(F64).copy()
    ys = np.zeros((B, T, Hv, Dv))
    deltas = np.zeros((B, T, Hv, Dv))
    eye = np.eye(Dk)
    for b in range(B):
        for h in range(Hv):
            M = S[b, h]                                   # [Dv, Dk]
            for t in range(T):
                kk = k[b, t, h // rf].astype(F64)
                qq = q[b, t, h // rf].astype(F64)
                gv = g[b, t, h].astype(F64)
                G = np.diag(np.broadcast_to(gv, (Dk,)))
                bt = F64(beta[b, t, h])
                Md = M @ G
                deltas[b, t, h] = bt * (v[b, t, h].astype(F64) - Md @ kk)
                M = Md @ (eye - bt * np.outer(kk, kk)) + bt * np.outer(v[b, t, h].astype(F64), kk)
                ys[b, t, h] = M @ qq
            S[b, h] = M
    return ys, S, deltas


@pytest.mark.parametrize("vec", [False, True])
def test_gated_delta_matches_matrix_form(vec):
    d = _gdn(10, vec=vec)
    y, S, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], dtype=F64)
    yw, Sw, tw = _matrix_form(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"])
    np.testing.assert_allclose(y, yw, rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(S, Sw, rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(tape, tw, rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("vec", [False, True])
def test_signed_and_degenerate_gates_match_matrix_and_closed_forms(vec):
    """The reference micro-benchmark draws EVERYTHING from uniform(-0.1, 0.1), gates and betas included
    (Sources/DFlashKernelBench/main.swift:28-30), so the oracle must hold for negative decays and betas and for
    the degenerate values 0 and 1: checked against the matrix form of the delta rule and, for the replay, the
    closed form (neither takes a logarithm, a quotient or a root of a gate)."""
    rng = np.random.default_rng(21)
    B, T, Hk, Hv, Dk, Dv = 2, 7, 2, 4, 8, 5
    u = lambda *s: rng.uniform(-0.1, 0.1, s).astype(np.float32)
    gshape = (B, T, Hv, Dk) if vec else (B, T, Hv)
    q, k, v, g, beta, S0 = u(B, T, Hk, Dk), u(B, T, Hk, Dk), u(B, T, Hv, Dv), u(*gshape), u(B, T, Hv), u(B, Hv, Dv, Dk)
    g[:, 1], g[:, 3], g[:, 5] = 0.0, 1.0, -0.5
    beta[:, 2], beta[:, 4] = 0.0, 1.0
    y, S, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0, dtype=F64)
    yw, Sw, tw = _matrix_form(q, k, v, g, beta, S0)
    np.testing.assert_allclose(y, yw, rtol=1e-11, atol=1e-15)
    np.testing.assert_allclose(S, Sw, rtol=1e-11, atol=1e-15)
    np.testing.assert_allclose(tape, tw, rtol=1e-11, atol=1e-15)
    # replay of that tape: closed form with suffix products of the signed gates
    got = O.tape_replay_ops(tape, k, g, S0, dtype=F64)
    gg = g.astype(F64) if vec else np.broadcast_to(g.astype(F64)[..., None], (B, T, Hv, Dk))
    c = np.ones_like(gg)
    for t in range(T - 2, -1, -1):
        c[:, t] = c[:, t + 1] * gg[:, t + 1]
    k_rep = np.repeat(k.astype(F64), Hv // Hk, axis=2)
    want = gg.prod(axis=1)[:, :, None, :] * S0.astype(F64) + np.einsum("bthk,bthv,bthk->bhvk", c, tape, k_rep)
    np.testing.assert_allclose(got, want, rtol=1e-11, atol=1e-15)
    np.testing.assert_allclose(got, S, rtol=1e-11, atol=1e-15)        # and it lands on the forward's state


def test_gated_delta_matches_kimi_restatement():
    # Second in-tree statement of the recurrence, vector gate, Hk == Hv
    # (Sources/SwiftLM/KimiLinearDFlash.swift:395-403), written with einsum.
    d = _gdn(11, Hk=4, Hv=4, vec=True)
    q, k, v, g, beta = (d[n].astype(F64) for n in ("q", "k", "v", "g", "beta"))
    s = d["state"].astype(F64)
    ys = []
    for t in range(q.shape[1]):
        s = s * g[:, t][:, :, None, :]
        kv = np.einsum("bhvk,bhk->bhv", s, k[:, t])
        delta = (v[:, t] - kv) * beta[:, t][..., None]
        s = s + np.einsum("bhk,bhv->bhvk", k[:, t], delta)
        ys.append(np.einsum("bhvk,bhk->bhv", s, q[:, t]))
    y, S, _ = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], dtype=F64)
    np.testing.assert_allclose(y, np.stack(ys, 1), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(S, s, rtol=1e-12, atol=1e-14)


def test_forward_low_precision_state_rounds_state_not_y():
    """One step by hand (DFlashKernels.swift:148-199 with a bf16 state): the stored state is the
    bf16 rounding of the updated state (:183-186) while y is read from the state before that
    rounding (:171-172).  Values are picked so that the two differ: 1 + 2^-9 is not a bf16 number."""
    eps = 2.0 ** -9
    S0 = np.array([[[[1.0, 0.0]]]], np.float32)            # one head, one row, Dk = 2
    k = np.array([[[[0.0, 1.0]]]], np.float32)
    q = np.array([[[[1.0, 1.0]]]], np.float32)
    v = np.array([[[[eps]]]], np.float32)
    g = np.ones((1, 1, 1), np.float32)
    beta = np.ones((1, 1, 1), np.float32)
    # by hand: S' = S0; m = S'k = 0; delta = (eps - 0) * 1 = eps; S = [1, eps]; y = S q = 1 + eps
    y, S, tape = O.gated_delta_ops_with_tape(q, k, v, g, beta, S0, requant="bf16")
    assert tape[0, 0, 0, 0] == np.float32(eps)
    assert y[0, 0, 0, 0] == np.float32(1.0 + eps)          # not re-rounded: bf16 would give 1.0
    np.testing.assert_array_equal(S[0, 0, 0], [1.0, eps])  # both entries are bf16 numbers
    # second step: now the update lands on the SAME entry, so the state must round and y must not
    k2 = np.array([[[[1.0, 0.0]]], [[[1.0, 0.0]]]], np.float32).reshape(1, 2, 1, 2)
    q2 = np.tile(q, (1, 2, 1, 1))
    v2 = np.array([1.0, 1.0 + 2 * eps + eps], np.float32).reshape(1, 2, 1, 1)   # step 2: delta = v - S[0]
    S1 = np.array([[[[1.0, 0.0]]]], np.float32)
    y2, S2, t2 = O.gated_delta_ops_with_tape(q2, k2, v2, np.ones((1, 2, 1), np.float32),
                                             np.ones((1, 2, 1), np.float32), S1, requant="bf16")
    # step 1: m = 1, delta = 0, S = [1, 0]; step 2: m = 1, delta = 3 eps, S = [1 + 3 eps, 0] -> y = 1 + 3 eps,
    # stored state rounds 1 + 3*2^-9 (= 1.005859375) to the bf16 grid {1, 1 + 2^-7}: nearest is 1 + 2^-7
    assert t2[0, 1, 0, 0] == np.float32(3 * eps)
    assert y2[0, 1, 0, 0] == np.float32(1.0 + 3 * eps)
    np.testing.assert_array_equal(S2[0, 0, 0], [1.0 + 2.0 ** -7, 0.0])
    # and the un-rounded path keeps the exact value
    _, S3, _ = O.gated_delta_ops_with_tape(q2, k2, v2, np.ones((1, 2, 1), np.float32),
                                           np.ones((1, 2, 1), np.float32), S1)
    np.testing.assert_array_equal(S3[0, 0, 0], [np.float32(1.0 + 3 * eps), 0.0])


@pytest.mark.parametrize("vec", [False, True])
def test_forward_tape_replays_to_forward_state(vec):
    """replay(tape[:n]) from S0 == state after the forward on the first n tokens."""
    d = _gdn(12, vec=vec)
    _, S_full, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], dtype=F64)
    T = d["q"].shape[1]
    for n in range(0, T + 1):
        _, S_n, _ = O.gated_delta_ops_with_tape(d["q"][:, :n], d["k"][:, :n], d["v"][:, :n], d["g"][:, :n],
                                                d["beta"][:, :n], d["state"], dtype=F64) if n else (0, d["state"].astype(F64), 0)
        rep = O.tape_replay_ops(tape[:, :n], d["k"][:, :n], d["g"][:, :n], d["state"], dtype=F64)
        np.testing.assert_allclose(rep, S_n, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(O.tape_replay_ops(tape, d["k"], d["g"], d["state"], dtype=F64), S_full,
                               rtol=1e-12, atol=1e-14)


def test_gated_delta_special_cases():
    d = _gdn(13, B=1, T=3, Hk=1, Hv=2, Dk=6, Dv=4)
    # beta = 0: pure decay, delta = 0, y_t = decayed state . q_t
    y, S, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], np.zeros_like(d["beta"]),
                                             d["state"], dtype=F64)
    assert np.all(tape == 0)
    dec = d["state"].astype(F64)
    for t in range(3):
        dec = dec * d["g"][:, t, :, None, None]
        np.testing.assert_allclose(y[:, t], np.einsum("bhvk,bk->bhv", dec, d["q"][:, t, 0].astype(F64)),
                                   rtol=1e-13)
    np.testing.assert_allclose(S, dec, rtol=1e-13)
    # zero state: the first innovation is beta * v and y_0 = beta * v * (k . q)
    y, S, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"],
                                             np.zeros_like(d["state"]), dtype=F64)
    bv = d["beta"][:, 0, :, None].astype(F64) * d["v"][:, 0].astype(F64)
    np.testing.assert_allclose(tape[:, 0], bv, rtol=1e-13)
    kq = float(d["k"][0, 0, 0].astype(F64) @ d["q"][0, 0, 0].astype(F64))
    np.testing.assert_allclose(y[:, 0], bv * kq, rtol=1e-12)


@pytest.mark.parametrize("vec", [False, True])
def test_gated_delta_masked_equals_subsequence(vec):
    d = _gdn(14, B=1, vec=vec)
    mask = np.array([[0, 1, 1, 0, 1, 0]], np.float32)
    keep = mask[0] > 0.5
    y, S, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask)
    ys, Ss, ts = O.gated_delta_ops_with_tape(d["q"][:, keep], d["k"][:, keep], d["v"][:, keep], d["g"][:, keep],
                                             d["beta"][:, keep], d["state"])
    np.testing.assert_array_equal(S, Ss)
    np.testing.assert_array_equal(y[:, keep], ys)
    np.testing.assert_array_equal(tape[:, keep], ts)
    assert np.all(y[:, ~keep] == 0) and np.all(tape[:, ~keep] == 0)
    assert tape.dtype == np.float32


# ------------------------------------------------- acceptance and indexing --


def test_match_acceptance_length_doc_example():
    # DFlashRuntime.swift:130-132
    assert O.match_acceptance_length([1, 2, 3], [1, 2, 5]) == 2
    assert O.match_acceptance_length([], []) == 0
    assert O.match_acceptance_length([7], [7]) == 1
    assert O.match_acceptance_length([1, 2, 3], [9, 2, 3]) == 0     # later matches do not count
    assert O.match_acceptance_length([1, 2, 3], [1, 9, 3]) == 1


def test_match_acceptance_length_brute_force():
    rng = np.random.default_rng(0)
    for _ in range(500):
        n = int(rng.integers(0, 16))
        a = rng.integers(0, 3, n)
        b = rng.integers(0, 3, n)
        want = 0
        for x, y in zip(a, b):
            if x != y:
                break
            want += 1
        assert O.match_acceptance_length(a, b) == want


def test_accept_commit_indexing():
    rng = np.random.default_rng(1)
    for _ in range(200):
        V = int(rng.integers(1, 17))
        staged = int(rng.integers(0, 50))
        drafted = rng.integers(0, 4, V - 1)
        posterior = rng.integers(0, 4, V)
        start = int(rng.integers(0, 1000))
        r = O.accept_commit(staged, drafted, posterior, start)
        a = 0
        while a < V - 1 and drafted[a] == posterior[a]:
            a += 1
        assert r["acceptance_len"] == a and 0 <= a <= V - 1
        assert r["commit_count"] == a + 1
        assert list(r["committed"]) == [staged] + list(drafted[:a])
        assert r["staged_next"] == posterior[a]
        assert r["start"] == start + a + 1
        assert r["rollback_args"] == {"target_len": start + a + 1, "acceptance_length": a, "drafted_tokens": V - 1}


def test_rebuild_conv_state_brute_force():
    rng = np.random.default_rng(2)
    B, keep, C, T = 2, 3, 5, 8
    snap = rng.standard_normal((B, keep, C)).astype(np.float32)
    qkv = rng.standard_normal((B, T, C)).astype(np.float32)
    for steps in range(1, T + 1):
        got = O.rebuild_conv_state(snap, qkv, steps, keep)
        # the window is the last `keep` inputs seen after `steps` tokens
        hist = [snap[:, i] for i in range(keep)] + [qkv[:, t] for t in range(steps)]
        want = np.stack(hist[-keep:], axis=1)
        np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(O.rebuild_conv_state(None, qkv, 1, keep)[:, :2], 0)
    # the slice end is clamped (RecurrentRollbackCache.swift:156)
    assert O.rebuild_conv_state(snap, qkv, T + 2, keep).shape[1] == 1


def test_restore_target_cache_actions():
    caches = [("rollback", 0), ("kv", 116), ("mamba", 0), ("kv", 100)]
    # partial acceptance: replay nAccepted, trim KV down to targetLen
    assert O.restore_target_cache_after_acceptance(caches, 104, 3, 15) == [
        ("rollback", 3), ("trim", 12), ("set_offset", 104), ("none",)]
    # fully accepted: no replay (DFlashRuntime.swift:194,199-202)
    assert O.restore_target_cache_after_acceptance(caches, 116, 15, 15)[0] == ("clear",)
    # draftedTokens == 0 is never "fully accepted"
    assert O.restore_target_cache_after_acceptance(caches, 101, 0, 0)[0] == ("rollback", 0)


def test_rollback_cache_state_machine():
    d = _gdn(20, B=1, T=8, Hk=2, Hv=4, Dk=8, Dv=8)
    rng = np.random.default_rng(3)
    conv0 = rng.standard_normal((1, 3, 10)).astype(np.float32)
    qkv = rng.standard_normal((1, 8, 10)).astype(np.float32)
    c = O.RecurrentRollbackCacheOracle()
    c.slots = [conv0, d["state"]]
    c.arm_rollback(prefix_len=5)
    assert c.armed
    y, S_full, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"])
    c.slots = [qkv[:, -3:], S_full]        # what the verify forward leaves behind
    c.record_tape(tape, d["k"], d["g"], qkv)
    c.rollback(n_accepted=2)               # acceptedSteps = 3
    _, S3, _ = O.gated_delta_ops_with_tape(d["q"][:, :3], d["k"][:, :3], d["v"][:, :3], d["g"][:, :3],
                                           d["beta"][:, :3], d["state"])
    np.testing.assert_allclose(c.slots[1], S3, rtol=1e-5, atol=1e-6)
    np.testing.assert_array_equal(c.slots[0], qkv[:, 0:3])
    assert not c.armed and c._snapshot is None
    # rollback without arm is a no-op that clears
    before = c.slots[1].copy()
    c.rollback(n_accepted=0)
    np.testing.assert_array_equal(c.slots[1], before)
    c.offset = 5
    assert c.trim(8) == 5 and c.offset == 0


# -------------------------------------------------------------------- sdpa --


def _sdpa_library(q, k, v, scale):
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1:3]
    kk = np.repeat(k.astype(F64), Hq // Hk, axis=1)
    vv = np.repeat(v.astype(F64), Hq // Hk, axis=1)
    s = np.einsum("bhmd,bhnd->bhmn", q.astype(F64), kk) * scale
    vis = np.arange(N)[None, :] <= (N - M + np.arange(M))[:, None]
    s = np.where(vis, s, -np.inf)
    return np.einsum("bhmn,bhnd->bhmd", softmax(s, axis=-1), vv), logsumexp(s, axis=-1)


def test_sdpa_matches_library_softmax():
    q, k, v = O.make_sdpa_inputs(0, B=2, Hq=4, Hk=2, M=16, L=37, D=8)
    o, lse = O.sdpa_block_causal(q, k, v, 0.3)
    ow, lw = _sdpa_library(q, k, v, 0.3)
    np.testing.assert_allclose(o, ow, rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(lse, lw, rtol=1e-12, atol=1e-14)


def test_sdpa_invariants():
    q, k, v = O.make_sdpa_inputs(1, B=1, Hq=4, Hk=2, M=16, L=20, D=8)
    # constant V -> constant O (rows of the softmax sum to one)
    o, _ = O.sdpa_block_causal(q, k, np.full_like(v, 2.5), 0.2)
    np.testing.assert_allclose(o, 2.5, rtol=1e-13)
    # L = 0: plain causal attention over the block; row 0 sees only key 0
    q, k, v = O.make_sdpa_inputs(2, B=1, Hq=2, Hk=1, M=16, L=0, D=8)
    o, lse = O.sdpa_block_causal(q, k, v, 0.5)
    np.testing.assert_allclose(o[0, :, 0], np.broadcast_to(v[0, 0, 0], (2, 8)), rtol=1e-13)
    s = np.einsum("hmd,nd->hmn", q[0].astype(F64), k[0, 0].astype(F64)) * 0.5
    s = np.where(np.tril(np.ones((16, 16), bool)), s, -np.inf)
    np.testing.assert_allclose(o[0], softmax(s, -1) @ v[0, 0].astype(F64), rtol=1e-12)
    np.testing.assert_allclose(lse[0], logsumexp(s, -1), rtol=1e-12)
    # GQA: query heads 0,1 read kv head 0 and heads 2,3 read kv head 1
    q, k, v = O.make_sdpa_inputs(3, B=1, Hq=4, Hk=2, M=16, L=8, D=8)
    v2 = v.copy()
    v2[:, 1] += 1.0
    o1, _ = O.sdpa_block_causal(q, k, v, 0.3)
    o2, _ = O.sdpa_block_causal(q, k, v2, 0.3)
    np.testing.assert_allclose(o2[:, :2], o1[:, :2], rtol=1e-13)
    np.testing.assert_allclose(o2[:, 2:], o1[:, 2:] + 1.0, rtol=1e-12)


def test_sdpa_additive_mask():
    q, k, v = O.make_sdpa_inputs(4, B=1, Hq=2, Hk=1, M=16, L=16, D=8)
    mask = np.zeros((1, 2, 16, 32))
    mask[..., :5] = -np.inf                               # hide the first five keys
    o, _ = O.sdpa_block_causal(q, k, v, 0.3, mask)
    ow, _ = O.sdpa_block_causal(q, k[:, :, 5:], v[:, :, 5:], 0.3)
    np.testing.assert_allclose(o, ow, rtol=1e-12)


def test_sdpa_additive_mask_bias_and_empty_rows():
    """A finite mask is a bias on the score (DFlashKernels.swift:553): adding log(w_n) weights key n
    by w_n in the softmax.  A row whose keys are all dropped yields zeros, not NaN (:711)."""
    q, k, v = (a.astype(np.float64) for a in O.make_sdpa_inputs(6, B=1, Hq=2, Hk=1, M=16, L=8, D=8))
    N = 24
    rng = np.random.default_rng(0)
    w = rng.uniform(0.5, 2.0, size=(1, 2, 16, N))
    o, lse = O.sdpa_block_causal(q, k, v, 0.3, np.log(w))
    s = np.einsum("bhmd,bhnd->bhmn", q * 0.3, np.repeat(k, 2, axis=1))
    vis = np.arange(N)[None, :] <= (N - 16 + np.arange(16))[:, None]
    p = np.where(vis, w * np.exp(s), 0.0)
    np.testing.assert_allclose(o, np.einsum("bhmn,bhnd->bhmd", p / p.sum(-1, keepdims=True), np.repeat(v, 2, axis=1)), rtol=1e-12)
    np.testing.assert_allclose(lse, np.log(p.sum(-1)), rtol=1e-12)
    mask = np.zeros((1, 2, 16, N))
    mask[0, 1, 3, :] = -np.inf
    o, lse = O.sdpa_block_causal(q, k, v, 0.3, mask)
    assert np.all(o[0, 1, 3] == 0.0) and lse[0, 1, 3] == -np.inf
    assert np.isfinite(o).all()


@pytest.mark.parametrize("blocks", [32, 64])
def test_sdpa_2pass_agrees_with_single_pass(blocks):
    q, k, v = O.make_sdpa_inputs(5, B=1, Hq=4, Hk=2, M=16, L=200, D=16)
    want, _ = O.sdpa_block_causal(q, k, v, 0.25)
    exact = O.sdpa_2pass(q, k, v, 0.25, blocks, partial_dtype="f32")
    np.testing.assert_allclose(exact, want, rtol=2e-5, atol=2e-6)
    rounded = O.sdpa_2pass(q, k, v, 0.25, blocks, partial_dtype="bf16")
    np.testing.assert_allclose(rounded, want, rtol=2e-2, atol=2e-2)


# ---------------------------------------------------------------- C oracle --


@pytest.mark.parametrize("variant", ["fused", "opbyop"])
@pytest.mark.parametrize("vec", [False, True])
@pytest.mark.parametrize("masked", [False, True])
def test_c_oracle_matches_numpy_oracle(variant, vec, masked):
    from oracle import c_oracle

    d = _gdn(30, B=2, T=5, Hk=2, Hv=4, Dk=16, Dv=8, vec=vec)
    mask = np.array([[1, 0, 1, 1, 0], [0, 1, 1, 0, 1]], np.float32) if masked else None
    got = c_oracle.tape_replay(d["tape"], d["k"], d["g"], d["state"], mask, variant=variant)
    want = O.tape_replay_ops(d["tape"], d["k"], d["g"], d["state"], mask, dtype=F64)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
    y, S, tape = c_oracle.gated_delta(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask,
                                      variant=variant)
    yw, Sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask,
                                             dtype=F64)
    np.testing.assert_allclose(y, yw, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(S, Sw, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(tape, tw, rtol=1e-4, atol=1e-5)


def test_c_oracle_sdpa_and_accept():
    from oracle import c_oracle

    q, k, v = O.make_sdpa_inputs(6, B=2, Hq=4, Hk=2, M=16, L=50, D=16)
    o, lse = c_oracle.sdpa_block_causal(q, k, v, 0.25)
    ow, lw = O.sdpa_block_causal(q, k, v, 0.25)
    np.testing.assert_allclose(o, ow, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(lse, lw, rtol=1e-5, atol=1e-5)
    assert c_oracle.match_acceptance_length([1, 2, 3], [1, 2, 5]) == 2
    assert c_oracle.match_acceptance_length([], []) == 0


# ---- greedy tokens (DFlashRuntime.swift:105-128) ----

def test_greedy_tokens_with_mask_brute_force():
    rng = np.random.default_rng(3)
    T, V = 5, 37
    logits = rng.standard_normal((T, V)).astype(np.float32)
    ids = [3, 36, -1, 99, 3]                                   # out-of-range ids are dropped (:109)
    mask = O.build_suppress_token_mask(V, ids)
    assert mask.sum() == 2 and mask[3] and mask[36]
    assert O.build_suppress_token_mask(V, [-5, 400]) is None and O.build_suppress_token_mask(V, None) is None
    got = O.greedy_tokens_with_mask(logits, mask)
    for t in range(T):
        best, arg = None, None
        for v in range(V):
            x = -1e9 if mask[v] else logits[t, v]
            if best is None or x > best:
                best, arg = x, v
        assert got[t] == arg
    assert got.dtype == np.uint32
    # the row maximum sits on a suppressed token: the runner-up is returned
    logits[0, 3] = 50.0
    assert O.greedy_tokens_with_mask(logits, mask)[0] != 3
    assert O.greedy_tokens_with_mask(logits, None)[0] == 3
    # ties: lowest index
    logits[1, :] = 0.0
    assert O.greedy_tokens_with_mask(logits, None)[1] == 0


def test_greedy_floor_is_rounded_to_the_logits_type():
    """where(mask, MLXArray(-1e9, dtype: logits.dtype), logits): with every token suppressed the
    floor ties everywhere and index 0 wins; a logit below the rounded floor loses to it."""
    V = 8
    mask = np.ones(V, bool)
    assert O.greedy_tokens_with_mask(np.zeros((1, V), np.float32), mask, dtype="bf16")[0] == 0
    mask[:] = False
    mask[5] = True
    low = np.full((1, V), -2e9, np.float32)
    assert O.greedy_tokens_with_mask(low, mask, dtype="bf16")[0] == 5


# ---- GatedDelta pre-ops (KimiLinearDFlash.swift:274-293, :362-363, :390-391) ----

def test_short_conv_is_a_causal_correlation_with_carried_window():
    from scipy.signal import correlate
    rng = np.random.default_rng(0)
    B, T, C, K = 2, 9, 5, 4
    x = rng.standard_normal((B, T, C))
    st = rng.standard_normal((B, K - 1, C))
    w = rng.standard_normal((C, K))
    out, new = O.short_conv_silu(x, st, w)
    for b in range(B):
        for c in range(C):
            full = np.concatenate([st[b, :, c], x[b, :, c]])
            pre = correlate(full, w[c], mode="valid")                 # sum_j full[t+j] w[j]
            np.testing.assert_allclose(out[b, :, c], pre / (1 + np.exp(-pre)), rtol=1e-12)
    np.testing.assert_array_equal(new, np.concatenate([st, x], 1)[:, T:])
    # processing the block in two pieces with the carried window equals one pass (what makes the
    # window a sufficient state, and what rebuildConvState relies on)
    o1, s1 = O.short_conv_silu(x[:, :4], st, w)
    o2, s2 = O.short_conv_silu(x[:, 4:], s1, w)
    np.testing.assert_allclose(np.concatenate([o1, o2], 1), out, rtol=1e-12)
    np.testing.assert_array_equal(s2, new)
    # no state = zeros (:288); T shorter than the window keeps old rows
    o0, _ = O.short_conv_silu(x, None, w)
    oz, _ = O.short_conv_silu(x, np.zeros_like(st), w)
    np.testing.assert_array_equal(o0, oz)
    _, s_short = O.short_conv_silu(x[:, :2], st, w)
    np.testing.assert_array_equal(s_short, np.concatenate([st[:, 2:], x[:, :2]], 1))
    # the rollback cache's rebuilt window after accepting n steps is the window a forward over the
    # first n tokens would have left (RecurrentRollbackCache.swift:139-158)
    for n in range(1, T + 1):
        _, want = O.short_conv_silu(x[:, :n], st, w)
        np.testing.assert_array_equal(O.rebuild_conv_state(st, x, n, K - 1), want)


def test_rms_norm_and_gates_against_library_forms():
    from scipy.special import expit
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 3, 4, 16))
    y = O.rms_norm_scaled(x, 16 ** -0.5, eps=0.0)
    np.testing.assert_allclose(np.linalg.norm(y, axis=-1), 1.0, rtol=1e-12)      # scale * rmsNorm = L2 normalisation
    a = rng.standard_normal((2, 3, 4)) * 3
    b = rng.standard_normal((2, 3, 4)) * 3
    al = rng.standard_normal(4)
    db = rng.standard_normal(4)
    g, beta = O.gdn_gates(a, b, al, db)
    np.testing.assert_allclose(beta, expit(b), rtol=1e-12)
    np.testing.assert_allclose(np.log(g), -np.exp(al) * np.log1p(np.exp(a + db)), rtol=1e-10)
    assert np.all((g > 0) & (g <= 1))
    # per-channel gate: each channel follows the scalar formula with its own bias
    a4 = rng.standard_normal((1, 2, 4, 8))
    db4 = rng.standard_normal((4, 8))
    g4, _ = O.gdn_gates(a4, b[:1, :2], al, db4)
    for d in range(8):
        gd, _ = O.gdn_gates(a4[..., d], b[:1, :2], al, db4[:, d])
        np.testing.assert_allclose(g4[..., d], gd, rtol=1e-12)


def test_gdn_finish_against_library_forms():
    from scipy.special import expit
    rng = np.random.default_rng(2)
    y = rng.standard_normal((2, 3, 4, 16))
    z = rng.standard_normal((2, 3, 4, 16)) * 3
    w = rng.standard_normal(16)
    out = O.gdn_finish(y, z, w, 0.0)
    # with eps = 0 and unit weight the normalised rows have RMS 1; undo the gate to see it
    unit = O.gdn_finish(y, z, np.ones(16), 0.0) / expit(z)
    np.testing.assert_allclose(np.sqrt((unit ** 2).mean(-1)), 1.0, rtol=1e-12)
    np.testing.assert_allclose(out, unit * w * expit(z), rtol=1e-12)
    np.testing.assert_allclose(O.gdn_finish(y, z, w, 1e-6, "silu"), O.gdn_finish(y, z, w, 1e-6) * z, rtol=1e-12)


def test_page_gather_scatter_brute_force():
    """gather_pages against an element-by-element loop over the page table, scatter_pages as its inverse,
    and the attention on a gathered cache equal to the attention on the dense one."""
    rng = np.random.default_rng(11)
    B, Hk, N, D, P, pages = 2, 3, 75, 4, 32, 9
    dense = rng.standard_normal((B, Hk, N, D)).astype(np.float32)
    table = np.array([[7, 2, 5], [0, 8, 3]])
    pool = O.scatter_pages(dense, table, pages, P, fill=-1.0)
    for b in range(B):
        for n in range(N):
            assert np.array_equal(pool[table[b, n // P], :, n % P], dense[b, :, n])
    untouched = np.ones(pages, bool)
    untouched[table.ravel()] = False
    assert np.all(pool[untouched] == -1.0)                       # pages nobody maps keep the fill
    assert np.all(pool[table[0, 2], :, N - 2 * P:] == -1.0)      # and so does the unused end of a last page
    got = O.gather_pages(pool, table, N)
    assert got.shape == dense.shape and np.array_equal(got, dense)
    assert np.array_equal(O.gather_pages(pool, table, 40), dense[:, :, :40])
    q = rng.standard_normal((B, 6, 16, D)).astype(np.float32)
    o1, l1 = O.sdpa_block_causal(q, dense, dense[::-1].copy(), 0.5)
    o2, l2 = O.sdpa_block_causal(q, got, O.gather_pages(O.scatter_pages(dense[::-1].copy(), table, pages, P), table, N), 0.5)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)
