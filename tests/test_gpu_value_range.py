"""GPU parity over the VALUE RANGE the reference feeds these kernels, not only the benchmark's
well-conditioned draws (L2-normalised q/k, gates and betas in (0, 1), a small state).

The chunked GatedDelta forward is algebraically different from the step-by-step recurrence
(decay-product tables, a 16x16 unit-triangular solve, a three-term bf16 split of the state), so it
is held against the float64 oracle on:
  * the reference micro-benchmark's own distribution: uniform(-0.1, 0.1) for q, k, v, g, beta and
    the state alike -- i.e. NEGATIVE gates and betas -- at its shape B=1, T=16, Hk=8, Hv=16,
    Dk=Dv=128 (Sources/DFlashKernelBench/main.swift:28-30, :551), masked and unmasked;
  * rows of special gates g in {0, 1, -0.5} and beta in {0, 1};
  * un-normalised keys with beta * |k|^2 up to 2 (the edge of the delta rule's stable range);
  * a state of magnitude 1e3;
each at T = 16 (one chunk) and T = 40 (the path that carries the state tile between chunks), with
bf16 and f32 inputs, scalar and per-channel gate.  The tape replay gets the same inputs.

Errors are measured against the largest magnitude of the expected array: fp32 state and tape
1e-4 * max|want|, low-precision y 2e-2 * max|want| (the stated bars, with the scale of the data in
place of an absolute floor that means nothing at |S| ~ 1e3 or ~ 1e-2).
"""

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

TORCH_DT = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def dev(a, dt="f32"):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", TORCH_DT[dt])


def host(t):
    return t.detach().float().cpu().numpy()


def assert_close_to_scale(got, want, tol, what):
    """max |got - want| <= tol * max |want| (and no NaN / inf where the oracle has none)."""
    want = np.asarray(want, np.float64)
    got = np.asarray(got, np.float64)
    assert np.isfinite(got).all() == np.isfinite(want).all(), f"{what}: non-finite values"
    scale = max(float(np.abs(want).max()), 1e-30)
    err = float(np.abs(got - want).max())
    assert err <= tol * scale, f"{what}: max abs err {err:.3e} > {tol:g} * max|want| = {tol * scale:.3e}"


def draw(kind, seed, B, T, Hk, Hv, Dk, Dv, in_dt, vec):
    """Inputs of one value-range case, rounded to the input type (the oracle sees what the device sees)."""
    rng = np.random.default_rng(seed)
    gshape = (B, T, Hv, Dk) if vec else (B, T, Hv)
    if kind == "refbench":
        u = lambda *s: rng.uniform(-0.1, 0.1, s).astype(np.float32)
        d = dict(q=u(B, T, Hk, Dk), k=u(B, T, Hk, Dk), v=u(B, T, Hv, Dv), g=u(*gshape), beta=u(B, T, Hv),
                 state=u(B, Hv, Dv, Dk))
    else:
        d = O.make_gdn_inputs(seed, B, T, Hk, Hv, Dk, Dv, in_dtype="f32", vec_gate=vec)
        if kind == "special_gates":
            gv = np.array([0.0, 1.0, -0.5, 0.3, 1.0, 0.0], np.float32)
            bv = np.array([0.0, 1.0, 0.5, 1.0, 0.0], np.float32)
            # step t of head h takes gv[(t + h) % 6] / bv[(t + 2h) % 5]: every head meets every value, in different orders
            tt, hh = np.meshgrid(np.arange(T), np.arange(Hv), indexing="ij")
            g = gv[(tt + hh) % len(gv)][None].repeat(B, 0)
            d["g"] = np.broadcast_to(g[..., None], gshape).copy() if vec else g
            d["beta"] = bv[(tt + 2 * hh) % len(bv)][None].repeat(B, 0).astype(np.float32)
        elif kind == "unnormalised_k":
            # |k_t|^2 = c / beta_t with c ~ U(1, 2) per (b, t, key head): beta |k|^2 up to 2 for the value heads
            # whose beta is the largest of their group
            rf = Hv // Hk
            bmax = d["beta"].reshape(B, T, Hk, rf).max(-1)
            c = rng.uniform(1.0, 2.0, (B, T, Hk)).astype(np.float32)
            d["k"] = d["k"] * np.sqrt(c / bmax)[..., None]
            d["q"] = d["q"] * rng.uniform(0.5, 3.0, (B, T, Hk, 1)).astype(np.float32)
        elif kind == "big_state":
            d["state"] = (1e3 * rng.standard_normal((B, Hv, Dv, Dk))).astype(np.float32)
        else:
            raise ValueError(kind)
    for n in ("q", "k", "v", "g", "beta"):
        d[n] = O.quantize(np.ascontiguousarray(d[n], np.float32), in_dt)
    return d


KINDS = ["refbench", "special_gates", "unnormalised_k", "big_state"]
# (name, B, T, Hk, Hv, Dk, Dv): the reference bench's shape; two chunks and a half; Dk = 64 with a padded last chunk
SHAPES = [("refbench_shape", 1, 16, 8, 16, 128, 128), ("two_chunks", 1, 40, 2, 4, 128, 32), ("dk64_T24", 2, 24, 1, 2, 64, 16)]


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("in_dt", ["bf16", "f32"])
@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
def test_forward_value_range(gpu_lib, shape, kind, in_dt, vec):
    from swiftlm_amd import DFlashKernels as K

    name, B, T, Hk, Hv, Dk, Dv = shape
    d = draw(kind, 31 + len(name) + len(kind), B, T, Hk, Hv, Dk, Dv, in_dt, vec)
    y, s, tape = K.gated_delta_kernel_with_tape(*(dev(d[n], in_dt) for n in ("q", "k", "v", "g", "beta")), dev(d["state"]))
    torch.cuda.synchronize()
    yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], dtype=np.float64)
    assert_close_to_scale(host(s), sw, 1e-4, "state")
    assert_close_to_scale(host(tape), tw, 1e-4, "tape")
    assert_close_to_scale(host(y), yw, 1e-4 if in_dt == "f32" else 2e-2, "y")


@pytest.mark.parametrize("kind", ["refbench", "special_gates"])
@pytest.mark.parametrize("in_dt", ["bf16", "f32"])
def test_forward_value_range_masked(gpu_lib, kind, in_dt):
    """The reference bench's masked scalar-gate case (main.swift:551) on its own distribution."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 16, 8, 16, 128, 128
    d = draw(kind, 77, B, T, Hk, Hv, Dk, Dv, in_dt, False)
    mask = (np.random.default_rng(5).random((B, T)) < 0.6).astype(np.float32)
    mask[:, 0] = 1.0
    y, s, tape = K.gated_delta_kernel_with_tape(*(dev(d[n], in_dt) for n in ("q", "k", "v", "g", "beta")), dev(d["state"]),
                                                dev(mask))
    torch.cuda.synchronize()
    yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask, dtype=np.float64)
    assert_close_to_scale(host(s), sw, 1e-4, "state")
    assert_close_to_scale(host(tape), tw, 1e-4, "tape")
    assert_close_to_scale(host(y), yw, 1e-4 if in_dt == "f32" else 2e-2, "y")
    off = mask < 0.5
    assert np.all(host(y)[off] == 0) and np.all(host(tape)[off] == 0)


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("vec", [False, True], ids=["scalar_g", "vec_g"])
def test_replay_value_range(gpu_lib, shape, kind, vec):
    from swiftlm_amd import DFlashKernels as K

    name, B, T, Hk, Hv, Dk, Dv = shape
    d = draw(kind, 53 + len(name) + len(kind), B, T, Hk, Hv, Dk, Dv, "bf16", vec)
    rng = np.random.default_rng(9)
    scale = {"refbench": 0.1, "big_state": 1e3}.get(kind, 1.0)
    tape = (scale * rng.standard_normal((B, T, Hv, Dv))).astype(np.float32)
    for n in sorted({1, T // 2, T}):
        out = K.tape_replay_kernel(dev(tape[:, :n]), dev(d["k"][:, :n], "bf16"), dev(d["g"][:, :n], "bf16"), dev(d["state"]))
        torch.cuda.synchronize()
        want = O.tape_replay_ops(tape[:, :n], d["k"][:, :n], d["g"][:, :n], d["state"], dtype=np.float64)
        assert_close_to_scale(host(out), want, 1e-4, f"replayed state, n={n}")


def test_forward_then_replay_value_range_consistency(gpu_lib):
    """replay(tape from the forward, n) == forward on n tokens, on the reference bench's distribution."""
    from swiftlm_amd import DFlashKernels as K

    B, T, Hk, Hv, Dk, Dv = 1, 16, 8, 16, 128, 128
    d = draw("refbench", 91, B, T, Hk, Hv, Dk, Dv, "bf16", False)
    q, k, v, g, beta = (dev(d[n], "bf16") for n in ("q", "k", "v", "g", "beta"))
    s0 = dev(d["state"])
    _, s_full, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0)
    for n in (1, 5, 16):
        _, s_n, _ = K.gated_delta_kernel_with_tape(*(t[:, :n].contiguous() for t in (q, k, v, g, beta)), s0)
        rep = K.tape_replay_kernel(tape[:, :n], k[:, :n], g[:, :n], s0)
        assert_close_to_scale(host(rep), host(s_n), 1e-4, f"replay vs forward, n={n}")
