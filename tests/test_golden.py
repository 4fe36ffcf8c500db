"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py from the
oracle): the oracles must keep reproducing them on the CPU, and the HIP kernels must match them
on the GPU."""

import glob
import os

import numpy as np
import pytest

from oracle import c_oracle
from oracle import dflash_oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return dict(np.load(os.path.join(GOLD, name), allow_pickle=False))


def gdn_files():
    return sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLD, "gdn_*.npz")))


def sdpa_files():
    return sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLD, "sdpa_*.npz")))


@pytest.mark.parametrize("name", gdn_files())
def test_oracles_reproduce_gdn_fixture(name):
    f = load(name)
    mask = f["mask"] if f["mask"].size else None
    n = int(f["n_accept"])
    for impl in ("numpy", "c"):
        if impl == "numpy":
            y, S, tape = O.gated_delta_ops_with_tape(f["q"], f["k"], f["v"], f["g"], f["beta"], f["state"], mask)
            rep = O.tape_replay_ops(f["tape"][:, :n], f["k"][:, :n], f["g"][:, :n], f["state"],
                                    None if mask is None else mask[:, :n])
        else:
            y, S, tape = c_oracle.gated_delta(f["q"], f["k"], f["v"], f["g"], f["beta"], f["state"], mask)
            rep = c_oracle.tape_replay(f["tape"][:, :n], f["k"][:, :n], f["g"][:, :n], f["state"],
                                       None if mask is None else mask[:, :n])
        np.testing.assert_allclose(y, f["y"], rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(S, f["state_out"], rtol=1e-4, atol=1e-6)
        np.testing.assert_allclose(tape, f["tape"], rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(rep, f["replayed"], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("name", sdpa_files())
def test_oracles_reproduce_sdpa_fixture(name):
    f = load(name)
    o, lse = c_oracle.sdpa_block_causal(f["q"], f["k"], f["v"], float(f["scale"]))
    np.testing.assert_allclose(o, f["out"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(lse, f["lse"], rtol=1e-5, atol=1e-5)


def test_oracle_reproduces_accept_fixture():
    cases = load("accept_commit_cases.npz")["cases"]
    for row in cases:
        staged, drafted, posterior, start = int(row[0]), row[1:16], row[16:32], int(row[32])
        r = O.accept_commit(staged, drafted, posterior, start)
        assert [r["acceptance_len"], r["commit_count"], r["staged_next"], r["start"]] == list(row[33:37])
        assert c_oracle.match_acceptance_length(drafted, posterior[:15]) == row[33]


# ------------------------------------------------------------------ GPU ------


def _dev(a, dt):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", dt)


@pytest.mark.gpu
@pytest.mark.parametrize("name", gdn_files())
def test_hip_matches_gdn_fixture(gpu_lib, name):
    import torch

    from swiftlm_amd import DFlashKernels as K

    f = load(name)
    dt = {"f32": torch.float32, "bf16": torch.bfloat16}[str(f["in_dtype"])]
    mask = _dev(f["mask"], torch.float32) if f["mask"].size else None
    n = int(f["n_accept"])
    q, k, v, g, beta = (_dev(f[x], dt) for x in ("q", "k", "v", "g", "beta"))
    s0 = _dev(f["state"], torch.float32)
    y, S, tape = K.gated_delta_kernel_with_tape(q, k, v, g, beta, s0, mask)
    rep = K.tape_replay_kernel(tape[:, :n], k[:, :n], g[:, :n], s0, None if mask is None else mask[:, :n])
    h = lambda t: t.float().cpu().numpy()
    ytol = dict(rtol=1e-4, atol=1e-5) if dt == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    np.testing.assert_allclose(h(y), f["y"], **ytol)
    np.testing.assert_allclose(h(S), f["state_out"], rtol=1e-4, atol=1e-6)
    np.testing.assert_allclose(h(tape), f["tape"], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(h(rep), f["replayed"], rtol=1e-4, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sdpa_files())
def test_hip_matches_sdpa_fixture(gpu_lib, name):
    import torch

    from swiftlm_amd import DFlashKernels as K

    f = load(name)
    out, lse = K.batched_sdpa_2pass(_dev(f["q"], torch.bfloat16), _dev(f["k"], torch.bfloat16),
                                    _dev(f["v"], torch.bfloat16), float(f["scale"]), return_lse=True)
    np.testing.assert_allclose(out.float().cpu().numpy(), f["out"], rtol=2e-2, atol=2e-2)
    np.testing.assert_allclose(lse.cpu().numpy(), f["lse"], rtol=2e-3, atol=2e-3)


@pytest.mark.gpu
def test_hip_matches_accept_fixture(gpu_lib):
    import torch

    from swiftlm_amd import DFlashRuntime as R

    for row in load("accept_commit_cases.npz")["cases"]:
        r = R.accept_commit(torch.from_numpy(row[0:16]).cuda(), torch.from_numpy(row[16:32]).cuda(), int(row[32]))
        assert [r.acceptance_len, r.commit_count, r.staged_first_next, r.start] == list(row[33:37])


# ---- fixtures of the ops next to the verify path ----

def test_oracles_reproduce_new_fixtures():
    f = load("preops_gdn_bf16.npz")
    B, T, Hk, Hv, Dk, Dv, K = [int(x) for x in f["dims"]]
    o = O.gdn_prepare(f["x"], f["conv_state"], f["conv_weight"], f["a"], f["b"], f["a_log"], f["dt_bias"], Hk, Hv, Dk, Dv,
                      q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    for k, v in o.items():
        np.testing.assert_allclose(v, f["out_" + k], rtol=1e-6, atol=1e-7, err_msg=k)
    np.testing.assert_allclose(O.gdn_finish(o["v"], f["gate"], f["norm_weight"], 1e-6), f["out_finish"], rtol=1e-6, atol=1e-7)
    g = load("greedy_tokens_bf16.npz")
    mask = O.build_suppress_token_mask(g["logits"].shape[1], g["suppress_ids"].tolist())
    np.testing.assert_array_equal(O.greedy_tokens_with_mask(g["logits"], mask, dtype="bf16"), g["tokens_masked"])
    np.testing.assert_array_equal(O.greedy_tokens_with_mask(g["logits"], None, dtype="bf16"), g["tokens_plain"])
    assert g["tokens_masked"][0] != 7 and g["tokens_plain"][0] == 7 and g["tokens_plain"][1] == 50
    m = load("masked_sdpa_d128.npz")
    o2, lse = O.sdpa_block_causal(m["q"], m["k"], m["v"], float(m["scale"]), m["mask"].astype(np.float64))
    np.testing.assert_allclose(o2, m["out"], rtol=1e-5, atol=1e-6)
    assert np.all(m["out"][0, 0, 3] == 0) and m["lse"][0, 0, 3] == -np.inf


@pytest.mark.gpu
def test_hip_matches_new_fixtures(gpu_lib):
    import torch

    from swiftlm_amd import DFlashKernels as K, DFlashRuntime as R

    bf = torch.bfloat16
    f = load("preops_gdn_bf16.npz")
    B, T, Hk, Hv, Dk, Dv, Kc = [int(x) for x in f["dims"]]
    got = K.gdn_prepare(_dev(f["x"], bf), _dev(f["conv_state"], bf), _dev(f["conv_weight"], bf), _dev(f["a"], bf),
                        _dev(f["b"], bf), _dev(f["a_log"], torch.float32), _dev(f["dt_bias"], torch.float32),
                        Hk, Hv, Dk, Dv, q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    for name, t in zip(("q", "k", "v", "g", "beta"), got[:5]):
        np.testing.assert_allclose(t.float().cpu().numpy(), f["out_" + name], rtol=2e-2, atol=2e-2, err_msg=name)
    np.testing.assert_array_equal(got[5].float().cpu().numpy(), f["out_conv_state"])
    fin = K.gdn_finish(_dev(f["out_v"], bf), _dev(f["gate"], bf), _dev(f["norm_weight"], bf), 1e-6)
    np.testing.assert_allclose(fin.float().cpu().numpy(),
                               O.gdn_finish(O.round_to_bf16(f["out_v"]), f["gate"], f["norm_weight"], 1e-6), rtol=2e-2, atol=2e-2)
    g = load("greedy_tokens_bf16.npz")
    V = g["logits"].shape[1]
    mask = R.build_suppress_token_mask(V, g["suppress_ids"].tolist())
    lg = _dev(g["logits"], bf)
    np.testing.assert_array_equal(R.greedy_tokens_with_mask(lg, mask).cpu().numpy().astype(np.uint32), g["tokens_masked"])
    np.testing.assert_array_equal(R.greedy_tokens_with_mask(lg, None).cpu().numpy().astype(np.uint32), g["tokens_plain"])
    m = load("masked_sdpa_d128.npz")
    out, lse = K.batched_sdpa_2pass(_dev(m["q"], bf), _dev(m["k"], bf), _dev(m["v"], bf), float(m["scale"]),
                                    _dev(m["mask"], bf), return_lse=True)
    np.testing.assert_allclose(out.float().cpu().numpy(), m["out"], rtol=2e-2, atol=2e-2)
    fin_rows = np.isfinite(m["lse"])
    np.testing.assert_allclose(lse.cpu().numpy()[fin_rows], m["lse"][fin_rows], rtol=2e-3, atol=2e-3)
    assert lse.cpu().numpy()[0, 0, 3] == -np.inf
