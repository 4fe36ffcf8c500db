#!/usr/bin/env python3
"""Writes the small seeded fixtures under tests/golden/ from the CPU oracle.

The reference ships no golden vectors for this path (its dumps are git-ignored and need
model weights), so these pin the ORACLE's behaviour over time and give the GPU tests
fixed inputs with expected outputs; they are not vectors taken from the reference.
Run from the repository root:  python tests/golden/make_golden.py
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import dflash_oracle as O  # noqa: E402


def gdn_fixture(name, seed, B, T, Hk, Hv, Dk, Dv, in_dtype, vec, masked, n_accept):
    d = O.make_gdn_inputs(seed, B, T, Hk, Hv, Dk, Dv, in_dtype=in_dtype, vec_gate=vec)
    mask = None
    if masked:
        mask = (np.random.default_rng(seed + 1).random((B, T)) < 0.6).astype(np.float32)
        mask[:, 0] = 1
    y, S, tape = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask,
                                             dtype=np.float64)
    tape32 = tape.astype(np.float32)
    replayed = O.tape_replay_ops(tape32[:, :n_accept], d["k"][:, :n_accept], d["g"][:, :n_accept], d["state"],
                                 None if mask is None else mask[:, :n_accept], dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, name), in_dtype=in_dtype, n_accept=n_accept,
                        mask=np.zeros(0) if mask is None else mask, **d,
                        y=y.astype(np.float32), state_out=S.astype(np.float32), tape=tape32,
                        replayed=replayed.astype(np.float32))


def sdpa_fixture(name, seed, B, Hq, Hk, L, D, scale):
    q, k, v = O.make_sdpa_inputs(seed, B, Hq, Hk, 16, L, D)
    o, lse = O.sdpa_block_causal(q, k, v, scale)
    np.savez_compressed(os.path.join(HERE, name), q=q, k=k, v=v, scale=scale, out=o.astype(np.float32),
                        lse=lse.astype(np.float32))


def accept_fixture(name, seed, n_cases=64):
    rng = np.random.default_rng(seed)
    rows = []
    for _ in range(n_cases):
        V = 16
        staged = int(rng.integers(0, 50000))
        drafted = rng.integers(0, 4, V - 1)
        posterior = rng.integers(0, 4, V)
        cut = int(rng.integers(0, V))
        posterior[:cut] = drafted[:cut] if cut < V else posterior[:cut]
        start = int(rng.integers(0, 100000))
        r = O.accept_commit(staged, drafted, posterior, start)
        rows.append(np.concatenate([[staged], drafted, posterior, [start, r["acceptance_len"], r["commit_count"],
                                                                     r["staged_next"], r["start"]]]))
    np.savez_compressed(os.path.join(HERE, name), cases=np.array(rows, dtype=np.int64))


def preops_fixture(name, seed, B, T, Hk, Hv, Dk, Dv, K):
    """bf16-representable inputs of the GatedDelta pre/post-ops and their float64 results."""
    rng = np.random.default_rng(seed)
    C = 2 * Hk * Dk + Hv * Dv
    r = lambda a: O.round_to_bf16(a.astype(np.float32))
    d = dict(x=r(rng.standard_normal((B, T, C))), conv_state=r(rng.standard_normal((B, K - 1, C))),
             conv_weight=r(0.5 * rng.standard_normal((C, K))), a=r(2 * rng.standard_normal((B, T, Hv))),
             b=r(2 * rng.standard_normal((B, T, Hv))), a_log=(0.5 * rng.standard_normal(Hv)).astype(np.float32),
             dt_bias=rng.standard_normal(Hv).astype(np.float32), gate=r(2 * rng.standard_normal((B, T, Hv, Dv))),
             norm_weight=r(1 + 0.1 * rng.standard_normal(Dv)))
    o = O.gdn_prepare(d["x"], d["conv_state"], d["conv_weight"], d["a"], d["b"], d["a_log"], d["dt_bias"], Hk, Hv, Dk, Dv,
                      q_scale=1.0 / Dk, k_scale=Dk ** -0.5)
    fin = O.gdn_finish(o["v"], d["gate"], d["norm_weight"], 1e-6)        # the post-op applied to v as a stand-in for y
    np.savez_compressed(os.path.join(HERE, name), dims=np.array([B, T, Hk, Hv, Dk, Dv, K]), **d,
                        **{"out_" + k: v.astype(np.float32) for k, v in o.items()}, out_finish=fin.astype(np.float32))


def greedy_fixture(name, seed, T, V):
    rng = np.random.default_rng(seed)
    logits = O.round_to_bf16((4 * rng.standard_normal((T, V))).astype(np.float32))
    ids = [0, 7, V - 1, V + 5] + list(range(100, 140))
    logits[0, 7] = 64.0                 # the unmasked winner is suppressed
    logits[1, 50] = logits[1, 900] = 63.0   # a tie: the lower index wins
    mask = O.build_suppress_token_mask(V, ids)
    np.savez_compressed(os.path.join(HERE, name), logits=logits, suppress_ids=np.array(ids),
                        tokens_masked=O.greedy_tokens_with_mask(logits, mask, dtype="bf16"),
                        tokens_plain=O.greedy_tokens_with_mask(logits, None, dtype="bf16"))


def sdpa_masked_fixture(name, seed, B, Hq, Hk, L, D, scale):
    q, k, v = O.make_sdpa_inputs(seed, B, Hq, Hk, 16, L, D)
    rng = np.random.default_rng(seed + 1)
    N = L + 16
    mask = O.round_to_bf16(rng.standard_normal((B, Hq, 16, N)).astype(np.float32))
    mask[rng.random((B, Hq, 16, N)) < 0.25] = -np.inf
    mask[0, 0, 3, :] = -np.inf          # a row without usable keys: zeros
    o, lse = O.sdpa_block_causal(q, k, v, scale, mask.astype(np.float64))
    np.savez_compressed(os.path.join(HERE, name), q=q, k=k, v=v, mask=mask, scale=scale, out=o.astype(np.float32),
                        lse=lse.astype(np.float32))


if __name__ == "__main__":
    # benchmark configuration 0 (fp32, the reference's CPU-runnable case), n ~ U{1..8} drawn with the seed
    gdn_fixture("gdn_config0_f32.npz", 0, 1, 8, 4, 8, 64, 64, "f32", False, False,
                O.draw_accepted(np.random.default_rng(0), 8, "uniform"))
    # a slice of the Qwen3-Next shape (4 of 32 value heads), bf16 inputs, n ~ Geometric(0.25)
    gdn_fixture("gdn_qwen3next_slice_bf16.npz", 1, 1, 16, 2, 4, 128, 128, "bf16", False, False,
                O.draw_accepted(np.random.default_rng(1), 16, "geometric"))
    gdn_fixture("gdn_vecgate_masked_bf16.npz", 2, 2, 6, 2, 4, 64, 32, "bf16", True, True, 4)
    sdpa_fixture("sdpa_small_d256.npz", 3, 1, 16, 2, 200, 256, 1.0 / 16)
    sdpa_fixture("sdpa_small_d128.npz", 4, 2, 8, 2, 77, 128, 1.0 / np.sqrt(128))
    accept_fixture("accept_commit_cases.npz", 5)
    preops_fixture("preops_gdn_bf16.npz", 6, 1, 6, 2, 4, 64, 64, 4)
    greedy_fixture("greedy_tokens_bf16.npz", 7, 16, 5000)
    sdpa_masked_fixture("masked_sdpa_d128.npz", 8, 1, 4, 2, 60, 128, 1.0 / np.sqrt(128))
    print("wrote", sorted(f for f in os.listdir(HERE) if f.endswith(".npz")))
