"""GPU parity over seeded random shapes: the attention entry points (plain, ragged, fused append,
additive mask) and the GatedDelta forward / replay pair against the CPU oracle.  Shapes are drawn
from the awkward corners: head groups that do not fill a workgroup, contexts shorter than a tile,
lengths one off a tile or chunk boundary, every supported Dk, value-head dims that are not a
multiple of the row tile.  Tolerances are the ones of the dedicated tests."""

import math

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

TD = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16}


def host(t):
    return t.detach().float().cpu().numpy()


def dev(a, dt):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda", TD[dt])


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_attention_random_shapes(gpu_lib, seed):
    from swiftlm_amd import DFlashKernels as K

    rng = np.random.default_rng(seed)
    for it in range(25):
        D = int(rng.choice([128, 256]))
        Hk = int(rng.choice([1, 2, 3, 4]))
        Hq = Hk * int(rng.choice([1, 2, 3, 4, 7, 8, 9, 12]))
        B = int(rng.choice([1, 1, 2, 3]))
        L = int(rng.choice([0, 1, 15, 16, 17, 31, 33, 100, 257, 700, 1500]))
        dt = torch.bfloat16 if rng.random() < 0.7 else torch.float16
        mode = str(rng.choice(["plain", "ragged", "append", "mask"]))
        case = f"seed {seed} case {it}: {mode} B={B} Hq={Hq} Hk={Hk} L={L} D={D} {dt}"
        N = L + 16
        g = torch.Generator(device="cuda").manual_seed(int(rng.integers(1 << 30)))
        q = torch.randn(B, Hq, 16, D, generator=g, device="cuda").to(dt)
        k = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dt)
        v = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dt)
        scale = 1.0 / math.sqrt(D)
        if mode == "plain":
            out, lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
            ow, lw = O.sdpa_block_causal(host(q), host(k), host(v), scale)
        elif mode == "mask":
            m = torch.randn(B, Hq, 16, N, generator=g, device="cuda")
            m = m.masked_fill(torch.rand(B, Hq, 16, N, generator=g, device="cuda") < 0.2, float("-inf")).to(dt)
            out, lse = K.batched_sdpa_2pass(q, k, v, scale, m, return_lse=True)
            ow, lw = O.sdpa_block_causal(host(q), host(k), host(v), scale, host(m).astype(np.float64))
        elif mode == "ragged":
            lens = torch.tensor([int(rng.integers(16, N + 1)) for _ in range(B)], dtype=torch.int32, device="cuda")
            out, lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True, kv_len=lens)
            ow, lw = np.zeros((B, Hq, 16, D)), np.zeros((B, Hq, 16))
            for b in range(B):
                n = int(lens[b])
                o1, l1 = O.sdpa_block_causal(host(q)[b:b + 1], host(k)[b:b + 1, :, :n], host(v)[b:b + 1, :, :n], scale)
                ow[b], lw[b] = o1[0], l1[0]
        else:
            cap = N + int(rng.integers(0, 40))
            kc = torch.zeros(B, Hk, cap, D, dtype=dt, device="cuda")
            vc = torch.zeros_like(kc)
            clen = torch.tensor([int(rng.integers(0, L + 1)) for _ in range(B)], dtype=torch.int32, device="cuda")
            for b in range(B):
                c = int(clen[b])
                kc[b, :, :c], vc[b, :, :c] = k[b, :, :c], v[b, :, :c]
            kn = torch.randn(B, Hk, 16, D, generator=g, device="cuda").to(dt)
            vn = torch.randn(B, Hk, 16, D, generator=g, device="cuda").to(dt)
            out, lse = K.batched_sdpa_2pass_append(q, kc, vc, kn, vn, scale, N, return_lse=True, cache_len=clen)
            ow, lw = np.zeros((B, Hq, 16, D)), np.zeros((B, Hq, 16))
            for b in range(B):
                c = int(clen[b])
                kk = np.concatenate([host(k)[b:b + 1, :, :c], host(kn)[b:b + 1]], axis=2)
                vv = np.concatenate([host(v)[b:b + 1, :, :c], host(vn)[b:b + 1]], axis=2)
                o1, l1 = O.sdpa_block_causal(host(q)[b:b + 1], kk, vv, scale)
                ow[b], lw[b] = o1[0], l1[0]
                assert torch.equal(kc[b, :, c:c + 16], kn[b]) and torch.equal(vc[b, :, c:c + 16], vn[b]), case
        torch.cuda.synchronize()
        np.testing.assert_allclose(host(out), ow, rtol=2e-2, atol=2e-2, err_msg=case)
        fin = np.isfinite(lw)
        np.testing.assert_allclose(host(lse)[fin], lw[fin], rtol=2e-3, atol=2e-3, err_msg=case)
        assert np.all(host(lse)[~fin] == -np.inf), case


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_gated_delta_random_shapes(gpu_lib, seed):
    from swiftlm_amd import DFlashKernels as K

    rng = np.random.default_rng(seed)
    for it in range(30):
        Dk = int(rng.choice([32, 64, 96, 128, 160, 192, 224, 256]))
        Dv = int(rng.choice([8, 16, 24, 32, 48, 64, 128]))
        Hk = int(rng.choice([1, 2, 4]))
        Hv = Hk * int(rng.choice([1, 2, 3]))
        B = int(rng.choice([1, 1, 2]))
        T = int(rng.choice([1, 2, 5, 15, 16, 17, 31, 33, 48]))
        vec = bool(rng.random() < 0.35)
        in_dt = str(rng.choice(["f32", "bf16", "bf16", "f16"]))
        masked = bool(rng.random() < 0.4)
        case = f"seed {seed} case {it}: B={B} T={T} Hk={Hk} Hv={Hv} Dk={Dk} Dv={Dv} vec={vec} {in_dt} masked={masked}"
        d = O.make_gdn_inputs(int(rng.integers(1 << 30)), B, T, Hk, Hv, Dk, Dv, in_dtype=in_dt, vec_gate=vec)
        mask = (rng.random((B, T)) < 0.6).astype(np.float32) if masked else None
        args = [dev(d[n], in_dt) for n in ("q", "k", "v", "g", "beta")]
        m_d = None if mask is None else dev(mask, "f32")
        y, s, tape = K.gated_delta_kernel_with_tape(*args, dev(d["state"], "f32"), m_d)
        torch.cuda.synchronize()
        yw, sw, tw = O.gated_delta_ops_with_tape(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], mask,
                                                  dtype=np.float64)
        np.testing.assert_allclose(host(s), sw, rtol=1e-4, atol=2e-6, err_msg=case)
        np.testing.assert_allclose(host(tape), tw, rtol=1e-4, atol=2e-6, err_msg=case)
        ytol = dict(rtol=1e-4, atol=1e-5) if in_dt == "f32" else dict(rtol=2e-2, atol=2e-2)
        np.testing.assert_allclose(host(y), yw, err_msg=case, **ytol)
        n = int(rng.integers(0, T + 1))
        rep = K.tape_replay_kernel(tape[:, :n].contiguous(), args[1][:, :n].contiguous(), args[3][:, :n].contiguous(),
                                   dev(d["state"], "f32"), None if m_d is None else m_d[:, :n].contiguous())
        torch.cuda.synchronize()
        rw = O.tape_replay_ops(host(tape)[:, :n], d["k"][:, :n], d["g"][:, :n], d["state"],
                               None if mask is None else mask[:, :n], dtype=np.float64)
        np.testing.assert_allclose(host(rep), rw, rtol=1e-4, atol=2e-6, err_msg=case)
