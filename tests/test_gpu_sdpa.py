"""GPU parity: block-causal batched GQA SDPA (HIP, through the C ABI) against the
CPU oracle, and at the long-context sizes against size-independent properties and
a float32 torch restatement of the same op.

Bar: bf16/f16 outputs within 2e-2 abs/rel; the float32
logsumexp is held to 2e-3 (its inputs are bf16 products accumulated in fp32)."""

import math

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

OUT_TOL = dict(rtol=2e-2, atol=2e-2)
LSE_TOL = dict(rtol=2e-3, atol=2e-3)


def host(t):
    return t.detach().float().cpu().numpy()


def torch_reference(q, k, v, scale, kv_len=None):
    """float32 restatement on the GPU for sizes the CPU oracle would take minutes on."""
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    outs, lses = [], []
    for b in range(B):
        n = N if kv_len is None else int(kv_len[b])
        kk = k[b, :, :n].float().repeat_interleave(Hq // Hk, dim=0)
        vv = v[b, :, :n].float().repeat_interleave(Hq // Hk, dim=0)
        s = torch.einsum("hmd,hnd->hmn", q[b].float() * scale, kk)
        vis = torch.arange(n, device=q.device)[None, :] <= (n - M + torch.arange(M, device=q.device))[:, None]
        s = s.masked_fill(~vis, float("-inf"))
        lses.append(torch.logsumexp(s, dim=-1))
        outs.append(torch.einsum("hmn,hnd->hmd", torch.softmax(s, dim=-1), vv))
    return torch.stack(outs), torch.stack(lses)


def gpu_inputs(seed, B, Hq, Hk, L, D, dtype=torch.bfloat16):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(B, Hq, 16, D, generator=g, device="cuda").to(dtype)
    k = torch.randn(B, Hk, L + 16, D, generator=g, device="cuda").to(dtype)
    v = torch.randn(B, Hk, L + 16, D, generator=g, device="cuda").to(dtype)
    return q, k, v


# (B, Hq, Hk, L, D)
SMALL = [
    (1, 16, 2, 0, 256),       # only the block itself: plain causal attention
    (1, 16, 2, 5, 256),
    (1, 16, 2, 100, 256),
    (2, 4, 2, 333, 128),      # group of 2
    (1, 32, 8, 512, 128),     # the reference bench's shape (DFlashKernelBench/main.swift:201-204)
    (1, 3, 3, 70, 128),       # no grouping, odd head count
    (1, 24, 2, 200, 128),     # group of 12: two workgroups per KV head
    (1, 16, 2, 1000, 256),
]


@pytest.mark.parametrize("cfg", SMALL, ids=[f"B{c[0]}_Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}" for c in SMALL])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_sdpa_matches_oracle_small(gpu_lib, cfg, dtype):
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D = cfg
    q, k, v = gpu_inputs(B * 1000 + L, B, Hq, Hk, L, D, dtype)
    scale = 1.0 / math.sqrt(D)
    out, lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    torch.cuda.synchronize()
    ow, lw = O.sdpa_block_causal(host(q), host(k), host(v), scale)
    assert out.dtype == dtype and out.shape == q.shape and lse.shape == (B, Hq, 16)
    np.testing.assert_allclose(host(out), ow, **OUT_TOL)
    np.testing.assert_allclose(host(lse), lw, **LSE_TOL)


def test_sdpa_config2_against_c_oracle(gpu_lib):
    """Benchmark configuration 2: Hq=16, Hkv=2, D=256, L=4096, scale 1/16."""
    from swiftlm_amd import DFlashKernels as K

    q, k, v = gpu_inputs(2, 1, 16, 2, 4096, 256)
    out, lse = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, return_lse=True)
    ow, lw = c_oracle.sdpa_block_causal(host(q), host(k), host(v), 1.0 / 16)
    np.testing.assert_allclose(host(out), ow, **OUT_TOL)
    np.testing.assert_allclose(host(lse), lw, **LSE_TOL)
    # without LSE the result is the same array
    assert torch.equal(K.batched_sdpa_2pass(q, k, v, 1.0 / 16), out)
    # inputs untouched, K/V taken as a view into a larger cache
    cache_k = torch.zeros(1, 2, 8192, 256, dtype=torch.bfloat16, device="cuda")
    cache_v = torch.zeros_like(cache_k)
    cache_k[:, :, :4112] = k
    cache_v[:, :, :4112] = v
    out2 = K.batched_sdpa_2pass(q, cache_k[:, :, :4112], cache_v[:, :, :4112], 1.0 / 16)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("cfg", [(1, 8, 1, 40000, 256), (1, 4, 1, 40000, 128), (1, 1, 1, 70000, 256)],
                         ids=lambda c: f"Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}")
def test_sdpa_single_kv_head_uses_every_split(gpu_lib, cfg):
    """One KV head and one batch: the key axis is cut into as many splits as the GPU has CUs (256 on the
    benchmark's GPU), so the combine kernel walks its partials in more than one pass, and with Hq = 1 most of
    a workgroup's query rows are absent.  Checked against a float32 restatement, logsumexp included."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D = cfg
    q, k, v = gpu_inputs(L + 11, B, Hq, Hk, L, D)
    scale = 1.0 / math.sqrt(D)
    out, lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    ow, lw = torch_reference(q, k, v, scale)
    np.testing.assert_allclose(host(out), host(ow), **OUT_TOL)
    np.testing.assert_allclose(host(lse), host(lw), **LSE_TOL)


@pytest.mark.parametrize("L", [32768, 40960, 102400])
def test_sdpa_long_context_properties(gpu_lib, L):
    """Benchmark configuration 3 sizes.  Properties that do not need a CPU pass: constant V gives
    constant O; the result matches a float32 restatement; appending hidden (future) keys
    changes nothing for the rows that cannot see them."""
    from swiftlm_amd import DFlashKernels as K

    q, k, v = gpu_inputs(L, 1, 16, 2, L, 256)
    out, lse = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, return_lse=True)
    ow, lw = torch_reference(q, k, v, 1.0 / 16)
    np.testing.assert_allclose(host(out), host(ow), **OUT_TOL)
    np.testing.assert_allclose(host(lse), host(lw), **LSE_TOL)
    const = K.batched_sdpa_2pass(q, k, torch.full_like(v, 0.75), 1.0 / 16)
    np.testing.assert_allclose(host(const), 0.75, rtol=1e-2)
    # row 0 sees keys 0..L only: changing the last 15 keys must not move it
    k2, v2 = k.clone(), v.clone()
    k2[:, :, L + 1:] = 3.0
    v2[:, :, L + 1:] = -5.0
    out2 = K.batched_sdpa_2pass(q, k2, v2, 1.0 / 16)
    assert torch.equal(out2[:, :, 0], out[:, :, 0])


def test_sdpa_ragged_batch(gpu_lib):
    """Benchmark configuration 3's ragged batch: 4 sequences with L ~ U[8K, 64K], one launch,
    per-sequence key counts on the device."""
    from swiftlm_amd import DFlashKernels as K

    rng = np.random.default_rng(0)
    Ls = rng.integers(8192, 65536, 4)
    Nmax = int(Ls.max()) + 16
    q, k, v = gpu_inputs(77, 4, 16, 2, Nmax - 16, 256)
    kv_len = torch.tensor([int(l) + 16 for l in Ls], dtype=torch.int32, device="cuda")
    out, lse = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, return_lse=True, kv_len=kv_len)
    ow, lw = torch_reference(q, k, v, 1.0 / 16, kv_len=kv_len.tolist())
    np.testing.assert_allclose(host(out), host(ow), **OUT_TOL)
    np.testing.assert_allclose(host(lse), host(lw), **LSE_TOL)
    # each sequence alone gives the same rows
    for b in (0, 3):
        n = int(kv_len[b])
        single = K.batched_sdpa_2pass(q[b:b + 1], k[b:b + 1, :, :n].contiguous(), v[b:b + 1, :, :n].contiguous(),
                                      1.0 / 16)
        np.testing.assert_allclose(host(single), host(out[b:b + 1]), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("cfg", [(1, 16, 2, 100, 256), (2, 4, 2, 333, 128), (1, 16, 2, 1003, 256)],
                         ids=["L100_D256", "B2_L333_D128", "L1003_odd_row_pitch"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_sdpa_additive_mask_matches_oracle(gpu_lib, cfg, dtype):
    """The masked partials kernel (DFlashKernels.swift:546-555): finite biases, dropped keys
    (-inf), a value at the lowest finite number of the type (still a usable key, :551), and one
    row with no usable key at all (zeros, :711)."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D = cfg
    N = L + 16
    q, k, v = gpu_inputs(B * 77 + L, B, Hq, Hk, L, D, dtype)
    g = torch.Generator(device="cuda").manual_seed(L)
    mask = torch.randn(B, Hq, 16, N, generator=g, device="cuda")
    drop = torch.rand(B, Hq, 16, N, generator=g, device="cuda") < 0.3
    mask = mask.masked_fill(drop, float("-inf"))
    mask[0, 0, 5, :] = float("-inf")                      # no usable key
    mask[0, 1, 2, :] = float("-inf")
    mask[0, 1, 2, 3] = torch.finfo(dtype).min             # only key 3, at the lowest finite value
    mask = mask.to(dtype)
    scale = 1.0 / math.sqrt(D)
    out, lse = K.batched_sdpa_2pass(q, k, v, scale, mask, return_lse=True)
    torch.cuda.synchronize()
    ow, lw = O.sdpa_block_causal(host(q), host(k), host(v), scale, host(mask).astype(np.float64))
    np.testing.assert_allclose(host(out), ow, **OUT_TOL)
    got_lse = host(lse)
    assert np.all(got_lse[0, 0, 5] == -np.inf) and np.all(host(out)[0, 0, 5] == 0)
    np.testing.assert_allclose(host(out)[0, 1, 2], host(v)[0, 0, 3], **OUT_TOL)      # all weight on key 3
    fin = np.isfinite(lw) & (np.abs(lw) < 1e30)
    np.testing.assert_allclose(got_lse[fin], lw[fin], **LSE_TOL)


def test_sdpa_broadcast_mask_and_zero_mask(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    q, k, v = gpu_inputs(11, 1, 16, 2, 200, 256)
    plain = K.batched_sdpa_2pass(q, k, v, 1.0 / 16)
    zero = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, torch.zeros(1, 1, 16, 216, device="cuda"))
    assert torch.equal(plain, zero)


def test_sdpa_unsupported_shapes_return_none(gpu_lib):
    """The reference's guards (DFlashKernels.swift:744-758): nil instead of an error."""
    from swiftlm_amd import DFlashKernels as K, DFlashUnsupported

    q, k, v = gpu_inputs(1, 1, 4, 2, 64, 128)
    assert K.batched_sdpa_2pass(q[:, :, :8], k, v, 0.1) is None                  # qLen != 16
    assert K.batched_sdpa_2pass(q.float(), k.float(), v.float(), 0.1) is None    # float32
    q64, k64, v64 = gpu_inputs(1, 1, 4, 2, 64, 64)
    assert K.batched_sdpa_2pass(q64, k64, v64, 0.1) is None                      # D = 64
    q3, _, _ = gpu_inputs(1, 1, 3, 2, 64, 128)
    assert K.batched_sdpa_2pass(q3, k, v, 0.1) is None                           # Hq % Hk != 0
    assert K.batched_sdpa_2pass(q[0], k[0], v[0], 0.1) is None                   # ndim != 4
    with pytest.raises(DFlashUnsupported):
        K.sdpa_fallback(q64, k64, v64, 0.1)


@pytest.mark.parametrize("cfg", [(1, 16, 2, 0, 256), (1, 16, 2, 7, 256), (2, 8, 2, 300, 128), (1, 16, 2, 4096, 256)],
                         ids=lambda c: f"B{c[0]}_Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}")
def test_sdpa_fused_append_equals_append_then_sdpa(gpu_lib, cfg):
    """The fused entry must give the bytes of `append, then attend`: same O and LSE, and the
    block's rows stored bit for bit at rows L .. L+15 of the cache, nothing else touched."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D = cfg
    q, k, v = gpu_inputs(L + 5, B, Hq, Hk, L, D)
    cap = L + 16 + 37
    kc = torch.full((B, Hk, cap, D), 3.0, dtype=torch.bfloat16, device="cuda")
    vc = torch.full((B, Hk, cap, D), -3.0, dtype=torch.bfloat16, device="cuda")
    kc[:, :, :L], vc[:, :, :L] = k[:, :, :L], v[:, :, :L]
    k_new, v_new = k[:, :, L:].contiguous(), v[:, :, L:].contiguous()
    scale = 1.0 / math.sqrt(D)
    want, want_lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    got, got_lse = K.batched_sdpa_2pass_append(q, kc, vc, k_new, v_new, scale, L + 16, return_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    assert torch.equal(kc[:, :, : L + 16], k) and torch.equal(vc[:, :, : L + 16], v)
    assert bool((kc[:, :, L + 16:] == 3.0).all()) and bool((vc[:, :, L + 16:] == -3.0).all())
    # and the next step reads them back from the cache
    again = K.batched_sdpa_2pass(q, kc[:, :, : L + 16], vc[:, :, : L + 16], scale)
    assert torch.equal(again, want)


def test_sdpa_fused_append_ragged(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, D, cap = 3, 16, 2, 256, 700
    Ls = [100, 333, 650]
    q, k, v = gpu_inputs(9, B, Hq, Hk, cap - 16, D)
    kc, vc = k.clone(), v.clone()
    k_new = torch.stack([k[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
    v_new = torch.stack([v[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
    for b in range(B):                                  # poison the rows the append must fill
        kc[b, :, Ls[b]:Ls[b] + 16] = 9.0
        vc[b, :, Ls[b]:Ls[b] + 16] = 9.0
    kv_len = torch.tensor([l + 16 for l in Ls], dtype=torch.int32, device="cuda")
    cache_len = torch.tensor(Ls, dtype=torch.int32, device="cuda")
    want = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, kv_len=kv_len)
    got = K.batched_sdpa_2pass_append(q, kc, vc, k_new, v_new, 1.0 / 16, cap, cache_len=cache_len)
    assert torch.equal(got, want)
    assert torch.equal(kc, k) and torch.equal(vc, v)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["f16", "bf16"])
def test_sdpa_partial_rows_do_not_overflow_f16(gpu_lib, dtype):
    """Scores that rise by just under the lazy-rescale threshold after the first tile make the
    unnormalised partial sums of a split large (2^7.9 x 224 keys x |V| = 2e5 here): the partial rows
    are stored normalised, so an f16 run still returns the exact answer (every V row is 4)."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, D, L = 1, 8, 1, 128, 32768
    N = L + 16
    q = torch.zeros(B, Hq, 16, D, dtype=dtype, device="cuda")
    q[..., 0] = 1.0
    k = torch.zeros(B, Hk, N, D, dtype=dtype, device="cuda")
    k[:, :, 32:, 0] = 7.9 / 1.4426950408889634
    v = torch.full((B, Hk, N, D), 4.0, dtype=dtype, device="cuda")
    out, lse = K.batched_sdpa_2pass(q, k, v, 1.0, return_lse=True)
    want, want_lse = torch_reference(q, k, v, 1.0)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    np.testing.assert_allclose(host(out), 4.0, rtol=1e-2)
    np.testing.assert_allclose(host(lse), host(want_lse), **LSE_TOL)


@pytest.mark.parametrize("cfg", SMALL + [(1, 16, 2, 4099, 256), (2, 8, 2, 2500, 128)],
                         ids=lambda c: f"B{c[0]}_Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}")
def test_sdpa_zero_mask_equals_plain_bitwise(gpu_lib, cfg):
    """The masked entry is another instantiation of the same kernel: with an all-zero mask it adds 0 to every score,
    so its result is the plain entry's to the bit; both are held to the oracle's tolerance where the oracle is
    affordable."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D = cfg
    q, k, v = gpu_inputs(L + 3, B, Hq, Hk, L, D)
    scale = 1.0 / math.sqrt(D)
    o_plain, l_plain = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    mask = torch.zeros(B, Hq, 16, L + 16, dtype=q.dtype, device="cuda")
    o_mask, l_mask = K.batched_sdpa_2pass(q, k, v, scale, mask, return_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(o_plain, o_mask)
    assert torch.equal(l_plain, l_mask)
    if L <= 1100:
        ow, lw = O.sdpa_block_causal(host(q), host(k), host(v), scale)
        np.testing.assert_allclose(host(o_plain), ow, **OUT_TOL)
        np.testing.assert_allclose(host(l_plain), lw, **LSE_TOL)
