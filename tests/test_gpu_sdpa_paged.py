"""GPU parity: the block-causal attention over a PAGED K/V cache, through the C ABI.

The reference's cache is dense (batchedSDPA2Pass, DFlashKernels.swift:737-743), so the paged
entry is pinned three ways: bit for bit against the dense entry on the gathered cache (same
arithmetic in the same order, only the addresses differ), against the CPU oracle on the
gathered cache (bf16/f16 outputs within 2e-2 abs/rel, logsumexp within 2e-3), and, for the
fused append, by reading the pool back: the block's rows land in the pages the table names,
bit for bit, and nothing else changes."""

import math

import numpy as np
import pytest
import torch

from oracle import dflash_oracle as O

pytestmark = pytest.mark.gpu

OUT_TOL = dict(rtol=2e-2, atol=2e-2)
LSE_TOL = dict(rtol=2e-3, atol=2e-3)


def host(t):
    return t.detach().float().cpu().numpy()


def torch_reference(q, k, v, scale, kv_len):
    """float32 restatement on the GPU over the first kv_len[b] keys of each sequence."""
    B, Hq, M, D = q.shape
    Hk = k.shape[1]
    outs, lses = [], []
    for b in range(B):
        n = int(kv_len[b])
        kk = k[b, :, :n].float().repeat_interleave(Hq // Hk, dim=0)
        vv = v[b, :, :n].float().repeat_interleave(Hq // Hk, dim=0)
        s = torch.einsum("hmd,hnd->hmn", q[b].float() * scale, kk)
        vis = torch.arange(n, device=q.device)[None, :] <= (n - M + torch.arange(M, device=q.device))[:, None]
        s = s.masked_fill(~vis, float("-inf"))
        lses.append(torch.logsumexp(s, dim=-1))
        outs.append(torch.einsum("hmn,hnd->hmd", torch.softmax(s, dim=-1), vv))
    return torch.stack(outs), torch.stack(lses)


def paged_case(seed, B, Hq, Hk, lengths, D, page_size, dtype=torch.bfloat16, spare_pages=3, head_pad=0, page_pad=0):
    """Dense K/V per sequence plus a pool that holds them under a shuffled page table.
    lengths: keys per sequence, block included.  head_pad / page_pad add unused elements to the
    pool's head and page pitches."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    N = max(lengths)
    q = torch.randn(B, Hq, 16, D, generator=g, device="cuda").to(dtype)
    k = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dtype)
    v = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dtype)
    pages_per_seq = (N + page_size - 1) // page_size
    num_pages = B * pages_per_seq + spare_pages
    perm = torch.randperm(num_pages, generator=torch.Generator().manual_seed(seed))[: B * pages_per_seq]
    table = perm.view(B, pages_per_seq).to(torch.int32).cuda()
    head_pitch = page_size * D + head_pad
    page_pitch = Hk * head_pitch + page_pad
    store_k = torch.full((num_pages * page_pitch,), 7.0, dtype=dtype, device="cuda")
    store_v = torch.full((num_pages * page_pitch,), -7.0, dtype=dtype, device="cuda")
    k_pool = store_k.as_strided((num_pages, Hk, page_size, D), (page_pitch, head_pitch, D, 1))
    v_pool = store_v.as_strided((num_pages, Hk, page_size, D), (page_pitch, head_pitch, D, 1))
    for b in range(B):
        for p in range(pages_per_seq):
            lo, hi = p * page_size, min((p + 1) * page_size, N)
            k_pool[table[b, p], :, : hi - lo] = k[b, :, lo:hi]
            v_pool[table[b, p], :, : hi - lo] = v[b, :, lo:hi]
    return q, k, v, k_pool, v_pool, table


# (B, Hq, Hk, L, D, page_size)
CASES = [
    (1, 16, 2, 0, 256, 32),        # only the block
    (1, 16, 2, 5, 256, 32),
    (1, 16, 2, 100, 256, 64),
    (2, 4, 2, 333, 128, 32),
    (1, 32, 8, 512, 128, 128),
    (1, 3, 3, 70, 128, 32),
    (1, 24, 2, 200, 128, 64),      # two workgroups per KV head
    (1, 16, 2, 1000, 256, 256),
    (1, 16, 2, 4099, 256, 32),     # many pages per workgroup
    (1, 16, 2, 4099, 256, 1024),   # one page spans several workgroups
]


@pytest.mark.parametrize("cfg", CASES, ids=lambda c: f"B{c[0]}_Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}_P{c[5]}")
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_paged_equals_dense_and_oracle(gpu_lib, cfg, dtype):
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D, P = cfg
    N = L + 16
    q, k, v, k_pool, v_pool, table = paged_case(L + P, B, Hq, Hk, [N] * B, D, P, dtype)
    scale = 1.0 / math.sqrt(D)
    want, want_lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, N, return_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    if N <= 1100:                                  # the CPU oracle on the gathered cache
        kd = O.gather_pages(host(k_pool), table.cpu().numpy(), N)
        vd = O.gather_pages(host(v_pool), table.cpu().numpy(), N)
        assert np.array_equal(kd, host(k)) and np.array_equal(vd, host(v))
        ref, ref_lse = O.sdpa_block_causal(host(q), kd, vd, scale)
        np.testing.assert_allclose(host(got), ref, **OUT_TOL)
        np.testing.assert_allclose(host(got_lse), ref_lse, **LSE_TOL)


def test_paged_padded_pitches_and_ragged_lengths(gpu_lib):
    """Pool pitches larger than the packed ones, and per-sequence lengths read on the device."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, D, P = 3, 16, 2, 256, 64
    lens = [116, 349, 666]
    q, k, v, k_pool, v_pool, table = paged_case(3, B, Hq, Hk, lens, D, P, head_pad=64, page_pad=128)
    kv_len = torch.tensor(lens, dtype=torch.int32, device="cuda")
    want = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, kv_len=kv_len)
    got = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, 1.0 / 16, max(lens), lengths=kv_len)
    assert torch.equal(got, want)
    for b in range(B):                             # each sequence against the oracle on its own keys
        kd = O.gather_pages(host(k_pool), table.cpu().numpy()[b:b + 1], lens[b])
        vd = O.gather_pages(host(v_pool), table.cpu().numpy()[b:b + 1], lens[b])
        ref, _ = O.sdpa_block_causal(host(q[b:b + 1]), kd, vd, 1.0 / 16)
        np.testing.assert_allclose(host(got[b:b + 1]), ref, **OUT_TOL)


@pytest.mark.parametrize("cfg", [(1, 16, 2, 0, 256, 32), (1, 16, 2, 7, 256, 32), (1, 16, 2, 25, 256, 32), (2, 8, 2, 300, 128, 64),
                                 (1, 16, 2, 4090, 256, 256)],
                         ids=lambda c: f"B{c[0]}_Hq{c[1]}_Hk{c[2]}_L{c[3]}_D{c[4]}_P{c[5]}")
def test_paged_fused_append(gpu_lib, cfg):
    """With k_new / v_new the paged entry equals the dense append entry, and the block's rows are
    stored into the pages that hold keys L .. L+15 (two pages when the block straddles a boundary:
    L = 25 with 32-key pages, L = 4090 with 256-key pages), everything else untouched."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D, P = cfg
    N = L + 16
    q, k, v, k_pool, v_pool, table = paged_case(L + 11, B, Hq, Hk, [N] * B, D, P)
    k_new, v_new = k[:, :, L:].contiguous(), v[:, :, L:].contiguous()
    full_k, full_v = k_pool.clone(), v_pool.clone()          # the pool as it must look afterwards
    tb = table.cpu().numpy()
    for b in range(B):                                       # poison the rows the append must fill
        for n in range(L, N):
            k_pool[tb[b, n // P], :, n % P] = 5.0
            v_pool[tb[b, n // P], :, n % P] = 5.0
    scale = 1.0 / math.sqrt(D)
    want, want_lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, N, k_new=k_new, v_new=v_new, return_lse=True)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    assert torch.equal(k_pool, full_k) and torch.equal(v_pool, full_v)
    # the next call finds the rows in the pages
    again = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, N)
    assert torch.equal(again, want)


def test_paged_fused_append_ragged_device_lengths(gpu_lib):
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, D, P = 3, 16, 2, 256, 128
    Ls = [100, 333, 650]
    lens = [l + 16 for l in Ls]
    q, k, v, k_pool, v_pool, table = paged_case(21, B, Hq, Hk, lens, D, P)
    k_new = torch.stack([k[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
    v_new = torch.stack([v[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
    full_k, full_v = k_pool.clone(), v_pool.clone()
    tb = table.cpu().numpy()
    for b in range(B):
        for n in range(Ls[b], lens[b]):
            k_pool[tb[b, n // P], :, n % P] = 9.0
            v_pool[tb[b, n // P], :, n % P] = 9.0
    kv_len = torch.tensor(lens, dtype=torch.int32, device="cuda")
    cache_len = torch.tensor(Ls, dtype=torch.int32, device="cuda")
    want = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, kv_len=kv_len)
    got = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, 1.0 / 16, max(lens), k_new=k_new, v_new=v_new, lengths=cache_len)
    assert torch.equal(got, want)
    # rows beyond a sequence's own length in its last page are not compared: they were never defined
    for b in range(B):
        for n in range(lens[b]):
            pg, r = tb[b, n // P], n % P
            assert torch.equal(k_pool[pg, :, r], full_k[pg, :, r]) and torch.equal(v_pool[pg, :, r], full_v[pg, :, r])


def test_paged_long_context_equals_dense(gpu_lib):
    """The benchmark's context length, 256-key pages in a shuffled pool."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D, P = 1, 16, 2, 32768, 256, 256
    q, k, v, k_pool, v_pool, table = paged_case(2, B, Hq, Hk, [L + 16], D, P)
    want, want_lse = K.batched_sdpa_2pass(q, k, v, 1.0 / 16, return_lse=True)
    got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, 1.0 / 16, L + 16, return_lse=True)
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)


def test_paged_many_tiles_per_workgroup_equals_dense(gpu_lib):
    """A batch wide enough that the key axis is split only 8 ways: every workgroup walks 150 tiles, so the
    producers' per-lane store of page entries (64 tiles a batch) is refilled twice."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D, P = 16, 2, 2, 38400, 128, 64
    q, k, v, k_pool, v_pool, table = paged_case(6, B, Hq, Hk, [L + 16] * B, D, P)
    scale = 1.0 / math.sqrt(D)
    want, want_lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True)
    got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, L + 16, return_lse=True)
    assert torch.equal(got, want) and torch.equal(got_lse, want_lse)
    # and the dense result itself against plain fp32 attention on one sequence
    b = 5
    s = torch.einsum("hmd,hnd->hmn", q[b].float() * scale, k[b].float())
    n = L + 16
    vis = torch.arange(n, device="cuda")[None, :] <= (n - 16 + torch.arange(16, device="cuda"))[:, None]
    ref = torch.einsum("hmn,hnd->hmd", torch.softmax(s.masked_fill(~vis, float("-inf")), -1), v[b].float())
    np.testing.assert_allclose(host(got[b]), host(ref), rtol=2e-2, atol=2e-2)


def test_paged_out_of_range_table_entries_stay_inside_the_pool(gpu_lib):
    """Entries outside [0, num_pages) are clamped on the device: the call completes and equals the
    call with the clamped table."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, L, D, P = 1, 16, 2, 200, 256, 32
    q, k, v, k_pool, v_pool, table = paged_case(4, B, Hq, Hk, [L + 16], D, P)
    bad = table.clone()
    bad[0, 1] = 10 ** 6
    bad[0, 2] = -5
    clamped = bad.clamp(0, k_pool.shape[0] - 1)
    got = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, bad, 1.0 / 16, L + 16)
    want = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, clamped, 1.0 / 16, L + 16)
    torch.cuda.synchronize()
    assert torch.equal(got, want)


def test_paged_rejects_what_it_does_not_take(gpu_lib):
    from swiftlm_amd import DFlashKernels as K
    from swiftlm_amd._lib import DFlashError

    q, k, v, k_pool, v_pool, table = paged_case(5, 1, 16, 2, [116], 256, 32)
    # page size below the tile, or not a power of two: unsupported, not an error
    small = k_pool[:, :, :16]
    assert K.batched_sdpa_2pass_paged(q, small.contiguous(), v_pool[:, :, :16].contiguous(), table, 1.0 / 16, 48) is None
    k48 = torch.zeros(4, 2, 48, 256, dtype=torch.bfloat16, device="cuda")
    assert K.batched_sdpa_2pass_paged(q, k48, k48.clone(), table, 1.0 / 16, 116) is None
    # a table that does not cover N
    with pytest.raises(DFlashError):
        K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table[:, :2].contiguous(), 1.0 / 16, 116)
    with pytest.raises(DFlashError):
        K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table.long(), 1.0 / 16, 116)
    # the same through the C ABI: a row pitch of 2 entries (64 keys) cannot hold 116 keys
    import ctypes as C
    from swiftlm_amd import _lib
    ws = torch.empty(int(gpu_lib.dflash_sdpa_workspace_bytes(1, 16, 2, 16, 116, 256)), dtype=torch.uint8, device="cuda")
    out = torch.empty_like(q)
    p = lambda t: C.c_void_p(t.data_ptr())
    rc = gpu_lib.dflash_sdpa_block_causal_paged(
        None, p(q), p(k_pool), p(v_pool), p(table), 2, 32, k_pool.shape[0], k_pool.stride(0), k_pool.stride(1), None, None,
        p(out), None, _lib.BF16, 1.0 / 16, 1, 16, 2, 16, 116, 256, None, p(ws), ws.numel())
    assert rc == _lib.INVALID
    rc = gpu_lib.dflash_sdpa_block_causal_paged(      # k_new without v_new
        None, p(q), p(k_pool), p(v_pool), p(table), 4, 32, k_pool.shape[0], k_pool.stride(0), k_pool.stride(1), p(q), None,
        p(out), None, _lib.BF16, 1.0 / 16, 1, 16, 2, 16, 116, 256, None, p(ws), ws.numel())
    assert rc == _lib.INVALID


@pytest.mark.parametrize("seed", [1, 2])
def test_paged_random_shapes(gpu_lib, seed):
    """Seeded random shapes, page sizes and ragged lengths, with and without the fused append:
    bit-identical to the dense entries, and within tolerance of the oracle on the gathered cache."""
    from swiftlm_amd import DFlashKernels as K

    rng = np.random.default_rng(seed)
    for it in range(20):
        D = int(rng.choice([128, 256]))
        Hk = int(rng.choice([1, 2, 3]))
        Hq = Hk * int(rng.choice([1, 2, 4, 8, 9]))
        B = int(rng.choice([1, 2, 3]))
        P = int(rng.choice([32, 64, 128, 512]))
        dt = torch.bfloat16 if rng.random() < 0.7 else torch.float16
        Ls = [int(rng.choice([0, 1, 15, 16, 17, 31, 33, 100, 257, 700])) for _ in range(B)]
        lens = [l + 16 for l in Ls]
        append = bool(rng.random() < 0.5)
        case = f"seed {seed} case {it}: B={B} Hq={Hq} Hk={Hk} Ls={Ls} D={D} P={P} {dt} append={append}"
        q, k, v, k_pool, v_pool, table = paged_case(int(rng.integers(1 << 30)), B, Hq, Hk, lens, D, P, dt,
                                                    head_pad=int(rng.choice([0, 8, 64])), page_pad=int(rng.choice([0, 16])))
        scale = 1.0 / math.sqrt(D)
        kv_len = torch.tensor(lens, dtype=torch.int32, device="cuda")
        want, want_lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True, kv_len=kv_len)
        if append:
            k_new = torch.stack([k[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
            v_new = torch.stack([v[b, :, Ls[b]:Ls[b] + 16] for b in range(B)]).contiguous()
            tb = table.cpu().numpy()
            for b in range(B):
                for n in range(Ls[b], lens[b]):
                    k_pool[tb[b, n // P], :, n % P] = 3.0
                    v_pool[tb[b, n // P], :, n % P] = 3.0
            got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, max(lens), k_new=k_new, v_new=v_new,
                                                      lengths=torch.tensor(Ls, dtype=torch.int32, device="cuda"), return_lse=True)
        else:
            got, got_lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, max(lens), lengths=kv_len, return_lse=True)
        torch.cuda.synchronize()
        assert torch.equal(got, want) and torch.equal(got_lse, want_lse), case
        for b in range(B):
            kd = O.gather_pages(host(k_pool), table.cpu().numpy()[b:b + 1], lens[b])
            vd = O.gather_pages(host(v_pool), table.cpu().numpy()[b:b + 1], lens[b])
            assert np.array_equal(kd, host(k[b:b + 1, :, : lens[b]])) and np.array_equal(vd, host(v[b:b + 1, :, : lens[b]])), case
            ref, ref_lse = O.sdpa_block_causal(host(q[b:b + 1]), kd, vd, scale)
            np.testing.assert_allclose(host(got[b:b + 1]), ref, err_msg=case, **OUT_TOL)
            np.testing.assert_allclose(host(got_lse[b:b + 1]), ref_lse, err_msg=case, **LSE_TOL)


@pytest.mark.parametrize("variant", ["plain", "masked", "append", "paged", "paged_append"])
@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_device_side_length_shorter_than_bound_in_every_instantiation(gpu_lib, variant, D, dtype):
    """Every instantiation of the partial kernel (two element types x two head dims x plain / masked / paged, with
    and without the fused append) reads the per-sequence key count from device memory through the scalar cache and
    waits for it by hand.  Each is run with ragged counts well below the host-side bound N -- a count taken too early
    would attend N keys (or garbage) -- and checked against the float32 restatement on exactly the live keys."""
    from swiftlm_amd import DFlashKernels as K

    B, Hq, Hk, P = 3, 8, 2, 64
    lens = [16 + 37, 16 + 700, 16 + 1501]                      # keys per sequence, block included
    N = 2000                                                   # the host-side bound (a cache capacity), never reached
    q, k, v, k_pool, v_pool, table = paged_case(D + len(variant), B, Hq, Hk, [N] * B, D, P, dtype)
    scale = 1.0 / math.sqrt(D)
    kv_len = torch.tensor(lens, dtype=torch.int32, device="cuda")
    cache_len = kv_len - 16
    g = torch.Generator(device="cuda").manual_seed(4)
    k_new = torch.randn(B, Hk, 16, D, generator=g, device="cuda").to(dtype)
    v_new = torch.randn(B, Hk, 16, D, generator=g, device="cuda").to(dtype)
    if "append" in variant:                                    # what the attention must see: the block's rows at cache_len
        for b in range(B):
            k[b, :, lens[b] - 16:lens[b]] = k_new[b]
            v[b, :, lens[b] - 16:lens[b]] = v_new[b]
    ow, lw = torch_reference(q, k, v, scale, kv_len=lens)
    if variant == "plain":
        out, lse = K.batched_sdpa_2pass(q, k, v, scale, return_lse=True, kv_len=kv_len)
    elif variant == "masked":
        zero = torch.zeros(B, Hq, 16, N, dtype=dtype, device="cuda")
        out, lse = K.batched_sdpa_2pass(q, k, v, scale, zero, return_lse=True, kv_len=kv_len)
    elif variant == "append":
        kc, vc = k.clone(), v.clone()
        for b in range(B):                                     # the cache does not hold the block yet
            kc[b, :, lens[b] - 16:lens[b]] = 0
            vc[b, :, lens[b] - 16:lens[b]] = 0
        out, lse = K.batched_sdpa_2pass_append(q, kc, vc, k_new, v_new, scale, N, return_lse=True, cache_len=cache_len)
        for b in range(B):
            assert torch.equal(kc[b, :, lens[b] - 16:lens[b]], k_new[b]) and torch.equal(vc[b, :, lens[b] - 16:lens[b]], v_new[b])
    elif variant == "paged":
        out, lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, N, lengths=kv_len, return_lse=True)
    else:
        out, lse = K.batched_sdpa_2pass_paged(q, k_pool, v_pool, table, scale, N, k_new=k_new, v_new=v_new,
                                              lengths=cache_len, return_lse=True)
    torch.cuda.synchronize()
    np.testing.assert_allclose(host(out), host(ow), **OUT_TOL)
    np.testing.assert_allclose(host(lse), host(lw), **LSE_TOL)
