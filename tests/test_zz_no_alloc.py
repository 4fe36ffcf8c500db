"""dflash_sdpa_block_causal_static (the entry that allocates nothing: its split-KV scratch is an
array inside the library) against dflash_sdpa_block_causal with a caller-provided workspace,
through the C ABI, bit for bit, on calls that follow one another in one process and share the
array: a large shape, then smaller ones that find the previous call's contents in it."""

import ctypes as C

import pytest
import torch

from swiftlm_amd import _lib

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 18 * 1024 * 1024          # DFLASH_SDPA_STATIC_SCRATCH_BYTES


def _p(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _inputs(seed, B, Hq, Hk, N, D, dtype):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(B, Hq, 16, D, generator=g, device="cuda").to(dtype)
    k = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dtype)
    v = torch.randn(B, Hk, N, D, generator=g, device="cuda").to(dtype)
    return q, k, v


def _both(lib, q, k, v, kv_len=None):
    """(out, lse) of the workspace entry and of the static entry on the same inputs."""
    B, Hq, M, D = q.shape
    Hk, N = k.shape[1], k.shape[2]
    code = _lib.BF16 if q.dtype == torch.bfloat16 else _lib.F16
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    scale = 1.0 / D ** 0.5
    need = int(lib.dflash_sdpa_workspace_bytes(B, Hq, Hk, M, N, D))
    assert 0 < need <= SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out_a, out_b = torch.empty_like(q), torch.full_like(q, float("nan"))
    lse_a = torch.empty(B, Hq, M, dtype=torch.float32, device="cuda")
    lse_b = torch.full_like(lse_a, float("nan"))
    tail = (code, scale, B, Hq, Hk, M, N, D, k.stride(0), k.stride(1), _p(kv_len))
    _lib.check(lib.dflash_sdpa_block_causal(st, _p(q), _p(k), _p(v), _p(out_a), _p(lse_a), *tail, _p(ws), need),
               "sdpa_block_causal")
    _lib.check(lib.dflash_sdpa_block_causal_static(st, _p(q), _p(k), _p(v), _p(out_b), _p(lse_b), *tail),
               "sdpa_block_causal_static")
    torch.cuda.synchronize()
    return (out_a, lse_a), (out_b, lse_b)


def _same(a, b):
    assert torch.equal(a[0].view(torch.int16), b[0].view(torch.int16)), "output rows differ"
    assert torch.equal(a[1].view(torch.int32), b[1].view(torch.int32)), "logsumexp differs"
    assert torch.isfinite(b[1]).all()


def test_static_entry_equals_workspace_entry_on_consecutive_calls(gpu_lib):
    lib = gpu_lib
    _lib.check(lib.dflash_init(), "dflash_init")
    # 1: the benchmark's attention shape (17.0 MB of scratch, nearly the whole array)
    q, k, v = _inputs(1, 1, 16, 2, 32768 + 16, 256, torch.bfloat16)
    _same(*_both(lib, q, k, v))
    # 2: a much smaller call right behind it, other head dim and type; the array still holds call 1's rows
    q, k, v = _inputs(2, 1, 8, 2, 300, 128, torch.float16)
    _same(*_both(lib, q, k, v))
    # 3: ragged batch with device-side lengths, splits left empty by the short sequences
    q, k, v = _inputs(3, 3, 16, 2, 4112, 256, torch.bfloat16)
    kv_len = torch.tensor([4112, 16, 1000], dtype=torch.int32, device="cuda")
    _same(*_both(lib, q, k, v, kv_len))
    # 4: call 1's shape again on fresh data
    q, k, v = _inputs(4, 1, 16, 2, 32768 + 16, 256, torch.bfloat16)
    _same(*_both(lib, q, k, v))


def test_static_entry_rejects_what_the_array_cannot_hold(gpu_lib):
    lib = gpu_lib
    B, Hq, Hk, N, D = 160, 16, 2, 16, 256          # 40,960 rows x 1 split x 520 B > 18 MiB
    need = int(lib.dflash_sdpa_workspace_bytes(B, Hq, Hk, 16, N, D))
    assert need > SCRATCH_BYTES
    q, k, v = _inputs(5, B, Hq, Hk, N, D, torch.bfloat16)
    out = torch.zeros_like(q)
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.dflash_sdpa_block_causal_static(st, _p(q), _p(k), _p(v), _p(out), None, _lib.BF16, 1.0 / 16, B, Hq, Hk, 16, N, D,
                                             k.stride(0), k.stride(1), None)
    assert rc == _lib.UNSUPPORTED
    msg = _lib.last_error()
    assert str(need) in msg and str(SCRATCH_BYTES) in msg, msg
    torch.cuda.synchronize()
    assert not out.any()                            # nothing was launched
