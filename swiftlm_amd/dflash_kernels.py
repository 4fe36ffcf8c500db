"""Host-side mirror of ``DFlashKernels`` (Sources/DFlash/DFlashKernels.swift) and
``DFlashKernelProvider`` / ``DFlashKernelRegistry``
(Sources/DFlash/DFlashKernelProvider.swift) over the HIP C ABI.

Same entry-point names, argument meaning and error behaviour as the reference:
each call is functional (inputs untouched, freshly allocated outputs).  torch is
used only to own device memory and to name the current stream; every result is
computed by libdflash_hip.so.
"""

from __future__ import annotations

import ctypes as C
from typing import Optional, Sequence, Tuple

import torch

from . import _lib
from ._lib import DFlashError, DFlashUnsupported  # noqa: F401  (re-exported)

_DT = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16,
       torch.uint8: _lib.U8, torch.bool: _lib.U8}


# arrival counters of gdn_layer's in-launch gated norm: int32 zeros per (device, stream, B*Hv), left zero by every call
_ARRIVALS = {}


def _code(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise DFlashUnsupported(f"dtype {t.dtype} is not supported") from None


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev(*ts: Optional[torch.Tensor]) -> None:
    for t in ts:
        if t is not None and not t.is_cuda:
            raise DFlashError("DFlash kernels run on the GPU only: got a CPU tensor (there is no CPU path)")


def _ptr_array(ts: Sequence[torch.Tensor]):
    arr = (C.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    return C.cast(arr, _lib.vpp), arr


class DFlashKernels:
    """Static entry points, named as in the reference."""

    shared: "DFlashKernelsInstance"

    # -- tape replay ---------------------------------------------------------
    @staticmethod
    def tape_replay_kernel(tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, state: torch.Tensor,
                           mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``tapeReplayKernel(tape:k:g:state:mask:)`` (DFlashKernels.swift:252-301).

        tape [B,T,Hv,Dv], k [B,T,Hk,Dk], g [B,T,Hv] or [B,T,Hv,Dk], state
        [B,Hv,Dv,Dk], mask [B,T]; returns the replayed state (same dtype as ``state``).
        """
        _dev(tape, k, g, state, mask)
        tape, k, g, state = (t.contiguous() for t in (tape, k, g, state))
        if g.dtype != k.dtype:
            g = g.to(k.dtype)
        mask = None if mask is None else mask.contiguous()
        B, T, Hk, Dk = k.shape
        Hv, Dv = tape.shape[2], tape.shape[3]
        out = torch.empty_like(state)
        rc = _lib.load().dflash_tape_replay(
            _stream(), _ptr(tape), _code(tape), _ptr(k), _ptr(g), _code(k), g.dim(),
            _ptr(state), _ptr(out), _code(state), _ptr(mask), _code(mask) if mask is not None else 0,
            B, T, Hk, Hv, Dk, Dv)
        _lib.check(rc, "tape_replay_kernel")
        return out

    @staticmethod
    def tape_replay_batched(tapes: Sequence[torch.Tensor], ks: Sequence[torch.Tensor], gs: Sequence[torch.Tensor],
                            states_in: Sequence[torch.Tensor], states_out: Sequence[torch.Tensor], steps: int,
                            steps_dev: Optional[torch.Tensor] = None, skip_if_full: bool = False) -> None:
        """One launch for the per-cache replays that
        ``restoreTargetCacheAfterAcceptance`` issues one by one
        (DFlashRuntime.swift:197-205).  All layers share shapes; results are written
        into ``states_out``."""
        _dev(*tapes, *ks, *gs, *states_in, *states_out, steps_dev)
        n = len(tapes)
        B, T, Hk, Dk = ks[0].shape
        Hv, Dv = tapes[0].shape[2], tapes[0].shape[3]
        for seq in (tapes, ks, gs, states_in, states_out):
            if len(seq) != n or any(not t.is_contiguous() for t in seq):
                raise DFlashError("tape_replay_batched: ragged or non-contiguous layer list")
        pt, _k1 = _ptr_array(tapes)
        pk, _k2 = _ptr_array(ks)
        pg, _k3 = _ptr_array(gs)
        pi, _k4 = _ptr_array(states_in)
        po, _k5 = _ptr_array(states_out)
        rc = _lib.load().dflash_tape_replay_batched(
            _stream(), n, pt, _code(tapes[0]), pk, pg, _code(ks[0]), gs[0].dim(), pi, po, _code(states_in[0]),
            int(steps), _ptr(steps_dev), int(bool(skip_if_full)), B, T, Hk, Hv, Dk, Dv)
        _lib.check(rc, "tape_replay_batched")

    # -- gated delta with tape -------------------------------------------------
    @staticmethod
    def gated_delta_kernel_with_tape(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                                     beta: torch.Tensor, state: torch.Tensor,
                                     mask: Optional[torch.Tensor] = None, want_state: bool = True
                                     ) -> Tuple[torch.Tensor, Optional[torch.Tensor], torch.Tensor]:
        """``gatedDeltaKernelWithTape(q:k:v:g:beta:state:mask:)`` (DFlashKernels.swift:316-367).

        Returns (y [B,T,Hv,Dv] in q's dtype, new state in ``state``'s dtype,
        innovation tape [B,T,Hv,Dv] float32).  ``want_state=False`` (no counterpart in the reference) leaves the
        post-block state out -- None is returned in its place -- for a caller that replays the tape whatever is
        accepted; only the verify-block form supports it (``DFlashUnsupported`` otherwise)."""
        _dev(q, k, v, g, beta, state, mask)
        q, k, v, g, beta, state = (t.contiguous() for t in (q, k, v, g, beta, state))
        for name, t in (("k", k), ("v", v), ("g", g), ("beta", beta)):
            if t.dtype != q.dtype:
                raise DFlashUnsupported(f"gated_delta_kernel_with_tape: {name} dtype {t.dtype} differs from q's {q.dtype}")
        mask = None if mask is None else mask.contiguous()
        B, T, Hk, Dk = k.shape
        Hv, Dv = v.shape[2], v.shape[3]
        y = torch.empty((B, T, Hv, Dv), dtype=q.dtype, device=q.device)
        tape = torch.empty((B, T, Hv, Dv), dtype=torch.float32, device=q.device)
        out = torch.empty_like(state) if want_state else None
        rc = _lib.load().dflash_gated_delta_tape(
            _stream(), _ptr(q), _ptr(k), _ptr(v), _ptr(g), g.dim(), _ptr(beta), _code(q),
            _ptr(state), _ptr(out), _code(state), _ptr(y), _ptr(tape),
            _ptr(mask), _code(mask) if mask is not None else 0, B, T, Hk, Hv, Dk, Dv)
        _lib.check(rc, "gated_delta_kernel_with_tape")
        return y, out, tape

    # -- block-causal SDPA -------------------------------------------------------
    @staticmethod
    def sdpa_workspace_bytes(B: int, Hq: int, Hk: int, M: int, N: int, D: int) -> int:
        return int(_lib.load().dflash_sdpa_workspace_bytes(B, Hq, Hk, M, N, D))

    @staticmethod
    def gdn_prepare(mixed_qkv: torch.Tensor, conv_state: Optional[torch.Tensor], conv_weight: torch.Tensor,
                    a_logits: torch.Tensor, b_logits: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                    Hk: int, Hv: int, Dk: int, Dv: int, q_scale: float, k_scale: float, eps: float = 1e-6):
        """The layer's steps between its projections and the recurrence, in one launch
        (Sources/SwiftLM/KimiLinearDFlash.swift: ShortConv1d :274-293, q/k normalisation :362-363,
        gates :390-391).  ``mixed_qkv`` [B,T,2*Hk*Dk+Hv*Dv] with channels q|k|v; ``conv_state``
        [B,K-1,C] or None; ``conv_weight`` [C,K]; ``a_logits`` [B,T,Hv] or [B,T,Hv,Dk];
        ``a_log`` [Hv] and ``dt_bias`` float32.  Returns (q, k, v, g, beta, new_conv_state), ready for
        ``gated_delta_kernel_with_tape``; ``mixed_qkv`` is what ``record_tape`` keeps as qkv."""
        _dev(mixed_qkv, conv_state, conv_weight, a_logits, b_logits, a_log, dt_bias)
        B, T, C = mixed_qkv.shape
        if C != 2 * Hk * Dk + Hv * Dv:
            raise DFlashError(f"gdn_prepare: {C} channels, expected 2*{Hk}*{Dk} + {Hv}*{Dv}")
        K = int(conv_weight.shape[1])
        dt = mixed_qkv.dtype
        x = mixed_qkv.contiguous()
        w = conv_weight.to(dt).contiguous()
        st = None if conv_state is None else conv_state.to(dt).contiguous()
        a = a_logits.to(dt).contiguous()
        bl = b_logits.to(dt).contiguous()
        al = a_log.float().contiguous()
        db = dt_bias.float().contiguous().reshape(-1)
        q = torch.empty(B, T, Hk, Dk, dtype=dt, device=x.device)
        k = torch.empty_like(q)
        v = torch.empty(B, T, Hv, Dv, dtype=dt, device=x.device)
        g = torch.empty_like(a)
        beta = torch.empty(B, T, Hv, dtype=dt, device=x.device)
        new_state = torch.empty(B, K - 1, C, dtype=dt, device=x.device)
        rc = _lib.load().dflash_gdn_prepare(
            _stream(), _ptr(x), _ptr(st), _ptr(w), _ptr(a), a.dim(), _ptr(bl), _ptr(al), _ptr(db), _code(x),
            float(q_scale), float(k_scale), float(eps), _ptr(q), _ptr(k), _ptr(v), _ptr(g), _ptr(beta), _ptr(new_state),
            B, T, Hk, Hv, Dk, Dv, K)
        _lib.check(rc, "gdn_prepare")
        return q, k, v, g, beta, new_state

    @staticmethod
    def gdn_finish(y: torch.Tensor, gate: torch.Tensor, norm_weight: torch.Tensor, eps: float,
                   gate_kind: str = "sigmoid") -> torch.Tensor:
        """``oNorm(out) * sigmoid(gate)`` per head (KimiLinearDFlash.swift:377-378); ``gate_kind="silu"``
        is the gated RMSNorm of Qwen3-Next's layer.  y, gate [B,T,Hv,Dv]; norm_weight [Dv]."""
        _dev(y, gate, norm_weight)
        if y.dim() != 4 or gate.shape != y.shape or norm_weight.shape != (y.shape[3],):
            raise DFlashError("gdn_finish: y and gate must be [B,T,Hv,Dv], norm_weight [Dv]")
        B, T, Hv, Dv = y.shape
        y = y.contiguous()
        out = torch.empty_like(y)
        rc = _lib.load().dflash_gdn_finish(_stream(), _ptr(y), _ptr(gate.to(y.dtype).contiguous()),
                                           _ptr(norm_weight.to(y.dtype).contiguous()), _ptr(out), _code(y), float(eps),
                                           {"sigmoid": 0, "silu": 1}[gate_kind], B, T, Hv, Dv)
        _lib.check(rc, "gdn_finish")
        return out

    @staticmethod
    def gdn_layer(mixed_qkv: torch.Tensor, conv_state: Optional[torch.Tensor], conv_weight: torch.Tensor,
                  a_logits: torch.Tensor, b_logits: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor,
                  state: torch.Tensor, Hk: int, Hv: int, Dk: int, Dv: int, q_scale: float, k_scale: float,
                  eps: float = 1e-6, gate: Optional[torch.Tensor] = None, norm_weight: Optional[torch.Tensor] = None,
                  norm_eps: float = 1e-6, gate_kind: str = "sigmoid", want_intermediates: bool = False,
                  arrivals: Optional[torch.Tensor] = None, one_launch: bool = True,
                  out: Optional[torch.Tensor] = None):
        """The body of a GatedDelta layer between its projections (KimiLinearDFlash.swift:351-378) in one
        call: ``gdn_prepare`` -> ``gated_delta_kernel_with_tape`` -> ``gdn_finish`` with the pre-ops done
        inside the forward kernel.  Returns a dict: ``out`` (None without ``gate``), ``y``, ``state``,
        ``tape``, ``k``, ``g`` (what ``record_tape`` keeps), ``conv_state``, and with
        ``want_intermediates`` also ``q``, ``v``, ``beta``.  Raises DFlashUnsupported outside the verify
        block's case (float32 state, scalar gate, K == 4, T <= 16), where the three calls apply.

        With a ``gate`` the gated norm runs inside the same launch, done by the last workgroup of each head;
        the heads' arrival counters are ``arrivals`` (int32 [B*Hv], zero before and after every call) or, when
        it is None, an array this module keeps per device, stream and size.  ``one_launch=False`` runs the gated
        norm as a second launch instead.  ``out`` (optional, [B,T,Hv,Dv] in the input type) receives the gated norm
        instead of a fresh tensor; it may be ``gate`` itself (the library then takes the second launch)."""
        _dev(mixed_qkv, conv_state, conv_weight, a_logits, b_logits, a_log, dt_bias, state, gate, norm_weight)
        B, T, C = mixed_qkv.shape
        if C != 2 * Hk * Dk + Hv * Dv:
            raise DFlashError(f"gdn_layer: {C} channels, expected 2*{Hk}*{Dk} + {Hv}*{Dv}")
        if a_logits.dim() != 3:
            raise DFlashUnsupported("gdn_layer: one decay per head and step only (a_logits [B,T,Hv])")
        if state.dtype != torch.float32:
            raise DFlashUnsupported("gdn_layer: float32 state only")
        K = int(conv_weight.shape[1])
        dt = mixed_qkv.dtype
        dv = mixed_qkv.device
        x = mixed_qkv.contiguous()
        w = conv_weight.to(dt).contiguous()
        st = None if conv_state is None else conv_state.to(dt).contiguous()
        a = a_logits.to(dt).contiguous()
        bl = b_logits.to(dt).contiguous()
        al = a_log.float().contiguous()
        db = dt_bias.float().contiguous().reshape(-1)
        state = state.contiguous()
        k = torch.empty(B, T, Hk, Dk, dtype=dt, device=dv)
        g = torch.empty(B, T, Hv, dtype=dt, device=dv)
        y = torch.empty(B, T, Hv, Dv, dtype=dt, device=dv)
        tape = torch.empty(B, T, Hv, Dv, dtype=torch.float32, device=dv)
        new_state = torch.empty_like(state)
        new_conv = torch.empty(B, K - 1, C, dtype=dt, device=dv)
        q = torch.empty_like(k) if want_intermediates else None
        v = torch.empty_like(y) if want_intermediates else None
        beta = torch.empty_like(g) if want_intermediates else None
        zg = nw = None
        if gate is None:
            out = None
        if gate is not None:
            if norm_weight is None or gate.shape != y.shape or norm_weight.shape != (Dv,):
                raise DFlashError("gdn_layer: gate must be [B,T,Hv,Dv] and come with norm_weight [Dv]")
            zg, nw = gate.to(dt).contiguous(), norm_weight.to(dt).contiguous()
            if out is None:
                out = torch.empty_like(y)
            elif out.shape != y.shape or out.dtype != dt or not out.is_contiguous() or not out.is_cuda:
                raise DFlashError("gdn_layer: out must be a contiguous device tensor [B,T,Hv,Dv] of the input type")
            if not one_launch:
                arrivals = None
            elif arrivals is None:
                key = (dv.index, torch.cuda.current_stream().cuda_stream, B * Hv)
                arrivals = _ARRIVALS.get(key)
                if arrivals is None:
                    if torch.cuda.is_current_stream_capturing():
                        # zeros created here would only be RECORDED (and live in the graph's private pool): an eager call
                        # on this stream before the first replay would count into uninitialised memory
                        raise DFlashError("gdn_layer: first use on this stream happens inside a graph capture; pass "
                                          "`arrivals` (int32 zeros [B*Hv]) or call gdn_layer once on this stream beforehand")
                    arrivals = _ARRIVALS[key] = torch.zeros(B * Hv, dtype=torch.int32, device=dv)
            elif arrivals.dtype != torch.int32 or arrivals.numel() < B * Hv or not arrivals.is_contiguous():
                raise DFlashError("gdn_layer: arrivals must be a contiguous int32 tensor of at least B*Hv elements")
        else:
            arrivals = None
        rc = _lib.load().dflash_gdn_layer(
            _stream(), _ptr(x), _ptr(st), _ptr(w), _ptr(a), _ptr(bl), _ptr(al), _ptr(db), _code(x),
            float(q_scale), float(k_scale), float(eps), _ptr(state), _ptr(new_state), _ptr(k), _ptr(g), _ptr(tape),
            _ptr(new_conv), _ptr(y), _ptr(zg), _ptr(nw), float(norm_eps), {"sigmoid": 0, "silu": 1}[gate_kind],
            _ptr(out), _ptr(arrivals), _ptr(q), _ptr(v), _ptr(beta), B, T, Hk, Hv, Dk, Dv, K)
        _lib.check(rc, "gdn_layer")
        res = dict(out=out, y=y, state=new_state, tape=tape, k=k, g=g, conv_state=new_conv)
        if want_intermediates:
            res.update(q=q, v=v, beta=beta)
        return res

    @staticmethod
    def batched_sdpa_2pass(queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scale: float,
                           mask: Optional[torch.Tensor] = None, *, return_lse: bool = False,
                           kv_len: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None):
        """``batchedSDPA2Pass(queries:keys:values:scale:mask:)`` (DFlashKernels.swift:737-815).

        queries [B,Hq,16,D]; keys/values [B,Hk,N,D] with N including the 16 block
        tokens (a view into a larger cache is fine as long as the last dimension is
        contiguous and rows are D apart).  ``mask`` is the reference's optional additive
        mask [B,Hq,16,N].  Returns None where the reference returns nil (unsupported
        shape/dtype).  ``return_lse`` additionally returns the
        float32 logsumexp [B,Hq,16]; ``kv_len`` (int32 [B] on the device) gives
        per-sequence key counts for ragged batches."""
        if queries.dim() != 4 or keys.dim() != 4 or values.dim() != 4:
            return None
        _dev(queries, keys, values, kv_len, workspace, mask)
        B, Hq, M, D = queries.shape
        Hk, N = keys.shape[1], keys.shape[2]
        if mask is not None:
            # additive [B,Hq,16,N] (anything that broadcasts to it), cast to the input type (:783-787)
            try:
                mask = mask.to(queries.dtype).expand(B, Hq, M, N).contiguous()
            except RuntimeError:
                raise DFlashError(f"batched_sdpa_2pass: mask {tuple(mask.shape)} does not broadcast to {(B, Hq, M, N)}")
        if values.shape != keys.shape or values.shape[3] != D or keys.dtype != queries.dtype or values.dtype != queries.dtype:
            return None
        queries = queries.contiguous()
        if keys.stride(3) != 1 or keys.stride(2) != D or keys.stride() != values.stride():
            keys, values = keys.contiguous(), values.contiguous()
        lib = _lib.load()
        need = int(lib.dflash_sdpa_workspace_bytes(B, Hq, Hk, M, N, D))
        if need == 0:
            return None
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=queries.device)
        out = torch.empty_like(queries)
        lse = torch.empty((B, Hq, M), dtype=torch.float32, device=queries.device) if return_lse else None
        try:
            code = _code(queries)
        except DFlashUnsupported:
            return None
        tail = (code, float(scale), B, Hq, Hk, M, N, D, keys.stride(0), keys.stride(1), _ptr(kv_len), _ptr(workspace),
                workspace.numel() * workspace.element_size())
        if mask is None:
            rc = lib.dflash_sdpa_block_causal(_stream(), _ptr(queries), _ptr(keys), _ptr(values), _ptr(out), _ptr(lse), *tail)
        else:
            rc = lib.dflash_sdpa_block_causal_masked(_stream(), _ptr(queries), _ptr(keys), _ptr(values), _ptr(mask),
                                                     _ptr(out), _ptr(lse), *tail)
        if rc == _lib.UNSUPPORTED:
            return None
        _lib.check(rc, "batched_sdpa_2pass")
        return (out, lse) if return_lse else out

    @staticmethod
    def batched_sdpa_2pass_append(queries: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                                  k_new: torch.Tensor, v_new: torch.Tensor, scale: float, n_keys: int, *,
                                  return_lse: bool = False, cache_len: Optional[torch.Tensor] = None,
                                  workspace: Optional[torch.Tensor] = None):
        """The verify block's attention with its KV append fused in (one launch pair instead of
        ``KVCacheSimple.update`` + ``batchedSDPA2Pass``).  ``k_cache``/``v_cache`` [B,Hk,capacity,D]
        hold ``n_keys - 16`` valid rows per sequence (``cache_len[b]`` when the int32 device
        tensor ``cache_len`` is given; ``n_keys`` is then the upper bound of cache_len + 16);
        ``k_new``/``v_new`` [B,Hk,16,D] are the block's rows, attended as keys n_keys-16 .. n_keys-1
        and written into those cache rows.  Returns None for unsupported shapes."""
        _dev(queries, k_cache, v_cache, k_new, v_new, cache_len, workspace)
        if queries.dim() != 4 or k_cache.dim() != 4 or k_cache.shape != v_cache.shape:
            return None
        B, Hq, M, D = queries.shape
        Hk, cap = k_cache.shape[1], k_cache.shape[2]
        if (k_new.shape != (B, Hk, M, D) or v_new.shape != (B, Hk, M, D) or k_cache.shape[3] != D
                or any(t.dtype != queries.dtype for t in (k_cache, v_cache, k_new, v_new))):
            return None
        if not (M <= n_keys <= cap):
            raise DFlashError(f"batched_sdpa_2pass_append: n_keys={n_keys} outside [{M}, capacity={cap}]")
        if k_cache.stride(3) != 1 or k_cache.stride(2) != D or k_cache.stride() != v_cache.stride():
            raise DFlashError("batched_sdpa_2pass_append: the caches must be row-contiguous and laid out alike")
        queries, k_new, v_new = queries.contiguous(), k_new.contiguous(), v_new.contiguous()
        lib = _lib.load()
        need = int(lib.dflash_sdpa_workspace_bytes(B, Hq, Hk, M, n_keys, D))
        if need == 0:
            return None
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=queries.device)
        out = torch.empty_like(queries)
        lse = torch.empty((B, Hq, M), dtype=torch.float32, device=queries.device) if return_lse else None
        try:
            code = _code(queries)
        except DFlashUnsupported:
            return None
        rc = lib.dflash_sdpa_block_causal_append(
            _stream(), _ptr(queries), _ptr(k_cache), _ptr(v_cache), _ptr(k_new), _ptr(v_new), _ptr(out), _ptr(lse),
            code, float(scale), B, Hq, Hk, M, int(n_keys), D, k_cache.stride(0), k_cache.stride(1), _ptr(cache_len),
            _ptr(workspace), workspace.numel() * workspace.element_size())
        if rc == _lib.UNSUPPORTED:
            return None
        _lib.check(rc, "batched_sdpa_2pass_append")
        return (out, lse) if return_lse else out

    @staticmethod
    def batched_sdpa_2pass_paged(queries: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                                 page_table: torch.Tensor, scale: float, n_keys: int, *,
                                 k_new: Optional[torch.Tensor] = None, v_new: Optional[torch.Tensor] = None,
                                 lengths: Optional[torch.Tensor] = None, return_lse: bool = False,
                                 workspace: Optional[torch.Tensor] = None):
        """The verify block's attention over a paged K/V cache.  ``k_pool``/``v_pool``
        [num_pages, Hk, page_size, D] (page_size a power of two >= 32); ``page_table`` int32
        [B, pages_per_sequence] maps key n of sequence b to page ``page_table[b, n // page_size]``.
        Without ``k_new``/``v_new`` this is ``batched_sdpa_2pass`` on the gathered cache (``lengths``:
        keys per sequence, block included); with them it is ``batched_sdpa_2pass_append`` (``lengths``:
        rows already cached, block excluded; the block's rows are stored into their pages).  The
        reference's cache is dense (``batchedSDPA2Pass``, DFlashKernels.swift:737-743, takes one
        [B,Hk,N,D] array), so paging has no counterpart there.  Returns None for unsupported shapes."""
        _dev(queries, k_pool, v_pool, page_table, k_new, v_new, lengths, workspace)
        if queries.dim() != 4 or k_pool.dim() != 4 or k_pool.shape != v_pool.shape or page_table.dim() != 2:
            return None
        B, Hq, M, D = queries.shape
        num_pages, Hk, page_size = k_pool.shape[0], k_pool.shape[1], k_pool.shape[2]
        if k_pool.shape[3] != D or k_pool.dtype != queries.dtype or v_pool.dtype != queries.dtype:
            return None
        if (k_new is None) != (v_new is None):
            raise DFlashError("batched_sdpa_2pass_paged: k_new and v_new go together")
        if k_new is not None and (k_new.shape != (B, Hk, M, D) or v_new.shape != (B, Hk, M, D)
                                  or k_new.dtype != queries.dtype or v_new.dtype != queries.dtype):
            return None
        if page_table.dtype != torch.int32 or page_table.shape[0] != B or page_table.stride(1) != 1:
            raise DFlashError("batched_sdpa_2pass_paged: page_table must be int32 [B, pages] with unit inner stride")
        if k_pool.stride(3) != 1 or k_pool.stride(2) != D or k_pool.stride() != v_pool.stride():
            raise DFlashError("batched_sdpa_2pass_paged: the pools must be row-contiguous and laid out alike")
        if page_table.shape[1] * page_size < n_keys:
            raise DFlashError(f"batched_sdpa_2pass_paged: {page_table.shape[1]} pages of {page_size} keys do not cover n_keys={n_keys}")
        table_pitch = page_table.stride(0) if B > 1 else page_table.shape[1]      # a single row's stride means nothing
        queries = queries.contiguous()
        if k_new is not None:
            k_new, v_new = k_new.contiguous(), v_new.contiguous()
        lib = _lib.load()
        need = int(lib.dflash_sdpa_workspace_bytes(B, Hq, Hk, M, n_keys, D))
        if need == 0:
            return None
        if workspace is None:
            workspace = torch.empty(need, dtype=torch.uint8, device=queries.device)
        out = torch.empty_like(queries)
        lse = torch.empty((B, Hq, M), dtype=torch.float32, device=queries.device) if return_lse else None
        try:
            code = _code(queries)
        except DFlashUnsupported:
            return None
        rc = lib.dflash_sdpa_block_causal_paged(
            _stream(), _ptr(queries), _ptr(k_pool), _ptr(v_pool), _ptr(page_table), table_pitch, page_size, num_pages,
            k_pool.stride(0), k_pool.stride(1), _ptr(k_new), _ptr(v_new), _ptr(out), _ptr(lse), code, float(scale),
            B, Hq, Hk, M, int(n_keys), D, _ptr(lengths), _ptr(workspace), workspace.numel() * workspace.element_size())
        if rc == _lib.UNSUPPORTED:
            return None
        _lib.check(rc, "batched_sdpa_2pass_paged")
        return (out, lse) if return_lse else out

    @staticmethod
    def sdpa_fallback(queries: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, scale: float,
                      mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``sdpaFallback`` (DFlashKernels.swift:818-828) delegates to the array library's
        general attention.  This package ships only the verify-block kernel, so shapes
        it does not cover are an error here instead of a silent second path."""
        out = DFlashKernels.batched_sdpa_2pass(queries, keys, values, scale, mask)
        if out is None:
            raise DFlashUnsupported("sdpa_fallback: shape/dtype not covered by the verify-block attention kernel")
        return out


class DFlashKernelProvider:
    """``protocol DFlashKernelProvider`` (DFlashKernelProvider.swift:8-14)."""

    def gated_delta_kernel_with_tape(self, q, k, v, g, beta, state, mask):  # pragma: no cover - protocol
        raise NotImplementedError


class DFlashKernelsInstance(DFlashKernelProvider):
    """``DFlashKernelsInstance`` (DFlashKernels.swift:832-843)."""

    def gated_delta_kernel_with_tape(self, q, k, v, g, beta, state, mask=None):
        return DFlashKernels.gated_delta_kernel_with_tape(q, k, v, g, beta, state, mask)


DFlashKernels.shared = DFlashKernelsInstance()


class DFlashKernelRegistry:
    """``DFlashKernelRegistry.provider`` (DFlashKernelProvider.swift:17-19)."""

    provider: Optional[DFlashKernelProvider] = None
