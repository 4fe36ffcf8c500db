"""Host-side mirror of the accept / commit / rollback part of ``DFlashRuntime``
(Sources/DFlash/DFlashRuntime.swift) and of the two ``DFlashEngine``
implementations (Sources/DFlash/DFlashEngine.swift), over the HIP C ABI.

Only the verify side of the loop is here: acceptance length, commit indexing,
cache arming and restoration.  Drafting, the target model and token streaming
are the caller's.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Sequence

import torch

from . import _lib
from .dflash_kernels import _code, _ptr, _stream
from .rollback_cache import RecurrentRollbackCache, _NativeCache, _RollbackCache


@dataclass
class AcceptResult:
    """What one verify cycle decides (names as in DFlashRuntime.swift:523-547, :571)."""
    acceptance_len: int
    commit_count: int
    staged_first_next: int
    start: int


_greedy_ws = {}


def _greedy_workspace(T: int, V: int, device) -> torch.Tensor:
    """One scratch tensor per (T, V, device, stream): launches sharing it must not overlap, which
    one stream guarantees."""
    key = (T, V, str(device), int(_stream().value or 0))
    ws = _greedy_ws.get(key)
    if ws is None:
        need = int(_lib.load().dflash_greedy_workspace_bytes(T, V))
        ws = torch.empty(need, dtype=torch.uint8, device=device)
        _greedy_ws[key] = ws
    return ws


class DFlashRuntime:
    # -- token utilities -------------------------------------------------------------
    @staticmethod
    def build_suppress_token_mask(vocab_size: int, suppress_token_ids, device="cuda"):
        """``buildSuppressTokenMask(vocabSize:suppressTokenIDs:)`` (DFlashRuntime.swift:105-115):
        uint8 [vocab] on the device, or None when no id is in range."""
        ids = sorted({int(i) for i in (suppress_token_ids or []) if 0 <= int(i) < vocab_size})
        if not ids:
            return None
        mask = torch.zeros(vocab_size, dtype=torch.uint8)
        mask[ids] = 1
        return mask.to(device)

    @staticmethod
    def greedy_tokens_with_mask(logits: torch.Tensor, suppress_token_mask=None) -> torch.Tensor:
        """``greedyTokensWithMask(logits:suppressTokenMask:)`` (DFlashRuntime.swift:118-128):
        logits [T, V] -> int32 [T] holding the reference's uint32 token ids."""
        if not logits.is_cuda or logits.dim() != 2:
            raise _lib.DFlashError("greedy_tokens_with_mask: logits must be a [T, V] tensor on the GPU")
        logits = logits.contiguous()
        T, V = logits.shape
        m = None if suppress_token_mask is None else suppress_token_mask.to(torch.uint8).contiguous()
        out = torch.empty(T, dtype=torch.int32, device=logits.device)
        ws = _greedy_workspace(T, V, logits.device)
        rc = _lib.load().dflash_greedy_tokens_with_mask(_stream(), _ptr(logits), _code(logits), T, V, _ptr(m), _ptr(out),
                                                        _ptr(ws), ws.numel())
        _lib.check(rc, "greedy_tokens_with_mask")
        return out

    @staticmethod
    def greedy_accept_commit(logits: torch.Tensor, suppress_token_mask, verify_ids: torch.Tensor, start: int):
        """The cycle's greedy tokens, acceptance length and commit bookkeeping in one call
        (DFlashRuntime.swift:513-547): returns (AcceptResult, posterior int32 [T])."""
        logits = logits.contiguous()
        T, V = logits.shape
        if int(verify_ids.shape[0]) != T:
            raise _lib.DFlashError("greedy_accept_commit: one logits row per verify position")
        m = None if suppress_token_mask is None else suppress_token_mask.to(torch.uint8).contiguous()
        v = verify_ids.to(torch.int32).contiguous()
        post = torch.empty(T, dtype=torch.int32, device=logits.device)
        out = torch.empty(4, dtype=torch.int32, device=logits.device)
        st = torch.tensor([start], dtype=torch.int32, device=logits.device)
        ws = _greedy_workspace(T, V, logits.device)
        rc = _lib.load().dflash_greedy_accept_commit(_stream(), _ptr(logits), _code(logits), T, V, _ptr(m), _ptr(v), _ptr(st),
                                                     _ptr(out), _ptr(post), _ptr(ws), ws.numel())
        _lib.check(rc, "greedy_accept_commit")
        a, c, s, n = out.tolist()
        return AcceptResult(a, c, s, n), post

    # -- acceptance ----------------------------------------------------------------
    @staticmethod
    def match_acceptance_length(drafted_tokens: torch.Tensor, posterior_tokens: torch.Tensor) -> torch.Tensor:
        """``matchAcceptanceLength(draftedTokens:posteriorTokens:)`` (DFlashRuntime.swift:133-142):
        number of leading matches as an int32 device scalar; 0 for empty input."""
        n = int(drafted_tokens.shape[0])
        out = torch.empty((), dtype=torch.int32, device=drafted_tokens.device)
        d = drafted_tokens.to(torch.int32).contiguous()     # same 32-bit pattern as the reference's uint32
        p = posterior_tokens.to(torch.int32).contiguous()
        if p.shape[0] < n:
            raise _lib.DFlashError("match_acceptance_length: posterior shorter than drafted")
        rc = _lib.load().dflash_match_acceptance_length(_stream(), _ptr(d) if n else None, _ptr(p) if n else None, n, _ptr(out))
        _lib.check(rc, "match_acceptance_length")
        return out

    @staticmethod
    def accept_commit(verify_ids: torch.Tensor, posterior: torch.Tensor, start: int) -> AcceptResult:
        """One cycle's integer bookkeeping done on the device and read back in a single
        16-byte copy (the reference blocks on ``.item()`` at DFlashRuntime.swift:525-530
        and then derives commitCount / stagedFirstNext / start on the host, :544-571)."""
        V = int(verify_ids.shape[0])
        v = verify_ids.to(torch.int32).contiguous()
        p = posterior.to(torch.int32).contiguous()
        if p.shape[0] < V:
            raise _lib.DFlashError("accept_commit: posterior must cover every verify position")
        out = torch.empty(4, dtype=torch.int32, device=v.device)
        st = torch.tensor([start], dtype=torch.int32, device=v.device)
        rc = _lib.load().dflash_accept_commit(_stream(), _ptr(v), _ptr(p), V, _ptr(st), _ptr(out))
        _lib.check(rc, "accept_commit")
        a, c, s, n = out.tolist()
        return AcceptResult(a, c, s, n)

    # -- caches ----------------------------------------------------------------------
    @staticmethod
    def arm_target_rollback(target_cache: Sequence[_NativeCache], prefix_len: int) -> None:
        """``armTargetRollback`` (DFlashRuntime.swift:170-176)."""
        for cache in target_cache:
            if isinstance(cache, _RollbackCache):
                cache.arm_rollback(prefix_len)

    @staticmethod
    def restore_target_cache_after_acceptance(cache_entries: Sequence[_NativeCache], target_len: int,
                                              acceptance_length: int, drafted_tokens: int) -> int:
        """``restoreTargetCacheAfterAcceptance`` (DFlashRuntime.swift:188-223); returns the
        nanoseconds spent enqueuing the rollbacks.  Every tape cache's replay goes out in one
        launch instead of one launch per cache."""
        n = len(cache_entries)
        arr = (C.c_void_p * max(n, 1))(*[c._h.value for c in cache_entries])
        ns = C.c_int64(0)
        rc = _lib.load().dflash_restore_target_cache_after_acceptance(
            C.cast(arr, _lib.vpp), n, _stream(), int(target_len), int(acceptance_length), int(drafted_tokens),
            C.byref(ns))
        for c in cache_entries:
            if isinstance(c, _RollbackCache):
                c._after_rollback()
        _lib.check(rc, "restore_target_cache_after_acceptance")
        return int(ns.value)


class DFlashEngine:
    """``protocol DFlashEngine`` (DFlashEngine.swift:17-28)."""

    def arm_rollback(self, target_cache, prefix_len: int) -> None:  # pragma: no cover - protocol
        raise NotImplementedError

    def rollback(self, target_cache, target_len: int, acceptance_length: int, drafted_tokens: int) -> int:
        return DFlashRuntime.restore_target_cache_after_acceptance(
            target_cache, target_len, acceptance_length, drafted_tokens)


class FullAttentionEngine(DFlashEngine):
    """``FullAttentionEngine`` (DFlashEngine.swift:34-54): nothing to arm; rollback trims KV."""

    def arm_rollback(self, target_cache, prefix_len: int) -> None:
        pass


class HybridGDNEngine(DFlashEngine):
    """``HybridGDNEngine`` (DFlashEngine.swift:60-84): arms the tape caches only."""

    def arm_rollback(self, target_cache, prefix_len: int) -> None:
        for cache in target_cache:
            if isinstance(cache, RecurrentRollbackCache):
                cache.arm_rollback(prefix_len)


def verify_ids_for_block(staged_first: torch.Tensor, drafted: torch.Tensor, verify_token_count: int) -> torch.Tensor:
    """``verifyTokenIDs`` (DFlashRuntime.swift:485-496): the staged first token followed by the
    first ``verify_token_count - 1`` drafted tokens."""
    if verify_token_count <= 1 or drafted is None or drafted.numel() == 0:
        return staged_first[:1]
    return torch.cat([staged_first[:1], drafted[: verify_token_count - 1]], dim=0)


def committed_segment(verify_ids: torch.Tensor, commit_count: int) -> List[int]:
    """``committedSegment`` (DFlashRuntime.swift:545)."""
    return verify_ids[:commit_count].tolist()
