"""Host-side mirror of the rollback caches
(Sources/DFlash/RecurrentRollbackCache.swift) over the C handles of
include/dflash_cache.h.

The native handle does the bookkeeping and enqueues the kernels; these classes
keep the torch tensors alive (the handle only stores their device pointers) and
give the caches the reference's names.  ``cache[0]`` is the conv window
[B, keep, C], ``cache[1]`` the recurrent state [B, Hv, Dv, Dk].
"""

from __future__ import annotations

import ctypes as C
from typing import List, Optional

import torch

from . import _lib
from .dflash_kernels import _code, _stream


class _NativeCache:
    KIND = _lib.CACHE_MAMBA

    def __init__(self, conv_kernel_size: int = 4):
        self._h = C.c_void_p(_lib.load().dflash_cache_create(self.KIND, conv_kernel_size))
        if not self._h:
            raise _lib.DFlashError("cache_create: " + _lib.last_error())
        self._slots: List[Optional[torch.Tensor]] = [None, None]
        self._by_ptr = {}

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            _lib.load().dflash_cache_destroy(h)

    # slots -------------------------------------------------------------------
    def __getitem__(self, i: int) -> Optional[torch.Tensor]:
        p = _lib.load().dflash_cache_get_slot(self._h, i)
        return self._by_ptr.get(p) if p else None

    def __setitem__(self, i: int, t: Optional[torch.Tensor]) -> None:
        if t is not None:
            if not t.is_cuda or not t.is_contiguous():
                raise _lib.DFlashError("cache slots hold contiguous device tensors")
            self._by_ptr[t.data_ptr()] = t
        _lib.check(_lib.load().dflash_cache_set_slot(self._h, i, C.c_void_p(t.data_ptr()) if t is not None else None),
                   "cache_set_slot")
        self._slots[i] = t
        if not self._holds_snapshot():
            self._forget_dead()

    def _holds_snapshot(self) -> bool:
        return False

    def _forget_dead(self) -> None:
        live = {_lib.load().dflash_cache_get_slot(self._h, i) for i in (0, 1)}
        self._by_ptr = {p: t for p, t in self._by_ptr.items() if p in live}

    @property
    def offset(self) -> int:
        return int(_lib.load().dflash_cache_offset(self._h))

    @offset.setter
    def offset(self, v: int) -> None:
        _lib.check(_lib.load().dflash_cache_set_offset(self._h, int(v)), "cache_set_offset")

    def trim(self, n: int) -> int:
        return int(_lib.load().dflash_cache_trim(self._h, int(n)))

    @property
    def is_trimmable(self) -> bool:
        return False


class MambaCache(_NativeCache):
    """Plain recurrent cache without rollback (the reference's MambaCache lives in mlx-swift-lm;
    only its use at DFlashRuntime.swift:206-211 matters here)."""

    KIND = _lib.CACHE_MAMBA


class KVCacheSimple(_NativeCache):
    """Trimmable attention cache as seen by restoreTargetCacheAfterAcceptance
    (DFlashRuntime.swift:212-218): an offset that ``trim`` lowers."""

    KIND = _lib.CACHE_KV

    @property
    def is_trimmable(self) -> bool:
        return True


class _RollbackCache(_NativeCache):
    """``protocol DFlashRollbackCache`` (RecurrentRollbackCache.swift:12-18)."""

    @property
    def is_armed(self) -> bool:
        return bool(_lib.load().dflash_cache_is_armed(self._h))

    def _holds_snapshot(self) -> bool:
        return self.is_armed

    def arm_rollback(self, prefix_len: int = 0) -> None:
        _lib.check(_lib.load().dflash_cache_arm_rollback(self._h, int(prefix_len)), "arm_rollback")

    def record_tape(self, tape: torch.Tensor, k: torch.Tensor, g: torch.Tensor, qkv: Optional[torch.Tensor]) -> None:
        state = self[1]
        if state is None:
            raise _lib.DFlashError("record_tape: slot 1 (recurrent state) is empty")
        tape, k, g = tape.contiguous(), k.contiguous(), g.contiguous()
        qkv = None if qkv is None else qkv.contiguous()
        self._tape_refs = (tape, k, g, qkv)
        B, T, Hk, Dk = k.shape
        Hv, Dv = tape.shape[2], tape.shape[3]
        rc = _lib.load().dflash_cache_record_tape(
            self._h, C.c_void_p(tape.data_ptr()), _code(tape), C.c_void_p(k.data_ptr()), C.c_void_p(g.data_ptr()),
            _code(k), g.dim(), C.c_void_p(qkv.data_ptr()) if qkv is not None else None,
            qkv.element_size() if qkv is not None else 2, _code(state), B, T, Hk, Hv, Dk, Dv,
            qkv.shape[-1] if qkv is not None else 0)
        _lib.check(rc, "record_tape")

    def rollback(self, n_accepted: int) -> None:
        rc = _lib.load().dflash_cache_rollback(self._h, _stream(), int(n_accepted))
        self._after_rollback()
        _lib.check(rc, "rollback")

    def clear_transients(self) -> None:
        _lib.check(_lib.load().dflash_cache_clear_transients(self._h), "clear_transients")
        self._after_rollback()

    def _after_rollback(self) -> None:
        # tape tensors stay referenced until the next cycle records new ones: the replay
        # that reads them may still be queued on the stream.
        self._forget_dead()


class RecurrentRollbackCache(_RollbackCache):
    """``RecurrentRollbackCache`` (RecurrentRollbackCache.swift:34-182): tape-replay rollback."""

    KIND = _lib.CACHE_TAPE
    default_conv_kernel_size = 4            # :135


class MambaSnapshotCache(_RollbackCache):
    """``MambaSnapshotCache`` (RecurrentRollbackCache.swift:193-232): snapshot-only rollback."""

    KIND = _lib.CACHE_SNAPSHOT
