"""ctypes binding of libdflash_hip.so, the C ABI declared in include/dflash_hip.h
and include/dflash_cache.h (plus the measurement hooks of include/dflash_profile.h).

There is no CPU or PyTorch fallback anywhere in this package: if the library is
not built, or the device is not a gfx950, loading fails with an error.
"""

from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdflash_hip.so")

OK, UNSUPPORTED, INVALID = 0, 1, 2
F32, BF16, F16, U8 = 0, 1, 2, 3
CACHE_TAPE, CACHE_SNAPSHOT, CACHE_MAMBA, CACHE_KV = 0, 1, 2, 3
MAX_BATCHED_LAYERS = 64
STATUS_SDPA_LEN, STATUS_APPEND_RANGE, STATUS_CONV_STEPS, STATUS_LAYER_ARRIVALS = 1, 2, 4, 8
KERNEL_SDPA_PARTIAL, KERNEL_SDPA_COMBINE, KERNEL_GDN_FORWARD, KERNEL_TAPE_REPLAY = 0, 1, 2, 3
KERNEL_GREEDY_PARTIAL, KERNEL_GDN_PREPARE, KERNEL_EMPTY, KERNEL_GDN_LAYER, KERNEL_GDN_FINISH = 4, 5, 6, 7, 8

vp, i32, i64, f32, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
vpp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); the single source of truth the symbol test walks.
SIGNATURES = {
    "dflash_version": (i32, []),
    "dflash_last_error": (C.c_char_p, []),
    "dflash_init": (i32, []),
    "dflash_tape_replay": (i32, [vp, vp, i32, vp, vp, i32, i32, vp, vp, i32, vp, i32] + [i32] * 6),
    "dflash_tape_replay_batched": (i32, [vp, i32, vpp, i32, vpp, vpp, i32, i32, vpp, vpp, i32, i32, vp, i32] + [i32] * 6),
    "dflash_gated_delta_tape": (i32, [vp, vp, vp, vp, vp, i32, vp, i32, vp, vp, i32, vp, vp, vp, i32] + [i32] * 6),
    "dflash_gdn_prepare": (i32, [vp, vp, vp, vp, vp, i32, vp, vp, vp, i32, f32, f32, f32, vp, vp, vp, vp, vp, vp] + [i32] * 7),
    "dflash_gdn_finish": (i32, [vp, vp, vp, vp, vp, i32, f32, i32, i32, i32, i32, i32]),
    "dflash_gdn_layer": (i32, [vp] * 8 + [i32, f32, f32, f32] + [vp] * 9 + [f32, i32] + [vp] * 5 + [i32] * 7),
    "dflash_sdpa_workspace_bytes": (sz, [i32] * 6),
    "dflash_sdpa_block_causal": (i32, [vp, vp, vp, vp, vp, vp, i32, f32] + [i32] * 6 + [i64, i64, vp, vp, sz]),
    "dflash_sdpa_block_causal_static": (i32, [vp, vp, vp, vp, vp, vp, i32, f32] + [i32] * 6 + [i64, i64, vp]),
    "dflash_sdpa_block_causal_masked": (i32, [vp, vp, vp, vp, vp, vp, vp, i32, f32] + [i32] * 6 + [i64, i64, vp, vp, sz]),
    "dflash_sdpa_block_causal_append": (i32, [vp, vp, vp, vp, vp, vp, vp, vp, i32, f32] + [i32] * 6 + [i64, i64, vp, vp, sz]),
    "dflash_sdpa_block_causal_paged": (i32, [vp, vp, vp, vp, vp, i32, i32, i32, i64, i64, vp, vp, vp, vp, i32, f32] + [i32] * 6 +
                                       [vp, vp, sz]),
    "dflash_match_acceptance_length": (i32, [vp, vp, vp, i32, vp]),
    "dflash_accept_commit": (i32, [vp, vp, vp, i32, vp, vp]),
    "dflash_accept_commit_replay_batched": (i32, [vp, vp, vp, i32, vp, vp, i32, vpp, i32, vpp, vpp, i32, i32, vpp, vpp, i32,
                                                  i32, i32, i32, i32, i32, i32, i32]),
    "dflash_greedy_workspace_bytes": (sz, [i32, i32]),
    "dflash_greedy_tokens_with_mask": (i32, [vp, vp, i32, i32, i32, vp, vp, vp, sz]),
    "dflash_greedy_accept_commit": (i32, [vp, vp, i32, i32, i32, vp, vp, vp, vp, vp, vp, sz]),
    "dflash_rebuild_conv_state": (i32, [vp, vp, vp, vp] + [i32] * 6 + [vp]),
    "dflash_kv_append": (i32, [vp, vp, vp, vp, vp] + [i32] * 5 + [i64, i64, i32, vp, i32, vp]),
    "dflash_set_status_word": (i32, [vp]),
    "dflash_profile_next_launch": (i32, [i32, vp, vp]),
    "dflash_profile_empty_launch": (i32, [vp, i32, i32, i32, i32, i32]),
    "dflash_cache_create": (vp, [i32, i32]),
    "dflash_cache_destroy": (None, [vp]),
    "dflash_cache_kind": (i32, [vp]),
    "dflash_cache_set_slot": (i32, [vp, i32, vp]),
    "dflash_cache_get_slot": (vp, [vp, i32]),
    "dflash_cache_offset": (i64, [vp]),
    "dflash_cache_set_offset": (i32, [vp, i64]),
    "dflash_cache_is_armed": (i32, [vp]),
    "dflash_cache_arm_rollback": (i32, [vp, i64]),
    "dflash_cache_record_tape": (i32, [vp, vp, i32, vp, vp, i32, i32, vp, i32, i32] + [i32] * 7),
    "dflash_cache_rollback": (i32, [vp, vp, i32]),
    "dflash_cache_clear_transients": (i32, [vp]),
    "dflash_cache_trim": (i64, [vp, i64]),
    "dflash_restore_target_cache_after_acceptance": (i32, [vpp, i32, vp, i64, i32, i32, C.POINTER(i64)]),
}


class DFlashError(RuntimeError):
    """A HIP call failed or the arguments were inconsistent."""


class DFlashUnsupported(DFlashError):
    """The shape/dtype is outside what the kernels cover (the reference would fall back)."""


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise DFlashError(
                f"{LIB_PATH} is missing: build it with `make -C swiftlm_amd/csrc` "
                "(or __graft_entry__.build()); there is no fallback path")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def last_error() -> str:
    return load().dflash_last_error().decode()


def check(rc: int, what: str) -> None:
    if rc == OK:
        return
    msg = f"{what}: {last_error()} (status {rc})"
    if rc == UNSUPPORTED:
        raise DFlashUnsupported(msg)
    raise DFlashError(msg)
