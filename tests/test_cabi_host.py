"""CPU-side checks of the C-ABI library: it loads, exports every symbol the
headers declare, and its host-only logic (cache bookkeeping, argument
validation) behaves like the reference.  No kernel is launched here."""

import ctypes as C
import os
import re

import pytest

from oracle import dflash_oracle as O
from swiftlm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    names = set()
    for h in ("dflash_hip.h", "dflash_cache.h", "dflash_profile.h"):
        text = open(os.path.join(ROOT, "include", h)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names |= set(re.findall(r"\b(dflash_[a-z0-9_]+)\s*\(", text))
    return names


def test_library_exports_every_declared_symbol():
    lib = C.CDLL(_lib.LIB_PATH)
    declared = _declared_symbols()
    assert len(declared) >= 26
    for name in sorted(declared):
        assert hasattr(lib, name), f"{name} declared in include/ but not exported"
    assert declared == set(_lib.SIGNATURES), "ctypes table and headers disagree"


def test_version_and_error_text():
    lib = _lib.load()
    assert lib.dflash_version() == 100
    assert isinstance(_lib.last_error(), str)


def test_modulemap_names_the_header():
    mm = open(os.path.join(ROOT, "include", "module.modulemap")).read()
    assert 'header "dflash_hip.h"' in mm and 'header "dflash_cache.h"' in mm and 'link "dflash_hip"' in mm


# ---- cache bookkeeping (host only; device pointers are never dereferenced) ----


def _cache(kind):
    h = C.c_void_p(_lib.load().dflash_cache_create(kind, 4))
    assert h
    return h


def test_cache_create_rejects_bad_kind():
    assert not _lib.load().dflash_cache_create(9, 4)
    assert "bad kind" in _lib.last_error()


def test_cache_arm_snapshot_and_clear():
    lib = _lib.load()
    c = _cache(_lib.CACHE_TAPE)
    lib.dflash_cache_set_slot(c, 0, 0x1000)
    lib.dflash_cache_set_slot(c, 1, 0x2000)
    assert not lib.dflash_cache_is_armed(c)
    assert lib.dflash_cache_arm_rollback(c, 7) == 0
    assert lib.dflash_cache_is_armed(c)
    # rollback without a recorded tape restores the snapshot pointers and disarms
    lib.dflash_cache_set_slot(c, 0, 0x3000)
    lib.dflash_cache_set_slot(c, 1, 0x4000)
    assert lib.dflash_cache_rollback(c, None, 2) == 0
    assert lib.dflash_cache_get_slot(c, 0) == 0x1000 and lib.dflash_cache_get_slot(c, 1) == 0x2000
    assert not lib.dflash_cache_is_armed(c)
    # rollback when never armed is a no-op (RecurrentRollbackCache.swift:96-99)
    lib.dflash_cache_set_slot(c, 1, 0x5000)
    assert lib.dflash_cache_rollback(c, None, 0) == 0
    assert lib.dflash_cache_get_slot(c, 1) == 0x5000
    lib.dflash_cache_destroy(c)


def test_cache_rollback_requires_functional_update():
    lib = _lib.load()
    c = _cache(_lib.CACHE_TAPE)
    lib.dflash_cache_set_slot(c, 0, 0x1000)
    lib.dflash_cache_set_slot(c, 1, 0x2000)
    lib.dflash_cache_arm_rollback(c, 0)
    rc = lib.dflash_cache_record_tape(c, 0x10, _lib.F32, 0x20, 0x30, _lib.BF16, 3, None, 2, _lib.F32,
                                      1, 16, 16, 32, 128, 128, 0)
    assert rc == 0
    # slot 1 still points at the pre-verify buffer: refusing beats corrupting the snapshot
    assert lib.dflash_cache_rollback(c, None, 3) == _lib.INVALID
    assert "pre-verify" in _lib.last_error()
    # a refused rollback changes nothing: still armed, slots as they were, so the caller can correct and retry
    assert lib.dflash_cache_is_armed(c)
    assert lib.dflash_cache_get_slot(c, 0) == 0x1000 and lib.dflash_cache_get_slot(c, 1) == 0x2000
    lib.dflash_cache_destroy(c)


def test_restore_validates_every_cache_before_touching_any():
    """A list whose LAST cache cannot be rolled back (slot 1 still holds the pre-verify buffer), or that holds a
    null handle, is refused as a whole: the caches before it keep their snapshot, tape, armed flag and offsets."""
    lib = _lib.load()
    good, kv, bad = _cache(_lib.CACHE_SNAPSHOT), _cache(_lib.CACHE_KV), _cache(_lib.CACHE_TAPE)
    lib.dflash_cache_set_slot(good, 1, 0x2000)
    lib.dflash_cache_arm_rollback(good, 100)
    lib.dflash_cache_set_slot(good, 1, 0x4000)
    lib.dflash_cache_set_offset(kv, 116)
    lib.dflash_cache_set_slot(bad, 0, 0x1000)
    lib.dflash_cache_set_slot(bad, 1, 0x2000)
    lib.dflash_cache_arm_rollback(bad, 100)
    assert lib.dflash_cache_record_tape(bad, 0x10, _lib.F32, 0x20, 0x30, _lib.BF16, 3, None, 2, _lib.F32,
                                        1, 16, 16, 32, 128, 128, 0) == 0
    for handles in ([good, kv, bad], [good, kv, C.c_void_p(None)]):
        arr = (C.c_void_p * 3)(*[h.value for h in handles])
        rc = lib.dflash_restore_target_cache_after_acceptance(C.cast(arr, _lib.vpp), 3, None, 104, 3, 15, None)
        assert rc == _lib.INVALID
        assert lib.dflash_cache_is_armed(good) and lib.dflash_cache_get_slot(good, 1) == 0x4000
        assert lib.dflash_cache_offset(kv) == 116
        assert lib.dflash_cache_is_armed(bad) and lib.dflash_cache_get_slot(bad, 1) == 0x2000
    for h in (good, kv, bad):
        lib.dflash_cache_destroy(h)


def test_snapshot_cache_restores_pointers():
    lib = _lib.load()
    c = _cache(_lib.CACHE_SNAPSHOT)
    lib.dflash_cache_set_slot(c, 0, 0x1000)
    lib.dflash_cache_set_slot(c, 1, 0x2000)
    lib.dflash_cache_arm_rollback(c, 0)
    assert lib.dflash_cache_record_tape(c, 0x10, 0, 0x20, 0x30, 1, 3, None, 2, 0, 1, 16, 16, 32, 128, 128, 0) == 0
    lib.dflash_cache_set_slot(c, 0, 0x3000)
    lib.dflash_cache_set_slot(c, 1, 0x4000)
    assert lib.dflash_cache_rollback(c, None, 5) == 0
    assert lib.dflash_cache_get_slot(c, 0) == 0x1000 and lib.dflash_cache_get_slot(c, 1) == 0x2000
    lib.dflash_cache_destroy(c)


def test_trim_semantics():
    lib = _lib.load()
    c = _cache(_lib.CACHE_KV)
    lib.dflash_cache_set_offset(c, 5)
    assert lib.dflash_cache_trim(c, 8) == 5 and lib.dflash_cache_offset(c) == 0
    lib.dflash_cache_set_offset(c, 20)
    assert lib.dflash_cache_trim(c, 8) == 8 and lib.dflash_cache_offset(c) == 12
    assert lib.dflash_cache_arm_rollback(c, 0) == _lib.INVALID
    lib.dflash_cache_destroy(c)


@pytest.mark.parametrize("acc,drafted", [(15, 15), (3, 15), (0, 15), (0, 0)])
def test_restore_matches_oracle_actions(acc, drafted):
    """Offsets and armed flags after restoreTargetCacheAfterAcceptance follow the
    oracle's action list (DFlashRuntime.swift:188-223).  No tape is recorded, so no
    kernel is launched."""
    lib = _lib.load()
    kinds = [_lib.CACHE_TAPE, _lib.CACHE_KV, _lib.CACHE_MAMBA, _lib.CACHE_KV, _lib.CACHE_SNAPSHOT]
    names = {_lib.CACHE_TAPE: "rollback", _lib.CACHE_SNAPSHOT: "rollback", _lib.CACHE_MAMBA: "mamba",
             _lib.CACHE_KV: "kv"}
    offsets = [0, 116, 90, 100, 0]
    target_len = 100 + acc + 1
    hs = [_cache(k) for k in kinds]
    for h, k, off in zip(hs, kinds, offsets):
        lib.dflash_cache_set_offset(h, off)
        if k in (_lib.CACHE_TAPE, _lib.CACHE_SNAPSHOT):
            lib.dflash_cache_set_slot(h, 1, 0x2000)
            lib.dflash_cache_arm_rollback(h, 100)
            lib.dflash_cache_set_slot(h, 1, 0x4000)
    arr = (C.c_void_p * len(hs))(*[h.value for h in hs])
    ns = C.c_int64(-1)
    rc = lib.dflash_restore_target_cache_after_acceptance(C.cast(arr, _lib.vpp), len(hs), None, target_len, acc,
                                                          drafted, C.byref(ns))
    assert rc == 0 and ns.value >= 0
    want = O.restore_target_cache_after_acceptance([(names[k], o) for k, o in zip(kinds, offsets)], target_len, acc,
                                                   drafted)
    for h, k, off, action in zip(hs, kinds, offsets, want):
        if action[0] == "clear":
            assert not lib.dflash_cache_is_armed(h)
            assert lib.dflash_cache_get_slot(h, 1) == 0x4000          # keeps the verify forward's state
        elif action[0] == "rollback":
            assert not lib.dflash_cache_is_armed(h)
            assert lib.dflash_cache_get_slot(h, 1) == 0x2000          # snapshot restored (no tape recorded)
        elif action[0] == "set_offset":
            assert lib.dflash_cache_offset(h) == action[1]
        elif action[0] == "trim":
            assert lib.dflash_cache_offset(h) == off - action[1] == target_len
        else:
            assert lib.dflash_cache_offset(h) == off
        lib.dflash_cache_destroy(h)


def test_argument_validation_needs_no_gpu_for_null_checks():
    # Null handles are rejected before anything touches a device.
    lib = _lib.load()
    assert lib.dflash_cache_rollback(None, None, 0) == _lib.INVALID
    assert lib.dflash_cache_set_slot(None, 0, None) == _lib.INVALID
    assert lib.dflash_restore_target_cache_after_acceptance(None, 3, None, 0, 0, 0, None) == _lib.INVALID


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits non-zero without touching a device."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr)
