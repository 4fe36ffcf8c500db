"""Verify-step driver for a hybrid GatedDelta / attention stack.

One DFlash verify step over the layers' hot path, in the order the reference's
loop runs it (Sources/DFlash/DFlashRuntime.swift:484-581):

  1. per GatedDelta layer: forward-with-tape from the pre-verify state into a second
     state buffer (the rollback cache is armed by reference, so nothing is copied);
     per attention layer: the block-causal SDPA over offset+16 keys with the append of the
     block's 16 K/V rows at the cache offset fused in (dense caches, or paged pools when
     ``StackConfig.page_size`` is set);
  2. acceptance length / commit count on the device (no host round trip);
  3. rollback: ONE batched tape-replay launch for all GatedDelta layers that reads the
     commit count from device memory and leaves a fully accepted block alone; the KV
     caches "trim" by taking the new offset.

Everything is enqueued through the C ABI on preallocated buffers, with no host
synchronisation and no allocation, so a step can be captured in a HIP graph and
replayed.  The state buffers ping-pong, hence steps come in even/odd pairs.
The per-layer activations (q, k, v, g, beta, the block's K/V rows) are the target
model's; here they are fixed synthetic tensors.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import List, Optional

import torch

from . import _lib


@dataclass
class StackConfig:
    n_layers: int = 48
    attn_every: int = 4            # layer i is attention when (i + 1) % attn_every == 0
    block: int = 16
    # GatedDelta layers (Qwen3-Next linear attention)
    Hk: int = 16
    Hv: int = 32
    Dk: int = 128
    Dv: int = 128
    # attention layers
    Hq: int = 16
    Hkv: int = 2
    D: int = 256
    context: int = 32768           # L0: cached tokens before the first step
    max_steps: int = 64            # sizes the KV capacity
    page_size: int = 0             # 0: dense KV caches; otherwise paged pools with pages of this many keys

    @property
    def capacity(self) -> int:
        return self.context + self.block * (self.max_steps + 1)

    def kinds(self) -> List[str]:
        return ["attn" if (i + 1) % self.attn_every == 0 else "gdn" for i in range(self.n_layers)]


def _p(t: Optional[torch.Tensor]):
    return None if t is None else C.c_void_p(t.data_ptr())


class HybridVerifyStack:
    """Buffers plus the enqueue routine of one verify step."""

    def __init__(self, cfg: StackConfig, seed: int = 0, device: str = "cuda", n_slots: int = 2):
        self.cfg = cfg
        self.lib = _lib.load()
        self.fuse_accept = True      # acceptance decided inside the batched replay launch (one launch fewer per step)
        # False: the forwards do not store the post-block state and the rollback replays the tape also when the whole
        # block is accepted (no counterpart in the reference, whose forward returns that state; the committed state
        # is the same either way)
        self.post_block_state = True
        g = torch.Generator(device=device).manual_seed(seed)
        bf = torch.bfloat16
        T = cfg.block

        def randn(*shape):
            return torch.randn(*shape, generator=g, device=device)

        self.gdn, self.attn = [], []
        for kind in cfg.kinds():
            if kind == "gdn":
                q = torch.nn.functional.normalize(randn(1, T, cfg.Hk, cfg.Dk), dim=-1).to(bf)
                k = torch.nn.functional.normalize(randn(1, T, cfg.Hk, cfg.Dk), dim=-1).to(bf)
                layer = dict(
                    q=q, k=k, v=randn(1, T, cfg.Hv, cfg.Dv).to(bf),
                    beta=torch.sigmoid(randn(1, T, cfg.Hv)).to(bf),
                    g=torch.exp(-torch.nn.functional.softplus(randn(1, T, cfg.Hv))).to(bf),
                    state=[(0.1 * randn(1, cfg.Hv, cfg.Dv, cfg.Dk)).contiguous(),
                           torch.zeros(1, cfg.Hv, cfg.Dv, cfg.Dk, device=device)],
                    y=torch.empty(1, T, cfg.Hv, cfg.Dv, dtype=bf, device=device),
                    tape=torch.empty(1, T, cfg.Hv, cfg.Dv, dtype=torch.float32, device=device))
                self.gdn.append(layer)
            else:
                kc = torch.zeros(1, cfg.Hkv, cfg.capacity, cfg.D, dtype=bf, device=device)
                vc = torch.zeros_like(kc)
                kc[:, :, : cfg.context] = randn(1, cfg.Hkv, cfg.context, cfg.D).to(bf)
                vc[:, :, : cfg.context] = randn(1, cfg.Hkv, cfg.context, cfg.D).to(bf)
                layer = dict(
                    q=randn(1, cfg.Hq, T, cfg.D).to(bf), k_new=randn(1, cfg.Hkv, T, cfg.D).to(bf),
                    v_new=randn(1, cfg.Hkv, T, cfg.D).to(bf), k_cache=kc, v_cache=vc,
                    out=torch.empty(1, cfg.Hq, T, cfg.D, dtype=bf, device=device),
                    lse=torch.empty(1, cfg.Hq, T, dtype=torch.float32, device=device))
                if cfg.page_size:
                    # the same keys in a pool [pages, Hkv, page_size, D] under a shuffled page table
                    P = cfg.page_size
                    pages = (cfg.capacity + P - 1) // P
                    perm = torch.randperm(pages, generator=torch.Generator().manual_seed(seed + len(self.attn)))
                    layer["page_table"] = perm.to(torch.int32).view(1, pages).to(device)
                    for name, dense in (("k_pool", kc), ("v_pool", vc)):
                        padded = torch.zeros(cfg.Hkv, pages * P, cfg.D, dtype=bf, device=device)
                        padded[:, : cfg.capacity] = dense[0]
                        pool = torch.empty(pages, cfg.Hkv, P, cfg.D, dtype=bf, device=device)
                        pool[perm.to(device)] = padded.view(cfg.Hkv, pages, P, cfg.D).transpose(0, 1)
                        layer[name] = pool
                    del layer["k_cache"], layer["v_cache"]
                self.attn.append(layer)
        self.scale = 1.0 / (cfg.D ** 0.5)
        n_max = cfg.capacity
        ws = int(self.lib.dflash_sdpa_workspace_bytes(1, cfg.Hq, cfg.Hkv, T, n_max, cfg.D))
        if self.attn and ws == 0:
            raise _lib.DFlashError("sdpa workspace query failed: " + _lib.last_error())
        self.workspace = torch.empty(max(ws, 256), dtype=torch.uint8, device=device)
        self.n_max = n_max
        # device-side scalars: cache offset L (advanced by the accept kernel) and that kernel's outputs
        self.offset = torch.tensor([cfg.context], dtype=torch.int32, device=device)
        self.accept = torch.zeros(4, dtype=torch.int32, device=device)
        # acceptance inputs of the step being enqueued, one pair per ping-pong phase
        # (one block [phase, ids | posterior, T], so that a caller can hand over both phases with a single copy)
        # (n_slots > 2: a graph that holds more than two steps gives every step its own slot)
        self.accept_inputs = torch.zeros(max(n_slots, 2), 2, T, dtype=torch.int32, device=device)
        self.verify_ids = [self.accept_inputs[i, 0] for i in range(self.accept_inputs.shape[0])]
        self.posterior = [self.accept_inputs[i, 1] for i in range(self.accept_inputs.shape[0])]
        self.phase = 0               # which state buffer holds the pre-verify state
        # host pointer tables for the batched replay, one per phase
        self._tables = []
        for ph in (0, 1):
            mk = lambda ts: (C.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
            self._tables.append(dict(
                tape=mk([l["tape"] for l in self.gdn]), k=mk([l["k"] for l in self.gdn]),
                g=mk([l["g"] for l in self.gdn]), sin=mk([l["state"][ph] for l in self.gdn]),
                sout=mk([l["state"][1 - ph] for l in self.gdn])))

    # -- one step ------------------------------------------------------------------
    def enqueue_step(self, stream: Optional[int] = None, before_launch=None, slot: Optional[int] = None) -> None:
        """Enqueue one verify step.  ``before_launch(name)`` is called ahead of each kernel-launching
        C call with name in {"gdn_forward", "sdpa", "tape_replay"} (used to arm timing brackets).
        ``slot``: which row of ``accept_inputs`` holds this step's token ids (default: the phase)."""
        cfg, lib, T = self.cfg, self.lib, self.cfg.block
        note = before_launch or (lambda name: None)
        st = C.c_void_p(torch.cuda.current_stream().cuda_stream if stream is None else stream)
        ph = self.phase
        slot = ph if slot is None else slot
        gi = ai = 0
        for kind in cfg.kinds():
            if kind == "gdn":
                l = self.gdn[gi]; gi += 1
                note("gdn_forward")
                rc = lib.dflash_gated_delta_tape(
                    st, _p(l["q"]), _p(l["k"]), _p(l["v"]), _p(l["g"]), 3, _p(l["beta"]), _lib.BF16,
                    _p(l["state"][ph]), _p(l["state"][1 - ph]) if self.post_block_state else None, _lib.F32, _p(l["y"]),
                    _p(l["tape"]), None, 0, 1, T, cfg.Hk, cfg.Hv, cfg.Dk, cfg.Dv)
                _lib.check(rc, "gated_delta_tape")
            else:
                l = self.attn[ai]; ai += 1
                hs = cfg.capacity * cfg.D
                note("sdpa")
                if cfg.page_size:
                    kp = l["k_pool"]
                    rc = lib.dflash_sdpa_block_causal_paged(
                        st, _p(l["q"]), _p(kp), _p(l["v_pool"]), _p(l["page_table"]), l["page_table"].shape[1], cfg.page_size,
                        kp.shape[0], kp.stride(0), kp.stride(1), _p(l["k_new"]), _p(l["v_new"]), _p(l["out"]), _p(l["lse"]),
                        _lib.BF16, self.scale, 1, cfg.Hq, cfg.Hkv, T, self.n_max, cfg.D, _p(self.offset), _p(self.workspace),
                        self.workspace.numel())
                    _lib.check(rc, "sdpa_block_causal_paged")
                    continue
                rc = lib.dflash_sdpa_block_causal_append(
                    st, _p(l["q"]), _p(l["k_cache"]), _p(l["v_cache"]), _p(l["k_new"]), _p(l["v_new"]), _p(l["out"]),
                    _p(l["lse"]), _lib.BF16, self.scale, 1, cfg.Hq, cfg.Hkv, T, self.n_max, cfg.D, cfg.Hkv * hs, hs,
                    _p(self.offset), _p(self.workspace), self.workspace.numel())
                _lib.check(rc, "sdpa_block_causal")
        cast = lambda a: C.cast(a, _lib.vpp)
        if self.gdn and self.fuse_accept:
            # acceptance + rollback of every GatedDelta layer in ONE launch: the replay kernel counts the
            # leading matches itself, writes accept[0..3] and advances the offset
            tb = self._tables[ph]
            note("tape_replay")
            rc = lib.dflash_accept_commit_replay_batched(
                st, _p(self.verify_ids[slot]), _p(self.posterior[slot]), T, _p(self.offset), _p(self.accept),
                len(self.gdn), cast(tb["tape"]), _lib.F32, cast(tb["k"]), cast(tb["g"]), _lib.BF16, 3,
                cast(tb["sin"]), cast(tb["sout"]), _lib.F32, 1 if self.post_block_state else 0, 1, T, cfg.Hk, cfg.Hv,
                cfg.Dk, cfg.Dv)
            _lib.check(rc, "accept_commit_replay_batched")
            self.phase = 1 - ph
            return
        # accept: commit count -> accept[1]; offset += commit count
        rc = lib.dflash_accept_commit(st, _p(self.verify_ids[slot]), _p(self.posterior[slot]), T, _p(self.offset),
                                      _p(self.accept))
        _lib.check(rc, "accept_commit")
        # rollback: every GatedDelta layer in one launch, step count read on the device
        if self.gdn:
            tb = self._tables[ph]
            note("tape_replay")
            rc = lib.dflash_tape_replay_batched(
                st, len(self.gdn), cast(tb["tape"]), _lib.F32, cast(tb["k"]), cast(tb["g"]), _lib.BF16, 3,
                cast(tb["sin"]), cast(tb["sout"]), _lib.F32, 0, C.c_void_p(self.accept.data_ptr() + 4),
                1 if self.post_block_state else 0, 1, T, cfg.Hk, cfg.Hv, cfg.Dk, cfg.Dv)
            _lib.check(rc, "tape_replay_batched")
        self.phase = 1 - ph

    # -- launch shapes --------------------------------------------------------------
    def launch_shapes(self):
        """(grid_x, grid_y, grid_z, threads, lds_bytes) of every kernel one step launches, in launch order:
        the shapes the library's host code picks for this configuration (csrc: launch_gdn_chunk, launch_sdpa,
        launch_replay_nr), for pricing a step's launches with empty kernels of the same shapes.  Only the
        benchmark's kernel choices are covered (chunked GatedDelta forward, dense or paged attention with at
        most 8 query heads per KV head, 4 state rows per replay thread)."""
        cfg, T = self.cfg, self.cfg.block
        assert cfg.Dk in (64, 128, 256) and cfg.Dv % 16 == 0 and cfg.Hq // cfg.Hkv <= 8 and cfg.D in (128, 256)
        ld = cfg.Dk + 4
        gdn_lds = (4 * (2 * 32 * ld + 16 * 33 + 2 * 16 * 16 + 16 * 17 + 16 * 16 + 4 * 16 + 16)   # fp32 operands and tables
                   + 2 * 5 * 16 * (cfg.Dk + 8))                                                    # bf16 operands
        gdn = (cfg.Dv // 16, cfg.Hv, 1, 256, gdn_lds)
        # splits: the S whose workspace layout gives the size the library reports
        rows = cfg.Hq * T
        need = int(self.lib.dflash_sdpa_workspace_bytes(1, cfg.Hq, cfg.Hkv, T, self.n_max, cfg.D))
        a256 = lambda x: (x + 255) & ~255
        splits = [S for S in range(1, 513) if a256(a256(a256(rows * S * cfg.D * 2) + rows * S * 4) + rows * S * 4) == need]
        assert len(splits) == 1, "cannot recover the split count from the workspace size"
        row_bytes = cfg.D * 2
        partial = (splits[0], cfg.Hkv, 1, 384, 4 * 32 * row_bytes + 2 * 3 * 32 * row_bytes)
        combine = (rows, 1, 1, 256, 4 * 512 + 16 + 4 * (256 // (cfg.D // 8)) * cfg.D)
        rpp = 256 // (cfg.Dk // 4)
        n_gdn = len(self.gdn)
        assert (cfg.Dv // rpp) * cfg.Hv * n_gdn >= 16 * 256 and cfg.Dv >= 4 * rpp
        tc = 8 if cfg.Dk >= 256 else 16
        replay = (cfg.Dv // (4 * rpp), cfg.Hv, n_gdn, 256, 4 * (tc * cfg.Dk + tc + tc * 4 * rpp + tc))
        out = []
        for kind in cfg.kinds():
            out += [gdn] if kind == "gdn" else [partial, combine]
        if n_gdn:
            out.append(replay)
        return out

    def set_acceptance(self, phase: int, commit_count: int, seed: int = 0) -> None:
        """Stage token ids for the step that will run in ``phase`` so that exactly
        ``commit_count`` tokens get committed (acceptance length commit_count - 1)."""
        T = self.cfg.block
        gen = torch.Generator().manual_seed(seed)
        ids = torch.randint(0, 1000, (T,), generator=gen, dtype=torch.int32)
        post = torch.empty(T, dtype=torch.int32)
        post[: T - 1] = ids[1:]
        post[T - 1] = 7
        a = commit_count - 1
        if a < T - 1:
            post[a] = ids[a + 1] + 1          # first mismatch at position a
        self.verify_ids[phase].copy_(ids, non_blocking=False)
        self.posterior[phase].copy_(post, non_blocking=False)

    # -- algorithmic bytes (the figures the roofline is priced against) -----------
    def gdn_forward_bytes(self) -> int:
        c, T = self.cfg, self.cfg.block
        state = c.Hv * c.Dv * c.Dk * 4
        return 2 * state + (2 * T * c.Hk * c.Dk + T * c.Hv * c.Dv + 2 * T * c.Hv) * 2 + T * c.Hv * c.Dv * 2 + T * c.Hv * c.Dv * 4

    def replay_bytes(self, n: int) -> int:
        c = self.cfg
        return 2 * c.Hv * c.Dv * c.Dk * 4 + n * c.Hv * c.Dv * 4 + n * c.Hk * c.Dk * 2 + n * c.Hv * 2

    def sdpa_bytes(self, n_keys: int) -> int:
        c, T = self.cfg, self.cfg.block
        return 2 * c.Hq * T * c.D * 2 + 2 * c.Hkv * n_keys * c.D * 2 + c.Hq * T * 4
