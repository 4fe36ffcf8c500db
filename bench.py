#!/usr/bin/env python3
"""DFlash verify-step benchmark on one MI355X.

A "step" is one verify step of the hybrid stack of the headline benchmark configuration: 48 layers =
12 x (GatedDelta, GatedDelta, GatedDelta, attention), 16-token draft block, 32K
context, accepted length ~ Geometric(0.25) clipped to [1, 16].  Per step: 36
GatedDelta forwards with tape, 12 KV appends + block-causal SDPAs, the accept kernel
and one batched tape replay, all resident in HBM, enqueued through the C ABI.
Steps are captured in HIP graphs (two steps per graph, the state buffers ping-pong)
unless --no-graph is given.

Prints ONE JSON line.  `value` is microseconds per layer (step time / 48).  The
`roofline` object prices the dominant kernel (the split-KV SDPA partial kernel) against
the 8 TB/s HBM peak using per-launch durations measured with HIP events on the launch
stream; `cpu_baseline` times the C restatement of the reference's CPU (ops) path on
this box's host cores on a bounded sample of the same workload.
"""

from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0


class HipEvents:
    """hipEvent_t pairs created and read through the HIP runtime torch already loaded."""

    def __init__(self):
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [C.c_void_p]
        self.hip.hipEventDestroy.argtypes = [C.c_void_p]
        self.pairs = []

    def pair(self):
        a, b = C.c_void_p(), C.c_void_p()
        assert self.hip.hipEventCreate(C.byref(a)) == 0 and self.hip.hipEventCreate(C.byref(b)) == 0
        self.pairs.append((a, b))
        return a, b

    def durations_us(self):
        out = []
        for a, b in self.pairs:
            assert self.hip.hipEventSynchronize(b) == 0
            ms = C.c_float()
            assert self.hip.hipEventElapsedTime(C.byref(ms), a, b) == 0
            out.append(ms.value * 1e3)
        return out

    def destroy(self):
        for a, b in self.pairs:
            self.hip.hipEventDestroy(a)
            self.hip.hipEventDestroy(b)
        self.pairs = []


def draw_commit_counts(n_steps: int, block: int, seed: int = 1234):
    rng = np.random.default_rng(seed)
    return [int(min(rng.geometric(0.25), block)) for _ in range(n_steps)]


def cpu_baseline(stack_cfg, mean_commit: int):
    """The reference's CPU path is its ops graph on MLX's CPU stream, which cannot be
    built here; its C restatement (oracle/dflash_oracle.c, one full-state pass per array
    op per step) is timed instead, on all host threads, on one GatedDelta layer
    (forward + replay) and one attention layer, scaled by the stack's 36:12 layer mix."""
    from oracle import c_oracle
    from oracle import dflash_oracle as O

    c = stack_cfg
    T = c.block
    d = O.make_gdn_inputs(0, 1, T, c.Hk, c.Hv, c.Dk, c.Dv, in_dtype="bf16")
    threads = c_oracle.num_threads()

    def best(fn, reps):
        fn()
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return min(ts), float(np.median(ts))

    out = {}
    for variant in ("opbyop", "fused"):
        fwd = lambda: c_oracle.gated_delta(d["q"], d["k"], d["v"], d["g"], d["beta"], d["state"], variant=variant)
        y, s, tape = fwd()
        rep = lambda: c_oracle.tape_replay(tape[:, :mean_commit], d["k"][:, :mean_commit], d["g"][:, :mean_commit],
                                           d["state"], variant=variant)
        out[variant] = (best(fwd, 20)[1], best(rep, 20)[1])
    q, k, v = O.make_sdpa_inputs(1, 1, c.Hq, c.Hkv, T, c.context, c.D)
    t_sdpa = best(lambda: c_oracle.sdpa_block_causal(q, k, v, 1.0 / np.sqrt(c.D)), 3)[1]
    n_gdn = sum(1 for x in c.kinds() if x == "gdn")
    n_attn = c.n_layers - n_gdn
    per_layer = lambda fr: (n_gdn * (fr[0] + fr[1]) + n_attn * t_sdpa) / c.n_layers * 1e6
    return {
        "value": round(per_layer(out["opbyop"]), 1),
        "unit": "us/layer",
        "cores": threads,
        "kind": "port",
        "sample": (f"C restatement of the ops path, {threads} OpenMP threads: 1 GatedDelta layer (forward T={T} + "
                   f"replay n={mean_commit}, median of 20) and 1 SDPA layer at L={c.context} (median of 3), weighted "
                   f"{n_gdn}:{n_attn} over {c.n_layers} layers"),
        "fused_variant_us_per_layer": round(per_layer(out["fused"]), 1),
        "gdn_forward_us": round(out["opbyop"][0] * 1e6, 1),
        "tape_replay_us": round(out["opbyop"][1] * 1e6, 1),
        "sdpa_us": round(t_sdpa * 1e6, 1),
    }


def aux_kernels(lib, cfg, reps=48):
    """The kernels on either side of the measured path, at the benchmark's shapes, each timed with
    events attached to its dispatch over `reps` launches on rotating buffers (inputs come from HBM):
    the GatedDelta pre-ops of one layer's 16-token block and the greedy tokens over [16, vocab]
    logits fused with the acceptance bookkeeping.  Not part of `value`."""
    import torch
    from swiftlm_amd import DFlashKernels as K, DFlashRuntime as R, _lib

    out = {}
    dev, bf = "cuda", torch.bfloat16
    g = torch.Generator(device=dev).manual_seed(11)
    B, T, Hk, Hv, Dk, Dv, Kc = 1, cfg.block, cfg.Hk, cfg.Hv, cfg.Dk, cfg.Dv, 4
    C = 2 * Hk * Dk + Hv * Dv
    sets = [(torch.randn(B, T, C, generator=g, device=dev).to(bf), torch.randn(B, Kc - 1, C, generator=g, device=dev).to(bf),
             torch.randn(B, T, Hv, generator=g, device=dev).to(bf), torch.randn(B, T, Hv, generator=g, device=dev).to(bf))
            for _ in range(reps)]
    w = (0.5 * torch.randn(C, Kc, generator=g, device=dev)).to(bf)
    a_log = torch.randn(Hv, generator=g, device=dev)
    dt_bias = torch.randn(Hv, generator=g, device=dev)
    ev = HipEvents()
    for x, st, a, b in sets[:4]:
        K.gdn_prepare(x, st, w, a, b, a_log, dt_bias, Hk, Hv, Dk, Dv, 1.0 / Dk, Dk ** -0.5)
    for x, st, a, b in sets:
        e0, e1 = ev.pair()
        _lib.check(lib.dflash_profile_next_launch(_lib.KERNEL_GDN_PREPARE, e0, e1), "profile_next_launch")
        K.gdn_prepare(x, st, w, a, b, a_log, dt_bias, Hk, Hv, Dk, Dv, 1.0 / Dk, Dk ** -0.5)
    torch.cuda.synchronize()
    us = float(np.median(ev.durations_us()))
    nbytes = (2 * T * C + 2 * (Kc - 1) * C + Kc * C + 4 * T * Hv) * 2        # x in/out, window in/out, taps, a/b/g/beta
    out["gdn_prepare"] = {"us": round(us, 2), "algorithmic_bytes": nbytes, "gbs": round(nbytes / us / 1e3, 1),
                          "shape": "B=1 T=%d C=%d K=%d bf16" % (T, C, Kc)}
    ev.destroy()
    del sets

    V = 151936
    logits = [torch.randn(T, V, generator=g, device=dev).to(bf) for _ in range(reps)]      # 48 x 4.9 MB
    mask = R.build_suppress_token_mask(V, [1, 2, 3])
    verify = torch.randint(0, V, (T,), generator=g, device=dev, dtype=torch.int32)
    for lg in logits[:4]:
        R.greedy_accept_commit(lg, mask, verify, 0)
    ev = HipEvents()
    for lg in logits:
        e0, e1 = ev.pair()
        _lib.check(lib.dflash_profile_next_launch(_lib.KERNEL_GREEDY_PARTIAL, e0, e1), "profile_next_launch")
        R.greedy_accept_commit(lg, mask, verify, 0)
    torch.cuda.synchronize()
    us = float(np.median(ev.durations_us()))
    nbytes = T * V * 2 + V
    out["greedy_partial"] = {"us": round(us, 2), "algorithmic_bytes": nbytes, "gbs": round(nbytes / us / 1e3, 1),
                             "shape": "T=%d V=%d bf16, uint8 suppress mask" % (T, V)}
    ev.destroy()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-graph", action="store_true", help="enqueue every step from the host instead of replaying graphs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--context", type=int, default=32768)
    ap.add_argument("--aux", action="store_true",
                    help="also time the kernels next to the measured path (pre-ops, greedy tokens) and report them "
                         "under aux_kernels; they are not part of the step time")
    ap.add_argument("--page-size", type=int, default=0,
                    help="keep the attention layers' K/V in paged pools with pages of this many keys (0: dense caches, "
                         "the configuration the headline number is quoted on)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB device copy, the known-size kernel the rocprof byte counters are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")

    import torch

    from swiftlm_amd import _lib
    from swiftlm_amd.verify_step import HybridVerifyStack, StackConfig

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU (there is no CPU path in the product)")
    torch.cuda.set_device(0)
    lib = _lib.load()
    _lib.check(lib.dflash_init(), "dflash_init")

    K, W = args.steps, args.warmup
    brk_steps = min(max(K, 1), 16)                 # eager pass with events attached to the kernels
    total = 2 + W + K + brk_steps
    cfg = StackConfig(context=args.context, max_steps=total + 2, page_size=args.page_size)
    stack = HybridVerifyStack(cfg, seed=0)
    T = cfg.block
    commits = draw_commit_counts(total, T)
    # token ids of every step, staged on the device once
    ids = torch.empty(total, T, dtype=torch.int32)
    post = torch.empty(total, T, dtype=torch.int32)
    gen = torch.Generator().manual_seed(5)
    for s, cc in enumerate(commits):
        row = torch.randint(0, 1000, (T,), generator=gen, dtype=torch.int32)
        p = torch.empty(T, dtype=torch.int32)
        p[: T - 1] = row[1:]
        p[T - 1] = 7
        if cc - 1 < T - 1:
            p[cc - 1] = row[cc] + 1                # first mismatch -> acceptance length cc - 1
        ids[s], post[s] = row, p
    # [step, ids | posterior, T]: one device-to-device copy hands a step its token ids (what the drafter and the
    # target's argmax would leave on the device), two consecutive steps' worth when a graph holds two steps
    staged_d = torch.stack([ids, post], dim=1).cuda()
    step_no = [0]

    def stage(phase):
        s = step_no[0]
        stack.accept_inputs[phase].copy_(staged_d[s], non_blocking=True)
        step_no[0] += 1

    def stage_pair(phase):
        s = step_no[0]
        if phase == 0:
            stack.accept_inputs.copy_(staged_d[s:s + 2], non_blocking=True)
        else:
            stage(phase); stage(1 - phase)
            return
        step_no[0] += 2

    def eager_step(before_launch=None):
        stage(stack.phase)
        stack.enqueue_step(before_launch=before_launch)

    # two eager steps first: loads code objects, sets LDS attributes (not legal during capture)
    eager_step(); eager_step()
    torch.cuda.synchronize()
    assert int(stack.offset) == cfg.context + commits[0] + commits[1], "device-side commit bookkeeping is off"

    graphs = None
    if not args.no_graph:
        # one graph per starting phase of the ping-pong state buffers, two steps each
        graphs = {}
        side = torch.cuda.Stream()
        for ph in (0, 1):
            stack.phase = ph
            side.wait_stream(torch.cuda.current_stream())
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                stack.enqueue_step()
                stack.enqueue_step()
            torch.cuda.current_stream().wait_stream(side)
            graphs[ph] = g
        stack.phase = 0
        torch.cuda.synchronize()

    def run(n_steps):
        for _ in range(n_steps // 2):
            if graphs is not None:
                ph = stack.phase
                stage_pair(ph)
                graphs[ph].replay()
            else:
                eager_step(); eager_step()
        if n_steps & 1:
            eager_step()

    run(W)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    run(K)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    timed_steps = K
    ms_per_step = dt * 1e3 / max(K, 1)
    us_per_layer = ms_per_step * 1e3 / cfg.n_layers

    # ---- per-kernel durations with HIP events on the launch stream (eager pass) ----
    ev = HipEvents()
    n_attn, n_gdn = len(stack.attn), len(stack.gdn)
    kv_before = int(stack.offset)
    idx = {"sdpa_partial": [], "sdpa_combine": [], "gdn_forward": [], "tape_replay": []}

    def arm(name):
        def one(kernel_id, key):
            a, b = ev.pair()
            idx[key].append(len(ev.pairs) - 1)
            _lib.check(lib.dflash_profile_next_launch(kernel_id, a, b), "profile_next_launch")
        if name == "sdpa":
            one(_lib.KERNEL_SDPA_PARTIAL, "sdpa_partial")
            one(_lib.KERNEL_SDPA_COMBINE, "sdpa_combine")
        elif name == "gdn_forward":
            one(_lib.KERNEL_GDN_FORWARD, "gdn_forward")
        else:
            one(_lib.KERNEL_TAPE_REPLAY, "tape_replay")

    for _ in range(brk_steps):
        eager_step(before_launch=arm)
    torch.cuda.synchronize()
    durs = ev.durations_us()
    avg = lambda key: float(np.mean([durs[i] for i in idx[key]])) if idx[key] else float("nan")
    sdpa_us, comb_us, fwd_us, rep_us = avg("sdpa_partial"), avg("sdpa_combine"), avg("gdn_forward"), avg("tape_replay")
    sdpa_launches = len(idx["sdpa_partial"])
    ev.destroy()
    kv_mid = (kv_before + int(stack.offset)) // 2 + T
    sdpa_bytes = stack.sdpa_bytes(kv_mid)
    achieved = sdpa_bytes / (sdpa_us * 1e-6) / 1e9

    # counter-measured bytes per launch: only for the workload the counters were collected on
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "sdpa_partial_traffic.json")
    if os.path.exists(tpath) and args.context == 32768 and not args.page_size:
        try:
            tj = json.load(open(tpath))
            if tj.get("workload") == "config4 L=32768":
                traffic = tj.get("hbm_bytes_per_launch")
        except Exception:
            traffic = None

    mean_commit = int(round(float(np.mean(commits))))
    step_bytes = n_gdn * (stack.gdn_forward_bytes() + stack.replay_bytes(mean_commit)) + n_attn * sdpa_bytes
    result = {
        "metric": "dflash_verify_us_per_layer",
        "value": round(us_per_layer, 3),
        "unit": "us/layer",
        "n_gpus": 1,
        "steps": timed_steps,
        "warmup": W,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": ("config4: DFlash verify step of a hybrid stack, 48 layers = 12 x (3 GatedDelta + 1 attention), "
                         "16-token block, L=%d, accepted n ~ Geometric(0.25) in [1,16]; GatedDelta Hk=16 Hv=32 dk=dv=128 "
                         "fp32 state; attention Hq=16 Hkv=2 D=256 bf16") % cfg.context,
            "layers": cfg.n_layers, "block": T, "context": cfg.context,
            "launch": "eager" if graphs is None else "hip-graph, 2 steps per graph",
            "kv_layout": "dense" if not cfg.page_size else "paged, %d-key pages" % cfg.page_size,
        },
        "step_hbm_algorithmic_gbs": round(step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
        "step_frac_of_hbm_peak": round(step_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
        "kernel_us": {"sdpa_partial": round(sdpa_us, 2), "sdpa_combine": round(comb_us, 2),
                      "gdn_forward_tape": round(fwd_us, 2), "tape_replay_batched_36_layers": round(rep_us, 2)},
        "roofline": {
            "kernel": "sdpa_partial_kernel<bf16,256>",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": traffic,
            "algorithmic_bytes_per_launch": sdpa_bytes,
            "avg_launch_us": round(sdpa_us, 2),
            "launches_timed": sdpa_launches,
        },
    }
    if args.aux:
        result["aux_kernels"] = aux_kernels(lib, cfg)
    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        result["calibration_copy_bytes"] = int(src.numel())
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cfg, mean_commit)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
