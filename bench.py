#!/usr/bin/env python3
"""Benchmark of the SR-AdamW step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama8b]

A "step" is one ``AdamW.step()`` over the whole synthetic parameter set, with
params, grads and both states already resident in HBM (or, for the streamed
workload, params/states in pinned host memory).  Prints ONE JSON line:

  value      elements updated per second over the K timed steps (wall clock
             around the steps, device synchronised on both sides)
  roofline   algorithmic HBM bytes per launch / mean kernel time of the update
             kernel, the kernel time taken with HIP events on the launch stream
             inside the library; peak = 8 TB/s
  cpu_baseline  the same ATen op sequence the reference issues
             (ramtorch/stochastic_optimizers/adamw.py:160-222), on CPU tensors
             with all host threads, on a bounded sample; plus the scalar C
             oracle on one thread

Workloads (synthetic, value distributions param~N(0,0.02), grad~N(0,1e-3),
ema~N(0,1e-4), ema_squared=N(0,1e-3)^2, stored bf16):
  llama8b   Llama-3-8B-shaped set, 290 tensors, 8 030 257 152 elements, all bf16,
            Philox seed 1234, first timed step is step 100            [default]
  cfg0      one 4096x4096 weight, explicit int16 noise, step 10
  small     20 000 small tensors (length log-uniform in [1,4096]) + 64 x 1024x1024
  mixed     Llama-3-8B shapes; bf16 p and ema, fp32 ema_squared, fp32 grads scaled
            by 1024 and unscaled in-kernel, global-norm clip to 1.0
  streamed  Llama-3-8B shapes with p/ema/ema_squared in pinned host memory,
            bf16 grads on the GPU, 256 MB chunks (--stream-gb bounds the host set)
  hooked    the same set, but each tensor is updated by AdamW.step_param() as a
            backward pass would hand its gradient over (last tensor first), and
            step() only waits: the grad hand-off from ramtorch.Linear's
            post-accumulate hook
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the update kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script (scaled by the counters' readings for kernels of known size in the same runs).
MEASURED_TRAFFIC_BYTES = {"llama8b": 112_546_390_426}
HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
METRIC = "SR-AdamW step: params/sec + achieved HBM GB/s (% of peak), 8B bf16 set, 1 GPU"


# ---- workload shapes -------------------------------------------------------------------------
def llama3_8b_shapes(layers: int = 32):
    """embed and lm_head 128256x4096; per layer q/o 4096x4096, k/v 1024x4096,
    gate/up 14336x4096, down 4096x14336, two RMSNorm vectors of 4096."""
    shapes = [(128256, 4096)]
    for _ in range(layers):
        shapes += [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096),      # q k v o
                   (14336, 4096), (14336, 4096), (4096, 14336), (4096,), (4096,)]
    shapes.append((128256, 4096))
    return shapes


def small_tensor_shapes(seed: int = 1234, count: int = 20_000, big: int = 64):
    import numpy as np
    rng = np.random.default_rng(seed)
    lens = np.floor(np.exp(rng.uniform(0.0, math.log(4096.0), count))).astype(np.int64).clip(1, 4096)
    return [(int(n),) for n in lens] + [(1024, 1024)] * big


def numel(shape):
    n = 1
    for s in shape:
        n *= s
    return n


def fill_tensor(shape, kind: str, seed: int, dtype, device):
    """Synthetic values of one array, drawn in fp32 on `device` and stored as `dtype`."""
    import torch
    gen = torch.Generator(device=device).manual_seed(seed)
    n = numel(shape)
    out = torch.empty(n, dtype=dtype, device=device)
    step = 1 << 28  # bound the fp32 temporary
    for lo in range(0, n, step):
        k = min(step, n - lo)
        x = torch.randn(k, device=device, generator=gen)
        if kind == "p":
            x.mul_(0.02)
        elif kind == "g":
            x.mul_(1e-3)
        elif kind == "m":
            x.mul_(1e-4)
        else:
            x.mul_(1e-3).square_()
        out[lo:lo + k] = x
    return out.view(shape)


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


# ---- CPU baseline ----------------------------------------------------------------------------
def cpu_baseline():
    """The reference's op sequence on CPU tensors (its step() cannot run without a GPU, so
    this restatement is what is timed), all host threads, including the three randint
    draws per tensor that the reference pays for.  Bounded sample of the same workload: the
    nine tensors of one transformer layer of the Llama-3-8B-shaped set (218 112 000 elements),
    best of 2 passes after a warm-up pass."""
    import numpy as np
    import torch
    import oracle
    from oracle import torch_ops

    shapes = llama3_8b_shapes(1)[1:-1]
    n = sum(numel(s) for s in shapes)
    sets = [tuple(fill_tensor(shp, kind, 4 * i + k, torch.bfloat16, "cpu") for k, kind in enumerate("pgmv"))
            for i, shp in enumerate(shapes)]
    best = float("inf")
    for it in range(3):
        t0 = time.perf_counter()
        for P, G, M, V in sets:
            torch_ops.reference_step_ops(P, G, M, V, step=10 + it, noise=None, **HP)
        dt = time.perf_counter() - t0
        if it:
            best = min(best, dt)
    threads = torch.get_num_threads()
    del sets

    # scalar C restatement, one thread, explicit noise (no RNG cost)
    k = 1 << 22
    p, g, m, v = oracle.synth_inputs(k, 1)
    noise = oracle.synth_noise(k, 1)
    sc = oracle.scalars_from_hparams(step=10, **HP)
    t0 = time.perf_counter()
    oracle.step_tensor(p, g, m, v, sc, noise=noise)
    c_dt = time.perf_counter() - t0
    return {
        "value": n / best, "unit": "elements/s", "cores": threads, "kind": "port",
        "sample": f"torch-op restatement of adamw.py:160-222 on CPU tensors, one transformer layer of the set "
                  f"({len(shapes)} tensors, {n} elements), best of 2 passes, {threads} threads, {cpu_model()}",
        "ms_per_sample": best * 1e3,
        "c_oracle_1thread_elements_per_s": k / c_dt,
    }


# ---- GPU workloads ----------------------------------------------------------------------------
def build_resident(shapes, *, g_dtype, v_dtype, device, seed=1234):
    import torch
    # parameters first, gradients afterwards: the order a framework allocates them in (model
    # construction, then the backward pass), so a parameter and its gradient are not neighbours
    params, grads = [], []
    for i, shp in enumerate(shapes):
        params.append(torch.nn.Parameter(fill_tensor(shp, "p", seed + 4 * i, torch.bfloat16, device),
                                         requires_grad=False))
    for i, shp in enumerate(shapes):
        g = fill_tensor(shp, "g", seed + 4 * i + 1, torch.float32 if g_dtype == torch.float32 else torch.bfloat16,
                        device)
        if g_dtype == torch.float32:
            g.mul_(1024.0)
        grads.append(g)
    return params, grads


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama8b", choices=["llama8b", "cfg0", "small", "mixed", "streamed", "hooked"])
    ap.add_argument("--layers", type=int, default=32, help="transformer layers of the Llama-shaped set")
    ap.add_argument("--stream-gb", type=float, default=48.2, help="upper bound on pinned host bytes (streamed)")
    ap.add_argument("--stream-chunk-mb", type=int, default=256, help="bytes of bf16 per staged chunk and array (streamed)")
    ap.add_argument("--state-placement", default="auto", choices=["auto", "plain"],
                    help="AdamW(state_placement=...): 'auto' puts ema and ema_squared into different HBM regions")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibrate", action="store_true",
                    help="also launch one plain elementwise kernel that reads 1 GiB and writes 1 GiB, so that "
                         "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can be scaled to bytes")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; the step needs no exchange between GPUs and a multi-GPU "
              "figure is not part of it (it would shard by tensor, as ZeRO-1 does). Use --gpus 1.", file=sys.stderr)
        return 2

    import torch
    import ramtorch_amd
    from ramtorch_amd.stochastic_optimizers import adamw as adamw_mod

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        return 1
    dev = "cuda:0"
    torch.cuda.set_device(0)
    wl = args.workload
    first_step = 100
    noise = None
    opt_kw = dict(storage_device="cuda", seed=1234, state_placement=args.state_placement)
    bytes_per_elem = 14
    dtype_label = "f32"  # arithmetic type; storage is bf16 (or fp32 for the mixed layout)
    if wl == "llama8b":
        shapes = llama3_8b_shapes(args.layers)
        params, grads = build_resident(shapes, g_dtype=torch.bfloat16, v_dtype=torch.bfloat16, device=dev)
        state_dtype = torch.bfloat16
    elif wl == "cfg0":
        shapes = [(4096, 4096)]
        params, grads = build_resident(shapes, g_dtype=torch.bfloat16, v_dtype=torch.bfloat16, device=dev)
        state_dtype = torch.bfloat16
        first_step = 10
        bytes_per_elem = 20
    elif wl == "small":
        shapes = small_tensor_shapes()
        params, grads = build_resident(shapes, g_dtype=torch.bfloat16, v_dtype=torch.bfloat16, device=dev)
        state_dtype = torch.bfloat16
    elif wl == "mixed":
        shapes = llama3_8b_shapes(args.layers)
        params, grads = build_resident(shapes, g_dtype=torch.float32, v_dtype=torch.float32, device=dev)
        state_dtype = torch.bfloat16
        opt_kw.update(loss_scale=1024.0, max_grad_norm=1.0, ema_squared_dtype=torch.float32)
        bytes_per_elem = 24
    else:  # streamed / hooked
        shapes = llama3_8b_shapes(args.layers)
        budget = int(args.stream_gb * 1e9)
        kept, used = [], 0
        for shp in shapes:
            if used + 6 * numel(shp) > budget:
                break
            kept.append(shp)
            used += 6 * numel(shp)
        shapes = kept
        params, grads = [], []
        for i, shp in enumerate(shapes):
            p = fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev).cpu().pin_memory()
            params.append(torch.nn.Parameter(p, requires_grad=False))
            grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.bfloat16, dev))
        state_dtype = torch.bfloat16
        opt_kw = dict(storage_device="cpu", seed=1234, stream_chunk_bytes=args.stream_chunk_mb << 20)
        bytes_per_elem = 12
        if wl == "hooked":
            gmap_needed = False

    total = sum(numel(s) for s in shapes)
    opt = ramtorch_amd.AdamW(params, dtype=state_dtype, **HP, **opt_kw)
    for i, p in enumerate(params):
        st = opt.state[p]
        st["step"] = first_step - 1 - args.warmup
        # the states stay the tensors the optimizer allocated (and placed); only their contents are set
        st["ema"].copy_(fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev))
        st["ema_squared"].copy_(fill_tensor(p.shape, "v", 1234 + 4 * i + 3, st["ema_squared"].dtype, dev))
    if wl == "cfg0":
        noise = {params[0]: tuple(torch.randint(-32768, 32768, (4096, 4096), dtype=torch.int16, device=dev,
                                                generator=torch.Generator(dev).manual_seed(1234 + k))
                                  for k in (1, 2, 3))}
    gmap = dict(zip(params, grads))
    if wl in ("small", "llama8b"):
        # bf16 gradients of bf16 params live in .grad, as after a backward pass; from 256
        # tensors on step() then collects its descriptors in C++
        for p, g in zip(params, grads):
            p.grad = g
        gmap = None
    torch.cuda.synchronize()

    handle = adamw_mod._handle(0)
    if "RT_MAX_INFLIGHT_CALLS" in os.environ:  # experiment knob: chunks step_param may queue ahead
        opt.max_inflight_calls = int(os.environ["RT_MAX_INFLIGHT_CALLS"])
    if "RT_POLL_SECONDS" in os.environ:
        opt._poll_seconds = float(os.environ["RT_POLL_SECONDS"])

    def one_step():
        if wl == "hooked":
            for p, g in zip(reversed(params), reversed(grads)):
                opt.step_param(p, g)
            opt.step()
        else:
            opt.step(noise=noise, grads=gmap)

    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize()
    resident = wl not in ("streamed", "hooked")
    if resident:
        # the library records a HIP event pair around the update kernels of every launch, on the
        # launch stream; nothing is read back before the timed region has ended
        handle.set_timing(True)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    kernel_times = handle.kernel_ms_history(min(args.steps, 256)) if resident else []
    if resident:
        handle.set_timing(False)

    # kernel time of the update launch: mean over the launches of the timed region (the most
    # recent 256 when there were more), from the event pairs recorded above
    roofline = None
    stream_info = None
    if resident:
        ks = kernel_times
        k_ms = sum(ks) / len(ks)
        # the update launch moves 14 (20 with explicit noise; 20 for the mixed layout, whose
        # norm pass is a separate launch of 4 B/elem) bytes per element
        upd_bytes = {"llama8b": 14, "small": 14, "cfg0": 20, "mixed": 20}[wl] * total
        achieved = upd_bytes / (k_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                    "frac": achieved / HBM_PEAK_GBPS,
                    "traffic": MEASURED_TRAFFIC_BYTES.get(wl) if args.layers == 32 else None,
                    "kernel": "sr_adamw_fast_wide_kernel" if wl == "mixed" else "sr_adamw_fast_kernel",
                    "kernel_ms": k_ms, "kernel_launches_timed": len(ks), "algorithmic_bytes_per_launch": upd_bytes}
        # What the same traffic pattern reaches with the arithmetic removed (the all-bf16 pattern:
        # 8 B read + 6 B written per element).  Where the arrays lie in HBM matters (see
        # ramtorch_amd/placement.py), so it is measured twice: on four fresh buffers allocated
        # side by side, and on the workload's own largest tensor (p, its gradient and its two
        # states, where the optimizer placed them).  The probe overwrites what it runs on, which
        # is why it comes last.
        n_probe = 1 << 30
        bufs = [torch.zeros(n_probe, dtype=torch.bfloat16, device=dev) for _ in range(4)]
        torch.cuda.synchronize()
        probe_ms = handle.stream_probe(*[b.data_ptr() for b in bufs], n_probe, reps=5)
        roofline["pattern_ceiling_fresh_buffers_GBps"] = 14 * n_probe / (probe_ms * 1e-3) / 1e9
        del bufs
        roofline["pattern_ceiling_GBps"] = roofline["pattern_ceiling_fresh_buffers_GBps"]
        big = max(range(len(params)), key=lambda i: params[i].numel())
        arrs = [params[big].data, grads[big], opt.state[params[big]]["ema"], opt.state[params[big]]["ema_squared"]]
        n_own = min(a.numel() * a.element_size() // 2 for a in arrs) // 8192 * 8192
        if n_own >= (1 << 24) and all(a.data_ptr() % 16 == 0 for a in arrs):
            probe_ms = handle.stream_probe(*[a.data_ptr() for a in arrs], n_own, reps=5)
            roofline["pattern_ceiling_GBps"] = 14 * n_own / (probe_ms * 1e-3) / 1e9
        roofline["frac_of_pattern_ceiling"] = achieved / roofline["pattern_ceiling_GBps"] if wl in ("llama8b", "small") else None
        roofline["state_placement"] = {"mode": args.state_placement, **(opt.state_placement_report or {})}
    else:
        if wl == "streamed":
            st = handle.streamed_stats()
        else:  # per-tensor asynchronous calls: the whole step is the unit
            st = {"bytes_h2d": 6.0 * total, "bytes_d2h": 6.0 * total, "seconds": ms_per_step * 1e-3}
        stream_info = {"h2d_GBps": st["bytes_h2d"] / st["seconds"] / 1e9, "d2h_GBps": st["bytes_d2h"] / st["seconds"] / 1e9,
                       "seconds_last_call": st["seconds"], "host_bytes": 6 * total}
        # same-run pinned-copy peaks with the same chunk size
        chunk = args.stream_chunk_mb << 20
        hbuf = torch.empty(chunk, dtype=torch.uint8).pin_memory()
        dbuf = torch.empty(chunk, dtype=torch.uint8, device=dev)
        for name, (dst, src) in (("h2d", (dbuf, hbuf)), ("d2h", (hbuf, dbuf))):
            dst.copy_(src, non_blocking=True)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            for _ in range(8):
                dst.copy_(src, non_blocking=True)
            torch.cuda.synchronize()
            stream_info[f"pinned_{name}_peak_GBps"] = 8 * chunk / (time.perf_counter() - t1) / 1e9
        stream_info["h2d_frac_of_peak"] = stream_info["h2d_GBps"] / stream_info["pinned_h2d_peak_GBps"]
        # both directions at once (what the pipeline does in steady state): two streams, one chunk each way
        hbuf2 = torch.empty(chunk, dtype=torch.uint8).pin_memory()
        dbuf2 = torch.empty(chunk, dtype=torch.uint8, device=dev)
        s_up, s_down = torch.cuda.Stream(), torch.cuda.Stream()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(8):
            with torch.cuda.stream(s_up):
                dbuf.copy_(hbuf, non_blocking=True)
            with torch.cuda.stream(s_down):
                hbuf2.copy_(dbuf2, non_blocking=True)
        torch.cuda.synchronize()
        stream_info["pinned_duplex_peak_GBps_each_way"] = 8 * chunk / (time.perf_counter() - t1) / 1e9
        stream_info["frac_of_duplex_peak"] = stream_info["d2h_GBps"] / stream_info["pinned_duplex_peak_GBps_each_way"]
        del hbuf2, dbuf2
        if wl == "streamed":
            # per-chunk copy durations of one more step, from events the library records on its copy streams
            handle.set_timing(True)
            one_step()
            tl = handle.streamed_timeline()
            handle.set_timing(False)
            if tl:
                h2d = [r[1] - r[0] for r in tl]
                d2h = [r[3] - r[2] for r in tl]
                stream_info["chunks"] = len(tl)
                stream_info["h2d_chunk_ms"] = {"first": h2d[0], "median": sorted(h2d)[len(h2d) // 2], "max": max(h2d)}
                stream_info["d2h_chunk_ms"] = {"median": sorted(d2h)[len(d2h) // 2], "max": max(d2h), "last": d2h[-1]}
                stream_info["pipeline_ms"] = tl[-1][3] - tl[0][0]
        roofline = {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": None,
                    "traffic": None, "note": "host-link bound; see host_link"}

    if args.pmc_calibrate:
        x = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        y = torch.empty_like(x)
        torch.cuda.synchronize()
        torch.add(x, 1.0, out=y)  # vectorized_elementwise_kernel: 2^30 bytes in, 2^30 bytes out
        torch.cuda.synchronize()
        del x, y

    out = {
        "metric": METRIC, "value": total / (ms_per_step * 1e-3), "unit": "elements/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": dtype_label, "data": "synthetic",
        "config": {"workload": wl, "tensors": len(shapes), "elements": total, "bytes_per_element": bytes_per_elem,
                   "first_timed_step": first_step, "noise": "explicit int16" if noise else "philox seed 1234",
                   "hparams": {"lr": HP["lr"], "betas": list(HP["betas"]), "eps": HP["eps"],
                               "weight_decay": HP["weight_decay"]}},
        "achieved_GBps_wall": bytes_per_elem * total / (ms_per_step * 1e-3) / 1e9,
        "roofline": roofline,
    }
    if stream_info:
        out["host_link"] = stream_info
    if not args.no_cpu_baseline:
        del params, grads, opt, gmap
        torch.cuda.empty_cache()
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
