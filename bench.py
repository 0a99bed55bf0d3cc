#!/usr/bin/env python3
"""Benchmark of the SR-AdamW step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload llama8b] [--secondary all|none|a,b,...]

A "step" is one ``AdamW.step()`` over the whole synthetic parameter set, with
params, grads and both states already resident in HBM (or, for the host-resident
workloads, params/states in pinned host memory).  Prints ONE JSON line:

  value      elements updated per second over the K timed steps of the main workload
             (wall clock around the steps, device synchronised on both sides)
  roofline   algorithmic HBM bytes per launch / mean kernel time of the update
             kernel, the kernel time taken with HIP events on the launch stream
             inside the library; peak = 8 TB/s.  ``roofline.settling``: the untimed
             steps that run before the W warm-up steps until the driver has finished
             clearing the device memory that set-up released (see ``settle``), with
             the kernel time of every batch of them
  secondary  the other configurations, each measured the same way in the same
             process with fewer steps (only when the main workload is the
             default one; ``--secondary none`` leaves them out)
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
  central   the default set with centralization=1.0 (adamw.py:179-184): one launch in which a
            wavefront sums a gradient row and then updates it (14 B per element from HBM; the
            row is read a second time out of the L2); next to it the same steps with a row-mean
            pass of their own first (16 B per element)
  streamed  Llama-3-8B shapes with p/ema/ema_squared in pinned host memory,
            bf16 grads on the GPU, 256 MB chunks (--stream-gb bounds the host set)
  hooked    the same set, but each tensor is updated by AdamW.step_param() as a
            backward pass would hand its gradient over (last tensor first), and
            step() only waits: the grad hand-off from ramtorch.Linear's
            post-accumulate hook
  any       one transformer layer of the set (9 tensors, 218 112 000 elements) with bf16 parameters
            and gradients and both states in fp64 (the reference upcasts any dtype, adamw.py:160-170,
            and writes what is not bf16 back with a plain copy_): the runtime-typed kernel that
            serves the layouts without a templated instance; 34 bytes per element
  pageable  a 16 GB prefix of the set with parameters and states in ordinary (not pinned) CPU memory,
            the third kind of input adamw.py:152-170 accepts: up through the library's pinned
            bounce buffers, filled by host threads, and down through them again
  offload_ref  the same set as the reference's own offload flow leaves it
            (linear.py:416-427 -> adamw.py:167): pinned CPU params and states
            and the gradients on the CPU too (in the pinned memory that
            ``.to("cpu", non_blocking=True)`` allocates); 8 bytes per element
            go up the host link, 6 come down.  Without the two embedding tensors
            (6 979 584 000 elements): a process can pin about 64 GiB on the box.
            Also timed with the gradients in ordinary CPU memory
            (``unpinned_gradients``)
"""
from __future__ import annotations

import argparse
import gc
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
# HBM bytes per launch of the dominant update kernel.  NOT measured in this run: rocprofv3 --pmc
# FETCH_SIZE / WRITE_SIZE figures of earlier runs of this script (each scaled by what the same
# counter reads for a plain kernel of known size in the same run), kept under profiles/.
_TRAFFIC_FILE = "profiles/sr_adamw_kernels_hbm_traffic.txt"
OFFLINE_TRAFFIC = {
    "llama8b": (112_422_266_998, _TRAFFIC_FILE),
    "mixed": (160_597_606_615, _TRAFFIC_FILE),      # the update launch; its norm pass fetches 32 120 545 889 B more
    "small": (1_090_935_301, _TRAFFIC_FILE),
    "cfg0": (335_774_529, _TRAFFIC_FILE),
    "central": (116_001_647_514, _TRAFFIC_FILE),   # row-wise kernels: the rows of 14 336 elements are read twice, the second time mostly from HBM
    "any": (8_292_259_533, _TRAFFIC_FILE),
}
HP = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
METRIC = "SR-AdamW step: params/sec + achieved HBM GB/s (% of peak), 8B bf16 set, 1 GPU"
RESIDENT = ("llama8b", "cfg0", "small", "mixed", "central", "any")
HOST = ("streamed", "hooked", "offload_ref", "pageable")
UPDATE_BYTES = {"llama8b": 14, "small": 14, "cfg0": 20, "mixed": 20, "central": 14, "any": 38}   # per element, update launch only
STEP_BYTES = {"llama8b": 14, "small": 14, "cfg0": 20, "mixed": 24, "central": 14, "any": 38, "streamed": 12, "hooked": 12,
              "offload_ref": 14, "pageable": 12}


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


_FILL_SCRATCH = {}


def fill_tensor(shape, kind: str, seed: int, dtype, device):
    """Synthetic values of one array, drawn in fp32 on `device` and stored as `dtype`.  The fp32 values
    are drawn into one scratch buffer per device that is allocated once, before anything else: the
    tensors of a set then follow each other in device memory as a model's do, instead of landing in
    whatever blocks earlier temporaries left behind in torch's allocator."""
    import torch
    gen = torch.Generator(device=device).manual_seed(seed)
    n = numel(shape)
    step = 1 << 28  # bound the fp32 scratch
    scratch = _FILL_SCRATCH.get(str(device))
    if scratch is None:
        scratch = _FILL_SCRATCH[str(device)] = torch.empty(step, dtype=torch.float32, device=device)
    out = torch.empty(n, dtype=dtype, device=device)
    for lo in range(0, n, step):
        k = min(step, n - lo)
        x = scratch[:k].normal_(generator=gen)
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
    # the same op sequence at config-0 size (one 4096 x 4096 tensor), 1 warm-up pass + best of 5
    P, G, M, V = (fill_tensor((4096, 4096), kind, 1234 + k, torch.bfloat16, "cpu") for k, kind in enumerate("pgmv"))
    best0 = float("inf")
    for it in range(6):
        t0 = time.perf_counter()
        torch_ops.reference_step_ops(P, G, M, V, step=10 + it, noise=None, **HP)
        dt = time.perf_counter() - t0
        if it:
            best0 = min(best0, dt)
    del P, G, M, V

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
        "cfg0_size": {"elements": 4096 * 4096, "ms_per_step": best0 * 1e3, "elements_per_s": 4096 * 4096 / best0,
                      "algorithmic_GBps": 14 * 4096 * 4096 / best0 / 1e9,
                      "sample": "the same op sequence on one 4096 x 4096 bf16 tensor, 1 warm-up pass + best of 5"},
        "c_oracle_1thread_elements_per_s": k / c_dt,
    }


# ---- GPU workloads ----------------------------------------------------------------------------
def build_resident(shapes, *, g_dtype, device, seed=1234, flat=False):
    """(params, grads, refill): ``refill()`` draws the parameters' values again into the same storage."""
    import torch
    gdt = torch.float32 if g_dtype == torch.float32 else torch.bfloat16
    if flat:
        # thousands of short tensors: carved out of one parameter buffer and one gradient buffer at
        # 512-byte steps, which is how torch's allocator packs small tensors anyway, and filled by two
        # kernels instead of tens of thousands
        offs, total = [], 0
        for shp in shapes:
            offs.append(total)
            total += (numel(shp) + 255) // 256 * 256
        pbuf = fill_tensor((total,), "p", seed, torch.bfloat16, device)
        gbuf = fill_tensor((total,), "g", seed + 1, gdt, device)
        if g_dtype == torch.float32:
            gbuf.mul_(1024.0)
        params = [torch.nn.Parameter(pbuf[o:o + numel(shp)].view(shp), requires_grad=False) for o, shp in zip(offs, shapes)]
        grads = [gbuf[o:o + numel(shp)].view(shp) for o, shp in zip(offs, shapes)]
        return params, grads, lambda: pbuf.copy_(fill_tensor((total,), "p", seed, torch.bfloat16, device))
    # parameters first, gradients afterwards: the order a framework allocates them in (model
    # construction, then the backward pass), so a parameter and its gradient are not neighbours
    params, grads = [], []
    for i, shp in enumerate(shapes):
        params.append(torch.nn.Parameter(fill_tensor(shp, "p", seed + 4 * i, torch.bfloat16, device),
                                         requires_grad=False))
    for i, shp in enumerate(shapes):
        g = fill_tensor(shp, "g", seed + 4 * i + 1, gdt, device)
        if g_dtype == torch.float32:
            g.mul_(1024.0)
        grads.append(g)

    def refill():
        for i, (p, shp) in enumerate(zip(params, shapes)):
            p.data.copy_(fill_tensor(shp, "p", seed + 4 * i, torch.bfloat16, device))
    return params, grads, refill


def set_states(opt, params, first_step, warmup, dev):
    import torch
    pools = getattr(opt, "_state_pools", None) or {}
    pooled = "ema" in pools and all(s is not None for s in pools.get("slots", [None]))
    if pooled and len(params) > 1000:
        # all states are views into two pools: fill the pools, not 2 x 20 000 views (padding included; harmless)
        for k, key in ((2, "ema"), (3, "ema_squared")):
            dt = opt.state[params[0]][key].dtype
            view = pools[key].view(dt)
            view.copy_(fill_tensor((view.numel(),), "m" if key == "ema" else "v", 1234 + k, dt, dev))
    for i, p in enumerate(params):
        st = opt.state[p]
        st["step"] = first_step - 1 - warmup
        if pooled and len(params) > 1000:
            continue
        # the states stay the tensors the optimizer allocated (and placed); only their contents are set
        st["ema"].copy_(fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev))   # (copy_ widens for wider states)
        st["ema_squared"].copy_(fill_tensor(p.shape, "v", 1234 + 4 * i + 3, st["ema_squared"].dtype, dev))


def _unpin_free_host_blocks():
    """Give the pinned host blocks that torch's allocator holds but nothing uses back to the system."""
    import torch
    fn = getattr(torch._C, "_host_emptyCache", None)
    if fn is not None:
        fn()


def timed_steps(one_step, steps, warmup, handle, resident):
    import torch
    for _ in range(warmup):
        one_step()
    torch.cuda.synchronize()
    if resident:
        # the library records a HIP event pair around the update kernels of every launch, on the
        # launch stream; nothing is read back before the timed region has ended
        handle.set_timing(True)
    t0 = time.perf_counter()
    for _ in range(steps):
        one_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ks = handle.kernel_ms_history(min(steps, 256)) if resident else []
    if resident:
        handle.set_timing(False)
    return wall * 1e3 / steps, ks


def settle(one_step, handle, seconds, max_seconds):
    """Untimed steps of the workload itself until the device's memory is the workload's alone.
    Device memory that a process gives back to the driver (here: the filler blocks of the optimizer's
    placement search, what torch's allocator releases between workloads, what an earlier process
    held) is cleared by the driver in the background, at about 33 GB/s on the MI355X boxes, and while
    that runs the same launch over the same tensors takes 1.0 - 1.5 % longer (8B set: 17.75 ms for
    1.9 s after 64 GiB were released, 3.8 s after 128 GiB; 17.56 ms before and after; compute-bound
    kernels or idling beforehand change nothing).  A training job pays that once, in its first
    seconds.  Steps run in batches for at least ``seconds``; from then on until a batch is 0.6 % faster
    than the first ones were (the clearing has ended) or ``max_seconds`` have passed (there was
    none).  Returns what was seen, for the bench line: the mean kernel time of every batch."""
    import torch
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    means = []
    steps = 0
    batch = 10
    while True:
        handle.set_timing(True)
        for _ in range(batch):
            one_step()
        torch.cuda.synchronize()
        ks = handle.kernel_ms_history(min(batch, 256))
        handle.set_timing(False)
        steps += batch
        means.append(sum(ks) / len(ks))
        if len(means) == 1:
            # short launches: batches long enough that the loop is not all synchronisation
            batch = int(min(2000, max(10, 0.15 / max(means[0] * 1e-3, 1e-6))))
        elapsed = time.perf_counter() - t0
        head = sorted(means[1:4])[len(means[1:4]) // 2] if len(means) >= 4 else None   # the first batch holds the ramp
        dropped = head is not None and means[-1] < 0.994 * head
        if elapsed >= max_seconds or (elapsed >= seconds and dropped):
            break
    return {"steps": steps, "seconds": time.perf_counter() - t0, "kernel_ms_first_batch": means[min(1, len(means) - 1)],
            "kernel_ms_last_batch": means[-1], "saw_the_clearing_end": bool(dropped),
            "kernel_ms_batches": [round(m, 4) for m in means[:64]]}


def config_of(wl, shapes, total, first_step, explicit):
    return {"workload": wl, "tensors": len(shapes), "elements": total, "bytes_per_element": STEP_BYTES[wl],
            "first_timed_step": first_step, "noise": "explicit int16" if explicit else "philox seed 1234",
            "hparams": {"lr": HP["lr"], "betas": list(HP["betas"]), "eps": HP["eps"],
                        "weight_decay": HP["weight_decay"]}}


def class_table(opt, params, grads, handle):
    """The update kernel's rate per shape class of the Llama-shaped set, on the tensors where the bench and
    the optimizer put them: five steps over the tensors of each class alone (kernel time from the
    library's events), and afterwards the math-free probe of the same traffic on one tensor of the class
    with its gradient and its two states (the probe overwrites what it runs on)."""
    import torch
    layer = lambda l, k: 1 + 9 * l + k
    classes = {"embed, lm_head (128256x4096)": [0, 289],
               "q, o (4096x4096)": [layer(l, k) for l in range(32) for k in (0, 3)],
               "k, v (1024x4096)": [layer(l, k) for l in range(32) for k in (1, 2)],
               "gate, up (14336x4096)": [layer(l, k) for l in range(32) for k in (4, 5)],
               "down (4096x14336)": [layer(l, 6) for l in range(32)]}
    out = {}
    for name, idx in classes.items():
        gm = {params[i]: grads[i] for i in idx}
        for p in params:
            p.grad = None
        opt.step(grads=gm)
        torch.cuda.synchronize()
        handle.set_timing(True)
        for _ in range(5):
            opt.step(grads=gm)
        torch.cuda.synchronize()
        ks = handle.kernel_ms_history(5)
        handle.set_timing(False)
        n = sum(params[i].numel() for i in idx)
        ms = sum(ks) / len(ks)
        out[name] = {"tensors": len(idx), "elements": n, "kernel_ms": ms, "achieved": 14 * n / (ms * 1e-3) / 1e9,
                     "frac": 14 * n / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
    for name, idx in classes.items():
        rates = []
        for i in (idx[0], idx[len(idx) // 2], idx[-1]):
            st = opt.state[params[i]]
            n = params[i].numel() // 8192 * 8192
            ms = handle.stream_probe(params[i].data_ptr(), grads[i].data_ptr(), st["ema"].data_ptr(),
                                     st["ema_squared"].data_ptr(), n, reps=max(5, int(3e8 // n)))
            rates.append(14 * n / (ms * 1e-3) / 1e9)
        out[name]["probe_GBps_first_middle_last_tensor"] = rates
    return out


def run_resident(wl, args, steps, warmup, *, full):
    """One resident workload.  ``full``: also the math-free ceilings and the plain-placement comparison."""
    import torch
    import ramtorch_amd
    from ramtorch_amd.stochastic_optimizers import adamw as adamw_mod

    dev = "cuda:0"
    first_step = 100
    opt_kw = dict(storage_device="cuda", seed=1234, state_placement=args.state_placement)
    g_dtype = torch.bfloat16
    state_dtype = torch.bfloat16
    if wl == "llama8b":
        shapes = llama3_8b_shapes(args.layers)
    elif wl == "central":
        shapes = llama3_8b_shapes(args.layers)
        opt_kw.update(centralization=1.0)
    elif wl == "cfg0":
        shapes = [(4096, 4096)]
        first_step = 10
    elif wl == "small":
        shapes = small_tensor_shapes()
        opt_kw.update(state_pool_min_bytes=0)   # states as views into two pools, like the large sets
    elif wl == "any":
        shapes = llama3_8b_shapes(1)[1:-1]
        state_dtype = torch.float64
    else:  # mixed
        shapes = llama3_8b_shapes(args.layers)
        g_dtype = torch.float32
        opt_kw.update(loss_scale=1024.0, max_grad_norm=1.0, ema_squared_dtype=torch.float32)
    params, grads, refill_params = build_resident(shapes, g_dtype=g_dtype, device=dev, flat=wl == "small")
    total = sum(numel(s) for s in shapes)
    opt = ramtorch_amd.AdamW(params, dtype=state_dtype, **HP, **opt_kw)
    set_states(opt, params, first_step, warmup, dev)
    noise = None
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

    one_step = lambda: opt.step(noise=noise, grads=gmap)
    settled = None
    if args.release_gib > 0 and full:
        # diagnostic: take this much device memory from the driver and give it straight back, so that the
        # settling steps below run while the driver clears it (their kernel times show for how long)
        time.sleep(max(0.0, args.idle_before_release))
        held = [handle.dev_hold(2 << 30) for _ in range(int(args.release_gib // 2))]
        for addr in held:
            handle.dev_release(addr)
    if args.settle_seconds > 0:
        # the device runs under the workload's own load until its clocks have settled; then parameters
        # and states are drawn again (same seeds, same distributions) and the step counts put back,
        # so that the timed steps start from the configuration's inputs at the configuration's step
        settled = settle(one_step, handle, args.settle_seconds, args.settle_max_seconds if full else min(args.settle_max_seconds, 6.0))
        refill_params()
        set_states(opt, params, first_step, warmup, dev)
        torch.cuda.synchronize()
    ms_per_step, ks = timed_steps(one_step, steps, warmup, handle, True)
    k_ms = sum(ks) / len(ks)
    upd_bytes = UPDATE_BYTES[wl] * total
    achieved = upd_bytes / (k_ms * 1e-3) / 1e9
    traffic = OFFLINE_TRAFFIC.get(wl) if args.layers == 32 else None
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBPS, "traffic": traffic[0] if traffic else None,
                "traffic_source": (f"not measured in this run: rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE of an earlier "
                                   f"run, {traffic[1]}") if traffic else None,
                "kernel": {"mixed": "sr_adamw_fast_wide_kernel", "central": "sr_adamw_rowwise_kernel",
                           "any": "sr_adamw_any_kernel"}.get(wl, "sr_adamw_fast_kernel"),
                "kernel_ms": k_ms, "kernel_launches_timed": len(ks), "algorithmic_bytes_per_launch": upd_bytes}
    if settled is not None:
        unsettled = upd_bytes / (settled["kernel_ms_first_batch"] * 1e-3) / 1e9
        roofline["settling"] = dict(settled, achieved_first_batch=unsettled, frac_first_batch=unsettled / HBM_PEAK_GBPS,
                                    note="untimed steps of this workload before the warm-up steps; parameters and "
                                         "states drawn again and step counts reset afterwards")
    out = {"ms_per_step": ms_per_step, "elements_per_s": total / (ms_per_step * 1e-3),
           "achieved_GBps_wall": STEP_BYTES[wl] * total / (ms_per_step * 1e-3) / 1e9,
           "config": config_of(wl, shapes, total, first_step, noise is not None), "roofline": roofline}
    if wl == "small":
        # the same steps with the layout recorded once (AdamW.freeze_layout): the host only checks that
        # no parameter or gradient has moved instead of gathering 20 064 descriptors again
        opt.freeze_layout()
        opt.step()
        ms2, ks2 = timed_steps(lambda: opt.step(), steps, 2, handle, True)
        out["static_layout"] = {"ms_per_step": ms2, "kernel_ms": sum(ks2) / len(ks2),
                                "elements_per_s": total / (ms2 * 1e-3), "recorded": opt._frozen is not None}
        opt.unfreeze_layout()
        # and once with every tensor an allocation of its own (torch's allocator packs them into its
        # 2 MiB small-tensor blocks at 512-byte steps), as a model's parameters and gradients are
        sep_p = [torch.nn.Parameter(p.detach().clone(), requires_grad=False) for p in params]
        for p, g in zip(sep_p, grads):
            p.grad = g.clone()
        sep = ramtorch_amd.AdamW(sep_p, dtype=torch.bfloat16, **HP, **dict(opt_kw, state_placement="plain"))
        for p in sep_p:
            sep.state[p]["step"] = first_step - 1
        ms3, ks3 = timed_steps(lambda: sep.step(), max(5, steps // 2), 3, handle, True)
        k3 = sum(ks3) / len(ks3)
        out["separate_allocations"] = {"ms_per_step": ms3, "kernel_ms": k3, "achieved": upd_bytes / (k3 * 1e-3) / 1e9,
                                       "frac": upd_bytes / (k3 * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                                       "note": "one torch allocation per parameter, gradient and state (plain placement)"}
        del sep, sep_p
    if full:
        # The same state tensors allocated one by one, as the reference allocates them, instead of
        # in two pools placed in different HBM regions: what the placement is worth on this box.
        if args.state_placement == "auto" and opt.state_placement_report is not None and len(params) < 1000:
            plain = ramtorch_amd.AdamW(params, dtype=torch.bfloat16, **HP, **dict(opt_kw, state_placement="plain"))
            for p in params:
                plain.state[p]["step"] = first_step - 1
            _, ks2 = timed_steps(lambda: plain.step(noise=noise, grads=gmap), max(3, steps // 4), 2, handle, True)
            k2 = sum(ks2) / len(ks2)
            roofline["plain_placement"] = {"kernel_ms": k2, "achieved": upd_bytes / (k2 * 1e-3) / 1e9,
                                           "frac": upd_bytes / (k2 * 1e-3) / 1e9 / HBM_PEAK_GBPS}
            del plain
        if args.class_table and wl == "llama8b" and args.layers == 32:
            roofline["classes"] = class_table(opt, params, grads, handle)
        # What the same traffic pattern reaches with the arithmetic removed (the all-bf16 pattern:
        # 8 B read + 6 B written per element).  Where the arrays lie in HBM matters, so it is measured
        # twice: on four fresh buffers allocated side by side, and on the workload's own largest
        # tensor (p, its gradient and its two states, where the optimizer placed them).  The probe
        # overwrites what it runs on, which is why it comes last.
        n_probe = 1 << 30
        bufs = [torch.zeros(n_probe, dtype=torch.bfloat16, device=dev) for _ in range(4)]
        torch.cuda.synchronize()
        probe_ms = handle.stream_probe(*[b.data_ptr() for b in bufs], n_probe, reps=5)
        roofline["pattern_ceiling_fresh_buffers_GBps"] = 14 * n_probe / (probe_ms * 1e-3) / 1e9
        del bufs
        roofline["pattern_ceiling_GBps"] = roofline["pattern_ceiling_fresh_buffers_GBps"]
        # (the largest tensor; when several share that size -- embedding and lm_head -- the first and the last of
        # them, and the better figure counts: the probe, unlike the kernel, is sensitive to where the gradient of
        # a tensor lies relative to its parameter, and reads 3 - 5 % low on some quadruples the kernel runs at full rate on)
        top = max(p.numel() for p in params)
        bigs = [i for i, p in enumerate(params) if p.numel() == top]
        own = []
        for big in sorted({bigs[0], bigs[-1]}):
            arrs = [params[big].data, grads[big], opt.state[params[big]]["ema"], opt.state[params[big]]["ema_squared"]]
            n_own = min(a.numel() * a.element_size() // 2 for a in arrs) // 8192 * 8192
            if n_own >= (1 << 24) and all(a.data_ptr() % 16 == 0 for a in arrs):
                probe_ms = handle.stream_probe(*[a.data_ptr() for a in arrs], n_own, reps=5)
                own.append(14 * n_own / (probe_ms * 1e-3) / 1e9)
        if own:
            roofline["pattern_ceiling_GBps"] = max(own)
            roofline["pattern_ceiling_own_tensors_GBps"] = own
        roofline["frac_of_pattern_ceiling"] = (achieved / roofline["pattern_ceiling_GBps"]
                                               if wl in ("llama8b", "small") else None)
    roofline["state_placement"] = {"mode": args.state_placement, **(opt.state_placement_report or {})}
    if wl == "central":
        # the same steps with the row means taken by a pass of their own first (what tensors whose rows do
        # not fit a wavefront get): 2 B per element more from HBM and one launch more
        opt.fuse_row_means = False
        ms2, ks2 = timed_steps(one_step, max(3, steps // 4), 2, handle, True)
        k2 = sum(ks2) / len(ks2)
        opt.fuse_row_means = True
        roofline["separate_row_mean_pass"] = {
            "ms_per_step": ms2, "update_kernel_ms": k2, "row_mean_pass_ms": ms2 - k2,
            "note": "row_mean_table_kernel (16.06 GB read) + the fast kernel's centralizing instance, 16 B per element"}
    if wl == "mixed":
        # the norm pass is a launch of its own (4 B per element read); time it apart
        from ramtorch_amd import functional as F
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        F.grad_norm(handle, grads, inv_loss_scale=1 / 1024, max_norm=1.0)
        ev[0].record()
        for _ in range(3):
            F.grad_norm(handle, grads, inv_loss_scale=1 / 1024, max_norm=1.0)
        ev[1].record()
        torch.cuda.synchronize()
        n_ms = ev[0].elapsed_time(ev[1]) / 3
        roofline["norm_pass"] = {"kernel": "grad_sumsq_table_kernel", "ms": n_ms, "achieved": 4 * total / (n_ms * 1e-3) / 1e9,
                                 "frac": 4 * total / (n_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS}
    del opt, params, grads, gmap, noise
    gc.collect()
    torch.cuda.empty_cache()
    return out


def run_host(workloads, args, steps, warmup):
    """The host-resident workloads, on one set of pinned host arrays (pinning 48 GB takes a while)."""
    import torch
    import ramtorch_amd
    from ramtorch_amd.stochastic_optimizers import adamw as adamw_mod

    dev = "cuda:0"
    shapes = llama3_8b_shapes(args.layers)
    budget = int(args.stream_gb * 1e9)
    kept, used = [], 0
    for shp in shapes:
        if used + 6 * numel(shp) > budget:
            break
        kept.append(shp)
        used += 6 * numel(shp)
    shapes = kept
    total = sum(numel(s) for s in shapes)
    t_pin = time.perf_counter()
    params, grads = [], []
    for i, shp in enumerate(shapes):
        p = fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev).cpu().pin_memory()
        params.append(torch.nn.Parameter(p, requires_grad=False))
        grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.bfloat16, dev))
    opt = ramtorch_amd.AdamW(params, dtype=torch.bfloat16, **HP, storage_device="cpu", seed=1234,
                             stream_chunk_bytes=args.stream_chunk_mb << 20)
    set_states(opt, params, 100, warmup * len(workloads), dev)
    torch.cuda.synchronize()
    setup_s = time.perf_counter() - t_pin
    handle = adamw_mod._handle(0)
    gmap = dict(zip(params, grads))
    results = {}
    link = None
    if "offload_ref" in workloads:   # it rebuilds the optimizer on a subset: last
        workloads = [w for w in workloads if w != "offload_ref"] + ["offload_ref"]
    for wl in workloads:
        cpu_grads = None
        wl_shapes, wl_total = shapes, total
        if wl == "hooked":
            def one_step():
                for p, g in zip(reversed(params), reversed(grads)):
                    opt.step_param(p, g)
                opt.step()
        elif wl == "offload_ref":
            # Gradients where Linear.backward leaves them (linear.py:416-427): on the CPU, in the pinned memory
            # that .to("cpu", non_blocking=True) allocates.  A process can pin about 64 GiB on the GPU box and
            # torch's pinned allocator rounds every tensor up to a power of two, so 16 GB of pinned gradients do
            # not fit next to the 48.2 GB of parameters and states: this workload runs without the two
            # 525 M-element embedding tensors (whose 1.05 GB arrays cost 2 GiB of pinned memory each).  The new
            # optimizer's states reuse the pinned blocks of the old one; what the embeddings held is unpinned.
            keep = [i for i, s_ in enumerate(shapes) if numel(s_) < (1 << 28)]
            wl_shapes = [shapes[i] for i in keep]
            wl_params = [params[i] for i in keep]
            wl_grads = [grads[i] for i in keep]
            del opt, gmap
            params = grads = None
            gc.collect()
            opt = ramtorch_amd.AdamW(wl_params, dtype=torch.bfloat16, **HP, storage_device="cpu", seed=1234,
                                     stream_chunk_bytes=args.stream_chunk_mb << 20)
            set_states(opt, wl_params, 100, warmup + 1, dev)
            gc.collect()
            _unpin_free_host_blocks()
            wl_total = sum(numel(s_) for s_ in wl_shapes)
            pinned_ok = True
            try:
                cpu_grads = {p: g.to("cpu", non_blocking=True) for p, g in zip(wl_params, wl_grads)}
                torch.cuda.synchronize()
                pinned_ok = all(g.is_pinned() for g in cpu_grads.values())
            except RuntimeError:   # no more memory to pin on this machine
                pinned_ok = False
            if not pinned_ok:      # measured with ordinary CPU memory only, and said so
                cpu_grads = None
                gc.collect()
                _unpin_free_host_blocks()
                cpu_grads = {p: g.to("cpu") for p, g in zip(wl_params, wl_grads)}
            one_step = lambda: opt.step(grads=cpu_grads)
        else:
            one_step = lambda: opt.step(grads=gmap)
        ms_per_step, _ = timed_steps(one_step, steps, warmup, handle, False)
        up = {"streamed": 6.0, "hooked": 6.0, "offload_ref": 8.0}[wl] * wl_total
        down = 6.0 * wl_total
        secs = ms_per_step * 1e-3
        info = {"h2d_GBps": up / secs / 1e9, "d2h_GBps": down / secs / 1e9, "host_bytes_up": up, "host_bytes_down": down}
        if wl == "offload_ref":
            info["gradients_pinned"] = pinned_ok
        if wl == "offload_ref" and pinned_ok:
            # the same with the gradients in ordinary (not pinned) CPU memory, as a plain .to("cpu") leaves
            # them: they go up through the library's pinned bounce buffers, filled by host threads
            del cpu_grads
            gc.collect()
            _unpin_free_host_blocks()
            plain_grads = {p: g.to("cpu") for p, g in zip(wl_params, wl_grads)}
            b0 = handle.streamed_bounce_stats()
            ms2, _ = timed_steps(lambda: opt.step(grads=plain_grads), 2, 1, handle, False)
            b1 = handle.streamed_bounce_stats()
            info["unpinned_gradients"] = {"ms_per_step": ms2, "h2d_GBps": up / (ms2 * 1e-3) / 1e9,
                                          "bounced_bytes_per_step": (b1["bytes"] - b0["bytes"]) / 3}
            del plain_grads
            cpu_grads = None
        if link is None:
            # same-run pinned-copy peaks with the same chunk size, each direction alone and both at
            # once (what the pipeline does in steady state), on the library's own copy streams
            link = handle.host_link_probe(args.stream_chunk_mb << 20, reps=8)
        info["pinned_h2d_peak_GBps"] = link["h2d_GBps"]
        info["pinned_d2h_peak_GBps"] = link["d2h_GBps"]
        info["pinned_duplex_peak_GBps_each_way"] = link["duplex_GBps_each_way"]
        info["h2d_frac_of_peak"] = info["h2d_GBps"] / link["h2d_GBps"]
        info["frac_of_duplex_peak"] = info["d2h_GBps"] / link["duplex_GBps_each_way"]
        if wl == "streamed":
            # per-chunk copy durations of one more step, from events the library records on its copy streams
            handle.set_timing(True)
            one_step()
            tl = handle.streamed_timeline()
            handle.set_timing(False)
            if tl:
                h2d = [r[1] - r[0] for r in tl]
                d2h = [r[3] - r[2] for r in tl]
                info["chunks"] = len(tl)
                info["h2d_chunk_ms"] = {"first": h2d[0], "median": sorted(h2d)[len(h2d) // 2], "max": max(h2d)}
                info["d2h_chunk_ms"] = {"median": sorted(d2h)[len(d2h) // 2], "max": max(d2h), "last": d2h[-1]}
                info["pipeline_ms"] = tl[-1][3] - tl[0][0]
        del cpu_grads
        results[wl] = {"ms_per_step": ms_per_step, "elements_per_s": wl_total / secs,
                       "config": config_of(wl, wl_shapes, wl_total, 100, False), "host_link": info,
                       "roofline": {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                    "frac": None, "traffic": None, "note": "host-link bound; see host_link"}}
    for r in results.values():
        r["setup_seconds"] = setup_s
    del opt, params, grads
    gc.collect()
    torch.cuda.empty_cache()
    _unpin_free_host_blocks()
    return results


def run_pageable(args, steps, warmup):
    """Parameters and states in ordinary CPU memory (not pinned), gradients on the GPU: a prefix of the
    Llama-shaped set.  Runs before the large pinned set exists: the bounce buffers are pinned memory, and a
    process can pin about 64 GiB on the GPU boxes."""
    import torch
    import ramtorch_amd
    from ramtorch_amd.stochastic_optimizers import adamw as adamw_mod

    dev = "cuda:0"
    shapes, used = [], 0
    for shp in llama3_8b_shapes(args.layers):
        if used + 6 * numel(shp) > int(args.pageable_gb * 1e9):
            break
        shapes.append(shp)
        used += 6 * numel(shp)
    total = sum(numel(s) for s in shapes)
    params, grads = [], []
    for i, shp in enumerate(shapes):
        params.append(torch.nn.Parameter(fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev).cpu(), requires_grad=False))
        grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.bfloat16, dev))
    opt = ramtorch_amd.AdamW(params, dtype=torch.bfloat16, **HP, storage_device="cpu", seed=1234,
                             stream_chunk_bytes=args.stream_chunk_mb << 20)
    for i, p in enumerate(params):
        st = opt.state[p]      # the constructor pins "cpu" states (adamw.py:91-97): these are plain CPU tensors instead
        st["step"] = 100 - 1 - warmup
        st["ema"] = fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev).cpu()
        st["ema_squared"] = fill_tensor(p.shape, "v", 1234 + 4 * i + 3, torch.bfloat16, dev).cpu()
        assert not (p.is_pinned() or st["ema"].is_pinned() or st["ema_squared"].is_pinned())
    gc.collect()
    _unpin_free_host_blocks()
    torch.cuda.synchronize()
    handle = adamw_mod._handle(0)
    gmap = dict(zip(params, grads))
    b0 = handle.streamed_bounce_stats()
    ms_per_step, _ = timed_steps(lambda: opt.step(grads=gmap), steps, warmup, handle, False)
    b1 = handle.streamed_bounce_stats()
    link = handle.host_link_probe(args.stream_chunk_mb << 20, reps=8)
    secs = ms_per_step * 1e-3
    info = {"h2d_GBps": 6.0 * total / secs / 1e9, "d2h_GBps": 6.0 * total / secs / 1e9,
            "host_bytes_up": 6.0 * total, "host_bytes_down": 6.0 * total,
            "bounced_bytes_per_step": (b1["bytes"] - b0["bytes"]) / (steps + warmup),
            "pinned_h2d_peak_GBps": link["h2d_GBps"], "pinned_d2h_peak_GBps": link["d2h_GBps"],
            "pinned_duplex_peak_GBps_each_way": link["duplex_GBps_each_way"],
            "note": "parameters and states in CPU memory that is not pinned: up and down through pinned bounce "
                    "buffers that host threads fill and empty"}
    info["h2d_frac_of_peak"] = info["h2d_GBps"] / link["h2d_GBps"]
    info["frac_of_duplex_peak"] = info["d2h_GBps"] / link["duplex_GBps_each_way"]
    out = {"ms_per_step": ms_per_step, "elements_per_s": total / secs, "config": config_of("pageable", shapes, total, 100, False),
           "host_link": info, "roofline": {"bound": "hbm", "achieved": None, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                                           "frac": None, "traffic": None, "note": "host-link bound; see host_link"}}
    del opt, params, grads, gmap
    gc.collect()
    torch.cuda.empty_cache()
    # the handle's bounce buffers (6 GB of pinned memory) go back before the large pinned set is built
    h = adamw_mod._handles.pop(0, None)
    if h is not None:
        h.close()
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="llama8b", choices=list(RESIDENT + HOST))
    ap.add_argument("--secondary", default=None,
                    help="'all', 'none' or a comma-separated list of workloads measured after the main one "
                         "(default: all when the main workload is llama8b, none otherwise)")
    ap.add_argument("--layers", type=int, default=32, help="transformer layers of the Llama-shaped set")
    ap.add_argument("--stream-gb", type=float, default=48.2, help="upper bound on pinned host bytes (host-resident workloads)")
    ap.add_argument("--stream-chunk-mb", type=int, default=256, help="bytes of bf16 per staged chunk and array")
    ap.add_argument("--pageable-gb", type=float, default=16.0, help="host bytes of the 'pageable' workload (p, ema, ema_squared)")
    ap.add_argument("--state-placement", default="auto", choices=["auto", "plain"],
                    help="AdamW(state_placement=...): 'auto' puts ema and ema_squared into different HBM regions")
    ap.add_argument("--settle-seconds", type=float, default=1.0,
                    help="resident workloads: untimed steps for at least this long before the warm-up steps, and on "
                         "until the driver has finished clearing released device memory in the background (a step "
                         "gets 0.6 %% faster) or --settle-max-seconds have passed (0 = no such steps)")
    ap.add_argument("--settle-max-seconds", type=float, default=8.0,
                    help="upper bound of that phase for the main workload (the secondary ones: at most 6 s)")
    ap.add_argument("--release-gib", type=float, default=0.0,
                    help="diagnostic (main workload): hold and release this much device memory right before the "
                         "settling steps, to see what the driver's background clearing of it costs and for how long")
    ap.add_argument("--idle-before-release", type=float, default=6.0,
                    help="with --release-gib: idle this long first, so that what set-up released has been cleared")
    ap.add_argument("--class-table", action="store_true",
                    help="llama8b: also the kernel's rate and the math-free probe's per shape class of the set")
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

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X", file=sys.stderr)
        return 1
    torch.cuda.set_device(0)
    wl = args.workload
    everything = [w for w in RESIDENT + HOST if w != wl]
    if args.secondary is None:
        secondary = everything if wl == "llama8b" else []
    elif args.secondary == "all":
        secondary = everything
    elif args.secondary == "none":
        secondary = []
    else:
        secondary = [w for w in args.secondary.split(",") if w]
        bad = [w for w in secondary if w not in RESIDENT + HOST]
        if bad:
            print(f"bench.py: unknown workload(s) {bad}", file=sys.stderr)
            return 2

    t_begin = time.perf_counter()
    if wl in RESIDENT:
        main_res = run_resident(wl, args, args.steps, args.warmup, full=True)
    elif wl == "pageable":
        main_res = run_pageable(args, args.steps, args.warmup)
    else:
        main_res = run_host([wl], args, args.steps, args.warmup)[wl]

    if args.pmc_calibrate:
        x = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")
        y = torch.empty_like(x)
        torch.cuda.synchronize()
        torch.add(x, 1.0, out=y)  # vectorized_elementwise_kernel: 2^30 bytes in, 2^30 bytes out
        torch.cuda.synchronize()
        del x, y

    sec = {}
    # fewer steps for the secondary configurations: the whole default run has to fit a few minutes
    for w in [w for w in secondary if w in RESIDENT]:
        k = {"cfg0": max(args.steps, 20), "small": max(args.steps, 20)}.get(w, max(3, min(args.steps, 10)))
        r = run_resident(w, args, k, min(args.warmup, 3), full=False)
        r["steps"] = k
        sec[w] = r
    if "pageable" in secondary:
        k = max(2, min(args.steps, 3))
        sec["pageable"] = run_pageable(args, k, 1)
        sec["pageable"]["steps"] = k
    host = [w for w in secondary if w in HOST and w != "pageable"]
    if host:
        k = max(2, min(args.steps, 3))
        for w, r in run_host(host, args, k, 1).items():
            r["steps"] = k
            sec[w] = r

    for w, r in sec.items():
        if w in RESIDENT and r["roofline"].get("achieved") and main_res["roofline"].get("achieved"):
            r["roofline"]["rate_vs_main_workload"] = r["roofline"]["achieved"] / main_res["roofline"]["achieved"]

    out = {
        "metric": METRIC, "value": main_res["elements_per_s"], "unit": "elements/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"], "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "f32",  # arithmetic type; storage is bf16 (or fp32 for the mixed layout)
        "data": "synthetic", "config": main_res["config"],
        "achieved_GBps_wall": main_res.get("achieved_GBps_wall"),
        "roofline": main_res["roofline"],
    }
    for extra in ("host_link", "static_layout"):
        if extra in main_res:
            out[extra] = main_res[extra]
    if sec:
        out["secondary"] = sec
    out["gpu_seconds_total"] = time.perf_counter() - t_begin
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
