"""Where the optimizer states sit in HBM.

Measured on MI355X (288 GiB as three regions of 96 GiB in physical address order; ``python -m
ramtorch_amd.placement`` prints the map): the
update's traffic -- four arrays read, three of them written in place -- runs at about 5.7 TB/s
when p, ema and ema_squared all lie in one region and at about 6.4 TB/s as soon as one of the
*written* arrays lies in another region; where the read-only gradient lies makes no difference.
The optimizer owns the two state arrays, so it can always arrange that: ``ema`` and
``ema_squared`` go into two pools that are placed in different regions.

Physical addresses are not visible from user space, so the placement is found by measurement:
``split_probe`` times the math-free copy of the update's access pattern (``rt_stream_probe``)
with all arrays inside one pool and with one written array in the other pool.  The pools hold
zeros when this runs and the probe only xors arrays with each other, so they still hold zeros
afterwards.
"""
from __future__ import annotations

from typing import Callable, Optional, Tuple

import torch

from . import _native as N

GIB = 1 << 30
_CHUNK = 8192            # elements per workgroup of the probe kernel
_MIN_ELEMS = 1 << 22     # below 8 MB per array the probe says little
_MAX_ELEMS = 1 << 27     # 256 MB per array is plenty


def split_probe(handle: N.Handle, a: torch.Tensor, b: torch.Tensor):
    """[(GB/s with p, g, ema, ema_squared all inside ``a``, GB/s with ema_squared in ``b`` instead), ...]
    at the beginning, middle and end of the two buffers, or None when they are too small to tell.
    ``a`` and ``b`` are 1-D GPU byte buffers of which corresponding parts will be used together (slot
    k of one pool with slot k of the other): a pool that straddles a region boundary shows the gain
    at some positions only."""
    na, nb = a.numel() * a.element_size() // 2, b.numel() * b.element_size() // 2
    n = min(na // 4, nb, _MAX_ELEMS)
    n -= n % _CHUNK
    if n < _MIN_ELEMS or (a.data_ptr() | b.data_ptr()) & 15:
        return None
    stream = torch.cuda.current_stream(a.device).cuda_stream
    gb = 14.0 * n / 1e6
    out = []
    with torch.cuda.device(a.device):
        for frac in (0.0, 0.5, 1.0):
            # the same relative position in both pools; in `a` four consecutive pieces are needed
            oa = int((na - 4 * n) * frac) // _CHUNK * _CHUNK
            ob = int((nb - n) * frac) // _CHUNK * _CHUNK
            pa = [a.data_ptr() + 2 * (oa + n * k) for k in range(4)]
            same = gb / handle.stream_probe(pa[0], pa[1], pa[2], pa[3], n, reps=3, stream=stream)
            cross = gb / handle.stream_probe(pa[0], pa[1], pa[2], b.data_ptr() + 2 * ob, n, reps=3, stream=stream)
            out.append((same, cross))
    return out


def place_pair(handle: N.Handle, device: torch.device, bytes_a: int, bytes_b: int, *,
               min_gain: float = 1.05, filler_bytes: int = 2 * GIB, step_bytes: int = 16 * GIB,
               max_filler_bytes: int = 112 * GIB, max_seconds: float = 8.0,
               log: Optional[Callable[[str], None]] = None):
    """Two zeroed byte pools on ``device`` such that arrays in the second are, as far as it can be
    arranged, in another HBM region than the corresponding arrays in the first.  Returns
    (pool_a, pool_b, report).

    The second pool is first allocated right after the first.  Unless the probe shows the gain
    (mean over the beginning, middle and end of the pools), filler blocks are allocated (memory
    the driver hands out in moderate blocks follows in physical address order; one huge block
    does not) and after every ``step_bytes`` of them a new candidate for the second pool is
    allocated and probed, until one shows the gain, or ``max_filler_bytes`` (a region is 96 GiB),
    free memory or ``max_seconds`` run out; the candidate with the best mean rate is kept.
    Fillers and the other candidates are released again and ``torch.cuda.empty_cache()`` returns
    them to the driver, which also drops whatever else torch had cached."""
    import time

    def zeros(nbytes):
        return torch.zeros(nbytes, dtype=torch.uint8, device=device)

    t0 = time.monotonic()
    report = {"placed": False, "filler_GiB": 0.0, "same_GBps": None, "cross_GBps": None, "tries": 0, "seconds": 0.0}
    a = zeros(bytes_a)
    best = zeros(bytes_b)
    res = split_probe(handle, a, best)
    if res is None:
        return a, best, report

    def summary(r):
        same = sum(x[0] for x in r) / len(r)
        cross = sum(x[1] for x in r) / len(r)
        return same, cross, cross >= min_gain * same

    same, cross, full = summary(res)
    report.update(same_GBps=same, cross_GBps=cross, tries=1, placed=full)
    held, filled = [], 0          # fillers and candidates that lost
    try:
        while not report["placed"]:
            free, _ = torch.cuda.mem_get_info(device)
            if (filled + step_bytes > max_filler_bytes or step_bytes + bytes_b + 4 * GIB > free
                    or time.monotonic() - t0 > max_seconds):
                break
            for _ in range(max(1, step_bytes // filler_bytes)):
                held.append(torch.empty(filler_bytes, dtype=torch.uint8, device=device))
            filled += step_bytes
            cand = zeros(bytes_b)
            same, cross, full = summary(split_probe(handle, a, cand))
            report["tries"] += 1
            if log:
                log(f"{filled / GIB:.0f} GiB of fillers: same {same:.0f} GB/s, split {cross:.0f} GB/s")
            if full or cross > report["cross_GBps"]:
                held.append(best)
                best = cand
                report.update(placed=full, filler_GiB=filled / GIB, same_GBps=same, cross_GBps=cross)
            else:
                held.append(cand)
            del cand
    except torch.cuda.OutOfMemoryError:
        pass
    del held
    torch.cuda.empty_cache()
    report["seconds"] = time.monotonic() - t0
    return a, best, report


def _device_map(block_gib: int = 2, reserve_gib: int = 6) -> None:
    """``python -m ramtorch_amd.placement``: maps how the update's traffic pattern runs depending on
    where its four arrays lie.  Allocates nearly all free memory of the current GPU in blocks (memory
    handed out block after block follows in physical address order) and probes combinations of blocks."""
    from .stochastic_optimizers.adamw import _handle

    dev = torch.device("cuda", torch.cuda.current_device())
    handle = _handle(dev.index)
    free, total = torch.cuda.mem_get_info(dev)
    block = block_gib * GIB
    n_blocks = int((free - reserve_gib * GIB) // block)
    n = block // 2  # bf16 elements per block
    blocks = [torch.empty(block, dtype=torch.uint8, device=dev) for _ in range(n_blocks)]
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream(dev).cuda_stream

    def probe(idx, reps=3):
        ms = handle.stream_probe(*(blocks[i].data_ptr() for i in idx), n, reps=reps, stream=stream)
        return 14.0 * n / ms / 1e6

    print(f"{torch.cuda.get_device_name(dev)}: {total / GIB:.0f} GiB, {n_blocks} blocks of {block_gib} GiB; "
          "GB/s of 8 B read + 6 B written per element (p, g, ema, ema_squared; p, ema, ema_squared written)")
    print("\n1. four neighbouring blocks (p, g, ema, ema_squared = blocks b .. b+3):")
    print("   " + "  ".join(f"{b * block_gib}GiB:{probe((b, b + 1, b + 2, b + 3)):.0f}" for b in range(0, n_blocks - 3, 4)))
    for base in (0, n_blocks // 2):
        print(f"\n2. p, g, ema at blocks {base}..{base + 2}; ema_squared at block k (GiB into the allocation order : GB/s):")
        ks = [k for k in range(0, n_blocks, 3) if not base <= k <= base + 2]
        print("   " + "  ".join(f"{k * block_gib}:{probe((base, base + 1, base + 2, k)):.0f}" for k in ks))
    a, b, c = 0, n_blocks // 2, n_blocks - 8
    where = {"A": a, "B": b, "C": c}
    print(f"\n3. which array has to move (A = block {a}.., B = block {b}.., C = block {c}..; order p g ema ema_squared):")
    for pat in ("AAAA", "BBBB", "CCCC", "ABAA", "AAAB", "AABA", "BAAA", "AABB", "ABAB", "ABBA", "ABBB", "AABC", "ABCA", "ABCC"):
        idx = tuple(where[r] + j for j, r in enumerate(pat))
        print(f"   {pat}  {probe(idx, 5):.0f}")


if __name__ == "__main__":
    _device_map()
