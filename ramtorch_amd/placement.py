"""Where the optimizer states sit in HBM.

Measured on MI355X (288 GiB as three regions of 96 GiB in physical address order): the update's
traffic -- four arrays read, three of them written in place -- runs at about 5.7 TB/s when p, ema
and ema_squared all lie in one region and at about 6.4 TB/s as soon as one of the *written* arrays
lies in another region; where the read-only gradient lies makes no difference.  The optimizer owns
the two state arrays, so it can always arrange that: ``ema`` and ``ema_squared`` go into two pools
that are placed in different regions.

Physical addresses are not visible from user space, so the placement is found by measurement:
``split_probe`` times the math-free copy of the update's access pattern (``rt_stream_probe``) with
all arrays inside one pool and with one written array in the other place.  The pools hold zeros
when this runs and the probe only xors arrays with each other, so they still hold zeros afterwards.
"""
from __future__ import annotations

import time
from typing import Callable, Optional

import torch

from . import _native as N

GIB = 1 << 30
_CHUNK = 8192            # elements per workgroup of the probe kernel
_MIN_ELEMS = 1 << 22     # below 8 MB per array the probe says little
_MAX_ELEMS = 1 << 27     # 256 MB per array is plenty


def split_probe(handle: N.Handle, a_ptr: int, a_bytes: int, b_ptr: int, b_bytes: int, device, stream: int):
    """[(GB/s with p, g, ema, ema_squared all inside block a, GB/s with ema_squared in block b instead), ...]
    at the beginning, middle and end of the two blocks, or None when they are too small to tell.
    Corresponding parts of the blocks will be used together (slot k of one pool with slot k of the
    other): a block that straddles a region boundary shows the gain at some positions only."""
    na, nb = a_bytes // 2, b_bytes // 2
    n = min(na // 4, nb, _MAX_ELEMS)
    n -= n % _CHUNK
    if n < _MIN_ELEMS or (a_ptr | b_ptr) & 15:
        return None
    gb = 14.0 * n / 1e6
    out = []
    with torch.cuda.device(device):
        for frac in (0.0, 0.5, 1.0):
            # the same relative position in both blocks; in `a` four consecutive pieces are needed
            oa = int((na - 4 * n) * frac) // _CHUNK * _CHUNK
            ob = int((nb - n) * frac) // _CHUNK * _CHUNK
            pa = [a_ptr + 2 * (oa + n * k) for k in range(4)]
            same = gb / handle.stream_probe(pa[0], pa[1], pa[2], pa[3], n, reps=3, stream=stream)
            cross = gb / handle.stream_probe(pa[0], pa[1], pa[2], b_ptr + 2 * ob, n, reps=3, stream=stream)
            out.append((same, cross))
    return out


class _HeldBlock:
    """A device block held through the library, seen by torch as a 1-D uint8 tensor (``tensor()``).
    The tensor and every view of it keep this object alive; the block is given back when the last
    of them has gone."""

    def __init__(self, addr: int, nbytes: int, device: torch.device):
        self.addr, self.nbytes, self.device = addr, nbytes, device
        self.__cuda_array_interface__ = {"shape": (nbytes,), "typestr": "|u1", "data": (addr, False), "version": 2,
                                         "strides": None}

    def tensor(self) -> torch.Tensor:
        return torch.as_tensor(self, device=self.device)

    def __del__(self):
        try:
            N.dev_release(self.addr)
        except Exception:
            pass  # interpreter shutdown: the process is about to return the memory anyway


#: Whether the optimizer lets the chunk-wise placement probe with the parameters' own memory (it writes
#: them back bit for bit as they are).  Set to False when something else may be writing parameters while
#: optimizers are constructed: chunks are then sorted relative to the first chunk taken, which keeps the
#: two pools apart from each other but not necessarily the first one with the parameters.
PROBE_WITH_PARAMETERS = True


def reference_arrays(params, device):
    """(address, address, address, elements) of three disjoint arrays inside the largest contiguous
    parameter on ``device`` for the chunk-wise placement to probe with (they are written back bit for
    bit as they are), or None when no parameter is large enough."""
    if not PROBE_WITH_PARAMETERS:
        return None
    best = None
    for p in params:
        if p.is_cuda and p.device == device and p.is_contiguous() and p.data_ptr() % 16 == 0:
            if best is None or p.numel() * p.element_size() > best.numel() * best.element_size():
                best = p
    if best is None:
        return None
    third = best.numel() * best.element_size() // 3 // 16 * 16    # bytes per array, 16-byte granules
    elems = min(third // 2, 1 << 27) // 8192 * 8192                # 16-bit elements per array
    if elems < (1 << 25):
        return None
    return best.data_ptr(), best.data_ptr() + third, best.data_ptr() + 2 * third, elems


_ENDED = {0: None, 1: "the search reached the memory it may occupy", 2: "the search reached its time limit",
          3: "the device had no free chunk left"}


def _place_pair_by_chunks(handle, device, bytes_a, bytes_b, free0, max_filler_bytes, max_fraction_of_free, max_seconds,
                          stream, report, log, ref):
    """The two pools from individually probed 1 GiB chunks (see rt_dev_hold_pair); None when the runtime
    cannot do that (the caller then searches with whole allocations)."""
    chunk = GIB
    need = -(-bytes_a // chunk) * chunk + -(-bytes_b // chunk) * chunk
    extra = min(max_filler_bytes, int(max_fraction_of_free * max(0, free0 - need)))
    if need + 2 * GIB > free0:
        return None
    try:
        a_ptr, b_ptr, rep = handle.dev_hold_pair(bytes_a, bytes_b, extra, max_seconds, ref, stream)
    except N.NativeError as e:
        if log:
            log(f"chunk-wise placement not used: {e}")
        return None
    a = _HeldBlock(a_ptr, -(-bytes_a // chunk) * chunk, device).tensor()[:bytes_a]
    b = _HeldBlock(b_ptr, -(-bytes_b // chunk) * chunk, device).tensor()[:bytes_b]
    report.update(placed=bool(rep[0]), filler_GiB=max(0.0, rep[2] * chunk - need) / GIB, tries=int(rep[2]),
                  same_GBps=rep[4], cross_GBps=rep[5], by_chunks=True, share_apart=rep[1],
                  relative_to_parameters=rep[7] == 2.0)
    reason = _ENDED.get(int(rep[6]))
    if reason and not rep[0]:
        report["reason"] = f"{reason}; {100 * rep[1]:.0f} % of the second pool lies apart from the first"
    res = split_probe(handle, a.data_ptr(), bytes_a, b.data_ptr(), bytes_b, device, stream)
    if res is not None:   # what the pools themselves show, beginning / middle / end
        report.update(same_GBps=sum(x[0] for x in res) / len(res), cross_GBps=sum(x[1] for x in res) / len(res))
    return a, b


def place_pair(handle: N.Handle, device: torch.device, bytes_a: int, bytes_b: int, *,
               min_gain: float = 1.05, min_gain_anywhere: float = 1.02, filler_bytes: int = 2 * GIB,
               step_bytes: int = 16 * GIB, max_filler_bytes: int = 112 * GIB, max_fraction_of_free: float = 0.5,
               max_seconds: float = 1.0, by_chunks: bool = True, ref=None,
               log: Optional[Callable[[str], None]] = None):
    """Two zeroed byte pools on ``device`` such that arrays in the second are, as far as it can be
    arranged, in another HBM region than the corresponding arrays in the first.  Returns
    (pool_a, pool_b, report).

    Pools of at least 1 GiB are first built chunk by chunk (``by_chunks``, ``rt_dev_hold_pair``): physical
    chunks of 1 GiB are taken one at a time, each is probed against the first one, and the two pools
    are mapped from chunks of the two kinds -- which also works in a process whose earlier
    allocations left the free memory in scattered order, where a single allocation of many GiB
    straddles regions.  Both pools are then memory held through the library.  ``ref``: three disjoint
    arrays in the memory of the parameters (see ``reference_arrays``):
    the first pool then lies where the parameters are and the second elsewhere.  What follows describes
    the search that is used when that is not available or does not apply.

    The place right behind the first pool is tried first.  A place is taken when the probe shows
    the gain there: ``min_gain`` on the mean over the beginning, the middle and the end of the pools,
    and at least ``min_gain_anywhere`` at each of them (in a process that has already allocated and
    released a lot, a block of many GiB rarely lies in one region from end to end; asking for the full
    gain everywhere turned such places down and the search ran out of time holding half of the
    memory).  Otherwise memory is occupied with filler blocks (memory the driver hands out in moderate
    blocks follows in physical address order; one huge block does not) and after every
    ``step_bytes`` of them the place a block of the pool's size gets is tried, until one is taken or
    the search runs out of ``max_filler_bytes`` (a region is 96 GiB), ``max_fraction_of_free`` of the
    memory that was free at the start, or ``max_seconds`` -- ``report["reason"]`` then says which.

    Everything the search occupies on the way -- fillers and the places it tried -- is held through
    the library (``rt_dev_hold``), not through torch, and given back before this returns; the place
    that shows the gain stays held and *is* the second pool (a torch tensor over that block, which
    goes back to the driver when its last view has gone).  torch's caching allocator only ever sees
    the first pool.  With little free memory the search simply ends early and the second pool is an
    ordinary torch allocation, wherever that lands (``placed: False``)."""
    stream = torch.cuda.current_stream(device).cuda_stream

    def zeros(nbytes):
        return torch.zeros(nbytes, dtype=torch.uint8, device=device)

    t0 = time.monotonic()
    report = {"placed": False, "filler_GiB": 0.0, "same_GBps": None, "cross_GBps": None, "tries": 0, "seconds": 0.0,
              "reason": None}
    free0, _ = torch.cuda.mem_get_info(device)
    if by_chunks and min(bytes_a, bytes_b) >= GIB:
        got = _place_pair_by_chunks(handle, device, bytes_a, bytes_b, free0, max_filler_bytes, max_fraction_of_free,
                                    max_seconds, stream, report, log, ref)
        if got is not None:
            report["seconds"] = time.monotonic() - t0
            return got[0], got[1], report
    a = zeros(bytes_a)
    # Pools under 1 GiB are not worth occupying -- and having the driver clear afterwards -- a hundred
    # GiB for: their launches are short and the probe on them says little.  From 1 GiB on the place
    # decides as much as for the largest sets (states of 1.7 GB each, fp64: 1.36 against 1.63 ms).
    by_size = max_filler_bytes if bytes_b >= GIB else 8 * bytes_b
    budget = min(by_size, int(max_fraction_of_free * max(0, free0 - bytes_a - bytes_b)))
    held, held_bytes = [], 0      # addresses of filler blocks held through the library
    best = None                   # (address, same, cross) of the best place seen that fell short of min_gain
    b = None

    def summary(r):
        # mean rates, and whether the place is good enough: the gain on the mean and some gain at every
        # probed position (a block that straddles two regions shows it at some of them only)
        same = sum(x[0] for x in r) / len(r)
        cross = sum(x[1] for x in r) / len(r)
        return same, cross, cross >= min_gain * same and all(x[1] >= min_gain_anywhere * x[0] for x in r)

    def adopt(addr, same, cross, placed):
        # this very block becomes the second pool: nothing is released and allocated again
        t = _HeldBlock(addr, bytes_b, device).tensor()
        t.zero_()
        report.update(placed=placed, filler_GiB=held_bytes / GIB, same_GBps=same, cross_GBps=cross)
        return t

    def out_of_time(next_cost=0.0):
        # (allocations take their time while the driver is still clearing memory that was released
        # shortly before: a block of 16 GiB up to half a second)
        if time.monotonic() - t0 + next_cost > max_seconds:
            report["reason"] = f"no place showed the whole gain within {max_seconds:g} s"
            return True
        return False

    try_cost = 0.0   # what the last try took, the allocation of its block included
    try:
        while b is None:
            free, _ = torch.cuda.mem_get_info(device)
            if bytes_b + 2 * GIB > free:
                report["reason"] = "not enough free device memory to try another place"
                break
            if report["tries"] and out_of_time(try_cost):
                break
            t_try = time.monotonic()
            try:
                cand = handle.dev_hold(bytes_b)   # the place the second pool would get right now
            except N.NativeError:
                report["reason"] = "not enough free device memory to try another place"
                break
            res = split_probe(handle, a.data_ptr(), bytes_a, cand, bytes_b, device, stream)
            if res is None:                       # pools too small to tell
                handle.dev_release(cand)
                report["reason"] = "pools too small for the probe to tell places apart"
                break
            same, cross, full = summary(res)
            try_cost = time.monotonic() - t_try
            report["tries"] += 1
            if report["cross_GBps"] is None:
                report.update(same_GBps=same, cross_GBps=cross)
            if log:
                log(f"{held_bytes / GIB:.0f} GiB occupied: same {same:.0f} GB/s, split {cross:.0f} GB/s")
            if full:
                b = adopt(cand, same, cross, True)
                break
            # Not here, or only in part (a block that straddles two regions shows the gain at some of
            # the probed positions).  The best such place stays held in case nothing better turns up;
            # any other is given back and occupied again, together with what follows it, by moderate
            # filler blocks: those the driver hands out in physical address order, which it does not
            # do for one huge block.
            if best is None or cross / same > best[2] / best[1]:
                if best is not None:
                    handle.dev_release(best[0])
                best = (cand, same, cross)
            else:
                handle.dev_release(cand)
            free, _ = torch.cuda.mem_get_info(device)
            if out_of_time():
                break
            if held_bytes + step_bytes > budget or step_bytes + bytes_b + 4 * GIB > free:
                report["reason"] = (f"no place showed the whole gain with {held_bytes / GIB:.0f} GiB occupied "
                                    f"(the search may hold {budget / GIB:.0f} GiB)")
                break
            try:
                for _ in range(max(1, step_bytes // filler_bytes)):
                    held.append(handle.dev_hold(filler_bytes))
                    held_bytes += filler_bytes
                    if out_of_time():
                        break
            except N.NativeError:
                report["reason"] = "not enough free device memory to occupy more"
                break
            if report["reason"]:
                break
        if b is None and best is not None and best[2] >= 1.01 * best[1]:
            report["reason"] = (report["reason"] or "") + "; the best place seen was taken"
            b = adopt(best[0], best[1], best[2], False)   # part of the gain is better than none
            best = None
    finally:
        for addr in held:
            handle.dev_release(addr)
        if best is not None:
            handle.dev_release(best[0])
    if b is None:
        b = zeros(bytes_b)
        report["reason"] = (report["reason"] or "") + "; the second pool is an ordinary allocation"
    report["seconds"] = time.monotonic() - t0
    return a, b, report
