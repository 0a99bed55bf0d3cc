"""ctypes binding of the C ABI in ``include/ramtorch_sr_adamw.h``.

The library is the only implementation of the step: if it is missing or does
not load, every entry point raises -- there is no fallback path.
"""
from __future__ import annotations

import atexit
import ctypes
import os
import sys
import threading
import weakref

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_lib", "libramtorch_sr_adamw.so")

ABI_VERSION = 4

RT_OK = 0
RT_EINVAL, RT_EHIP, RT_ENOMEM, RT_EUNSUPPORTED = -1, -2, -3, -4
RT_DT_BF16, RT_DT_F32, RT_DT_F16, RT_DT_F64 = 0, 1, 2, 3
RT_NOISE_PHILOX, RT_NOISE_EXPLICIT = 0, 1
RT_HOST_P, RT_HOST_G, RT_HOST_M, RT_HOST_V = 1, 2, 4, 8
RT_HOST_ORDERED = 16

#: every symbol the header declares
EXPORTS = (
    "rt_version", "rt_last_error", "rt_create", "rt_destroy", "rt_step_multi", "rt_step_streamed",
    "rt_grad_norm", "rt_row_means", "rt_sr_copy", "rt_set_timing", "rt_last_kernel_ms", "rt_kernel_ms_history", "rt_streamed_stats",
    "rt_stream_probe", "rt_streamed_timeline", "rt_streamed_plan",
    "rt_step_streamed_async", "rt_streamed_wait", "rt_streamed_completed",
    "rt_grad_norm_static", "rt_host_link_probe", "rt_selftest_sqrt", "rt_dev_hold", "rt_dev_release", "rt_dev_hold_pair",
    "rt_streamed_bounce_stats", "rt_row_means_multi", "rt_streamed_schedule",
)


class RtScalars(ctypes.Structure):
    _fields_ = [
        ("beta1", ctypes.c_float),
        ("one_m_beta1", ctypes.c_float),
        ("beta2", ctypes.c_float),
        ("one_m_beta2", ctypes.c_float),
        ("inv_bcs", ctypes.c_float),
        ("eps", ctypes.c_float),
        ("decay", ctypes.c_float),
        ("neg_step_size", ctypes.c_float),
        ("inv_loss_scale", ctypes.c_float),
        ("centralization", ctypes.c_float),
        ("apply_decay", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class RtTensorDesc(ctypes.Structure):
    _fields_ = [
        ("p", ctypes.c_void_p),
        ("g", ctypes.c_void_p),
        ("m", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("noise_p", ctypes.c_void_p),
        ("noise_m", ctypes.c_void_p),
        ("noise_v", ctypes.c_void_p),
        ("dbg_p", ctypes.c_void_p),
        ("dbg_m", ctypes.c_void_p),
        ("dbg_v", ctypes.c_void_p),
        ("row_mean", ctypes.c_void_p),
        ("numel", ctypes.c_uint64),
        ("elem_offset", ctypes.c_uint64),
        ("row_len", ctypes.c_uint64),
        ("tensor_id", ctypes.c_uint32),
        ("step", ctypes.c_uint32),
        ("scalars_idx", ctypes.c_uint32),
        ("p_dtype", ctypes.c_uint8),
        ("g_dtype", ctypes.c_uint8),
        ("m_dtype", ctypes.c_uint8),
        ("v_dtype", ctypes.c_uint8),
        ("host_mask", ctypes.c_uint32),
        ("reserved", ctypes.c_uint32),
    ]


class RtSchedOp(ctypes.Structure):
    """One operation of a streamed call's schedule (``rt_sched_op``)."""
    _fields_ = [
        ("kind", ctypes.c_uint32),
        ("chunk", ctypes.c_uint32),
        ("stage", ctypes.c_uint32),
        ("bounce", ctypes.c_uint32),
        ("wait_event", ctypes.c_uint32),
        ("record_event", ctypes.c_uint32),
        ("value", ctypes.c_uint64),
    ]


(RT_OP_HOST_WAIT_BACK, RT_OP_HOST_FILL, RT_OP_HOST_WAIT_FILL, RT_OP_HOST_DRAIN, RT_OP_HOST_WAIT_DRAIN, RT_OP_H2D,
 RT_OP_KERNEL, RT_OP_D2H, RT_OP_PUBLISH, RT_OP_TICKET, RT_OP_HOST_WAIT_IDLE) = range(11)
RT_EV_H2D_DONE, RT_EV_COMP_DONE, RT_EV_D2H_DONE = 0, 2, 4
RT_SCHED_NONE = 0xFFFFFFFF

assert ctypes.sizeof(RtSchedOp) == 32
assert ctypes.sizeof(RtScalars) == 48
assert ctypes.sizeof(RtTensorDesc) == 136


class NativeError(RuntimeError):
    """A C-ABI call returned a non-zero code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"ramtorch_sr_adamw error {code}: {message}")
        self.code = code


_lib = None


def lib() -> ctypes.CDLL:
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. "
            "Run `python -m ramtorch_amd.build` (needs hipcc); there is no fallback implementation.")
    L = ctypes.CDLL(LIB_PATH)
    vp, u32, u64, i32 = ctypes.c_void_p, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_int
    descs, scal = ctypes.POINTER(RtTensorDesc), ctypes.POINTER(RtScalars)
    L.rt_version.restype = i32
    L.rt_version.argtypes = []
    L.rt_last_error.restype = ctypes.c_char_p
    L.rt_last_error.argtypes = []
    L.rt_create.restype = i32
    L.rt_create.argtypes = [i32, ctypes.POINTER(vp)]
    L.rt_destroy.restype = i32
    L.rt_destroy.argtypes = [vp]
    L.rt_step_multi.restype = i32
    L.rt_step_multi.argtypes = [vp, descs, u32, scal, u32, u64, i32, vp, vp, vp]
    L.rt_step_streamed.restype = i32
    L.rt_step_streamed.argtypes = [vp, descs, u32, scal, u32, u64, i32, u64, vp, vp, vp]
    L.rt_grad_norm.restype = i32
    L.rt_grad_norm.argtypes = [vp, descs, u32, ctypes.c_float, ctypes.c_float, vp, vp]
    L.rt_grad_norm_static.restype = i32
    L.rt_grad_norm_static.argtypes = [vp, descs, u32, ctypes.c_float, ctypes.c_float, vp, vp]
    L.rt_host_link_probe.restype = i32
    L.rt_host_link_probe.argtypes = [vp, u64, i32, ctypes.POINTER(ctypes.c_double)]
    L.rt_dev_hold.restype = i32
    L.rt_dev_hold.argtypes = [vp, u64, ctypes.POINTER(vp)]
    L.rt_dev_release.restype = i32
    L.rt_dev_release.argtypes = [vp, vp]
    L.rt_dev_hold_pair.restype = i32
    L.rt_dev_hold_pair.argtypes = [vp, u64, u64, u64, ctypes.c_double, vp, vp, vp, u64, ctypes.POINTER(vp),
                                   ctypes.POINTER(vp), ctypes.POINTER(ctypes.c_double), vp]
    L.rt_selftest_sqrt.restype = i32
    L.rt_selftest_sqrt.argtypes = [vp, ctypes.POINTER(u64)]
    L.rt_row_means_multi.restype = i32
    L.rt_row_means_multi.argtypes = [vp, descs, u32, ctypes.c_float, vp]
    L.rt_row_means.restype = i32
    L.rt_row_means.argtypes = [vp, vp, i32, u64, u64, ctypes.c_float, vp, vp]
    L.rt_sr_copy.restype = i32
    L.rt_sr_copy.argtypes = [vp, vp, u64, vp, u64, vp]
    L.rt_set_timing.restype = i32
    L.rt_set_timing.argtypes = [vp, i32]
    L.rt_last_kernel_ms.restype = i32
    L.rt_last_kernel_ms.argtypes = [vp, ctypes.POINTER(ctypes.c_float)]
    L.rt_kernel_ms_history.restype = i32
    L.rt_kernel_ms_history.argtypes = [vp, ctypes.POINTER(ctypes.c_float), u32, ctypes.POINTER(u32)]
    L.rt_stream_probe.restype = i32
    L.rt_stream_probe.argtypes = [vp, vp, vp, vp, vp, u64, i32, ctypes.POINTER(ctypes.c_float), vp]
    L.rt_streamed_timeline.restype = i32
    L.rt_streamed_timeline.argtypes = [vp, ctypes.POINTER(ctypes.c_float), u32, ctypes.POINTER(u32)]
    L.rt_step_streamed_async.restype = i32
    L.rt_step_streamed_async.argtypes = [vp, descs, u32, scal, u32, u64, i32, u64, vp, vp, vp, ctypes.POINTER(u64)]
    L.rt_streamed_wait.restype = i32
    L.rt_streamed_wait.argtypes = [vp]
    L.rt_streamed_completed.restype = i32
    L.rt_streamed_completed.argtypes = [vp, ctypes.POINTER(u64)]
    L.rt_streamed_plan.restype = i32
    L.rt_streamed_plan.argtypes = [descs, u32, u64, ctypes.POINTER(u64), u32, ctypes.POINTER(u32)]
    L.rt_streamed_schedule.restype = i32
    L.rt_streamed_schedule.argtypes = [u32, u64, u32, i32, i32, u64, ctypes.POINTER(RtSchedOp), u32, ctypes.POINTER(u32)]
    L.rt_streamed_stats.restype = i32
    L.rt_streamed_stats.argtypes = [vp, ctypes.POINTER(ctypes.c_double)]
    L.rt_streamed_bounce_stats.restype = i32
    L.rt_streamed_bounce_stats.argtypes = [vp, ctypes.POINTER(ctypes.c_uint64)]
    v = L.rt_version()
    if v != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {v}, this package expects {ABI_VERSION}; rebuild it")
    _lib = L
    return L


def check(code: int) -> None:
    if code != RT_OK:
        raise NativeError(code, lib().rt_last_error().decode("utf-8", "replace"))


class Handle:
    """Owns one ``rt_handle`` (workspace of one device)."""

    def __init__(self, device: int):
        self._h = ctypes.c_void_p()
        check(lib().rt_create(int(device), ctypes.byref(self._h)))
        self.device = int(device)
        # ctypes drops the GIL during a call and an rt_handle is not re-entrant: calls on one handle
        # from several Python threads (the main thread and autograd's hook threads) take turns.
        self._lock = threading.RLock()
        _live_handles.add(self)

    @property
    def ptr(self) -> ctypes.c_void_p:
        if not self._h:
            raise RuntimeError("handle already destroyed")
        return self._h

    def close(self) -> None:
        if self._h:
            lib().rt_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        # During interpreter shutdown the HIP runtime may already be gone; the
        # atexit hook below has released everything that was still open.
        if sys is None or sys.is_finalizing():
            return
        try:
            self.close()
        except Exception:
            pass

    # -- thin wrappers ---------------------------------------------------------
    def step_multi(self, descs, n, scalars, n_scalars, seed, noise_mode, d_clip_coef=None, d_skip=None, stream=0):
        with self._lock:
            check(lib().rt_step_multi(self.ptr, descs, n, scalars, n_scalars, seed, noise_mode, d_clip_coef,
                                      d_skip, stream))

    def step_streamed(self, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems, d_clip_coef=None,
                      d_skip=None, stream=0):
        with self._lock:
            check(lib().rt_step_streamed(self.ptr, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems,
                                         d_clip_coef, d_skip, stream))

    def step_streamed_async(self, descs, n, scalars, n_scalars, seed, noise_mode, chunk_elems, d_clip_coef=None,
                            d_skip=None, stream=0) -> int:
        """Enqueue only; returns the ticket of the call."""
        t = ctypes.c_uint64()
        with self._lock:
            check(lib().rt_step_streamed_async(self.ptr, descs, n, scalars, n_scalars, seed, noise_mode,
                                               chunk_elems, d_clip_coef, d_skip, stream, ctypes.byref(t)))
        return t.value

    def streamed_wait(self) -> None:
        with self._lock:
            check(lib().rt_streamed_wait(self.ptr))

    def streamed_completed(self) -> int:
        t = ctypes.c_uint64()
        with self._lock:
            check(lib().rt_streamed_completed(self.ptr, ctypes.byref(t)))
        return t.value

    def grad_norm(self, descs, n, inv_loss_scale, max_norm, d_out, stream=0):
        with self._lock:
            check(lib().rt_grad_norm(self.ptr, descs, n, inv_loss_scale, max_norm, d_out, stream))

    def grad_norm_static(self, descs, n, inv_loss_scale, max_norm, d_out, stream=0):
        """rt_grad_norm without any device allocation (at most 4096 non-empty gradients)."""
        with self._lock:
            check(lib().rt_grad_norm_static(self.ptr, descs, n, inv_loss_scale, max_norm, d_out, stream))

    def host_link_probe(self, nbytes: int, reps: int = 8):
        """Pinned-copy rates of the host link in GB/s: host to device, device to host, each way with both at once."""
        out = (ctypes.c_double * 3)()
        with self._lock:
            check(lib().rt_host_link_probe(self.ptr, int(nbytes), int(reps), out))
        return {"h2d_GBps": out[0], "d2h_GBps": out[1], "duplex_GBps_each_way": out[2]}

    def dev_hold(self, nbytes: int) -> int:
        """Address of a device block of ``nbytes`` that is only held (see rt_dev_hold); raises NativeError
        with code RT_ENOMEM when there is none."""
        out = ctypes.c_void_p()
        with self._lock:
            check(lib().rt_dev_hold(self.ptr, int(nbytes), ctypes.byref(out)))
        return out.value

    def dev_hold_pair(self, bytes_a: int, bytes_b: int, max_extra_bytes: int, max_seconds: float, ref=None, stream=0):
        """(address a, address b, report) of two zeroed blocks that never share an HBM region (see
        rt_dev_hold_pair); ``ref``: optional (address, address, address, elements) of three arrays in parameter memory."""
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        rep = (ctypes.c_double * 8)()
        rp, rm, rv, rn = ref if ref else (None, None, None, 0)
        with self._lock:
            check(lib().rt_dev_hold_pair(self.ptr, int(bytes_a), int(bytes_b), int(max_extra_bytes), float(max_seconds),
                                         rp, rm, rv, int(rn), ctypes.byref(a), ctypes.byref(b), rep, stream))
        return a.value, b.value, list(rep)

    def dev_release(self, addr: int) -> None:
        with self._lock:
            check(lib().rt_dev_release(self.ptr, ctypes.c_void_p(addr)))

    def selftest_sqrt(self) -> int:
        """Number of floats in [2^-96, inf) on which the kernels' short sqrt differs from sqrtf (expected 0)."""
        n = ctypes.c_uint64()
        with self._lock:
            check(lib().rt_selftest_sqrt(self.ptr, ctypes.byref(n)))
        return n.value

    def row_means_multi(self, descs, n, inv_loss_scale, stream=0):
        with self._lock:
            check(lib().rt_row_means_multi(self.ptr, descs, n, inv_loss_scale, stream))

    def row_means(self, g, g_dtype, rows, row_len, inv_loss_scale, d_row_mean, stream=0):
        with self._lock:
            check(lib().rt_row_means(self.ptr, g, g_dtype, rows, row_len, inv_loss_scale, d_row_mean, stream))

    def set_timing(self, enabled: bool) -> None:
        with self._lock:
            check(lib().rt_set_timing(self.ptr, int(enabled)))

    def last_kernel_ms(self) -> float:
        ms = ctypes.c_float()
        with self._lock:
            check(lib().rt_last_kernel_ms(self.ptr, ctypes.byref(ms)))
        return ms.value

    def kernel_ms_history(self, cap: int = 256):
        """Durations (ms) of the most recent timed launches since set_timing(True), oldest first."""
        buf = (ctypes.c_float * cap)()
        n = ctypes.c_uint32()
        with self._lock:
            check(lib().rt_kernel_ms_history(self.ptr, buf, cap, ctypes.byref(n)))
        return [buf[i] for i in range(n.value)]

    def stream_probe(self, p, g, m, v, numel, reps=5, stream=0) -> float:
        """Mean ms per pass of the math-free traffic pattern (see rt_stream_probe)."""
        ms = ctypes.c_float()
        with self._lock:
            check(lib().rt_stream_probe(self.ptr, p, g, m, v, numel, reps, ctypes.byref(ms), stream))
        return ms.value

    def streamed_timeline(self):
        """[(h2d_begin, h2d_end, d2h_begin, d2h_end), ...] in ms for the last timed streamed call."""
        n = ctypes.c_uint32()
        with self._lock:
            check(lib().rt_streamed_timeline(self.ptr, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_float * max(n.value, 1))()
        with self._lock:
            check(lib().rt_streamed_timeline(self.ptr, buf, n.value, ctypes.byref(n)))
        return [tuple(buf[i:i + 4]) for i in range(0, n.value, 4)]

    def streamed_stats(self):
        out = (ctypes.c_double * 3)()
        with self._lock:
            check(lib().rt_streamed_stats(self.ptr, out))
        return {"bytes_h2d": out[0], "bytes_d2h": out[1], "seconds": out[2]}

    def streamed_bounce_stats(self):
        """Calls that met host arrays that are not pinned, and the bytes host threads copied for them."""
        out = (ctypes.c_uint64 * 2)()
        with self._lock:
            check(lib().rt_streamed_bounce_stats(self.ptr, out))
        return {"calls": int(out[0]), "bytes": int(out[1])}


_live_handles: "weakref.WeakSet[Handle]" = weakref.WeakSet()


@atexit.register
def _close_all_handles() -> None:
    """Release device workspaces while the HIP runtime is still alive."""
    for h in list(_live_handles):
        try:
            h.close()
        except Exception:
            pass


def streamed_plan(descs, n: int, chunk_elems: int):
    """[(chunk, tensor, start, count, stage_offset), ...]: the schedule of rt_step_streamed (host only)."""
    k = ctypes.c_uint32()
    check(lib().rt_streamed_plan(descs, n, chunk_elems, None, 0, ctypes.byref(k)))
    buf = (ctypes.c_uint64 * max(5 * k.value, 1))()
    check(lib().rt_streamed_plan(descs, n, chunk_elems, buf, k.value, ctypes.byref(k)))
    return [tuple(buf[5 * i:5 * i + 5]) for i in range(k.value)]


def streamed_schedule(n_chunks: int, seq0: int = 0, used_mask: int = 0, paced_up: bool = False,
                      paced_down: bool = False, batch_chunks: int = 64):
    """The operations of a streamed call in the order the host issues them (host only): a list of
    ``RtSchedOp``.  This is the list the library itself executes."""
    k = ctypes.c_uint32()
    args = (int(n_chunks), int(seq0), int(used_mask), int(paced_up), int(paced_down), int(batch_chunks))
    check(lib().rt_streamed_schedule(*args, None, 0, ctypes.byref(k)))
    buf = (RtSchedOp * max(k.value, 1))()
    check(lib().rt_streamed_schedule(*args, buf, k.value, ctypes.byref(k)))
    return list(buf[:k.value])


def dev_release(addr: int) -> None:
    """Give a block of rt_dev_hold back without a handle (hipFree finds the device by the address)."""
    check(lib().rt_dev_release(None, ctypes.c_void_p(addr)))


def sr_copy(target_ptr, source_ptr, numel, noise_ptr, seed, stream=0) -> None:
    check(lib().rt_sr_copy(target_ptr, source_ptr, numel, noise_ptr, seed, stream))
