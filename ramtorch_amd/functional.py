"""Host-side packing for the fused SR-AdamW step: torch tensors in, C-ABI
descriptor tables out.  Mirrors what ``AdamW.step`` of the reference computes in
Python before it touches a tensor (ramtorch/stochastic_optimizers/adamw.py:173-188)
and hands the rest to the HIP library.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _native as N

_DT_CODE = {torch.bfloat16: N.RT_DT_BF16, torch.float32: N.RT_DT_F32, torch.float16: N.RT_DT_F16}
#: params and states may also be fp64 (upcast / plain copy_ semantics of adamw.py:160-170, 208-222)
_DT_CODE_PMV = dict(_DT_CODE)
_DT_CODE_PMV[torch.float64] = N.RT_DT_F64

#: numpy mirror of ``rt_tensor_desc`` (same field order and offsets)
DESC_DTYPE = np.dtype(
    [("p", "<u8"), ("g", "<u8"), ("m", "<u8"), ("v", "<u8"),
     ("noise_p", "<u8"), ("noise_m", "<u8"), ("noise_v", "<u8"),
     ("dbg_p", "<u8"), ("dbg_m", "<u8"), ("dbg_v", "<u8"), ("row_mean", "<u8"),
     ("numel", "<u8"), ("elem_offset", "<u8"), ("row_len", "<u8"),
     ("tensor_id", "<u4"), ("step", "<u4"), ("scalars_idx", "<u4"),
     ("p_dtype", "u1"), ("g_dtype", "u1"), ("m_dtype", "u1"), ("v_dtype", "u1"),
     ("host_mask", "<u4"), ("reserved", "<u4")], align=False)
assert DESC_DTYPE.itemsize == ctypes.sizeof(N.RtTensorDesc)


def dtype_code(dt: torch.dtype, what: str) -> int:
    try:
        return (_DT_CODE if what == "grad" else _DT_CODE_PMV)[dt]
    except KeyError:
        raise NotImplementedError(f"{what} dtype {dt} is not supported by the HIP step (bf16 / fp32 / fp16; "
                                  "fp64 for params and states)") from None


def make_scalars(lr: float, betas: Tuple[float, float], eps: float, weight_decay: float, step: int,
                 centralization: float = 0.0, inv_loss_scale: float = 1.0) -> N.RtScalars:
    """The Python-double scalar math of adamw.py:173-188, each value rounded to
    float32 where an ATen call of adamw.py:190-200 consumes it.  ``step`` is the
    value after the increment of adamw.py:177."""
    beta1, beta2 = betas
    bias_correction = 1 - beta1 ** step
    bias_correction_sqrt = (1 - beta2 ** step) ** (1 / 2)
    step_size = lr / bias_correction
    f32 = np.float32
    # `tensor / python_float` on the GPU multiplies by the reciprocal of the scalar, taken in
    # double precision and then rounded to float32
    inv_bcs = f32(1.0 / bias_correction_sqrt)
    apply_decay = weight_decay != 0
    return N.RtScalars(
        beta1=f32(beta1), one_m_beta1=f32(1 - beta1), beta2=f32(beta2), one_m_beta2=f32(1 - beta2),
        inv_bcs=inv_bcs, eps=f32(eps),
        decay=f32(1 - step_size * weight_decay) if apply_decay else f32(1.0),
        neg_step_size=f32(-step_size), inv_loss_scale=f32(inv_loss_scale), centralization=f32(centralization),
        apply_decay=int(apply_decay), reserved=0)


@dataclass
class Entry:
    """One tensor of one step.  All four arrays hold ``p.numel()`` contiguous elements."""
    p: torch.Tensor
    g: torch.Tensor
    m: torch.Tensor
    v: torch.Tensor
    step: int
    scalars_idx: int
    tensor_id: int
    noise: Optional[Tuple[Optional[torch.Tensor], Optional[torch.Tensor], Optional[torch.Tensor]]] = None
    dbg: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None
    row_mean: Optional[torch.Tensor] = None
    row_len: int = 0
    elem_offset: int = 0
    ordered: bool = False  # host arrays may still be written by work queued on the stream: uploads wait for it
    keep: list = field(default_factory=list)  # temporaries that must outlive the launch


ROWWISE_MIN_LEN, ROWWISE_MAX_LEN = 512, 32768


def rowwise_ok(e: "Entry", row_len: int, explicit_noise: bool = False) -> bool:
    """Whether the update kernel can take the row means of this entry's gradient itself
    (centralization, adamw.py:179-184) instead of reading them from ``row_mean``: whole tensors of
    16-bit arrays on the GPU, 16-byte aligned, Philox noise, no debug outputs, rows a multiple of 8
    and 512 .. 32768 elements long -- the same rule as the library's (it rejects anything else)."""
    if explicit_noise or e.noise is not None or e.dbg is not None or e.elem_offset or e.row_mean is not None:
        return False
    if row_len % 8 or not (ROWWISE_MIN_LEN <= row_len <= ROWWISE_MAX_LEN) or e.p.numel() % row_len:
        return False
    for t in (e.p, e.g, e.m, e.v):
        if not t.is_cuda or t.dtype not in (torch.bfloat16, torch.float16) or t.data_ptr() % 16 or not t.is_contiguous():
            return False
    # fp16 states come in pairs in the templated kernels; anything else is the runtime-typed kernel's
    return (e.m.dtype == torch.float16) == (e.v.dtype == torch.float16)


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def pack_descs(entries: Sequence[Entry], streamed: bool) -> np.ndarray:
    """Build the ``rt_tensor_desc`` array.  For the resident entry point every
    tensor must be on the GPU; for the streamed one ``host_mask`` marks the CPU ones."""
    n = len(entries)
    d = np.zeros(n, DESC_DTYPE)
    if n == 0:
        return d
    d["p"] = [e.p.data_ptr() for e in entries]
    d["g"] = [e.g.data_ptr() for e in entries]
    d["m"] = [e.m.data_ptr() for e in entries]
    d["v"] = [e.v.data_ptr() for e in entries]
    d["numel"] = [e.p.numel() for e in entries]
    d["tensor_id"] = [e.tensor_id for e in entries]
    d["step"] = [e.step & 0xFFFFFFFF for e in entries]
    d["scalars_idx"] = [e.scalars_idx for e in entries]
    d["p_dtype"] = [dtype_code(e.p.dtype, "param") for e in entries]
    d["g_dtype"] = [dtype_code(e.g.dtype, "grad") for e in entries]
    d["m_dtype"] = [dtype_code(e.m.dtype, "state") for e in entries]
    d["v_dtype"] = [dtype_code(e.v.dtype, "state") for e in entries]
    if any(e.elem_offset for e in entries):
        d["elem_offset"] = [e.elem_offset for e in entries]
    for i, e in enumerate(entries):
        if e.g.numel() != e.p.numel() or e.m.numel() != e.p.numel() or e.v.numel() != e.p.numel():
            raise ValueError(f"tensor {i}: p/g/m/v element counts differ")
        if e.noise is not None:
            for name, t, tgt in zip(("noise_p", "noise_m", "noise_v"), e.noise, (e.p, e.m, e.v)):
                if t is None:
                    continue
                if t.dtype not in (torch.int16, torch.uint16) or t.numel() != tgt.numel() or not t.is_cuda \
                        or not t.is_contiguous():
                    raise ValueError(f"tensor {i}: {name} must be a contiguous int16 CUDA tensor of p's size")
                d[name][i] = t.data_ptr()
        if e.dbg is not None:
            for name, t in zip(("dbg_p", "dbg_m", "dbg_v"), e.dbg):
                if t.dtype != torch.float32 or t.numel() != e.p.numel() or not t.is_cuda or not t.is_contiguous():
                    raise ValueError(f"tensor {i}: {name} must be a contiguous fp32 CUDA tensor of p's size")
                d[name][i] = t.data_ptr()
        if e.row_mean is not None:
            d["row_mean"][i] = e.row_mean.data_ptr()
            d["row_len"][i] = e.row_len
        elif e.row_len:
            d["row_len"][i] = e.row_len   # the update kernel takes the row means itself (see rowwise_ok)
        mask = 0
        for bit, t in ((N.RT_HOST_P, e.p), (N.RT_HOST_G, e.g), (N.RT_HOST_M, e.m), (N.RT_HOST_V, e.v)):
            if not t.is_contiguous():
                raise ValueError(f"tensor {i}: arrays must be contiguous")
            if not t.is_cuda:
                mask |= bit
        if mask and not streamed:
            raise ValueError(f"tensor {i}: a CPU tensor reached the resident entry point")
        if mask and e.ordered:
            mask |= N.RT_HOST_ORDERED
        d["host_mask"][i] = mask
    return d


def scalars_array(scalars: Sequence[N.RtScalars]):
    arr = (N.RtScalars * max(len(scalars), 1))()
    for i, s in enumerate(scalars):
        arr[i] = s
    return arr


def _descs_ptr(d: np.ndarray):
    return d.ctypes.data_as(ctypes.POINTER(N.RtTensorDesc))


def launch_resident(handle: N.Handle, descs: np.ndarray, scalars: Sequence[N.RtScalars], *, seed: int,
                    explicit_noise: bool, clip_coef: Optional[torch.Tensor] = None,
                    skip: Optional[torch.Tensor] = None, stream: Optional[int] = None) -> None:
    """``rt_step_multi`` over an already packed ``rt_tensor_desc`` array (every
    pointer a device address).  Enqueues on ``stream`` (default: torch's current
    stream) and returns without synchronising; the caller keeps the tensors alive."""
    if len(descs) == 0:
        return
    descs = np.ascontiguousarray(descs)
    if stream is None:
        stream = torch.cuda.current_stream(handle.device).cuda_stream
    handle.step_multi(_descs_ptr(descs), len(descs), scalars_array(scalars), len(scalars), seed & (2 ** 64 - 1),
                      N.RT_NOISE_EXPLICIT if explicit_noise else N.RT_NOISE_PHILOX,
                      None if clip_coef is None else clip_coef.data_ptr(),
                      None if skip is None else skip.data_ptr(), stream)


def step_resident(handle: N.Handle, entries: Sequence[Entry], scalars: Sequence[N.RtScalars], *, seed: int,
                  explicit_noise: bool, clip_coef: Optional[torch.Tensor] = None,
                  skip: Optional[torch.Tensor] = None, stream: Optional[int] = None) -> None:
    """One launch (per dtype combination) over GPU-resident tensors on ``stream``
    (default: torch's current stream).  Returns without synchronising."""
    if not entries:
        return
    launch_resident(handle, pack_descs(entries, streamed=False), scalars, seed=seed, explicit_noise=explicit_noise,
                    clip_coef=clip_coef, skip=skip, stream=stream)


def step_streamed(handle: N.Handle, entries: Sequence[Entry], scalars: Sequence[N.RtScalars], *, seed: int,
                  explicit_noise: bool, chunk_elems: int, stream: Optional[int] = None,
                  wait: bool = True, clip_coef: Optional[torch.Tensor] = None,
                  skip: Optional[torch.Tensor] = None, descs: Optional[np.ndarray] = None) -> Optional[int]:
    """Chunked H2D / update / D2H for tensors with CPU-resident arrays.  With
    ``wait`` (default) host memory is final when this returns.  Without it the
    call only enqueues and returns a ticket: until ``handle.streamed_completed()``
    reaches it (or ``handle.streamed_wait()`` returns) the caller must keep the
    tensors alive and leave p / m / v alone."""
    if not entries:
        return None
    d = pack_descs(entries, streamed=True) if descs is None else descs
    if stream is None:
        stream = torch.cuda.current_stream(handle.device).cuda_stream
    args = (_descs_ptr(d), len(entries), scalars_array(scalars), len(scalars), seed & (2 ** 64 - 1),
            N.RT_NOISE_EXPLICIT if explicit_noise else N.RT_NOISE_PHILOX, int(chunk_elems),
            None if clip_coef is None else clip_coef.data_ptr(), None if skip is None else skip.data_ptr(), stream)
    if wait:
        handle.step_streamed(*args)
        return None
    return handle.step_streamed_async(*args)


def grad_norm(handle: N.Handle, grads: Sequence[torch.Tensor], *, inv_loss_scale: float = 1.0,
              max_norm: float = 1.0, out: Optional[torch.Tensor] = None,
              stream: Optional[int] = None) -> torch.Tensor:
    """Global L2 norm of GPU gradients.  Returns a 4-float CUDA tensor:
    [total_norm, clip_coef, found_inf (as uint32 bits), unused]."""
    if out is None:
        out = torch.zeros(4, dtype=torch.float32, device=f"cuda:{handle.device}")
    n = len(grads)
    d = np.zeros(n, DESC_DTYPE)
    if n:
        for g in grads:
            if not g.is_cuda or not g.is_contiguous():
                raise ValueError("grad_norm needs contiguous CUDA gradients")
        d["g"] = [g.data_ptr() for g in grads]
        d["numel"] = [g.numel() for g in grads]
        d["g_dtype"] = [dtype_code(g.dtype, "grad") for g in grads]
    if stream is None:
        stream = torch.cuda.current_stream(handle.device).cuda_stream
    handle.grad_norm(_descs_ptr(d), n, float(inv_loss_scale), float(max_norm), out.data_ptr(), stream)
    return out


def row_means(handle: N.Handle, g: torch.Tensor, rows: int, row_len: int, inv_loss_scale: float = 1.0,
              stream: Optional[int] = None) -> torch.Tensor:
    out = torch.empty(max(rows, 1), dtype=torch.float32, device=g.device)
    if stream is None:
        stream = torch.cuda.current_stream(handle.device).cuda_stream
    handle.row_means(g.data_ptr(), dtype_code(g.dtype, "grad"), rows, row_len, float(inv_loss_scale),
                     out.data_ptr(), stream)
    return out


def row_means_multi(handle: N.Handle, jobs: Sequence[Tuple[Entry, int, int]], inv_loss_scale: float = 1.0,
                    stream: Optional[int] = None) -> None:
    """Row means of the GPU gradients of many entries in one launch.  ``jobs`` holds
    (entry, rows, row_len); every entry gets ``row_mean`` (a view into one fp32 buffer) and ``row_len``."""
    jobs = [j for j in jobs if j[1] > 0 and j[2] > 0]
    if not jobs:
        return
    dev = jobs[0][0].g.device
    buf = torch.empty(sum(rows for _, rows, _ in jobs), dtype=torch.float32, device=dev)
    d = np.zeros(len(jobs), DESC_DTYPE)
    off = 0
    for k, (e, rows, row_len) in enumerate(jobs):
        if not e.g.is_cuda or not e.g.is_contiguous():
            raise ValueError("row_means_multi needs contiguous CUDA gradients")
        e.row_mean = buf[off:off + rows]
        e.row_len = row_len
        off += rows
        d["g"][k] = e.g.data_ptr()
        d["g_dtype"][k] = dtype_code(e.g.dtype, "grad")
        d["numel"][k] = rows * row_len
        d["row_len"][k] = row_len
        d["row_mean"][k] = e.row_mean.data_ptr()
    if stream is None:
        stream = torch.cuda.current_stream(handle.device).cuda_stream
    handle.row_means_multi(_descs_ptr(d), len(jobs), float(inv_loss_scale), stream)
