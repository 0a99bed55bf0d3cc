"""CPU oracle for the stochastic-rounding AdamW step -- TEST INFRASTRUCTURE ONLY.

Python face of ``sr_adamw_oracle.c`` (plain scalar C restating the reference's
``ramtorch/stochastic_optimizers/adamw.py``).  Only ``tests/``, the smoke check
and the benchmark's ``cpu_baseline`` leg may import this package; the shipped
library never does, and nothing here touches a GPU.

Arrays are numpy: bf16 and fp16 data travel as ``uint16`` bit patterns, fp32 as
``float32``.  The dtype of an argument is stated explicitly where it matters.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

# flavour bits (mirrors of the C defines)
FMA_ADD = 1
FMA_ADDCMUL = 2
FMA_ADDCDIV = 4
DIV_RECIP = 8
ADDCMUL_AG_FIRST = 16
ADDCDIV_AM_FIRST = 32

#: rounding sequence of torch's CPU kernels (adamw.py:190-200 run on CPU tensors)
TORCH_CPU_FLAVOUR = FMA_ADD | FMA_ADDCMUL | ADDCMUL_AG_FIRST | ADDCDIV_AM_FIRST
#: rounding sequence of torch's GPU (ROCm) kernels -- what the reference executes,
#: since adamw.py:152-157 always computes on a GPU.  Pinned on the GPU box by
#: tests/test_gpu_parity.py against the ATen kernels themselves, and here by the
#: golden vectors those kernels produced (tests/golden/torch_gpu_step.npz).
REFERENCE_FLAVOUR = FMA_ADD | FMA_ADDCMUL | FMA_ADDCDIV | DIV_RECIP

DT_BF16, DT_F32, DT_F16, DT_F64 = 0, 1, 2, 3
NOISE_PHILOX, NOISE_EXPLICIT = 0, 1


class Scalars(ctypes.Structure):
    _fields_ = [
        ("beta1", ctypes.c_float),
        ("one_m_beta1", ctypes.c_float),
        ("beta2", ctypes.c_float),
        ("one_m_beta2", ctypes.c_float),
        ("bcs", ctypes.c_float),
        ("inv_bcs", ctypes.c_float),
        ("eps", ctypes.c_float),
        ("decay", ctypes.c_float),
        ("neg_step_size", ctypes.c_float),
        ("inv_loss_scale", ctypes.c_float),
        ("apply_decay", ctypes.c_int32),
        ("apply_clip", ctypes.c_int32),
    ]


def build(force: bool = False) -> str:
    """Compile liboracle.so with the committed Makefile (gcc only)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        u16p = ctypes.POINTER(ctypes.c_uint16)
        f32p = ctypes.POINTER(ctypes.c_float)
        vp = ctypes.c_void_p
        L.orc_sr_bf16.restype = ctypes.c_uint16
        L.orc_sr_bf16.argtypes = [ctypes.c_float, ctypes.c_uint16]
        L.orc_bf16_to_f32.restype = ctypes.c_float
        L.orc_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_f16_rne.restype = ctypes.c_uint16
        L.orc_f32_to_f16_rne.argtypes = [ctypes.c_float]
        L.orc_f32_to_f16_array.restype = None
        L.orc_f32_to_f16_array.argtypes = [f32p, u16p, ctypes.c_uint64]
        L.orc_philox4x32_10.restype = None
        L.orc_philox4x32_10.argtypes = [ctypes.POINTER(ctypes.c_uint32)] * 3
        L.orc_philox_noise.restype = ctypes.c_uint16
        L.orc_philox_noise.argtypes = [ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint32,
                                       ctypes.c_uint64]
        L.orc_update_elem.restype = None
        L.orc_update_elem.argtypes = [ctypes.c_float] * 4 + [ctypes.POINTER(Scalars), ctypes.c_float,
                                                             ctypes.c_uint32, f32p, f32p, f32p]
        L.orc_step_tensor.restype = ctypes.c_int
        L.orc_step_tensor.argtypes = [vp, ctypes.c_int, vp, ctypes.c_int, vp, ctypes.c_int, vp, ctypes.c_int,
                                      ctypes.c_uint64, ctypes.POINTER(Scalars), ctypes.c_float, ctypes.c_int,
                                      u16p, u16p, u16p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_uint32,
                                      ctypes.c_uint64, ctypes.c_uint32, f32p, f32p, f32p]
        L.orc_sr_copy.restype = None
        L.orc_sr_copy.argtypes = [u16p, f32p, ctypes.c_uint64, ctypes.c_int, u16p, ctypes.c_uint64]
        L.orc_grad_sumsq.restype = ctypes.c_double
        L.orc_grad_sumsq.argtypes = [vp, ctypes.c_int, ctypes.c_uint64, ctypes.c_float]
        L.orc_row_means.restype = None
        L.orc_row_means.argtypes = [vp, ctypes.c_int, ctypes.c_uint64, ctypes.c_uint64, f32p]
        _lib = L
    return _lib


def scalars_from_hparams(lr, betas, eps, weight_decay, step, inv_loss_scale=1.0, apply_clip=False) -> Scalars:
    """adamw.py:173-177,186-188: Python doubles, each cast to float32 where an
    ATen call consumes it.  ``step`` is the post-increment value."""
    beta1, beta2 = betas
    bias_correction = 1 - beta1 ** step
    bias_correction_sqrt = (1 - beta2 ** step) ** (1 / 2)
    step_size = lr / bias_correction
    bcs32 = np.float32(bias_correction_sqrt)
    return Scalars(
        beta1=np.float32(beta1),
        one_m_beta1=np.float32(1 - beta1),
        beta2=np.float32(beta2),
        one_m_beta2=np.float32(1 - beta2),
        bcs=bcs32,
        # torch's GPU `tensor / python_float` multiplies by the reciprocal taken in double and
        # then rounded to float32 (pinned by tests/golden/torch_gpu_step.npz, case step1)
        inv_bcs=np.float32(1.0 / bias_correction_sqrt),
        eps=np.float32(eps),
        decay=np.float32(1 - step_size * weight_decay),
        neg_step_size=np.float32(-step_size),
        inv_loss_scale=np.float32(inv_loss_scale),
        apply_decay=int(weight_decay != 0),
        apply_clip=int(bool(apply_clip)),
    )


_NP_DT = {DT_BF16: np.uint16, DT_F16: np.uint16, DT_F32: np.float32, DT_F64: np.float64}


def _ptr(a, ctype):
    return None if a is None else a.ctypes.data_as(ctypes.POINTER(ctype))


def _check(a, dt, name):
    if a.dtype != _NP_DT[dt] or not a.flags.c_contiguous:
        raise TypeError(f"{name}: need contiguous {_NP_DT[dt].__name__} for dtype code {dt}, got {a.dtype}")


def step_tensor(p, g, m, v, scalars: Scalars, *, p_dtype=DT_BF16, g_dtype=DT_BF16, m_dtype=DT_BF16,
                v_dtype=DT_BF16, clip_coef=1.0, noise=None, seed=0, step=0, tensor_id=0, elem_offset=0,
                flavour=REFERENCE_FLAVOUR, debug=False):
    """In-place step on numpy arrays.  ``noise`` = (np, nm, nv) uint16 arrays selects
    the explicit mode; otherwise Philox(seed, step, tensor_id).  Returns the fp32
    pre-rounding (p, m, v) when ``debug``."""
    n = p.size
    _check(p, p_dtype, "p"); _check(g, g_dtype, "g"); _check(m, m_dtype, "m"); _check(v, v_dtype, "v")
    assert g.size == n and m.size == n and v.size == n
    dbg = [np.empty(n, np.float32) if debug else None for _ in range(3)]
    if noise is not None:
        mode = NOISE_EXPLICIT
        nz = [None if a is None else np.ascontiguousarray(a).view(np.uint16) for a in noise]
    else:
        mode = NOISE_PHILOX
        nz = [None, None, None]
    rc = lib().orc_step_tensor(
        p.ctypes.data, p_dtype, g.ctypes.data, g_dtype, m.ctypes.data, m_dtype, v.ctypes.data, v_dtype, n,
        ctypes.byref(scalars), np.float32(clip_coef), mode,
        _ptr(nz[0], ctypes.c_uint16), _ptr(nz[1], ctypes.c_uint16), _ptr(nz[2], ctypes.c_uint16),
        seed, step & 0xFFFFFFFF, tensor_id, elem_offset, flavour,
        _ptr(dbg[0], ctypes.c_float), _ptr(dbg[1], ctypes.c_float), _ptr(dbg[2], ctypes.c_float))
    if rc != 0:
        raise ValueError(f"orc_step_tensor rejected its arguments (code {rc})")
    return tuple(dbg) if debug else None


def update_elem(p, g, m, v, scalars: Scalars, clip_coef=1.0, flavour=REFERENCE_FLAVOUR):
    out = [ctypes.c_float() for _ in range(3)]
    lib().orc_update_elem(p, g, m, v, ctypes.byref(scalars), np.float32(clip_coef), flavour,
                          *[ctypes.byref(o) for o in out])
    return tuple(np.float32(o.value) for o in out)


def philox4x32_10(ctr, key):
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    lib().orc_philox4x32_10(c, k, o)
    return tuple(o)


def philox_noise(seed, step, tensor_id, which, elem) -> int:
    return lib().orc_philox_noise(seed, step & 0xFFFFFFFF, tensor_id, which, elem)


def philox_noise_array(seed, step, tensor_id, which, start, count) -> np.ndarray:
    """uint16 noise for elements [start, start+count) (start a multiple of 8)."""
    assert start % 8 == 0
    out = np.empty(((count + 7) // 8) * 8, np.uint16)
    words = out.view(np.uint32).reshape(-1, 4)
    for b in range(words.shape[0]):
        blk = start // 8 + b
        words[b] = philox4x32_10((blk & 0xFFFFFFFF, blk >> 32, tensor_id * 4 + which, step & 0xFFFFFFFF),
                                 (seed & 0xFFFFFFFF, seed >> 32))
    return out[:count]


def sr_bf16(x, noise) -> int:
    return lib().orc_sr_bf16(np.float32(x), noise)


def sr_copy(source: np.ndarray, noise=None, seed=0) -> np.ndarray:
    """copy_stochastic_ (adamw.py:6-30): float32 array -> uint16 bf16 bits."""
    src = np.ascontiguousarray(source, np.float32).ravel()
    tgt = np.empty(src.size, np.uint16)
    nz = None if noise is None else np.ascontiguousarray(noise).view(np.uint16).ravel()
    lib().orc_sr_copy(_ptr(tgt, ctypes.c_uint16), _ptr(src, ctypes.c_float), src.size,
                      NOISE_PHILOX if nz is None else NOISE_EXPLICIT, _ptr(nz, ctypes.c_uint16), seed)
    return tgt.reshape(source.shape)


def grad_sumsq(g: np.ndarray, g_dtype=DT_BF16, inv_loss_scale=1.0) -> float:
    _check(g, g_dtype, "g")
    return lib().orc_grad_sumsq(g.ctypes.data, g_dtype, g.size, np.float32(inv_loss_scale))


def clip_coef(total_norm: float, max_norm: float) -> np.float32:
    """torch.nn.utils.clip_grad_norm_: min(1, max_norm / (total + 1e-6)), in float32."""
    c = np.float32(max_norm) / (np.float32(total_norm) + np.float32(1e-6))
    return np.float32(min(np.float32(1.0), c))


def row_means(g: np.ndarray, rows: int, row_len: int, g_dtype=DT_BF16) -> np.ndarray:
    _check(g, g_dtype, "g")
    out = np.empty(rows, np.float32)
    lib().orc_row_means(g.ctypes.data, g_dtype, rows, row_len, _ptr(out, ctypes.c_float))
    return out


# ---- small numpy helpers shared by the tests --------------------------------------
def f32_to_bf16_rne(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bf16 bits (how the synthetic inputs are stored)."""
    b = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def f32_to_f16_rne(x: np.ndarray) -> np.ndarray:
    """The oracle's float32 -> binary16 conversion (bits), for fp16 params / states."""
    x = np.ascontiguousarray(x, np.float32).ravel()
    out = np.empty(x.size, np.uint16)
    lib().orc_f32_to_f16_array(_ptr(x, ctypes.c_float), _ptr(out, ctypes.c_uint16), x.size)
    return out


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    return (h.astype(np.uint32) << 16).view(np.float32)


def synth_inputs(n: int, seed: int = 1234):
    """The synthetic value distributions of the benchmark configurations:
    param ~ N(0, 0.02), grad ~ N(0, 1e-3), ema ~ N(0, 1e-4), ema_squared = N(0, 1e-3)^2,
    drawn in float32 and stored as bf16 bits."""
    rng = np.random.default_rng(seed)
    p = f32_to_bf16_rne(rng.normal(0, 0.02, n).astype(np.float32))
    g = f32_to_bf16_rne(rng.normal(0, 1e-3, n).astype(np.float32))
    m = f32_to_bf16_rne(rng.normal(0, 1e-4, n).astype(np.float32))
    v = f32_to_bf16_rne((rng.normal(0, 1e-3, n).astype(np.float32)) ** 2)
    return p, g, m, v


def synth_noise(n: int, seed: int = 1234):
    rng = np.random.default_rng(seed + 7)
    return tuple(rng.integers(0, 65536, n, dtype=np.uint16) for _ in range(3))
