"""Parity of the HIP path (through the C ABI) with the CPU oracle and with
torch's own GPU kernels.  Needs an MI355X: run with ``-m gpu``.

Bar: bit-exact for every bf16 result and for the fp32 values before rounding.
"""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ops
from ramtorch_amd import _native as N
from ramtorch_amd import functional as F

pytestmark = pytest.mark.gpu

HP0 = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)
_NP2T = {np.dtype(np.uint16): torch.int16, np.dtype(np.float32): torch.float32}


@pytest.fixture(scope="module")
def handle():
    assert torch.cuda.is_available(), "these tests need the GPU"
    h = N.Handle(0)
    yield h
    torch.cuda.synchronize()
    h.close()


def dev16(a, dt=torch.bfloat16):
    """uint16 bit patterns -> GPU tensor of a 16-bit dtype."""
    return torch.from_numpy(a.view(np.int16).copy()).view(dt).cuda()


def nmis(a, b):
    """Number of elements whose bits differ (keeps assertion messages short)."""
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    assert a.shape == b.shape and a.dtype == b.dtype, (a.shape, b.shape, a.dtype, b.dtype)
    it = {2: torch.int16, 4: torch.int32}[a.element_size()]
    return int((a.view(it) != b.view(it)).sum())


def bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).ravel()


def bits32(t):
    return t.detach().cpu().contiguous().numpy().view(np.uint32)


def run_both(handle, p, g, m, v, *, hp=HP0, step=10, noise=None, seed=1234, tensor_id=0, debug=True,
             g_dtype=oracle.DT_BF16, p_dtype=oracle.DT_BF16, m_dtype=oracle.DT_BF16, v_dtype=oracle.DT_BF16,
             inv_loss_scale=1.0, clip_coef=None, pad=0):
    """One tensor through the HIP library and through the oracle; returns both result sets.
    pad: the arrays are the first elements of allocations that many elements longer, and what lies
    behind them has to be the same afterwards."""
    tdt = {oracle.DT_BF16: torch.bfloat16, oracle.DT_F16: torch.float16}
    padded = []

    def up(a, code):
        t = torch.from_numpy(a.copy()).cuda() if code in (oracle.DT_F32, oracle.DT_F64) else dev16(a, tdt[code])
        if pad:
            whole = torch.empty(a.size + pad, dtype=t.dtype, device="cuda")
            whole.view(torch.uint8).fill_(0xA5)
            whole[:a.size] = t
            padded.append(whole)
            t = whole[:a.size]
        return t

    P, G, M, V = up(p, p_dtype), up(g, g_dtype), up(m, m_dtype), up(v, v_dtype)
    n = p.size
    NZ = None if noise is None else tuple(torch.from_numpy(z.view(np.int16).copy()).cuda() for z in noise)
    dbg = tuple(torch.full((n,), float("nan"), device="cuda") for _ in range(3)) if debug else None
    e = F.Entry(p=P, g=G, m=M, v=V, step=step, scalars_idx=0, tensor_id=tensor_id, noise=NZ, dbg=dbg)
    sc = F.make_scalars(step=step, inv_loss_scale=inv_loss_scale, **hp)
    coef_t = None if clip_coef is None else torch.tensor([clip_coef], dtype=torch.float32, device="cuda")
    F.step_resident(handle, [e], [sc], seed=seed, explicit_noise=noise is not None, clip_coef=coef_t)
    torch.cuda.synchronize()
    for whole in padded:
        assert bool((whole[n:].view(torch.uint8) == 0xA5).all()), "bytes behind the tensor were written"

    po, mo, vo = p.copy(), m.copy(), v.copy()
    sco = oracle.scalars_from_hparams(step=step, inv_loss_scale=inv_loss_scale, apply_clip=clip_coef is not None, **hp)
    d = oracle.step_tensor(po, g, mo, vo, sco, p_dtype=p_dtype, g_dtype=g_dtype, m_dtype=m_dtype, v_dtype=v_dtype,
                           clip_coef=1.0 if clip_coef is None else clip_coef, noise=noise, seed=seed, step=step,
                           tensor_id=tensor_id, debug=True)
    def tbits(t):
        if t.dtype == torch.float64:
            return t.detach().cpu().contiguous().numpy().view(np.uint64)
        return bits32(t) if t.dtype == torch.float32 else bits16(t)
    nbits = {np.dtype(np.float32): np.uint32, np.dtype(np.float64): np.uint64, np.dtype(np.uint16): np.uint16}
    got = [tbits(t) for t in (P, M, V)]
    want = [a.view(nbits[a.dtype]) for a in (po, mo, vo)]
    return got, want, (None if dbg is None else [bits32(t) for t in dbg]), [x.view(np.uint32) for x in d]


def assert_same(got, want, dbg, pre, what=""):
    for name, a, b in zip("pmv", got, want):
        np.testing.assert_array_equal(a, b, err_msg=f"{what} {name} (stored)")
    if dbg is not None:
        for name, a, b in zip("pmv", dbg, pre):
            np.testing.assert_array_equal(a, b, err_msg=f"{what} {name} (fp32 before rounding)")


# ---- the flavour pin: torch's GPU kernels are the reference's arithmetic -----------------
def test_reference_flavour_is_what_torch_gpu_kernels_compute():
    n = 1 << 20
    p, g, m, v = oracle.synth_inputs(n, 1234)
    noise = oracle.synth_noise(n, 1234)
    P, G, M, V = dev16(p), dev16(g), dev16(m), dev16(v)
    NZ = [torch.from_numpy(z.view(np.int16).copy()).cuda() for z in noise]
    p32, m32, v32 = torch_ops.reference_step_ops(P, G, M, V, step=10, noise=NZ, **HP0)
    torch.cuda.synchronize()
    sc = oracle.scalars_from_hparams(step=10, **HP0)
    po, mo, vo = p.copy(), m.copy(), v.copy()
    d = oracle.step_tensor(po, g, mo, vo, sc, noise=noise, flavour=oracle.REFERENCE_FLAVOUR, debug=True)
    for name, t, a in zip("pmv", (p32, m32, v32), d):
        np.testing.assert_array_equal(bits32(t), a.view(np.uint32), err_msg=f"fp32 {name}")
    for name, t, a in zip("pmv", (P, M, V), (po, mo, vo)):
        np.testing.assert_array_equal(bits16(t), a, err_msg=f"bf16 {name}")
    # and the CPU flavour is measurably different, so the pin is sharp
    d2 = oracle.step_tensor(p.copy(), g, m.copy(), v.copy(), sc, noise=noise, flavour=oracle.TORCH_CPU_FLAVOUR,
                            debug=True)
    assert (d2[0].view(np.uint32) != bits32(p32)).sum() > 0


# ---- config 0: one 4096 x 4096 weight, explicit noise, bit-exact ----------------------------
def test_config0_bit_exact_against_oracle_and_torch_gpu_ops(handle):
    n = 4096 * 4096
    p, g, m, v = oracle.synth_inputs(n, 1234)
    noise = oracle.synth_noise(n, 1234)
    got, want, dbg, pre = run_both(handle, p, g, m, v, noise=noise, step=10)
    assert_same(got, want, dbg, pre, "config0")
    # fast path (no debug outputs) gives the same stored bits
    got2, _, _, _ = run_both(handle, p, g, m, v, noise=noise, step=10, debug=False)
    assert_same(got2, want, None, None, "config0 fast path")
    # the reference's own op sequence on the GPU
    P, G, M, V = (dev16(a).view(4096, 4096) for a in (p, g, m, v))
    NZ = [torch.from_numpy(z.view(np.int16).copy()).cuda().view(4096, 4096) for z in noise]
    p32, m32, v32 = torch_ops.reference_step_ops(P, G, M, V, step=10, noise=NZ, **HP0)
    for name, t, a in zip("pmv", (P, M, V), got2):
        np.testing.assert_array_equal(bits16(t).ravel(), a, err_msg=f"torch GPU ops vs HIP {name}")
    for name, t, a in zip("pmv", (p32, m32, v32), dbg):
        np.testing.assert_array_equal(bits32(t).ravel(), a, err_msg=f"torch GPU ops vs HIP fp32 {name}")


# ---- sizes: empty, tiny, ragged, chunk boundaries -------------------------------------------
@pytest.mark.parametrize("n", [1, 7, 8, 9, 2047, 2048, 8191, 8192, 8193, 3 * 8192 + 5, 100_003])
@pytest.mark.parametrize("mode", ["explicit", "philox"])
def test_sizes_and_tails(handle, n, mode):
    p, g, m, v = oracle.synth_inputs(n, n)
    noise = oracle.synth_noise(n, n) if mode == "explicit" else None
    for debug in (True, False):
        got, want, dbg, pre = run_both(handle, p, g, m, v, noise=noise, step=3, tensor_id=5, debug=debug)
        assert_same(got, want, dbg, pre, f"n={n} {mode}")


def test_empty_inputs(handle):
    F.step_resident(handle, [], [], seed=0, explicit_noise=False)
    z = torch.zeros(0, dtype=torch.bfloat16, device="cuda")
    e = F.Entry(p=z, g=z.clone(), m=z.clone(), v=z.clone(), step=1, scalars_idx=0, tensor_id=0)
    F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False)
    torch.cuda.synchronize()


def test_unaligned_views(handle):
    # a view that starts 2 bytes into an allocation: no 128-bit access is legal
    n = 5000
    p, g, m, v = oracle.synth_inputs(n, 21)
    base = [torch.zeros(n + 8, dtype=torch.bfloat16, device="cuda") for _ in range(4)]
    views = []
    for b, a, off in zip(base, (p, g, m, v), (1, 3, 0, 5)):
        b[off:off + n] = dev16(a)
        views.append(b[off:off + n])
    e = F.Entry(p=views[0], g=views[1], m=views[2], v=views[3], step=10, scalars_idx=0, tensor_id=1)
    F.step_resident(handle, [e], [F.make_scalars(step=10, **HP0)], seed=7, explicit_noise=False)
    torch.cuda.synchronize()
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.step_tensor(po, g, mo, vo, oracle.scalars_from_hparams(step=10, **HP0), seed=7, step=10, tensor_id=1)
    for name, t, a in zip("pmv", (views[0], views[2], views[3]), (po, mo, vo)):
        np.testing.assert_array_equal(bits16(t), a, err_msg=name)
    # nothing outside the views was written
    assert float(base[0][0]) == 0 and not base[0][n + 1:].any() and not base[3][:5].any()


# ---- value edge cases -------------------------------------------------------------------------
def test_edge_values(handle):
    import itertools
    vals = [0x0000, 0x8000, 0x0001, 0x8001, 0x007F, 0x0080, 0x0100, 0x3F80, 0xBF80, 0x7F7F, 0xFF7F, 0x4000, 0x3F00,
            0x1234, 0x9234, 0x2B00, 0x6000, 0x0F00, 0x3DCC, 0x3A83, 0x7F80, 0xFF80]
    combos = list(itertools.product(range(len(vals)), repeat=2))
    p = np.array([vals[a] for a, b in combos], np.uint16)
    g = np.array([vals[b] for a, b in combos], np.uint16)
    m = np.array([vals[(a + b) % len(vals)] for a, b in combos], np.uint16)
    v = np.array([vals[(a * 7 + b) % len(vals)] & 0x7FFF for a, b in combos], np.uint16)
    noise = oracle.synth_noise(p.size, 99)
    got, want, dbg, pre = run_both(handle, p, g, m, v, noise=noise)
    # NaN payloads are not part of the contract; everything else is bit-exact
    for name, a, b, d_, q in zip("pmv", got, want, dbg, pre):
        ok = ~np.isnan(q.view(np.float32))
        np.testing.assert_array_equal(d_[ok], q[ok], err_msg=f"fp32 {name}")
        np.testing.assert_array_equal(a[ok], b[ok], err_msg=f"bf16 {name}")
        assert np.isnan(d_.view(np.float32)[~ok]).all()


# ---- hyper-parameters and steps -------------------------------------------------------------------
@pytest.mark.parametrize("hp,step", [
    (dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), 1),
    (dict(lr=3e-4, betas=(0.95, 0.99), eps=1e-6, weight_decay=0.0), 100),
    (dict(lr=2.5e-3, betas=(0.8, 0.9999), eps=1e-10, weight_decay=0.1), 5000),
    (dict(lr=1e-4, betas=(0.0, 0.5), eps=1e-8, weight_decay=1.0), 2),
])
def test_hyperparameters(handle, hp, step):
    n = 50_000
    p, g, m, v = oracle.synth_inputs(n, step)
    got, want, dbg, pre = run_both(handle, p, g, m, v, hp=hp, step=step, noise=oracle.synth_noise(n, step))
    assert_same(got, want, dbg, pre, f"{hp} step {step}")


# ---- dtype combinations (fp32 params / states are stored without rounding) ------------------------
@pytest.mark.parametrize("p_dt,g_dt,m_dt,v_dt", [
    (oracle.DT_BF16, oracle.DT_F32, oracle.DT_BF16, oracle.DT_F32),   # config 4 layout
    (oracle.DT_F32, oracle.DT_F32, oracle.DT_F32, oracle.DT_F32),
    (oracle.DT_BF16, oracle.DT_F16, oracle.DT_BF16, oracle.DT_BF16),
    (oracle.DT_F32, oracle.DT_BF16, oracle.DT_BF16, oracle.DT_BF16),
    (oracle.DT_BF16, oracle.DT_BF16, oracle.DT_F32, oracle.DT_BF16),
    # fp16 / fp64 params and states: upcast like everything else, plain copy_ on the way back
    # (adamw.py:208,214,221-222).  fp16 params, and states that are both fp16, have templated kernels ...
    (oracle.DT_F16, oracle.DT_F16, oracle.DT_F16, oracle.DT_F16),
    (oracle.DT_BF16, oracle.DT_BF16, oracle.DT_F16, oracle.DT_F16),
    (oracle.DT_F16, oracle.DT_F16, oracle.DT_F32, oracle.DT_F32),
    (oracle.DT_F16, oracle.DT_F32, oracle.DT_BF16, oracle.DT_BF16),
    (oracle.DT_F32, oracle.DT_F16, oracle.DT_F16, oracle.DT_F16),
    # ... fp64 anywhere, or one fp16 state next to another dtype, take the runtime-typed kernel
    (oracle.DT_BF16, oracle.DT_BF16, oracle.DT_F16, oracle.DT_F32),
    (oracle.DT_F64, oracle.DT_F32, oracle.DT_BF16, oracle.DT_F64),
    (oracle.DT_F16, oracle.DT_BF16, oracle.DT_F64, oracle.DT_F32),
])
@pytest.mark.parametrize("mode", ["explicit", "philox"])
def test_dtype_combinations(handle, p_dt, g_dt, m_dt, v_dt, mode):
    n = 20_000 + 3
    p, g, m, v = oracle.synth_inputs(n, 31)

    def conv(a, dt):
        if dt == oracle.DT_F32:
            return (oracle.bf16_to_f32(a) * np.float32(1.0009765625)).astype(np.float32)  # not bf16-exact
        if dt == oracle.DT_F16:
            return oracle.bf16_to_f32(a).astype(np.float16).view(np.uint16)
        if dt == oracle.DT_F64:  # not representable in fp32: the upcast to fp32 has to round
            return oracle.bf16_to_f32(a).astype(np.float64) * (1.0 + 2.0 ** -30)
        return a
    p, g, m, v = conv(p, p_dt), conv(g, g_dt), conv(m, m_dt), conv(v, v_dt)
    noise = oracle.synth_noise(n, 31) if mode == "explicit" else None
    for debug in (True, False):
        got, want, dbg, pre = run_both(handle, p, g, m, v, noise=noise, p_dtype=p_dt, g_dtype=g_dt, m_dtype=m_dt,
                                       v_dtype=v_dt, debug=debug)
        assert_same(got, want, dbg, pre, f"dtypes {p_dt}{g_dt}{m_dt}{v_dt} {mode}")


@pytest.mark.parametrize("n", [8, 504, 511, 512, 513, 520, 1024, 2047, 2048, 2056, 8192, 8192 + 512, 8192 + 519, 3 * 8192 - 1])
def test_runtime_typed_kernel_around_a_wavefronts_run(handle, n):
    """The runtime-typed kernel moves fp32 and fp64 arrays a whole wavefront (512 elements) at a time where
    all 512 exist and lane by lane behind that: sizes on both sides of those edges, the three wide
    layouts, both noise modes, and the memory behind the arrays has to stay as it was."""
    for p_dt, g_dt, m_dt, v_dt in [(oracle.DT_BF16, oracle.DT_BF16, oracle.DT_F64, oracle.DT_F64),
                                   (oracle.DT_F64, oracle.DT_F32, oracle.DT_F32, oracle.DT_F64),
                                   (oracle.DT_F16, oracle.DT_BF16, oracle.DT_F64, oracle.DT_F32)]:
        p, g, m, v = oracle.synth_inputs(n, 100 + n)

        def conv(a, dt):
            f = oracle.bf16_to_f32(a)
            if dt == oracle.DT_F32:
                return (f * np.float32(1.0009765625)).astype(np.float32)
            if dt == oracle.DT_F16:
                return f.astype(np.float16).view(np.uint16)
            if dt == oracle.DT_F64:
                return f.astype(np.float64) * (1.0 + 2.0 ** -30)
            return a
        for mode in ("philox", "explicit"):
            noise = oracle.synth_noise(n, 7) if mode == "explicit" else None
            got, want, dbg, pre = run_both(handle, conv(p, p_dt), conv(g, g_dt), conv(m, m_dt), conv(v, v_dt), noise=noise,
                                           p_dtype=p_dt, g_dtype=g_dt, m_dtype=m_dt, v_dtype=v_dt, debug=False, step=3,
                                           pad=1024)
            assert_same(got, want, dbg, pre, f"n={n} dtypes {p_dt}{g_dt}{m_dt}{v_dt} {mode}")


def test_fp16_param_overflow_and_gradual_underflow(handle):
    """An fp16 param written back past the fp16 range becomes inf, tiny values land on
    fp16 subnormals (round to nearest even), as Tensor.copy_ does."""
    n = 4096 + 5
    p, g, m, v = oracle.synth_inputs(n, 77)
    p16 = oracle.bf16_to_f32(p).astype(np.float16)
    p16[:8] = [65504.0, -65504.0, 6e-8, -6e-8, 6.1e-5, 1.2e-7, 0.0, -0.0]
    g16 = oracle.bf16_to_f32(g).astype(np.float16)
    g16[:2] = [-60000.0, 60000.0]  # pushes the two largest values over the edge
    g16[8:12] = [6e-8, 1e-6, -3e-7, 2e-5]  # ema = 0.1 * g: fp16 subnormals and zero
    hp = dict(lr=100.0, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    m0 = np.zeros(n, np.uint16)
    got, want, dbg, pre = run_both(handle, p16.view(np.uint16), g16.view(np.uint16), m0, m0.copy(), hp=hp, step=1,
                                   p_dtype=oracle.DT_F16, g_dtype=oracle.DT_F16, m_dtype=oracle.DT_F16,
                                   v_dtype=oracle.DT_F16)
    assert_same(got, want, dbg, pre, "fp16 edges")
    out = got[0].view(np.float16)
    assert np.isinf(out[0]) and out[0] > 0 and np.isinf(out[1]) and out[1] < 0
    assert np.isinf(got[2].view(np.float16)[0])  # g*g overflows fp16 in ema_squared as well
    ema = got[1].view(np.float16)[8:12]
    # below half the smallest subnormal -> 0; a subnormal; exactly -2^-25, a tie -> -0 (even)
    assert ema[0] == 0 and 0 < ema[1] < 6.1e-5 and got[1][10] == 0x8000


def test_loss_scale_and_clip_coefficient(handle):
    n = 30_000
    p, g, m, v = oracle.synth_inputs(n, 41)
    g32 = (oracle.bf16_to_f32(g) * np.float32(1024)).astype(np.float32)
    v32 = oracle.bf16_to_f32(v).copy()
    got, want, dbg, pre = run_both(handle, p, g32, m, v32, g_dtype=oracle.DT_F32, v_dtype=oracle.DT_F32,
                                   inv_loss_scale=1.0 / 1024, clip_coef=0.37, step=100)
    assert_same(got, want, dbg, pre, "loss scale + clip")


# ---- many tensors in one launch ---------------------------------------------------------------------
def test_multi_tensor_launch_with_groups_and_steps(handle):
    rng = np.random.default_rng(5)
    lens = [int(x) for x in np.exp(rng.uniform(0, np.log(4096), 300)).astype(np.int64).clip(1, 4096)]
    lens += [0, 8192, 8192 * 2 + 1, 1, 65_537]
    hps = [HP0, dict(lr=3e-4, betas=(0.95, 0.99), eps=1e-6, weight_decay=0.0)]
    scal, sco, entries, inputs = [], [], [], []
    for gi, hp in enumerate(hps):
        for st in (4, 9):
            scal.append(F.make_scalars(step=st, **hp))
            sco.append((oracle.scalars_from_hparams(step=st, **hp), st))
    for i, n in enumerate(lens):
        p, g, m, v = oracle.synth_inputs(n, 1000 + i)
        si = i % len(scal)
        P, G, M, V = dev16(p), dev16(g), dev16(m), dev16(v)
        entries.append(F.Entry(p=P, g=G, m=M, v=V, step=sco[si][1], scalars_idx=si, tensor_id=i))
        inputs.append((p, g, m, v, si))
    F.step_resident(handle, entries, scal, seed=99, explicit_noise=False)
    torch.cuda.synchronize()
    for i, (e, (p, g, m, v, si)) in enumerate(zip(entries, inputs)):
        po, mo, vo = p.copy(), m.copy(), v.copy()
        oracle.step_tensor(po, g, mo, vo, sco[si][0], seed=99, step=sco[si][1], tensor_id=i)
        for name, t, a in zip("pmv", (e.p, e.m, e.v), (po, mo, vo)):
            np.testing.assert_array_equal(bits16(t), a, err_msg=f"tensor {i} (n={lens[i]}) {name}")


def test_mixed_dtype_tensors_in_one_call(handle):
    n = 10_000
    p, g, m, v = oracle.synth_inputs(n, 61)
    sc, sco = F.make_scalars(step=2, **HP0), oracle.scalars_from_hparams(step=2, **HP0)
    e0 = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=2, scalars_idx=0, tensor_id=0)
    p32 = oracle.bf16_to_f32(p).copy()
    e1 = F.Entry(p=torch.from_numpy(p32.copy()).cuda(), g=dev16(g), m=dev16(m), v=dev16(v), step=2, scalars_idx=0,
                 tensor_id=1)
    F.step_resident(handle, [e0, e1], [sc], seed=3, explicit_noise=False)
    torch.cuda.synchronize()
    a = [p.copy(), m.copy(), v.copy()]
    oracle.step_tensor(a[0], g, a[1], a[2], sco, seed=3, step=2, tensor_id=0)
    b = [p32.copy(), m.copy(), v.copy()]
    oracle.step_tensor(b[0], g, b[1], b[2], sco, p_dtype=oracle.DT_F32, seed=3, step=2, tensor_id=1)
    np.testing.assert_array_equal(bits16(e0.p), a[0])
    np.testing.assert_array_equal(bits32(e1.p), b[0].view(np.uint32))
    np.testing.assert_array_equal(bits16(e1.m), b[1])


# ---- pieces of a tensor draw the same noise as the whole -----------------------------------------
def test_elem_offset_pieces_equal_whole(handle):
    n = 40_000
    p, g, m, v = oracle.synth_inputs(n, 71)
    sc = F.make_scalars(step=6, **HP0)
    whole = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=6, scalars_idx=0, tensor_id=9)
    F.step_resident(handle, [whole], [sc], seed=5, explicit_noise=False)
    P, G, M, V = dev16(p), dev16(g), dev16(m), dev16(v)
    cuts = [0, 8, 8200, 24_000, n]
    pieces = [F.Entry(p=P[a:b], g=G[a:b], m=M[a:b], v=V[a:b], step=6, scalars_idx=0, tensor_id=9, elem_offset=a)
              for a, b in zip(cuts[:-1], cuts[1:])]
    F.step_resident(handle, pieces, [sc], seed=5, explicit_noise=False)
    torch.cuda.synchronize()
    assert nmis(whole.p, P) == 0 and nmis(whole.m, M) == 0 and nmis(whole.v, V) == 0


# ---- skip flag ----------------------------------------------------------------------------------------
def test_skip_flag_leaves_everything_untouched(handle):
    n = 9000
    p, g, m, v = oracle.synth_inputs(n, 81)
    e = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=1, scalars_idx=0, tensor_id=0)
    skip = torch.ones(1, dtype=torch.int32, device="cuda")
    F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False, skip=skip)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(bits16(e.p), p)
    np.testing.assert_array_equal(bits16(e.m), m)
    skip.zero_()
    F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False, skip=skip)
    torch.cuda.synchronize()
    assert (bits16(e.m) != m).any()


# ---- argument errors come back as error codes, not crashes ------------------------------------------------
def test_bad_arguments_are_rejected(handle):
    z = torch.zeros(16, dtype=torch.bfloat16, device="cuda")
    e = F.Entry(p=z, g=z.clone(), m=z.clone(), v=z.clone(), step=1, scalars_idx=3, tensor_id=0)
    with pytest.raises(N.NativeError, match="scalars_idx"):
        F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False)
    e.scalars_idx = 0
    with pytest.raises(N.NativeError, match="explicit noise"):
        F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=True)
    e.elem_offset = 4
    with pytest.raises(N.NativeError, match="elem_offset"):
        F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False)
    e.elem_offset = 0
    e.tensor_id = 1 << 30
    with pytest.raises(N.NativeError, match="tensor_id"):
        F.step_resident(handle, [e], [F.make_scalars(step=1, **HP0)], seed=0, explicit_noise=False)
    # centralization without row means: only for tensors the row-wise kernel takes (rows a multiple of 8, 512 .. 32768)
    e.tensor_id = 0
    cen = [F.make_scalars(step=1, centralization=0.5, **HP0)]
    with pytest.raises(N.NativeError, match="row_len"):
        F.step_resident(handle, [e], cen, seed=0, explicit_noise=False)
    e.row_len = 16
    with pytest.raises(N.NativeError, match="without row_mean"):
        F.step_resident(handle, [e], cen, seed=0, explicit_noise=False)
    big = torch.zeros(1024, dtype=torch.bfloat16, device="cuda")
    e2 = F.Entry(p=big, g=big.clone(), m=big.clone(), v=big.clone(), step=1, scalars_idx=0, tensor_id=0, row_len=520)
    with pytest.raises(N.NativeError, match="without row_mean"):     # 1024 is not a multiple of 520
        F.step_resident(handle, [e2], cen, seed=0, explicit_noise=False)
    e2.row_len = 512
    F.step_resident(handle, [e2], cen, seed=0, explicit_noise=False)   # two rows of 512: taken
    torch.cuda.synchronize()


def test_kernel_timing_history(handle):
    """rt_set_timing / rt_last_kernel_ms / rt_kernel_ms_history: one event pair per launch, read back
    after the fact, oldest first; switching timing on again forgets earlier launches."""
    n = 1 << 20
    p, g, m, v = oracle.synth_inputs(n, 5)
    e = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=1, scalars_idx=0, tensor_id=0)
    sc = [F.make_scalars(step=1, **HP0)]
    with pytest.raises(N.NativeError, match="no timed launch"):
        handle.set_timing(True)
        handle.last_kernel_ms()
    for _ in range(5):
        F.step_resident(handle, [e], sc, seed=1, explicit_noise=False)
    hist = handle.kernel_ms_history()
    assert len(hist) == 5 and all(0.0 < t < 50.0 for t in hist), hist
    assert handle.kernel_ms_history(2) == hist[-2:]
    assert handle.last_kernel_ms() == hist[-1]
    handle.set_timing(True)
    assert handle.kernel_ms_history() == []
    F.step_resident(handle, [e], sc, seed=1, explicit_noise=False)
    assert len(handle.kernel_ms_history()) == 1
    handle.set_timing(False)
    F.step_resident(handle, [e], sc, seed=1, explicit_noise=False)   # not recorded
    assert len(handle.kernel_ms_history()) == 1
    torch.cuda.synchronize()


# ---- seeded random cases: sizes, dtypes, hyper-parameters, steps, noise modes, scaling -----------------
def test_random_cases_match_the_oracle(handle):
    rng = np.random.default_rng(20240)
    dts = [oracle.DT_BF16, oracle.DT_F32, oracle.DT_F16, oracle.DT_F64]

    def conv(a, dt, scale=1.0):
        f = oracle.bf16_to_f32(a) * np.float32(scale)
        if dt == oracle.DT_F32:
            return (f * np.float32(1.0009765625)).astype(np.float32)
        if dt == oracle.DT_F16:
            return f.astype(np.float16).view(np.uint16)
        if dt == oracle.DT_F64:
            return f.astype(np.float64) * (1.0 + 2.0 ** -30)
        return a

    for case in range(400):
        n = max(1, int(rng.choice([rng.integers(1, 64), rng.integers(1, 9000), rng.integers(8000, 70000),
                                   8192 * rng.integers(1, 6) + rng.integers(-9, 9)])))
        p_dt, m_dt, v_dt = (int(rng.choice(dts, p=[0.55, 0.25, 0.1, 0.1])) for _ in range(3))
        g_dt = int(rng.choice(dts[:3], p=[0.5, 0.35, 0.15]))
        hp = dict(lr=float(10 ** rng.uniform(-5, -1)),
                  betas=(float(rng.choice([0.0, 0.5, 0.9, 0.95])), float(rng.choice([0.9, 0.99, 0.999, 0.9999]))),
                  eps=float(rng.choice([1e-8, 1e-6, 1e-12])), weight_decay=float(rng.choice([0.0, 0.01, 0.1])))
        ls = float(rng.choice([1.0, 1.0, 1024.0, 65536.0]))
        if g_dt == oracle.DT_F16:
            ls = min(ls, 1024.0)
        p, g, m, v = oracle.synth_inputs(n, int(rng.integers(0, 1 << 30)))
        kw = dict(hp=hp, step=int(rng.choice([1, 2, 10, 1000, 123456])), seed=int(rng.integers(0, 1 << 62)),
                  tensor_id=int(rng.integers(0, 1 << 20)), p_dtype=p_dt, g_dtype=g_dt, m_dtype=m_dt, v_dtype=v_dt,
                  inv_loss_scale=1.0 / ls, clip_coef=None if rng.random() < 0.7 else float(rng.uniform(0.01, 1.0)),
                  noise=oracle.synth_noise(n, int(rng.integers(0, 1 << 30))) if rng.random() < 0.4 else None,
                  debug=bool(rng.random() < 0.5))
        got, want, dbg, pre = run_both(handle, conv(p, p_dt), conv(g, g_dt, ls), conv(m, m_dt), conv(v, v_dt), **kw)
        assert_same(got, want, dbg, pre, f"random case {case}: n={n} dtypes={(p_dt, g_dt, m_dt, v_dt)}")


def test_random_centralized_pieces_match_the_oracle(handle):
    """Centralization (adamw.py:179-184) through both kernels that carry it: random row lengths
    (shorter and longer than a lane's vector, a unit, a wave's run), pieces that start and end in the middle of
    rows, 16-bit layouts (whole units take the fast kernel's centralizing instance) and layouts with
    an fp32 array (generic kernel).  The means are arbitrary numbers: the kernels only consume them."""
    rng = np.random.default_rng(777)
    for case in range(60):
        row_len = int(rng.choice([rng.integers(1, 8), rng.integers(8, 40), rng.integers(100, 5000), 4096,
                                  8192 + rng.integers(-9, 9), rng.integers(20_000, 40_000)]))
        rows = int(max(1, min(rng.integers(1, 60), 300_000 // row_len)))
        total = rows * row_len
        start = int(rng.integers(0, max(1, total // 2))) // 8 * 8 if rng.random() < 0.7 else 0
        count = int(rng.integers(1, total - start + 1)) if rng.random() < 0.5 else total - start
        wide = rng.random() < 0.25
        p_dt = int(rng.choice([oracle.DT_BF16, oracle.DT_F16]))
        g_dt = int(rng.choice([oracle.DT_BF16, oracle.DT_F16])) if not wide else oracle.DT_F32
        mv_dt = int(rng.choice([oracle.DT_BF16, oracle.DT_F16]))
        cen = float(rng.choice([1.0, 0.5, 0.3]))
        p, g, m, v = oracle.synth_inputs(total, int(rng.integers(0, 1 << 30)))
        means = (rng.standard_normal(rows) * 1e-3).astype(np.float32)
        tdt = {oracle.DT_BF16: torch.bfloat16, oracle.DT_F16: torch.float16}

        def conv(a, dt):
            f = oracle.bf16_to_f32(a)
            if dt == oracle.DT_F32:
                return (f * np.float32(1.0009765625)).astype(np.float32)
            return f.astype(np.float16).view(np.uint16) if dt == oracle.DT_F16 else a

        def up(a, dt):
            return torch.from_numpy(a.copy()).cuda() if dt == oracle.DT_F32 else dev16(a, tdt[dt])

        hp = dict(HP0, lr=float(10 ** rng.uniform(-4, -2)))
        step, seed, tid = int(rng.choice([1, 7, 1000])), int(rng.integers(0, 1 << 62)), int(rng.integers(0, 1 << 20))
        arrs = [conv(p, p_dt), conv(g, g_dt), conv(m, mv_dt), conv(v, mv_dt)]
        P, G, M, V = (up(a, dt) for a, dt in zip(arrs, (p_dt, g_dt, mv_dt, mv_dt)))
        sl = slice(start, start + count)
        e = F.Entry(p=P[sl], g=G[sl], m=M[sl], v=V[sl], step=step, scalars_idx=0, tensor_id=tid,
                    row_mean=torch.from_numpy(means).cuda(), row_len=row_len, elem_offset=start)
        F.step_resident(handle, [e], [F.make_scalars(step=step, centralization=cen, **hp)], seed=seed, explicit_noise=False)
        torch.cuda.synchronize()

        g32 = arrs[1][sl].astype(np.float32) if g_dt == oracle.DT_F32 else (
            oracle.bf16_to_f32(arrs[1][sl]) if g_dt == oracle.DT_BF16 else arrs[1][sl].view(np.float16).astype(np.float32))
        row_of = (np.arange(start, start + count) // row_len)
        g32 = (g32 - (means[row_of] * np.float32(cen)).astype(np.float32)).astype(np.float32)
        po, mo, vo = arrs[0][sl].copy(), arrs[2][sl].copy(), arrs[3][sl].copy()
        oracle.step_tensor(po, g32, mo, vo, oracle.scalars_from_hparams(step=step, **hp), p_dtype=p_dt,
                           g_dtype=oracle.DT_F32, m_dtype=mv_dt, v_dtype=mv_dt, seed=seed, step=step, tensor_id=tid,
                           elem_offset=start)
        what = f"case {case}: rows={rows} row_len={row_len} start={start} count={count} dtypes={(p_dt, g_dt, mv_dt)}"
        for name, t, a in zip("pmv", (P, M, V), (po, mo, vo)):
            np.testing.assert_array_equal(bits16(t)[sl], a, err_msg=f"{what} {name}")
        # nothing outside the piece was touched
        for name, t, a in zip("pmv", (P, M, V), (arrs[0], arrs[2], arrs[3])):
            np.testing.assert_array_equal(bits16(t)[:start], a[:start], err_msg=f"{what} {name} before the piece")
            np.testing.assert_array_equal(bits16(t)[start + count:], a[start + count:], err_msg=f"{what} {name} behind it")
