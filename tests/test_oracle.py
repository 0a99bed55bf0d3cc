"""Pins for the CPU oracle (oracle/sr_adamw_oracle.c).  No GPU needed.

Each check is chosen so that a plausible mistake in the oracle (dropped term,
wrong sign, wrong association, wrong scalar cast) fails at least one of them:
known-answer vectors, vectors produced by torch's own GPU kernels on an
MI355X (tests/golden/torch_gpu_step.npz), torch's CPU kernels run here, the
Random123 Philox vectors, an independent pure-Python Philox, brute force over
all 65536 noises, and a float64 evaluation of the textbook formula.
"""
import itertools
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ops

HP0 = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)


def _hex16(s):
    return np.array([int(x, 16) for x in s.split()], dtype=np.uint16)


def _hex32(s):
    return np.array([int(x, 16) for x in s.split()], dtype=np.uint32)


@pytest.fixture(scope="module")
def kat(golden_dir):
    with open(os.path.join(golden_dir, "kat8.json")) as f:
        return json.load(f)


@pytest.fixture(scope="module")
def gpu_golden(golden_dir):
    return np.load(os.path.join(golden_dir, "torch_gpu_step.npz"))


# ---- scalars -------------------------------------------------------------------------
def test_scalar_bit_patterns(kat):
    hp = kat["hparams"]
    sc = oracle.scalars_from_hparams(hp["lr"], tuple(hp["betas"]), hp["eps"], hp["weight_decay"], hp["step"])
    for name, bits in kat["scalars_f32_bits"].items():
        got = np.float32(getattr(sc, name)).view(np.uint32)
        assert got == int(bits, 16), f"{name}: {got:08x} != {bits}"


def test_scalars_follow_python_double_order():
    # float32(1 - (lr/bc)*wd) must come from the double expression, not from float32 pieces
    sc = oracle.scalars_from_hparams(2.5e-3, (0.8, 0.9999), 1e-10, 0.1, 5000)
    bc = 1 - 0.8 ** 5000
    assert np.float32(sc.decay) == np.float32(1 - (2.5e-3 / bc) * 0.1)
    assert np.float32(sc.neg_step_size) == np.float32(-(2.5e-3 / bc))
    assert np.float32(sc.inv_bcs) == np.float32(1.0 / (1 - 0.9999 ** 5000) ** 0.5)


# ---- the 8-element known-answer vector ------------------------------------------------
@pytest.mark.parametrize("flavour", [oracle.REFERENCE_FLAVOUR, oracle.TORCH_CPU_FLAVOUR,
                                     oracle.REFERENCE_FLAVOUR & ~oracle.DIV_RECIP])
def test_kat8(kat, flavour):
    hp = kat["hparams"]
    sc = oracle.scalars_from_hparams(hp["lr"], tuple(hp["betas"]), hp["eps"], hp["weight_decay"], hp["step"])
    p, g, m, v = (_hex16(kat[k]) for k in "pgmv")
    noise = tuple(np.array(kat[k], np.uint16) for k in ("noise_p", "noise_m", "noise_v"))
    d = oracle.step_tensor(p, g, m, v, sc, noise=noise, flavour=flavour, debug=True)
    for got, key in zip(d, ("p32", "m32", "v32")):
        np.testing.assert_array_equal(got.view(np.uint32), _hex32(kat[key]), err_msg=key)
    for got, key in zip((p, m, v), ("p16", "m16", "v16")):
        np.testing.assert_array_equal(got, _hex16(kat[key]), err_msg=key)


# ---- vectors from torch's GPU kernels (the reference's real arithmetic) -----------------
def _golden_cases():
    import importlib.util
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "make_torch_gpu_golden.py")
    spec = importlib.util.spec_from_file_location("make_torch_gpu_golden", here)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    cases = []
    for name, n, seed, hp, step in mod.CASES:
        cases.append((name, oracle.synth_inputs(n, seed), oracle.synth_noise(n, seed), hp, step))
    e = mod.edge_inputs()
    cases.append(("edge", e, oracle.synth_noise(e[0].size, 99), HP0, 10))
    return cases


@pytest.mark.parametrize("case", _golden_cases(), ids=lambda c: c[0])
def test_reference_flavour_matches_torch_gpu_vectors(gpu_golden, case):
    name, (p, g, m, v), noise, hp, step = case
    sc = oracle.scalars_from_hparams(step=step, **hp)
    p, m, v = p.copy(), m.copy(), v.copy()
    d = oracle.step_tensor(p, g, m, v, sc, noise=noise, flavour=oracle.REFERENCE_FLAVOUR, debug=True)
    for got, key in zip(d, ("p32", "m32", "v32")):
        want = gpu_golden[f"{name}/{key}"]
        nan = np.isnan(want.view(np.float32))
        np.testing.assert_array_equal(got.view(np.uint32)[~nan], want[~nan], err_msg=f"{name}/{key}")
        assert np.isnan(got[nan]).all()
    for got, key, pre in zip((p, m, v), ("p16", "m16", "v16"), d):
        want = gpu_golden[f"{name}/{key}"]
        finite = np.isfinite(pre)
        np.testing.assert_array_equal(got[finite], want[finite], err_msg=f"{name}/{key}")


def test_other_flavours_do_not_match_torch_gpu_vectors(gpu_golden):
    # the vectors are sharp enough to tell the flavours apart (fp32 values; bf16 alone would not be)
    name, (p, g, m, v), noise, hp, step = _golden_cases()[3]
    sc = oracle.scalars_from_hparams(step=step, **hp)
    for fl in (oracle.TORCH_CPU_FLAVOUR, oracle.REFERENCE_FLAVOUR & ~oracle.DIV_RECIP,
               oracle.REFERENCE_FLAVOUR & ~oracle.FMA_ADDCDIV, oracle.REFERENCE_FLAVOUR & ~oracle.FMA_ADD):
        d = oracle.step_tensor(p.copy(), g, m.copy(), v.copy(), sc, noise=noise, flavour=fl, debug=True)
        diff = sum(int((d[i].view(np.uint32) != gpu_golden[f"{name}/{k}"]).sum())
                   for i, k in enumerate(("p32", "m32", "v32")))
        assert diff > 0, f"flavour {fl} unexpectedly reproduces the GPU vectors"


# ---- torch's CPU kernels, run here, against the CPU flavour -----------------------------
def test_cpu_flavour_matches_torch_cpu_ops():
    n = 200_000
    p, g, m, v = oracle.synth_inputs(n, 77)
    noise = oracle.synth_noise(n, 77)
    step = 10
    to_t = lambda a: torch.from_numpy(oracle.bf16_to_f32(a).copy())
    P, G, M, V = to_t(p), to_t(g), to_t(m), to_t(v)
    beta1, beta2 = HP0["betas"]
    bc = 1 - beta1 ** step
    bcs = (1 - beta2 ** step) ** 0.5
    ss = HP0["lr"] / bc
    M.mul_(beta1).add_(G, alpha=1 - beta1)
    V.mul_(beta2).addcmul_(G, G, value=1 - beta2)
    # torch's CPU sqrt (MKL VML) is not correctly rounded on large tensors; the reference
    # never runs it (it computes on a GPU, whose sqrt is), so take the correctly rounded one
    sq = V.double().sqrt().float()
    den = (sq / bcs).add_(HP0["eps"])
    P.mul_(1 - ss * HP0["weight_decay"])
    P.addcdiv_(M, den, value=-ss)
    sc = oracle.scalars_from_hparams(step=step, **HP0)
    pp, mm, vv = p.copy(), m.copy(), v.copy()
    d = oracle.step_tensor(pp, g, mm, vv, sc, noise=noise, flavour=oracle.TORCH_CPU_FLAVOUR, debug=True)
    for got, want, name in zip(d, (P, M, V), "pmv"):
        np.testing.assert_array_equal(got.view(np.uint32), want.numpy().view(np.uint32), err_msg=name)
    # and the stochastic-rounding write-back against raw torch integer ops
    for pre, nz, got in zip((P, M, V), noise, (pp, mm, vv)):
        tgt = torch.empty(n, dtype=torch.bfloat16)
        torch_ops.sr_write_(tgt, pre, torch.from_numpy(nz.astype(np.int32)))
        np.testing.assert_array_equal(got, tgt.view(torch.int16).numpy().view(np.uint16))


# ---- textbook formula in float64 --------------------------------------------------------
@pytest.mark.parametrize("flavour", [oracle.REFERENCE_FLAVOUR, oracle.TORCH_CPU_FLAVOUR, 0])
@pytest.mark.parametrize("hp,step", [(HP0, 10), (dict(lr=3e-4, betas=(0.95, 0.99), eps=1e-6, weight_decay=0.0), 3),
                                     (dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.1), 1)])
def test_update_matches_float64_formula(flavour, hp, step):
    n = 20_000
    p, g, m, v = oracle.synth_inputs(n, 5)
    sc = oracle.scalars_from_hparams(step=step, **hp)
    d = oracle.step_tensor(p.copy(), g, m.copy(), v.copy(), sc, noise=oracle.synth_noise(n, 5), flavour=flavour,
                           debug=True)
    P, G, M, V = (oracle.bf16_to_f32(a).astype(np.float64) for a in (p, g, m, v))
    b1, b2 = hp["betas"]
    m1 = b1 * M + (1 - b1) * G
    v1 = b2 * V + (1 - b2) * G * G
    ss = hp["lr"] / (1 - b1 ** step)
    den = np.sqrt(v1) / np.sqrt(1 - b2 ** step) + hp["eps"]
    p1 = P * (1 - ss * hp["weight_decay"]) - ss * m1 / den
    # m' and p' are sums that can cancel: bound the error by the magnitude of their terms
    assert np.max(np.abs(d[1] - m1) / (np.abs(b1 * M) + np.abs((1 - b1) * G))) < 3e-7
    np.testing.assert_allclose(d[2], v1, rtol=3e-7, atol=0)
    scale = np.abs(P) + np.abs(ss * m1 / den)
    assert np.max(np.abs(d[0] - p1) / scale) < 5e-7


def test_update_special_cases():
    sc = oracle.scalars_from_hparams(step=10, **HP0)
    # zero grad and zero states: pure decay, states stay zero
    po, mo, vo = oracle.update_elem(0.5, 0.0, 0.0, 0.0, sc)
    assert (po, mo, vo) == (np.float32(0.5) * np.float32(sc.decay), 0.0, 0.0)
    # weight_decay == 0 leaves p untouched by the decay multiply
    sc0 = oracle.scalars_from_hparams(step=10, lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0)
    po, _, _ = oracle.update_elem(0.5, 0.0, 0.0, 0.0, sc0)
    assert po == np.float32(0.5)
    # sign: a positive gradient moves the parameter down, a negative one up
    lo, _, _ = oracle.update_elem(0.0, 1e-3, 0.0, 0.0, sc0)
    hi, _, _ = oracle.update_elem(0.0, -1e-3, 0.0, 0.0, sc0)
    assert lo < 0 < hi and lo == -hi
    # loss scale and clip multiply the gradient before anything else
    scs = oracle.scalars_from_hparams(step=10, inv_loss_scale=1 / 1024, apply_clip=True, **HP0)
    a = oracle.update_elem(0.1, 1.024, 1e-4, 1e-6, scs, clip_coef=0.5)
    b = oracle.update_elem(0.1, 1.024 / 1024 * 0.5, 1e-4, 1e-6, sc)
    assert a == b


# ---- stochastic rounding -----------------------------------------------------------------
@pytest.mark.parametrize("bits", [0x3F800001, 0x3F80FFFF, 0xBF808000, 0x00000001, 0x3FFFFFFF, 0x7F7F0001, 0x3F800000])
def test_sr_round_up_count_equals_low16(bits):
    x = np.array([bits], np.uint32).view(np.float32)[0]
    noises = np.arange(65536, dtype=np.uint16)
    out = oracle.sr_copy(np.full(65536, x, np.float32), noise=noises)
    truncated = bits >> 16
    ups = int((out != truncated).sum())
    assert ups == (bits & 0xFFFF)
    assert set(np.unique(out)) <= {truncated, (truncated + 1) & 0xFFFF}


def test_sr_edge_cases():
    f = lambda b: np.array([b], np.uint32).view(np.float32)[0]
    assert oracle.sr_bf16(f(0x7F800000), 0xFFFF) == 0x7F80      # +inf stays
    assert oracle.sr_bf16(f(0xFF800000), 0xFFFF) == 0xFF80      # -inf stays
    assert oracle.sr_bf16(f(0x00000000), 0xFFFF) == 0x0000      # +0 stays
    assert oracle.sr_bf16(f(0x80000000), 0xFFFF) == 0x8000      # -0 stays
    assert oracle.sr_bf16(f(0x3F800000), 0xFFFF) == 0x3F80      # bf16-exact values never move
    assert oracle.sr_bf16(f(0x7F7FFFFF), 0x0001) == 0x7F80      # largest finite can carry into inf
    assert oracle.sr_bf16(f(0x3FFFFFFF), 0x0001) == 0x4000      # mantissa carry into the exponent
    assert oracle.sr_bf16(f(0x00000001), 0xFFFF) == 0x0001      # denormal rounds up to the smallest bf16
    assert oracle.sr_bf16(f(0x00000001), 0xFFFE) == 0x0000
    assert oracle.sr_bf16(f(0xBF808000), 0x8000) == 0xBF81      # negative values round away from zero
    assert oracle.sr_bf16(f(0xBF808000), 0x7FFF) == 0xBF80
    assert oracle.sr_bf16(f(0xFFFFFFFF), 0xFFFF) == 0x0000      # int32 wrap of a NaN pattern (reference quirk)


def test_sr_is_unbiased_in_expectation():
    # E[round(x)] over all noises equals x exactly
    for bits in (0x3F812345, 0xBE00F00F, 0x00FF8001):
        x = np.array([bits], np.uint32).view(np.float32)[0]
        out = oracle.sr_copy(np.full(65536, x, np.float32), noise=np.arange(65536, dtype=np.uint16))
        mean = oracle.bf16_to_f32(out).astype(np.float64).mean()
        assert mean == np.float64(x)


# ---- Philox ------------------------------------------------------------------------------
def test_philox_random123_vectors(kat):
    for vec in kat["philox4x32_10"]:
        got = oracle.philox4x32_10([int(x, 16) for x in vec["ctr"]], [int(x, 16) for x in vec["key"]])
        assert list(got) == [int(x, 16) for x in vec["out"]]


def _philox_py(ctr, key):
    """Independent pure-Python Philox4x32-10 (Salmon et al. 2011, fig. 2)."""
    c, k = list(ctr), list(key)
    for _ in range(10):
        hi0, lo0 = divmod(0xD2511F53 * c[0], 1 << 32)
        hi1, lo1 = divmod(0xCD9E8D57 * c[2], 1 << 32)
        c = [hi1 ^ c[1] ^ k[0], lo1, hi0 ^ c[3] ^ k[1], lo0]
        k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
    return c


def test_noise_counter_layout():
    seed, step, tid = 0x1234_5678_9ABC_DEF0, 100, 17
    for which, elem in itertools.product((0, 1, 2), (0, 1, 7, 8, 9, 4095, (1 << 35) + 13)):
        blk = elem >> 3
        out = _philox_py([blk & 0xFFFFFFFF, blk >> 32, tid * 4 + which, step], [seed & 0xFFFFFFFF, seed >> 32])
        word = out[(elem & 7) >> 1]
        want = (word >> 16) if (elem & 1) else (word & 0xFFFF)
        assert oracle.philox_noise(seed, step, tid, which, elem) == want


def test_noise_is_uniform_and_independent_between_arrays():
    n = 1 << 16
    a = oracle.philox_noise_array(1234, 100, 0, 0, 0, n).astype(np.float64)
    b = oracle.philox_noise_array(1234, 100, 0, 1, 0, n).astype(np.float64)
    c = oracle.philox_noise_array(1234, 101, 0, 0, 0, n).astype(np.float64)
    for x in (a, b, c):
        assert abs(x.mean() - 32767.5) < 4 * 18918 / np.sqrt(n)
    assert abs(np.corrcoef(a, b)[0, 1]) < 0.02 and abs(np.corrcoef(a, c)[0, 1]) < 0.02


# ---- whole-tensor plumbing -----------------------------------------------------------------
def test_pieces_equal_whole_in_philox_mode():
    n = 4096 + 24
    p, g, m, v = oracle.synth_inputs(n, 3)
    sc = oracle.scalars_from_hparams(step=7, **HP0)
    whole = [a.copy() for a in (p, m, v)]
    oracle.step_tensor(whole[0], g, whole[1], whole[2], sc, seed=9, step=7, tensor_id=2)
    parts = [a.copy() for a in (p, m, v)]
    for lo, hi in ((0, 1024), (1024, 4000), (4000, n)):
        sl = [np.ascontiguousarray(a[lo:hi]) for a in parts]
        oracle.step_tensor(sl[0], np.ascontiguousarray(g[lo:hi]), sl[1], sl[2], sc, seed=9, step=7, tensor_id=2,
                           elem_offset=lo)
        for a, s in zip(parts, sl):
            a[lo:hi] = s
    for w, q in zip(whole, parts):
        np.testing.assert_array_equal(w, q)


def test_mixed_dtypes_store_plain_fp32():
    n = 64
    p, g, m, v = oracle.synth_inputs(n, 8)
    sc = oracle.scalars_from_hparams(step=2, **HP0)
    v32 = oracle.bf16_to_f32(v).copy()
    g32 = oracle.bf16_to_f32(g).copy()
    pp, mm = p.copy(), m.copy()
    d = oracle.step_tensor(pp, g32, mm, v32, sc, g_dtype=oracle.DT_F32, v_dtype=oracle.DT_F32, seed=1, step=2,
                           debug=True)
    np.testing.assert_array_equal(v32, d[2])  # fp32 state: stored as computed (adamw.py:221-222)
    ref = [a.copy() for a in (p, m, v)]
    d2 = oracle.step_tensor(ref[0], g, ref[1], ref[2], sc, seed=1, step=2, debug=True)
    np.testing.assert_array_equal(d[0], d2[0])
    np.testing.assert_array_equal(pp, ref[0])


def test_f16_gradient_decode():
    h = np.array([0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x3C00, 0xBC00, 0x7BFF, 0x1234], np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.lib().orc_f16_to_f32(int(x)) for x in h], np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_matches_numpy_and_torch():
    """fp16 params / states take a plain copy_ (adamw.py:208,214,221-222): round to nearest even
    with gradual underflow.  Pinned against numpy's and torch's own conversions on every
    high-half pattern crossed with the low halves that decide the rounding, plus random bits."""
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x0FFF, 0x1000, 0x1001, 0x1FFF, 0x2000, 0x2FFF, 0x3000, 0x3001, 0x7FFF,
                     0x8000, 0x8001, 0xEFFF, 0xF000, 0xF001, 0xFFFF], np.uint32)
    bits = (hi[:, None] | lows[None, :]).ravel()
    rng = np.random.default_rng(3)
    bits = np.concatenate([bits, rng.integers(0, 1 << 32, 2_000_000, dtype=np.uint64).astype(np.uint32)])
    x = bits.view(np.float32)
    finite = ~np.isnan(x)  # NaN payloads are not part of the contract
    got = oracle.f32_to_f16_rne(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(got[finite], want[finite])
    want_t = torch.from_numpy(x.copy()).to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got[finite], want_t[finite])
    nan16 = got[~finite]
    assert np.all((nan16 & 0x7C00) == 0x7C00) and np.all((nan16 & 0x03FF) != 0)


@pytest.mark.parametrize("dts", [("f16", "f16", "f16"), ("f64", "f16", "f32"), ("bf16", "f64", "f16"),
                                 ("f16", "bf16", "f64")])
def test_fp16_and_fp64_targets_take_a_plain_copy(dts):
    """Write-back dtype only changes the last conversion: the fp32 result (debug output) is the
    same as in the all-fp32 run fed the same upcast inputs, and the stored value is its plain
    conversion (numpy's), not a stochastic rounding."""
    n = 4099
    pb, gb, mb, vb = oracle.synth_inputs(n, 21)
    f32 = [oracle.bf16_to_f32(a).copy() for a in (pb, gb, mb, vb)]
    f32[0][:4] = [70000.0, -70000.0, 1e-7, -3e-8]  # fp16 overflow and gradual underflow of the param
    code = {"bf16": oracle.DT_BF16, "f32": oracle.DT_F32, "f16": oracle.DT_F16, "f64": oracle.DT_F64}

    def store(x32, dt):
        if dt == "f16":
            with np.errstate(over="ignore"):
                return x32.astype(np.float16).view(np.uint16).copy()
        if dt == "f64":
            return x32.astype(np.float64)
        if dt == "bf16":
            return oracle.f32_to_bf16_rne(x32)
        return x32.copy()

    def load(a, dt):
        if dt == "f16":
            return a.view(np.float16).astype(np.float32)
        if dt == "f64":
            return a.astype(np.float32)
        if dt == "bf16":
            return oracle.bf16_to_f32(a)
        return a

    arrs = [store(f32[0], dts[0]), store(f32[2], dts[1]), store(f32[3], dts[2])]
    ups = [load(a, dt).copy() for a, dt in zip(arrs, dts)]
    sc = oracle.scalars_from_hparams(step=7, **HP0)
    ref = oracle.step_tensor(ups[0], f32[1], ups[1], ups[2], sc, p_dtype=oracle.DT_F32, g_dtype=oracle.DT_F32,
                             m_dtype=oracle.DT_F32, v_dtype=oracle.DT_F32, seed=5, step=7, debug=True)
    dbg = oracle.step_tensor(arrs[0], f32[1], arrs[1], arrs[2], sc, p_dtype=code[dts[0]], g_dtype=oracle.DT_F32,
                             m_dtype=code[dts[1]], v_dtype=code[dts[2]], seed=5, step=7, tensor_id=3, debug=True)
    for k in range(3):
        np.testing.assert_array_equal(dbg[k].view(np.uint32), ref[k].view(np.uint32))
        if dts[k] == "bf16":
            nz = oracle.philox_noise_array(5, 7, 3, k, 0, n)
            want = ((dbg[k].view(np.uint32).astype(np.uint64) + nz) >> 16).astype(np.uint16)
            np.testing.assert_array_equal(arrs[k], want)
        else:
            w = store(dbg[k], dts[k])
            np.testing.assert_array_equal(arrs[k].view(np.uint16 if dts[k] == "f16" else arrs[k].dtype),
                                          w.view(np.uint16 if dts[k] == "f16" else w.dtype))


def test_grad_sumsq_and_clip_coef():
    g = oracle.f32_to_bf16_rne(np.random.default_rng(0).normal(0, 1e-3, 10_000).astype(np.float32) * 1024)
    want = float(np.sum((oracle.bf16_to_f32(g).astype(np.float64) / 1024) ** 2))
    assert oracle.grad_sumsq(g, inv_loss_scale=1 / 1024) == pytest.approx(want, rel=1e-12)
    assert oracle.clip_coef(0.5, 1.0) == np.float32(1.0)
    assert oracle.clip_coef(4.0, 1.0) == np.float32(1.0) / (np.float32(4.0) + np.float32(1e-6))


def test_row_means():
    g = oracle.f32_to_bf16_rne(np.arange(12, dtype=np.float32))
    np.testing.assert_array_equal(oracle.row_means(g, 3, 4), np.array([1.5, 5.5, 9.5], np.float32))
