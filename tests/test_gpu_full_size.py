"""Parity at the benchmark's full sizes.  The whole result cannot go through
the scalar oracle in reasonable time, so windows of the big tensors are
checked bit for bit instead (the oracle can start anywhere in a tensor through
``elem_offset``), together with properties that do not depend on size.
Run with ``-m gpu``; needs about 70 GB of HBM.
"""
import numpy as np
import pytest
import torch

import oracle
import ramtorch_amd
from bench import HP, fill_tensor, llama3_8b_shapes, numel, small_tensor_shapes
from ramtorch_amd import _native as N
from ramtorch_amd import functional as F

pytestmark = pytest.mark.gpu


def bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).ravel()


def test_llama8b_set_sampled_windows_match_oracle():
    """Config 1: 290 tensors, 8 030 257 152 elements, all bf16, Philox seed 1234, step 100."""
    dev = "cuda:0"
    shapes = llama3_8b_shapes()
    total = sum(numel(s) for s in shapes)
    assert len(shapes) == 290 and total == 8_030_257_152
    params, grads = [], []
    for i, shp in enumerate(shapes):
        params.append(torch.nn.Parameter(fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev), requires_grad=False))
        grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.bfloat16, dev))
    opt = ramtorch_amd.AdamW(params, storage_device="cuda", seed=1234, **HP)
    for i, p in enumerate(params):
        st = opt.state[p]
        st["step"] = 99
        st["ema"] = fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev)
        st["ema_squared"] = fill_tensor(p.shape, "v", 1234 + 4 * i + 3, torch.bfloat16, dev)

    # windows: (tensor index, first element, length); starts are multiples of 8 (a Philox block)
    rng = np.random.default_rng(7)
    W = 4096
    sizes = np.array([numel(s) for s in shapes], dtype=np.float64)
    wins = []
    for ti in rng.choice(len(shapes), size=40, p=sizes / sizes.sum()):
        n = numel(shapes[ti])
        wins.append((int(ti), int(rng.integers(0, max(1, (n - W) // 8 + 1))) * 8, min(W, n)))
    big = 0  # embedding: 525 336 576 elements
    nb = numel(shapes[big])
    wins += [(big, 0, W), (big, nb - W, W), (big, 8192 * 1000 - 8, 64), (len(shapes) - 1, nb - W, W),
             (8, 0, 4096), (9, 0, 4096)]  # the two norm vectors of layer 0 (shorter than one chunk)
    before = []
    for ti, lo, ln in wins:
        p = params[ti]
        st = opt.state[p]
        before.append(tuple(bits16(t.view(-1)[lo:lo + ln]) for t in (p, grads[ti], st["ema"], st["ema_squared"])))
    sums_before = [float(p.float().sum()) for p in params[:3]]

    opt.step(grads=dict(zip(params, grads)))
    torch.cuda.synchronize()

    sc = oracle.scalars_from_hparams(step=100, **HP)
    for (ti, lo, ln), (p0, g0, m0, v0) in zip(wins, before):
        po, mo, vo = p0.copy(), m0.copy(), v0.copy()
        oracle.step_tensor(po, g0, mo, vo, sc, seed=1234, step=100, tensor_id=ti, elem_offset=lo)
        st = opt.state[params[ti]]
        for name, t, want in (("p", params[ti], po), ("ema", st["ema"], mo), ("ema_squared", st["ema_squared"], vo)):
            got = bits16(t.view(-1)[lo:lo + ln])
            bad = int((got != want).sum())
            assert bad == 0, f"tensor {ti} window [{lo}, {lo + ln}) {name}: {bad} of {ln} values differ"
    # size-independent properties: every tensor advanced one step; every parameter tensor moved;
    # second moments stay non-negative
    assert all(opt.state[p]["step"] == 100 for p in params)
    assert all(float(p.float().sum()) != s for p, s in zip(params[:3], sums_before))
    for p in params[:12]:
        assert int((opt.state[p]["ema_squared"].view(torch.int16) < 0).sum()) == 0


def test_single_tensor_past_2_to_the_32_elements():
    """One tensor longer than 2^32 elements: 64-bit element offsets in the chunk
    table, in the kernel and in the Philox counter; ragged tail through the generic kernel."""
    n = (1 << 32) + 3 * 8192 + 5
    dev = "cuda:0"
    h = N.Handle(0)
    P = fill_tensor((n,), "p", 1, torch.bfloat16, dev)
    G = fill_tensor((n,), "g", 2, torch.bfloat16, dev)
    M = fill_tensor((n,), "m", 3, torch.bfloat16, dev)
    V = fill_tensor((n,), "v", 4, torch.bfloat16, dev)
    wins = [(0, 4096), ((1 << 32) - 2048, 4096), ((1 << 32) + 8192, 4096), (n - 8192 - 5 - 8192 + 8, 4096),
            (n - 1029, 1029)]
    wins = [(lo - lo % 8, ln + lo % 8) for lo, ln in wins]
    before = [tuple(bits16(t[lo:lo + ln]) for t in (P, G, M, V)) for lo, ln in wins]
    e = F.Entry(p=P, g=G, m=M, v=V, step=100, scalars_idx=0, tensor_id=17)
    F.step_resident(h, [e], [F.make_scalars(step=100, **HP)], seed=99, explicit_noise=False)
    torch.cuda.synchronize()
    sc = oracle.scalars_from_hparams(step=100, **HP)
    for (lo, ln), (p0, g0, m0, v0) in zip(wins, before):
        po, mo, vo = p0.copy(), m0.copy(), v0.copy()
        oracle.step_tensor(po, g0, mo, vo, sc, seed=99, step=100, tensor_id=17, elem_offset=lo)
        for name, t, want in (("p", P, po), ("m", M, mo), ("v", V, vo)):
            bad = int((bits16(t[lo:lo + ln]) != want).sum())
            assert bad == 0, f"window [{lo}, {lo + ln}) {name}: {bad} of {ln} values differ"
    h.close()


def test_philox_block_index_above_32_bits():
    n = 10_000
    p, g, m, v = oracle.synth_inputs(n, 5)
    h = N.Handle(0)
    off = (1 << 36) + 4096  # block index (off / 8) needs 34 bits
    dev16 = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).cuda()
    e = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=3, scalars_idx=0, tensor_id=2, elem_offset=off)
    F.step_resident(h, [e], [F.make_scalars(step=3, **HP)], seed=(1 << 63) + 12345, explicit_noise=False)
    torch.cuda.synchronize()
    po, mo, vo = p.copy(), m.copy(), v.copy()
    oracle.step_tensor(po, g, mo, vo, oracle.scalars_from_hparams(step=3, **HP), seed=(1 << 63) + 12345, step=3,
                       tensor_id=2, elem_offset=off)
    for name, t, want in (("p", e.p, po), ("m", e.m, mo), ("v", e.v, vo)):
        assert int((bits16(t) != want).sum()) == 0, name
    h.close()


def test_config2_every_tensor_matches_oracle():
    """Config 2 at full size: 20 000 tensors of 1..4096 elements plus 64 of 1024 x 1024, one step
    through AdamW.step (descriptors gathered in C++ when the helper is built), every tensor
    compared bit for bit."""
    dev = "cuda:0"
    shapes = small_tensor_shapes()
    assert len(shapes) == 20_064
    params, grads, before = [], [], []
    rng = np.random.default_rng(5)
    for i, shp in enumerate(shapes):
        n = numel(shp)
        p, g, m, v = oracle.synth_inputs(n, int(rng.integers(0, 1 << 30)))
        t = torch.from_numpy(p.view(np.int16).copy()).view(torch.bfloat16).view(shp).to(dev)
        params.append(torch.nn.Parameter(t, requires_grad=False))
        grads.append(torch.from_numpy(g.view(np.int16).copy()).view(torch.bfloat16).view(shp).to(dev))
        before.append((p, g, m, v))
    opt = ramtorch_amd.AdamW(params, storage_device="cuda", seed=1234, **HP)
    for p, g, (_, _, m, v) in zip(params, grads, before):
        p.grad = g
        st = opt.state[p]
        st["step"] = 99
        st["ema"].copy_(torch.from_numpy(m.view(np.int16).copy()).view(torch.bfloat16).view(p.shape))
        st["ema_squared"].copy_(torch.from_numpy(v.view(np.int16).copy()).view(torch.bfloat16).view(p.shape))
    opt.step()
    torch.cuda.synchronize()
    sc = oracle.scalars_from_hparams(step=100, **HP)
    bad = []
    for i, (p, (p0, g0, m0, v0)) in enumerate(zip(params, before)):
        po, mo, vo = p0.copy(), m0.copy(), v0.copy()
        oracle.step_tensor(po, g0, mo, vo, sc, seed=1234, step=100, tensor_id=i)
        st = opt.state[p]
        if (st["step"] != 100 or (bits16(p) != po).any() or (bits16(st["ema"]) != mo).any()
                or (bits16(st["ema_squared"]) != vo).any()):
            bad.append(i)
    assert not bad, f"{len(bad)} of {len(params)} tensors differ, first {bad[:5]}"


def test_config4_layout_sampled_windows_match_oracle():
    """Config 4 at full size: bf16 p / ema, fp32 gradients scaled by 1024, fp32 ema_squared, global-norm
    clip to 1.0.  The norm is an order-dependent sum (checked to 1e-5 relative against float64 partial
    sums on the GPU); given the coefficient the kernel used, sampled windows are bit-exact."""
    dev = "cuda:0"
    shapes = llama3_8b_shapes()
    params, grads = [], []
    for i, shp in enumerate(shapes):
        params.append(torch.nn.Parameter(fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev), requires_grad=False))
    for i, shp in enumerate(shapes):
        grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.float32, dev).mul_(1024.0))
    opt = ramtorch_amd.AdamW(params, storage_device="cuda", seed=1234, loss_scale=1024.0, max_grad_norm=1.0,
                             ema_squared_dtype=torch.float32, **HP)
    for i, p in enumerate(params):
        st = opt.state[p]
        st["step"] = 99
        st["ema"].copy_(fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev))
        st["ema_squared"].copy_(fill_tensor(p.shape, "v", 1234 + 4 * i + 3, torch.float32, dev))
    rng = np.random.default_rng(9)
    W = 4096
    sizes = np.array([numel(s) for s in shapes], dtype=np.float64)
    wins = []
    for ti in rng.choice(len(shapes), size=24, p=sizes / sizes.sum()):
        n = numel(shapes[ti])
        wins.append((int(ti), int(rng.integers(0, max(1, (n - W) // 8 + 1))) * 8, min(W, n)))
    wins += [(0, 0, W), (len(shapes) - 1, numel(shapes[-1]) - W, W), (8, 0, 4096)]
    before = []
    for ti, lo, ln in wins:
        p, st = params[ti], opt.state[params[ti]]
        before.append((bits16(p.view(-1)[lo:lo + ln]), grads[ti].view(-1)[lo:lo + ln].cpu().numpy().copy(),
                       bits16(st["ema"].view(-1)[lo:lo + ln]), st["ema_squared"].view(-1)[lo:lo + ln].cpu().numpy().copy()))
    want_sq = sum(float((g.double() / 1024.0).square().sum()) for g in grads)
    opt.step(grads=dict(zip(params, grads)))
    torch.cuda.synchronize()
    norm, coef, found_inf = (float(opt.last_grad_norm[0]), np.float32(opt.last_grad_norm[1].item()),
                             int(opt.last_grad_norm.view(torch.int32)[2]))
    assert found_inf == 0 and abs(norm - want_sq ** 0.5) <= 1e-5 * want_sq ** 0.5
    assert coef == oracle.clip_coef(np.float32(norm), 1.0)
    sc = oracle.scalars_from_hparams(step=100, inv_loss_scale=1.0 / 1024.0, apply_clip=True, **HP)
    for (ti, lo, ln), (p0, g0, m0, v0) in zip(wins, before):
        po, mo, vo = p0.copy(), m0.copy(), v0.copy()
        oracle.step_tensor(po, g0, mo, vo, sc, g_dtype=oracle.DT_F32, v_dtype=oracle.DT_F32, clip_coef=coef, seed=1234,
                           step=100, tensor_id=ti, elem_offset=lo)
        st = opt.state[params[ti]]
        assert int((bits16(params[ti].view(-1)[lo:lo + ln]) != po).sum()) == 0, (ti, lo)
        assert int((bits16(st["ema"].view(-1)[lo:lo + ln]) != mo).sum()) == 0, (ti, lo)
        got_v = st["ema_squared"].view(-1)[lo:lo + ln].cpu().numpy().view(np.uint32)
        assert int((got_v != vo.view(np.uint32)).sum()) == 0, (ti, lo)


def test_config3_streamed_set_sampled_windows_match_oracle():
    """Config 3 at full size: parameters and both states of the 8 030 257 152-element set in pinned host
    memory (48.2 GB), bf16 gradients on the GPU, 256 MB chunks.  One step through the three-stream
    pipeline; sampled windows of the host arrays are bit-exact, including windows that straddle
    chunk boundaries (a chunk holds 134 217 728 staged elements and cuts tensors at multiples of 8)."""
    dev = "cuda:0"
    shapes = llama3_8b_shapes()
    params, grads = [], []
    for i, shp in enumerate(shapes):
        t = fill_tensor(shp, "p", 1234 + 4 * i, torch.bfloat16, dev).cpu().pin_memory()
        params.append(torch.nn.Parameter(t, requires_grad=False))
        grads.append(fill_tensor(shp, "g", 1234 + 4 * i + 1, torch.bfloat16, dev))
    opt = ramtorch_amd.AdamW(params, storage_device="cpu", seed=1234, stream_chunk_bytes=256 << 20, **HP)
    for i, p in enumerate(params):
        st = opt.state[p]
        st["step"] = 99
        st["ema"].copy_(fill_tensor(p.shape, "m", 1234 + 4 * i + 2, torch.bfloat16, dev))
        st["ema_squared"].copy_(fill_tensor(p.shape, "v", 1234 + 4 * i + 3, torch.bfloat16, dev))
        assert st["ema"].is_pinned() and p.is_pinned()
    rng = np.random.default_rng(13)
    W = 4096
    sizes = np.array([numel(s) for s in shapes], dtype=np.float64)
    wins = []
    for ti in rng.choice(len(shapes), size=30, p=sizes / sizes.sum()):
        n = numel(shapes[ti])
        wins.append((int(ti), int(rng.integers(0, max(1, (n - W) // 8 + 1))) * 8, min(W, n)))
    chunk = (256 << 20) // 2
    # the embedding (tensor 0, 525 336 576 elements) is cut at every multiple of `chunk`: windows across the cuts
    wins += [(0, k * chunk - 2048, W) for k in (1, 2, 3)] + [(0, 0, W), (len(shapes) - 1, numel(shapes[-1]) - W, W)]
    before = []
    for ti, lo, ln in wins:
        p, st = params[ti], opt.state[params[ti]]
        # copies: for host tensors bits16() is a view of the live memory
        before.append(tuple(bits16(t.view(-1)[lo:lo + ln]).copy() for t in (p, grads[ti], st["ema"], st["ema_squared"])))
    opt.step(grads=dict(zip(params, grads)))   # returns when host memory is final
    sc = oracle.scalars_from_hparams(step=100, **HP)
    for (ti, lo, ln), (p0, g0, m0, v0) in zip(wins, before):
        po, mo, vo = p0.copy(), m0.copy(), v0.copy()
        oracle.step_tensor(po, g0, mo, vo, sc, seed=1234, step=100, tensor_id=ti, elem_offset=lo)
        st = opt.state[params[ti]]
        for name, t, want in (("p", params[ti], po), ("ema", st["ema"], mo), ("ema_squared", st["ema_squared"], vo)):
            bad = int((bits16(t.view(-1)[lo:lo + ln]) != want).sum())
            assert bad == 0, f"tensor {ti} window [{lo}, {lo + ln}) {name}: {bad} of {ln} values differ"
    assert all(opt.state[p]["step"] == 100 for p in params)
