"""The host-resident (streamed) path: params / states in pinned host memory,
chunked H2D -> update -> D2H.  Results must be bit-identical to the resident
path and to the oracle, whatever the chunk size.  Run with ``-m gpu``.
"""
import numpy as np
import pytest
import torch

import oracle
import ramtorch_amd
from ramtorch_amd import _native as N
from ramtorch_amd import functional as F

pytestmark = pytest.mark.gpu
HP0 = dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01)


def host16(a, pin=True):
    t = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return t.pin_memory() if pin else t


def dev16(a):
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).cuda()


def nmis(a, b):
    """Number of elements whose bits differ (keeps assertion messages short)."""
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    assert a.shape == b.shape and a.dtype == b.dtype, (a.shape, b.shape, a.dtype, b.dtype)
    it = {2: torch.int16, 4: torch.int32}[a.element_size()]
    return int((a.view(it) != b.view(it)).sum())


def bits16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).ravel()


@pytest.fixture(scope="module")
def handle():
    h = N.Handle(0)
    yield h
    torch.cuda.synchronize()
    h.close()


LENS = [1, 5, 8, 4096, 8191, 8193, 30_011, 16, 100_000, 0, 7]


@pytest.mark.parametrize("chunk_elems", [8, 64, 4096, 8192, 65_536, 1 << 22])
def test_streamed_equals_oracle_for_any_chunk_size(handle, chunk_elems):
    sc, sco = F.make_scalars(step=10, **HP0), oracle.scalars_from_hparams(step=10, **HP0)
    entries, inputs = [], []
    lens = [n for n in LENS if n < 10_000] if chunk_elems < 64 else LENS  # keep the call count sane
    for i, n in enumerate(lens):
        p, g, m, v = oracle.synth_inputs(n, 50 + i)
        entries.append(F.Entry(p=host16(p), g=dev16(g), m=host16(m), v=host16(v), step=10, scalars_idx=0,
                               tensor_id=i))
        inputs.append((p, g, m, v))
    F.step_streamed(handle, entries, [sc], seed=77, explicit_noise=False, chunk_elems=chunk_elems)
    # no synchronisation here on purpose: host memory must be final when the call returns
    for i, (e, (p, g, m, v)) in enumerate(zip(entries, inputs)):
        po, mo, vo = p.copy(), m.copy(), v.copy()
        oracle.step_tensor(po, g, mo, vo, sco, seed=77, step=10, tensor_id=i)
        for name, t, a in zip("pmv", (e.p, e.m, e.v), (po, mo, vo)):
            np.testing.assert_array_equal(t.view(torch.int16).numpy().view(np.uint16), a,
                                          err_msg=f"chunk {chunk_elems} tensor {i} (n={lens[i]}) {name}")
    stats = handle.streamed_stats()
    total = sum(lens)
    assert stats["bytes_h2d"] == 6 * total and stats["bytes_d2h"] == 6 * total


def test_streamed_mixed_residency_and_dtypes(handle):
    """GPU params with host states (the constructor's default layout), host
    unpinned gradients, fp32 state on the host, explicit noise."""
    n = 50_000
    p, g, m, v = oracle.synth_inputs(n, 90)
    noise = oracle.synth_noise(n, 90)
    NZ = tuple(torch.from_numpy(z.view(np.int16).copy()).cuda() for z in noise)
    sc, sco = F.make_scalars(step=3, **HP0), oracle.scalars_from_hparams(step=3, **HP0)
    v32 = oracle.bf16_to_f32(v).copy()
    e0 = F.Entry(p=dev16(p), g=dev16(g), m=host16(m), v=host16(v), step=3, scalars_idx=0, tensor_id=0, noise=NZ)
    e1 = F.Entry(p=host16(p), g=host16(g, pin=False), m=host16(m), v=torch.from_numpy(v32.copy()).pin_memory(),
                 step=3, scalars_idx=0, tensor_id=1, noise=NZ)
    F.step_streamed(handle, [e0, e1], [sc], seed=0, explicit_noise=True, chunk_elems=16_384)
    torch.cuda.synchronize()
    a = [p.copy(), m.copy(), v.copy()]
    oracle.step_tensor(a[0], g, a[1], a[2], sco, noise=noise)
    for name, t, w in zip("pmv", (e0.p, e0.m, e0.v), a):
        np.testing.assert_array_equal(bits16(t), w, err_msg=f"e0 {name}")
    b = [p.copy(), m.copy(), v32.copy()]
    oracle.step_tensor(b[0], g, b[1], b[2], sco, v_dtype=oracle.DT_F32, noise=noise)
    np.testing.assert_array_equal(bits16(e1.p), b[0])
    np.testing.assert_array_equal(bits16(e1.m), b[1])
    np.testing.assert_array_equal(e1.v.numpy().view(np.uint32), b[2].view(np.uint32))


@pytest.mark.parametrize("chunk_elems", [64, 4096, 65_536])
def test_unpinned_gradients_go_up_through_bounce_buffers(handle, chunk_elems):
    """The reference's offload flow leaves the gradients in ordinary CPU memory (linear.py:416-427):
    host threads copy them into pinned bounce buffers chunk by chunk.  More chunks than bounce
    buffers, pinned and unpinned gradients in one call, two calls in a row (the buffer index
    runs on across calls), and an unpinned parameter next to pinned states (it goes up through the
    upload slots and its update comes back through the download slots)."""
    lens = [30_011, 8, 0, 4096, 100_000, 5, 8193]
    before = handle.streamed_bounce_stats()
    state = []
    for i, n in enumerate(lens):
        p, g, m, v = oracle.synth_inputs(n, 500 + i)
        state.append([p, g, m, v, host16(p, pin=(i != 4)), host16(m), host16(v)])
    expect_bytes = 0
    for step in (7, 8):
        sc, sco = F.make_scalars(step=step, **HP0), oracle.scalars_from_hparams(step=step, **HP0)
        entries = []
        for i, (p, g, m, v, P, M, V) in enumerate(state):
            unpinned = i % 3 != 1
            G = host16(g, pin=not unpinned)
            assert G.is_pinned() != unpinned or len(g) == 0
            entries.append(F.Entry(p=P, g=G, m=M, v=V, step=step, scalars_idx=0, tensor_id=i))
            expect_bytes += 2 * len(g) * unpinned + 2 * 2 * len(p) * (i == 4)   # the unpinned parameter goes up and comes down
        F.step_streamed(handle, entries, [sc], seed=31, explicit_noise=False, chunk_elems=chunk_elems)
        for i, (p, g, m, v, P, M, V) in enumerate(state):
            oracle.step_tensor(p, g, m, v, sco, seed=31, step=step, tensor_id=i)
            for name, t, a in zip("pmv", (P, M, V), (p, m, v)):
                np.testing.assert_array_equal(bits16(t), a, err_msg=f"step {step} chunk {chunk_elems} tensor {i} {name}")
    after = handle.streamed_bounce_stats()
    assert after["calls"] - before["calls"] == 2
    assert after["bytes"] - before["bytes"] == expect_bytes


def test_unpinned_uploads_can_be_left_to_the_runtime(monkeypatch):
    """RT_STREAM_BOUNCE_THREADS=0 (read when a handle first streams): no bounce buffers, no host
    threads; the runtime stages the copies from ordinary CPU memory itself.  Same results."""
    monkeypatch.setenv("RT_STREAM_BOUNCE_THREADS", "0")
    h = N.Handle(0)
    try:
        n = 50_000
        p, g, m, v = oracle.synth_inputs(n, 520)
        e = F.Entry(p=host16(p), g=host16(g, pin=False), m=host16(m), v=host16(v), step=4, scalars_idx=0, tensor_id=3)
        F.step_streamed(h, [e], [F.make_scalars(step=4, **HP0)], seed=8, explicit_noise=False, chunk_elems=8192)
        assert h.streamed_bounce_stats() == {"calls": 0, "bytes": 0}
        oracle.step_tensor(p, g, m, v, oracle.scalars_from_hparams(step=4, **HP0), seed=8, step=4, tensor_id=3)
        for name, t, a in zip("pmv", (e.p, e.m, e.v), (p, m, v)):
            np.testing.assert_array_equal(bits16(t), a, err_msg=name)
    finally:
        torch.cuda.synchronize()
        h.close()


@pytest.mark.parametrize("blocking", [True, False])
@pytest.mark.parametrize("which", ["pinned gradient", "ordered parameter"])
def test_uploads_wait_for_host_arrays_the_stream_is_still_filling(handle, which, blocking):
    """A gradient in pinned host memory may still be on its way there (grad.to("cpu", non_blocking=True)
    on a busy stream): the upload must wait for the caller's stream.  The same for a host parameter
    when the caller says so (RT_HOST_ORDERED); without either, uploads do not wait."""
    n = 3_000_000
    p, g, m, v = oracle.synth_inputs(n, 530)
    stale = torch.zeros(n, dtype=torch.bfloat16).pin_memory()
    # everything is prepared first: a blocking copy further down would drain the stream
    if which == "pinned gradient":
        fresh = dev16(g)
        e = F.Entry(p=host16(p), g=stale, m=host16(m), v=host16(v), step=6, scalars_idx=0, tensor_id=1)
    else:
        fresh = dev16(p)
        e = F.Entry(p=stale, g=dev16(g), m=host16(m), v=host16(v), step=6, scalars_idx=0, tensor_id=1, ordered=True)
    sc = [F.make_scalars(step=6, **HP0)]
    busy = torch.randn(4096, 4096, device="cuda")
    torch.cuda.synchronize()
    for _ in range(150):                      # a hundred milliseconds of work ahead of the copy
        busy = (busy @ busy) * 1e-4
    stale.copy_(fresh, non_blocking=True)     # not there yet when the call below is made
    # the call that returns when all is done waits for the stream on the host, the asynchronous one on the GPU
    F.step_streamed(handle, [e], sc, seed=12, explicit_noise=False, chunk_elems=1 << 20, wait=blocking)
    if not blocking:
        handle.streamed_wait()
    oracle.step_tensor(p, g, m, v, oracle.scalars_from_hparams(step=6, **HP0), seed=12, step=6, tensor_id=1)
    for name, t, a in zip("pmv", (e.p, e.m, e.v), (p, m, v)):
        np.testing.assert_array_equal(bits16(t), a, err_msg=name)


def test_streamed_and_resident_agree_bit_for_bit(handle):
    n = 300_000
    p, g, m, v = oracle.synth_inputs(n, 95)
    sc = F.make_scalars(step=42, **HP0)
    r = F.Entry(p=dev16(p), g=dev16(g), m=dev16(m), v=dev16(v), step=42, scalars_idx=0, tensor_id=4)
    F.step_resident(handle, [r], [sc], seed=5, explicit_noise=False)
    s = F.Entry(p=host16(p), g=dev16(g), m=host16(m), v=host16(v), step=42, scalars_idx=0, tensor_id=4)
    F.step_streamed(handle, [s], [sc], seed=5, explicit_noise=False, chunk_elems=40_000)
    torch.cuda.synchronize()
    for a, b in ((r.p, s.p), (r.m, s.m), (r.v, s.v)):
        assert nmis(a.cpu(), b) == 0


def test_optimizer_default_layout_cpu_params_and_pinned_states():
    """The reference's offload flow: pinned CPU bf16 params (as ramtorch.Linear
    creates them), CPU gradients, pinned CPU states, several steps."""
    shapes = [(128, 96), (96,), (33, 7)]
    ps, gs, refs = [], [], []
    for i, shp in enumerate(shapes):
        n = int(np.prod(shp))
        p, g, _, _ = oracle.synth_inputs(n, 900 + i)
        t = torch.nn.Parameter(host16(p).view(shp))
        t.is_ramtorch = True
        ps.append(t)
        gs.append(g)
        refs.append([p.copy(), np.zeros(n, np.uint16), np.zeros(n, np.uint16)])
    opt = ramtorch_amd.AdamW(ps, seed=21, stream_chunk_bytes=16_384, **HP0)
    assert all(opt.state[p]["ema"].is_pinned() and opt.state[p]["ema"].device.type == "cpu" for p in ps)
    for step in (1, 2, 3):
        for p, g in zip(ps, gs):
            p.grad = host16(g, pin=False).view(p.shape)        # Linear.backward leaves CPU grads
        opt.step()
        sco = oracle.scalars_from_hparams(step=step, **HP0)
        for i, (p, g) in enumerate(zip(ps, gs)):
            oracle.step_tensor(refs[i][0], g, refs[i][1], refs[i][2], sco, seed=21, step=step, tensor_id=i)
            np.testing.assert_array_equal(bits16(p), refs[i][0], err_msg=f"step {step} param {i}")
            np.testing.assert_array_equal(bits16(opt.state[p]["ema"]), refs[i][1])
            np.testing.assert_array_equal(bits16(opt.state[p]["ema_squared"]), refs[i][2])
    assert all(p.is_pinned() for p in ps)  # params were updated in place


def test_optimizer_plain_pageable_cpu_params():
    """Plain (not pinned) CPU parameters and gradients, the third input kind the reference accepts:
    the copies are staged by the runtime instead of going by DMA, results are the same."""
    shapes = [(70_000,), (257, 31)]
    ps, gs, refs = [], [], []
    for i, shp in enumerate(shapes):
        n = int(np.prod(shp))
        p, g, _, _ = oracle.synth_inputs(n, 950 + i)
        t = torch.nn.Parameter(host16(p, pin=False).view(shp))
        assert not t.is_pinned()
        ps.append(t)
        gs.append(g)
        refs.append([p.copy(), np.zeros(n, np.uint16), np.zeros(n, np.uint16)])
    opt = ramtorch_amd.AdamW(ps, seed=22, stream_chunk_bytes=65_536, **HP0)
    for step in (1, 2):
        for p, g in zip(ps, gs):
            p.grad = host16(g, pin=False).view(p.shape)
        opt.step()
        sco = oracle.scalars_from_hparams(step=step, **HP0)
        for i, (p, g) in enumerate(zip(ps, gs)):
            oracle.step_tensor(refs[i][0], g, refs[i][1], refs[i][2], sco, seed=22, step=step, tensor_id=i)
            np.testing.assert_array_equal(bits16(p), refs[i][0], err_msg=f"step {step} param {i}")
            np.testing.assert_array_equal(bits16(opt.state[p]["ema"]), refs[i][1])
            np.testing.assert_array_equal(bits16(opt.state[p]["ema_squared"]), refs[i][2])


def test_optimizer_gpu_params_with_default_cpu_states():
    n = 20_000
    p, g, _, _ = oracle.synth_inputs(n, 950)
    P = torch.nn.Parameter(dev16(p))
    P.grad = dev16(g)
    opt = ramtorch_amd.AdamW([P], seed=1, **HP0)          # storage_device defaults to "cpu"
    opt.step()
    po, mo, vo = p.copy(), np.zeros(n, np.uint16), np.zeros(n, np.uint16)
    oracle.step_tensor(po, g, mo, vo, oracle.scalars_from_hparams(step=1, **HP0), seed=1, step=1, tensor_id=0)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(bits16(P), po)
    np.testing.assert_array_equal(bits16(opt.state[P]["ema"]), mo)


# ---- updates started from inside backward (the post-accumulate-grad hook of ramtorch.Linear) ----------
def _offload_params(shapes, seed):
    ps, gs, refs = [], [], []
    for i, shp in enumerate(shapes):
        n = int(np.prod(shp))
        p, g, _, _ = oracle.synth_inputs(n, seed + i)
        t = torch.nn.Parameter(host16(p).view(shp))
        t.is_ramtorch = True
        ps.append(t)
        gs.append(g)
        refs.append([p.copy(), np.zeros(n, np.uint16), np.zeros(n, np.uint16)])
    return ps, gs, refs


def test_post_accumulate_hook_updates_from_the_gpu_gradient():
    shapes = [(256, 128), (128,), (64, 64), (40_000,)]
    ps, gs, refs = _offload_params(shapes, 1200)
    opt = ramtorch_amd.AdamW(ps, seed=31, stream_chunk_bytes=32_768, **HP0)
    hook = opt.make_post_accumulate_hook()
    for step in (1, 2):
        # what Linear.backward does per layer, last layer first (linear.py:341-430)
        for p, g in reversed(list(zip(ps, gs))):
            p.ramtorch_grad = dev16(g).view(p.shape)          # accumulated gradient, on the GPU
            hook(p)
            cpu_grad = p.ramtorch_grad.to("cpu", non_blocking=True)
            del p.ramtorch_grad
            p.grad = cpu_grad                                  # the reference still ships it to the CPU
        assert all(opt.state[p]["step"] == step for p in ps)
        opt.step()                                             # waits; must not apply the update twice
        sco = oracle.scalars_from_hparams(step=step, **HP0)
        for i, (p, g) in enumerate(zip(ps, gs)):
            oracle.step_tensor(refs[i][0], g, refs[i][1], refs[i][2], sco, seed=31, step=step, tensor_id=i)
            np.testing.assert_array_equal(bits16(p), refs[i][0], err_msg=f"step {step} param {i}")
            np.testing.assert_array_equal(bits16(opt.state[p]["ema"]), refs[i][1])
            np.testing.assert_array_equal(bits16(opt.state[p]["ema_squared"]), refs[i][2])
            assert opt.state[p]["step"] == step
    # with the hook switched off (gradient-accumulation micro-step) nothing happens until step()
    opt.fuse_in_backward = False
    for p, g in zip(ps, gs):
        p.ramtorch_grad = dev16(g).view(p.shape)
        hook(p)
        del p.ramtorch_grad
        p.grad = host16(g, pin=False).view(p.shape)
    assert all(opt.state[p]["step"] == 2 for p in ps)
    opt.step()
    sco = oracle.scalars_from_hparams(step=3, **HP0)
    for i, (p, g) in enumerate(zip(ps, gs)):
        oracle.step_tensor(refs[i][0], g, refs[i][1], refs[i][2], sco, seed=31, step=3, tensor_id=i)
        np.testing.assert_array_equal(bits16(p), refs[i][0], err_msg=f"step 3 param {i}")


def test_step_param_with_centralization_equals_step():
    """Updates handed over tensor by tensor (the hook of ramtorch.Linear) with gradient centralization
    (adamw.py:179-184): the row means are taken from the whole gradient, the update then goes in
    staged pieces that start in the middle of rows.  Same bits as step() on the same data."""
    shapes = [(64, 300), (5, 4099), (129,), (9000, 12)]
    out = []
    for early in (False, True):
        ps, gs, _ = _offload_params(shapes, 1250)
        q = torch.nn.Parameter(dev16(gs[1]).view(shapes[1]).clone())   # a GPU-resident parameter as well
        opt = ramtorch_amd.AdamW(ps + [q], seed=9, centralization=0.5, stream_chunk_bytes=2 * 10_000, **HP0)
        for k in ("ema", "ema_squared"):
            opt.state[q][k] = opt.state[q][k].cuda()
        for _ in range(2):
            grads = [dev16(g).view(shp) for g, shp in zip(gs, shapes)] + [dev16(gs[3])[:q.numel()].view(q.shape)]
            if early:
                for p, g in zip(ps + [q], grads):
                    opt.step_param(p, g)
                opt.step()
            else:
                opt.step(grads=dict(zip(ps + [q], grads)))
        torch.cuda.synchronize()
        out.append([(bits16(p), bits16(opt.state[p]["ema"]), bits16(opt.state[p]["ema_squared"])) for p in ps + [q]])
        assert all(opt.state[p]["step"] == 2 for p in ps + [q])
    for a, b in zip(*out):
        for x, y in zip(a, b):
            np.testing.assert_array_equal(x, y)


def test_step_param_mixes_with_step_and_rejects_double_use():
    ps, gs, refs = _offload_params([(3000,), (5000,)], 1300)
    gpu_p, gpu_g, _, _ = oracle.synth_inputs(7000, 1310)
    q = torch.nn.Parameter(dev16(gpu_p))                       # a GPU-resident parameter in the same optimizer
    opt = ramtorch_amd.AdamW([{"params": ps}, {"params": [q], "lr": 3e-4}], seed=2, storage_device="cpu", **HP0)
    opt.state[q]["ema"] = opt.state[q]["ema"].cuda()
    opt.state[q]["ema_squared"] = opt.state[q]["ema_squared"].cuda()
    opt.step_param(ps[0], dev16(gs[0]))                        # early
    opt.step_param(q, dev16(gpu_g))                            # early, resident
    with pytest.raises(RuntimeError, match="twice"):
        opt.step_param(ps[0], dev16(gs[0]))
    ps[1].grad = host16(gs[1], pin=False)                      # this one waits for step()
    ps[0].grad = host16(gs[0], pin=False)
    opt.step()
    torch.cuda.synchronize()
    sco = oracle.scalars_from_hparams(step=1, **HP0)
    for i in (0, 1):
        oracle.step_tensor(refs[i][0], gs[i], refs[i][1], refs[i][2], sco, seed=2, step=1, tensor_id=i)
        np.testing.assert_array_equal(bits16(ps[i]), refs[i][0], err_msg=f"param {i}")
    qo, mo, vo = gpu_p.copy(), np.zeros(7000, np.uint16), np.zeros(7000, np.uint16)
    hp = dict(HP0, lr=3e-4)
    oracle.step_tensor(qo, gpu_g, mo, vo, oracle.scalars_from_hparams(step=1, **hp), seed=2, step=1, tensor_id=2)
    np.testing.assert_array_equal(bits16(q), qo)
    with pytest.raises(ValueError):
        opt.step_param(torch.nn.Parameter(torch.zeros(4)), torch.zeros(4))


def test_async_calls_chain_through_the_shared_staging_buffers(handle):
    """Many asynchronous single-tensor calls in a row, sizes that do not divide the
    chunk: buffers alternate across calls and a grown staging buffer is handled."""
    sc, sco = F.make_scalars(step=5, **HP0), oracle.scalars_from_hparams(step=5, **HP0)
    lens = [100, 9000, 70_001, 8192, 33, 250_000, 4096, 12_345]
    entries, inputs, tickets = [], [], []
    for i, n in enumerate(lens):
        p, g, m, v = oracle.synth_inputs(n, 1400 + i)
        e = F.Entry(p=host16(p), g=dev16(g), m=host16(m), v=host16(v), step=5, scalars_idx=0, tensor_id=i)
        entries.append(e)
        inputs.append((p, g, m, v))
        tickets.append(F.step_streamed(handle, [e], [sc], seed=8, explicit_noise=False, chunk_elems=16_384,
                                       wait=False))
    assert tickets == sorted(tickets) and len(set(tickets)) == len(tickets)
    handle.streamed_wait()
    assert handle.streamed_completed() == tickets[-1]
    for i, (e, (p, g, m, v)) in enumerate(zip(entries, inputs)):
        po, mo, vo = p.copy(), m.copy(), v.copy()
        oracle.step_tensor(po, g, mo, vo, sco, seed=8, step=5, tensor_id=i)
        for name, t, a in zip("pmv", (e.p, e.m, e.v), (po, mo, vo)):
            np.testing.assert_array_equal(bits16(t), a, err_msg=f"tensor {i} (n={lens[i]}) {name}")


def test_load_state_dict_restores_pinned_host_states():
    import copy
    ps, gs, _ = _offload_params([(64, 32)], 1500)
    a = ramtorch_amd.AdamW(ps, seed=3, **HP0)
    ps[0].grad = host16(gs[0], pin=False).view(64, 32)
    a.step()
    sd = copy.deepcopy(a.state_dict())
    ps2 = [torch.nn.Parameter(ps[0].detach().clone().pin_memory())]
    b = ramtorch_amd.AdamW(ps2, **HP0)
    b.load_state_dict(sd)
    st = b.state[ps2[0]]
    assert st["ema"].is_pinned() and st["ema_squared"].is_pinned() and b.seed == 3 and st["step"] == 1
    for opt, params in ((a, ps), (b, ps2)):
        params[0].grad = host16(gs[0], pin=False).view(64, 32)
        opt.step()
    assert nmis(ps[0].detach(), ps2[0].detach()) == 0
    assert nmis(a.state[ps[0]]["ema_squared"], st["ema_squared"]) == 0


@pytest.mark.parametrize("grads_on", ["cuda", "cpu"])
def test_max_grad_norm_with_host_resident_params_and_states(grads_on):
    """Global-norm clip for the offload layout (pinned CPU params and states; gradients on the GPU as
    config 3 has them, or on the CPU as ramtorch.Linear leaves them): the norm is taken on the GPU over
    every gradient and the streamed update multiplies by the coefficient.  The norm against a float64
    sum (1e-6 relative: reduction order), the update bit-exact given the coefficient the kernel used."""
    shapes = [(300, 70), (4096,), (17,)]
    ps, gs, refs = [], [], []
    for i, shp in enumerate(shapes):
        n = int(np.prod(shp))
        p, g, _, _ = oracle.synth_inputs(n, 1300 + i)
        ps.append(torch.nn.Parameter(host16(p).view(shp)))
        gs.append(g)
        refs.append([p.copy(), np.zeros(n, np.uint16), np.zeros(n, np.uint16)])
    opt = ramtorch_amd.AdamW(ps, seed=4, stream_chunk_bytes=8192, max_grad_norm=1e-3, **HP0)
    for step in (1, 2):
        gmap = {}
        for p, g in zip(ps, gs):
            t = host16(g, pin=False).view(p.shape)
            gmap[p] = t.cuda() if grads_on == "cuda" else t
        opt.step(grads=gmap)
        total = float(opt.last_grad_norm[0])
        coef = np.float32(opt.last_grad_norm[1].item())
        want = sum(oracle.grad_sumsq(g, oracle.DT_BF16, 1.0) for g in gs) ** 0.5
        assert total == pytest.approx(want, rel=1e-6)
        assert coef < 1.0 and coef == oracle.clip_coef(np.float32(total), 1e-3)
        sco = oracle.scalars_from_hparams(step=step, apply_clip=True, **HP0)
        for i, (p, g) in enumerate(zip(ps, gs)):
            oracle.step_tensor(refs[i][0], g, refs[i][1], refs[i][2], sco, clip_coef=coef, seed=4, step=step,
                               tensor_id=i)
            np.testing.assert_array_equal(bits16(p), refs[i][0], err_msg=f"step {step} param {i}")
            np.testing.assert_array_equal(bits16(opt.state[p]["ema"]), refs[i][1])
            np.testing.assert_array_equal(bits16(opt.state[p]["ema_squared"]), refs[i][2])
    # a non-finite gradient: nothing moves
    snap = [bits16(p).copy() for p in ps]
    bad = {p: host16(g, pin=False).view(p.shape).cuda() for p, g in zip(ps, gs)}
    bad[ps[1]][3] = float("inf")
    opt.step(grads=bad)
    assert all((bits16(p) == s).all() for p, s in zip(ps, snap))
    assert opt.last_grad_norm.view(torch.int32)[2].item() == 1


def test_host_link_probe_reports_plausible_rates(handle):
    r = handle.host_link_probe(64 << 20, reps=4)
    assert all(5.0 < r[k] < 200.0 for k in ("h2d_GBps", "d2h_GBps", "duplex_GBps_each_way")), r
