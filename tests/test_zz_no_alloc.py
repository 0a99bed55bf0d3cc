"""rt_grad_norm_static -- the entry point that allocates no device memory -- against rt_grad_norm,
through the C ABI.  Needs an MI355X: run with ``-m gpu``.

Bar: the three output words (norm, clip coefficient, non-finite flag) are identical bit for bit:
both entry points add the same per-chunk sums in the same order.  The norm itself is also held
against a float64 sum, relative tolerance 1e-6 (an order-dependent fp32/fp64 reduction).
"""

import numpy as np
import pytest
import torch

from ramtorch_amd import _native as N
from ramtorch_amd import functional as F

pytestmark = pytest.mark.gpu


def _descs(grads):
    d = np.zeros(len(grads), F.DESC_DTYPE)
    d["g"] = [g.data_ptr() for g in grads]
    d["numel"] = [g.numel() for g in grads]
    d["g_dtype"] = [F.dtype_code(g.dtype, "grad") for g in grads]
    return d


def _both(handle, grads, inv_loss_scale=1.0, max_norm=1.0):
    d = _descs(grads)
    stream = torch.cuda.current_stream().cuda_stream
    a = torch.full((4,), float("nan"), device="cuda")
    b = torch.full((4,), float("nan"), device="cuda")
    handle.grad_norm(F._descs_ptr(d), len(d), inv_loss_scale, max_norm, a.data_ptr(), stream)
    handle.grad_norm_static(F._descs_ptr(d), len(d), inv_loss_scale, max_norm, b.data_ptr(), stream)
    torch.cuda.synchronize()
    return a.cpu().numpy().view(np.uint32)[:3], b.cpu().numpy().view(np.uint32)[:3]


def _make_grads(sizes, seed):
    gen = torch.Generator(device="cuda").manual_seed(seed)
    dts = (torch.bfloat16, torch.float32, torch.float16)
    grads = []
    for k, n in enumerate(sizes):
        dt = dts[k % 3]
        if k % 5 == 4 and n > 0:  # a view that starts 2 (or 4) bytes into its allocation: not 16-byte aligned
            base = torch.randn(n + 1, device="cuda", generator=gen).mul_(1e-3).to(dt)
            grads.append(base[1:])
        else:
            grads.append(torch.randn(n, device="cuda", generator=gen).mul_(1e-3).to(dt))
    return grads


def _ref_norm(grads, inv_loss_scale):
    tot = 0.0
    for g in grads:
        tot += float((g.double() * inv_loss_scale).square().sum())
    return tot ** 0.5


def test_static_grad_norm_matches_the_allocating_entry_point_twice_in_a_row():
    assert torch.cuda.is_available(), "this test needs the GPU"
    h = N.Handle(0)
    try:
        # first call: 300 gradients from 0 to 3 M elements, every dtype, whole chunks, tails, unaligned
        # views, more chunks than workgroups of the pass (so workgroups loop)
        rng = np.random.default_rng(7)
        sizes = [0, 1, 7, 8, 8191, 8192, 8193, 16384, 3 * 8192 + 5, 1 << 20, (3 << 20) + 17]
        sizes += [int(x) for x in np.floor(np.exp(rng.uniform(0, np.log(400_000), 289)))]
        grads = _make_grads(sizes, 11)
        # warm both paths up once so that the allocating one has its workspace, then measure memory
        _both(h, grads)
        d = _descs(grads)
        out = torch.zeros(4, device="cuda")
        torch.cuda.synchronize()
        free0, _ = torch.cuda.mem_get_info()
        h.grad_norm_static(F._descs_ptr(d), len(d), 1.0, 1.0, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        free1, _ = torch.cuda.mem_get_info()
        assert free1 == free0, "the static entry point changed the amount of free device memory"

        a, b = _both(h, grads, inv_loss_scale=1.0 / 1024.0, max_norm=1e-3)
        assert (a == b).all(), (a, b)
        norm = float(a[:1].view(np.float32)[0])
        ref = _ref_norm(grads, 1.0 / 1024.0)
        assert abs(norm - ref) <= 1e-6 * ref, (norm, ref)  # tolerance: 1e-6 relative (reduction order)
        assert a[2] == 0

        # second call, smaller input: what the first call left in the device array must not matter
        small = _make_grads([5, 8192, 100_003], 12)
        a2, b2 = _both(h, small, max_norm=0.5)
        assert (a2 == b2).all(), (a2, b2)
        ref2 = _ref_norm(small, 1.0)
        norm2 = float(b2[:1].view(np.float32)[0])
        assert abs(norm2 - ref2) <= 1e-6 * ref2, (norm2, ref2)

        # nothing to sum: norm 0, coefficient 1, flag clear -- same as the allocating entry point
        a3, b3 = _both(h, _make_grads([0, 0], 13))
        assert (a3 == b3).all() and float(b3[:1].view(np.float32)[0]) == 0.0

        # a non-finite gradient raises the flag in both
        bad = _make_grads([1000, 9000], 14)
        bad[1][17] = float("inf")
        a4, b4 = _both(h, bad)
        assert a4[2] == 1 and b4[2] == 1 and a4[1] == b4[1]

        # beyond the fixed table: refused with a clear error, nothing launched
        many = [torch.ones(1, device="cuda", dtype=torch.bfloat16) for _ in range(4097)]
        d = _descs(many)
        with pytest.raises(N.NativeError) as ei:
            h.grad_norm_static(F._descs_ptr(d), len(d), 1.0, 1.0, out.data_ptr(), 0)
        assert ei.value.code == N.RT_EUNSUPPORTED and "4096" in str(ei.value)
        # exactly at the limit it works
        a5, b5 = _both(h, many[:4096])
        assert (a5 == b5).all() and float(b5[:1].view(np.float32)[0]) == 64.0
    finally:
        torch.cuda.synchronize()
        h.close()


def test_static_grad_norm_calls_from_two_handles_and_streams_take_turns():
    """Two handles, each on a stream of its own, call the static entry point back to back without any
    synchronisation in between: both use the GPU's one array, and each call waits on the GPU for the one
    before it, so every result is the one the allocating entry point gives."""
    h1, h2 = N.Handle(0), N.Handle(0)
    try:
        s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
        sets = [_make_grads([200_000 + 8192 * k, 1 << 20, 77], 20 + k) for k in range(6)]
        want = []
        for g in sets:
            a, _ = _both(h1, g, max_norm=0.25)
            want.append(a)
        outs = [torch.full((4,), float("nan"), device="cuda") for _ in sets]
        ds = [_descs(g) for g in sets]
        torch.cuda.synchronize()
        for k, (d, out) in enumerate(zip(ds, outs)):
            h, s = ((h1, s1), (h2, s2))[k % 2]
            h.grad_norm_static(F._descs_ptr(d), len(d), 1.0, 0.25, out.data_ptr(), s.cuda_stream)
        torch.cuda.synchronize()
        for k, (out, a) in enumerate(zip(outs, want)):
            assert (out.cpu().numpy().view(np.uint32)[:3] == a).all(), k
    finally:
        torch.cuda.synchronize()
        h1.close()
        h2.close()
