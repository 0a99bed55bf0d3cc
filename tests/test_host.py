"""Host-side logic and the C-ABI surface.  No GPU needed, no compute calls."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest
import torch

import oracle
import ramtorch_amd
from ramtorch_amd import _native as N
from ramtorch_amd import functional as F

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "ramtorch_sr_adamw.h")


# ---- the shared library and its header ---------------------------------------------------
def test_library_loads_and_exports_every_declared_symbol():
    L = N.lib()
    assert L.rt_version() == N.ABI_VERSION
    text = open(HEADER).read()
    declared = set(re.findall(r"^\s*(?:int|const char\*)\s+(rt_\w+)\s*\(", text, flags=re.M))
    assert declared == set(N.EXPORTS), declared ^ set(N.EXPORTS)
    for name in declared:
        assert hasattr(L, name), f"{name} declared in the header but not exported"


def test_header_compiles_as_c_and_layouts_agree(tmp_path):
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "ramtorch_sr_adamw.h"\n'
        "int main(void){\n"
        'printf("%zu %zu\\n", sizeof(rt_scalars), sizeof(rt_tensor_desc));\n'
        + "".join(f'printf("d.{f} %zu\\n", offsetof(rt_tensor_desc, {f}));\n' for f, _ in N.RtTensorDesc._fields_)
        + "".join(f'printf("s.{f} %zu\\n", offsetof(rt_scalars, {f}));\n' for f, _ in N.RtScalars._fields_)
        + "return 0;}\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe)])
    lines = subprocess.check_output([str(exe)], text=True).split("\n")
    s_sz, d_sz = map(int, lines[0].split())
    assert s_sz == ctypes.sizeof(N.RtScalars) and d_sz == ctypes.sizeof(N.RtTensorDesc) == F.DESC_DTYPE.itemsize
    offs = dict(l.split() for l in lines[1:] if l)
    for f, _ in N.RtTensorDesc._fields_:
        assert int(offs["d." + f]) == getattr(N.RtTensorDesc, f).offset == F.DESC_DTYPE.fields[f][1], f
    for f, _ in N.RtScalars._fields_:
        assert int(offs["s." + f]) == getattr(N.RtScalars, f).offset, f


def test_errors_are_reported_without_a_gpu():
    L = N.lib()
    assert L.rt_step_multi(None, None, 0, None, 0, 0, 0, None, None, None) == N.RT_EINVAL
    assert b"handle" in L.rt_last_error()
    assert L.rt_sr_copy(None, None, 0, None, 0, None) == N.RT_OK  # empty copy is a no-op
    assert L.rt_sr_copy(None, None, 8, None, 0, None) == N.RT_EINVAL
    h = ctypes.c_void_p()
    rc = L.rt_create(0, ctypes.byref(h))
    if not torch.cuda.is_available():
        assert rc != N.RT_OK and L.rt_last_error() != b""
    with pytest.raises(N.NativeError):
        N.check(N.RT_EINVAL)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(N, "_lib", None)
    monkeypatch.setattr(N, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        N.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "ramtorch_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
                assert "liboracle" not in text, f


# ---- scalars -----------------------------------------------------------------------------
@pytest.mark.parametrize("hp,step", [
    (dict(lr=1e-4, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), 10),
    (dict(lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.01), 1),
    (dict(lr=2.5e-3, betas=(0.8, 0.9999), eps=1e-10, weight_decay=0.0), 5000),
])
def test_make_scalars_agrees_with_oracle_and_known_bits(hp, step):
    a = F.make_scalars(step=step, **hp)
    b = oracle.scalars_from_hparams(step=step, **hp)
    for f in ("beta1", "one_m_beta1", "beta2", "one_m_beta2", "inv_bcs", "eps", "neg_step_size", "apply_decay"):
        assert getattr(a, f) == getattr(b, f), f
    if hp["weight_decay"] != 0:
        assert a.decay == b.decay
    else:
        assert a.decay == 1.0 and a.apply_decay == 0
    if step == 10:
        bits = lambda x: int(np.float32(x).view(np.uint32))
        assert bits(a.inv_bcs) == 0x41205C3A and bits(a.neg_step_size) == 0xB920FDF8 and bits(a.decay) == 0x3F7FFFE6


# ---- optimizer interface (adamw.py:57-104) -------------------------------------------------
def _params(dtype=torch.bfloat16):
    return [torch.nn.Parameter(torch.zeros(4, 6, dtype=dtype)), torch.nn.Parameter(torch.zeros(5, dtype=dtype))]


def test_constructor_defaults_and_state_layout():
    ps = _params()
    opt = ramtorch_amd.AdamW(ps)
    g = opt.param_groups[0]
    assert (g["lr"], g["betas"], g["eps"], g["weight_decay"], g["centralization"]) == (1e-3, (0.9, 0.999), 1e-8, 1e-2, 0)
    assert opt.chunk_size == 64 and opt.optim_state_dtype == torch.bfloat16 and opt.optim_state_device == "cpu"
    for p in ps:
        st = opt.state[p]
        assert set(st) == {"step", "ema", "ema_squared"}
        assert st["step"] == 0 and isinstance(st["step"], int)
        for k in ("ema", "ema_squared"):
            assert st[k].shape == p.shape and st[k].dtype == torch.bfloat16 and st[k].device.type == "cpu"
            assert not st[k].any()


def test_state_dtype_and_positional_signature():
    ps = _params(torch.float32)
    opt = ramtorch_amd.AdamW(ps, 3e-4, (0.95, 0.99), 1e-6, 0.1, 0, 16, torch.float32, "cpu")
    assert opt.state[ps[0]]["ema"].dtype == torch.float32 and opt.chunk_size == 16
    assert opt.param_groups[0]["betas"] == (0.95, 0.99)


def test_param_groups_from_zero1_style_lists_with_empty_groups():
    ps = _params()
    groups = [{"params": [ps[0]], "lr": 1e-3, "weight_decay": 0.01}, {"params": [], "lr": 5e-4, "weight_decay": 0.0},
              {"params": [ps[1]], "lr": 5e-4}]
    opt = ramtorch_amd.AdamW(groups)
    assert [len(g["params"]) for g in opt.param_groups] == [1, 0, 1]
    assert opt.param_groups[2]["weight_decay"] == 1e-2 and opt.param_groups[1]["lr"] == 5e-4
    assert opt._tensor_ids() == {id(ps[0]): 0, id(ps[1]): 1}


def test_state_dict_round_trip_keeps_reference_keys():
    ps = _params()
    opt = ramtorch_amd.AdamW(ps, lr=2e-3)
    opt.state[ps[0]]["step"] = 7
    opt.state[ps[0]]["ema"].fill_(0.5)
    sd = opt.state_dict()
    assert set(sd) == {"state", "param_groups", "ramtorch_amd"}
    assert set(sd["state"][0]) == {"step", "ema", "ema_squared"}
    opt2 = ramtorch_amd.AdamW(_params(), lr=1e-3)
    opt2.load_state_dict(sd)
    p0 = opt2.param_groups[0]["params"][0]
    assert opt2.state[p0]["step"] == 7 and opt2.param_groups[0]["lr"] == 2e-3
    assert torch.equal(opt2.state[p0]["ema"], torch.full((4, 6), 0.5, dtype=torch.bfloat16))


def test_load_state_dict_keeps_state_dtype_device_and_seed():
    ps = [torch.nn.Parameter(torch.zeros(8, dtype=torch.bfloat16))]
    a = ramtorch_amd.AdamW(ps, dtype=torch.float32, seed=77)
    a.state[ps[0]]["ema_squared"].fill_(1.0 + 2.0 ** -20)      # not representable in bf16
    a.state[ps[0]]["step"] = 3
    sd = a.state_dict()
    assert sd["ramtorch_amd"] == {"seed": 77} and set(sd["state"][0]) == {"step", "ema", "ema_squared"}
    b = ramtorch_amd.AdamW([torch.nn.Parameter(torch.zeros(8, dtype=torch.bfloat16))], dtype=torch.float32)
    b.load_state_dict(sd)
    st = b.state[b.param_groups[0]["params"][0]]
    assert st["ema_squared"].dtype == torch.float32 and st["ema_squared"].device.type == "cpu"
    assert float(st["ema_squared"][0]) == 1.0 + 2.0 ** -20 and st["step"] == 3 and b.seed == 77
    assert st["ema_squared"].data_ptr() != a.state[ps[0]]["ema_squared"].data_ptr()   # a copy, not an alias
    # a checkpoint written by the reference (no extra entry) loads and keeps the current seed
    del sd["ramtorch_amd"]
    c = ramtorch_amd.AdamW([torch.nn.Parameter(torch.zeros(8, dtype=torch.bfloat16))], seed=5)
    c.load_state_dict(sd)
    assert c.seed == 5
    # and torch's own loader accepts ours
    torch.optim.SGD([torch.nn.Parameter(torch.zeros(8))], lr=0.1).state_dict()


def test_step_without_gpu_raises_and_leaves_state_alone():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    ps = _params()
    opt = ramtorch_amd.AdamW(ps)
    ps[0].grad = torch.ones_like(ps[0])
    with pytest.raises(RuntimeError, match="GPU"):
        opt.step()
    assert opt.state[ps[0]]["step"] == 0
    with pytest.raises(RuntimeError):
        ramtorch_amd.copy_stochastic_(torch.zeros(4, dtype=torch.bfloat16), torch.zeros(4))


def test_zero_grad_and_add_param_group_are_inherited():
    ps = _params()
    opt = ramtorch_amd.AdamW([ps[0]])
    ps[0].grad = torch.ones_like(ps[0])
    opt.zero_grad()
    assert ps[0].grad is None
    opt.add_param_group({"params": [ps[1]], "lr": 1e-5})
    assert len(opt.param_groups) == 2 and opt.param_groups[1]["betas"] == (0.9, 0.999)
    assert opt._tensor_ids()[id(ps[1])] == 1


# ---- descriptor packing ---------------------------------------------------------------------
def test_pack_descs_rejects_bad_inputs():
    t = lambda n, dt=torch.bfloat16: torch.zeros(n, dtype=dt)
    e = F.Entry(p=t(8), g=t(8), m=t(8), v=t(8), step=1, scalars_idx=0, tensor_id=0)
    with pytest.raises(ValueError, match="CPU tensor"):
        F.pack_descs([e], streamed=False)
    d = F.pack_descs([e], streamed=True)
    assert d["host_mask"][0] == 15 and d["numel"][0] == 8 and d["p"][0] == e.p.data_ptr()
    e.ordered = True   # host arrays the caller's stream may still be filling: uploads must wait for it
    assert F.pack_descs([e], streamed=True)["host_mask"][0] == 15 | N.RT_HOST_ORDERED == 31
    with pytest.raises(ValueError, match="element counts"):
        F.pack_descs([F.Entry(p=t(8), g=t(9), m=t(8), v=t(8), step=1, scalars_idx=0, tensor_id=0)], streamed=True)
    # fp16 / fp64 params and states are valid (plain copy_ on write-back, adamw.py:208-222) ...
    d = F.pack_descs([F.Entry(p=t(8, torch.float16), g=t(8), m=t(8, torch.float64), v=t(8, torch.float32), step=1,
                              scalars_idx=0, tensor_id=0)], streamed=True)
    assert (d["p_dtype"][0], d["g_dtype"][0], d["m_dtype"][0], d["v_dtype"][0]) == (2, 0, 3, 1)
    # ... other dtypes are not, and neither is an fp64 gradient at this level (AdamW.step downcasts it first)
    with pytest.raises(NotImplementedError):
        F.pack_descs([F.Entry(p=t(8, torch.int16), g=t(8), m=t(8), v=t(8), step=1, scalars_idx=0, tensor_id=0)],
                     streamed=True)
    with pytest.raises(NotImplementedError):
        F.pack_descs([F.Entry(p=t(8), g=t(8, torch.float64), m=t(8), v=t(8), step=1, scalars_idx=0, tensor_id=0)],
                     streamed=True)
    with pytest.raises(ValueError, match="contiguous"):
        F.pack_descs([F.Entry(p=torch.zeros(4, 4, dtype=torch.bfloat16).t(), g=t(16), m=t(16), v=t(16), step=1,
                              scalars_idx=0, tensor_id=0)], streamed=True)


def test_build_module_knows_its_sources():
    from ramtorch_amd import build
    for s in build.SOURCES:
        assert os.path.exists(os.path.join(build.CSRC, s))
    assert "--offload-arch=gfx950" in build.HIPCC_FLAGS and "-ffp-contract=off" in build.HIPCC_FLAGS
    i = build.HIPCC_FLAGS.index("-packed-fp32-ops")
    assert build.HIPCC_FLAGS[i - 3:i] == ["-Xclang", "-target-feature", "-Xclang"]


# ---- chunk schedule of the streamed path (pure host logic) -----------------------------------
@pytest.mark.parametrize("chunk_elems", [8, 64, 8192, 100_000, 1 << 27])
def test_streamed_chunk_schedule_covers_every_element_once(chunk_elems):
    rng = np.random.default_rng(chunk_elems)
    lens = [0, 1, 7, 8, 9, 4096, 8191, 8193, 250_007, 16, 0, 5] + [int(x) for x in rng.integers(1, 50_000, 20)]
    d = np.zeros(len(lens), F.DESC_DTYPE)
    d["numel"] = lens
    plan = N.streamed_plan(d.ctypes.data_as(ctypes.POINTER(N.RtTensorDesc)), len(lens), chunk_elems)
    covered = [0] * len(lens)
    per_chunk = {}
    last = (-1, -1)
    for chunk, tensor, start, count, off in plan:
        assert count > 0 and start % 8 == 0 and off % 8 == 0          # Philox blocks and 16-byte alignment
        assert start == covered[tensor], "pieces of a tensor must be consecutive"
        assert (chunk, tensor) >= last                                  # tensors in order, chunks in order
        last = (chunk, tensor)
        covered[tensor] += count
        lo, hi = per_chunk.get(chunk, (0, 0))
        assert off >= hi, "pieces overlap inside the staging buffer"
        per_chunk[chunk] = (lo, off + count)
        assert off + count <= chunk_elems
    assert covered == lens
    assert sorted(per_chunk) == list(range(len(per_chunk)))
    # no chunk but the last may be left mostly empty: a new chunk starts only when the previous one is full
    for c in sorted(per_chunk)[:-1]:
        assert per_chunk[c][1] > chunk_elems - 8


def test_streamed_plan_rejects_bad_chunk_size():
    d = np.zeros(1, F.DESC_DTYPE)
    with pytest.raises(N.NativeError):
        N.streamed_plan(d.ctypes.data_as(ctypes.POINTER(N.RtTensorDesc)), 1, 12)


# ---- the C++ descriptor gatherer (host logic only; CPU tensors stand in with dev = -1) ----------
def test_gatherer_writes_the_rows_the_python_loop_would():
    from ramtorch_amd import _gather as G
    g = G.module()
    if g is None:
        pytest.skip("gather helper not built")
    n = 300
    ps = [torch.nn.Parameter(torch.zeros(7 + i % 5, dtype=torch.bfloat16 if i % 2 else torch.float32)) for i in range(n)]
    sts = [{"step": i % 3, "ema": torch.zeros_like(p), "ema_squared": torch.zeros_like(p, dtype=torch.float32)}
           for i, p in enumerate(ps)]
    for i, p in enumerate(ps):
        if i % 7:
            p.grad = torch.ones_like(p)  # torch only stores a gradient of the parameter's own dtype
    sts[5] = {}                                                # state not initialised -> Python
    sts[9]["ema"] = torch.zeros(3, dtype=torch.bfloat16)       # size mismatch -> Python
    sts[10]["ema_squared"] = torch.zeros(4, 3).t()[:, :3]      # not contiguous -> Python
    sts[11]["step"] = torch.tensor(4)                          # step is not a plain int -> Python
    ps[12] = torch.nn.Parameter(torch.zeros(5, dtype=torch.float64))
    ps[12].grad = torch.ones_like(ps[12])                      # fp64 gradient -> Python (downcast there)
    sts[13]["ema"] = torch.zeros(ps[13].numel(), dtype=torch.int16)  # unsupported dtype -> Python
    old = [st.get("step") for st in sts]
    buf = np.zeros(n, F.DESC_DTYPE)
    stat = np.full(n, 255, np.uint8)
    rows, steps = g.gather_group(ps, sts, -1, buf.ctypes.data, n, stat.ctypes.data, 4, 100)
    assert sorted(steps) == [1, 2, 3]
    for i in (5, 9, 10, 11, 12, 13):
        assert stat[i] == g.PYTHON and (sts[i].get("step") is old[i])
    code = {torch.bfloat16: 0, torch.float32: 1, torch.float16: 2}
    j = 0
    for i, p in enumerate(ps):
        if p.grad is None:
            assert stat[i] == g.NO_GRAD and sts[i].get("step") == old[i]  # adamw.py:114: no step increment
            continue
        if stat[i] == g.PYTHON:
            continue
        d, st = buf[j], sts[i]
        j += 1
        assert stat[i] == g.WRITTEN and st["step"] == old[i] + 1
        assert (d["p"], d["g"], d["m"], d["v"]) == (p.data_ptr(), p.grad.data_ptr(), st["ema"].data_ptr(),
                                                    st["ema_squared"].data_ptr())
        assert d["numel"] == p.numel() and d["tensor_id"] == 100 + i and d["step"] == st["step"]
        assert d["scalars_idx"] == 4 + steps.index(st["step"])
        assert (d["p_dtype"], d["g_dtype"], d["m_dtype"], d["v_dtype"]) == (code[p.dtype], code[p.grad.dtype],
                                                                             code[p.dtype], 1)
        assert d["host_mask"] == 0 and d["elem_offset"] == 0 and d["noise_p"] == 0 and d["row_mean"] == 0
    assert j == rows
    # capacity is respected: what does not fit is left to Python, untouched
    old = [st.get("step") for st in sts]
    rows2, _ = g.gather_group(ps, sts, -1, buf.ctypes.data, 10, stat.ctypes.data, 0, 0)
    assert rows2 == 10 and int((stat == g.WRITTEN).sum()) == 10
    assert sum(st.get("step") != o for st, o in zip(sts, old)) == 10
    # a tensor subclass is never touched
    class T(torch.Tensor):
        pass
    sub = torch.zeros(4).as_subclass(T)
    rows3, _ = g.gather_group([sub], [{"step": 0, "ema": torch.zeros(4), "ema_squared": torch.zeros(4)}], -1,
                              buf.ctypes.data, 10, stat.ctypes.data, 0, 0)
    assert rows3 == 0 and stat[0] == g.PYTHON


def test_state_layout_options_are_validated_and_harmless_on_cpu():
    ps = [torch.nn.Parameter(torch.zeros(16, dtype=torch.bfloat16))]
    with pytest.raises(ValueError, match="state_placement"):
        ramtorch_amd.AdamW(ps, state_placement="somewhere")
    with pytest.raises(ValueError, match="noise_source"):
        ramtorch_amd.AdamW(ps, noise_source="dice")
    opt = ramtorch_amd.AdamW(ps, ema_squared_dtype=torch.float32)  # bf16 ema, fp32 ema_squared
    st = opt.state[ps[0]]
    assert st["ema"].dtype == torch.bfloat16 and st["ema_squared"].dtype == torch.float32
    assert opt.state_placement == "auto" and opt.state_placement_report is None and not opt._state_pools


def test_copies_and_unpickled_optimizers_keep_their_configuration():
    import copy
    import pickle
    ps = [torch.nn.Parameter(torch.zeros(16, dtype=torch.bfloat16))]
    opt = ramtorch_amd.AdamW(ps, seed=7, loss_scale=4.0, max_grad_norm=1.5, noise_source="reference",
                             ema_squared_dtype=torch.float32, state_placement="plain", chunk_size=3)
    opt.max_inflight_calls = 5
    for other in (copy.deepcopy(opt), pickle.loads(pickle.dumps(opt))):
        assert (other.seed, other.loss_scale, other.max_grad_norm, other.noise_source) == (7, 4.0, 1.5, "reference")
        assert other.ema_squared_dtype == torch.float32 and other.optim_state_dtype == torch.bfloat16
        assert other.state_placement == "plain" and other.chunk_size == 3 and other.max_inflight_calls == 5
        assert other._stepped_early == set() and other._inflight == [] and other._recs is None
        q = other.param_groups[0]["params"][0]
        assert other.state[q]["ema_squared"].dtype == torch.float32 and other.state[q]["step"] == 0
    # load_state_dict goes through __setstate__ too and must leave the live configuration alone
    opt.load_state_dict(copy.deepcopy(opt.state_dict()))
    assert opt.max_inflight_calls == 5 and opt.loss_scale == 4.0


def test_layout_check_notices_every_kind_of_change():
    """verify_layout (the per-step check of a recorded layout) on CPU tensors: true while nothing moved,
    false for a moved / new / vanished / retyped / non-contiguous gradient and for a moved parameter."""
    from ramtorch_amd import _gather as G
    g = G.module()
    if g is None or not hasattr(g, "verify_layout"):
        pytest.skip("gather helper not built")
    from ramtorch_amd import _native as N
    ps = [torch.nn.Parameter(torch.zeros(6, 4, dtype=torch.bfloat16)) for _ in range(40)]
    for i, p in enumerate(ps):
        if i % 7:
            p.grad = torch.ones(6, 4, dtype=torch.bfloat16)

    def record():
        e = np.zeros((len(ps), 3), np.uint64)
        for i, p in enumerate(ps):
            e[i, 0] = p.data_ptr()
            if p.grad is not None:
                e[i, 1] = p.grad.data_ptr()
                e[i, 2] = {torch.bfloat16: N.RT_DT_BF16, torch.float32: N.RT_DT_F32, torch.float16: N.RT_DT_F16}[p.grad.dtype]
        return e

    def check(e):
        return g.verify_layout(ps, e.ctypes.data, len(ps))

    e = record()
    assert check(e) is True
    ps[3].grad.add_(1)                       # in-place accumulation keeps the layout
    assert check(e) is True
    keep = ps[3].grad
    ps[3].grad = torch.ones(6, 4, dtype=torch.bfloat16)   # a new gradient tensor
    assert check(e) is False
    ps[3].grad = keep
    assert check(e) is True
    ps[0].grad = torch.ones(6, 4, dtype=torch.bfloat16)   # index 0 had none
    assert check(e) is False
    ps[0].grad = None
    ps[5].grad = None                        # one vanished
    assert check(e) is False
    e = record()
    assert check(e) is True
    e2 = e.copy()
    e2[8, 2] = N.RT_DT_F32                   # recorded with another dtype
    assert check(e2) is False
    base = torch.ones(4, 6, dtype=torch.bfloat16)
    ps[9].grad = base.t()                    # same storage as a contiguous tensor would have, other strides
    e3 = record()
    assert check(e3) is False
    ps[9].grad = torch.ones(6, 4, dtype=torch.bfloat16)
    e = record()
    ps[2].data = torch.zeros(6, 4, dtype=torch.bfloat16)  # the parameter moved
    assert check(e) is False
    assert g.verify_layout(ps[:-1], e.ctypes.data, len(ps)) is False   # list length differs


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it exits with a message instead of a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                         capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert "ONE GPU" in res.stderr and res.stdout.strip() == ""


def test_copy_pool_copies_every_byte_and_waits_per_group(tmp_path):
    """The host threads that fill the streamed path's bounce buffers (csrc/copy_pool.h): many groups
    of copies of odd sizes submitted at once, each waited for on its own, compared byte for byte;
    waiting on a group with nothing in it returns; the pool shuts down with idle workers."""
    src = tmp_path / "pool.cpp"
    src.write_text(r'''
#include "copy_pool.h"
#include <cstdio>
#include <random>
int main() {
    std::mt19937_64 rng(7);
    const size_t sizes[] = {0, 1, 63, 4096, (2u << 20) - 1, (2u << 20), (2u << 20) + 1, 9u << 20};
    std::vector<std::vector<uint8_t>> from, to;
    for (int rep = 0; rep < 3; ++rep)
        for (size_t n : sizes) {
            from.emplace_back(n);
            to.emplace_back(n, (uint8_t)0);
            for (auto& b : from.back()) b = (uint8_t)rng();
        }
    {
        rt::CopyPool pool(5);
        std::vector<rt::CopyPool::Group> groups(from.size());
        rt::CopyPool::Group empty;
        pool.wait(&empty);
        for (size_t i = 0; i < from.size(); ++i) pool.submit(&groups[i], to[i].data(), from[i].data(), from[i].size());
        for (size_t i = from.size(); i-- > 0;) {  // waited for in the opposite order
            pool.wait(&groups[i]);
            if (to[i] != from[i]) { std::printf("group %zu differs\n", i); return 1; }
        }
    }
    { rt::CopyPool idle(3); }
    std::printf("ok\n");
    return 0;
}
''')
    exe = tmp_path / "pool"
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-pthread", "-fsanitize=thread",
                           "-I", os.path.join(ROOT, "ramtorch_amd", "csrc"), str(src), "-o", str(exe)])
    assert subprocess.check_output([str(exe)], text=True).strip() == "ok"


# ---- the streamed pipeline's order of operations, replayed on the CPU ---------------------------------
# rt_streamed_schedule hands out the very list of operations the library executes for a streamed call
# (three streams, two staging buffers per array, four bounce slots each way, events, host waits).  The
# replay below runs such lists as the hardware may: the host issues operations in order and blocks where
# the list says it waits; every stream runs its operations in order, each starting no earlier than the
# event it waits for; host copies run beside all of that; which of the possible next things happens is
# drawn at random.  Two things are checked at every start of an operation: nothing else that is running
# touches a buffer it writes (or writes one it reads), and every buffer it reads holds what it is
# supposed to hold.  The reference keeps its transfers apart with ping-pong buffers and events
# (ramtorch/modules/linear.py:163-197, 267-308) and device-wide syncs (adamw.py:227-232).
class _Replay:
    def __init__(self, calls, rng):
        """calls: [(ops, seq0)] executed back to back on one handle."""
        self.rng = rng
        self.calls = calls
        self.violations = []
        self.content = {}            # buffer -> tag of what it holds
        self.running = []            # [name, reads, writes, on_finish]
        self.queues = {s: [] for s in ("h2d", "comp", "d2h")}   # issued, not yet started: (op, awaited record or None, abs chunk)
        self.stream_busy = {s: None for s in self.queues}
        self.records = {}            # event id -> index of its most recent record among the issued ones
        self.record_done = set()     # (event id, index) of completed records
        self.record_count = {}
        self.back = 0                # the published chunk counter
        self.copies = {}             # ("fill" | "drain", abs chunk) -> running entry or "done"
        speeds = [0.02, 1.0, 50.0]
        self.weight = {k: speeds[rng.integers(3)] for k in ("host", "start", "finish", "copy")}
        self.stream_weight = {s: speeds[rng.integers(3)] for s in ("h2d", "comp", "d2h")}
        self._copy_weight = {}

    def copy_weight(self, key):
        if key not in self._copy_weight:     # every host copy has a speed of its own
            self._copy_weight[key] = [0.02, 1.0, 50.0][self.rng.integers(3)]
        return self._copy_weight[key]

    def _conflict(self, name, reads, writes):
        for other, oreads, owrites, *_ in self.running:
            for b in writes:
                if b in oreads or b in owrites:
                    self.violations.append(f"{name} writes {b} while {other} uses it")
            for b in reads:
                if b in owrites:
                    self.violations.append(f"{name} reads {b} while {other} writes it")

    def _expect(self, name, buf, tag):
        if self.content.get(buf) != tag:
            self.violations.append(f"{name} finds {self.content.get(buf)} in {buf}, not {tag}")

    def _start(self, name, reads, writes, expects, results):
        self._conflict(name, reads, writes)
        for buf, tag in expects:
            self._expect(name, buf, tag)
        for buf in writes:
            self.content[buf] = ("being written by", name)
        entry = [name, set(reads), set(writes), results]
        self.running.append(entry)
        return entry

    def _finish(self, entry):
        self.running.remove(entry)
        for buf, tag in entry[3]:
            self.content[buf] = tag

    def run(self, paced_up, paced_down):
        K = N
        stream_of = {K.RT_OP_H2D: "h2d", K.RT_OP_KERNEL: "comp", K.RT_OP_D2H: "d2h", K.RT_OP_PUBLISH: "d2h", K.RT_OP_TICKET: "d2h"}
        flat = [(op, seq0) for ops, seq0 in self.calls for op in ops]
        pc = 0
        steps = 0
        while True:
            steps += 1
            assert steps < 200000, "the replay does not end"
            actions = []
            # -- the host: issue the next operation, unless it has to wait
            if pc < len(flat):
                op, seq0 = flat[pc]
                c = seq0 + op.chunk
                if op.kind == K.RT_OP_HOST_WAIT_BACK:
                    if self.back >= op.value:
                        actions.append(("host", None))
                elif op.kind == K.RT_OP_HOST_WAIT_FILL:
                    if self.copies.get(("fill", c), "done") == "done":
                        actions.append(("host", None))
                elif op.kind == K.RT_OP_HOST_WAIT_DRAIN:
                    if self.copies.get(("drain", c), "done") == "done":
                        actions.append(("host", None))
                elif op.kind == K.RT_OP_HOST_WAIT_IDLE:
                    if not any(self.queues.values()) and not any(self.stream_busy.values()):
                        actions.append(("host", None))
                else:
                    actions.append(("host", None))
            # -- streams: start the head operation when its event has fired; finish what runs
            for s, q in self.queues.items():
                if self.stream_busy[s] is not None:
                    actions.append(("finish", s))
                elif q:
                    op, awaited, c = q[0]
                    if awaited is None or awaited in self.record_done:
                        actions.append(("start", s))
            for key, entry in self.copies.items():
                if entry != "done":
                    actions.append(("copy", key))
            if not actions:
                assert pc >= len(flat) and not any(self.queues.values()), "the replay is stuck: a wait that nothing satisfies"
                return self.violations
            # Which of them happens: drawn with weights that differ from replay to replay by orders of
            # magnitude (a host far ahead of the device, copies that crawl, a stream that stalls ...)
            w = np.array([self.weight[a[0]] * (self.copy_weight(a[1]) if a[0] == "copy" else self.stream_weight.get(a[1], 1.0))
                          for a in actions])
            kind, arg = actions[self.rng.choice(len(actions), p=w / w.sum())]
            if kind == "host":
                op, seq0 = flat[pc]
                pc += 1
                if pc == len(flat):    # the call returns to its caller: host memory must be final
                    for key, entry in self.copies.items():
                        if entry != "done":
                            self.violations.append(f"the call returns while {key} is still copying")
                c = seq0 + op.chunk
                if op.kind == K.RT_OP_HOST_FILL:
                    e = self._start(f"fill({c})", [("user", c)], [("up", op.bounce)], [], [(("up", op.bounce), ("chunk", c))])
                    self.copies[("fill", c)] = e
                elif op.kind == K.RT_OP_HOST_DRAIN:
                    e = self._start(f"drain({c})", [("down", op.bounce)], [("user", c)], [(("down", op.bounce), ("result", c))],
                                    [(("user", c), ("result", c))])
                    self.copies[("drain", c)] = e
                elif op.kind in stream_of:
                    awaited = None
                    if op.wait_event != K.RT_SCHED_NONE and op.wait_event in self.records:
                        awaited = (op.wait_event, self.records[op.wait_event])
                    if op.record_event != K.RT_SCHED_NONE:
                        k = self.record_count.get(op.record_event, 0)
                        self.record_count[op.record_event] = k + 1
                        self.records[op.record_event] = k
                        op_record = (op.record_event, k)
                    else:
                        op_record = None
                    self.queues[stream_of[op.kind]].append(((op, op_record), awaited, c))
            elif kind == "start":
                (op, op_record), _, c = self.queues[arg].pop(0)
                stage = ("stage", op.stage)
                if op.kind == K.RT_OP_H2D:
                    src = ("up", op.bounce) if op.bounce != K.RT_SCHED_NONE else ("user", c)
                    expects = [(src, ("chunk", c))] if op.bounce != K.RT_SCHED_NONE else []
                    e = self._start(f"h2d({c})", [src], [stage], expects, [(stage, ("chunk", c))])
                elif op.kind == K.RT_OP_KERNEL:
                    e = self._start(f"kernel({c})", [stage], [stage], [(stage, ("chunk", c))], [(stage, ("result", c))])
                elif op.kind == K.RT_OP_D2H:
                    dst = ("down", op.bounce) if op.bounce != K.RT_SCHED_NONE else ("user", c)
                    e = self._start(f"d2h({c})", [stage], [dst], [(stage, ("result", c))], [(dst, ("result", c))])
                else:
                    e = self._start("publish", [], [], [], [])
                    e.append(op)
                self.stream_busy[arg] = (e, op_record)
            elif kind == "finish":
                e, op_record = self.stream_busy[arg]
                self.stream_busy[arg] = None
                self._finish(e)
                if op_record is not None:
                    self.record_done.add(op_record)
                if len(e) > 4 and e[4].kind == K.RT_OP_PUBLISH:
                    self.back = max(self.back, e[4].value)
            else:
                e = self.copies[arg]
                self._finish(e)
                self.copies[arg] = "done"


def _two_calls(n1, n2, paced_up, paced_down, batch=3):
    """Two streamed calls on one handle, the second chained behind the first as the library chains them."""
    a = N.streamed_schedule(n1, 0, 0, paced_up, paced_down, batch)
    used = (1 if n1 >= 1 else 0) | (2 if n1 >= 2 else 0)     # staging buffers 0 and 1 hold chunks of the first call
    b = N.streamed_schedule(n2, n1, used, paced_up, paced_down, batch)
    return [(a, 0), (b, n1)]


@pytest.mark.parametrize("paced_up,paced_down", [(False, False), (True, False), (True, True), (False, True)])
def test_streamed_schedule_keeps_buffers_apart_under_any_interleaving(paced_up, paced_down):
    for n1, n2 in ((1, 1), (2, 3), (5, 4), (9, 7)):
        calls = _two_calls(n1, n2, paced_up, paced_down)
        for seed in range(60):
            bad = _Replay(calls, np.random.default_rng(seed)).run(paced_up, paced_down)
            assert not bad, (n1, n2, seed, bad[:3])
        # every chunk went through all three stages exactly once, in chunk order on every stream
        for ops, _ in calls:
            for kind in (N.RT_OP_H2D, N.RT_OP_KERNEL, N.RT_OP_D2H):
                assert [o.chunk for o in ops if o.kind == kind] == list(range(len([o for o in ops if o.kind == N.RT_OP_H2D])))
            assert [o.kind for o in ops].count(N.RT_OP_TICKET) == 1


def _without(ops, index):
    """The schedule with one wait taken out: a stream operation loses its event, a host wait disappears."""
    out = []
    for i, o in enumerate(ops):
        if i != index:
            out.append(o)
        elif o.kind in (N.RT_OP_H2D, N.RT_OP_KERNEL, N.RT_OP_D2H):
            c = N.RtSchedOp.from_buffer_copy(o)
            c.wait_event = N.RT_SCHED_NONE
            out.append(c)
    return out


@pytest.mark.parametrize("paced_up,paced_down", [(False, False), (True, True)])
def test_streamed_schedule_replay_notices_a_missing_wait(paced_up, paced_down):
    """The check has teeth: take any single wait that protects a buffer out of the list and some interleaving
    shows the damage.  (The waits of a long unpaced call between its batches of chunks only keep the
    streams' queues short; nothing is unsafe without them, and they are left out here.)"""
    ops = N.streamed_schedule(8, 0, 0, paced_up, paced_down, 64)
    # (paced, an upload's wait for its staging buffer is implied by the host's own wait for that chunk to
    # have come back, two chunks earlier; it stays in the list because asynchronous calls chain on it)
    evented = (N.RT_OP_KERNEL, N.RT_OP_D2H) if (paced_up or paced_down) else (N.RT_OP_H2D, N.RT_OP_KERNEL, N.RT_OP_D2H)
    waits = [i for i, o in enumerate(ops)
             if (o.kind in evented and o.wait_event != N.RT_SCHED_NONE)
             or o.kind in (N.RT_OP_HOST_WAIT_BACK, N.RT_OP_HOST_WAIT_FILL, N.RT_OP_HOST_WAIT_DRAIN)]   # (a single call: nothing before it to wait for)
    assert len(waits) >= 20
    for i in waits:
        broken = _without(ops, i)
        caught = False
        for seed in range(300):
            try:
                bad = _Replay([(broken, 0)], np.random.default_rng(seed)).run(paced_up, paced_down)
            except AssertionError:     # a replay that cannot end is a broken schedule too
                bad = ["stuck"]
            if bad:
                caught = True
                break
        assert caught, (i, ops[i].kind, ops[i].chunk)


def test_recorded_layout_keeps_its_step_counts_in_step_with_the_states():
    """Bringing the lagging step counts of a recorded layout up to date (state_dict(), pickling) must move
    the recorded counts along: the next recorded step builds its bias corrections from them."""
    from ramtorch_amd import _gather as G
    if G.module() is None:
        pytest.skip("the gather helper is not built")
    p = torch.nn.Parameter(torch.zeros(8, dtype=torch.bfloat16))
    opt = ramtorch_amd.AdamW([p], storage_device="cpu")
    st = opt.state[p]
    st["step"] = 2
    dicts = [st, opt.state]
    versions = np.zeros(2, np.uint64)
    G.module().dict_versions(dicts, versions.ctypes.data, 2)
    opt._frozen = {"pending": 3, "states": [st], "keys": [(0, 2)], "state_dicts": dicts, "versions": versions}
    opt._materialize_frozen_steps()
    assert st["step"] == 5 and opt._frozen["keys"] == [(0, 5)] and opt._frozen["pending"] == 0
    # the optimizer's own writes do not count as somebody else's: the stamps were taken again
    assert G.module().verify_versions(dicts, versions.ctypes.data, 2)
    st["ema"] = st["ema"].clone()            # somebody else's does
    assert not G.module().verify_versions(dicts, versions.ctypes.data, 2)
    opt._frozen = None
