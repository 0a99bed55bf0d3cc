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
