// Host-side helper of AdamW.step for parameter sets with very many tensors: walks one
// param group and writes the rt_tensor_desc rows of every "plain" tensor (param, gradient
// and both states contiguous on one GPU, supported dtypes) straight into a caller-owned
// buffer, advancing state["step"] as adamw.py:177 does.  It does, per tensor, what the Python
// loop of AdamW.step does (the checks of adamw.py:112-119 and the lazy-state test of
// adamw.py:125), only without ~2 us of interpreter and binding overhead per tensor; whatever
// is not plain is handed back to that Python loop untouched.
//
// A CPython extension that reads torch tensors through torch's C++ API.  It moves no tensor
// data and launches nothing: the update itself runs behind the C ABI of
// include/ramtorch_sr_adamw.h.  Optional: AdamW.step works without it.
#include <Python.h>

#include <torch/csrc/autograd/python_variable.h>
#include <ATen/core/Tensor.h>

#include <cstdint>
#include <algorithm>
#include <cstring>
#include <thread>
#include <vector>

#include "../../include/ramtorch_sr_adamw.h"

static_assert(sizeof(rt_tensor_desc) == 136, "rt_tensor_desc layout");

namespace {

PyObject* k_ema = nullptr;
PyObject* k_ema_squared = nullptr;
PyObject* k_step = nullptr;
PyTypeObject* t_tensor = nullptr;     // torch.Tensor
PyTypeObject* t_parameter = nullptr;  // torch.nn.Parameter

enum Status : uint8_t {
    kWritten = 0,  // row written, state["step"] advanced
    kNoGrad = 1,   // grad is None: skipped, step not advanced (adamw.py:114)
    kPython = 2,   // not plain (or not initialised yet): the Python loop handles it
};

inline bool exact_tensor(PyObject* o) {
    PyTypeObject* t = Py_TYPE(o);
    return t == t_tensor || t == t_parameter;
}

// dtype code of a param / state (bf16, f32, f16, f64) or -1
inline int pmv_code(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kBFloat16: return RT_DT_BF16;
        case at::kFloat: return RT_DT_F32;
        case at::kHalf: return RT_DT_F16;
        case at::kDouble: return RT_DT_F64;
        default: return -1;
    }
}

// dtype code of a gradient (bf16, f32, f16) or -1
inline int grad_code(const at::Tensor& t) {
    switch (t.scalar_type()) {
        case at::kBFloat16: return RT_DT_BF16;
        case at::kFloat: return RT_DT_F32;
        case at::kHalf: return RT_DT_F16;
        default: return -1;
    }
}

// dev >= 0: on that GPU; dev < 0: in host memory (exercised by the CPU-only tests of this
// helper; the optimizer only ever passes a GPU index)
inline bool dense_on(const at::Tensor& t, int dev) {
    if (t.layout() != at::kStrided || !t.is_contiguous()) return false;
    return dev >= 0 ? (t.is_cuda() && t.get_device() == dev) : t.is_cpu();
}

// The walk below is a chain of dependent loads per tensor (list item -> Python wrapper ->
// TensorImpl -> autograd meta -> gradient -> storage, and the same through the state dict), and
// with tens of thousands of tensors none of it is in cache: the chain's latency is the cost.
// Warm runs ahead of the main loop as a software pipeline: level k of the chain is prefetched
// for tensor i + (kLevels - k) * kLead while tensor i is processed, so each level finds the
// previous one already in cache.  It reads what the main loop reads and decides nothing.
constexpr int kLevels = 5;
constexpr Py_ssize_t kLead = 6;
constexpr Py_ssize_t kRing = 64;  // > kLevels * kLead

inline void touch(const void* p, int lines = 1) {
    const char* c = static_cast<const char*>(p);
    for (int k = 0; k < lines; ++k) __builtin_prefetch(c + 64 * k, 0, 3);
}

struct Warm {
    PyObject* params;
    PyObject* states;
    Py_ssize_t n;
    const c10::TensorImpl* impl[kRing][4];
    PyObject* obj[kRing][3];

    void level(int k, Py_ssize_t i) {
        if (i < 0 || i >= n) return;
        const Py_ssize_t r = i % kRing;
        PyObject* po = PyList_GET_ITEM(params, i);
        PyObject* so = PyList_GET_ITEM(states, i);
        switch (k) {
            case 0:  // wrappers and dict headers
                touch(po);
                touch(so);
                break;
            case 1:  // TensorImpl of the param; key table of the dict
                impl[r][0] = exact_tensor(po) ? THPVariable_Unpack(po).unsafeGetTensorImpl() : nullptr;
                if (impl[r][0]) touch(impl[r][0], 4);
                if (PyDict_CheckExact(so)) touch(reinterpret_cast<PyDictObject*>(so)->ma_keys, 4);
                break;
            case 2:  // autograd meta + storage of the param; state objects
                if (impl[r][0]) {
                    touch(impl[r][0]->autograd_meta(), 2);
                    touch(impl[r][0]->unsafe_storage().unsafeGetStorageImpl());
                }
                obj[r][0] = obj[r][1] = obj[r][2] = nullptr;
                if (PyDict_CheckExact(so)) {
                    obj[r][0] = PyDict_GetItem(so, k_ema);
                    obj[r][1] = PyDict_GetItem(so, k_ema_squared);
                    obj[r][2] = PyDict_GetItem(so, k_step);
                    for (int j = 0; j < 3; ++j)
                        if (obj[r][j]) touch(obj[r][j]);
                }
                break;
            case 3:  // TensorImpl of the gradient and of both states
                impl[r][1] = impl[r][2] = impl[r][3] = nullptr;
                if (impl[r][0]) {
                    const at::Tensor& g = THPVariable_Unpack(po).grad();
                    if (g.defined()) impl[r][1] = g.unsafeGetTensorImpl();
                }
                for (int j = 0; j < 2; ++j)
                    if (obj[r][j] && exact_tensor(obj[r][j]))
                        impl[r][2 + j] = THPVariable_Unpack(obj[r][j]).unsafeGetTensorImpl();
                for (int j = 1; j < 4; ++j)
                    if (impl[r][j]) touch(impl[r][j], 4);
                break;
            default:  // their storages
                for (int j = 1; j < 4; ++j)
                    if (impl[r][j]) touch(impl[r][j]->unsafe_storage().unsafeGetStorageImpl());
        }
    }

    // called before tensor i is processed
    void ahead_of(Py_ssize_t i) {
        if (i == 0) {  // fill the pipeline
            for (int k = 0; k < kLevels; ++k)
                for (Py_ssize_t j = 0; j < (kLevels - k) * kLead; ++j) level(k, j);
        }
        for (int k = 0; k < kLevels; ++k) level(k, i + (kLevels - k) * kLead);
    }
};

// gather_group(params, states, dev, desc_addr, desc_cap, status_addr, scalars_base, tensor_id_base)
//   -> (rows_written, [distinct new step values, in order of first use])
// params: list of tensors; states: list of the per-param state dicts (same order);
// desc_addr / desc_cap: address and capacity (rows) of an rt_tensor_desc buffer;
// status_addr: address of a uint8 buffer with len(params) entries.
// Row r of a written tensor gets scalars_idx = scalars_base + (index of its step in the returned list).
PyObject* gather_group(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
    if (nargs != 8) {
        PyErr_SetString(PyExc_TypeError, "gather_group takes 8 arguments");
        return nullptr;
    }
    PyObject* params = args[0];
    PyObject* states = args[1];
    if (!PyList_CheckExact(params) || !PyList_CheckExact(states)) {
        PyErr_SetString(PyExc_TypeError, "params and states must be lists");
        return nullptr;
    }
    const long dev = PyLong_AsLong(args[2]);
    auto* rows = reinterpret_cast<rt_tensor_desc*>(PyLong_AsUnsignedLongLong(args[3]));
    const Py_ssize_t cap = PyLong_AsSsize_t(args[4]);
    auto* status = reinterpret_cast<uint8_t*>(PyLong_AsUnsignedLongLong(args[5]));
    const unsigned long scalars_base = PyLong_AsUnsignedLong(args[6]);
    const unsigned long id_base = PyLong_AsUnsignedLong(args[7]);
    if (PyErr_Occurred()) return nullptr;
    const Py_ssize_t n = PyList_GET_SIZE(params);
    if (PyList_GET_SIZE(states) != n || !rows || !status) {
        PyErr_SetString(PyExc_ValueError, "params / states length mismatch or NULL buffer");
        return nullptr;
    }
    std::vector<long long> steps;
    Py_ssize_t w = 0;
    Warm warm;
    warm.params = params;
    warm.states = states;
    warm.n = n;
    for (Py_ssize_t i = 0; i < n; ++i) {
        warm.ahead_of(i);
        status[i] = kPython;
        PyObject* po = PyList_GET_ITEM(params, i);
        PyObject* so = PyList_GET_ITEM(states, i);
        if (!exact_tensor(po) || !PyDict_CheckExact(so)) continue;
        const at::Tensor& p = THPVariable_Unpack(po);
        const at::Tensor& g = p.grad();
        if (!g.defined()) {
            status[i] = kNoGrad;
            continue;
        }
        if (w >= cap) continue;
        PyObject* mo = PyDict_GetItem(so, k_ema);           // borrowed
        PyObject* vo = PyDict_GetItem(so, k_ema_squared);
        PyObject* st = PyDict_GetItem(so, k_step);
        if (!mo || !vo || !st || !exact_tensor(mo) || !exact_tensor(vo) || !PyLong_CheckExact(st)) continue;
        const at::Tensor& m = THPVariable_Unpack(mo);
        const at::Tensor& v = THPVariable_Unpack(vo);
        const int pc = pmv_code(p), mc = pmv_code(m), vc = pmv_code(v), gc = grad_code(g);
        if (pc < 0 || mc < 0 || vc < 0 || gc < 0) continue;
        if (!dense_on(p, (int)dev) || !dense_on(g, (int)dev) || !dense_on(m, (int)dev) || !dense_on(v, (int)dev))
            continue;
        const int64_t numel = p.numel();
        if (g.numel() != numel || m.numel() != numel || v.numel() != numel) continue;
        int overflow = 0;
        const long long step = PyLong_AsLongLongAndOverflow(st, &overflow);
        if (overflow || step < 0) continue;
        const long long new_step = step + 1;  // adamw.py:177
        PyObject* ns = PyLong_FromLongLong(new_step);
        if (!ns) return nullptr;
        const int rc = PyDict_SetItem(so, k_step, ns);
        Py_DECREF(ns);
        if (rc != 0) return nullptr;
        size_t si = steps.size();
        for (size_t k = steps.size(); k-- > 0;)
            if (steps[k] == new_step) {
                si = k;
                break;
            }
        if (si == steps.size()) steps.push_back(new_step);

        rt_tensor_desc& d = rows[w++];
        std::memset(&d, 0, sizeof(d));
        d.p = p.data_ptr();
        d.g = g.data_ptr();
        d.m = m.data_ptr();
        d.v = v.data_ptr();
        d.numel = (uint64_t)numel;
        d.tensor_id = (uint32_t)(id_base + (unsigned long)i);
        d.step = (uint32_t)((unsigned long long)new_step & 0xFFFFFFFFull);
        d.scalars_idx = (uint32_t)(scalars_base + si);
        d.p_dtype = (uint8_t)pc;
        d.g_dtype = (uint8_t)gc;
        d.m_dtype = (uint8_t)mc;
        d.v_dtype = (uint8_t)vc;
        status[i] = kWritten;
    }
    PyObject* lst = PyList_New((Py_ssize_t)steps.size());
    if (!lst) return nullptr;
    for (size_t k = 0; k < steps.size(); ++k) {
        PyObject* v = PyLong_FromLongLong(steps[k]);
        if (!v) {
            Py_DECREF(lst);
            return nullptr;
        }
        PyList_SET_ITEM(lst, (Py_ssize_t)k, v);
    }
    PyObject* out = Py_BuildValue("(nN)", w, lst);
    return out;
}

// verify_layout(params, expect_addr, n) -> bool
// The cheap per-step check of a frozen layout: params is the flat list of parameters the layout was
// recorded for, expect_addr the address of n triples of uint64 (data pointer of the parameter, data
// pointer of its gradient or 0 for "no gradient", RT_DT_* code of the gradient).  True when every
// parameter is still an exact Tensor / Parameter at the recorded address whose gradient is where it
// was (or still absent), dense, contiguous, of the recorded dtype and of the parameter's size.
// Reads what gather_group reads of a parameter and its gradient, with the same software prefetch,
// and nothing of the states; it changes nothing.
// One contiguous range of the check.  Only reads: object headers, tensor records, storages.
bool verify_range(PyObject* params, const uint64_t* expect, Py_ssize_t lo, Py_ssize_t hi) {
    constexpr Py_ssize_t kAhead = 8;
    constexpr Py_ssize_t kSlots = 4 * kAhead;
    const c10::TensorImpl* pimpl[kSlots] = {};
    auto stage = [&](int level, Py_ssize_t i) {
        if (i < lo || i >= hi) return;
        const Py_ssize_t r = i % kSlots;
        PyObject* po = PyList_GET_ITEM(params, i);
        switch (level) {
            case 0: touch(po); break;
            case 1:
                pimpl[r] = exact_tensor(po) ? THPVariable_Unpack(po).unsafeGetTensorImpl() : nullptr;
                if (pimpl[r]) touch(pimpl[r], 4);
                break;
            case 2:
                if (pimpl[r]) {
                    touch(pimpl[r]->autograd_meta(), 2);
                    touch(pimpl[r]->unsafe_storage().unsafeGetStorageImpl());
                }
                break;
            default:
                if (pimpl[r]) {
                    const at::Tensor& g = THPVariable_Unpack(po).grad();
                    if (g.defined()) touch(g.unsafeGetTensorImpl(), 4);
                }
        }
    };
    for (int level = 0; level < 4; ++level)
        for (Py_ssize_t j = 0; j < (4 - level) * kAhead; ++j) stage(level, lo + j);
    for (Py_ssize_t i = lo; i < hi; ++i) {
        for (int level = 0; level < 4; ++level) stage(level, i + (4 - level) * kAhead);
        PyObject* po = PyList_GET_ITEM(params, i);
        if (!exact_tensor(po)) return false;
        const at::Tensor& p = THPVariable_Unpack(po);
        if (reinterpret_cast<uint64_t>(p.data_ptr()) != expect[3 * i]) return false;
        const at::Tensor& g = p.grad();
        const uint64_t want = expect[3 * i + 1];
        if (!g.defined()) {
            if (want != 0) return false;
            continue;
        }
        if (want == 0 || g.layout() != at::kStrided || !g.is_contiguous() || g.numel() != p.numel() ||
            reinterpret_cast<uint64_t>(g.data_ptr()) != want || (uint64_t)grad_code(g) != expect[3 * i + 2])
            return false;
    }
    return true;
}

PyObject* verify_layout(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
    if (nargs != 3) {
        PyErr_SetString(PyExc_TypeError, "verify_layout takes 3 arguments");
        return nullptr;
    }
    PyObject* params = args[0];
    if (!PyList_CheckExact(params)) {
        PyErr_SetString(PyExc_TypeError, "params must be a list");
        return nullptr;
    }
    const auto* expect = reinterpret_cast<const uint64_t*>(PyLong_AsUnsignedLongLong(args[1]));
    const Py_ssize_t n = PyLong_AsSsize_t(args[2]);
    if (PyErr_Occurred()) return nullptr;
    if (PyList_GET_SIZE(params) != n || (n > 0 && !expect)) Py_RETURN_FALSE;
    // The walk is bound by the latency of dependent loads, so long lists are split over a few
    // threads.  The calling thread keeps the interpreter lock throughout: nothing can change the
    // objects while the helpers read them, and the helpers call nothing of the interpreter.
    const Py_ssize_t kPerThread = 2048;
    const int threads = (int)std::min<Py_ssize_t>(8, std::max<Py_ssize_t>(1, n / kPerThread));
    if (threads <= 1) {
        if (verify_range(params, expect, 0, n)) Py_RETURN_TRUE;
        Py_RETURN_FALSE;
    }
    std::vector<char> ok(threads, 0);
    std::vector<std::thread> pool;
    const Py_ssize_t per = (n + threads - 1) / threads;
    for (int t = 1; t < threads; ++t)
        pool.emplace_back([&, t] { ok[t] = verify_range(params, expect, t * per, std::min(n, (t + 1) * per)); });
    ok[0] = verify_range(params, expect, 0, std::min(n, per));
    for (auto& th : pool) th.join();
    for (char c : ok)
        if (!c) Py_RETURN_FALSE;
    Py_RETURN_TRUE;
}

// dict_versions(dicts, out_addr, n) / verify_versions(dicts, expect_addr, n) -> bool
// A recorded layout keeps the addresses of the two state tensors of every parameter and does not
// read the state dicts again while it is in use, so nothing else may change them either.  CPython
// stamps every dict with a version that changes whenever the dict is modified (ma_version_tag);
// dict_versions writes the stamps of n dicts as uint64 to out_addr, verify_versions compares them:
// a state tensor that was replaced, removed or added shows as a changed stamp, for one load per
// dict.  (Interpreters without the stamp, 3.12 and later: dict_versions fails and no layout is recorded.)
PyObject* dict_versions(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
#if PY_VERSION_HEX >= 0x030C0000
    PyErr_SetString(PyExc_NotImplementedError, "this interpreter's dicts carry no version stamp");
    return nullptr;
#else
    if (nargs != 3 || !PyList_CheckExact(args[0])) {
        PyErr_SetString(PyExc_TypeError, "dict_versions(list, address, n)");
        return nullptr;
    }
    auto* out = reinterpret_cast<uint64_t*>(PyLong_AsUnsignedLongLong(args[1]));
    const Py_ssize_t n = PyLong_AsSsize_t(args[2]);
    if (PyErr_Occurred()) return nullptr;
    if (PyList_GET_SIZE(args[0]) != n || (n > 0 && !out)) {
        PyErr_SetString(PyExc_ValueError, "list length and n differ");
        return nullptr;
    }
    for (Py_ssize_t i = 0; i < n; ++i) {
        PyObject* d = PyList_GET_ITEM(args[0], i);
        if (!PyDict_Check(d)) {
            PyErr_SetString(PyExc_TypeError, "not a dict");
            return nullptr;
        }
        out[i] = reinterpret_cast<PyDictObject*>(d)->ma_version_tag;
    }
    Py_RETURN_NONE;
#endif
}

PyObject* verify_versions(PyObject*, PyObject* const* args, Py_ssize_t nargs) {
#if PY_VERSION_HEX >= 0x030C0000
    Py_RETURN_FALSE;
#else
    if (nargs != 3 || !PyList_CheckExact(args[0])) {
        PyErr_SetString(PyExc_TypeError, "verify_versions(list, address, n)");
        return nullptr;
    }
    const auto* expect = reinterpret_cast<const uint64_t*>(PyLong_AsUnsignedLongLong(args[1]));
    const Py_ssize_t n = PyLong_AsSsize_t(args[2]);
    if (PyErr_Occurred()) return nullptr;
    if (PyList_GET_SIZE(args[0]) != n || (n > 0 && !expect)) Py_RETURN_FALSE;
    constexpr Py_ssize_t kAhead = 16;
    for (Py_ssize_t i = 0; i < n; ++i) {
        if (i + kAhead < n) touch(PyList_GET_ITEM(args[0], i + kAhead));
        PyObject* d = PyList_GET_ITEM(args[0], i);
        if (!PyDict_Check(d) || reinterpret_cast<PyDictObject*>(d)->ma_version_tag != expect[i]) Py_RETURN_FALSE;
    }
    Py_RETURN_TRUE;
#endif
}

// set_types(torch.Tensor, torch.nn.Parameter): only objects of exactly these types take the fast path.
PyObject* set_types(PyObject*, PyObject* args) {
    PyObject *a = nullptr, *b = nullptr;
    if (!PyArg_ParseTuple(args, "OO", &a, &b)) return nullptr;
    if (!PyType_Check(a) || !PyType_Check(b)) {
        PyErr_SetString(PyExc_TypeError, "expected two types");
        return nullptr;
    }
    Py_INCREF(a);
    Py_INCREF(b);
    t_tensor = reinterpret_cast<PyTypeObject*>(a);
    t_parameter = reinterpret_cast<PyTypeObject*>(b);
    Py_RETURN_NONE;
}

PyMethodDef methods[] = {
    {"gather_group", reinterpret_cast<PyCFunction>(reinterpret_cast<void (*)()>(gather_group)), METH_FASTCALL,
     "rt_tensor_desc rows of the plain tensors of one param group"},
    {"verify_layout", reinterpret_cast<PyCFunction>(reinterpret_cast<void (*)()>(verify_layout)), METH_FASTCALL,
     "whether every parameter and gradient of a recorded layout is still where it was"},
    {"dict_versions", reinterpret_cast<PyCFunction>(reinterpret_cast<void (*)()>(dict_versions)), METH_FASTCALL,
     "modification stamps of a list of dicts"},
    {"verify_versions", reinterpret_cast<PyCFunction>(reinterpret_cast<void (*)()>(verify_versions)), METH_FASTCALL,
     "whether none of the dicts has been modified since dict_versions"},
    {"set_types", set_types, METH_VARARGS, "register torch.Tensor and torch.nn.Parameter"},
    {nullptr, nullptr, 0, nullptr},
};

PyModuleDef moddef = {PyModuleDef_HEAD_INIT, "_rt_gather", "descriptor gathering for ramtorch_amd.AdamW", -1, methods,
                      nullptr, nullptr, nullptr, nullptr};

}  // namespace

PyMODINIT_FUNC PyInit__rt_gather(void) {
    k_ema = PyUnicode_InternFromString("ema");
    k_ema_squared = PyUnicode_InternFromString("ema_squared");
    k_step = PyUnicode_InternFromString("step");
    if (!k_ema || !k_ema_squared || !k_step) return nullptr;
    PyObject* m = PyModule_Create(&moddef);
    if (!m) return nullptr;
    PyModule_AddIntConstant(m, "DESC_SIZE", (long)sizeof(rt_tensor_desc));
    PyModule_AddIntConstant(m, "WRITTEN", kWritten);
    PyModule_AddIntConstant(m, "NO_GRAD", kNoGrad);
    PyModule_AddIntConstant(m, "PYTHON", kPython);
    return m;
}
