// Host-side helper: turns the optimizer's Python tensor lists into FsAdamTensor rows (include/fsadam.h)
// in one C++ loop per step instead of several Python-level passes over every tensor.
//
// It stands where the reference converts list[list[Tensor]] to vector<vector<Tensor>> in pybind
// (fairscale/clib/fused_adam_cuda/fused_adam_cuda.cpp:4-8), validates the lists
// (fairscale/clib/fused_adam_cuda/multi_tensor_apply.cuh:49-67) and walks the parameters
// (fairscale/optim/adam.py:207-254).  It reads pointers and metadata only: no tensor operation is
// dispatched and nothing is computed here.
//
// Built as a CPython extension module against the installed torch: python -m fairscale_amd.csrc.build
#include <Python.h>

#include <torch/csrc/autograd/python_variable.h>
#include <pybind11/pybind11.h>

#include <cstdint>
#include <string>

namespace py = pybind11;

namespace {

// Status codes shared with fairscale_amd/_rows.py.  Non-negative: the rows were written.
enum Status : int {
    kUnchanged = 0,      // rows equal to what the buffer already held
    kChanged = 1,        // at least one word differs
    kNotTensor = -1,     // an entry is not a plain torch.Tensor / Parameter
    kNotContiguous = -2,  // multi_tensor_apply.cuh:59
    kNotCuda = -3,        // multi_tensor_apply.cuh:61
    kNumel = -4,          // multi_tensor_apply.cuh:65
    kDtype = -5,
    kDevice = -6,
    kLength = -7,         // multi_tensor_apply.cuh:55
    kNoGrad = -8,         // a parameter has no gradient: the general walk decides
    kSparse = -9,         // adam.py:218
    kNoState = -10,       // state dict without exp_avg / exp_avg_sq / step
    kError = -11,         // torch raised while reading metadata
    kStale = -12,         // the parameter list no longer holds the objects the states belong to
};

struct Result {
    int status = kUnchanged;
    int64_t list = -1;   // which list (0 p, 1 m, 2 v, 3 g, 4 p_copy)
    int64_t index = -1;  // which tensor
};

c10::ScalarType dtype_of_code(int code) { return code == 1 ? c10::ScalarType::Half : c10::ScalarType::Float; }

// The checks of multi_tensor_apply.cuh:59-65 in the reference's order, then dtype and device.
// device >= 0: that GPU.  device == -1: host tensors, which only tests of this walk ask for (the
// kernels' library refuses to run without a GPU).
inline int check_tensor(const at::Tensor& t, c10::ScalarType dtype, int device, int64_t numel) {
    if (t.layout() != c10::kStrided) return kSparse;
    if (!t.is_contiguous()) return kNotContiguous;
    if (device >= 0 && !t.is_cuda()) return kNotCuda;
    if (t.numel() != numel) return kNumel;
    if (t.scalar_type() != dtype) return kDtype;
    if (t.get_device() != device) return kDevice;
    return 0;
}

inline void put(int64_t* slot, int64_t value, bool* changed) {
    if (*slot != value) {
        *slot = value;
        *changed = true;
    }
}

inline const at::Tensor* plain_tensor(PyObject* obj) {
    if (!THPVariable_CheckExact(obj)) return nullptr;
    return &THPVariable_Unpack(obj);
}

// rows: n x 6 int64 (p, m, v, g, p_copy, numel).  lists: 4 or 5 Python lists of n tensors.
Result fill_rows_impl(PyObject* lists, const int* dtype_codes, int device, int64_t* rows, int64_t n) {
    Result r;
    bool changed = false;
    const Py_ssize_t depth = PyList_GET_SIZE(lists);
    PyObject* first = PyList_GET_ITEM(lists, 0);
    for (Py_ssize_t d = 0; d < depth; ++d) {
        PyObject* lst = PyList_GET_ITEM(lists, d);
        if (!PyList_Check(lst) || PyList_GET_SIZE(lst) != n) {
            r.status = kLength;
            r.list = d;
            return r;
        }
        const c10::ScalarType dtype = dtype_of_code(dtype_codes[d]);
        for (int64_t t = 0; t < n; ++t) {
            const at::Tensor* x = plain_tensor(PyList_GET_ITEM(lst, t));
            const at::Tensor* x0 = d == 0 ? x : plain_tensor(PyList_GET_ITEM(first, t));
            if (!x || !x0) {
                r.status = kNotTensor;
                r.list = d;
                r.index = t;
                return r;
            }
            const int bad = check_tensor(*x, dtype, device, x0->numel());
            if (bad) {
                r.status = bad;
                r.list = d;
                r.index = t;
                return r;
            }
            put(&rows[t * 6 + d], reinterpret_cast<int64_t>(x->data_ptr()), &changed);
            if (d == 0) put(&rows[t * 6 + 5], x->numel(), &changed);
        }
    }
    if (depth == 4)
        for (int64_t t = 0; t < n; ++t) put(&rows[t * 6 + 4], 0, &changed);
    r.status = changed ? kChanged : kUnchanged;
    return r;
}

py::tuple as_tuple(const Result& r, py::object extra = py::none()) { return py::make_tuple(r.status, r.list, r.index, extra); }

// fill_rows(lists, dtype_codes, device_index, rows_address, n) -> (status, list, index, None)
py::tuple fill_rows(py::list lists, py::tuple dtype_codes, int device, uintptr_t rows_address, int64_t n) {
    Result r;
    const Py_ssize_t depth = PyList_GET_SIZE(lists.ptr());
    if ((depth != 4 && depth != 5) || (Py_ssize_t)py::len(dtype_codes) != depth || n < 1 || !rows_address) {
        r.status = kLength;
        return as_tuple(r);
    }
    for (Py_ssize_t d = 0; d < depth; ++d)
        if (!PyList_Check(PyList_GET_ITEM(lists.ptr(), d))) {
            r.status = kLength;
            r.list = d;
            return as_tuple(r);
        }
    int codes[5] = {0, 0, 0, 0, 0};
    for (Py_ssize_t d = 0; d < depth; ++d) codes[d] = dtype_codes[d].cast<int>();
    try {
        r = fill_rows_impl(lists.ptr(), codes, device, reinterpret_cast<int64_t*>(rows_address), n);
    } catch (const std::exception& e) {
        r.status = kError;
        return as_tuple(r, py::str(e.what()));
    }
    return as_tuple(r);
}

// The steady-state walk of Adam.step.  `states[t]` is the state dict {step, exp_avg, exp_avg_sq} of
// parameter t, or None for a parameter that had no gradient when the lists were collected: such a
// parameter must still have none (adam.py:214-215 skips it), the others must have a dense one.  p
// comes from `masters` when given (MIXED_PRECISION: the fp32 copies, with the fp16 parameters as
// p_copy), else from `params`; `outs` are attached fp16 copies (None where states is None).  Rows are
// written for the parameters that take part, in order.  When everything checks, each state's step
// is incremented and the last one is returned.
//
// `snapshot` is the tuple of parameter objects `states` was collected for: a list edited in place since
// then is reported as stale instead of pairing a new parameter with another one's state.
//
// gather(params, snapshot, masters|None, states, outs|None, dtype_codes(p, s, g), device, rows_address)
//   -> (status, list, index, step|None)
py::tuple gather(py::list params, py::tuple snapshot, py::object masters, py::list states, py::object outs, py::tuple dtype_codes,
                 int device, uintptr_t rows_address) {
    static PyObject* k_avg = PyUnicode_InternFromString("exp_avg");
    static PyObject* k_sq = PyUnicode_InternFromString("exp_avg_sq");
    static PyObject* k_step = PyUnicode_InternFromString("step");
    static PyObject* one = PyLong_FromLong(1);
    Result r;
    const int64_t n = PyList_GET_SIZE(params.ptr());
    const bool mixed = !masters.is_none();
    const bool with_outs = !outs.is_none();
    if (PyTuple_GET_SIZE(snapshot.ptr()) != n) {
        r.status = kStale;
        return as_tuple(r);
    }
    if (n < 1 || !rows_address || PyList_GET_SIZE(states.ptr()) != n || py::len(dtype_codes) != 3 ||
        (mixed && (!PyList_Check(masters.ptr()) || PyList_GET_SIZE(masters.ptr()) != n)) ||
        (with_outs && (!PyList_Check(outs.ptr()) || PyList_GET_SIZE(outs.ptr()) != n)) || (mixed && with_outs)) {
        r.status = kLength;
        return as_tuple(r);
    }
    const c10::ScalarType p_dtype = dtype_of_code(dtype_codes[0].cast<int>());
    const c10::ScalarType s_dtype = dtype_of_code(dtype_codes[1].cast<int>());
    const c10::ScalarType g_dtype = dtype_of_code(dtype_codes[2].cast<int>());
    int64_t* rows = reinterpret_cast<int64_t*>(rows_address);
    bool changed = false;
    int64_t active = 0;  // rows written so far
    auto stop = [&](int status, int64_t list, int64_t index) {
        r.status = status;
        r.list = list;
        r.index = index;
        return as_tuple(r);
    };
    try {
        for (int64_t t = 0; t < n; ++t) {
            PyObject* param_obj = PyList_GET_ITEM(params.ptr(), t);
            if (param_obj != PyTuple_GET_ITEM(snapshot.ptr(), t)) return stop(kStale, 0, t);
            const at::Tensor* param = plain_tensor(param_obj);
            if (!param) return stop(kNotTensor, mixed ? 4 : 0, t);
            const at::Tensor* p = mixed ? plain_tensor(PyList_GET_ITEM(masters.ptr(), t)) : param;
            if (!p) return stop(kNotTensor, 0, t);
            const at::Tensor& g = param->grad();
            PyObject* st = PyList_GET_ITEM(states.ptr(), t);
            if (st == Py_None) {  // sat out when the lists were collected
                if (g.defined()) return stop(kStale, 3, t);
                continue;
            }
            if (!g.defined()) return stop(kNoGrad, 3, t);
            if (!PyDict_Check(st)) return stop(kNoState, 1, t);
            PyObject* m_obj = PyDict_GetItemWithError(st, k_avg);
            PyObject* v_obj = PyDict_GetItemWithError(st, k_sq);
            if (!m_obj || !v_obj || !PyDict_GetItemWithError(st, k_step)) {
                PyErr_Clear();
                return stop(kNoState, 1, t);
            }
            const at::Tensor* m = plain_tensor(m_obj);
            const at::Tensor* v = plain_tensor(v_obj);
            if (!m) return stop(kNotTensor, 1, t);
            if (!v) return stop(kNotTensor, 2, t);
            const int64_t numel = p->numel();
            int bad;
            if ((bad = check_tensor(*p, p_dtype, device, numel))) return stop(bad, 0, t);
            if ((bad = check_tensor(*m, s_dtype, device, numel))) return stop(bad, 1, t);
            if ((bad = check_tensor(*v, s_dtype, device, numel))) return stop(bad, 2, t);
            if ((bad = check_tensor(g, g_dtype, device, numel))) return stop(bad, 3, t);
            int64_t* row = rows + active * 6;
            active += 1;
            put(row + 0, reinterpret_cast<int64_t>(p->data_ptr()), &changed);
            put(row + 1, reinterpret_cast<int64_t>(m->data_ptr()), &changed);
            put(row + 2, reinterpret_cast<int64_t>(v->data_ptr()), &changed);
            put(row + 3, reinterpret_cast<int64_t>(g.data_ptr()), &changed);
            if (mixed || with_outs) {
                const at::Tensor* c = mixed ? param : plain_tensor(PyList_GET_ITEM(outs.ptr(), t));
                if (!c) return stop(kNotTensor, 4, t);
                if ((bad = check_tensor(*c, c10::ScalarType::Half, device, numel))) return stop(bad, 4, t);
                put(row + 4, reinterpret_cast<int64_t>(c->data_ptr()), &changed);
            } else {
                put(row + 4, 0, &changed);
            }
            put(row + 5, numel, &changed);
        }
    } catch (const std::exception& e) {
        r.status = kError;
        return as_tuple(r, py::str(e.what()));
    }
    if (active == 0) return stop(kNoGrad, 3, 0);
    // everything checked: advance the step counters (adam.py:230)
    PyObject* last = nullptr;
    for (int64_t t = 0; t < n; ++t) {
        PyObject* st = PyList_GET_ITEM(states.ptr(), t);
        if (st == Py_None) continue;
        PyObject* next = PyNumber_Add(PyDict_GetItemWithError(st, k_step), one);
        if (!next) throw py::error_already_set();
        if (PyDict_SetItem(st, k_step, next) != 0) {
            Py_DECREF(next);
            throw py::error_already_set();
        }
        Py_XDECREF(last);
        last = next;  // keeps the reference of the newest counter
    }
    r.status = changed ? kChanged : kUnchanged;
    return as_tuple(r, py::reinterpret_steal<py::object>(last));
}

// Gradients of one pass (include/fsadam.h: FsGradTensor rows, n x 2 int64: pointer, numel): dense,
// contiguous, one dtype, one device.
//
// fill_grad_rows(grads, dtype_code, device_index, rows_address) -> (status, 3, index, None)
py::tuple fill_grad_rows(py::list grads, int dtype_code, int device, uintptr_t rows_address) {
    Result r;
    r.list = 3;
    const int64_t n = PyList_GET_SIZE(grads.ptr());
    if (n < 1 || !rows_address) {
        r.status = kLength;
        return as_tuple(r);
    }
    const c10::ScalarType dtype = dtype_of_code(dtype_code);
    int64_t* rows = reinterpret_cast<int64_t*>(rows_address);
    try {
        for (int64_t t = 0; t < n; ++t) {
            const at::Tensor* g = plain_tensor(PyList_GET_ITEM(grads.ptr(), t));
            r.index = t;
            if (!g) {
                r.status = kNotTensor;
                return as_tuple(r);
            }
            const int bad = check_tensor(*g, dtype, device, g->numel());
            if (bad) {
                r.status = bad;
                return as_tuple(r);
            }
            rows[t * 2 + 0] = reinterpret_cast<int64_t>(g->data_ptr());
            rows[t * 2 + 1] = g->numel();
        }
    } catch (const std::exception& e) {
        r.status = kError;
        return as_tuple(r, py::str(e.what()));
    }
    r.index = -1;
    r.status = kUnchanged;
    return as_tuple(r);
}

}  // namespace

PYBIND11_MODULE(_tensor_rows, m) {
    m.doc() = "Tensor lists -> FsAdamTensor rows for libfsadam (pointers and metadata only)";
    m.def("fill_rows", &fill_rows);
    m.def("gather", &gather);
    m.def("fill_grad_rows", &fill_grad_rows);
    m.attr("UNCHANGED") = (int)kUnchanged;
    m.attr("CHANGED") = (int)kChanged;
    m.attr("NOT_TENSOR") = (int)kNotTensor;
    m.attr("NOT_CONTIGUOUS") = (int)kNotContiguous;
    m.attr("NOT_CUDA") = (int)kNotCuda;
    m.attr("NUMEL") = (int)kNumel;
    m.attr("DTYPE") = (int)kDtype;
    m.attr("DEVICE") = (int)kDevice;
    m.attr("LENGTH") = (int)kLength;
    m.attr("NO_GRAD") = (int)kNoGrad;
    m.attr("SPARSE") = (int)kSparse;
    m.attr("NO_STATE") = (int)kNoState;
    m.attr("ERROR") = (int)kError;
    m.attr("STALE") = (int)kStale;
}
