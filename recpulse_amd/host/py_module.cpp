// CPython extension `recpulse_cuda`: the Tensor type and module functions of the
// reference's Python surface for the matmul path (reference python/tensor_python.c),
// bound with pybind11 on top of rp_host.h.  The module keeps the reference's
// name so that `import recpulse_cuda as rp` and `recpulse.module.Linear` work
// unchanged; failures raise RuntimeError("<op> operation failed ...") like the
// reference (python/tensor_python.c:2294-2297).
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/eval.h>
#include <pybind11/stl.h>

#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "rp_host.h"

namespace py = pybind11;

namespace {

struct PyTensor {
    Tensor* t;                       // owns one reference (reference python/tensor_python.c:15-18, 74-80)
    explicit PyTensor(Tensor* tensor) : t(tensor) {}
    PyTensor(const PyTensor&) = delete;
    PyTensor& operator=(const PyTensor&) = delete;
    ~PyTensor() { if (t) free_tensor(t); }
};

using TensorPtr = std::unique_ptr<PyTensor>;

TensorPtr wrap(Tensor* t, const char* op) {
    if (!t) {
        std::string msg = std::string(op) + " operation failed";
        const char* why = rp_last_error();
        if (why && why[0]) msg += std::string(": ") + why;
        throw std::runtime_error(msg);
    }
    return std::make_unique<PyTensor>(t);
}

DType parse_dtype(const std::string& s) {             // reference python/tensor_python.c:23-40
    if (s == "float32") return DTYPE_FLOAT32;
    if (s == "float64") return DTYPE_FLOAT64;
    if (s == "float16") return DTYPE_FLOAT16;
    if (s == "bfloat16") return DTYPE_BFLOAT16;
    throw py::value_error("Invalid dtype '" + s + "'. Must be 'float32', 'float64', 'float16' or 'bfloat16'");
}

const char* dtype_name(DType d) {
    switch (d) {
        case DTYPE_FLOAT32: return "float32";
        case DTYPE_FLOAT64: return "float64";
        case DTYPE_FLOAT16: return "float16";
        default: return "bfloat16";
    }
}

int parse_device(const std::string& s) {              // reference python/tensor_python.c:42-62
    if (s == "cpu" || s == "host") return -1;
    if (s == "cuda" || s == "device") return 0;
    if (s.rfind("cuda:", 0) == 0) {
        try { return std::stoi(s.substr(5)); } catch (...) {}
    }
    throw py::value_error("Invalid device '" + s + "'. Must be 'cpu', 'cuda' or 'cuda:N'");
}

std::string device_name(int id) { return id < 0 ? "cpu" : "cuda:" + std::to_string(id); }

std::vector<int> to_shape(const py::object& o) {
    std::vector<int> shape;
    if (py::isinstance<py::int_>(o)) shape.push_back(o.cast<int>());
    else for (auto item : o) shape.push_back(item.cast<int>());
    if (shape.empty()) throw py::value_error("shape must not be empty");
    return shape;
}

py::array tensor_to_numpy(PyTensor& self) {           // bfloat16 comes back as float32 values (numpy has no bfloat16)
    Tensor* t = self.t;
    DType out_dt = t->dtype == DTYPE_BFLOAT16 ? DTYPE_FLOAT32 : t->dtype;
    Tensor* host = tensor_to(t, -1, out_dt, false);
    if (!host) throw std::runtime_error(std::string("to_numpy failed: ") + rp_last_error());
    std::vector<py::ssize_t> shape(host->shape, host->shape + host->ndim);
    py::array arr;
    if (out_dt == DTYPE_FLOAT32) arr = py::array_t<float>(shape);
    else if (out_dt == DTYPE_FLOAT64) arr = py::array_t<double>(shape);
    else arr = py::array(py::dtype("float16"), shape);
    std::memcpy(arr.mutable_data(), host->data, host->size * dtype_size(out_dt));
    free_tensor(host);
    return arr;
}

TensorPtr from_numpy(py::array arr) {                 // float32 / float64 / float16, always on the host (reference :3068-3107)
    py::array c = py::array::ensure(arr, py::array::c_style);
    DType dt;
    if (c.dtype().is(py::dtype::of<float>())) dt = DTYPE_FLOAT32;
    else if (c.dtype().is(py::dtype::of<double>())) dt = DTYPE_FLOAT64;
    else if (c.dtype().is(py::dtype("float16"))) dt = DTYPE_FLOAT16;
    else throw py::type_error("from_numpy supports float32, float64 and float16 arrays");
    std::vector<int> shape;
    for (py::ssize_t i = 0; i < c.ndim(); i++) shape.push_back((int)c.shape(i));
    if (shape.empty()) shape.push_back(1);
    Tensor* t = empty_tensor(dt, -1, (int)shape.size(), shape.data());
    if (!t) throw std::runtime_error("from_numpy failed");
    std::memcpy(t->data, c.data(), t->size * dtype_size(dt));
    return std::make_unique<PyTensor>(t);
}

std::vector<int> targets_from(const py::object& o) {  // a sequence of ints or a Tensor (reference :942-967, 1254-1264)
    std::vector<int> out;
    if (py::isinstance<PyTensor>(o)) {
        PyTensor& pt = o.cast<PyTensor&>();
        Tensor* host = tensor_to(pt.t, -1, DTYPE_FLOAT32, false);
        if (!host) throw std::runtime_error("targets: conversion failed");
        for (size_t i = 0; i < host->size; i++) out.push_back((int)((float*)host->data)[i]);
        free_tensor(host);
    } else {
        for (auto item : o) out.push_back(item.cast<int>());
    }
    return out;
}

}  // namespace

// Reference count that `self` shows inside a method called on a temporary (a call result that no name holds), or 0 when
// a temporary cannot be told from a named object on this interpreter: then nothing is ever treated as one.
static int g_temporary_refs = 0;

PYBIND11_MODULE(recpulse_cuda, m) {
    m.doc() = "RecPulse tensor module for the matmul path, MI355X device layer underneath";

    py::class_<PyTensor>(m, "Tensor")
        .def_property_readonly("shape", [](PyTensor& s) { py::tuple t(s.t->ndim); for (int i = 0; i < s.t->ndim; i++) t[i] = s.t->shape[i]; return t; })
        .def_property_readonly("strides", [](PyTensor& s) { py::tuple t(s.t->ndim); for (int i = 0; i < s.t->ndim; i++) t[i] = s.t->strides[i]; return t; })
        .def_property_readonly("dtype", [](PyTensor& s) { return std::string(dtype_name(s.t->dtype)); })
        .def_property_readonly("device", [](PyTensor& s) { return device_name(s.t->device_id); })
        .def_property_readonly("device_id", [](PyTensor& s) { return s.t->device_id; })
        .def_property_readonly("size", [](PyTensor& s) { return s.t->size; })
        .def_property_readonly("ndim", [](PyTensor& s) { return s.t->ndim; })
        .def_property_readonly("requires_grad", [](PyTensor& s) { return s.t->metadata && s.t->metadata->requires_grad; })
        .def_property_readonly("has_grad", [](PyTensor& s) { return s.t->metadata && s.t->metadata->grad != nullptr; })
        .def_property_readonly("is_contiguous", [](PyTensor& s) { return rp_is_contiguous(s.t); })
        .def_property_readonly("grad", [](PyTensor& s) -> py::object {          // a copy, as in the reference (:155-174)
            if (!s.t->metadata || !s.t->metadata->grad) return py::none();
            return py::cast(wrap(tensor_copy(s.t->metadata->grad), "grad"));
        })
        .def_property_readonly("T", [](PyTensor& s) {                           // 2-D only (:2219-2246)
            if (s.t->ndim != 2) throw std::runtime_error("T is defined for 2-D tensors");
            return wrap(op_transpose(s.t, 0, 1), "transpose");
        })
        .def("to", [](py::object self, py::object device, py::object dtype, bool inplace) -> py::object {
            PyTensor& s = self.cast<PyTensor&>();
            int dev = device.is_none() ? s.t->device_id : parse_device(device.cast<std::string>());
            DType dt = dtype.is_none() ? s.t->dtype : parse_dtype(dtype.cast<std::string>());
            Tensor* r = tensor_to(s.t, dev, dt, inplace);
            if (!r) throw std::runtime_error(std::string("to operation failed: ") + rp_last_error());
            if (inplace) return self;
            return py::cast(std::make_unique<PyTensor>(r));
        }, py::arg("device") = py::none(), py::arg("dtype") = py::none(), py::arg("inplace") = false)
        .def("to_numpy", &tensor_to_numpy)
        .def("copy", [](PyTensor& s) { return wrap(tensor_copy(s.t), "copy"); })
        .def("copy_", [](py::object self, PyTensor& other) {
            PyTensor& s = self.cast<PyTensor&>();
            if (tensor_copy_into(s.t, other.t) != 0) throw std::runtime_error(std::string("copy_ operation failed: ") + rp_last_error());
            return self;
        })
        .def("data", [](PyTensor& s) {                                           // flat list of Python floats
            py::array a = tensor_to_numpy(s);
            return a.attr("reshape")(-1).attr("astype")("float64").attr("tolist")();
        })
        .def("requires_grad_", [](py::object self, bool flag) {                 // marks a leaf (:2248-2272)
            PyTensor& s = self.cast<PyTensor&>();
            if (!s.t->metadata) s.t->metadata = (Meta*)calloc(1, sizeof(Meta));
            s.t->metadata->requires_grad = flag;
            s.t->metadata->is_leaf = true;
            return self;
        }, py::arg("flag") = true)
        .def("backward", [](PyTensor& s) {
            if (tensor_backward(s.t) != 0) throw std::runtime_error(std::string("backward operation failed: ") + rp_last_error());
        })
        .def("zero_grad", [](PyTensor& s) { tensor_zero_grad(s.t); })
        // ---- autograd ops ----
        .def("op_matmul", [](PyTensor& a, PyTensor& b) { return wrap(op_matmul(a.t, b.t), "op_matmul"); })
        .def("op_linear", [](PyTensor& x, PyTensor& w, py::object bias) {
            return wrap(op_linear(x.t, w.t, bias.is_none() ? nullptr : bias.cast<PyTensor&>().t), "op_linear");
        }, py::arg("weight"), py::arg("bias") = py::none())
        .def("op_conv2d", [](PyTensor& x, PyTensor& w, py::object bias, int stride_h, int stride_w, int pad_h, int pad_w, int dilation_h, int dilation_w) {
            return wrap(op_conv2d(x.t, w.t, bias.is_none() ? nullptr : bias.cast<PyTensor&>().t, stride_h, stride_w, pad_h, pad_w, dilation_h, dilation_w), "op_conv2d");
        }, py::arg("weight"), py::arg("bias") = py::none(), py::arg("stride_h") = 1, py::arg("stride_w") = 1, py::arg("pad_h") = 0, py::arg("pad_w") = 0,
             py::arg("dilation_h") = 1, py::arg("dilation_w") = 1)        // reference python/tensor_python.c:1139-1171
        .def("op_lstm_cell", [](PyTensor& x, PyTensor& h, PyTensor& c, PyTensor& w_ih, PyTensor& w_hh, py::object b_ih, py::object b_hh) {
            return wrap(op_lstm_cell(x.t, h.t, c.t, w_ih.t, w_hh.t, b_ih.is_none() ? nullptr : b_ih.cast<PyTensor&>().t,
                                     b_hh.is_none() ? nullptr : b_hh.cast<PyTensor&>().t), "op_lstm_cell");
        }, py::arg("h"), py::arg("c"), py::arg("weight_ih"), py::arg("weight_hh"), py::arg("bias_ih") = py::none(), py::arg("bias_hh") = py::none())
        .def("op_gru_cell", [](PyTensor& x, PyTensor& h, PyTensor& w_ih, PyTensor& w_hh, py::object b_ih, py::object b_hh) {
            return wrap(op_gru_cell(x.t, h.t, w_ih.t, w_hh.t, b_ih.is_none() ? nullptr : b_ih.cast<PyTensor&>().t,
                                    b_hh.is_none() ? nullptr : b_hh.cast<PyTensor&>().t), "op_gru_cell");
        }, py::arg("h"), py::arg("weight_ih"), py::arg("weight_hh"), py::arg("bias_ih") = py::none(), py::arg("bias_hh") = py::none())
        .def("op_attention", [](PyTensor& q, PyTensor& k, PyTensor& v, double scale) { return wrap(op_attention(q.t, k.t, v.t, scale), "op_attention"); },
             py::arg("k"), py::arg("v"), py::arg("scale"))
        .def("op_add", [](PyTensor& a, PyTensor& b) { return wrap(op_add(a.t, b.t), "op_add"); })
        .def("op_relu", [](PyTensor& a) { return wrap(op_relu(a.t), "op_relu"); })
        // `x.op_mul_scalar(s).op_softmax()`: the scaled tensor is a temporary that nothing can read once this call has
        // returned, which its reference count shows (g_temporary_refs, measured when the module is loaded)
        .def("op_softmax", [](py::object self, int dim) {
            PyTensor& a = self.cast<PyTensor&>();
            const bool temporary = g_temporary_refs > 0 && (int)self.ref_count() <= g_temporary_refs;
            return wrap(temporary ? op_softmax_consume(a.t, dim) : op_softmax(a.t, dim), "op_softmax");
        }, py::arg("dim") = -1)
        .def("_refs", [](py::object self, int) { return (int)self.ref_count(); }, py::arg("dim") = -1)      // the same argument shape as op_softmax: its count is the yardstick
        .def("op_log_softmax", [](PyTensor& a, int dim) { return wrap(op_log_softmax(a.t, dim), "op_log_softmax"); }, py::arg("dim") = -1)
        .def("op_mul_scalar", [](PyTensor& a, double s) { return wrap(op_mul_scalar(a.t, s), "op_mul_scalar"); })
        .def("op_sum_all", [](PyTensor& a) { return wrap(op_sum_all(a.t), "op_sum_all"); })
        .def("op_mean_all", [](PyTensor& a) { return wrap(op_mean_all(a.t), "op_mean_all"); })
        .def("op_cross_entropy_loss", [](PyTensor& a, py::object targets, const std::string& reduction, int from_logits) {
            std::vector<int> t = targets_from(targets);
            int red = reduction == "mean" ? 1 : (reduction == "sum" ? 2 : (reduction == "none" ? 0 : -1));
            if (red < 0) throw py::value_error("reduction must be 'none', 'mean' or 'sum'");
            if (a.t->ndim != 2 || (int)t.size() != a.t->shape[0]) throw std::runtime_error("op_cross_entropy_loss operation failed: one target per row of a 2-D input");
            return wrap(op_cross_entropy_loss(a.t, t.data(), a.t->shape[0], a.t->shape[1], red, from_logits), "op_cross_entropy_loss");
        }, py::arg("targets"), py::arg("reduction") = "mean", py::arg("from_logits") = -1)
        // ---- plain (no graph) variants the reference also exposes ----
        .def("add", [](PyTensor& a, PyTensor& b) {
            Tensor* r = op_add(a.t, b.t);
            return wrap(r, "add");
        })
        .def("relu", [](PyTensor& a) { return wrap(op_relu(a.t), "relu"); })
        .def("mul_scalar", [](PyTensor& a, double s) { return wrap(op_mul_scalar(a.t, s), "mul_scalar"); })
        .def("sum_all", [](PyTensor& a) {                                        // Python float, float32 / float64 only (:634-684)
            if (a.t->dtype != DTYPE_FLOAT32 && a.t->dtype != DTYPE_FLOAT64) throw std::runtime_error("sum_all returns a float for float32 / float64 tensors only");
            Tensor* dev = a.t->device_id >= 0 ? tensor_retain(a.t) : nullptr;
            double v = 0;
            if (dev) {
                TensorPtr r = wrap(op_sum_all(dev), "sum_all");
                free_tensor(dev);
                if (tensor_read_scalar(r->t, &v) != 0) throw std::runtime_error("sum_all failed");
                return v;
            }
            // host tensors: a read-out helper, summed in element order
            Tensor* h = tensor_to(a.t, -1, DTYPE_FLOAT64, false);
            for (size_t i = 0; i < h->size; i++) v += ((double*)h->data)[i];
            free_tensor(h);
            return v;
        })
        .def("mean_all", [](PyTensor& a) {
            if (a.t->dtype != DTYPE_FLOAT32 && a.t->dtype != DTYPE_FLOAT64) throw std::runtime_error("mean_all returns a float for float32 / float64 tensors only");
            double v = 0;
            if (a.t->device_id >= 0) {
                TensorPtr r = wrap(op_mean_all(a.t), "mean_all");
                if (tensor_read_scalar(r->t, &v) != 0) throw std::runtime_error("mean_all failed");
                return v;
            }
            Tensor* h = tensor_to(a.t, -1, DTYPE_FLOAT64, false);
            for (size_t i = 0; i < h->size; i++) v += ((double*)h->data)[i];
            v /= (double)h->size;
            free_tensor(h);
            return v;
        })
        // ---- views ----
        .def("transpose", [](PyTensor& a, int d0, int d1) { return wrap(op_transpose(a.t, d0, d1), "transpose"); })
        .def("permute", [](PyTensor& a, std::vector<int> dims) { return wrap(op_permute(a.t, dims.data(), (int)dims.size()), "permute"); })
        .def("reshape", [](PyTensor& a, py::object shape) { auto s = to_shape(shape); return wrap(op_reshape(a.t, (int)s.size(), s.data()), "reshape"); })
        .def("view", [](PyTensor& a, py::object shape) { auto s = to_shape(shape); return wrap(op_reshape(a.t, (int)s.size(), s.data()), "view"); })
        .def("flatten", [](PyTensor& a) { int s = -1; return wrap(op_reshape(a.t, 1, &s), "flatten"); })
        .def("contiguous", [](PyTensor& a) { return wrap(rp_is_contiguous(a.t) ? tensor_copy(a.t) : rp_contiguous(a.t), "contiguous"); })
        .def("slice", [](PyTensor& a, py::object start, py::object stop, py::object step) {
            auto get = [&](py::object o, const char* name) {
                std::vector<int> v;
                if (o.is_none()) return v;
                if (!py::isinstance<py::list>(o) && !py::isinstance<py::tuple>(o)) throw py::type_error(std::string(name) + " must be a list or tuple");
                for (auto item : o) v.push_back(item.cast<int>());
                if ((int)v.size() != a.t->ndim) throw py::value_error(std::string(name) + " must have " + std::to_string(a.t->ndim) + " elements");
                return v;
            };
            std::vector<int> b = get(start, "start"), e = get(stop, "stop"), s = get(step, "step");
            return wrap(op_slice(a.t, b.empty() ? nullptr : b.data(), e.empty() ? nullptr : e.data(), s.empty() ? nullptr : s.data()), "slice");      // reference python/tensor_python.c:2198
        }, py::arg("start") = py::none(), py::arg("stop") = py::none(), py::arg("step") = py::none())
        .def("__repr__", [](PyTensor& s) {
            std::string r = "Tensor(shape=(";
            for (int i = 0; i < s.t->ndim; i++) r += std::to_string(s.t->shape[i]) + (i + 1 < s.t->ndim ? ", " : "");
            return r + "), dtype=" + dtype_name(s.t->dtype) + ", device=" + device_name(s.t->device_id) + ")";
        });

    auto make = [](Tensor* (*ctor)(DType, int, int, int*, Meta*), const char* name) {
        return [ctor, name](py::object shape, const std::string& dtype, const std::string& device) {
            auto s = to_shape(shape);
            return wrap(ctor(parse_dtype(dtype), parse_device(device), (int)s.size(), s.data(), nullptr), name);
        };
    };
    m.def("zeros", make(zeros_tensor, "zeros"), py::arg("shape"), py::arg("dtype") = "float32", py::arg("device") = "cpu");
    m.def("ones", make(ones_tensor, "ones"), py::arg("shape"), py::arg("dtype") = "float32", py::arg("device") = "cpu");
    m.def("values", [](py::object data, const std::string& dtype, const std::string& device) {      // 1-D (reference :2882-2999)
        std::vector<double> v;
        for (auto item : data) v.push_back(item.cast<double>());
        if (v.empty()) throw py::value_error("values needs at least one element");
        int n = (int)v.size();
        return wrap(values_tensor(v.data(), DTYPE_FLOAT64, parse_dtype(dtype), -1, parse_device(device), 1, &n, nullptr), "values");
    }, py::arg("data"), py::arg("dtype") = "float32", py::arg("device") = "cpu");
    m.def("from_numpy", &from_numpy);
    m.def("randn", [](py::object shape, const std::string& dtype, const std::string& device, const std::string&) {
        auto s = to_shape(shape);
        return wrap(rp_randn(parse_dtype(dtype), parse_device(device), (int)s.size(), s.data()), "randn");
    }, py::arg("shape"), py::arg("dtype") = "float32", py::arg("device") = "cpu", py::arg("method") = "box_muller");
    m.def("rand", [](py::object shape, const std::string& dtype, const std::string& device) {
        auto s = to_shape(shape);
        return wrap(rp_rand(parse_dtype(dtype), parse_device(device), (int)s.size(), s.data()), "rand");
    }, py::arg("shape"), py::arg("dtype") = "float32", py::arg("device") = "cpu");
#ifdef RP_TEST_HOOKS
    m.def("_fail_gemm_after", [](int n) { rp_debug_fail_gemm_after(n); }, py::arg("n"));      // fault injection for tests of the error paths
#endif
    m.def("manual_seed", [](unsigned long long seed) { rp_manual_seed(seed); });
    // how a temporary looks to a method on this interpreter: call the yardstick on one, and on a named object
    try {
        py::dict scope;
        scope["T"] = m.attr("zeros");
        py::exec("named = T([1])\nn = named._refs()\nt = T([1]).copy()._refs()\nn2 = named.copy().copy()._refs()", py::globals(), scope);
        const int n = scope["n"].cast<int>(), t = scope["t"].cast<int>(), t2 = scope["n2"].cast<int>();
        if (t == t2 && t < n) g_temporary_refs = t;
    } catch (py::error_already_set& e) { g_temporary_refs = 0; }
    m.def("device_count", []() { int n = 0; for (int i = 0; i < 64 && validate_device_id(i); i++) n = i + 1; return n; });
}
