// pybind11 module `sparseops_backend`: the reference's Python surface
// (src/bindings.cpp:50-216) on top of the HIP implementation.  Same names, argument
// meaning and error behaviour (RuntimeError for X.ndim != 2, X.shape[0] != E.n,
// bias.size != E.m); additions are marked "extension".
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>

#include "../bench/data_gen.hpp"
#include "device.hpp"
#include "ellpack_encoder.hpp"
#include "ellpack_matmul.hpp"
#include "ellpack_matvec.hpp"
#include "onnx_wire.hpp"
#include "rbm_conv.hpp"
#include "sparse_onnx.hpp"

namespace py = pybind11;
using farray = py::array_t<float, py::array::c_style | py::array::forcecast>;

namespace {

template <typename T>
py::array_t<T> copy_2d(const T *src, uint32_t rows, uint32_t cols)
{
    py::array_t<T> out({py::ssize_t(rows), py::ssize_t(cols)});
    if (rows && cols) std::memcpy(out.mutable_data(), src, std::size_t(rows) * cols * sizeof(T));
    return out;
}

const float *optional_bias(const py::object &bias, farray &holder, uint32_t m)
{
    if (bias.is_none()) return nullptr;
    holder = farray::ensure(bias);
    if (!holder) throw std::runtime_error("bias must be convertible to a float32 array");
    if (uint64_t(holder.size()) != m) throw std::runtime_error("Bias length must equal E.m");
    return holder.data();
}

} // namespace

PYBIND11_MODULE(sparseops_backend, mod)
{
    mod.doc() = "Sparse ELLPACK kernels on AMD MI355X (HIP); drop-in for the CPU sparseops_backend";

    py::class_<Ellpack>(mod, "Ellpack")
        .def_readonly("m", &Ellpack::m)
        .def_readonly("n", &Ellpack::n)
        .def_readonly("r", &Ellpack::r)
        .def_property_readonly("Wd", [](const Ellpack &E) { return copy_2d(E.Wd.ptr, E.m, E.r); })
        .def_property_readonly("idx", [](const Ellpack &E) { return copy_2d(E.idx.data(), E.m, E.r); })
        // The reference exposes its host gather scratch; it is unused here and reads as zeros.
        .def_property_readonly("Xt", [](const Ellpack &E) {
            py::array_t<float> out({py::ssize_t(E.m), py::ssize_t(E.r)});
            if (out.size()) std::memset(out.mutable_data(), 0, std::size_t(out.size()) * sizeof(float));
            return out;
        })
        // extension: per-row stored-nonzero counts
        .def_property_readonly("nnz", [](const Ellpack &E) {
            py::array_t<uint32_t> out(py::ssize_t(E.m));
            if (E.m) std::memcpy(out.mutable_data(), E.nnz.data(), std::size_t(E.m) * sizeof(uint32_t));
            return out;
        });

    mod.def("convert_to_ellpack", [](farray W) {
        if (W.ndim() != 2) throw std::runtime_error("W must be 2D (m x n)");
        return convert_to_ellpack(W.data(), uint32_t(W.shape(0)), uint32_t(W.shape(1)));
    }, "Convert dense NumPy matrix -> ELLPACK handle");

    mod.def("decode_from_ellpack", [](const Ellpack &E) {
        py::array_t<float> W({py::ssize_t(E.m), py::ssize_t(E.n)});
        decode_from_ellpack(E, W.mutable_data());
        return W;
    }, "Convert ELLPACK handle -> dense NumPy matrix");

    mod.def("ellpack_matvec", [](const Ellpack &E, farray x, py::object bias) {
        if (uint64_t(x.size()) != E.n) throw std::runtime_error("Input length must equal E.n");
        farray holder;
        const float *b = optional_bias(bias, holder, E.m);
        py::array_t<float> y(py::ssize_t(E.m));
        {
            py::gil_scoped_release nogil;
            ellpack_matvec(E, x.data(), b, y.mutable_data());
        }
        return y;
    }, py::arg("E"), py::arg("x"), py::arg("bias") = py::none(), "y = E @ x + bias (ELLPACK, on the GPU)");

    mod.def("ellpack_matmul", [](const Ellpack &E, farray X, py::object bias) {
        if (X.ndim() != 2) throw std::runtime_error("X must be 2D (n × C)");
        if (uint32_t(X.shape(0)) != E.n) throw std::runtime_error("Input row count must equal E.n");
        farray holder;
        const float *b = optional_bias(bias, holder, E.m);
        const uint32_t C = uint32_t(X.shape(1));
        py::array_t<float> Y({py::ssize_t(E.m), py::ssize_t(C)});
        {
            py::gil_scoped_release nogil;
            ellpack_matmul(E, X.data(), C, b, Y.mutable_data());
        }
        return Y;
    }, py::arg("E"), py::arg("X"), py::arg("bias") = py::none(),
       "Y = E @ X + bias[:, None] (ELLPACK x dense, on the GPU); X is (n, C), returns (m, C)");

    // extension: whether the HIP path can run in this process
    mod.def("device_available", []() {
        int n = 0;
        return so_device_count(&n) == SO_OK && n > 0;
    });

    // extension: what the built-in protobuf reader sees in an .onnx file (no device needed)
    mod.def("parse_onnx", [](const std::string &path) {
        const onnxwire::Model m = onnxwire::load_model(path);
        py::dict out;
        out["ir_version"] = m.ir_version;
        out["producer_name"] = m.producer_name;
        py::list opsets;
        for (const auto &o : m.opset_import) opsets.append(py::make_tuple(o.first, o.second));
        out["opset_import"] = opsets;
        py::list nodes;
        for (const auto &n : m.graph.node) {
            py::dict d, attrs;
            d["op_type"] = n.op_type;
            d["name"] = n.name;
            d["input"] = n.input;
            d["output"] = n.output;
            for (const auto &a : n.attribute) {
                if (!a.ints.empty()) attrs[py::str(a.name)] = a.ints;
                else if (!a.floats.empty()) attrs[py::str(a.name)] = a.floats;
                else if (a.type == 1) attrs[py::str(a.name)] = a.f;
                else if (a.type == 3) attrs[py::str(a.name)] = py::bytes(a.s);
                else attrs[py::str(a.name)] = a.i;
            }
            d["attrs"] = attrs;
            nodes.append(d);
        }
        out["nodes"] = nodes;
        py::dict inits;
        for (const auto &t : m.graph.initializer) {
            std::vector<py::ssize_t> shape(t.dims.begin(), t.dims.end());
            py::array_t<float> a(shape);
            const std::vector<float> v = t.floats();
            if (!v.empty()) std::memcpy(a.mutable_data(), v.data(), v.size() * sizeof(float));
            inits[py::str(t.name)] = a;
        }
        out["initializers"] = inits;
        auto vis = [](const std::vector<onnxwire::ValueInfo> &v) {
            py::list l;
            for (const auto &vi : v) {
                py::list dims;
                for (const auto &d : vi.dims) {
                    if (d.has_value) dims.append(d.value);
                    else dims.append(d.param);
                }
                l.append(py::make_tuple(vi.name, py::tuple(dims)));
            }
            return l;
        };
        out["inputs"] = vis(m.graph.input);
        out["outputs"] = vis(m.graph.output);
        return out;
    });

    // The row-block-merged plan (include/rbm_conv.hpp of the reference; not bound there).
    py::class_<RBMBlock>(mod, "RBMBlock")
        .def_readonly("M0", &RBMBlock::M0)
        .def_readonly("Ct", &RBMBlock::Ct)
        .def_property_readonly("krel", [](const RBMBlock &b) { return py::array_t<uint32_t>(py::ssize_t(b.krel.size()), b.krel.data()); })
        .def_property_readonly("colptr", [](const RBMBlock &b) { return py::array_t<uint32_t>(py::ssize_t(b.colptr.size()), b.colptr.data()); })
        .def_property_readonly("pair_row", [](const RBMBlock &b) {
            py::array_t<uint16_t> out(py::ssize_t(b.pairs.size()));
            for (std::size_t i = 0; i < b.pairs.size(); ++i) out.mutable_data()[i] = b.pairs[i].row;
            return out;
        })
        .def_property_readonly("pair_w", [](const RBMBlock &b) {
            py::array_t<float> out(py::ssize_t(b.pairs.size()));
            for (std::size_t i = 0; i < b.pairs.size(); ++i) out.mutable_data()[i] = b.pairs[i].w;
            return out;
        })
        .def_property_readonly("bias", [](const RBMBlock &b) { return py::array_t<float>(py::ssize_t(b.bias.size()), b.bias.data()); });
    py::class_<RBMPlan>(mod, "RBMPlan")
        .def_readonly("M", &RBMPlan::M)
        .def_readonly("N", &RBMPlan::N)
        .def_readonly("Ct_max", &RBMPlan::Ct_max)
        .def_property_readonly("blocks", [](const RBMPlan &p) { return p.blocks; });
    mod.def("build_rbm_from_ellpack", [](const Ellpack &E, const py::object &bias, uint32_t Ct_max) {
        farray holder;
        return build_rbm_from_ellpack(E, optional_bias(bias, holder, E.m), Ct_max);
    }, py::arg("E"), py::arg("bias") = py::none(), py::arg("Ct_max") = 8,
       "Row-block-merged re-encoding of an ELLPACK matrix (blocks of Ct_max rows, union columns, (row, weight) pairs)");

    // The benchmark harness's generator (bench/data_gen.hpp; the reference's recipe,
    // benchmark-mkl/common/data_gen.cpp:23-96): what bench_vendor runs for the same arguments.
    mod.def("benchmark_dense", [](int64_t M, int64_t N, double sparsity, uint64_t seed, bool irregular) {
        if (M < 0 || N < 0 || !(sparsity >= 0.0 && sparsity <= 1.0)) throw std::runtime_error("benchmark_dense: bad arguments");
        const std::vector<float> W = sparseops_bench::dense_matrix(M, N, sparsity, seed, irregular);
        py::array_t<float> out({py::ssize_t(M), py::ssize_t(N)});
        std::copy(W.begin(), W.end(), out.mutable_data());
        return out;
    }, py::arg("M"), py::arg("N"), py::arg("sparsity"), py::arg("seed") = 42, py::arg("irregular") = false,
       "Dense (M, N) float32 matrix of the benchmark recipe: Bernoulli(1 - sparsity) mask over N(0, 1) values");
    mod.def("benchmark_operand", [](py::ssize_t rows, py::ssize_t cols, uint64_t seed) {
        if (rows < 0 || cols < 0) throw std::runtime_error("benchmark_operand: bad arguments");
        const std::vector<float> X = sparseops_bench::dense_operand(std::size_t(rows) * std::size_t(cols), seed);
        py::array_t<float> out({rows, cols});
        std::copy(X.begin(), X.end(), out.mutable_data());
        return out;
    }, py::arg("rows"), py::arg("cols"), py::arg("seed") = 42, "Dense (rows, cols) float32 operand, uniform in [-1, 1)");
    mod.def("reload_tuning", []() { sparseops::check(so_tuning_reload(sparseops::context()), "so_tuning_reload"); },
            "Read the SPARSEOPS_* tuning overrides from the environment again (they are read when the process-wide "
            "context is created); models pick the change up at their next resize_buffers");

    py::class_<SparseOnnxModel>(mod, "SparseOnnxModel")
        .def(py::init<const std::string &>(), "Load an ONNX model and pre-encode weights to ELLPACK")
        .def("run", [](const SparseOnnxModel &model, py::array X) {
            // Accepts a (B, ...) array in either memory order and returns the
            // (B, ...) result a framework would: a Fortran-ordered 2-D input is
            // already [features x B] and is used as is (what the reference's model
            // tests feed, tests/full_test.py:77-80); anything else is taken in C
            // order and transposed on the device.
            if (X.ndim() < 2) throw std::runtime_error("Input tensor must have rank >= 2");
            const uint32_t B = uint32_t(X.shape(0));
            if (B == 0) throw std::runtime_error("Input batch must be positive");
            if (uint64_t(X.size()) != uint64_t(B) * model.input_features())
                throw std::runtime_error("Input has " + std::to_string(X.size() / B) + " features per sample, model expects " +
                                         std::to_string(model.input_features()));
            const bool f32 = py::isinstance<py::array_t<float>>(X);
            const bool fortran2d = f32 && X.ndim() == 2 && (X.flags() & py::array::f_style) && !(X.flags() & py::array::c_style);
            if (fortran2d) {
                const float *in = static_cast<const float *>(X.data());
                std::vector<std::size_t> shape{B, model.output_features()};
                py::array_t<float, py::array::f_style> Y(shape);
                {
                    py::gil_scoped_release nogil;
                    model.run(in, B, Y.mutable_data());
                }
                return py::array(Y);
            }
            farray Xc = farray::ensure(X);
            if (!Xc) throw std::runtime_error("Input must be convertible to a float32 array");
            std::vector<std::size_t> shape = model.output_shape();
            shape[0] = B;
            py::array_t<float> Y(shape);
            {
                py::gil_scoped_release nogil;
                model.run_batch_major(Xc.data(), B, Y.mutable_data());
            }
            return py::array(Y);
        }, "Run inference on a (B, ...) input; returns the (B, ...) output")
        .def("run_device", [](const SparseOnnxModel &model, std::uintptr_t d_input, uint32_t B, std::uintptr_t d_output) {
            // Device pointers as integers (e.g. the .ptr of a ctypes-side allocation on the same
            // device): [input_features x B] in, [output_features x B] out, both in HBM.  Waits for the
            // chain, so the caller may read d_output from any stream afterwards.
            py::gil_scoped_release nogil;
            model.run_device(reinterpret_cast<const float *>(d_input), B, reinterpret_cast<float *>(d_output));
            sparseops::check(so_sync(sparseops::context()), "so_sync");
        }, py::arg("d_input"), py::arg("B"), py::arg("d_output"),
           "Run the layer chain on device buffers ([features x B] row-major); no host copies")
        .def("resize_buffers", &SparseOnnxModel::resize_buffers, py::arg("batch"),
             "Pre-size every activation buffer for `batch` samples (run() then allocates nothing)")
        .def("output_shape", &SparseOnnxModel::output_shape)
        .def("input_shape", &SparseOnnxModel::input_shape)
        .def("batch", &SparseOnnxModel::batch)
        .def("time_device", &SparseOnnxModel::time_device, py::arg("steps"), py::arg("warmup") = 3)
        .def("describe", &SparseOnnxModel::describe)
        .def("nnz_flops_per_sample", &SparseOnnxModel::nnz_flops_per_sample);
}
