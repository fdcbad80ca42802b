// pybind11 module `hip_ext`: the HIP counterpart of the reference's `metal_ext`
// (metal_ext.mm:770-796).  HipContext exposes the same method names the Python
// host layer calls on MetalContext and forwards each one to the C ABI of
// libautograd_hip.so; no kernel code lives here.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/autograd_hip.h"

namespace py = pybind11;

namespace {

void raise_for(int rc) {
    if (rc == AGRAD_OK) return;
    const std::string msg = agrad_last_error();
    switch (rc) {
        case AGRAD_EINDEX: throw py::index_error(msg);
        case AGRAD_EINVAL: throw py::value_error(msg);
        case AGRAD_EWORKSPACE: throw py::value_error(msg);
        default: throw std::runtime_error(msg);
    }
}

uint32_t float_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}

class HipContext {
public:
    explicit HipContext(int device = 0) { raise_for(agrad_ctx_create(device, &ctx_)); }
    ~HipContext() { agrad_ctx_destroy(ctx_); }
    HipContext(const HipContext&) = delete;
    HipContext& operator=(const HipContext&) = delete;

    uint64_t max_buffer_length() {
        uint64_t v = 0;
        raise_for(agrad_max_buffer_length(ctx_, &v));
        return v;
    }
    uint64_t alloc(uint64_t bytes) {
        uint64_t id = 0;
        raise_for(agrad_alloc(ctx_, bytes, &id));
        return id;
    }
    void free(uint64_t id) { raise_for(agrad_free(ctx_, id)); }
    void begin_pass() { raise_for(agrad_begin_pass(ctx_)); }
    void end_pass() {
        py::gil_scoped_release nogil;
        int rc = agrad_end_pass(ctx_);
        py::gil_scoped_acquire gil;
        raise_for(rc);
    }
    // record the launches between graph_begin and graph_end, replay them with graph_launch
    void graph_begin() { raise_for(agrad_graph_begin(ctx_)); }
    // column sums that backward launches with DEFER_PARAM_GRAD left unfolded: fold them all / count them
    void finalize_param_grads() { raise_for(agrad_finalize_param_grads(ctx_)); }
    uint32_t pending_param_grads() {
        uint32_t n = 0;
        raise_for(agrad_pending_param_grads(ctx_, &n));
        return n;
    }
    uint64_t graph_end() {
        uint64_t id = 0;
        raise_for(agrad_graph_end(ctx_, &id));
        return id;
    }
    void graph_launch(uint64_t id) { raise_for(agrad_graph_launch(ctx_, id)); }
    void graph_destroy(uint64_t id) { raise_for(agrad_graph_destroy(ctx_, id)); }
    void synchronize() {
        py::gil_scoped_release nogil;
        int rc = agrad_synchronize(ctx_);
        py::gil_scoped_acquire gil;
        raise_for(rc);
    }
    // GPU time between the two calls, in the spirit of begin/end_pass_profiled
    // (metal_ext.mm:215-286): returns {"gpu_ms": ...}.
    void begin_pass_profiled() { raise_for(agrad_timer_start(ctx_)); }
    py::dict end_pass_profiled() {
        float ms = 0.0f;
        raise_for(agrad_timer_stop(ctx_, &ms));
        raise_for(agrad_end_pass(ctx_));
        py::dict d;
        d["gpu_ms"] = ms;
        return d;
    }

    void dispatch_with_args_3d(const std::string& name, const std::vector<uint64_t>& ids,
                               const std::vector<uint64_t>& offs, const std::vector<uint32_t>& args,
                               uint64_t gx, uint64_t gy, uint64_t gz, uint64_t tg) {
        if (ids.size() != offs.size()) throw py::value_error("buffer_ids and offsets differ in length");
        raise_for(agrad_dispatch(ctx_, name.c_str(), ids.data(), offs.data(), (int)ids.size(), args.data(),
                                 (int)args.size(), gx, gy, gz, tg));
    }

    // dst[dense index] (+)= src[strided index]: the reference's dispatch_contiguous and
    // dispatch_strided (metal_ext.mm:512-557) with the element type and the write mode
    // as optional trailing arguments; grid_size is implied by the shape
    void dispatch_gather_strided(const std::string& name, uint64_t src_id, uint64_t src_off, uint64_t dst_id,
                                 uint64_t dst_off, const std::vector<uint32_t>& shape,
                                 const std::vector<uint64_t>& strides, uint64_t grid_size, int dtype,
                                 uint32_t flags) {
        (void)grid_size;
        if (shape.size() != strides.size()) throw py::value_error("shape and strides differ in length");
        if (shape.size() > AGRAD_MAX_DIMS) throw py::value_error("too many dimensions");
        std::vector<uint32_t> args(3 + 3 * AGRAD_MAX_DIMS, 0u);
        args[0] = (uint32_t)dtype;
        args[1] = flags;
        args[2] = (uint32_t)shape.size();
        for (size_t i = 0; i < shape.size(); ++i) {
            args[3 + i] = shape[i];
            args[3 + AGRAD_MAX_DIMS + 2 * i] = (uint32_t)(strides[i] & 0xffffffffull);
            args[3 + AGRAD_MAX_DIMS + 2 * i + 1] = (uint32_t)(strides[i] >> 32);
        }
        const uint64_t ids[2] = {src_id, dst_id}, offs[2] = {src_off, dst_off};
        raise_for(agrad_dispatch(ctx_, name.c_str(), ids, offs, 2, args.data(), (int)args.size(), 0, 0, 0, 0));
    }

    void fill_scalar(const std::string& name, const std::vector<uint64_t>& ids,
                     const std::vector<uint64_t>& offs, float value, uint64_t n) {
        (void)name;
        if (ids.size() != 1 || offs.size() != 1) throw py::value_error("fill_scalar takes one buffer");
        raise_for(agrad_fill(ctx_, ids[0], offs[0], float_bits(value), 4, n));
    }
    void fill_scalar2(const std::string& name, const std::vector<uint64_t>& ids,
                      const std::vector<uint64_t>& offs, uint32_t bits, int itemsize, uint64_t n) {
        (void)name;
        if (ids.size() != 1 || offs.size() != 1) throw py::value_error("fill_scalar2 takes one buffer");
        raise_for(agrad_fill(ctx_, ids[0], offs[0], bits, itemsize, n));
    }

    // Any C-contiguous array; bytes are copied as they are.
    void copy_from_host(uint64_t id, uint64_t off, py::array host) {
        py::array c = py::array::ensure(host, py::array::c_style);
        if (!c) throw py::value_error("copy_from_host needs an array");
        raise_for(agrad_copy_from_host(ctx_, id, off, c.data(), (uint64_t)c.nbytes()));
    }
    py::array copy_to_host(uint64_t id, uint64_t off, const std::vector<py::ssize_t>& shape,
                           const std::string& dtype) {
        py::array out(py::dtype(dtype), shape);
        raise_for(agrad_copy_to_host(ctx_, id, off, out.mutable_data(), (uint64_t)out.nbytes()));
        return out;
    }

    uint64_t norm_backward_workspace_bytes(uint64_t rows, uint32_t C, int dtype) {
        return agrad_norm_backward_workspace_bytes(rows, C, dtype);
    }
    uint64_t embedding_sort_workspace_bytes(uint64_t N, uint32_t V) {
        return agrad_embedding_sort_workspace_bytes(N, V);
    }
    uint64_t embedding_backward_sorted_workspace_bytes(uint64_t N, uint32_t C) {
        return agrad_embedding_backward_sorted_workspace_bytes(N, C);
    }
    uint64_t broadcast_grad_workspace_bytes(uint64_t lead, uint64_t inner) {
        return agrad_broadcast_grad_workspace_bytes(lead, inner);
    }
    uint64_t gelu_bias_backward_workspace_bytes(uint64_t rows, uint32_t C) {
        return agrad_gelu_bias_backward_workspace_bytes(rows, C);
    }
    uint64_t mul_backward_workspace_bytes(int kind, uint64_t lead, uint64_t inner) {
        return agrad_mul_backward_workspace_bytes(kind, lead, inner);
    }
    uint64_t embedding_backward_workspace_bytes(uint64_t N, uint32_t C, uint32_t V, int dtype) {
        return agrad_embedding_backward_workspace_bytes(N, C, V, dtype);
    }
    std::vector<std::string> kernel_names() {
        std::vector<std::string> v;
        for (int i = 0; i < agrad_kernel_count(); ++i) v.push_back(agrad_kernel_name(i));
        return v;
    }
    py::object kernel_signature(const std::string& name) {
        const char* s = agrad_kernel_signature(name.c_str());
        if (s == nullptr) return py::none();
        return py::str(s);
    }
    // agrad_ctx* as an integer, for callers that bind the C ABI with ctypes
    uint64_t handle() { return reinterpret_cast<uint64_t>(ctx_); }

private:
    agrad_ctx* ctx_ = nullptr;
};

}  // namespace

PYBIND11_MODULE(hip_ext, m) {
    m.doc() = "MI355X (gfx950) native context for the autograd fused layer-op path";
    m.attr("F32") = (int)AGRAD_F32;
    m.attr("BF16") = (int)AGRAD_BF16;
    m.attr("ACC_INPUT_GRAD") = (unsigned)AGRAD_ACC_INPUT_GRAD;
    m.attr("ACC_PARAM_GRAD") = (unsigned)AGRAD_ACC_PARAM_GRAD;
    m.attr("ACC_PARAM_GRAD2") = (unsigned)AGRAD_ACC_PARAM_GRAD2;
    m.attr("DEFER_PARAM_GRAD") = (unsigned)AGRAD_DEFER_PARAM_GRAD;
    m.attr("PARAM_GRAD_BF16") = (unsigned)AGRAD_PARAM_GRAD_BF16;
    m.def("device_count", [] {
        int n = 0;
        agrad_device_count(&n);
        return n;
    });
    py::class_<HipContext>(m, "HipContext")
        .def(py::init<int>(), py::arg("device") = 0)
        .def("max_buffer_length", &HipContext::max_buffer_length)
        .def("alloc", &HipContext::alloc)
        .def("free", &HipContext::free)
        .def("begin_pass", &HipContext::begin_pass)
        .def("end_pass", &HipContext::end_pass)
        .def("begin_pass_profiled", &HipContext::begin_pass_profiled)
        .def("end_pass_profiled", &HipContext::end_pass_profiled)
        .def("dispatch_with_args_3d", &HipContext::dispatch_with_args_3d)
        .def("dispatch_contiguous", &HipContext::dispatch_gather_strided, py::arg("kernel_name"),
             py::arg("x_id"), py::arg("x_offset"), py::arg("out_id"), py::arg("out_offset"), py::arg("shape"),
             py::arg("strides"), py::arg("grid_size") = 0, py::arg("dtype") = (int)AGRAD_F32, py::arg("flags") = 0u)
        .def("dispatch_strided", &HipContext::dispatch_gather_strided, py::arg("kernel_name"),
             py::arg("grad_out_id"), py::arg("grad_out_offset"), py::arg("grad_x_id"), py::arg("grad_x_offset"),
             py::arg("shape"), py::arg("strides"), py::arg("grid_size") = 0, py::arg("dtype") = (int)AGRAD_F32,
             py::arg("flags") = 0u)
        .def("fill_scalar", &HipContext::fill_scalar)
        .def("fill_scalar2", &HipContext::fill_scalar2)
        .def("copy_from_host", &HipContext::copy_from_host)
        .def("copy_to_host", &HipContext::copy_to_host, py::arg("buffer_id"), py::arg("offset"),
             py::arg("shape"), py::arg("dtype") = "float32")
        .def("norm_backward_workspace_bytes", &HipContext::norm_backward_workspace_bytes)
        .def("embedding_backward_workspace_bytes", &HipContext::embedding_backward_workspace_bytes)
        .def("broadcast_grad_workspace_bytes", &HipContext::broadcast_grad_workspace_bytes)
        .def("mul_backward_workspace_bytes", &HipContext::mul_backward_workspace_bytes)
        .def("gelu_bias_backward_workspace_bytes", &HipContext::gelu_bias_backward_workspace_bytes)
        .def("embedding_sort_workspace_bytes", &HipContext::embedding_sort_workspace_bytes)
        .def("embedding_backward_sorted_workspace_bytes", &HipContext::embedding_backward_sorted_workspace_bytes)
        .def("kernel_names", &HipContext::kernel_names)
        .def("kernel_signature", &HipContext::kernel_signature)
        .def("handle", &HipContext::handle)
        .def("finalize_param_grads", &HipContext::finalize_param_grads)
        .def("pending_param_grads", &HipContext::pending_param_grads)
        .def("graph_begin", &HipContext::graph_begin)
        .def("graph_end", &HipContext::graph_end)
        .def("graph_launch", &HipContext::graph_launch)
        .def("graph_destroy", &HipContext::graph_destroy)
        .def("synchronize", &HipContext::synchronize);
}
