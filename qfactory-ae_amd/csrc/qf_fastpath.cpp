// Host-side fast path of QLinear.forward(x): one native call that validates the activation, allocates the
// output with torch's caching allocator and calls the specialisation's C-ABI `launch` through its address.
//
// The reference's forward allocates in Python and goes through a ctypes closure that re-checks five tensors
// per call (qfactory/qlinear.py:52-61, qfactory/core/matmul.py:124-151).  At one row the kernels here run in
// 4 - 10 us, so that interpreter work (tensor attribute reads, torch.empty's argument parsing, the ctypes
// marshalling of eight arguments) is what a caller in eager mode waits for.  Nothing here touches HIP: the
// stream handle comes from the caller and the launch goes through the function pointer, so the module
// builds with the host compiler alone and loads without a GPU.
//
// Built in-tree by qfactory.fastpath.build() (g++ against the installed torch's headers and libraries).
#include <torch/extension.h>

#include <cstdint>
#include <stdexcept>
#include <string>

namespace {

// include/qfactory_launch.h: launch(m, activation, weight, output, scale, zero, stream, rc) for grouped layers,
// launch(m, activation, weight, output, stream, rc) for layers without scales
using launch_grouped_t = void (*)(int, void*, void*, void*, void*, void*, void*, int*);
using launch_plain_t = void (*)(int, void*, void*, void*, void*, int*);

class BoundLaunch {
public:
    BoundLaunch(std::uintptr_t fn, std::uintptr_t weight, std::uintptr_t scale, std::uintptr_t zero, bool grouped,
                std::int64_t n, std::int64_t k, at::ScalarType dtype, int device_index)
        : fn_(reinterpret_cast<void*>(fn)), w_(reinterpret_cast<void*>(weight)), s_(reinterpret_cast<void*>(scale)),
          z_(reinterpret_cast<void*>(zero)), grouped_(grouped), n_(n), k_(k), dtype_(dtype), device_(device_index) {
        if (fn_ == nullptr) throw std::invalid_argument("BoundLaunch: null launch address");
    }

    // Launch into a caller's (m, n) output: the return code of `launch`, or None when either tensor is not what
    // the specialisation was bound for.
    py::object into(const at::Tensor& x, const at::Tensor& out, std::uintptr_t stream) const {
        if (!accepts(x) || out.dim() != 2 || out.size(0) != x.size(0) || out.size(1) != n_ || out.scalar_type() != dtype_ ||
            !out.is_contiguous() || !out.device().is_cuda() || out.device().index() != device_)
            return py::none();
        return py::int_(x.size(0) > 0 ? run(x, out, stream) : 0);
    }

    // (m, k) activation -> freshly allocated (m, n) output with the launch enqueued on `stream`.  None when the
    // activation is not what the specialisation was bound for: the caller's slower path then names the problem.
    py::object operator()(const at::Tensor& x, std::uintptr_t stream) const {
        if (!accepts(x)) return py::none();
        at::Tensor out = at::empty({x.size(0), n_}, x.options());
        if (x.size(0) > 0) {
            const int rc = run(x, out, stream);
            if (rc != 0)
                throw std::runtime_error("quantized linear launch failed with return code " + std::to_string(rc));
        }
        return py::cast(out);
    }

private:
    bool accepts(const at::Tensor& x) const {
        return x.dim() == 2 && x.size(1) == k_ && x.scalar_type() == dtype_ && x.is_contiguous() &&
               x.device().is_cuda() && x.device().index() == device_;
    }

    int run(const at::Tensor& x, const at::Tensor& out, std::uintptr_t stream) const {
        int rc = 0;
        const int m = static_cast<int>(x.size(0));
        void* sp = reinterpret_cast<void*>(stream);
        if (grouped_)
            reinterpret_cast<launch_grouped_t>(fn_)(m, x.data_ptr(), w_, out.data_ptr(), s_, z_, sp, &rc);
        else
            reinterpret_cast<launch_plain_t>(fn_)(m, x.data_ptr(), w_, out.data_ptr(), sp, &rc);
        return rc;
    }

    void *fn_, *w_, *s_, *z_;
    bool grouped_;
    std::int64_t n_, k_;
    at::ScalarType dtype_;
    int device_;
};

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "allocate-and-launch fast path of the quantized linear layers";
#ifdef QF_FASTPATH_SOURCE_DIGEST
    m.attr("source_digest") = QF_FASTPATH_SOURCE_DIGEST;      // md5 of this file at build time: load() refuses a stale build
#endif
    py::class_<BoundLaunch>(m, "BoundLaunch")
        .def(py::init<std::uintptr_t, std::uintptr_t, std::uintptr_t, std::uintptr_t, bool, std::int64_t, std::int64_t,
                      at::ScalarType, int>(),
             py::arg("fn"), py::arg("weight"), py::arg("scale"), py::arg("zero"), py::arg("grouped"), py::arg("n"),
             py::arg("k"), py::arg("dtype"), py::arg("device_index"))
        .def("__call__", &BoundLaunch::operator(), py::arg("activation"), py::arg("stream"))
        .def("into", &BoundLaunch::into, py::arg("activation"), py::arg("output"), py::arg("stream"));
}
