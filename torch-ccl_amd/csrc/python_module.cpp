// Python module torch_ccl_amd._C: registers the c10d backend "ccl" for ROCm ("cuda") tensors and
// exposes torch.distributed.ProcessGroupCCL(store, rank, size, timeout) -- the registration
// contract of the reference's module init (oneccl_bindings_for_pytorch/csrc/init.cpp:123-154).
#include <pybind11/chrono.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/csrc/utils/pybind.h>

#include "process_group_ccl.hpp"

namespace py = pybind11;

namespace {

// Holder that drops the GIL while the last reference dies: the backend's destructor waits
// (bounded) for the other ranks and must not stall the interpreter's other threads.
template <typename T>
class ReleaseGilHolder {
 public:
  ReleaseGilHolder() = default;
  ReleaseGilHolder(const ReleaseGilHolder&) = default;
  ReleaseGilHolder(ReleaseGilHolder&&) noexcept = default;
  ReleaseGilHolder& operator=(const ReleaseGilHolder&) = default;
  ReleaseGilHolder& operator=(ReleaseGilHolder&&) noexcept = default;
  /* implicit */ ReleaseGilHolder(c10::intrusive_ptr<T> p) : p_(std::move(p)) {}
  explicit ReleaseGilHolder(T* raw) : p_(c10::intrusive_ptr<T>::unsafe_steal_from_new(raw)) {}
  ~ReleaseGilHolder() {
    if (p_ && p_.use_count() == 1 && Py_IsInitialized() && PyGILState_Check()) {
      py::gil_scoped_release nogil;
      p_.reset();
    }
  }
  T* get() const noexcept { return p_.get(); }
  T& operator*() const noexcept { return *p_; }
  T* operator->() const noexcept { return p_.get(); }
  explicit operator bool() const noexcept { return (bool)p_; }

 private:
  c10::intrusive_ptr<T> p_;
};

}  // namespace

PYBIND11_DECLARE_HOLDER_TYPE(T, ReleaseGilHolder<T>, true)

PYBIND11_MODULE(_C, m) {
  using mccl_pg::ProcessGroupCCL;
  m.doc() = "c10d backend 'ccl' on MI355X: local-reduce and pack/permute kernels behind ProcessGroupCCL";

  py::object dist = py::module::import("torch.distributed");
  py::object register_backend = dist.attr("Backend").attr("register_backend");
  py::object backend_base = py::module::import("torch._C._distributed_c10d").attr("Backend");

  py::object creator = py::cpp_function(
      &ProcessGroupCCL::create, py::arg("store"), py::arg("rank"), py::arg("size"),
      py::arg("timeout") = std::chrono::milliseconds(ProcessGroupCCL::OP_TIMEOUT_MILLIS),
      py::call_guard<py::gil_scoped_release>());
  m.attr("create_process_group") = creator;

  m.def("register", [register_backend, creator](const std::string& name) {
    register_backend(name, creator, false, std::vector<std::string>{"cuda"});
  });

  // a Work without device work behind it, for tests of wait(timeout) that need no GPU
  m.def("_pending_work", &ProcessGroupCCL::pendingWork, py::arg("rank"), py::arg("polls"), py::arg("op_timeout"));

  py::class_<ProcessGroupCCL, ReleaseGilHolder<ProcessGroupCCL>>(m, "ProcessGroupCCL", backend_base)
      .def(py::init([](const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
                       std::chrono::milliseconds timeout) {
             return ReleaseGilHolder<ProcessGroupCCL>(
                 c10::make_intrusive<ProcessGroupCCL>(store, rank, size, timeout));
           }),
           py::arg("store"), py::arg("rank"), py::arg("size"),
           py::arg("timeout") = std::chrono::milliseconds(ProcessGroupCCL::OP_TIMEOUT_MILLIS))
      // what the bisecting switches of the environment parsed to: 1 = work only, 2 = sync only, + 4 = allreduce disabled
      .def("_bisect_mode", &ProcessGroupCCL::bisectMode)
      // collectives of this group that met at the host rendezvous / that reused a cached one
      .def("_rendezvous_counts", &ProcessGroupCCL::rendezvousCounts)
      // which way the collective this rank enqueued last took (what the verbose log prints)
      .def("_last_path", &ProcessGroupCCL::lastPath);
}
