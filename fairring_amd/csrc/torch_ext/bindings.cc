// Python module _fairring: ProcessGroup and ProcessGroup.Options, as the
// reference binds them (fairring/bindings.cc:20-47), on the c10d::Backend base
// that current PyTorch exposes as torch._C._distributed_c10d.Backend.
#include <pybind11/chrono.h>
#include <pybind11/pybind11.h>
#include <torch/csrc/utils/pybind.h>

#include "process_group.h"

namespace py = pybind11;

using fairring::ProcessGroupFairring;

PYBIND11_MODULE(_fairring, module) {
  py::module::import("torch.distributed");

  py::class_<ProcessGroupFairring, c10::intrusive_ptr<ProcessGroupFairring>, c10d::Backend>
      processGroupFairring(module, "ProcessGroup");

  py::class_<ProcessGroupFairring::OptionsFairring,
             c10::intrusive_ptr<ProcessGroupFairring::OptionsFairring>, c10d::Backend::Options>(
      processGroupFairring, "Options")
      .def(py::init<int64_t, int64_t, int64_t, bool, std::chrono::milliseconds, int64_t>(),
           py::arg("max_memory_allocated_in_bytes"),
           py::arg("max_padding_allocated_in_bytes"), py::arg("min_parallelism"),
           py::arg("is_high_priority_stream") = false,
           py::arg("timeout") = kBackendDefaultTimeout,
           py::arg("slice_size_in_bytes") = static_cast<int64_t>(0));

  processGroupFairring
      .def(py::init<const c10::intrusive_ptr<c10d::Store>&, int, int,
                    c10::intrusive_ptr<ProcessGroupFairring::OptionsFairring>>(),
           py::call_guard<py::gil_scoped_release>())
      .def("_set_simulated_peer_contributions",
           &ProcessGroupFairring::setSimulatedPeerContributions, py::arg("peers"),
           py::call_guard<py::gil_scoped_release>())
      .def("_set_fused_divide", &ProcessGroupFairring::setFusedDivide, py::arg("on"))
      .def("_layout", &ProcessGroupFairring::layout);
}
