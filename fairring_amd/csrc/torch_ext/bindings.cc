// Python module _fairring. It exposes the same two names the reference's
// module does (fairring/bindings.cc:20-47): ProcessGroup, constructed from
// (store, rank, size, options) with the GIL released, and the nested
// ProcessGroup.Options with keyword-capable staging parameters. The base class
// is c10d::Backend, which current PyTorch shows to Python as
// torch._C._distributed_c10d.Backend.
#include <pybind11/chrono.h>
#include <pybind11/pybind11.h>
#include <torch/csrc/utils/pybind.h>

#include "process_group.h"

namespace {

namespace py = pybind11;
using PG = fairring::ProcessGroupFairring;
using Opts = PG::OptionsFairring;
using Millis = std::chrono::milliseconds;

c10::intrusive_ptr<Opts> makeOptions(int64_t totalBytes, int64_t paddingBytes, int64_t parallelism,
                                     bool highPriority, Millis timeout, int64_t sliceBytes) {
  return Opts::create(totalBytes, paddingBytes, parallelism, highPriority, timeout, sliceBytes);
}

c10::intrusive_ptr<PG> makeGroup(const c10::intrusive_ptr<c10d::Store>& store, int rank, int size,
                                 c10::intrusive_ptr<Opts> options) {
  return c10::make_intrusive<PG>(store, rank, size, std::move(options));
}

void bind(py::module& m) {
  // torch.distributed must be loaded first: it registers the Backend base type
  py::module::import("torch.distributed");

  py::class_<PG, c10::intrusive_ptr<PG>, c10d::Backend> group(m, "ProcessGroup");
  py::class_<Opts, c10::intrusive_ptr<Opts>, c10d::Backend::Options> options(group, "Options");

  options.def(py::init(&makeOptions), py::arg("max_memory_allocated_in_bytes"),
              py::arg("max_padding_allocated_in_bytes"), py::arg("min_parallelism"),
              py::arg("is_high_priority_stream") = false,
              py::arg("timeout") = Millis(kBackendDefaultTimeout),
              py::arg("slice_size_in_bytes") = int64_t{0});

  group.def(py::init(&makeGroup), py::arg("store"), py::arg("rank"), py::arg("size"),
            py::arg("options"), py::call_guard<py::gil_scoped_release>());

  // one-GPU additions, not in the reference
  group.def("_set_simulated_peer_contributions", &PG::setSimulatedPeerContributions,
            py::arg("peers"), py::call_guard<py::gil_scoped_release>());
  group.def("_set_fused_divide", &PG::setFusedDivide, py::arg("on"));
  group.def("_layout", &PG::layout);
  // measurement hooks of the pipeline behind the group (include/fairring_hip.h)
  group.def("_profile_mark", &PG::profileMark, py::call_guard<py::gil_scoped_release>());
  group.def("_launch_records", &PG::launchRecords, py::call_guard<py::gil_scoped_release>());
  group.def("_synchronize", &PG::synchronizeAll, py::call_guard<py::gil_scoped_release>());
  // the allreduce with one of torch's DDP communication hooks folded in
  group.def("_allreduce_pre_divided", &PG::allreducePreDivided, py::arg("bucket"),
            py::call_guard<py::gil_scoped_release>());
  group.def("_allreduce_compressed", &PG::allreduceCompressed, py::arg("bucket"),
            py::arg("wire_dtype"), py::arg("grads") = std::vector<at::Tensor>(),
            py::call_guard<py::gil_scoped_release>());
  // the allreduce of a bucket read from the gradient tensors it is assembled from
  group.def("_allreduce_from_grads", &PG::allreduceFromGrads, py::arg("bucket"), py::arg("grads"),
            py::arg("pre_divide") = false, py::call_guard<py::gil_scoped_release>());
}

}  // namespace

PYBIND11_MODULE(_fairring, m) { bind(m); }
