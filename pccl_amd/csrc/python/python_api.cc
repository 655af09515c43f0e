// python_api.cc -- the Python extension module of the engine, pccl_amd.engine_c.
//
// Same layout as the reference's pccl.engine_c (csrc/python_api.cc:10-28, built by
// setup.py:105-112 as a torch C++ extension): class Engine(rank, world_size) with initEngine,
// regOp, exeOp, exportEndpoint, joinCluster, exitCluster, and submodule utils with
// LaunchEnvironments.listOpt / getEnv / registerOpt.  exeOp takes torch tensors, as
// include/engine.h:19 declares it (const std::string &, at::Tensor &, at::Tensor), and runs on
// torch's current stream of the input's device.  waitOp is this build's addition (the reference
// has no way to learn that an op finished).
#include <torch/extension.h>

#include <string>

#include "engine_torch.h"
#include "launch_env.h"

namespace py = pybind11;
using namespace engine_c;

namespace {

void wait_op(TorchEngine &engine, const std::string &name) {
  engine.waitOp(name, (void *)c10::hip::getCurrentHIPStream().stream());
}

}  // namespace

PYBIND11_MODULE(engine_c, m) {
  m.doc() = "PCCL engine on MI355X: registered collectives run by the HIP reduce-copy executor";

  py::class_<TorchEngine>(m, "Engine")
      .def(py::init<int, int>(), py::arg("rank"), py::arg("world_size"))
      .def("initEngine", &TorchEngine::initEngine)
      .def("regOp", static_cast<void (Engine::*)(const std::string &, const std::string &)>(&Engine::regOp),
           py::arg("name"), py::arg("filepath"))
      .def("exeOp", static_cast<void (TorchEngine::*)(const std::string &, at::Tensor &, at::Tensor)>(&TorchEngine::exeOp),
           py::arg("name"), py::arg("input"), py::arg("output"))
      .def("waitOp", &wait_op, py::arg("name"))
      .def("exportEndpoint", &TorchEngine::exportEndpoint)
      .def("joinCluster", &TorchEngine::joinCluster)
      .def("exitCluster", &TorchEngine::exitCluster);

  auto utils_submodule = m.def_submodule("utils");
  py::class_<utils::LaunchEnvironments>(utils_submodule, "LaunchEnvironments")
      .def_static("listOpt", &utils::LaunchEnvironments::listOpt)
      .def_static("getEnv", &utils::LaunchEnvironments::getEnv)
      .def_static("registerOpt", &utils::LaunchEnvironments::registerOpt);
}
