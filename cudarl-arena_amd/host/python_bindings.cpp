// pybind11 module `cudarl_core` (src/python_bindings.cpp:8-26): class
// Environment = EnvironmentBridge with the reference's snake_case methods.
// CudaQLearning is not bound upstream; binding it is additive.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include "environment_bridge.h"
#include "q_learning.h"

namespace py = pybind11;

PYBIND11_MODULE(cudarl_core, m) {
  m.doc() = "CudaRL-Arena Python bindings (MI355X engine)";

  py::class_<EnvironmentBridge>(m, "Environment")
      .def(py::init<int, int>(), py::arg("width") = 10, py::arg("height") = 10)
      .def("reset", &EnvironmentBridge::reset)
      .def("step", &EnvironmentBridge::step)
      .def("get_observation", &EnvironmentBridge::getObservation)
      .def("get_width", &EnvironmentBridge::getWidth)
      .def("get_height", &EnvironmentBridge::getHeight)
      .def("get_agent_position", &EnvironmentBridge::getAgentPosition)
      .def("add_obstacle", &EnvironmentBridge::addObstacle)
      .def("set_goal", &EnvironmentBridge::setGoal)
      .def("add_trap", &EnvironmentBridge::addTrap, py::arg("x"), py::arg("y"), py::arg("penalty") = -1.0f);

  py::class_<CudaQLearning>(m, "CudaQLearning")
      .def(py::init<int, int, int, float, float, int>(), py::arg("width"), py::arg("height"),
           py::arg("action_space_size"), py::arg("learning_rate") = 0.1f,
           py::arg("discount_factor") = 0.99f, py::arg("max_mode") = 0)
      .def("update_batch", &CudaQLearning::update_batch)
      .def("get_q_table", &CudaQLearning::get_q_table)
      .def("set_q_table", &CudaQLearning::set_q_table)
      .def("get_best_action", &CudaQLearning::get_best_action)
      .def("get_q_value", &CudaQLearning::get_q_value);

  // the raw Environment, for tests that mirror tests/test_environment.cpp
  py::class_<Environment>(m, "RawEnvironment")
      .def(py::init<int, int, int>(), py::arg("id") = 0, py::arg("width") = 10, py::arg("height") = 10)
      .def("reset", &Environment::reset)
      .def("step", &Environment::step)
      .def("getWidth", &Environment::getWidth)
      .def("getHeight", &Environment::getHeight)
      .def("getAgentX", &Environment::getAgentX)
      .def("getAgentY", &Environment::getAgentY)
      .def("getReward", &Environment::getReward)
      .def("isDone", &Environment::isDone)
      .def("getCellValue", &Environment::getCellValue)
      .def("getGrid", &Environment::getGrid)
      .def("setCellValue", &Environment::setCellValue, py::arg("x"), py::arg("y"), py::arg("value"),
           py::arg("trap") = false);

  m.attr("__version__") = "0.1.0";
}
