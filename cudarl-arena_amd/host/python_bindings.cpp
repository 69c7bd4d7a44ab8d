// pybind11 module `cudarl_core` (src/python_bindings.cpp:8-26): class
// Environment = EnvironmentBridge with the reference's snake_case methods.
// CudaQLearning is not bound upstream; binding it is additive.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>
#include <memory>
#include <stdexcept>

#include "batched_environment.h"
#include "environment.h"
#include "environment_bridge.h"
#include "npy.h"
#include "q_learning.h"

namespace py = pybind11;

namespace {

// DLPack (v0.8 layout) view of one device array, so that any DLPack consumer
// can wrap the engine's memory without a copy.  device_type 10 = ROCm.
struct DLDevice { int32_t device_type; int32_t device_id; };
struct DLDataType { uint8_t code; uint8_t bits; uint16_t lanes; };
struct DLTensor {
  void* data; DLDevice device; int32_t ndim; DLDataType dtype; int64_t* shape; int64_t* strides; uint64_t byte_offset;
};
struct DLManagedTensor { DLTensor dl_tensor; void* manager_ctx; void (*deleter)(DLManagedTensor*); };
constexpr int32_t kDLROCM = 10;

struct ViewCtx {
  int64_t shape[3];
  PyObject* owner;  // keeps the BatchedEnvironment alive while the view exists
};

void view_deleter(DLManagedTensor* t) {
  ViewCtx* ctx = static_cast<ViewCtx*>(t->manager_ctx);
  {
    py::gil_scoped_acquire gil;
    Py_DECREF(ctx->owner);
  }
  delete ctx;
  delete t;
}

void capsule_destructor(PyObject* cap) {
  // a consumer renames the capsule to "used_dltensor" and then owns the tensor
  if (PyCapsule_IsValid(cap, "dltensor")) {
    auto* t = static_cast<DLManagedTensor*>(PyCapsule_GetPointer(cap, "dltensor"));
    if (t && t->deleter) t->deleter(t);
  }
}

struct ArraySpec { int which; uint8_t code; uint8_t bits; int ndim; };

ArraySpec spec_of(const std::string& name) {
  if (name == "s") return {CRL_PTR_S, 0, 32, 1};
  if (name == "ep_step") return {CRL_PTR_EP_STEP, 0, 32, 1};
  if (name == "episode") return {CRL_PTR_EPISODE, 0, 32, 1};
  if (name == "reward") return {CRL_PTR_REWARD, 2, 32, 1};
  if (name == "done") return {CRL_PTR_DONE, 1, 8, 1};
  if (name == "action") return {CRL_PTR_ACTION, 1, 8, 1};
  if (name == "q") return {CRL_PTR_Q, 2, 32, 3};
  throw std::runtime_error("unknown device array '" + name + "'");
}

crl_config make_config(int n_envs, int width, int height, int n_actions, bool shared_table, bool shared_map,
                       float lr, float gamma, float epsilon, int episode_len, uint64_t seed, int max_mode,
                       int goal_mode, bool auto_reset, float step_reward, float goal_reward,
                       float trap_reward, int reward_flags, int eps_mode, float eps_decay, float eps_end,
                       int eps_span) {
  crl_config c{};
  c.struct_size = sizeof c;
  c.n_envs = n_envs;
  c.width = width;
  c.height = height;
  c.n_actions = n_actions;
  c.table_mode = shared_table ? CRL_TABLE_SHARED : CRL_TABLE_PER_ENV;
  c.map_mode = shared_map ? CRL_MAP_SHARED : CRL_MAP_PER_ENV;
  c.max_mode = max_mode;
  c.goal_mode = goal_mode;
  c.auto_reset = auto_reset ? 1 : 0;
  c.episode_len = episode_len;
  c.lr = lr;
  c.gamma = gamma;
  c.step_reward = step_reward;
  c.goal_reward = goal_reward;
  c.trap_reward = trap_reward;
  c.reward_flags = reward_flags;
  c.eps_mode = eps_mode;
  c.eps0 = epsilon;
  c.eps_decay = eps_decay;
  c.eps_end = eps_end;
  c.eps_span = eps_span;
  c.seed = seed;
  return c;
}

template <class T>
py::array_t<T> to_array(const std::vector<T>& v) {
  py::array_t<T> a((py::ssize_t)v.size());
  std::memcpy(a.mutable_data(), v.data(), v.size() * sizeof(T));
  return a;
}

// The reference's other Python surface (src/bindings/python_bindings.cpp:9-63,
// class PyEnvironment bound as `Environment` there): observations as an (H, W)
// numpy array, a dict for info, width / height / env_id as read-only properties.
// Bound here under its C++ name beside the current `Environment`.
class PyEnvironment {
 public:
  PyEnvironment(int width, int height, int env_id = 0)
      : width_(width), height_(height), env_id_(env_id), env_(env_id, width, height) {}

  py::array_t<float> reset() {
    env_.reset();
    return observation();
  }
  std::tuple<py::array_t<float>, float, bool, py::dict> step(int action) {
    env_.step(action);
    py::dict info;
    info["agent_x"] = env_.getAgentX();
    info["agent_y"] = env_.getAgentY();
    return std::make_tuple(observation(), env_.getReward(), env_.isDone(), info);
  }
  py::array_t<float> observation() const {
    const std::vector<float> grid = env_.getGrid();  // row-major [y][x]: already the (H, W) layout
    py::array_t<float> obs({(py::ssize_t)height_, (py::ssize_t)width_});
    std::memcpy(obs.mutable_data(), grid.data(), grid.size() * sizeof(float));
    return obs;
  }
  int width() const { return width_; }
  int height() const { return height_; }
  int env_id() const { return env_id_; }

 private:
  int width_, height_, env_id_;
  Environment env_;
};

}  // namespace

PYBIND11_MODULE(cudarl_core, m) {
  m.doc() = "CudaRL-Arena Python bindings (MI355X engine)";

  py::class_<PyEnvironment>(m, "PyEnvironment")
      .def(py::init<int, int, int>(), py::arg("width") = 10, py::arg("height") = 10, py::arg("env_id") = 0)
      .def("reset", &PyEnvironment::reset)
      .def("step", &PyEnvironment::step)
      .def("get_observation", &PyEnvironment::observation)
      .def_property_readonly("width", &PyEnvironment::width)
      .def_property_readonly("height", &PyEnvironment::height)
      .def_property_readonly("env_id", &PyEnvironment::env_id);

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
           py::arg("discount_factor") = 0.99f, py::arg("max_mode") = 1)
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

  // the batched surface (additive): N envs, their tables, the fused loop
  py::class_<BatchedEnvironment>(m, "BatchedEnvironment")
      .def(py::init([](int n_envs, int width, int height, int n_actions, bool shared_table, bool shared_map,
                       float learning_rate, float discount_factor, float exploration_rate, int episode_len,
                       uint64_t seed, int max_mode, int goal_mode, bool auto_reset, float step_reward,
                       float goal_reward, float trap_reward, int reward_flags, int eps_mode,
                       float exploration_decay, float exploration_end, int eps_span, int device) {
             return std::make_unique<BatchedEnvironment>(
                 make_config(n_envs, width, height, n_actions, shared_table, shared_map, learning_rate,
                             discount_factor, exploration_rate, episode_len, seed, max_mode, goal_mode,
                             auto_reset, step_reward, goal_reward, trap_reward, reward_flags, eps_mode,
                             exploration_decay, exploration_end, eps_span),
                 device);
           }),
           py::arg("n_envs"), py::arg("width") = 10, py::arg("height") = 10, py::arg("n_actions") = 4,
           py::arg("shared_table") = false, py::arg("shared_map") = false, py::arg("learning_rate") = 0.1f,
           py::arg("discount_factor") = 0.99f, py::arg("exploration_rate") = 0.1f, py::arg("episode_len") = 0,
           py::arg("seed") = 0, py::arg("max_mode") = 0, py::arg("goal_mode") = 0, py::arg("auto_reset") = true,
           py::arg("step_reward") = -0.01f, py::arg("goal_reward") = 1.0f, py::arg("trap_reward") = -1.0f,
           py::arg("reward_flags") = 0, py::arg("eps_mode") = 0, py::arg("exploration_decay") = 1.0f,
           py::arg("exploration_end") = 0.0f, py::arg("eps_span") = 1, py::arg("device") = 0)
      .def_property_readonly("num_envs", &BatchedEnvironment::numEnvs)
      .def_property_readonly("num_states", &BatchedEnvironment::numStates)
      .def_property_readonly("num_actions", &BatchedEnvironment::numActions)
      .def_property_readonly("num_tables", &BatchedEnvironment::numTables)
      .def_property_readonly("step_count", &BatchedEnvironment::stepCount)
      .def("set_maps",
           [](BatchedEnvironment& self, py::array_t<uint8_t, py::array::c_style | py::array::forcecast> cls,
              py::array_t<int32_t, py::array::c_style | py::array::forcecast> start, py::object cell_reward) {
             const size_t cells = (size_t)self.numMaps() * self.numStates();
             if ((size_t)cls.size() != cells) throw std::runtime_error("cell_class has the wrong size");
             if ((size_t)start.size() != (size_t)self.numEnvs()) throw std::runtime_error("start has the wrong size");
             if (cell_reward.is_none()) {
               self.setMaps(cls.data(), start.data(), nullptr);
             } else {
               auto cr = py::array_t<float, py::array::c_style | py::array::forcecast>::ensure(cell_reward);
               if (!cr || (size_t)cr.size() != cells) throw std::runtime_error("cell_reward has the wrong size");
               self.setMaps(cls.data(), start.data(), cr.data());
             }
           },
           py::arg("cell_class"), py::arg("start"), py::arg("cell_reward") = py::none())
      .def("reset", &BatchedEnvironment::reset)
      .def("step",
           [](BatchedEnvironment& self, py::object actions) {
             if (actions.is_none()) {
               self.step(nullptr);
             } else {
               auto a = py::array_t<int32_t, py::array::c_style | py::array::forcecast>::ensure(actions);
               if (!a || (size_t)a.size() != (size_t)self.numEnvs()) throw std::runtime_error("actions has the wrong size");
               self.step(a.data());
             }
           },
           py::arg("actions") = py::none())
      .def("select",
           [](BatchedEnvironment& self) {
             py::array_t<int32_t> out(self.numEnvs());
             self.select(out.mutable_data());
             return out;
           })
      .def("update", &BatchedEnvironment::update)
      .def("run", &BatchedEnvironment::run, py::arg("n_steps"), py::call_guard<py::gil_scoped_release>())
      // the same under the name a caller of select / step / update looks for: n fused rounds
      // in one call instead of 3 n launches (1M envs of 16x16: 1.4e10 env-steps/s one round
      // per call, 3.1e10 at 20, 8.8e10 at 1000)
      .def("step_n", &BatchedEnvironment::run, py::arg("n_steps"), py::call_guard<py::gil_scoped_release>())
      .def("sync", &BatchedEnvironment::sync)
      .def("state",
           [](const BatchedEnvironment& self) {
             const BatchedEnvironment::State st = self.state();
             py::dict d;
             d["s"] = to_array(st.s);
             d["ep_step"] = to_array(st.ep_step);
             d["episode"] = to_array(st.episode);
             d["reward"] = to_array(st.reward);
             d["done"] = to_array(st.done);
             d["action"] = to_array(st.action);
             return d;
           })
      .def("q_table",
           [](const BatchedEnvironment& self, int table) {
             const std::vector<float> q = self.qTable(table);
             py::array_t<float> a({(py::ssize_t)self.numStates(), (py::ssize_t)self.numActions()});
             std::memcpy(a.mutable_data(), q.data(), q.size() * sizeof(float));
             return a;
           },
           py::arg("table") = 0)
      .def("set_q_table",
           [](BatchedEnvironment& self, int table, py::array_t<float, py::array::c_style | py::array::forcecast> q) {
             self.setQTable(table, std::vector<float>(q.data(), q.data() + q.size()));
           })
      .def("device_pointer",
           [](const BatchedEnvironment& self, const std::string& name) {
             return reinterpret_cast<uintptr_t>(self.devicePointer(spec_of(name).which));
           })
      // zero-copy DLPack view ("dltensor" capsule, ROCm device) of s / ep_step / episode /
      // reward / done / action ([N]) or q ([tables, S, A]); the view keeps the engine alive
      .def("dlpack", [](py::object self_obj, const std::string& name) {
        const BatchedEnvironment& self = self_obj.cast<const BatchedEnvironment&>();
        const ArraySpec sp = spec_of(name);
        auto* ctx = new ViewCtx{};
        ctx->shape[0] = sp.ndim == 3 ? self.numTables() : self.numEnvs();
        ctx->shape[1] = self.numStates();
        ctx->shape[2] = self.numActions();
        ctx->owner = self_obj.ptr();
        Py_INCREF(ctx->owner);
        auto* t = new DLManagedTensor{};
        t->dl_tensor.data = self.devicePointer(sp.which);
        t->dl_tensor.device = DLDevice{kDLROCM, self.device()};
        t->dl_tensor.ndim = sp.ndim;
        t->dl_tensor.dtype = DLDataType{sp.code, sp.bits, 1};
        t->dl_tensor.shape = ctx->shape;
        t->dl_tensor.strides = nullptr;
        t->dl_tensor.byte_offset = 0;
        t->manager_ctx = ctx;
        t->deleter = view_deleter;
        return py::reinterpret_steal<py::object>(PyCapsule_New(t, "dltensor", capsule_destructor));
      });

  // QTableAgent.save / load (src/train.py:150-168): float64 (W, H, A) .npy files indexed
  // [x, y, a]; the table handed in / out is the engine's fp32 [(y*W + x)*A + a]
  m.def("save_agent_npy",
        [](const std::string& path, py::array_t<float, py::array::c_style | py::array::forcecast> q, int width,
           int height, int actions) {
          crl_npy::save_agent(path, std::vector<float>(q.data(), q.data() + q.size()), width, height, actions);
        },
        py::arg("path"), py::arg("q"), py::arg("width"), py::arg("height"), py::arg("actions") = 4);
  m.def("load_agent_npy",
        [](const std::string& path, int width, int height, int actions) {
          const std::vector<float> q = crl_npy::load_agent(path, width, height, actions);
          py::array_t<float> a({(py::ssize_t)(width * height), (py::ssize_t)actions});
          std::memcpy(a.mutable_data(), q.data(), q.size() * sizeof(float));
          return a;
        },
        py::arg("path"), py::arg("width"), py::arg("height"), py::arg("actions") = 4);
  m.def("save_table_npy",
        [](const std::string& path, py::array_t<float, py::array::c_style | py::array::forcecast> q) {
          std::vector<int64_t> shape(q.shape(), q.shape() + q.ndim());
          crl_npy::save_f32(path, shape, q.data());
        });

  m.attr("__version__") = "0.1.0";
}
