#include "environment.h"

#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>
#include <utility>

#include "crl.h"

namespace {

bool verbose() {
  static const bool v = std::getenv("CUDARL_VERBOSE") != nullptr;
  return v;
}

// like the reference's CUDA_CHECK (src/core/cuda_utils.h:11-19): status -> exception
void check(int rc, const char* what) {
  if (rc != CRL_OK) throw std::runtime_error(std::string(what) + ": " + crl_last_error());
}

}  // namespace

Environment::Environment(int id, int width, int height) : env_id(id), engine(nullptr) {
  if (width < 1 || height < 1) throw std::runtime_error("Environment: width and height must be >= 1");
  state.width = width;
  state.height = height;
  state.agent_x = width / 2;
  state.agent_y = height / 2;
  state.reward = 0.0f;
  state.done = false;
  grid_store.resize((size_t)width * height);
  state.grid = grid_store.data();
  initializeGrid();

  crl_config cfg{};
  cfg.struct_size = sizeof(cfg);
  cfg.n_envs = 1;
  cfg.width = width;
  cfg.height = height;
  cfg.n_actions = 4;
  cfg.table_mode = CRL_TABLE_SHARED;
  cfg.map_mode = CRL_MAP_SHARED;
  cfg.max_mode = CRL_MAX_TRUE;
  cfg.goal_mode = CRL_GOAL_ON_RESULT;  // src/environment.cu:43
  cfg.auto_reset = 0;                  // done is sticky (src/environment.cu:44-46)
  cfg.episode_len = 0;
  cfg.lr = 0.1f;
  cfg.gamma = 0.99f;
  cfg.step_reward = -0.01f;
  cfg.goal_reward = 1.0f;
  cfg.trap_reward = -1.0f;
  cfg.reward_flags = CRL_REWARD_CELLS;
  cfg.eps_mode = CRL_EPS_FIXED;
  cfg.eps0 = 0.0f;
  cfg.eps_span = 1;
  cfg.seed = (uint64_t)id;
  // (host buffers first: nothing below may throw while the engine is held by a raw pointer)
  std::vector<uint8_t> cls(grid_store.size());
  std::vector<float> rew(grid_store.size());
  crl_classify_grid(grid_store.data(), grid_store.size(), -0.01f, cls.data(), rew.data());
  check(crl_create(&cfg, 0, &engine), "Environment: crl_create");
  const int32_t start = (height / 2) * width + width / 2;  // src/environment.cu:9-10
  int rc = crl_set_maps(engine, cls.data(), &start, rew.data());
  if (rc != CRL_OK) {
    release();
    check(rc, "Environment: crl_set_maps");
  }
  if (verbose())
    std::cout << "Environment " << env_id << " constructed (" << width << "x" << height << ")." << std::endl;
}

Environment::~Environment() {
  const bool had = engine != nullptr;
  release();
  if (had && verbose()) std::cout << "Environment " << env_id << " destructed." << std::endl;
}

void Environment::release() noexcept {
  if (engine) crl_destroy(engine);
  engine = nullptr;
}

Environment::Environment(Environment&& o) noexcept
    : env_id(o.env_id), state(o.state), engine(o.engine), grid_store(std::move(o.grid_store)) {
  state.grid = grid_store.data();
  o.engine = nullptr;
  o.state.grid = nullptr;
}

Environment& Environment::operator=(Environment&& o) noexcept {
  if (this != &o) {
    release();
    env_id = o.env_id;
    state = o.state;
    engine = o.engine;
    grid_store = std::move(o.grid_store);
    state.grid = grid_store.data();
    o.engine = nullptr;
    o.state.grid = nullptr;
  }
  return *this;
}

void Environment::reset() {
  check(crl_reset(engine, 0, 1), "Environment::reset");
  updateHostState();
  if (verbose()) std::cout << "Environment " << env_id << " reset." << std::endl;
}

void Environment::step(int action) {
  const int32_t a = action;
  check(crl_step(engine, &a), "Environment::step");
  updateHostState();
  if (verbose())
    std::cout << "Environment " << env_id << " performed action " << action << ", reward: " << state.reward
              << ", position: (" << state.agent_x << "," << state.agent_y << ")"
              << ", done: " << (state.done ? "true" : "false") << std::endl;
}

float Environment::getCellValue(int x, int y) const {
  if (x >= 0 && x < state.width && y >= 0 && y < state.height) return grid_store[(size_t)y * state.width + x];
  return 0.0f;  // src/environment.cu:131
}

std::vector<float> Environment::getGrid() const { return grid_store; }

void Environment::setCellValue(int x, int y, float value, bool trap) {
  if (x < 0 || x >= state.width || y < 0 || y >= state.height)
    throw std::runtime_error("Environment::setCellValue: cell out of range");
  const size_t cell = (size_t)y * state.width + x;
  uint8_t cls;
  float rew;
  crl_classify_grid(&value, 1, -0.01f, &cls, &rew);
  if (trap) {
    cls = CRL_CELL_TRAP;
    rew = value;
  }
  check(crl_set_cell(engine, 0, (int32_t)cell, cls, rew), "Environment::setCellValue");
  grid_store[cell] = value;
}

void Environment::initializeGrid() {
  // cells uniform in [0, 0.5] (all FREE) and the goal in the top-right corner
  // (src/environment.cu:138-147).  The reference seeds rand() from the wall
  // clock; here the seed is the env id so that runs are reproducible.
  const uint32_t key[2] = {(uint32_t)env_id, 0x43524c45u};
  for (size_t i = 0; i < grid_store.size(); i += 4) {
    const uint32_t ctr[4] = {(uint32_t)(i / 4), 0u, 0u, 0u};
    uint32_t w[4];
    crl_philox4x32_10(ctr, key, w);
    for (size_t j = 0; j < 4 && i + j < grid_store.size(); ++j)
      grid_store[i + j] = (float)(w[j] >> 8) * (1.0f / 16777216.0f) * 0.5f;
  }
  grid_store[(size_t)state.width - 1] = 1.0f;
}

void Environment::updateHostState() {
  int32_t s = 0;
  float r = 0.0f;
  uint8_t d = 0;
  check(crl_get_state(engine, &s, &r, &d, nullptr, nullptr, nullptr), "Environment: crl_get_state");
  state.agent_x = s % state.width;
  state.agent_y = s / state.width;
  state.reward = r;
  state.done = d != 0;
}
