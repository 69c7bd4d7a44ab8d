#include "q_learning.h"

#include <cstdint>
#include <cstdlib>
#include <iostream>
#include <stdexcept>
#include <string>

#include "crl.h"

CudaQLearning::CudaQLearning(int width, int height, int action_space_size, float learning_rate,
                             float discount_factor, int max_mode)
    : width(width), height(height), action_space_size(action_space_size),
      learning_rate(learning_rate), discount_factor(discount_factor), engine(nullptr),
      max_batch_size(1024) {  // src/q_learning.cu:10
  crl_config cfg{};
  cfg.struct_size = sizeof(cfg);
  cfg.n_envs = 1;
  cfg.width = width;
  cfg.height = height;
  cfg.n_actions = action_space_size;
  cfg.table_mode = CRL_TABLE_SHARED;
  cfg.map_mode = CRL_MAP_SHARED;
  cfg.max_mode = max_mode;
  cfg.goal_mode = CRL_GOAL_ON_TARGET;
  cfg.auto_reset = 0;
  cfg.lr = learning_rate;
  cfg.gamma = discount_factor;
  cfg.step_reward = -0.01f;
  cfg.goal_reward = 1.0f;
  cfg.trap_reward = -1.0f;
  cfg.eps_mode = CRL_EPS_FIXED;
  cfg.eps_span = 1;
  if (width < 1 || height < 1 || action_space_size < 1)
    throw std::runtime_error("CudaQLearning: width, height and action_space_size must be >= 1");
  h_q_table.resize((size_t)width * height * action_space_size, 0.0f);  // (before the engine: may throw)
  if (crl_create(&cfg, 0, &engine) != CRL_OK)  // src/q_learning.cu:17-19
    throw std::runtime_error(std::string("Failed to allocate device memory for Q-table: ") + crl_last_error());
  if (std::getenv("CUDARL_VERBOSE"))
    std::cout << "CudaQLearning initialized with " << width << "x" << height << " states and "
              << action_space_size << " actions" << std::endl;
}

CudaQLearning::~CudaQLearning() { crl_destroy(engine); }

void CudaQLearning::update_batch(const std::vector<std::pair<int, int>>& states,
                                 const std::vector<int>& actions, const std::vector<float>& rewards,
                                 const std::vector<std::pair<int, int>>& next_states,
                                 const std::vector<bool>& dones) {
  const size_t batch_size = states.size();
  if (batch_size > (size_t)max_batch_size)  // src/q_learning.cu:117-119
    throw std::runtime_error("Batch size exceeds maximum batch size");
  if (batch_size != actions.size() || batch_size != rewards.size() || batch_size != next_states.size() ||
      batch_size != dones.size())  // src/q_learning.cu:121-124
    throw std::runtime_error("Inconsistent batch sizes");
  if (batch_size == 0) return;
  std::vector<int32_t> s(batch_size), a(batch_size), s2(batch_size);
  std::vector<uint8_t> d(batch_size);
  for (size_t i = 0; i < batch_size; ++i) {
    const int x = states[i].first, y = states[i].second;
    const int nx = next_states[i].first, ny = next_states[i].second;
    // the reference indexes unchecked (src/kernels.cu:96); an out-of-range
    // state would be an out-of-bounds device access, so it is refused here
    if (x < 0 || x >= width || y < 0 || y >= height || nx < 0 || nx >= width || ny < 0 || ny >= height)
      throw std::runtime_error("Invalid state");
    if (actions[i] < 0 || actions[i] >= action_space_size) throw std::runtime_error("Invalid state or action");
    s[i] = y * width + x;  // src/kernels.cu:96
    s2[i] = ny * width + nx;
    a[i] = actions[i];
    d[i] = dones[i] ? 1 : 0;
  }
  if (crl_td_update(engine, 0, (int32_t)batch_size, s.data(), a.data(), rewards.data(), s2.data(), d.data()) != CRL_OK)
    throw std::runtime_error(std::string("update_batch: ") + crl_last_error());
  // src/q_learning.cu:173: the host mirror follows every update
  if (crl_q_get(engine, 0, h_q_table.data()) != CRL_OK)
    throw std::runtime_error(std::string("update_batch: ") + crl_last_error());
}

std::vector<float> CudaQLearning::get_q_table() const { return h_q_table; }

void CudaQLearning::set_q_table(const std::vector<float>& q_table) {
  if (q_table.size() != (size_t)width * height * action_space_size)  // src/q_learning.cu:181-183
    throw std::runtime_error("Invalid Q-table size");
  if (crl_q_set(engine, 0, q_table.data()) != CRL_OK)
    throw std::runtime_error(std::string("set_q_table: ") + crl_last_error());
  h_q_table = q_table;
}

int CudaQLearning::get_best_action(int x, int y) const {
  if (x < 0 || x >= width || y < 0 || y >= height) throw std::runtime_error("Invalid state");
  const size_t base = ((size_t)y * width + x) * action_space_size;
  int best_action = 0;
  float best_value = h_q_table[base];
  for (int a = 1; a < action_space_size; a++) {  // strict >: lowest index wins ties
    if (h_q_table[base + a] > best_value) {
      best_value = h_q_table[base + a];
      best_action = a;
    }
  }
  return best_action;
}

float CudaQLearning::get_q_value(int x, int y, int action) const {
  if (x < 0 || x >= width || y < 0 || y >= height || action < 0 || action >= action_space_size)
    throw std::runtime_error("Invalid state or action");
  return h_q_table[((size_t)y * width + x) * action_space_size + action];
}
