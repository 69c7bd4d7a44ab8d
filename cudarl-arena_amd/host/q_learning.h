// CudaQLearning: the reference's tabular Q-learning host class
// (src/q_learning.cuh:8-95), same public signatures, on the HIP engine.
#pragma once
#include <utility>
#include <vector>

struct crl_engine;

class CudaQLearning {
 public:
  // max_mode (additive): 1 = max over the next row seeded with 0, which is what the
  // kernel behind this class upstream computes (update_q_values_kernel,
  // src/kernels.cu:101-110) and therefore the default of the five-argument
  // constructor; 0 = the true max (src/gpu/kernels.cu:35-45, np.max in src/train.py:134),
  // the default of the batched engine and of train().
  CudaQLearning(int width, int height, int action_space_size, float learning_rate = 0.1f,
                float discount_factor = 0.99f, int max_mode = 1);
  ~CudaQLearning();
  CudaQLearning(const CudaQLearning&) = delete;
  CudaQLearning& operator=(const CudaQLearning&) = delete;

  void update_batch(const std::vector<std::pair<int, int>>& states, const std::vector<int>& actions,
                    const std::vector<float>& rewards,
                    const std::vector<std::pair<int, int>>& next_states,
                    const std::vector<bool>& dones);
  std::vector<float> get_q_table() const;
  void set_q_table(const std::vector<float>& q_table);
  int get_best_action(int x, int y) const;
  float get_q_value(int x, int y, int action) const;

 private:
  int width;
  int height;
  int action_space_size;
  float learning_rate;
  float discount_factor;
  std::vector<float> h_q_table;  // host mirror, refreshed after every update
  crl_engine* engine;
  int max_batch_size;
};
