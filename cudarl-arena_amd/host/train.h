// train() / evaluate(): the reference's training driver (src/train.py:171-311)
// on the batched engine.  One call runs `num_episodes` episodes of at most
// `max_steps` steps for EVERY env of the batch (the reference has one env); the
// episode loop, the break on done and the reward / length bookkeeping of
// src/train.py:191-226 run on the device (episode budget + accumulators).
#pragma once
#include <cstdint>
#include <iosfwd>
#include <string>
#include <vector>

#include "batched_environment.h"

namespace cudarl {

struct TrainOptions {  // the argparse flags of src/train.py:361-385, same defaults
  int width = 10, height = 10;
  float learning_rate = 0.1f, discount_factor = 0.99f;
  float exploration_rate = 1.0f, exploration_decay = 0.995f;
  int episodes = 1000, max_steps = 500, eval_episodes = 10;
  std::string output_dir = "results";
  bool save_agent = false;
  bool plot = false;  // accepted for compatibility; plotting stays with the reference's Python
  // additive
  int n_envs = 1;
  uint64_t seed = 0;
  bool mock_env = false;  // the agent cannot move and nothing ends an episode (python/cudarl/mock_env.py)
};

struct TrainMetrics {
  std::vector<float> return_sum;    // per env, over its finished episodes
  std::vector<int32_t> length_sum;  // per env
  std::vector<float> last_return;   // per env
  double avg_reward = 0, avg_length = 0;  // over all episodes of all envs
  uint64_t env_steps = 0;
  double seconds = 0;
};

struct EvalMetrics {
  double avg_reward = 0, avg_length = 0;
  std::vector<float> rewards;    // one greedy episode per env (greedy episodes of one env are all alike)
  std::vector<int32_t> lengths;
};

// Engine configuration of a training run with these options (per-step epsilon
// decay as in src/train.py:140-141, episode budget, return tracking).
crl_config training_config(const TrainOptions& o);

// The reference's default world (src/environment.cu:9-10,138-147): every cell
// free, goal in the top-right corner, start in the centre; or the mock world.
void default_world(const TrainOptions& o, std::vector<uint8_t>& cell_class, std::vector<int32_t>& start);

// src/train.py:171-259.  `log` (may be null) receives the reference's progress lines.
TrainMetrics train(BatchedEnvironment& env, int num_episodes, int max_steps, std::ostream* log);

// src/train.py:262-311: greedy episodes (at most 1000 steps) with the trained
// tables, nothing is updated.  Uses a second engine with the same maps.
EvalMetrics evaluate(const BatchedEnvironment& trained, const std::vector<uint8_t>& cell_class,
                     const std::vector<int32_t>& start, int num_episodes, std::ostream* log);

}  // namespace cudarl
