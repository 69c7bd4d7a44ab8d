// cudarl_train: command line of the reference's src/train.py (same flags and
// defaults, :361-385) on the batched engine.  Additive flags: --envs, --seed,
// --mock-env.  --plot is accepted and ignored.
#include <sys/stat.h>

#include <cstdlib>
#include <cstring>
#include <iostream>
#include <stdexcept>
#include <string>

#include "npy.h"
#include "train.h"

namespace {

void usage() {
  std::cerr << "usage: cudarl_train [--width W] [--height H] [--learning-rate A] [--discount-factor G]\n"
               "                    [--exploration-rate E] [--exploration-decay D] [--episodes N]\n"
               "                    [--max-steps T] [--eval-episodes K] [--output-dir DIR] [--save-agent]\n"
               "                    [--plot] [--envs N] [--seed S] [--mock-env]\n";
}

}  // namespace

int main(int argc, char** argv) {
  cudarl::TrainOptions o;
  try {
    for (int i = 1; i < argc; ++i) {
      const std::string a = argv[i];
      auto value = [&]() -> const char* {
        if (i + 1 >= argc) throw std::runtime_error("missing value for " + a);
        return argv[++i];
      };
      if (a == "--width") o.width = std::atoi(value());
      else if (a == "--height") o.height = std::atoi(value());
      else if (a == "--learning-rate") o.learning_rate = (float)std::atof(value());
      else if (a == "--discount-factor") o.discount_factor = (float)std::atof(value());
      else if (a == "--exploration-rate") o.exploration_rate = (float)std::atof(value());
      else if (a == "--exploration-decay") o.exploration_decay = (float)std::atof(value());
      else if (a == "--episodes") o.episodes = std::atoi(value());
      else if (a == "--max-steps") o.max_steps = std::atoi(value());
      else if (a == "--eval-episodes") o.eval_episodes = std::atoi(value());
      else if (a == "--output-dir") o.output_dir = value();
      else if (a == "--save-agent") o.save_agent = true;
      else if (a == "--plot") o.plot = true;
      else if (a == "--envs") o.n_envs = std::atoi(value());
      else if (a == "--seed") o.seed = std::strtoull(value(), nullptr, 10);
      else if (a == "--mock-env") o.mock_env = true;
      else if (a == "--help" || a == "-h") { usage(); return 0; }
      else throw std::runtime_error("unknown argument " + a);
    }
    if (o.episodes < 1 || o.max_steps < 1 || o.n_envs < 1) throw std::runtime_error("episodes, max-steps and envs must be >= 1");

    if (o.save_agent) mkdir(o.output_dir.c_str(), 0777);
    std::vector<uint8_t> cls;
    std::vector<int32_t> start;
    cudarl::default_world(o, cls, start);
    BatchedEnvironment env(cudarl::training_config(o));
    env.setMaps(cls.data(), start.data(), nullptr);
    std::cout << "Initialized Q-table agent with " << o.width << "x" << o.height << " states and 4 actions" << std::endl;
    std::cout << "Starting training for " << o.episodes << " episodes" << std::endl;
    const cudarl::TrainMetrics m = cudarl::train(env, o.episodes, o.max_steps, &std::cout);
    if (o.eval_episodes > 0) {
      std::cout << "Evaluating agent for " << o.eval_episodes << " episodes" << std::endl;
      cudarl::evaluate(env, cls, start, o.eval_episodes, &std::cout);
    }
    if (o.save_agent) {
      const std::string path = o.output_dir + "/qtable_agent.npy";  // src/train.py:424-426
      crl_npy::save_agent(path, env.qTable(0), o.width, o.height, 4);
      std::cout << "Saved Q-table to " << path << std::endl;
    }
    if (o.plot) std::cout << "Plotting is left to the reference's Python tools" << std::endl;
    std::cout << "Done! (" << m.env_steps << " env-steps in " << m.seconds << " s)" << std::endl;
  } catch (const std::exception& e) {
    std::cerr << "cudarl_train: " << e.what() << std::endl;
    usage();
    return 1;
  }
  return 0;
}
