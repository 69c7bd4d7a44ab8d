#include "train.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <ostream>
#include <stdexcept>
#include <string>

namespace cudarl {

crl_config training_config(const TrainOptions& o) {
  crl_config c{};
  c.struct_size = sizeof c;
  c.n_envs = o.n_envs;
  c.width = o.width;
  c.height = o.height;
  c.n_actions = 4;
  c.table_mode = CRL_TABLE_PER_ENV;
  c.map_mode = CRL_MAP_SHARED;
  c.max_mode = CRL_MAX_TRUE;            // np.max, src/train.py:134
  c.goal_mode = CRL_GOAL_ON_TARGET;
  c.auto_reset = 1;                     // env.reset() at the top of every episode, src/train.py:193
  c.episode_len = o.max_steps;          // for step in range(max_steps), src/train.py:198
  c.lr = o.learning_rate;
  c.gamma = o.discount_factor;
  c.step_reward = -0.01f;
  c.goal_reward = 1.0f;
  c.trap_reward = -1.0f;
  c.eps_mode = CRL_EPS_STEP_MULT;       // decayed after every update, src/train.py:140-141
  c.eps0 = o.exploration_rate;
  c.eps_decay = o.exploration_decay;
  const int64_t span = (int64_t)o.episodes * o.max_steps + 1;
  c.eps_span = (int32_t)std::min<int64_t>(span, (int64_t)1 << 26);
  c.max_episodes = o.episodes;          // for episode in range(num_episodes), src/train.py:191
  c.track_returns = 1;
  c.seed = o.seed;
  return c;
}

void default_world(const TrainOptions& o, std::vector<uint8_t>& cls, std::vector<int32_t>& start) {
  const size_t S = (size_t)o.width * o.height;
  if (o.mock_env) {
    cls.assign(S, (uint8_t)CRL_CELL_WALL);
    cls[0] = CRL_CELL_FREE;
    start.assign((size_t)o.n_envs, 0);
    return;
  }
  cls.assign(S, (uint8_t)CRL_CELL_FREE);
  cls[(size_t)o.width - 1] = CRL_CELL_GOAL;
  start.assign((size_t)o.n_envs, (o.height / 2) * o.width + o.width / 2);
}

namespace {

double seconds_since(std::chrono::steady_clock::time_point t0) {
  return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
}

void summarise(const BatchedEnvironment::EpisodeStats& st, const std::vector<int32_t>& episodes,
               double& avg_reward, double& avg_length) {
  double r = 0, l = 0, n = 0;
  for (size_t i = 0; i < episodes.size(); ++i) {
    r += st.return_sum[i];
    l += st.length_sum[i];
    n += episodes[i];
  }
  avg_reward = n > 0 ? r / n : 0;
  avg_length = n > 0 ? l / n : 0;
}

}  // namespace

TrainMetrics train(BatchedEnvironment& env, int num_episodes, int max_steps, std::ostream* log) {
  if (!env.config().track_returns || env.config().max_episodes != num_episodes)
    throw std::runtime_error("train: the engine must be created from training_config()");
  const auto t0 = std::chrono::steady_clock::now();
  std::vector<float> eps_tab;
  {
    int32_t len = 0;
    if (crl_eps_table(&env.config(), nullptr, 0, &len) != CRL_OK || len < 1)
      throw std::runtime_error(std::string("train: epsilon table: ") + crl_last_error());
    eps_tab.resize((size_t)len);
    if (crl_eps_table(&env.config(), eps_tab.data(), len, &len) != CRL_OK)
      throw std::runtime_error(std::string("train: epsilon table: ") + crl_last_error());
  }
  const int log_every = std::max(1, num_episodes / 20);  // src/train.py:236
  int next_log = log_every;
  TrainMetrics m;
  // an episode is at most max_steps long, so num_episodes chunks always suffice;
  // envs that finish early stop by themselves (episode budget)
  for (int chunk = 0; chunk < num_episodes; ++chunk) {
    env.run(max_steps);
    const BatchedEnvironment::State st = env.state();
    const int done_min = *std::min_element(st.episode.begin(), st.episode.end());
    if (log && st.episode[0] >= next_log) {
      const BatchedEnvironment::EpisodeStats es = env.episodeStats();
      double ar, al;
      summarise(es, st.episode, ar, al);
      const uint64_t t = env.stepCount();
      const float eps = eps_tab[(size_t)std::min<uint64_t>(t, eps_tab.size() - 1)];
      char line[256];
      std::snprintf(line, sizeof line,
                    "Episode %d/%d | Reward: %.2f | Avg Reward: %.2f | Avg Length: %.1f | Epsilon: %.3f | Time: %.1fs",
                    st.episode[0], num_episodes, es.last_return[0], ar, al, eps, seconds_since(t0));
      *log << line << std::endl;
      while (next_log <= st.episode[0]) next_log += log_every;
    }
    if (done_min >= num_episodes) break;
  }
  const BatchedEnvironment::State st = env.state();
  const BatchedEnvironment::EpisodeStats es = env.episodeStats();
  m.return_sum = es.return_sum;
  m.length_sum = es.length_sum;
  m.last_return = es.last_return;
  summarise(es, st.episode, m.avg_reward, m.avg_length);
  for (int32_t l : es.length_sum) m.env_steps += (uint64_t)l;
  m.seconds = seconds_since(t0);
  if (log) {
    char line[128];
    std::snprintf(line, sizeof line, "Training completed in %.1f seconds", m.seconds);
    *log << line << std::endl;
  }
  return m;
}

EvalMetrics evaluate(const BatchedEnvironment& trained, const std::vector<uint8_t>& cell_class,
                     const std::vector<int32_t>& start, int num_episodes, std::ostream* log) {
  crl_config c = trained.config();
  c.lr = 0.0f;                 // no learning: Q + 0*(target - Q) = Q
  c.eps_mode = CRL_EPS_FIXED;  // training=False: no exploration (src/train.py:105)
  c.eps0 = 0.0f;
  c.eps_span = 1;
  c.episode_len = 1000;        // "for step in range(1000)", src/train.py:281
  c.max_episodes = 1;          // without exploration every episode of an env is the same one
  c.track_returns = 1;
  BatchedEnvironment ev(c, trained.device());
  ev.setMaps(cell_class.data(), start.data(), nullptr);
  for (int t = 0; t < trained.numTables(); ++t) ev.setQTable(t, trained.qTable(t));
  ev.run(1000);
  const BatchedEnvironment::EpisodeStats es = ev.episodeStats();
  EvalMetrics m;
  m.rewards = es.last_return;
  m.lengths = es.last_length;
  double r = 0, l = 0;
  for (size_t i = 0; i < m.rewards.size(); ++i) {
    r += m.rewards[i];
    l += m.lengths[i];
  }
  m.avg_reward = r / (double)m.rewards.size();
  m.avg_length = l / (double)m.lengths.size();
  if (log) {
    char line[160];
    for (int e = 0; e < num_episodes; ++e) {
      std::snprintf(line, sizeof line, "Evaluation episode %d: Reward = %.2f, Length = %d", e + 1,
                    m.rewards[0], m.lengths[0]);
      *log << line << std::endl;
    }
    std::snprintf(line, sizeof line, "Evaluation results: Avg Reward = %.2f, Avg Length = %.1f", m.avg_reward,
                  m.avg_length);
    *log << line << std::endl;
  }
  return m;
}

}  // namespace cudarl
