// BatchedEnvironment / the batched face of the engine for C++ and Python callers:
// N grid-worlds, their Q-tables and the fused select -> step -> update loop behind
// one object.  No counterpart upstream (the reference steps one Environment per
// call, src/environment.cu:113-125); the method names follow EnvironmentBridge
// (src/environment_bridge.h) and QTableAgent (src/train.py:36-168).
#pragma once
#include <cstdint>
#include <string>
#include <vector>

#include "crl.h"

class BatchedEnvironment {
 public:
  explicit BatchedEnvironment(const crl_config& cfg, int device = 0);
  ~BatchedEnvironment();
  BatchedEnvironment(const BatchedEnvironment&) = delete;
  BatchedEnvironment& operator=(const BatchedEnvironment&) = delete;

  const crl_config& config() const { return cfg; }
  int numEnvs() const { return cfg.n_envs; }
  int numStates() const { return cfg.width * cfg.height; }
  int numActions() const { return cfg.n_actions; }
  int numTables() const { return cfg.table_mode == CRL_TABLE_SHARED ? 1 : cfg.n_envs; }
  int numMaps() const { return cfg.map_mode == CRL_MAP_SHARED ? 1 : cfg.n_envs; }

  // cell_class: numMaps()*S bytes; start: N cells; cell_reward: numMaps()*S floats or empty
  void setMaps(const uint8_t* cell_class, const int32_t* start, const float* cell_reward);
  void reset();
  void step(const int32_t* actions);          // nullptr: the actions of the last select()
  void select(int32_t* actions_out);          // may be nullptr
  void update();
  void run(int n_steps);                      // fused select -> step -> update
  void sync();

  struct State {
    std::vector<int32_t> s, ep_step, episode;
    std::vector<float> reward;
    std::vector<uint8_t> done, action;
  };
  State state() const;
  // needs config().track_returns
  struct EpisodeStats {
    std::vector<float> last_return, return_sum;
    std::vector<int32_t> last_length, length_sum;
  };
  EpisodeStats episodeStats() const;
  std::vector<float> qTable(int table = 0) const;
  void setQTable(int table, const std::vector<float>& q);
  uint64_t stepCount() const;

  // raw device pointer of one SoA array (CRL_PTR_*), for zero-copy consumers
  void* devicePointer(int which) const;
  int device() const { return dev; }

 private:
  crl_config cfg;
  int dev;
  crl_engine* engine;
};
