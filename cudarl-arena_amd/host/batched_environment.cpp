#include "batched_environment.h"

#include <stdexcept>

namespace {
void check(int rc, const char* what) {
  if (rc != CRL_OK) throw std::runtime_error(std::string(what) + ": " + crl_last_error());
}
}  // namespace

BatchedEnvironment::BatchedEnvironment(const crl_config& c, int device) : cfg(c), dev(device), engine(nullptr) {
  cfg.struct_size = sizeof(crl_config);
  check(crl_create(&cfg, device, &engine), "BatchedEnvironment");
}

BatchedEnvironment::~BatchedEnvironment() { crl_destroy(engine); }

void BatchedEnvironment::setMaps(const uint8_t* cell_class, const int32_t* start, const float* cell_reward) {
  check(crl_set_maps(engine, cell_class, start, cell_reward), "setMaps");
}
void BatchedEnvironment::reset() { check(crl_reset(engine, 0, cfg.n_envs), "reset"); }
void BatchedEnvironment::step(const int32_t* actions) { check(crl_step(engine, actions), "step"); }
void BatchedEnvironment::select(int32_t* actions_out) { check(crl_select(engine, actions_out), "select"); }
void BatchedEnvironment::update() { check(crl_update(engine), "update"); }
void BatchedEnvironment::run(int n_steps) { check(crl_run_fused(engine, n_steps), "run"); }
void BatchedEnvironment::sync() { check(crl_sync(engine), "sync"); }

BatchedEnvironment::State BatchedEnvironment::state() const {
  State st;
  const size_t n = (size_t)cfg.n_envs;
  st.s.resize(n);
  st.ep_step.resize(n);
  st.episode.resize(n);
  st.reward.resize(n);
  st.done.resize(n);
  st.action.resize(n);
  check(crl_get_state(engine, st.s.data(), st.reward.data(), st.done.data(), st.action.data(),
                      st.ep_step.data(), st.episode.data()),
        "state");
  return st;
}

BatchedEnvironment::EpisodeStats BatchedEnvironment::episodeStats() const {
  EpisodeStats st;
  const size_t n = (size_t)cfg.n_envs;
  st.last_return.resize(n);
  st.return_sum.resize(n);
  st.last_length.resize(n);
  st.length_sum.resize(n);
  check(crl_get_episode_stats(engine, st.last_return.data(), st.last_length.data(), st.return_sum.data(),
                              st.length_sum.data()),
        "episodeStats");
  return st;
}

std::vector<float> BatchedEnvironment::qTable(int table) const {
  std::vector<float> q((size_t)numStates() * numActions());
  check(crl_q_get(engine, table, q.data()), "qTable");
  return q;
}

void BatchedEnvironment::setQTable(int table, const std::vector<float>& q) {
  if (q.size() != (size_t)numStates() * numActions()) throw std::runtime_error("Invalid Q-table size");
  check(crl_q_set(engine, table, q.data()), "setQTable");
}

uint64_t BatchedEnvironment::stepCount() const {
  uint64_t t = 0;
  check(crl_get_step_count(engine, &t), "stepCount");
  return t;
}

void* BatchedEnvironment::devicePointer(int which) const {
  void* p = nullptr;
  check(crl_device_ptr(engine, which, &p), "devicePointer");
  return p;
}
