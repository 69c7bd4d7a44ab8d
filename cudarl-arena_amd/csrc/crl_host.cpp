// Host-only part of the C ABI: configuration checks, epsilon schedules, the
// float-grid classifier, Philox for tests, and the synthetic map generators.
#include "crl_host.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <thread>

#include "crl_philox.h"

namespace crl {

std::string& last_error() {
  thread_local std::string text;
  return text;
}

int fail_with(int code, const char* why) {
  try {
    last_error() = why;
  } catch (...) {  // out of memory for the text: the code still says what happened
  }
  return code;
}


int validate_config(const crl_config* c, std::string& why) {
  char buf[256];
  auto bad = [&](int code, const char* msg) {
    why = msg;
    return code;
  };
  if (!c) return bad(CRL_E_ARG, "config is null");
  if (c->struct_size != sizeof(crl_config)) {
    snprintf(buf, sizeof buf, "config.struct_size is %u, this library expects %zu", c->struct_size,
             sizeof(crl_config));
    return bad(CRL_E_ARG, buf);
  }
  if (c->n_envs < 1) return bad(CRL_E_ARG, "n_envs must be >= 1");
  if (c->width < 1 || c->height < 1) return bad(CRL_E_ARG, "width and height must be >= 1");
  if ((int64_t)c->width * c->height > (int64_t)1 << 24)
    return bad(CRL_E_ARG, "more than 2^24 cells per map");
  if (c->n_actions != 4 && c->n_actions != 8) return bad(CRL_E_ARG, "n_actions must be 4 or 8");
  if (c->table_mode != CRL_TABLE_PER_ENV && c->table_mode != CRL_TABLE_SHARED)
    return bad(CRL_E_ARG, "bad table_mode");
  if (c->map_mode != CRL_MAP_PER_ENV && c->map_mode != CRL_MAP_SHARED) return bad(CRL_E_ARG, "bad map_mode");
  if (c->max_mode != CRL_MAX_TRUE && c->max_mode != CRL_MAX_ZERO_FLOOR) return bad(CRL_E_ARG, "bad max_mode");
  if (c->goal_mode != CRL_GOAL_ON_TARGET && c->goal_mode != CRL_GOAL_ON_RESULT)
    return bad(CRL_E_ARG, "bad goal_mode");
  if (c->auto_reset != 0 && c->auto_reset != 1) return bad(CRL_E_ARG, "auto_reset must be 0 or 1");
  if (c->episode_len < 0) return bad(CRL_E_ARG, "episode_len must be >= 0");
  if (c->reward_flags & ~3) return bad(CRL_E_ARG, "unknown reward_flags bits");
  if ((c->reward_flags & CRL_REWARD_BASE_CELLS) && !(c->reward_flags & CRL_REWARD_CELLS))
    return bad(CRL_E_ARG, "CRL_REWARD_BASE_CELLS needs CRL_REWARD_CELLS");
  if (c->eps_mode < CRL_EPS_FIXED || c->eps_mode > CRL_EPS_EPISODE_LINEAR) return bad(CRL_E_ARG, "bad eps_mode");
  if (c->eps_mode != CRL_EPS_FIXED && c->eps_span < 1) return bad(CRL_E_ARG, "eps_span must be >= 1");
  if (c->eps_span > (1 << 26)) return bad(CRL_E_ARG, "eps_span too large");
  if (c->max_episodes < 0) return bad(CRL_E_ARG, "max_episodes must be >= 0");
  if (c->track_returns != 0 && c->track_returns != 1) return bad(CRL_E_ARG, "track_returns must be 0 or 1");
  if ((uint64_t)c->n_envs * (uint64_t)c->width * c->height > ((uint64_t)1 << 40))
    return bad(CRL_E_ARG, "n_envs * cells too large");
  return CRL_OK;
}

std::vector<float> build_eps_table(const crl_config& c) {
  std::vector<float> tab;
  if (c.eps_mode == CRL_EPS_FIXED) {
    tab.push_back(c.eps0);
  } else if (c.eps_mode == CRL_EPS_STEP_MULT || c.eps_mode == CRL_EPS_EPISODE_MULT) {
    tab.resize((size_t)c.eps_span);
    double e = (double)c.eps0;
    for (int i = 0; i < c.eps_span; ++i) {
      tab[(size_t)i] = (float)e;
      e *= (double)c.eps_decay;
    }
  } else {
    tab.resize((size_t)c.eps_span + 1);
    for (int i = 0; i <= c.eps_span; ++i)
      tab[(size_t)i] = (float)((double)c.eps0 +
                               ((double)c.eps_end - (double)c.eps0) * (double)i / (double)c.eps_span);
  }
  return tab;
}

void pack_classes(const uint8_t* cls, size_t n_cells, uint32_t* words) {
  const size_t n_words = (n_cells + 15) / 16;
  for (size_t w = 0; w < n_words; ++w) {
    uint32_t v = 0;
    const size_t base = w * 16;
    const size_t lim = std::min<size_t>(16, n_cells - base);
    for (size_t j = 0; j < lim; ++j) v |= (uint32_t)(cls[base + j] & 3u) << (2 * j);
    words[w] = v;
  }
}

namespace {

// word `i` of the stream (seed; a, stream id): counter (a, id, i/4, 0), lane i%4
struct WordStream {
  uint64_t seed;
  uint32_t a, id;
  uint32_t cached_block = 0xffffffffu;
  Philox4 blk{};
  WordStream(uint64_t s, uint32_t a_, uint32_t id_) : seed(s), a(a_), id(id_) {}
  uint32_t word(uint32_t i) {
    const uint32_t b = i >> 2;
    if (b != cached_block) {
      blk = philox4x32_10(a, id, b, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
      cached_block = b;
    }
    const uint32_t w[4] = {blk.w0, blk.w1, blk.w2, blk.w3};
    return w[i & 3];
  }
};

// f(i) for i in [0, n) on up to 16 threads.  Nothing escapes: false if f, or
// starting a thread, threw (the C ABI above never lets an exception through).
template <class F>
bool parallel_for(int n, F f) {
  unsigned hw = std::thread::hardware_concurrency();
  int workers = (int)std::min<unsigned>(hw ? hw : 1u, 16u);
  if (n < 4096) workers = 1;
  std::atomic<bool> ok{true};
  auto run = [&](int lo, int hi) {
    try {
      for (int i = lo; i < hi; ++i) f(i);
    } catch (...) {
      ok = false;
    }
  };
  if (workers <= 1) {
    run(0, n);
    return ok;
  }
  std::vector<std::thread> pool;
  try {
    pool.reserve((size_t)workers);
    for (int w = 0; w < workers; ++w)
      pool.emplace_back(run, (int)((int64_t)n * w / workers), (int)((int64_t)n * (w + 1) / workers));
  } catch (...) {
    ok = false;  // the threads already started still finish their share
  }
  for (auto& t : pool) t.join();
  return ok;
}

// index of the j-th FREE cell
int nth_free(const uint8_t* cls, int S, int j) {
  for (int c = 0; c < S; ++c)
    if (cls[c] == CRL_CELL_FREE && j-- == 0) return c;
  return -1;
}

}  // namespace
}  // namespace crl

extern "C" {

void crl_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  const crl::Philox4 r = crl::philox4x32_10(ctr[0], ctr[1], ctr[2], ctr[3], key[0], key[1]);
  out[0] = r.w0;
  out[1] = r.w1;
  out[2] = r.w2;
  out[3] = r.w3;
}

void crl_explore_draw(uint64_t seed, uint32_t env, uint64_t t, int32_t n_actions, float* u,
                      int32_t* a_rand) {
  const crl::Philox4 b = crl::explore_block(seed, env, t >> 1);
  const uint32_t w0 = (t & 1) ? b.w2 : b.w0;
  const uint32_t w1 = (t & 1) ? b.w3 : b.w1;
  if (u) *u = crl::u01(w0);
  if (a_rand) *a_rand = (int32_t)crl::below(w1, (uint32_t)n_actions);
}

int crl_eps_table(const crl_config* cfg, float* out, int32_t cap, int32_t* len) {
  const int rc = crl::validate_config(cfg, crl::last_error());
  if (rc != CRL_OK) return rc;
  try {
    const std::vector<float> tab = crl::build_eps_table(*cfg);
    if (len) *len = (int32_t)tab.size();
    if (out)
      for (int32_t i = 0; i < cap && (size_t)i < tab.size(); ++i) out[i] = tab[(size_t)i];
  } catch (...) {
    return crl::fail_with(CRL_E_ALLOC, "crl_eps_table: host allocation failed");
  }
  return CRL_OK;
}

int crl_classify_grid(const float* grid, size_t n, float step_reward, uint8_t* out_class,
                      float* out_reward) {
  if (!grid || !out_class) return crl::fail_with(CRL_E_ARG, "crl_classify_grid: null array");
  for (size_t i = 0; i < n; ++i) {
    const float v = grid[i];
    uint8_t k;
    float r = step_reward;
    if (v >= 0.99f) {  // src/kernels.cu:55
      k = CRL_CELL_GOAL;
      r = 1.0f;
    } else if (v < 0.0f && v > -1.0f) {  // src/kernels.cu:60
      k = CRL_CELL_TRAP;
      r = v;
    } else if (v < 0.0f) {  // src/kernels.cu:34: blocks, no special reward
      k = CRL_CELL_WALL;
    } else {
      k = CRL_CELL_FREE;
    }
    out_class[i] = k;
    if (out_reward) out_reward[i] = r;
  }
  return CRL_OK;
}

int crl_gen_maps_bernoulli(uint64_t seed, int32_t n_maps, int32_t n_envs, int32_t width,
                           int32_t height, float p_wall, float p_trap, uint8_t* cell_class,
                           int32_t* start) {
  if (n_maps < 1 || n_envs < 1 || width < 1 || height < 1 || !cell_class || !start)
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_bernoulli: sizes must be >= 1 and the arrays not null");
  if (n_maps != 1 && n_maps != n_envs)
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_bernoulli: one shared map or one map per env");
  if ((int64_t)width * height < 2 || (int64_t)width * height > ((int64_t)1 << 30))
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_bernoulli: a map has 2 to 2^30 cells");
  const int S = width * height;
  try {
  std::vector<int> n_free((size_t)n_maps), goal((size_t)n_maps);
  bool ok = crl::parallel_for(n_maps, [&](int m) {
    uint8_t* cls = cell_class + (size_t)m * S;
    crl::WordStream walls(seed, (uint32_t)m, crl::kStreamMap);
    crl::WordStream traps(seed, (uint32_t)m, crl::kStreamTrap);
    crl::WordStream sg(seed, (uint32_t)m, crl::kStreamStartGoal);
    int nf = 0;
    for (int c = 0; c < S; ++c) {
      uint8_t k = CRL_CELL_FREE;
      if (crl::u01(walls.word((uint32_t)c)) < p_wall)
        k = CRL_CELL_WALL;
      else if (p_trap > 0.0f && crl::u01(traps.word((uint32_t)c)) < p_trap)
        k = CRL_CELL_TRAP;
      cls[c] = k;
      nf += k == CRL_CELL_FREE;
    }
    // a map needs two free cells: clear cells 0 and S-1 if the draw left fewer
    if (nf < 2) {
      if (cls[0] != CRL_CELL_FREE) { cls[0] = CRL_CELL_FREE; ++nf; }
      if (nf < 2 && cls[S - 1] != CRL_CELL_FREE) { cls[S - 1] = CRL_CELL_FREE; ++nf; }
    }
    const int g = crl::nth_free(cls, S, (int)crl::below(sg.word(0), (uint32_t)nf));
    cls[g] = CRL_CELL_GOAL;
    n_free[(size_t)m] = nf - 1;
    goal[(size_t)m] = g;
    if (n_maps == n_envs)
      start[m] = crl::nth_free(cls, S, (int)crl::below(sg.word(1), (uint32_t)(nf - 1)));
  });
  if (n_maps == 1 && n_envs >= 1) {
    // shared map: every env draws its own start among the free cells
    const uint8_t* cls = cell_class;
    std::vector<int> free_cells;
    for (int c = 0; c < S; ++c)
      if (cls[c] == CRL_CELL_FREE) free_cells.push_back(c);
    const uint32_t nf = (uint32_t)free_cells.size();
    ok = crl::parallel_for(n_envs, [&](int i) {
      crl::WordStream sg(seed, (uint32_t)i, crl::kStreamStartGoal);
      start[i] = free_cells[crl::below(sg.word(4), nf)];
    }) && ok;
  }
  return ok ? CRL_OK : crl::fail_with(CRL_E_ALLOC, "crl_gen_maps_bernoulli: host allocation or a worker thread failed");
  } catch (...) {
    return crl::fail_with(CRL_E_ALLOC, "crl_gen_maps_bernoulli: host allocation failed");
  }
}

int crl_gen_maps_noise(uint64_t seed, int32_t n_maps, int32_t width, int32_t height, int32_t pitch,
                       float wall_frac, float sigma, float goal_bonus, uint8_t* cell_class,
                       int32_t* start, float* cell_reward) {
  if (n_maps < 1 || width < 1 || height < 1 || pitch < 1 || !cell_class || !start)
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_noise: sizes must be >= 1 and the arrays not null");
  if (!(wall_frac >= 0.0f && wall_frac < 1.0f))
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_noise: wall_frac must be in [0, 1)");
  if ((int64_t)width * height > ((int64_t)1 << 30))
    return crl::fail_with(CRL_E_ARG, "crl_gen_maps_noise: a map has at most 2^30 cells");
  const int S = width * height;
  if (S < 2) return crl::fail_with(CRL_E_ARG, "crl_gen_maps_noise: a map needs two cells");
  const int lw = (width + pitch - 1) / pitch + 1, lh = (height + pitch - 1) / pitch + 1;
  const bool ok = crl::parallel_for(n_maps, [&](int m) {
    uint8_t* cls = cell_class + (size_t)m * S;
    crl::WordStream lat(seed, (uint32_t)m, crl::kStreamLattice);
    std::vector<float> lattice((size_t)lw * lh);
    for (int i = 0; i < lw * lh; ++i) lattice[(size_t)i] = crl::u01(lat.word((uint32_t)i));
    std::vector<float> val((size_t)S);
    for (int y = 0; y < height; ++y)
      for (int x = 0; x < width; ++x) {
        const int gx = x / pitch, gy = y / pitch;
        float fx = (float)(x % pitch) / (float)pitch, fy = (float)(y % pitch) / (float)pitch;
        fx = fx * fx * (3.0f - 2.0f * fx);
        fy = fy * fy * (3.0f - 2.0f * fy);
        const float v00 = lattice[(size_t)gy * lw + gx], v10 = lattice[(size_t)gy * lw + gx + 1];
        const float v01 = lattice[(size_t)(gy + 1) * lw + gx], v11 = lattice[(size_t)(gy + 1) * lw + gx + 1];
        const float top = v00 + (v10 - v00) * fx, bot = v01 + (v11 - v01) * fx;
        val[(size_t)y * width + x] = top + (bot - top) * fy;
      }
    // the n_wall highest-valued cells are walls (ties broken by cell index)
    int n_wall = (int)((double)wall_frac * (double)S);
    if (n_wall > S - 2) n_wall = S - 2;
    std::vector<int> order((size_t)S);
    for (int c = 0; c < S; ++c) order[(size_t)c] = c;
    std::nth_element(order.begin(), order.begin() + n_wall, order.end(), [&](int a, int b) {
      return val[(size_t)a] > val[(size_t)b] || (val[(size_t)a] == val[(size_t)b] && a < b);
    });
    std::fill(cls, cls + S, (uint8_t)CRL_CELL_FREE);
    for (int i = 0; i < n_wall; ++i) cls[order[(size_t)i]] = CRL_CELL_WALL;
    const int nf = S - n_wall;
    crl::WordStream sg(seed, (uint32_t)m, crl::kStreamStartGoal);
    const int g = crl::nth_free(cls, S, (int)crl::below(sg.word(0), (uint32_t)nf));
    cls[g] = CRL_CELL_GOAL;
    start[m] = crl::nth_free(cls, S, (int)crl::below(sg.word(1), (uint32_t)(nf - 1)));
    if (cell_reward) {
      float* cr = cell_reward + (size_t)m * S;
      crl::WordStream rw(seed, (uint32_t)m, crl::kStreamReward);
      for (int c = 0; c < S; c += 2) {
        // Box-Muller on two words
        const float u1 = ((float)(rw.word((uint32_t)c) >> 8) + 1.0f) * (1.0f / 16777216.0f);
        const float u2 = crl::u01(rw.word((uint32_t)c + 1));
        const float rad = std::sqrt(-2.0f * std::log(u1));
        const float ang = 6.28318530717958647692f * u2;
        cr[c] = sigma * rad * std::cos(ang);
        if (c + 1 < S) cr[c + 1] = sigma * rad * std::sin(ang);
      }
      cr[g] += goal_bonus;
    }
  });
  return ok ? CRL_OK : crl::fail_with(CRL_E_ALLOC, "crl_gen_maps_noise: host allocation or a worker thread failed");
}

}  // extern "C"
