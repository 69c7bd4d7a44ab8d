// gfx950 kernels of the batched grid-world + tabular Q-learning engine.
//
// Data layout in HBM (all structure-of-arrays, one entry per env):
//   s, ep_step, episode : int32    reward : fp32    done, action : uint8
//   start               : int32 cell index
//   map                 : 2 bits per cell, 16 cells per uint32, map_words per map
//   cell_reward         : fp32 per cell (optional)
//   Q                   : fp32 [table][s][a], one table per env or one shared
//
// Nothing here is a contraction, so there is no MFMA: every kernel is bound by
// HBM traffic or by dependent-access latency.
#pragma once
#include "crl_device.h"
#include "crl_reduce.h"

namespace crl {

struct Ptrs {
  int32_t* s;
  int32_t* ep_step;
  int32_t* episode;
  const int32_t* start;
  float* reward;
  uint8_t* done;
  uint8_t* action;
  const uint32_t* map;
  const float* cell_reward;
  float* Q;
  const float* eps_tab;
  // supplied exploration stream [sup_n][N], valid for steps sup_t0 .. sup_t0+sup_n-1
  const float* u_sup;
  const int32_t* a_sup;
  uint64_t sup_t0;
  int sup_n;
  // trace [cap][trace_n]
  int32_t* tr_s;
  uint8_t* tr_a;
  float* tr_r;
  uint8_t* tr_d;
  int trace_n, trace_cursor, trace_cap;
  // geometry
  int N;
  int map_words;   // uint32 words per map
  int map_shared;  // 1: one map for all envs
  int table_shared;  // 1: one table for all envs
  size_t S;        // cells per map
};

// the two draws of step t for one env
struct Draw {
  float u;
  int a;
};

__device__ __forceinline__ Draw pick_draw(const Philox4 blk, uint64_t t, int A) {
  const uint32_t w0 = (t & 1) ? blk.w2 : blk.w0;
  const uint32_t w1 = (t & 1) ? blk.w3 : blk.w1;
  Draw d;
  d.u = u01(w0);
  d.a = (int)below(w1, (uint32_t)A);
  return d;
}

// ---------------------------------------------------------------------------
// Fused select -> step -> update, per-env tables, one lane per env, n_steps per
// launch.  The env's position, episode counters and the Q row of the cell it
// stands on live in registers for the whole launch: per step the only memory
// traffic is one row read (the new cell) and one 4-byte write.
//
// MAP = 0: per-env maps staged once into LDS, word-interleaved across lanes
//          (word w of lane l at lds[w*blockDim + l]: conflict-free reads)
// MAP = 1: one shared map staged into LDS
// MAP = 2: maps read from global memory (too large for LDS)
// ---------------------------------------------------------------------------
template <int A, int MAP>
__global__ __launch_bounds__(256) void k_fused_per_env(const Rules R, const Ptrs P,
                                                        const uint64_t t0, const int n_steps) {
  extern __shared__ uint32_t lds[];
  const int tid = threadIdx.x;
  const int bdim = blockDim.x;
  const int n_chunks = (P.N + bdim - 1) / bdim;

  if (MAP == 1) {
    for (int i = tid; i < P.map_words; i += bdim) lds[i] = P.map[i];
    __syncthreads();
  }

  // A block takes chunks blockIdx, blockIdx + gridDim, ... and runs each for all
  // n_steps.  The grid size therefore sets how many envs (and how many bytes of
  // their tables) are live on the chip at once: small enough and the rows an
  // env keeps returning to are still in the last-level cache.
  for (int chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int env0 = chunk * bdim;
    const int env = env0 + tid;
    const bool live = env < P.N;

    if (MAP == 0) {
      __syncthreads();  // the previous chunk's readers are done with the map
      // the chunk's maps are contiguous in HBM: coalesced read, transposing write
      const int n_here = min(bdim, P.N - env0);
      const uint32_t* src = P.map + (size_t)env0 * P.map_words;
      const int total = n_here * P.map_words;
      for (int i = tid; i < total; i += bdim) {
        const int e = i / P.map_words, w = i - e * P.map_words;
        lds[w * bdim + e] = src[i];
      }
      __syncthreads();
    }
    if (!live) continue;  // only in the last chunk, after its barriers

    const uint32_t* gmap = P.map + (P.map_shared ? 0 : (size_t)env * P.map_words);
    auto cls = [&](int cell) -> int {
      uint32_t word;
      if (MAP == 0)
        word = lds[(cell >> 4) * bdim + tid];
      else if (MAP == 1)
        word = lds[cell >> 4];
      else
        word = gmap[cell >> 4];
      return cell_class_of(word, cell);
    };
    const float* cr =
        P.cell_reward ? P.cell_reward + (P.map_shared ? 0 : (size_t)env * P.S) : nullptr;

    float* __restrict__ Qe = P.Q + (size_t)env * P.S * A;
    const int start = P.start[env];
    const int sx = start % R.W, sy = start / R.W;
    int s = P.s[env];
    int x = s % R.W, y = s / R.W;
    int ep_step = P.ep_step[env];
    int episode = P.episode[env];
    bool done = P.done[env] != 0;
    float reward = 0.0f;
    int action = 0;
    Row<A> row = load_row<A>(Qe + (size_t)s * A);
    Philox4 blk = explore_block(R.seed, (uint32_t)env, t0 >> 1);

    for (int k = 0; k < n_steps; ++k) {
      const uint64_t t = t0 + (uint64_t)k;
      Draw d = pick_draw(blk, t, A);
      if (P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
        const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
        d.u = P.u_sup[o];
        d.a = P.a_sup[o];
      }
      const float eps = eps_of(R, P.eps_tab, t, episode);
      const int a = (d.u < eps) ? d.a : row_argmax(row);

      const int s0 = s;
      bool hit;
      step_rule(R, cls, cr, x, y, a, reward, hit);
      const int s2 = y * R.W + x;
      done = hit || (!R.auto_reset && done);

      // Q row of the new cell; when the env did not move it is the row in registers
      Row<A> row2 = row;
      if (s2 != s0) row2 = load_row<A>(Qe + (size_t)s2 * A);
      // the next step's draws depend on nothing: the Philox rounds run while the
      // row load is in flight
      if ((t & 1) == 1) blk = explore_block(R.seed, (uint32_t)env, (t + 1) >> 1);
      const float m = row_max(row2, done, R.max_mode);
      const float qn = td_value(row_get(row, a), reward, m, R.lr, R.gamma);
      Qe[(size_t)s0 * A + a] = qn;
      if (s2 == s0) row2 = row_set(row2, a, qn);

      ep_step += 1;
      action = a;
      if (env < P.trace_n && P.trace_cursor + k < P.trace_cap) {
        const size_t o = (size_t)(P.trace_cursor + k) * P.trace_n + env;
        P.tr_s[o] = s2;
        P.tr_a[o] = (uint8_t)a;
        P.tr_r[o] = reward;
        P.tr_d[o] = done ? 1 : 0;
      }
      if (R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len))) {
        x = sx;
        y = sy;
        s = start;
        ep_step = 0;
        episode += 1;
        row = load_row<A>(Qe + (size_t)start * A);
        if (start == s0) row = row_set(row, a, qn);  // the value just written, from registers
      } else {
        s = s2;
        row = row2;
      }
    }

    P.s[env] = s;
    P.ep_step[env] = ep_step;
    P.episode[env] = episode;
    P.reward[env] = reward;
    P.done[env] = done ? 1 : 0;
    P.action[env] = (uint8_t)action;
  }
}

// ---------------------------------------------------------------------------
// Stand-alone pieces: select, step, update.  They reproduce one fused step when
// called in that order and back the reference-shaped host classes.
// ---------------------------------------------------------------------------

// Epsilon-greedy select with A lanes per env: lane a holds Q[s][a] (one
// coalesced read of the row), and the argmax runs over the lane group with
// cross-lane shuffles on (value, index) so that the lowest index wins ties
// (src/q_learning.cu:200-206).  The group's first lane draws and writes.
template <int A>
__global__ __launch_bounds__(256) void k_select(const Rules R, const Ptrs P, const uint64_t t,
                                                 int32_t* __restrict__ act_out) {
  const int gid = blockIdx.x * blockDim.x + threadIdx.x;
  const int env = gid / A;
  const int a = gid - env * A;
  const bool live = env < P.N;
  const int e = live ? env : P.N - 1;  // keep whole groups active for the shuffles
  const int s = P.s[e];
  const float* Qe = P.Q + (P.table_shared ? 0 : (size_t)e * P.S * A);
  float v = Qe[(size_t)s * A + a];
  int idx = a;
#pragma unroll
  for (int m = 1; m < A; m <<= 1) {
    const float ov = __shfl_xor(v, m);
    const int oi = __shfl_xor(idx, m);
    const bool take = (ov > v) || (ov == v && oi < idx);
    v = take ? ov : v;
    idx = take ? oi : idx;
  }
  if (!live || a != 0) return;
  Draw d = pick_draw(explore_block(R.seed, (uint32_t)env, t >> 1), t, A);
  if (P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
    const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
    d.u = P.u_sup[o];
    d.a = P.a_sup[o];
  }
  const float eps = eps_of(R, P.eps_tab, t, P.episode[env]);
  act_out[env] = (d.u < eps) ? d.a : idx;
}

// transition left behind by k_step for k_update_* : (s, a, r, s', done)
struct Transition {
  int32_t* s;
  int32_t* a;
  float* r;
  int32_t* s2;
  uint8_t* done;
};

// One move for every env with supplied actions (src/environment.cu:113-125,
// rules of src/kernels.cu:13-66), then the restart of finished envs.
__global__ __launch_bounds__(256) void k_step(const Rules R, const Ptrs P, const Transition T,
                                               const int32_t* __restrict__ act) {
  const int env = blockIdx.x * blockDim.x + threadIdx.x;
  if (env >= P.N) return;
  const uint32_t* gmap = P.map + (P.map_shared ? 0 : (size_t)env * P.map_words);
  auto cls = [&](int cell) -> int { return cell_class_of(gmap[cell >> 4], cell); };
  const float* cr = P.cell_reward ? P.cell_reward + (P.map_shared ? 0 : (size_t)env * P.S) : nullptr;
  const int s0 = P.s[env];
  int x = s0 % R.W, y = s0 / R.W;
  const int a = act[env];
  float reward;
  bool hit;
  step_rule(R, cls, cr, x, y, a, reward, hit);
  const int s2 = y * R.W + x;
  const bool done = hit || (!R.auto_reset && P.done[env] != 0);
  int ep_step = P.ep_step[env] + 1;
  T.s[env] = s0;
  T.a[env] = a;
  T.r[env] = reward;
  T.s2[env] = s2;
  T.done[env] = done ? 1 : 0;
  P.reward[env] = reward;
  P.done[env] = done ? 1 : 0;
  P.action[env] = (uint8_t)a;
  if (env < P.trace_n && P.trace_cursor < P.trace_cap) {
    const size_t o = (size_t)P.trace_cursor * P.trace_n + env;
    P.tr_s[o] = s2;
    P.tr_a[o] = (uint8_t)a;
    P.tr_r[o] = reward;
    P.tr_d[o] = done ? 1 : 0;
  }
  if (R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len))) {
    P.s[env] = P.start[env];
    P.ep_step[env] = 0;
    P.episode[env] += 1;
  } else {
    P.s[env] = s2;
    P.ep_step[env] = ep_step;
  }
}

// Environment::reset for envs [first, first+count) (src/environment.cu:6-14)
__global__ __launch_bounds__(256) void k_reset(const Ptrs P, const int first, const int count) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  const int env = first + i;
  P.s[env] = P.start[env];
  P.ep_step[env] = 0;
  P.reward[env] = 0.0f;
  P.done[env] = 0;
  P.action[env] = 0;
}

// TD update of one recorded transition per env on the env's own table
// (src/gpu/kernels.cu:7-54, one thread per sample; tables are disjoint)
template <int A>
__global__ __launch_bounds__(256) void k_update_per_env(const Rules R, const Ptrs P,
                                                         const Transition T) {
  const int env = blockIdx.x * blockDim.x + threadIdx.x;
  if (env >= P.N) return;
  float* Qe = P.Q + (size_t)env * P.S * A;
  const int s = T.s[env], a = T.a[env], s2 = T.s2[env];
  if ((unsigned)a >= (unsigned)A) return;  // an invalid action has no table entry
  const Row<A> row2 = load_row<A>(Qe + (size_t)s2 * A);
  const float m = row_max(row2, T.done[env] != 0, R.max_mode);
  const size_t k = (size_t)s * A + a;
  Qe[k] = td_value(Qe[k], T.r[env], m, R.lr, R.gamma);
}

// (key, delta) of n transitions against ONE table Q (K = S*A entries), all
// reads before any write.  key = s*A + a, or -1 for an invalid action.
template <int A>
__global__ __launch_bounds__(256) void k_delta(const float* __restrict__ Q, const int n,
                                                const int32_t* __restrict__ s,
                                                const int32_t* __restrict__ a,
                                                const float* __restrict__ r,
                                                const int32_t* __restrict__ s2,
                                                const uint8_t* __restrict__ done, const float lr,
                                                const float gamma, const int max_mode,
                                                int32_t* __restrict__ key,
                                                float* __restrict__ delta) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int ai = a[i];
  if ((unsigned)ai >= (unsigned)A) {
    key[i] = -1;
    delta[i] = 0.0f;
    return;
  }
  const Row<A> row2 = load_row<A>(Q + (size_t)s2[i] * A);
  const float m = row_max(row2, done[i] != 0, max_mode);
  const int k = s[i] * A + ai;
  key[i] = k;
  delta[i] = td_delta(Q[k], r[i], m, lr, gamma);
}

// Shared table, first half of a fused step: every env selects, moves and emits
// (key, delta) against the table as it stands; nothing is written to Q.  With
// REDUCE the workgroup (= one 256-sample block of the ordered reduction) also
// folds its own deltas and hands the block sums to the key owners.
// MAP = 1: shared map staged in LDS; MAP = 2: maps in global memory.
template <int A, int MAP, bool REDUCE>
__global__ __launch_bounds__(256) void k_shared_act(const Rules R, const Ptrs P, const uint64_t t,
                                                     const int trace_row,
                                                     int32_t* __restrict__ key,
                                                     float* __restrict__ delta, const ReduceGeom G,
                                                     uint2* __restrict__ handoff) {
  extern __shared__ unsigned char lds_raw[];
  uint32_t* lds_map = reinterpret_cast<uint32_t*>(lds_raw + (REDUCE ? sizeof(ReduceLds) : 0));
  const int tid = threadIdx.x;
  const int env = blockIdx.x * blockDim.x + tid;
  const bool live = env < P.N;
  // the env's cell is fetched while the map streams into LDS
  const int s_in = live ? P.s[env] : 0;
  if (MAP == 1) {
    for (int i = tid; i < P.map_words; i += blockDim.x) lds_map[i] = P.map[i];
    __syncthreads();
  }
  int my_key = 0;
  float my_delta = 0.0f;
  if (live) {
    const uint32_t* gmap = P.map + (P.map_shared ? 0 : (size_t)env * P.map_words);
    auto cls = [&](int cell) -> int {
      const uint32_t word = (MAP == 1) ? lds_map[cell >> 4] : gmap[cell >> 4];
      return cell_class_of(word, cell);
    };
    const float* cr =
        P.cell_reward ? P.cell_reward + (P.map_shared ? 0 : (size_t)env * P.S) : nullptr;
    const float* __restrict__ Q = P.Q;

    const int s0 = s_in;
    int x = s0 % R.W, y = s0 / R.W;
    const Row<A> row = load_row<A>(Q + (size_t)s0 * A);
    Draw d = pick_draw(explore_block(R.seed, (uint32_t)env, t >> 1), t, A);
    if (P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
      const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
      d.u = P.u_sup[o];
      d.a = P.a_sup[o];
    }
    const int episode = P.episode[env];
    const float eps = eps_of(R, P.eps_tab, t, episode);
    const int a = (d.u < eps) ? d.a : row_argmax(row);
    float reward;
    bool hit;
    step_rule(R, cls, cr, x, y, a, reward, hit);
    const int s2 = y * R.W + x;
    const bool done = hit || (!R.auto_reset && P.done[env] != 0);
    const Row<A> row2 = load_row<A>(Q + (size_t)s2 * A);
    const float m = row_max(row2, done, R.max_mode);
    my_key = s0 * A + a;
    my_delta = td_delta(row_get(row, a), reward, m, R.lr, R.gamma);
    key[env] = my_key;
    delta[env] = my_delta;

    const int ep_step = P.ep_step[env] + 1;
    P.reward[env] = reward;
    P.done[env] = done ? 1 : 0;
    P.action[env] = (uint8_t)a;
    if (env < P.trace_n && trace_row < P.trace_cap) {
      const size_t o = (size_t)trace_row * P.trace_n + env;
      P.tr_s[o] = s2;
      P.tr_a[o] = (uint8_t)a;
      P.tr_r[o] = reward;
      P.tr_d[o] = done ? 1 : 0;
    }
    if (R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len))) {
      P.s[env] = P.start[env];
      P.ep_step[env] = 0;
      P.episode[env] = episode + 1;
    } else {
      P.s[env] = s2;
      P.ep_step[env] = ep_step;
    }
  }
  if (REDUCE) {
    ReduceLds& L = *reinterpret_cast<ReduceLds*>(lds_raw);
    reduce_block(L, G, blockIdx.x, my_key, my_delta, live, handoff);
  }
}

// plain copy of n16 16-byte words: the known-size launch that calibrates the
// hardware traffic counters
__global__ __launch_bounds__(256) void k_probe_copy(const uint4* __restrict__ src,
                                                     uint4* __restrict__ dst, const size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

}  // namespace crl
