// Device-side building blocks shared by the gfx950 kernels: cell-class lookup,
// the grid-world step rule, row argmax and the TD arithmetic.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "crl_philox.h"

namespace crl {

constexpr int kFree = 0, kGoal = 1, kTrap = 2, kWall = 3;

// Everything a kernel needs to know about the rules; passed by value.
struct Rules {
  int W, H, A;
  int goal_mode;     // 0: class of the target cell, 1: class of the resulting cell
  int reward_flags;  // bit0: cell array for goal/trap, bit1: also for the base reward
  int auto_reset;
  int episode_len;
  int max_mode;  // 0 true max, 1 zero floor
  int eps_mode;  // 0 fixed, 1 by global step, 2/3 by per-env episode
  int eps_len;
  float lr, gamma;
  float step_reward, goal_reward, trap_reward;
  float eps0;
  uint64_t seed;
};

// 16 cells per 32-bit word, 2 bits per cell
__device__ __forceinline__ int cell_class_of(uint32_t word, int cell) {
  return (int)((word >> ((cell & 15) * 2)) & 3u);
}

// (dx,dy) of an action.  Actions outside [0,A) do not move
// (src/kernels.cu:15-23 has no default case).
__device__ __forceinline__ void action_delta(int a, int A, int& dx, int& dy) {
  // (d+1) in 2 bits per action: a = 0..7
  constexpr uint32_t kDx = 1u | (2u << 2) | (1u << 4) | (0u << 6) | (2u << 8) | (2u << 10) |
                           (0u << 12) | (0u << 14);
  constexpr uint32_t kDy = 0u | (1u << 2) | (2u << 4) | (1u << 6) | (0u << 8) | (2u << 10) |
                           (2u << 12) | (0u << 14);
  const bool ok = (unsigned)a < (unsigned)A;
  const int sh = (a & 7) * 2;
  dx = ok ? (int)((kDx >> sh) & 3u) - 1 : 0;
  dy = ok ? (int)((kDy >> sh) & 3u) - 1 : 0;
}

// One move (src/kernels.cu:13-66 on cell classes; goal_mode 1 gives
// src/environment.cu:17-48).  `cls(cell)` returns the class of a cell of this
// env's map, `cr` its per-cell rewards (may be null when unused).
template <class ClassOf>
__device__ __forceinline__ void step_rule(const Rules& R, ClassOf cls, const float* __restrict__ cr,
                                          int& x, int& y, int a, float& reward, bool& hit) {
  int dx, dy;
  action_delta(a, R.A, dx, dy);
  const int nx = x + dx, ny = y + dy;
  const bool in = (unsigned)nx < (unsigned)R.W && (unsigned)ny < (unsigned)R.H;
  const int tgt = ny * R.W + nx;
  const int k = in ? cls(tgt) : kFree;
  const bool moved = in && k < kTrap;
  if (moved) {
    x = nx;
    y = ny;
  }
  const int s2 = y * R.W + x;
  const bool cells = (R.reward_flags & 1) != 0;
  float r = (cells && (R.reward_flags & 2)) ? cr[s2] : R.step_reward;
  hit = false;
  if (R.goal_mode == 0) {
    if (in && k == kGoal) {
      r = cells ? cr[tgt] : R.goal_reward;
      hit = true;
    } else if (in && k == kTrap) {
      r = cells ? cr[tgt] : R.trap_reward;
    }
  } else {
    if (in && k == kTrap) r = cells ? cr[tgt] : R.trap_reward;
    if (cls(s2) == kGoal) {
      r = cells ? cr[s2] : R.goal_reward;
      hit = true;
    }
  }
  reward = r;
}

template <int A>
struct Row {
  float v[A];
};

template <int A>
__device__ __forceinline__ Row<A> load_row(const float* __restrict__ p) {
  Row<A> r;
  const float4* p4 = reinterpret_cast<const float4*>(p);
#pragma unroll
  for (int i = 0; i < A / 4; ++i) {
    const float4 t = p4[i];
    r.v[4 * i + 0] = t.x;
    r.v[4 * i + 1] = t.y;
    r.v[4 * i + 2] = t.z;
    r.v[4 * i + 3] = t.w;
  }
  return r;
}

// lowest index wins ties (src/q_learning.cu:200-206: strict >)
template <int A>
__device__ __forceinline__ int row_argmax(const Row<A>& r) {
  int best = 0;
  float bv = r.v[0];
#pragma unroll
  for (int a = 1; a < A; ++a) {
    const bool gt = r.v[a] > bv;
    bv = gt ? r.v[a] : bv;
    best = gt ? a : best;
  }
  return best;
}

template <int A>
__device__ __forceinline__ float row_get(const Row<A>& r, int a) {
  float q = r.v[0];
#pragma unroll
  for (int i = 1; i < A; ++i) q = (a == i) ? r.v[i] : q;
  return q;
}

template <int A>
__device__ __forceinline__ void row_set(Row<A>& r, int a, float q) {
#pragma unroll
  for (int i = 0; i < A; ++i) r.v[i] = (a == i) ? q : r.v[i];
}

// max_a' Q[s',a'] (src/gpu/kernels.cu:35-45), or floored at 0 (src/kernels.cu:101-110)
template <int A>
__device__ __forceinline__ float row_max(const Row<A>& r, bool done, int max_mode) {
  float m = r.v[0];
#pragma unroll
  for (int a = 1; a < A; ++a) m = fmaxf(m, r.v[a]);
  if (max_mode == 1) m = fmaxf(0.0f, m);
  return done ? 0.0f : m;
}

// Q + lr*((r + gamma*m) - Q) with the contractions written out
__device__ __forceinline__ float td_value(float q, float r, float m, float lr, float gamma) {
  const float target = __builtin_fmaf(gamma, m, r);
  return __builtin_fmaf(lr, target - q, q);
}
__device__ __forceinline__ float td_delta(float q, float r, float m, float lr, float gamma) {
  const float target = __builtin_fmaf(gamma, m, r);
  return lr * (target - q);
}

__device__ __forceinline__ float eps_of(const Rules& R, const float* __restrict__ tab, uint64_t t,
                                        int episode) {
  if (R.eps_mode == 0) return R.eps0;
  uint64_t i = (R.eps_mode == 1) ? t : (uint64_t)(episode < 0 ? 0 : episode);
  const uint64_t last = (uint64_t)(R.eps_len - 1);
  i = i > last ? last : i;
  return tab[i];
}

}  // namespace crl
