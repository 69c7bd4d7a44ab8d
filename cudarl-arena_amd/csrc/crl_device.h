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
  int max_episodes;  // > 0: envs that finished this many episodes stop stepping
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
// The reward is a class constant or ONE element of `cr`, at an index that is
// known as soon as the class of the target cell is: a single load that is in
// flight together with the table row of the new cell.
struct ClassRewards {
  float step, goal, trap;
};
template <class ClassOf>
__device__ __forceinline__ void step_rule(const Rules& R, const ClassRewards by, const ClassOf& cls,
                                          const float* __restrict__ cr, int& x, int& y, int a,
                                          float& reward, bool& hit) {
  int dx, dy;
  action_delta(a, R.A, dx, dy);
  const int nx = x + dx, ny = y + dy;
  const bool in = (unsigned)nx < (unsigned)R.W && (unsigned)ny < (unsigned)R.H;
  const int tgt = ny * R.W + nx;
  const int k = in ? cls(tgt) : kFree;
  const bool moved = in && k < kTrap;
  x = moved ? nx : x;
  y = moved ? ny : y;
  const int s2 = y * R.W + x;
  const bool trap = in && k == kTrap;
  // goal test: on the target cell, or (goal_mode 1) on the cell the env ends up on,
  // where it fires again while the env bumps into something next to the goal
  hit = R.goal_mode == 0 ? (in && k == kGoal) : (cls(s2) == kGoal);
  // goal beats trap; the goal pays on the goal cell (= s2 in both modes: a goal
  // target is moved onto), the trap on the target cell, anything else on s2
  const bool cells = (R.reward_flags & 1) != 0;
  const bool base_cells = cells && (R.reward_flags & 2) != 0;
  const float by_class = hit ? by.goal : trap ? by.trap : by.step;
  const bool from_cell = cells && (hit || trap || base_cells);
  float by_cell = 0.0f;
  if (cells) by_cell = cr[(trap && !hit) ? tgt : s2];  // uniform branch, index always inside the map
  reward = from_cell ? by_cell : by_class;
}

// Move codes: what each action does from one cell, 2 bits per action -
//   0 the env moves, 1 it moves onto the goal, 2 a trap (stays, trap reward),
//   3 blocked by a wall or by the edge of the grid (stays, step reward)
// - which is the class of the target cell, or 3 outside the grid.  Valid for the
// rule that tests the goal on the target cell (src/kernels.cu:34-66).  With the
// codes of the cell it stands on in a register, an env's next cell follows from
// its action without a map lookup or a bounds test.
// `word_of(i)` returns word i of the env's packed class map.
template <int A, class WordOf>
__device__ __forceinline__ uint32_t moves_of_cell(WordOf word_of, int W, int H, int x, int y, int s) {
  // all map words are asked for before the first one is looked at (a target
  // outside the grid reads the env's own cell instead, and the result is dropped)
  uint32_t word[A];
#pragma unroll
  for (int a = 0; a < A; ++a) {
    int dx, dy;
    action_delta(a, A, dx, dy);  // constants once the loop is unrolled
    const bool in = (dx == 0 || (unsigned)(x + dx) < (unsigned)W) &&
                    (dy == 0 || (unsigned)(y + dy) < (unsigned)H);
    const int tgt = in ? s + dy * W + dx : s;
    word[a] = word_of(tgt >> 4);
  }
#pragma unroll
  for (int a = 0; a < A; ++a) asm volatile("" : "+v"(word[a]));  // keeps the reads unconditional
  uint32_t mv = 0;
#pragma unroll
  for (int a = 0; a < A; ++a) {
    int dx, dy;
    action_delta(a, A, dx, dy);
    const bool in = (dx == 0 || (unsigned)(x + dx) < (unsigned)W) &&
                    (dy == 0 || (unsigned)(y + dy) < (unsigned)H);
    const int tgt = s + dy * W + dx;
    const uint32_t code = in ? (uint32_t)cell_class_of(word[a], tgt) : (uint32_t)kWall;
    mv |= code << (2 * a);
  }
  return mv;
}
// packed move codes: 16/A cells per 32-bit word
template <int A>
__device__ __forceinline__ constexpr int move_cells_per_word() { return 16 / A; }

// 16-byte loads / stores marked non-temporal: data that streams through once
typedef float crl_f4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 stream_load4(const float4* p) {
  const crl_f4 v = __builtin_nontemporal_load(reinterpret_cast<const crl_f4*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stream_store4(const float4 v, float4* p) {
  crl_f4 t;
  t.x = v.x;
  t.y = v.y;
  t.z = v.z;
  t.w = v.w;
  __builtin_nontemporal_store(t, reinterpret_cast<crl_f4*>(p));
}

// One table row in registers.  Named scalars passed BY VALUE: an element picked
// by a run-time action index must compile to a chain of selects.  Through a
// reference the optimiser folds "select of two loads" into one indexed load
// and the row ends up in scratch memory.
template <int A>
struct Row;

template <>
struct Row<4> {
  float q0, q1, q2, q3;
};
template <>
struct Row<8> {
  float q0, q1, q2, q3, q4, q5, q6, q7;
};

__device__ __forceinline__ Row<4> load_row4(const float* __restrict__ p) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  return Row<4>{t.x, t.y, t.z, t.w};
}
__device__ __forceinline__ Row<8> load_row8(const float* __restrict__ p) {
  const float4 t = reinterpret_cast<const float4*>(p)[0];
  const float4 u = reinterpret_cast<const float4*>(p)[1];
  return Row<8>{t.x, t.y, t.z, t.w, u.x, u.y, u.z, u.w};
}
template <int A>
__device__ __forceinline__ Row<A> load_row(const float* __restrict__ p);
template <>
__device__ __forceinline__ Row<4> load_row<4>(const float* __restrict__ p) { return load_row4(p); }
template <>
__device__ __forceinline__ Row<8> load_row<8>(const float* __restrict__ p) { return load_row8(p); }

// Keeps the optimiser from merging a conditionally loaded row with another one
// (which would make the conditional load wait for the other row first).
__device__ __forceinline__ void row_opaque(Row<4>& r) {
  asm volatile("" : "+v"(r.q0), "+v"(r.q1), "+v"(r.q2), "+v"(r.q3));
}
__device__ __forceinline__ void row_opaque(Row<8>& r) {
  asm volatile("" : "+v"(r.q0), "+v"(r.q1), "+v"(r.q2), "+v"(r.q3), "+v"(r.q4), "+v"(r.q5), "+v"(r.q6), "+v"(r.q7));
}

__device__ __forceinline__ Row<4> row_pick(bool c, const Row<4> a, const Row<4> b) {
  return Row<4>{c ? a.q0 : b.q0, c ? a.q1 : b.q1, c ? a.q2 : b.q2, c ? a.q3 : b.q3};
}
__device__ __forceinline__ Row<8> row_pick(bool c, const Row<8> a, const Row<8> b) {
  return Row<8>{c ? a.q0 : b.q0, c ? a.q1 : b.q1, c ? a.q2 : b.q2, c ? a.q3 : b.q3,
                c ? a.q4 : b.q4, c ? a.q5 : b.q5, c ? a.q6 : b.q6, c ? a.q7 : b.q7};
}

// lowest index wins ties (src/q_learning.cu:200-206: strict >)
__device__ __forceinline__ void amax_step(float v, int i, float& bv, int& bi) {
  const bool gt = v > bv;
  bv = gt ? v : bv;
  bi = gt ? i : bi;
}
__device__ __forceinline__ int row_argmax(const Row<4> r) {
  float bv = r.q0;
  int bi = 0;
  amax_step(r.q1, 1, bv, bi);
  amax_step(r.q2, 2, bv, bi);
  amax_step(r.q3, 3, bv, bi);
  return bi;
}
__device__ __forceinline__ int row_argmax(const Row<8> r) {
  float bv = r.q0;
  int bi = 0;
  amax_step(r.q1, 1, bv, bi);
  amax_step(r.q2, 2, bv, bi);
  amax_step(r.q3, 3, bv, bi);
  amax_step(r.q4, 4, bv, bi);
  amax_step(r.q5, 5, bv, bi);
  amax_step(r.q6, 6, bv, bi);
  amax_step(r.q7, 7, bv, bi);
  return bi;
}

__device__ __forceinline__ float row_get(const Row<4> r, int a) {
  float q = r.q0;
  q = (a == 1) ? r.q1 : q;
  q = (a == 2) ? r.q2 : q;
  q = (a == 3) ? r.q3 : q;
  return q;
}
__device__ __forceinline__ float row_get(const Row<8> r, int a) {
  float q = r.q0;
  q = (a == 1) ? r.q1 : q;
  q = (a == 2) ? r.q2 : q;
  q = (a == 3) ? r.q3 : q;
  q = (a == 4) ? r.q4 : q;
  q = (a == 5) ? r.q5 : q;
  q = (a == 6) ? r.q6 : q;
  q = (a == 7) ? r.q7 : q;
  return q;
}

__device__ __forceinline__ Row<4> row_set(const Row<4> r, int a, float q) {
  return Row<4>{(a == 0) ? q : r.q0, (a == 1) ? q : r.q1, (a == 2) ? q : r.q2, (a == 3) ? q : r.q3};
}
__device__ __forceinline__ Row<8> row_set(const Row<8> r, int a, float q) {
  return Row<8>{(a == 0) ? q : r.q0, (a == 1) ? q : r.q1, (a == 2) ? q : r.q2, (a == 3) ? q : r.q3,
                (a == 4) ? q : r.q4, (a == 5) ? q : r.q5, (a == 6) ? q : r.q6, (a == 7) ? q : r.q7};
}

// max_a' Q[s',a'] (src/gpu/kernels.cu:35-45), or floored at 0 (src/kernels.cu:101-110)
__device__ __forceinline__ float row_max(const Row<4> r, bool done, int max_mode) {
  float m = fmaxf(fmaxf(r.q0, r.q1), fmaxf(r.q2, r.q3));
  if (max_mode == 1) m = fmaxf(0.0f, m);
  return done ? 0.0f : m;
}
__device__ __forceinline__ float row_max(const Row<8> r, bool done, int max_mode) {
  float m = fmaxf(fmaxf(fmaxf(r.q0, r.q1), fmaxf(r.q2, r.q3)), fmaxf(fmaxf(r.q4, r.q5), fmaxf(r.q6, r.q7)));
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
