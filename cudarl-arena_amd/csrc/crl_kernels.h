// gfx950 kernels of the batched grid-world + tabular Q-learning engine.
//
// Data layout in HBM (all structure-of-arrays, one entry per env):
//   s, ep_step, episode : int32    reward : fp32    done, action : uint8
//   start               : int32 cell index
//   map                 : 2 bits per cell, 16 cells per uint32, map_words per map
//   moves               : 2 bits per (cell, action), derived from map, mv_words per map
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
  const uint32_t* moves;  // packed move codes of every cell, mv_words per map
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
  // episode statistics (all null unless tracked): running return of the open
  // episode, return / length of the last finished one, sums over finished ones
  float* ret_acc;
  float* ret_last;
  float* ret_sum;
  int32_t* len_last;
  int32_t* len_sum;
  // geometry
  int N;
  int map_words;   // uint32 words per map
  int mv_words;    // uint32 words of move codes per map
  int map_shared;  // 1: one map for all envs
  int table_shared;  // 1: one table for all envs
  size_t S;        // cells per map
};

// an episode of `env` just ended with return `ret` after `len` steps
__device__ __forceinline__ void record_episode(const Ptrs& P, int env, float ret, int len) {
  P.ret_last[env] = ret;
  P.len_last[env] = len;
  P.ret_sum[env] = P.ret_sum[env] + ret;
  P.len_sum[env] = P.len_sum[env] + len;
}

// trace row of an env that has used up its episode budget: it stays where it is
__device__ __forceinline__ void trace_idle(const Ptrs& P, int env, int row, int s) {
  if (env < P.trace_n && row < P.trace_cap) {
    const size_t o = (size_t)row * P.trace_n + env;
    P.tr_s[o] = s;
    P.tr_a[o] = 0;
    P.tr_r[o] = 0.0f;
    P.tr_d[o] = 0;
  }
}

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
// stands on live in registers for the whole launch: per step the only table
// traffic is the row of the new cell (asked for twice when the episode goes on:
// as the TD target's row and as the next row to act from - one cache line) and
// one 4-byte write.
// ---------------------------------------------------------------------------

// where an env's table lives while it is being stepped
constexpr int kTouchFloats = 2048;  // tables up to 8 KB are pulled into the caches whole ...
constexpr int kTouchMinSteps = 64;  // ... by launches long enough to use most of their lines
template <int A>
struct GlobalTable {  // in HBM / the caches
  float* __restrict__ q;
  __device__ __forceinline__ Row<A> load(int s) const { return load_row<A>(q + (size_t)s * A); }
  __device__ __forceinline__ void store(int s, int a, float v) const { q[(size_t)s * A + a] = v; }
  // Reads one word of every 128-byte line of a small table before its env starts
  // to step.  Left to the steps, each line's first use is a miss all the way to
  // HBM that holds up the whole wave - 64 envs x 32 lines, one or two at a time;
  // asked for together they cost one round trip (measured on 4 KB tables: +18 %).
  __device__ __forceinline__ void touch(int floats) const {
    if (floats > kTouchFloats) return;
    float acc = 0.0f;
    for (int i = 0; i < floats; i += 32) acc += q[i];
    asm volatile("" ::"v"(acc));
  }
};
template <int A>
struct LdsTable {  // staged into LDS for the whole launch
  float* q;
  __device__ __forceinline__ Row<A> load(int s) const { return load_row<A>(q + s * A); }
  __device__ __forceinline__ void store(int s, int a, float v) const { q[s * A + a] = v; }
};

// Where the fused loops get the move codes of a cell from.
// Pre-built codes staged in LDS, word-interleaved over the wave's lanes:
template <int A>
struct MovesLds {
  const uint32_t* base;  // the lane's first word
  int stride;            // words between two consecutive words of one env
  __device__ __forceinline__ uint32_t at(int s, int, int) const {
    constexpr unsigned kCells = (unsigned)move_cells_per_word<A>();
    const unsigned c = (unsigned)s;  // cell indices are never negative: shifts, not signed division
    return base[(c / kCells) * (unsigned)stride] >> ((c % kCells) * 2u * A);
  }
};
// Derived from the class map in LDS when the codes of all lanes do not fit: one
// map word per action, asked for while the table row is in flight.
template <int A>
struct MovesFromMap {
  const uint32_t* base;  // the lane's first map word, words 64 apart
  int W, H;
  __device__ __forceinline__ uint32_t at(int s, int x, int y) const {
    return moves_of_cell<A>([&](int word) -> uint32_t { return base[word * 64]; }, W, H, x, y, s);
  }
};

// Read from global memory, for maps whose codes do not fit LDS: one load, in
// flight together with the table row of the same cell.
template <int A>
struct MovesGlobal {
  const uint32_t* base;  // the env's (or the shared) packed move codes
  __device__ __forceinline__ uint32_t at(int s, int, int) const {
    constexpr unsigned kCells = (unsigned)move_cells_per_word<A>();
    const unsigned c = (unsigned)s;
    return base[c / kCells] >> ((c % kCells) * 2u * A);
  }
};

// n_steps of one env, any configuration.  `moves.at(cell, x, y)` gives the move
// codes of a cell of the env's map, `own_map` is the env's packed class map in
// global memory (read twice per launch, and only for the goal test on the
// resulting cell), `cr` its per-cell rewards (or null), `tab` its table.
// The step rule is step_rule()'s, restated on move codes: the class of the
// target cell is two bits of the codes of the cell the env stands on.
template <int A, class Table, class Moves>
__device__ __forceinline__ void run_env_steps(const Rules& R, const Ptrs& P, const int env,
                                              const uint64_t t0, const int n_steps, const Moves moves,
                                              const uint32_t* __restrict__ own_map,
                                              const float* __restrict__ cr, const Table tab) {
  // The class rewards as plain register values.  As loads from the kernel's
  // argument block, "cell reward or class reward" is turned into one load through
  // a selected pointer, which needs the class rewards copied to scratch memory.
  float r_step = R.step_reward, r_goal = R.goal_reward, r_trap = R.trap_reward;
  asm volatile("" : "+v"(r_step), "+v"(r_goal), "+v"(r_trap));
  const int W = R.W;
  const bool cells = (R.reward_flags & 1) != 0;
  const bool base_cells = cells && (R.reward_flags & 2) != 0;
  const bool goal_on_result = R.goal_mode != 0;
  int start = P.start[env];
  const int sx = start % W, sy = start / W;
  int s = P.s[env];
  int x = s % W, y = s / W;  // only followed when the move codes are derived from the map
  int ep_step = P.ep_step[env];
  int episode = P.episode[env];
  bool done = P.done[env] != 0;
  float reward = P.reward[env];  // rewritten unchanged if the env's episode budget is used up
  int action = P.action[env];
  Row<A> row = tab.load(s);
  uint32_t mv = moves.at(s, x, y);
  // goal test on the resulting cell: whether the env stands on a goal is carried
  // along (a move onto a cell tells its class); the start cell's answer is fixed
  int on_goal = 0, start_goal = 0;
  if (goal_on_result) {
    on_goal = cell_class_of(own_map[s >> 4], s) == kGoal;
    start_goal = cell_class_of(own_map[start >> 4], start) == kGoal;
  }
  Philox4 blk = explore_block(R.seed, (uint32_t)env, t0 >> 1);
  // Epsilon of a per-episode schedule stays in a register and is looked up again
  // only when an episode of the wave ends: as a load at the top of every step it
  // was a second round trip to memory per step, in front of the action.
  float eps = eps_of(R, P.eps_tab, t0, episode);
  const bool track = P.ret_acc != nullptr;
  float ret = track ? P.ret_acc[env] : 0.0f;
  // nothing loaded above is still in flight when the loop starts (a value still in
  // flight at the loop's entry makes the loop wait for ALL outstanding memory
  // operations on every iteration, the previous step's stores included)
  row_opaque(row);
  asm volatile("" : "+v"(ep_step), "+v"(episode), "+v"(reward), "+v"(action), "+v"(ret), "+v"(mv),
               "+v"(start), "+v"(s), "+v"(on_goal), "+v"(start_goal), "+v"(eps));

  for (int k = 0; k < n_steps; ++k) {
    if (R.max_episodes > 0 && episode >= R.max_episodes) {
      // budget used up: for ever, so the rest of the launch only fills the trace
      for (int kk = k; kk < n_steps; ++kk) trace_idle(P, env, P.trace_cursor + kk, s);
      break;
    }
    const uint64_t t = t0 + (uint64_t)k;
    Draw d = pick_draw(blk, t, A);
    if (P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
      const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
      d.u = P.u_sup[o];
      d.a = P.a_sup[o];
    }
    // indexed by the step: one address for the whole wave, read every step
    if (R.eps_mode == 1) eps = eps_of(R, P.eps_tab, t, episode);
    const int a = (d.u < eps) ? d.a : row_argmax(row);

    // the move (src/kernels.cu:13-66; goal on the resulting cell: src/environment.cu:43)
    const int s0 = s;
    const uint32_t code = (mv >> (2 * a)) & 3u;  // class of the target cell, WALL outside the grid
    const bool moved = code < (uint32_t)kTrap;
    const bool trap = code == (uint32_t)kTrap;
    int dx, dy;
    action_delta(a, A, dx, dy);
    const int tgt = s0 + __mul24(dy, W) + dx;  // inside the map whenever it is used
    const int s2 = moved ? tgt : s0;
    dx = moved ? dx : 0;
    dy = moved ? dy : 0;
    const int on_goal2 = moved ? (int)(code == (uint32_t)kGoal) : on_goal;
    const bool hit = goal_on_result ? on_goal2 != 0 : code == (uint32_t)kGoal;
    // goal beats trap; the goal pays on the goal cell (= s2 under both rules), the
    // trap on the target cell, anything else on s2: one load at one index
    const float by_class = hit ? r_goal : trap ? r_trap : r_step;
    float by_cell = 0.0f;
    if (cells) by_cell = cr[(trap && !hit) ? tgt : s2];
    reward = (cells && (hit || trap || base_cells)) ? by_cell : by_class;
    done = hit || (!R.auto_reset && done);

    // Everything the rest of this step and the start of the next one read from
    // memory is asked for here, in one go: the reward above, the row of the cell
    // the move ends on (for the TD target), the row and the move codes of the cell
    // the env acts from next - the same cell unless the episode ends with this
    // step and the env restarts.  One round trip per step, no branch around a
    // load.  An env that stays where it is reads its own row again (the pre-update
    // values: the write below comes later).
    ep_step += 1;
    const bool ends = R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len));
    s = ends ? start : s2;
    x = ends ? sx : x + dx;
    y = ends ? sy : y + dy;
    on_goal = ends ? start_goal : on_goal2;
    // (the second row only when an episode of the wave ends: a request that
    // nobody needs still takes its turn in the memory pipeline)
    const bool any_ends = __builtin_amdgcn_ballot_w64(ends) != 0;
    const Row<A> row2 = tab.load(s2);
    Row<A> row_restart{};
    if (any_ends) row_restart = tab.load(s);
    mv = moves.at(s, x, y);
    // the next step's draws depend on nothing: the Philox rounds run while the
    // loads are in flight
    if ((t & 1) == 1) blk = explore_block(R.seed, (uint32_t)env, (t + 1) >> 1);
    const float m = row_max(row2, done, R.max_mode);
    const float qn = td_value(row_get(row, a), reward, m, R.lr, R.gamma);
    tab.store(s0, a, qn);
    // the value just written, patched in from registers
    row = row_set(row_pick(ends, row_restart, row2), s == s0 ? a : -1, qn);

    action = a;
    ret = ret + reward;
    if (env < P.trace_n && P.trace_cursor + k < P.trace_cap) {
      const size_t o = (size_t)(P.trace_cursor + k) * P.trace_n + env;
      P.tr_s[o] = s2;
      P.tr_a[o] = (uint8_t)a;
      P.tr_r[o] = reward;
      P.tr_d[o] = done ? 1 : 0;
    }
    if (ends && track) record_episode(P, env, ret, ep_step);
    ret = ends ? 0.0f : ret;
    ep_step = ends ? 0 : ep_step;
    episode += ends ? 1 : 0;
    if (R.eps_mode >= 2 && any_ends) {
      eps = eps_of(R, P.eps_tab, t, episode);
      asm volatile("" : "+v"(eps));  // arrived before the loop goes round
    }
  }

  P.s[env] = s;
  P.ep_step[env] = ep_step;
  P.episode[env] = episode;
  if (track) P.ret_acc[env] = ret;
  P.reward[env] = reward;
  P.done[env] = done ? 1 : 0;
  P.action[env] = (uint8_t)action;
}

// The same loop for the common configuration, with everything that is fixed
// there folded away: fixed epsilon, class rewards (no per-cell array), goal test
// on the target cell, auto-reset, true max, no trace and no supplied stream.
// Fewer live scalars and no optional branches: about half the instructions of
// the general loop, which matters because a wave that waits for one row per
// step is also issue-bound on the arithmetic between two rows.
// Between the arrival of one row and the request for the next lie only the
// argmax, the draw and one shift of the cell's move codes; the codes of the next
// cell, the Philox rounds and the bookkeeping run while the row is in flight.
//
// PAIR: lanes l and l + 32 of the wave step the SAME env (a wave that can hold
// only 32 envs, because their tables fill the LDS, has half its lanes to spare).
// Both do everything twice - same addresses, same values - except the Philox
// rounds, the most expensive stretch of a step that waits for no memory: one
// lane computes the block of the next two steps, the other the block after, and
// they swap, so the rounds run every fourth step instead of every second.
//
// RICH adds the two things that configurations with large maps bring along and
// that cost one more request per step at most: per-cell rewards (`cr`, may be
// null) and an epsilon that follows the env's episode count.  The threshold
// stays in a register and is looked up again only when an episode of the wave
// ends, and so is the row of the start cell: with long episodes both are rare.
template <int A, bool PAIR, bool RICH, class Table, class Moves>
__device__ __forceinline__ void run_env_fast(const Rules& R, const Ptrs& P, const int env,
                                             const uint64_t t0, const int n_steps, const Moves moves,
                                             const float* __restrict__ cr, const Table tab) {
  const int W = R.W, T = R.episode_len;
  const float lr = R.lr, gamma = R.gamma;
  // u01(w) < eps  <=>  (w >> 8) < eps * 2^24, both sides exact: an integer compare
  auto threshold = [](float eps) -> uint32_t {
    const float scaled = ceilf(eps * 16777216.0f);
    return !(scaled > 0.0f) ? 0u : scaled >= 16777216.0f ? (1u << 24) : (uint32_t)scaled;
  };
  uint32_t explore_below = threshold(R.eps0);
  float r_step = R.step_reward, r_goal = R.goal_reward, r_trap = R.trap_reward;
  if (RICH) asm volatile("" : "+v"(r_step), "+v"(r_goal), "+v"(r_trap));  // plain values: no select of loads
  const bool cells = RICH && cr != nullptr;
  const bool base_cells = cells && (R.reward_flags & 2) != 0;
  const bool scheduled = RICH && R.eps_mode >= 2;
  int start = P.start[env];
  const int sx = start % W, sy = start / W;
  int s = P.s[env];
  int x = s % W, y = s / W;  // only followed when the move codes are derived from the map
  int ep_step = P.ep_step[env];
  int episode = P.episode[env];
  float reward = 0.0f;
  int action = 0;
  bool hit = false;
  Row<A> row = tab.load(s);
  uint32_t mv = moves.at(s, x, y);
  if (scheduled) explore_below = threshold(eps_of(R, P.eps_tab, t0, episode));
  const int lane = (int)__lane_id();
  const bool upper = PAIR && lane >= 32;
  // own block, and (PAIR) the partner lane's: {blk, nxt} = the next two blocks
  auto two_blocks = [&](uint64_t b, Philox4& first, Philox4& second) {
    const Philox4 own = explore_block(R.seed, (uint32_t)env, b + (upper ? 1 : 0));
    // v_permlane32_swap exchanges the upper 32 lanes of its first operand with the
    // lower 32 of its second: given the same value twice it returns the lower
    // half's words in both halves (block b) and the upper half's (block b + 1)
    const auto w0 = __builtin_amdgcn_permlane32_swap(own.w0, own.w0, false, false);
    const auto w1 = __builtin_amdgcn_permlane32_swap(own.w1, own.w1, false, false);
    const auto w2 = __builtin_amdgcn_permlane32_swap(own.w2, own.w2, false, false);
    const auto w3 = __builtin_amdgcn_permlane32_swap(own.w3, own.w3, false, false);
    first.w0 = w0[0];
    first.w1 = w1[0];
    first.w2 = w2[0];
    first.w3 = w3[0];
    second.w0 = w0[1];
    second.w1 = w1[1];
    second.w2 = w2[1];
    second.w3 = w3[1];
  };
  Philox4 blk, nxt{};
  bool have_nxt = PAIR;
  uint64_t next_block = (t0 >> 1) + (PAIR ? 2 : 1);
  if (PAIR)
    two_blocks(t0 >> 1, blk, nxt);
  else
    blk = explore_block(R.seed, (uint32_t)env, t0 >> 1);
  bool odd = (t0 & 1) != 0;
  // everything loaded above has arrived before the loop starts: a value still in
  // flight at the loop's entry makes the loop's first instruction wait for ALL
  // outstanding memory operations on every iteration, the previous step's store
  // included
  row_opaque(row);
  asm volatile("" : "+v"(ep_step), "+v"(episode), "+v"(mv), "+v"(start), "+v"(s));
  if (RICH) asm volatile("" : "+v"(explore_below));

  for (int k = 0; k < n_steps; ++k) {
    const uint32_t w0 = odd ? blk.w2 : blk.w0;
    const uint32_t w1 = odd ? blk.w3 : blk.w1;
    // both candidates are computed and one is selected: cheaper than a divergent branch
    const int greedy = row_argmax(row);
    const int a = ((w0 >> 8) < explore_below) ? (int)below(w1, (uint32_t)A) : greedy;

    const uint32_t code = (mv >> (2 * a)) & 3u;
    const bool moved = code < (uint32_t)kTrap;
    int dx, dy;
    action_delta(a, A, dx, dy);
    hit = code == (uint32_t)kGoal;
    const bool trap = code == (uint32_t)kTrap;
    reward = hit ? r_goal : (trap ? r_trap : r_step);
    float by_cell = 0.0f;
    if (RICH && cells) {
      // the goal pays on the goal cell (where the move ends), the trap on the
      // cell it guards, anything else where the move ends: one load at one index
      const int tgt = s + __mul24(dy, W) + dx;
      by_cell = cr[trap ? tgt : (moved ? tgt : s)];
    }
    dx = moved ? dx : 0;
    dy = moved ? dy : 0;
    const int s2 = s + __mul24(dy, W) + dx;

    // Two rows are asked for together: the one of the cell the move ends on (for
    // the TD target) and the one of the cell the env acts from next - the same
    // cell, and the same cache line, unless the episode ends with this step and the
    // env restarts.  No branch, and a restart costs no second round trip.  An env
    // that stays where it is reads its own row again (the pre-update values: the
    // write below comes later).
    ep_step += 1;
    const bool ends = hit || (T > 0 && ep_step >= T);
    const int s_next = ends ? start : s2;
    const Row<A> row2 = tab.load(s2);
    Row<A> row_next{};
    const bool any_ends = !RICH || __builtin_amdgcn_ballot_w64(ends) != 0;
    if (any_ends) row_next = tab.load(s_next);
    x = ends ? sx : x + dx;
    y = ends ? sy : y + dy;
    mv = moves.at(s_next, x, y);
    if (odd) {  // in the loads' shadow
      if (!PAIR) {
        blk = explore_block(R.seed, (uint32_t)env, next_block++);
      } else if (have_nxt) {
        blk = nxt;
        have_nxt = false;
      } else {
        two_blocks(next_block, blk, nxt);
        next_block += 2;
        have_nxt = true;
      }
    }
    if (RICH) reward = (cells && (hit || trap || base_cells)) ? by_cell : reward;
    const float m = row_max(row2, hit, 0);
    const float qn = td_value(row_get(row, a), reward, m, lr, gamma);
    tab.store(s, a, qn);

    // the cell to act from next, with the value just written patched in from registers
    row = row_set(RICH ? row_pick(ends, row_next, row2) : row_next, s_next == s ? a : -1, qn);
    ep_step = ends ? 0 : ep_step;
    episode += ends ? 1 : 0;
    s = s_next;
    action = a;
    odd = !odd;
    if (RICH && scheduled && any_ends) {
      explore_below = threshold(eps_of(R, P.eps_tab, t0, episode));
      asm volatile("" : "+v"(explore_below));  // arrived before the loop goes round
    }
  }

  P.s[env] = s;
  P.ep_step[env] = ep_step;
  P.episode[env] = episode;
  P.reward[env] = reward;
  P.done[env] = hit ? 1 : 0;
  P.action[env] = (uint8_t)action;
}

// Per-env tables whose maps are shared (MAP = 1: the one map's move codes staged
// in LDS) or too large for LDS (MAP = 2: move codes read from global memory, one
// load per step).  A block takes chunks blockIdx, blockIdx + gridDim, ... and runs
// each for all n_steps.  MODE 0: the general loop, 1: the folded loop, 2: the
// folded loop with two lanes per env (a batch too small to give every SIMD a wave
// of 64 envs: twice the waves, each with half the distinct addresses per request,
// and the Philox rounds shared between the lanes of a pair).
template <int A, int MAP, int MODE>
__global__ __launch_bounds__(256) void k_fused_per_env(const Rules R, const Ptrs P,
                                                        const uint64_t t0, const int n_steps) {
  constexpr bool FAST = MODE >= 1;
  constexpr bool PAIR = MODE == 2;  // two lanes per env: lanes l and l + 32 of a wave
  extern __shared__ uint32_t lds[];
  const int tid = threadIdx.x;
  const int bdim = blockDim.x;
  const int envs_per_block = PAIR ? bdim >> 1 : bdim;
  const int n_chunks = (P.N + envs_per_block - 1) / envs_per_block;
  const int slot = PAIR ? ((tid >> 6) << 5) + (tid & 31) : tid;

  if (MAP == 1) {
    for (int i = tid; i < P.mv_words; i += bdim) lds[i] = P.moves[i];
    __syncthreads();
  }
  for (int chunk = blockIdx.x; chunk < n_chunks; chunk += gridDim.x) {
    const int env = chunk * envs_per_block + slot;
    if (env >= P.N) continue;
    const float* cr =
        P.cell_reward ? P.cell_reward + (P.map_shared ? 0 : (size_t)env * P.S) : nullptr;
    const uint32_t* own_map = P.map + (P.map_shared ? 0 : (size_t)env * P.map_words);
    const GlobalTable<A> tab{P.Q + (size_t)env * P.S * A};
    if (MAP == 1) {
      if (FAST)
        run_env_fast<A, PAIR, true>(R, P, env, t0, n_steps, MovesLds<A>{lds, 1}, cr, tab);
      else
        run_env_steps<A>(R, P, env, t0, n_steps, MovesLds<A>{lds, 1}, own_map, cr, tab);
    } else {
      const MovesGlobal<A> moves{P.moves + (P.map_shared ? 0 : (size_t)env * P.mv_words)};
      if (FAST)
        run_env_fast<A, PAIR, true>(R, P, env, t0, n_steps, moves, cr, tab);
      else
        run_env_steps<A>(R, P, env, t0, n_steps, moves, own_map, cr, tab);
    }
  }
}

// Per-env tables with per-env maps small enough for LDS: every wave is an
// independent worker that draws env ranges from one ticket counter (32 envs per
// ticket), stages its envs' maps into its own LDS slice ([word][lane]: conflict
// free) and steps them for all n_steps.  The grid size sets how many envs - and
// how many bytes of their tables - are live on the chip at once: few enough and
// the rows an env keeps returning to are still in the last-level cache.
//
// All waves of a workgroup but the last step 64 envs each against tables in HBM /
// the caches, and spend most of their time waiting for one row per step.  With
// LDSW the last wave uses the idle issue slots and the LDS: it stages the WHOLE
// tables of 32 envs into LDS, steps them there and writes the tables back.  The
// split between the two kinds follows their speed; which worker steps an env does
// not change its results.
//
// MODE 0 is the general loop; 1 and 2 select the folded loop (run_env_fast; 2: its
// variant with per-cell rewards and per-episode epsilon), which works on move
// codes: the LDS wave always stages the pre-built codes of its envs; the table
// waves stage them too with MOVES, and otherwise stage the (four times smaller)
// class maps and derive the codes while their row loads are in flight.  With
// staged codes and `pair_tables` a table wave takes one ticket instead of two and
// gives every env two lanes, like the LDS wave: for batches too small to fill the
// chip with 64-env waves.
constexpr int kTicketEnvs = 32;

// `count` envs' words (`wpe` per env, contiguous in HBM) into [word][lane]; eight
// loads in flight per lane (one at a time, a short launch is spent waiting here)
__device__ __forceinline__ void stage_words(const uint32_t* __restrict__ src, const int count,
                                            const int wpe, const int stride, uint32_t* dst,
                                            const int lane) {
  const int total = count * wpe;
  auto put = [&](int i, uint32_t v) {
    const int e = i / wpe, w = i - e * wpe;
    dst[w * stride + e] = v;
  };
  int i0 = 0;
  for (; i0 + 64 * 8 <= total; i0 += 64 * 8) {
    uint32_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = __builtin_nontemporal_load(src + i0 + u * 64 + lane);  // read once per launch
#pragma unroll
    for (int u = 0; u < 8; ++u) put(i0 + u * 64 + lane, v[u]);
  }
  for (int i = i0 + lane; i < total; i += 64) put(i, __builtin_nontemporal_load(src + i));
}

template <int A, int MODE, bool LDSW, bool MOVES>
__global__ __launch_bounds__(LDSW ? 320 : 256) void k_fused_tickets(const Rules R, const Ptrs P,
                                                                     const uint64_t t0,
                                                                     const int n_steps,
                                                                     unsigned* __restrict__ ticket,
                                                                     const int tab_stride,
                                                                     const int fixed_tickets,
                                                                     const int pair_envs) {
  constexpr bool FAST = MODE >= 1;  // the folded loop ...
  constexpr bool RICH = MODE == 2;  // ... in its variant with per-cell rewards and per-episode epsilon
  extern __shared__ uint32_t lds[];
  const int n_waves = (int)(blockDim.x >> 6);  // with LDSW the last one works on LDS tables
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const bool lds_worker = LDSW && wave == n_waves - 1;
  // LDS: one slice per table wave, the LDS wave's slice, the tables
  constexpr bool kTableMoves = FAST && MOVES;
  const int slice = (kTableMoves ? P.mv_words : P.map_words) * 64;
  const int lds_slice = !LDSW ? 0 : FAST ? P.mv_words * kTicketEnvs : P.map_words * 64;
  uint32_t* my_words = lds + wave * slice;  // (the LDS wave is the last one)
  float* tabs = reinterpret_cast<float*>(lds + (n_waves - 1) * slice + lds_slice);
  // envs per ticket: 32, or what a thin table wave steps (never with an LDS wave beside it)
  const int unit = (FAST && MOVES && pair_envs) ? pair_envs : kTicketEnvs;
  const unsigned n_tickets = (unsigned)((P.N + unit - 1) / unit);
  // (pair_envs: the table waves, too, take one ticket and give every env several lanes)
  const bool thin = lds_worker || (FAST && MOVES && pair_envs);
  const int cap = thin ? unit : 64;
  const unsigned take = thin ? 1u : 2u;
  const size_t table = P.S * A;  // floats per table

  // fixed_tickets: the tickets are dealt by position, wave after wave, round after round
  // (workers that all take the same time need no counter).  With a wave for every pair of tickets (a short launch with all
  // envs in flight) the tickets are dealt by position: tens of thousands of
  // atomic draws from one counter would take longer than the few steps.
  if (fixed_tickets && blockIdx.x == 0 && threadIdx.x == 0) {
    ticket[1] = (unsigned)P.N;
    ticket[2] = 0u;
  }
  unsigned stepped = 0;  // envs this worker has stepped
  for (unsigned round = 0;; ++round) {
    unsigned base = 0;
    if (fixed_tickets) {
      base = ((round * gridDim.x + blockIdx.x) * (unsigned)n_waves + (unsigned)wave) * take;
    } else {
      if (lane == 0) base = atomicAdd(ticket, take);
      base = __shfl(base, 0);
    }
    if (base >= n_tickets) break;  // every worker gets here: the counter only grows
    const int env0 = (int)base * unit;
    const int n_here = min(cap, P.N - env0);
    const int env = env0 + lane;
    const bool live = lane < n_here;
    stepped += (unsigned)n_here;

    // this worker's maps: contiguous in HBM, transposed into [word][lane]
    __builtin_amdgcn_wave_barrier();
    const bool codes = FAST && (MOVES || lds_worker);
    if (codes)
      stage_words(P.moves + (size_t)env0 * P.mv_words, n_here, P.mv_words, cap, my_words, lane);
    else
      stage_words(P.map + (size_t)env0 * P.map_words, n_here, P.map_words, 64, my_words, lane);
    const float* cr = P.cell_reward ? P.cell_reward + (size_t)env * P.S : nullptr;

    if (!lds_worker) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (kTableMoves && pair_envs) {
        // lanes l, l + unit, ... step env l; the halves of the wave share the Philox rounds
        const int l = lane & (unit - 1);
        if (l < n_here) {
          const GlobalTable<A> tab{P.Q + (size_t)(env0 + l) * table};
          if (n_steps >= kTouchMinSteps) tab.touch((int)table);
          run_env_fast<A, true, RICH>(R, P, env0 + l, t0, n_steps, MovesLds<A>{my_words + l, unit},
                                      RICH && P.cell_reward ? P.cell_reward + (size_t)(env0 + l) * P.S : nullptr,
                                      tab);
        }
      } else if (live) {
        const GlobalTable<A> tab{P.Q + (size_t)env * table};
        if (n_steps >= kTouchMinSteps) tab.touch((int)table);
        if (kTableMoves)
          run_env_fast<A, false, RICH>(R, P, env, t0, n_steps, MovesLds<A>{my_words + lane, 64}, RICH ? cr : nullptr, tab);
        else if (FAST)
          run_env_fast<A, false, RICH>(R, P, env, t0, n_steps, MovesFromMap<A>{my_words + lane, R.W, R.H}, RICH ? cr : nullptr, tab);
        else
          run_env_steps<A>(R, P, env, t0, n_steps, MovesFromMap<A>{my_words + lane, R.W, R.H},
                           P.map + (size_t)env * P.map_words, cr, tab);
      }
    } else {
      // tables in: n_here consecutive tables are one contiguous run in HBM
      const float4* g4 = reinterpret_cast<const float4*>(P.Q + (size_t)env0 * table);
      const int t4 = (int)(table / 4);
      const int total4 = n_here * t4;
      // streamed once in and once out: marked non-temporal so that they do not
      // push the table waves' rows out of the L2
      auto ld = [&](int i) -> float4 { return stream_load4(g4 + i); };
      auto put = [&](int i, const float4 v) {
        const int e = i / t4, o = i - e * t4;
        reinterpret_cast<float4*>(tabs + e * tab_stride)[o] = v;
      };
      int i0 = 0;
      for (; i0 + 64 * 8 <= total4; i0 += 64 * 8) {  // eight loads in flight per lane
        const int i = i0 + lane;
        const float4 v0 = ld(i), v1 = ld(i + 64), v2 = ld(i + 128), v3 = ld(i + 192);
        const float4 v4 = ld(i + 256), v5 = ld(i + 320), v6 = ld(i + 384), v7 = ld(i + 448);
        put(i, v0);
        put(i + 64, v1);
        put(i + 128, v2);
        put(i + 192, v3);
        put(i + 256, v4);
        put(i + 320, v5);
        put(i + 384, v6);
        put(i + 448, v7);
      }
      for (int i = i0 + lane; i < total4; i += 64) put(i, ld(i));
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (FAST) {
        // lanes l and l + 32 both step env l of the ticket
        const int l = lane & (kTicketEnvs - 1);
        if (l < n_here) {
          const LdsTable<A> tab{tabs + l * tab_stride};
          run_env_fast<A, true, RICH>(R, P, env0 + l, t0, n_steps, MovesLds<A>{my_words + l, kTicketEnvs},
                                      RICH && P.cell_reward ? P.cell_reward + (size_t)(env0 + l) * P.S : nullptr,
                                      tab);
        }
      } else if (live) {
        const LdsTable<A> tab{tabs + lane * tab_stride};
        run_env_steps<A>(R, P, env, t0, n_steps, MovesFromMap<A>{my_words + lane, R.W, R.H},
                         P.map + (size_t)env * P.map_words, cr, tab);
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      float4* o4 = reinterpret_cast<float4*>(P.Q + (size_t)env0 * table);
      auto get = [&](int i) -> float4 {
        const int e = i / t4, o = i - e * t4;
        return reinterpret_cast<const float4*>(tabs + e * tab_stride)[o];
      };
      int j0 = 0;
      for (; j0 + 64 * 4 <= total4; j0 += 64 * 4) {
        const int i = j0 + lane;
        const float4 v0 = get(i), v1 = get(i + 64), v2 = get(i + 128), v3 = get(i + 192);
        stream_store4(v0, o4 + i);
        stream_store4(v1, o4 + i + 64);
        stream_store4(v2, o4 + i + 128);
        stream_store4(v3, o4 + i + 192);
      }
      for (int i = j0 + lane; i < total4; i += 64) stream_store4(get(i), o4 + i);
    }
  }
  // who did how much: once per worker (a pair of atomics per ticket had every wave of a
  // short launch queue at the counters whenever a round of tickets ended)
  if (!fixed_tickets && lane == 0 && stepped != 0u) atomicAdd(ticket + (lds_worker ? 2 : 1), stepped);
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
  if (R.max_episodes > 0 && P.episode[env] >= R.max_episodes) {
    T.s[env] = s0;  // budget used up: no move and, with action -1, no update
    T.a[env] = -1;
    T.r[env] = 0.0f;
    T.s2[env] = s0;
    T.done[env] = 0;
    trace_idle(P, env, P.trace_cursor, s0);
    return;
  }
  int x = s0 % R.W, y = s0 / R.W;
  const int a = act[env];
  float reward;
  bool hit;
  step_rule(R, ClassRewards{R.step_reward, R.goal_reward, R.trap_reward}, cls, cr, x, y, a, reward, hit);
  const int s2 = y * R.W + x;
  const bool done = hit || (!R.auto_reset && P.done[env] != 0);
  int ep_step = P.ep_step[env] + 1;
  const float ret = P.ret_acc ? P.ret_acc[env] + reward : 0.0f;
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
    if (P.ret_acc) {
      record_episode(P, env, ret, ep_step);
      P.ret_acc[env] = 0.0f;
    }
    P.s[env] = P.start[env];
    P.ep_step[env] = 0;
    P.episode[env] += 1;
  } else {
    if (P.ret_acc) P.ret_acc[env] = ret;
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
  if (P.ret_acc) P.ret_acc[env] = 0.0f;
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
                                                     unsigned long long* __restrict__ handoff) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  uint32_t* lds_map = reinterpret_cast<uint32_t*>(lds_raw + (REDUCE ? kReduceLdsBytes : 0));
  const int tid = threadIdx.x;
  const int env = blockIdx.x * blockDim.x + tid;
  bool live = env < P.N;
  // the env's cell is fetched while the map streams into LDS
  const int s_in = live ? P.s[env] : 0;
  if (REDUCE) reduce_block_init(*reinterpret_cast<ReduceLds*>(lds_raw));
  if (MAP == 1)
    for (int i = tid; i < P.map_words; i += blockDim.x) lds_map[i] = P.map[i];
  if (MAP == 1 || REDUCE) __syncthreads();
  int my_key = 0;
  float my_delta = 0.0f;
  if (live && R.max_episodes > 0 && P.episode[env] >= R.max_episodes) {
    live = false;  // budget used up: no move, no delta
    key[env] = -1;
    delta[env] = 0.0f;
    trace_idle(P, env, trace_row, s_in);
  }
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
    // The TD target needs the largest value of the row of the cell the move ends
    // on - one of the A neighbours, or this cell.  All of them are asked for now,
    // with the env's own row, instead of one more dependent round trip once the
    // action is known (the table is small and shared: these reads hit the caches).
    float nb_max[A];
#pragma unroll
    for (int i = 0; i < A; ++i) {
      int dx, dy;
      action_delta(i, A, dx, dy);
      const bool in = (unsigned)(x + dx) < (unsigned)R.W && (unsigned)(y + dy) < (unsigned)R.H;
      const int cell = in ? s0 + dy * R.W + dx : s0;
      nb_max[i] = row_max(load_row<A>(Q + (size_t)cell * A), false, 0);
    }
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
    step_rule(R, ClassRewards{R.step_reward, R.goal_reward, R.trap_reward}, cls, cr, x, y, a, reward, hit);
    const int s2 = y * R.W + x;
    const bool done = hit || (!R.auto_reset && P.done[env] != 0);
    float m = row_max(row, false, 0);  // the env stayed where it was
#pragma unroll
    for (int i = 0; i < A; ++i) m = (s2 != s0 && a == i) ? nb_max[i] : m;
    if (R.max_mode == 1) m = fmaxf(0.0f, m);
    m = done ? 0.0f : m;
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
    const float ret = P.ret_acc ? P.ret_acc[env] + reward : 0.0f;
    if (R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len))) {
      if (P.ret_acc) {
        record_episode(P, env, ret, ep_step);
        P.ret_acc[env] = 0.0f;
      }
      P.s[env] = P.start[env];
      P.ep_step[env] = 0;
      P.episode[env] = episode + 1;
    } else {
      if (P.ret_acc) P.ret_acc[env] = ret;
      P.s[env] = s2;
      P.ep_step[env] = ep_step;
    }
  }
  if (REDUCE) {
    ReduceLds& L = *reinterpret_cast<ReduceLds*>(lds_raw);
    reduce_block<false>(L, G, blockIdx.x, my_key, my_delta, live, handoff, 0u, reinterpret_cast<float*>(lds_raw + sizeof(ReduceLds)));
  }
}

// Move codes of maps [first, first + count) from their class maps: one thread per
// word of codes.
template <int A>
__global__ __launch_bounds__(256) void k_build_moves(const uint32_t* __restrict__ map,
                                                      const int map_words, const int W, const int H,
                                                      const int mv_words, const int first,
                                                      const int count, uint32_t* __restrict__ moves) {
  constexpr int kCells = move_cells_per_word<A>();
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= (size_t)count * mv_words) return;
  const int m = first + (int)(i / mv_words), w = (int)(i % mv_words);
  const uint32_t* g = map + (size_t)m * map_words;
  uint32_t out = 0;
#pragma unroll
  for (int j = 0; j < kCells; ++j) {
    const int c = w * kCells + j;
    if (c < W * H) {
      const uint32_t mv = moves_of_cell<A>([&](int word) -> uint32_t { return g[word]; }, W, H, c % W, c / W, c);
      out |= mv << (j * 2 * A);
    }
  }
  moves[(size_t)m * mv_words + w] = out;
}

__global__ void k_fill_u32(unsigned* p, const unsigned v, const size_t n) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
// (a launch instead of a device-to-device copy: a caller may record the call)
__global__ void k_copy3_u32(const unsigned* __restrict__ src, unsigned* __restrict__ dst) {
  if (threadIdx.x < 3) dst[threadIdx.x] = src[threadIdx.x];
}

// plain copy of n16 16-byte words: the known-size launch that calibrates the
// hardware traffic counters
__global__ __launch_bounds__(256) void k_probe_copy(const uint4* __restrict__ src,
                                                     uint4* __restrict__ dst, const size_t n16) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

}  // namespace crl
