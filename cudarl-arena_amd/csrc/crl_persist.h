// Shared table, all steps of a launch in ONE kernel: 256 workgroups, one per compute
// unit, every one of them a block of the ordered reduction (256 envs, state in
// registers for the whole launch; fewer envs: blocks without envs) and the owner of up
// to 64 keys (whole table rows, values in registers), and the two roles hand their
// data to each other through memory.  Always 256 owners, also where the table would
// fit fewer: an owner's 256 cells are then small ones, every workgroup has a part in
// both passes, and a table of few cells that many envs crowd on is spread as far as
// it goes (65,536 envs on a 16x16x4 table: 7.2 us per step with 256 owners of one row
// each, 14.3 with 16 owners of 16 rows).
//
// What is exchanged is only ever touched with device-scope accesses (st_dev64 /
// ld_dev64: coherent between the eight XCDs without fences), and every exchanged
// datum is a 64-bit unit that carries the tag of the step it belongs to.  A reader
// asks for the data itself, again and again until the tags are the step's: there
// are no flags, no "store, wait for the acknowledgement, then publish", and one
// trip through memory per exchange instead of two.
//
//   view[cell]   2 A units, side by side, everything a step of an env on that cell needs:
//                  [0, A)   {value, tag} of the cell's A keys, published by the row's owner
//                  [A, 2A)  {max of the row of the cell that action i leads to, tag},
//                           published by THAT row's owner (the cell itself where the move
//                           would leave the grid): one row maximum goes to up to A + 2 places
//   cell[block][owner]          block sums, records as in crl_reduce.h: a main half of 4 records,
//                               written whole every step ([block][owner]: 8 KB of whole lines per
//                               block), and an extension of 4 more ([owner][block]) that only a
//                               block with more than 4 distinct keys for that owner writes into
//   raw[env]     {delta, key, tag}   only from blocks whose cell for some owner overflowed
//
// One step k (tag k + 1 for what the blocks read, k + 2 for the table that results):
//   block:  what does not depend on the table (exploration draw, neighbour cells, move
//           codes; the owner's stores are on their way meanwhile) -> poll the view of
//           the env's cell -> select, move, (key, delta) -> ordered block sums -> cells
//   owner:  wave by wave (64 blocks = four groups of the tree each): clear the wave's
//           quarter of the tile -> poll the cells of its blocks -> into the tile -> its
//           four group sums; one barrier; totals in group order -> new values and row
//           maxima into the views
// An owner overwrites its values only after it has every block's cells of the step,
// which a block writes after all its threads have read theirs: one buffer of views
// suffices.  Cells and raw samples have two buffers, taken in turn: a workgroup that
// writes the cells of step k + 2 has read table values of step k + 2 (or, without
// envs, has had all cells of step k + 1 as an owner), so some owner has had the
// cells of step k + 1 of ALL workgroups, which - a workgroup does its two roles one
// after the other, and every workgroup writes cells every step, empty ones if it has
// no envs - were all through with their owner's part of step k by then.
//
// Every wait is bounded: a thread that polls `spin_limit` times in vain (or sees the
// give-up word set) makes its workgroup set the give-up word and leave.
#pragma once
#include <type_traits>

#include "crl_kernels.h"

namespace crl {

constexpr int kPersistSpinLimit = 1 << 20;  // polls of a fraction of a microsecond each
constexpr int kPersistMaxGroups = 256;      // workgroups: one per compute unit, all resident
constexpr int kPersistOwnShift = 8;         // log2(owners): always 256, every workgroup is one
constexpr int kMainShift = 2, kMainRecs = 1 << kMainShift;  // records in the half of a cell that is written every step
static_assert(main_shift_for(kPersistOwnShift) == kMainShift && cell_shift_for(kPersistOwnShift) == kMainShift + 1 &&
              (1 << kPersistOwnShift) == kPersistMaxGroups && (kPersistMaxGroups << (kMainShift - 1)) == kStagePieces,
              "the owner's loads are laid out for cells of 4 + 4 records");
constexpr int kPersistMaxSteps = 65535;     // per launch: the raw samples' tags have 17 bits
constexpr int kPersistClockWords = 20 + 8 * 256;  // 2 workgroups x (8 phases + polls of the two waits by thread 0),
                                                  // then the wall clock of every workgroup at the 8 marks of one step

struct alignas(16) PersistLds {
  ReduceLds red;
  alignas(16) float tile[kTileBlocks * kOwnKeys];       // the owner's [block][key] block sums: a quarter (64 blocks) to a wave, which
                                                        // clears, fills and adds up its quarter without waiting for the others
  alignas(16) unsigned long long stage[kPersistMaxGroups << kMainShift];  // the main halves of the block's cells on their way out
  alignas(16) float gsum[(kTileBlocks / kGroupBlocks) * kOwnKeys];  // [group][key] (written 16 bytes at a time)
  float o_delta[kBlockSamples];                         // raw samples of one overflowing block
  uint8_t o_slot[kBlockSamples];
  uint8_t o_list[kTileBlocks];  // blocks whose cell overflowed this step
  int o_count;
  int dead;  // some thread gave up waiting (never cleared)
};

struct PersistBufs {
  unsigned long long* table;   // view [S][2 A]
  unsigned long long* cells;   // 2 x [workgroups][owners][main half], then 2 x [owners][workgroups][extension]
  unsigned long long* raw;     // [N]
  unsigned* err;               // give-up word
  unsigned long long* clocks;  // kPersistClockWords phase clocks, or null
};

__device__ __forceinline__ unsigned long long tagged(uint32_t bits, uint32_t tag) {
  return (unsigned long long)bits | ((unsigned long long)tag << 32);
}
__device__ __forceinline__ uint32_t tag_of(unsigned long long v) { return (uint32_t)(v >> 32); }
__device__ __forceinline__ float value_of(unsigned long long v) { return __uint_as_float((uint32_t)v); }

// raw sample: delta in the low word; key, valid bit and a 17-bit tag in the high word
constexpr uint32_t kRawKeyMask = 0x3FFFu, kRawValid = 0x4000u;
constexpr int kRawTagShift = 15;
static_assert(kDenseKeys - 1 <= (int)kRawKeyMask, "raw samples hold 14-bit keys");
static_assert(kPersistMaxSteps + 1 < (1 << (32 - kRawTagShift)), "raw tags must be unique within a launch");
static_assert((uint32_t)kPersistMaxSteps + 1u <= kRecTagMask, "record tags must be unique within a launch");

template <int A>
__device__ __forceinline__ Row<A> row_of_tagged(const unsigned long long (&v)[A]);
template <>
__device__ __forceinline__ Row<4> row_of_tagged<4>(const unsigned long long (&v)[4]) {
  return Row<4>{value_of(v[0]), value_of(v[1]), value_of(v[2]), value_of(v[3])};
}
template <>
__device__ __forceinline__ Row<8> row_of_tagged<8>(const unsigned long long (&v)[8]) {
  return Row<8>{value_of(v[0]), value_of(v[1]), value_of(v[2]), value_of(v[3]),
                value_of(v[4]), value_of(v[5]), value_of(v[6]), value_of(v[7])};
}

// Phase clocks (CLK only): thread 0 of the first and the last workgroup add up the shader
// clocks between the marks of a step.  Phases: 0 work before the table is needed, 1 wait
// for the table, 2 select / move / delta, 3 ordered block sums + cells, 4 clearing the
// tile, 5 wait for the cells and put them into the tile, 6 group sums + barrier + totals +
// publish, 7 loop overhead.
#define CRL_MARK(i)                                                                         \
  do {                                                                                      \
    if (CLK) {                                                                              \
      const unsigned long long now_ = clock64();                                            \
      phase_[i] += now_ - last_;                                                            \
      last_ = now_;                                                                         \
      if (k == n_steps / 2 && tid == 0 && B.clocks) B.clocks[20 + wg * 8 + (i)] = wall_clock64(); \
    }                                                                                       \
  } while (0)

// MAP = 1: the shared map staged in LDS; MAP = 2: maps read from global memory
// (they do not change during a launch, so plain loads are fine).
// G.own_shift = kPersistOwnShift, G.n_blocks = 256 = the number of workgroups (blocks
// without envs hand over empty cells).
// Everything in B holds tag 0 at launch (cleared by the host), *B.err is zero.
// FOLD = the rules of the common configuration are compile-time facts (goal test on the
// target cell, restart at the end of an episode, true maximum, rewards by class, no trace,
// no supplied stream, no episode budget, no return statistics): the general kernel keeps
// a dozen lane masks and pointers for them that do not fit the scalar registers and are
// fetched back again and again (190 lane reads per step).
template <int A, int MAP, bool CLK, bool FOLD>
__global__ __launch_bounds__(256) void k_shared_persist(const Rules R, const Ptrs P, const uint64_t t0,
                                                         const int n_steps, const int trace_row0,
                                                         const ReduceGeom G, const PersistBufs B,
                                                         const int spin_limit) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  PersistLds& L = *reinterpret_cast<PersistLds*>(lds_raw);
  static_assert(sizeof(PersistLds) % 16 == 0 && offsetof(PersistLds, tile) % 16 == 0, "16-byte LDS accesses");
  static_assert(kSortBytes <= sizeof(L.tile) / 2, "the holders' line-up borrows the upper half of the tile");
  uint32_t* lds_map = reinterpret_cast<uint32_t*>(lds_raw + sizeof(PersistLds));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wg = blockIdx.x;
  const int env = wg * 256 + tid;
  const bool has_env = env < P.N;
  const int n_own = 1 << G.own_shift;  // = workgroups: every one of them is a block and an owner

  // a launch of this engine gave up earlier and nobody has set state and table again:
  // nothing to do (the word is read once, so that all threads take the same way)
  if (tid == 0) L.o_count = (int)ld_dev32(B.err);
  __syncthreads();
  if (L.o_count != 0) return;
  __syncthreads();
  reduce_block_init(L.red);
  if (tid == 0) {
    L.o_count = 0;
    L.dead = 0;
  }
  if (MAP == 1)
    for (int i = tid; i < P.map_words; i += 256) lds_map[i] = P.map[i];
  // env state lives in registers for the whole launch
  int s = has_env ? P.s[env] : 0;
  int ep_step = has_env ? P.ep_step[env] : 0;
  int episode = has_env ? P.episode[env] : 0;
  bool done = has_env ? P.done[env] != 0 : false;
  float reward = has_env ? P.reward[env] : 0.0f;
  int action = has_env ? P.action[env] : 0;
  const int start = has_env ? P.start[env] : 0;
  const bool track = !FOLD && P.ret_acc != nullptr;
  float ret = (track && has_env) ? P.ret_acc[env] : 0.0f;
  const uint32_t* gmap = P.map + ((P.map_shared || !has_env) ? 0 : (size_t)env * P.map_words);
  const float* cr = P.cell_reward ? P.cell_reward + ((P.map_shared || !has_env) ? 0 : (size_t)env * P.S) : nullptr;
  const DevWindow w_table = dev_window(B.table), w_cells = dev_window(B.cells);
  // 64-bit words of one buffer of main halves; cells with an extension: as many again, behind both buffers
  const size_t cells_half = ((size_t)n_own * G.n_blocks) << G.main_shift;
  const bool cells_flag = !FOLD && (R.reward_flags & 1) != 0;
  const bool base_cells = cells_flag && (R.reward_flags & 2) != 0;

  // owner: lane l of wave 0 keeps the table value of its key in a register; the A lanes
  // of a row sit side by side, each of them publishes its value and one copy of the row's
  // maximum
  const int own_key = key_of(wg, lane, G);
  const bool own_live = wave == 0 && own_key < G.K;
  float q_own = own_live ? P.Q[own_key] : 0.0f;
  // where the lane of action a publishes: its value in the view of its cell, and the row's
  // maximum in the view of the cell that reaches this one by action a (and in its own
  // cell's view if action a would leave the grid there)
  int pub_q = -1, pub_from = -1, pub_self = -1;
  if (own_live) {
    const int c = own_key >> G.a_shift, a = own_key & (A - 1);
    const int x = c % R.W, y = c / R.W;
    int dx, dy;
    action_delta(a, A, dx, dy);
    pub_q = c * 2 * A + a;
    if ((unsigned)(x - dx) < (unsigned)R.W && (unsigned)(y - dy) < (unsigned)R.H) pub_from = (c - dy * R.W - dx) * 2 * A + A + a;
    if (!((unsigned)(x + dx) < (unsigned)R.W && (unsigned)(y + dy) < (unsigned)R.H)) pub_self = c * 2 * A + A + a;
  }
  auto publish = [&](uint32_t tag) {  // wave 0 of an owner
    if (own_live) st_dev64(B.table + pub_q, tagged(__float_as_uint(q_own), tag));
    float qs[A];
    if constexpr (A == 4) {  // the four lanes of a row are a quad: a move within it, no trip through LDS
      qs[0] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(q_own), 0x00, 0xf, 0xf, true));
      qs[1] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(q_own), 0x55, 0xf, 0xf, true));
      qs[2] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(q_own), 0xaa, 0xf, 0xf, true));
      qs[3] = __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(q_own), 0xff, 0xf, 0xf, true));
    } else {
#pragma unroll
      for (int i = 0; i < A; ++i) qs[i] = __shfl(q_own, (lane & ~(A - 1)) + i);
    }
    if (own_live) {
      Row<A> row;
      if constexpr (A == 4) row = Row<4>{qs[0], qs[1], qs[2], qs[3]};
      else row = Row<8>{qs[0], qs[1], qs[2], qs[3], qs[4], qs[5], qs[6], qs[7]};
      const unsigned long long mx = tagged(__float_as_uint(row_max(row, false, 0)), tag);
      if (pub_from >= 0) st_dev64(B.table + pub_from, mx);
      if (pub_self >= 0) st_dev64(B.table + pub_self, mx);
    }
  };
  if (wave == 0) publish(1u);
  __syncthreads();

  // What a step needs that does not depend on the table: computed at the top of the step,
  // while the values of the step before are on their way from the owners.
  bool live = false;
  int s0 = 0, cls0 = kFree;
  int nb[A];
  uint32_t mv = 0;
  Draw d{0.0f, 0};
  float eps = 0.0f;
  auto prepare = [&](int k) {
    const uint64_t t = t0 + (uint64_t)k;
    live = has_env && (FOLD || !(R.max_episodes > 0 && episode >= R.max_episodes));
    if (!FOLD && has_env && !live) trace_idle(P, env, trace_row0 + k, s);
    s0 = s;
    const int x0 = s0 % R.W, y0 = s0 / R.W;
    if (live) {
#pragma unroll
      for (int i = 0; i < A; ++i) {
        int dx, dy;
        action_delta(i, A, dx, dy);
        const bool in = (unsigned)(x0 + dx) < (unsigned)R.W && (unsigned)(y0 + dy) < (unsigned)R.H;
        nb[i] = in ? s0 + dy * R.W + dx : s0;
      }
      auto word_of = [&](int w) -> uint32_t { return (MAP == 1) ? lds_map[w] : gmap[w]; };
      mv = moves_of_cell<A>(word_of, R.W, R.H, x0, y0, s0);
      cls0 = cell_class_of(word_of(s0 >> 4), s0);
      d = pick_draw(explore_block(R.seed, (uint32_t)env, t >> 1), t, A);
      if (!FOLD && P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
        const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
        d.u = P.u_sup[o];
        d.a = P.a_sup[o];
      }
      eps = eps_of(R, P.eps_tab, t, episode);
    } else {
#pragma unroll
      for (int i = 0; i < A; ++i) nb[i] = 0;
    }
  };

  unsigned long long phase_[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  unsigned long long last_ = CLK ? clock64() : 0ull;
  bool gave_up = false;
  for (int k = 0; k < n_steps; ++k) {
    const uint32_t want = (uint32_t)k + 1u;
    CRL_MARK(7);
    // (the values this workgroup published as an owner are on their way meanwhile)
    prepare(k);
    reduce_stage_init(L.stage, G, want);
    // (The values published at the end of the last step need about 1 us to be visible, which
    // is what the preparation above takes.  A look that comes too early costs a whole round
    // trip more; while a step was longer than now, a pause of 0.1-0.2 us here and before the
    // first look at the cells was worth 0.1-0.4 us per step, and now it no longer is.)
    CRL_MARK(0);

    // ---- the table of this step: the view of the env's cell ----------------------------
    unsigned long long rq[A], rn[A];
    {
      const uint32_t view = (uint32_t)s0 * (uint32_t)(2 * A * 8);  // byte offset of the cell's view
      bool ok = false;
      int spins = 0;
      while (!ok) {
        poll_fence();
        if (live) {
          // two units to a 16-byte load: the row, then the neighbours' maxima
#pragma unroll
          for (int i = 0; i < A; i += 2) {
            const uint4 r = ld_dev128(w_table, view + (uint32_t)i * 8u);
            rq[i] = tagged(r.x, r.y);
            rq[i + 1] = tagged(r.z, r.w);
          }
#pragma unroll
          for (int i = 0; i < A; i += 2) {
            const uint4 r = ld_dev128(w_table, view + (uint32_t)(A + i) * 8u);
            rn[i] = tagged(r.x, r.y);
            rn[i + 1] = tagged(r.z, r.w);
          }
        }
        ok = true;
        if (live) {
#pragma unroll
          for (int i = 0; i < A; ++i) ok = ok && tag_of(rq[i]) == want && tag_of(rn[i]) == want;
        }
        if (!ok && (++spins >= spin_limit || ((spins & 63) == 0 && ld_dev32(B.err) != 0u))) {
          L.dead = 1;
          break;
        }
      }
      if (CLK) phase_[8] += (unsigned long long)spins + 1ull;
      // (no barrier here: the block sums begin with one, behind which every thread of the
      // workgroup has read its view - cells are written later still - and whether some
      // thread gave up is looked at behind them; until then it works on whatever it got)
    }
    CRL_MARK(1);

    // ---- select, move, (key, delta) ---------------------------------------------------
    int my_key = 0;
    float my_delta = 0.0f;
    if (live) {
      const Row<A> row = row_of_tagged<A>(rq);
      const int greedy = row_argmax(row);  // (worked out for every env: cheaper than a branch around it)
      const int a = (d.u < eps) ? d.a : greedy;
      // (the key is known: its leader is being found while the delta is worked out)
      my_key = s0 * A + a;
      atomicMin(&L.red.lead[my_key], (uint32_t)tid);
      // the rule of step_rule() on the move code of the action: the class of the target
      // cell, or kWall outside the grid
      const int code = (int)((mv >> (2 * a)) & 3u);
      int tgt = nb[0];
      float m_tgt = value_of(rn[0]);
#pragma unroll
      for (int i = 1; i < A; ++i) {
        tgt = (a == i) ? nb[i] : tgt;
        m_tgt = (a == i) ? value_of(rn[i]) : m_tgt;
      }
      const bool moved = code < kTrap;
      const bool trap = code == kTrap;
      const int s2 = moved ? tgt : s0;
      const bool hit = (FOLD || R.goal_mode == 0) ? code == kGoal : ((moved ? code : cls0) == kGoal);
      const float by_class = hit ? R.goal_reward : trap ? R.trap_reward : R.step_reward;
      float by_cell = 0.0f;
      if (cells_flag) by_cell = cr[(trap && !hit) ? tgt : s2];
      reward = (cells_flag && (hit || trap || base_cells)) ? by_cell : by_class;
      done = hit || (!FOLD && !R.auto_reset && done);
      float m = (s2 != s0) ? m_tgt : row_max(row, false, 0);
      if (!FOLD && R.max_mode == 1) m = fmaxf(0.0f, m);
      m = done ? 0.0f : m;
      my_delta = td_delta(row_get(row, a), reward, m, R.lr, R.gamma);
      action = a;
      if (!FOLD && env < P.trace_n && trace_row0 + k < P.trace_cap) {
        const size_t o = (size_t)(trace_row0 + k) * P.trace_n + env;
        P.tr_s[o] = s2;
        P.tr_a[o] = (uint8_t)a;
        P.tr_r[o] = reward;
        P.tr_d[o] = done ? 1 : 0;
      }
      ep_step += 1;
      ret = ret + reward;
      const bool over_now = (FOLD || R.auto_reset) && (done || (R.episode_len > 0 && ep_step >= R.episode_len));
      if (!FOLD && track && over_now) record_episode(P, env, ret, ep_step);
      ret = over_now ? 0.0f : ret;
      s = over_now ? start : s2;
      ep_step = over_now ? 0 : ep_step;
      episode += over_now ? 1 : 0;
    }
    CRL_MARK(2);

    // ---- block sums to the owners' cells ------------------------------------------------
    const int half = k & 1;  // cells and raw samples: two buffers, taken in turn
    // (`sorted`: the upper half of the tile, which is free until the block sums are through)
    const bool over = reduce_block<true>(L.red, G, wg, my_key, my_delta, live, B.cells, want, L.tile + kTileBlocks * kOwnKeys / 2,
                                         L.stage, &w_cells,
                                         (uint32_t)((size_t)half * cells_half * 8), B.cells + (2 + half) * cells_half, true);
    if (over && has_env)
      st_dev64(B.raw + (size_t)half * P.N + env, tagged(__float_as_uint(my_delta),
                                   (uint32_t)my_key | (live ? kRawValid : 0u) | (want << kRawTagShift)));
    CRL_MARK(3);

    // ---- while the cells travel: the owner's tile cleared -------------------------------
    {  // (each wave its own quarter)
      float4* tile4 = reinterpret_cast<float4*>(L.tile) + wave * (kTileBlocks * kOwnKeys / 4 / 4);
#pragma unroll
      for (int i = 0; i < kTileBlocks * kOwnKeys / 4 / 256; ++i) tile4[i * 64 + lane] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
    // (no waiting for the own cells' acknowledgement before the first look at the others':
    // that costs 0.3 us per step; clearing the tile first is pause enough)
    if (L.dead) {  // some thread gave up waiting for the table
      gave_up = true;
      break;
    }
    CRL_MARK(4);

    // ---- as owner of 64 keys: all blocks' cells, added in tree order --------------------
    {
      // A wave takes 64 blocks' cells.  A main half is two pieces of 16 bytes = two records
      // each: two lanes read it side by side, so a load of the wave is 32 whole halves, and
      // the same two lanes read the cell's extension; all four loads are asked for at once.
      {
        const int pair = lane & 1;  // this lane's piece of its cells
        constexpr int GS = 2;       // loads of either kind per lane
        int spins = 0;
        bool stop = false;
        uint4 rec[GS], more[GS];
        int cnt[GS];
        uint32_t src[GS], src_more[GS];  // byte offsets into the cells
#pragma unroll
        for (int j = 0; j < GS; ++j) {
          const int blk = wave * 64 + j * 32 + (lane >> 1);
          src[j] = (uint32_t)(((size_t)half * cells_half + ((size_t)(blk * n_own + wg) << kMainShift) + 2 * pair) * 8);
          src_more[j] = (uint32_t)(((size_t)(2 + half) * cells_half + ((size_t)(wg * n_own + blk) << kMainShift) + 2 * pair) * 8);
        }
        for (;;) {
          poll_fence();
#pragma unroll
          for (int j = 0; j < GS; ++j) rec[j] = ld_dev128(w_cells, src[j]);
#pragma unroll
          for (int j = 0; j < GS; ++j) more[j] = ld_dev128(w_cells, src_more[j]);
          bool ok = true;
#pragma unroll
          for (int j = 0; j < GS; ++j) {
            // (record 0 of the cell is in the even lane of the two: a move within the quad)
            const uint32_t meta0 = (uint32_t)__builtin_amdgcn_mov_dpp((int)rec[j].x, 0xa0, 0xf, 0xf, true);
            cnt[j] = rec_count(meta0);
            // (every record of a main half is written every step)
            bool mine = rec_tag(meta0) == want && rec_tag(rec[j].x) == want && rec_tag(rec[j].z) == want;
            if (cnt[j] != kSlotOverflow) {  // (an extension record: only where the count says so)
              mine = mine && (kMainRecs + 2 * pair >= cnt[j] || rec_tag(more[j].x) == want) &&
                     (kMainRecs + 2 * pair + 1 >= cnt[j] || rec_tag(more[j].z) == want);
            }
            ok = ok && mine;
          }
          if (__all(ok)) break;
          if (++spins >= spin_limit || ((spins & 63) == 0 && ld_dev32(B.err) != 0u)) {
            L.dead = 1;
            stop = true;
            break;
          }
        }
        if (CLK) phase_[9] += (unsigned long long)spins + 1ull;
        if (!stop) {
#pragma unroll
          for (int j = 0; j < GS; ++j) {
            const int blk = wave * 64 + j * 32 + (lane >> 1);
            float* row = L.tile + blk * kOwnKeys;
            const bool too_many = cnt[j] == kSlotOverflow;
            if (__any(too_many)) {  // (rare)
              if (too_many && pair == 0) L.o_list[atomicAdd(&L.o_count, 1)] = (uint8_t)blk;
            }
            // (no branches: a record that is not there goes to a word of this thread's that
            // nobody reads)
            const int n = too_many ? 0 : cnt[j];
            float* none = &L.o_delta[tid];
            *(2 * pair < n ? &row[rec_slot(rec[j].x)] : none) = __uint_as_float(rec[j].y);
            *(2 * pair + 1 < n ? &row[rec_slot(rec[j].z)] : none) = __uint_as_float(rec[j].w);
            *(kMainRecs + 2 * pair < n ? &row[rec_slot(more[j].x)] : none) = __uint_as_float(more[j].y);
            *(kMainRecs + 2 * pair + 1 < n ? &row[rec_slot(more[j].z)] : none) = __uint_as_float(more[j].w);
          }
        }
      }
      CRL_MARK(5);
      // the wave's four groups: its own 64 rows of the tile, which only it has written
      auto group_sums = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // a lane takes four keys of one of the wave's four groups: 16 loads of 16 bytes
        const int grp = wave * 4 + (lane >> 4);
        const float4* rows = reinterpret_cast<const float4*>(L.tile + grp * kGroupBlocks * kOwnKeys) + (lane & 15);
        float4 v[kGroupBlocks];
#pragma unroll
        for (int bb = 0; bb < kGroupBlocks; ++bb) v[bb] = rows[bb * (kOwnKeys / 4)];
        float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
#pragma unroll
        for (int bb = 0; bb < kGroupBlocks; ++bb) {
          acc.x = acc.x + v[bb].x;
          acc.y = acc.y + v[bb].y;
          acc.z = acc.z + v[bb].z;
          acc.w = acc.w + v[bb].w;
        }
        reinterpret_cast<float4*>(L.gsum + grp * kOwnKeys)[lane & 15] = acc;
      };
      group_sums();
      __syncthreads();
      // (the totals are asked for along with the two words that say whether they stand)
      auto totals = [&]() {
        float total = 0.0f;
#pragma unroll
        for (int grp = 0; grp < kTileBlocks / kGroupBlocks; ++grp) total = total + L.gsum[grp * kOwnKeys + lane];
        return total;
      };
      float total = totals();
      if (L.dead) {  // some wave gave up waiting for its cells
        gave_up = true;
        break;
      }
      // blocks with more distinct keys for this owner than a cell holds (rare): their raw
      // samples, all threads at once, then one thread per key adds its matches in order,
      // and the group sums once more
      const int n_over = L.o_count;
      if (n_over > 0) {
        bool raw_failed = false;
        for (int q = 0; q < n_over; ++q) {
          const int bb = L.o_list[q];
          const int i = bb * kBlockSamples + tid;
          int slot = 255;
          float dv = 0.0f;
          if (i < P.N) {
            unsigned long long v = 0ull;
            int spins = 0;
            for (;;) {
              poll_fence();
              v = ld_dev64(B.raw + (size_t)half * P.N + i);
              if ((tag_of(v) >> kRawTagShift) == want) break;
              if (++spins >= spin_limit || ((spins & 63) == 0 && ld_dev32(B.err) != 0u)) {
                raw_failed = true;
                break;
              }
            }
            const int kk = (int)(tag_of(v) & kRawKeyMask);
            if (!raw_failed && (tag_of(v) & kRawValid) && owner_of(kk, G) == wg) {
              slot = slot_of(kk, G);
              dv = value_of(v);
            }
          }
          L.o_slot[tid] = (uint8_t)slot;
          L.o_delta[tid] = dv;
          __syncthreads();
          if (tid < kOwnKeys) {
            float acc = 0.0f;
            for (int j = 0; j < kBlockSamples; ++j)
              if (L.o_slot[j] == tid) acc = acc + L.o_delta[j];  // sample order
            L.tile[bb * kOwnKeys + tid] = acc;
          }
          __syncthreads();
        }
        if (tid == 0) L.o_count = 0;
        if (raw_failed) L.dead = 1;
        __syncthreads();
        if (L.dead) {
          gave_up = true;
          break;
        }
        group_sums();
        __syncthreads();
        total = totals();
      }
      if (wave == 0) {
        q_own = q_own + total;
        publish(want + 1u);
      }
      CRL_MARK(6);
    }
  }
#undef CRL_MARK
  if (gave_up && tid == 0) st_dev32(B.err, 1u);
  if (CLK && B.clocks && tid == 0 && (wg == 0 || wg == (int)gridDim.x - 1))
    for (int i = 0; i < 10; ++i) B.clocks[(wg ? 10 : 0) + i] = phase_[i];

  if (own_live) P.Q[own_key] = q_own;
  if (has_env) {
    P.s[env] = s;
    P.ep_step[env] = ep_step;
    P.episode[env] = episode;
    if (track) P.ret_acc[env] = ret;
    P.reward[env] = reward;
    P.done[env] = done ? 1 : 0;
    P.action[env] = (uint8_t)action;
  }
}

// ---------------------------------------------------------------------------
// Diagnostics: what a barrier over all resident workgroups costs when it is
// built from device-scope loads and stores, in three layouts.  `mem` is zeroed
// before the launch; out[0] receives the 100 MHz clock ticks of `rounds` barriers,
// out[1] the number of workgroups that gave up waiting.
//   0  one packed flag word per workgroup, every workgroup polls all of them with one
//      16-byte load per lane
//   1  one flag per 128-byte line, polled one load at a time
//   2  a tree in which every word has one writer and one reader: 16 members -> their
//      leader -> the root, which releases all workgroups through one word each
// ---------------------------------------------------------------------------
constexpr int kProbeLine = 32;  // words per 128-byte line
template <int PATTERN>
__global__ __launch_bounds__(256) void k_probe_barrier(unsigned* mem, const int rounds, unsigned long long* out) {
  const int n = (int)gridDim.x, w = (int)blockIdx.x, tid = (int)threadIdx.x;
  constexpr int kLimit = kPersistSpinLimit / 8;
  bool dead = false;  // the same in every thread of the workgroup
  // -> false when the limit was hit
  auto wait_word = [&](const unsigned* p, unsigned want) -> bool {
    int spins = 0;
    while ((int)(ld_dev32(p) - want) < 0)
      if (++spins >= kLimit) return false;
    return true;
  };
  const unsigned long long t0 = wall_clock64();
  for (int r = 1; r <= rounds && !dead; ++r) {
    bool ok = true;
    if (PATTERN == 0) {
      if (tid == 0) st_dev32(mem + w, (unsigned)r);
      if (tid < 64)
        for (int i = tid * 4; i < min(n, tid * 4 + 4); ++i) ok = ok && wait_word(mem + i, (unsigned)r);
    } else if (PATTERN == 1) {
      if (tid == 0) st_dev32(mem + (size_t)w * kProbeLine, (unsigned)r);
      if (tid < 64)
        for (int i = tid; i < n; i += 64) ok = ok && wait_word(mem + (size_t)i * kProbeLine, (unsigned)r);
    } else {
      unsigned* arrive = mem;                        // [16 groups][line]: word m of group g
      unsigned* garrive = mem + 16 * kProbeLine;     // word g
      unsigned* go = mem + 17 * kProbeLine;          // [workgroup][line]
      const int g = w >> 4, m = w & 15;
      const int members = min(16, n - g * 16), groups = (n + 15) >> 4;
      if (tid == 0) st_dev32(arrive + g * kProbeLine + m, (unsigned)r);
      if (m == 0) {
        if (tid < members) ok = wait_word(arrive + g * kProbeLine + tid, (unsigned)r);
        ok = __syncthreads_or(!ok) == 0;
        if (tid == 0) st_dev32(garrive + g, (unsigned)r);
        if (w == 0) {
          if (tid < groups) ok = ok && wait_word(garrive + tid, (unsigned)r);
          ok = __syncthreads_or(!ok) == 0;
          if (tid < n) st_dev32(go + (size_t)tid * kProbeLine, (unsigned)r);
        }
      }
      if (tid == 0) ok = ok && wait_word(go + (size_t)w * kProbeLine, (unsigned)r);
    }
    dead = __syncthreads_or(!ok) != 0;  // every thread leaves the loop in the same round
  }
  if (tid == 0 && dead) atomicAdd(out + 1, 1ull);
  if (tid == 0 && w == 0) out[0] = wall_clock64() - t0;
}

}  // namespace crl
