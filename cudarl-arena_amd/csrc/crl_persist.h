// Shared table, all steps of a launch in ONE kernel: every workgroup is a block of
// the ordered reduction (256 envs, state in registers for the whole launch) and
// the owner of 64 keys, and the two roles hand their data to each other through
// memory that is read and written past the caches' incoherent levels.
//
// gfx950 has eight XCDs, each with its own L2; plain loads and stores are
// coherent inside one XCD only, and the release / acquire fences that make them
// coherent across the chip write back and invalidate a whole L2.  Loads and stores
// carrying the `sc1` bit (device scope) are served past the L2: a value stored
// that way by one workgroup is seen by the next sc1 load of any other (measured:
// about 170 ns per dependent sc1 access, also between XCDs).  So everything the
// workgroups exchange - the table, the hand-off cells, the (key, delta) arrays
// and the step flags - is only ever touched with sc1 accesses inside this kernel,
// and an exchange is: sc1 stores, wait until they are acknowledged, sc1 store of
// the workgroup's flag; the reader polls the flags, then sc1-loads the data.
//
// One step:
//   1. wait until every owner has published the table of this step   (owner flags)
//   2. act: select, move, (key, delta) from the table as published
//   3. fold the block's deltas in order, hand the block sums to the owners'
//      cells, publish                                                 (block flag)
//   4. as owner: wait for every block's cells, add them in tree order, store
//      the 64 new table values, publish                               (owner flag)
// A workgroup writes its cells of step k+1 only after step 1 of k+1, when every
// owner has consumed the cells of step k, and an owner overwrites its table values
// only after step 4's wait, when every block has read them: one buffer of each.
//
// Every wait is bounded: a workgroup that waits for `spin_limit` polls (default
// kPersistSpinLimit) sets the error word and leaves; the others then leave, too.
#pragma once
#include "crl_kernels.h"

namespace crl {

constexpr int kPersistSpinLimit = 1 << 20;  // polls of about a quarter microsecond each
constexpr int kPersistMaxGroups = 256;      // workgroups: one per compute unit, all resident
constexpr size_t kPersistReduceLds =
    sizeof(ReduceLds) > (size_t)(kTileBlocks + kTileBlocks / kGroupBlocks) * kOwnKeys * sizeof(float)
        ? sizeof(ReduceLds)
        : (size_t)(kTileBlocks + kTileBlocks / kGroupBlocks) * kOwnKeys * sizeof(float);

// ---- device-scope (sc1) accesses -----------------------------------------------
// Stores are fire-and-forget until drain_stores().  Loads come in groups that are
// issued together and waited for inside ONE asm statement, with early-clobber
// outputs: the compiler does not know that a load writes its destination later
// and would otherwise reuse those registers while the load is in flight.

__device__ __forceinline__ void st_dev(unsigned* p, unsigned v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st_dev(int32_t* p, int32_t v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st_dev(float* p, float v) {
  asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void st_dev(uint2* p, uint2 v) {
  asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
}
__device__ __forceinline__ void drain_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ unsigned ld_dev(const unsigned* p) {
  unsigned v;
  asm volatile("global_load_dword %0, %1, off sc1\n s_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ uint4 ld_dev4(const uint4* p) {
  uint4 v;
  asm volatile("global_load_dwordx4 %0, %1, off sc1\n s_waitcnt vmcnt(0)" : "=&v"(v) : "v"(p) : "memory");
  return v;
}
__device__ __forceinline__ void ld_dev4x2(const uint4* p0, const uint4* p1, uint4& v0, uint4& v1) {
  asm volatile(
      "global_load_dwordx4 %0, %2, off sc1\n global_load_dwordx4 %1, %3, off sc1\n s_waitcnt vmcnt(0)"
      : "=&v"(v0), "=&v"(v1)
      : "v"(p0), "v"(p1)
      : "memory");
}
__device__ __forceinline__ void ld_dev4x4(const uint4* p0, const uint4* p1, const uint4* p2, const uint4* p3,
                                          uint4& v0, uint4& v1, uint4& v2, uint4& v3) {
  asm volatile(
      "global_load_dwordx4 %0, %4, off sc1\n global_load_dwordx4 %1, %5, off sc1\n"
      "global_load_dwordx4 %2, %6, off sc1\n global_load_dwordx4 %3, %7, off sc1\n s_waitcnt vmcnt(0)"
      : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3)
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3)
      : "memory");
}
__device__ __forceinline__ void ld_dev4x5(const uint4* p0, const uint4* p1, const uint4* p2, const uint4* p3,
                                          const uint4* p4, uint4& v0, uint4& v1, uint4& v2, uint4& v3,
                                          uint4& v4) {
  asm volatile(
      "global_load_dwordx4 %0, %5, off sc1\n global_load_dwordx4 %1, %6, off sc1\n"
      "global_load_dwordx4 %2, %7, off sc1\n global_load_dwordx4 %3, %8, off sc1\n"
      "global_load_dwordx4 %4, %9, off sc1\n s_waitcnt vmcnt(0)"
      : "=&v"(v0), "=&v"(v1), "=&v"(v2), "=&v"(v3), "=&v"(v4)
      : "v"(p0), "v"(p1), "v"(p2), "v"(p3), "v"(p4)
      : "memory");
}

__device__ __forceinline__ float max4(const uint4 r) {
  return fmaxf(fmaxf(__uint_as_float(r.x), __uint_as_float(r.y)), fmaxf(__uint_as_float(r.z), __uint_as_float(r.w)));
}

// row of cell `cell` of the shared table and the row maxima of the cells the A
// actions lead to (`nb[i]`: neighbour cell, or the cell itself at the grid's edge)
template <int A>
__device__ __forceinline__ void load_rows_dev(const float* Q, int cell, const int (&nb)[A], Row<A>& row,
                                              float (&nb_max)[A]);
template <>
__device__ __forceinline__ void load_rows_dev<4>(const float* Q, int cell, const int (&nb)[4], Row<4>& row,
                                                 float (&nb_max)[4]) {
  const uint4* T = reinterpret_cast<const uint4*>(Q);
  uint4 r, n0, n1, n2, n3;
  ld_dev4x5(T + cell, T + nb[0], T + nb[1], T + nb[2], T + nb[3], r, n0, n1, n2, n3);
  row = Row<4>{__uint_as_float(r.x), __uint_as_float(r.y), __uint_as_float(r.z), __uint_as_float(r.w)};
  nb_max[0] = max4(n0);
  nb_max[1] = max4(n1);
  nb_max[2] = max4(n2);
  nb_max[3] = max4(n3);
}
template <>
__device__ __forceinline__ void load_rows_dev<8>(const float* Q, int cell, const int (&nb)[8], Row<8>& row,
                                                 float (&nb_max)[8]) {
  const uint4* T = reinterpret_cast<const uint4*>(Q);  // a row is two 16-byte halves
  uint4 a, b, c, d;
  ld_dev4x2(T + 2 * cell, T + 2 * cell + 1, a, b);
  row = Row<8>{__uint_as_float(a.x), __uint_as_float(a.y), __uint_as_float(a.z), __uint_as_float(a.w),
               __uint_as_float(b.x), __uint_as_float(b.y), __uint_as_float(b.z), __uint_as_float(b.w)};
#pragma unroll
  for (int i = 0; i < 8; i += 2) {
    ld_dev4x4(T + 2 * nb[i], T + 2 * nb[i] + 1, T + 2 * nb[i + 1], T + 2 * nb[i + 1] + 1, a, b, c, d);
    nb_max[i] = fmaxf(max4(a), max4(b));
    nb_max[i + 1] = fmaxf(max4(c), max4(d));
  }
}

// Wave 0 polls the first `n` flags until all have reached `want` (or the limit is
// hit, or another workgroup has given up); every thread returns the same answer.
__device__ __forceinline__ bool wait_flags(const unsigned* flags, int n, unsigned want, unsigned* err,
                                           int* lds_dead, const int spin_limit) {
  if (threadIdx.x < 64) {
    const int i0 = (int)threadIdx.x * 4;
    bool ok = true;
    if (i0 < n) {
      int spins = 0;
      for (;;) {
        const uint4 v = ld_dev4(reinterpret_cast<const uint4*>(flags + i0));
        ok = (int)(v.x - want) >= 0 && (i0 + 1 >= n || (int)(v.y - want) >= 0) &&
             (i0 + 2 >= n || (int)(v.z - want) >= 0) && (i0 + 3 >= n || (int)(v.w - want) >= 0);
        if (ok) break;
        if (++spins >= spin_limit || ((spins & 255) == 0 && ld_dev(err) != 0u)) break;
      }
    }
    if (!__all(ok) && threadIdx.x == 0) {
      st_dev(err, 1u);
      *lds_dead = 1;
    }
  }
  __syncthreads();
  return *lds_dead == 0;
}

// reduce_block() with the hand-off written for readers on other XCDs
__device__ __forceinline__ void reduce_block_dev(ReduceLds& L, const ReduceGeom G, const int block,
                                                 const int key, const float delta, const bool valid,
                                                 uint2* handoff) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n_own = 1 << G.own_shift;
  unsigned long long peers = __ballot(valid);
  for (int b = 0; b < G.key_bits; ++b) {
    const bool bit = (key >> b) & 1;
    const unsigned long long m = __ballot(bit);
    peers &= bit ? m : ~m;
  }
  const bool leader = valid && (peers & ((1ull << lane) - 1ull)) == 0ull;
  const int owner = owner_of(key, G.own_shift);
  bool first = false;
  int slot = 0;
  constexpr int kAhead = 8;
  unsigned long long rest = leader ? peers : 0ull;
  float ahead[kAhead];
#pragma unroll
  for (int i = 0; i < kAhead; ++i) {
    const int j = rest ? __builtin_ctzll(rest) : lane;
    const float dj = __shfl(delta, j);
    ahead[i] = rest ? dj : 0.0f;
    rest &= rest - 1ull;
  }
  __syncthreads();
  for (int w = 0; w < 4; ++w) {
    if (wave == w) {
      float acc = 0.0f;
      if (leader) {
        first = L.seen[key] == 0;
        acc = first ? 0.0f : L.run[key];
      }
#pragma unroll
      for (int i = 0; i < kAhead; ++i) acc = acc + ahead[i];  // lane order = sample order
      while (__ballot(rest != 0ull) != 0ull) {
        const int j = rest ? __builtin_ctzll(rest) : lane;
        const float dj = __shfl(delta, j);
        if (rest) acc = acc + dj;
        rest &= rest - 1ull;
      }
      if (leader) {
        L.run[key] = acc;
        L.seen[key] = 1;
        if (first) slot = atomicAdd(&L.handed[owner], 1);
      }
    }
    __syncthreads();
  }
  if (leader && first && slot < kSlotCap) {
    const size_t at = ((size_t)owner * G.n_blocks + block) * kHandoffRecs + slot;
    uint32_t tag = (uint32_t)(key >> G.own_shift);
    if (slot == 0) {
      const int c = L.handed[owner];
      tag |= (uint32_t)(c > kSlotCap ? kSlotOverflow : c) << 8;
    }
    st_dev(handoff + at, make_uint2(tag, __float_as_uint(L.run[key])));
  }
  if (tid < n_own && L.handed[tid] == 0)
    st_dev(handoff + ((size_t)tid * G.n_blocks + block) * kHandoffRecs, make_uint2(0u, 0u));
}

// Phase clocks: thread 0 of the first and the last workgroup add up the shader clocks
// between the marks of a step and leave the sums behind the give-up word (16 x 64 bit),
// for crl_get_persist_clocks.  Phases: 0 wait for the owners, 1 act, 2 block sums,
// 3 drain + publish, 4 wait for the blocks, 5 cells into the tile, 6 tile sums + publish,
// 7 loop overhead.
#define CRL_MARK(i)                                   \
  do {                                                \
    const unsigned long long now_ = clock64();        \
    phase_[i] += now_ - last_;                        \
    last_ = now_;                                     \
  } while (0)

// MAP = 1: the shared map staged in LDS; MAP = 2: maps read from global memory
// (they do not change during a launch, so plain loads are fine).
// G.n_blocks is the number of workgroups (blocks without envs hand over empty cells).
// flags: [0, kPersistMaxGroups) block flags, [kPersistMaxGroups, 2 * kPersistMaxGroups)
// owner flags, all zero at launch; err: the give-up word, zero at launch.
template <int A, int MAP>
__global__ __launch_bounds__(256) void k_shared_persist(const Rules R, const Ptrs P, const uint64_t t0,
                                                         const int n_steps, const int trace_row0,
                                                         int32_t* key, float* delta, const ReduceGeom G,
                                                         uint2* handoff, unsigned* flags, unsigned* err,
                                                         const int spin_limit) {
  extern __shared__ unsigned char lds_raw[];
  ReduceLds& L = *reinterpret_cast<ReduceLds*>(lds_raw);
  float* tile = reinterpret_cast<float*>(lds_raw);  // the owner's [block][key] tile reuses the block's table
  float* gsum = tile + kTileBlocks * kOwnKeys;
  uint32_t* lds_map = reinterpret_cast<uint32_t*>(lds_raw + kPersistReduceLds);
  __shared__ int lds_dead;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wg = blockIdx.x;
  const int env = wg * 256 + tid;
  const bool has_env = env < P.N;
  const int n_groups = (int)gridDim.x;  // every workgroup publishes a block flag
  const int n_own = 1 << G.own_shift;   // workgroups [0, n_own) are owners, too
  const bool is_owner = wg < n_own;
  unsigned* block_flags = flags;
  unsigned* owner_flags = flags + kPersistMaxGroups;

  if (tid == 0) lds_dead = 0;
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
  const bool track = P.ret_acc != nullptr;
  float ret = (track && has_env) ? P.ret_acc[env] : 0.0f;
  // owner: lane l of wave 0 keeps the table value of its key in a register
  const int own_key = key_of(wg, lane, G.own_shift);
  const bool own_live = is_owner && wave == 0 && own_key < G.K;
  float q_own = own_live ? __uint_as_float(ld_dev(reinterpret_cast<const unsigned*>(P.Q + own_key))) : 0.0f;
  const uint32_t* gmap = P.map + ((P.map_shared || !has_env) ? 0 : (size_t)env * P.map_words);
  const float* cr = P.cell_reward ? P.cell_reward + ((P.map_shared || !has_env) ? 0 : (size_t)env * P.S) : nullptr;
  __syncthreads();

  unsigned long long phase_[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  unsigned long long last_ = clock64();
  for (int k = 0; k < n_steps; ++k) {
    const uint64_t t = t0 + (uint64_t)k;
    CRL_MARK(7);
    // 1. the table of this step: every owner has published its values of step k
    if (k > 0 && !wait_flags(owner_flags, n_own, (unsigned)k, err, &lds_dead, spin_limit)) break;
    CRL_MARK(0);
    reduce_block_clear(L, G);

    // 2. act
    const bool live = has_env && !(R.max_episodes > 0 && episode >= R.max_episodes);
    int my_key = 0;
    float my_delta = 0.0f;
    if (has_env && !live) trace_idle(P, env, trace_row0 + k, s);
    if (live) {
      auto cls = [&](int cell) -> int {
        const uint32_t word = (MAP == 1) ? lds_map[cell >> 4] : gmap[cell >> 4];
        return cell_class_of(word, cell);
      };
      const int s0 = s;
      int x = s0 % R.W, y = s0 / R.W;
      int nb[A];
#pragma unroll
      for (int i = 0; i < A; ++i) {
        int dx, dy;
        action_delta(i, A, dx, dy);
        const bool in = (unsigned)(x + dx) < (unsigned)R.W && (unsigned)(y + dy) < (unsigned)R.H;
        nb[i] = in ? s0 + dy * R.W + dx : s0;
      }
      Row<A> row;
      float nb_max[A];
      load_rows_dev<A>(P.Q, s0, nb, row, nb_max);
      Draw d = pick_draw(explore_block(R.seed, (uint32_t)env, t >> 1), t, A);
      if (P.u_sup && t >= P.sup_t0 && t - P.sup_t0 < (uint64_t)P.sup_n) {
        const size_t o = (size_t)(t - P.sup_t0) * P.N + env;
        d.u = P.u_sup[o];
        d.a = P.a_sup[o];
      }
      const float eps = eps_of(R, P.eps_tab, t, episode);
      const int a = (d.u < eps) ? d.a : row_argmax(row);
      bool hit;
      step_rule(R, ClassRewards{R.step_reward, R.goal_reward, R.trap_reward}, cls, cr, x, y, a, reward, hit);
      const int s2 = y * R.W + x;
      done = hit || (!R.auto_reset && done);
      float m = row_max(row, false, 0);  // the env stayed where it was
#pragma unroll
      for (int i = 0; i < A; ++i) m = (s2 != s0 && a == i) ? nb_max[i] : m;
      if (R.max_mode == 1) m = fmaxf(0.0f, m);
      m = done ? 0.0f : m;
      my_key = s0 * A + a;
      my_delta = td_delta(row_get(row, a), reward, m, R.lr, R.gamma);
      action = a;
      if (env < P.trace_n && trace_row0 + k < P.trace_cap) {
        const size_t o = (size_t)(trace_row0 + k) * P.trace_n + env;
        P.tr_s[o] = s2;
        P.tr_a[o] = (uint8_t)a;
        P.tr_r[o] = reward;
        P.tr_d[o] = done ? 1 : 0;
      }
      ep_step += 1;
      ret = ret + reward;
      if (R.auto_reset && (done || (R.episode_len > 0 && ep_step >= R.episode_len))) {
        if (track) record_episode(P, env, ret, ep_step);
        ret = 0.0f;
        s = start;
        ep_step = 0;
        episode += 1;
      } else {
        s = s2;
      }
    }
    CRL_MARK(1);
    // the raw samples, for an owner that finds more block sums than a cell holds
    if (has_env) {
      st_dev(key + env, live ? my_key : -1);
      st_dev(delta + env, my_delta);
    }

    // 3. block sums to the owners' cells
    reduce_block_dev(L, G, wg, my_key, my_delta, live, handoff);
    CRL_MARK(2);
    drain_stores();
    __syncthreads();
    if (tid == 0) st_dev(block_flags + wg, (unsigned)(k + 1));
    CRL_MARK(3);

    // 4. as owner of 64 keys: all blocks' cells, added in tree order
    if (is_owner) {
      if (!wait_flags(block_flags, n_groups, (unsigned)(k + 1), err, &lds_dead, spin_limit)) break;
      CRL_MARK(4);
      // (the wait's barrier also ends every thread's use of the block's LDS table)
      const int b = tid;
      uint4 c0 = make_uint4(0, 0, 0, 0), c1 = c0, c2 = c0, c3 = c0;
      if (b < G.n_blocks) {
        const uint4* src = reinterpret_cast<const uint4*>(handoff + ((size_t)wg * G.n_blocks + b) * kHandoffRecs);
        ld_dev4x4(src, src + 1, src + 2, src + 3, c0, c1, c2, c3);
      }
      float4* my_row = reinterpret_cast<float4*>(tile + tid * kOwnKeys);
#pragma unroll
      for (int i = 0; i < kOwnKeys / 4; ++i) my_row[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      const int c = (int)((c0.x >> 8) & 0xFFu);
      float* row = tile + tid * kOwnKeys;
      if (c != kSlotOverflow) {
        const uint4 cell[4] = {c0, c1, c2, c3};
#pragma unroll
        for (int i = 0; i < kHandoffRecs / 2; ++i) {
          if (c > 2 * i) row[cell[i].x & 0xFFu] = __uint_as_float(cell[i].y);
          if (c > 2 * i + 1) row[cell[i].z & 0xFFu] = __uint_as_float(cell[i].w);
        }
      } else {
        // more distinct keys than slots: redo the block's part from its samples, in order
        const int lo = b * kBlockSamples, hi = min(P.N, lo + kBlockSamples);
        for (int i = lo; i < hi; ++i) {
          const int kk = (int)ld_dev(reinterpret_cast<const unsigned*>(key + i));
          if (kk >= 0 && owner_of(kk, G.own_shift) == wg) {
            float& acc = row[kk >> G.own_shift];
            acc = acc + __uint_as_float(ld_dev(reinterpret_cast<const unsigned*>(delta + i)));
          }
        }
      }
      __syncthreads();
      CRL_MARK(5);
#pragma unroll
      for (int gi = 0; gi < 4; ++gi) {
        const int grp = wave * 4 + gi;
        float acc = 0.0f;
#pragma unroll
        for (int bb = 0; bb < kGroupBlocks; ++bb) acc = acc + tile[(grp * kGroupBlocks + bb) * kOwnKeys + lane];
        gsum[grp * kOwnKeys + lane] = acc;
      }
      __syncthreads();
      if (wave == 0) {
        float total = 0.0f;
#pragma unroll
        for (int grp = 0; grp < kTileBlocks / kGroupBlocks; ++grp) total = total + gsum[grp * kOwnKeys + lane];
        if (own_live) {
          q_own = q_own + total;
          st_dev(P.Q + own_key, q_own);
        }
        drain_stores();
        if (lane == 0) st_dev(owner_flags + wg, (unsigned)(k + 1));
      }
      __syncthreads();  // the tile is free again before the next step clears the block's table
      CRL_MARK(6);
    }
  }
  if (tid == 0 && (wg == 0 || wg == n_groups - 1))
    for (int i = 0; i < 8; ++i) reinterpret_cast<unsigned long long*>(err + 8)[(wg ? 8 : 0) + i] = phase_[i];
#undef CRL_MARK

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
// Measurement helper: what a barrier over all resident workgroups costs when it is
// built from device-scope loads and stores, in three layouts.  `mem` is zeroed
// before the launch; out[0] receives the 100 MHz clock ticks of `rounds` barriers,
// out[1] the number of workgroups that gave up waiting.
//   0  one packed flag word per workgroup, every workgroup polls all of them with one
//      16-byte load per lane (what k_shared_persist does)
//   1  one flag per 128-byte line, polled one load at a time
//   2  a tree in which every word has one writer and one reader: 16 members -> their
//      leader -> the root, which releases all workgroups through one word each
// ---------------------------------------------------------------------------
constexpr int kProbeLine = 32;  // words per 128-byte line
template <int PATTERN>
__global__ __launch_bounds__(256) void k_probe_barrier(unsigned* mem, const int rounds, unsigned long long* out) {
  const int n = (int)gridDim.x, w = (int)blockIdx.x, tid = (int)threadIdx.x;
  __shared__ int dead;
  if (tid == 0) dead = 0;
  __syncthreads();
  auto wait_word = [&](const unsigned* p, unsigned want) {
    int spins = 0;
    while ((int)(ld_dev(p) - want) < 0 && ++spins < kPersistSpinLimit / 8) {}
    if (spins >= kPersistSpinLimit / 8) dead = 1;
  };
  const unsigned long long t0 = wall_clock64();
  for (int r = 1; r <= rounds && !dead; ++r) {
    if (PATTERN == 0) {
      if (tid == 0) st_dev(mem + w, (unsigned)r);
      if (tid < 64 && tid * 4 < n) {
        int spins = 0;
        for (;;) {
          const uint4 v = ld_dev4(reinterpret_cast<const uint4*>(mem + tid * 4));
          const bool ok = (int)(v.x - r) >= 0 && (tid * 4 + 1 >= n || (int)(v.y - r) >= 0) &&
                          (tid * 4 + 2 >= n || (int)(v.z - r) >= 0) && (tid * 4 + 3 >= n || (int)(v.w - r) >= 0);
          if (ok) break;
          if (++spins >= kPersistSpinLimit / 8) {
            dead = 1;
            break;
          }
        }
      }
    } else if (PATTERN == 1) {
      if (tid == 0) st_dev(mem + (size_t)w * kProbeLine, (unsigned)r);
      if (tid < 64)
        for (int i = tid; i < n; i += 64) wait_word(mem + (size_t)i * kProbeLine, (unsigned)r);
    } else {
      unsigned* arrive = mem;                        // [16 groups][line]: word m of group g
      unsigned* garrive = mem + 16 * kProbeLine;     // word g
      unsigned* go = mem + 17 * kProbeLine;          // [workgroup][line]
      const int g = w >> 4, m = w & 15;
      const int members = min(16, n - g * 16), groups = (n + 15) >> 4;
      if (tid == 0) st_dev(arrive + g * kProbeLine + m, (unsigned)r);
      if (m == 0) {
        if (tid < members) wait_word(arrive + g * kProbeLine + tid, (unsigned)r);
        __syncthreads();
        if (tid == 0) st_dev(garrive + g, (unsigned)r);
        if (w == 0) {
          if (tid < groups) wait_word(garrive + tid, (unsigned)r);
          __syncthreads();
          if (tid < n) st_dev(go + (size_t)tid * kProbeLine, (unsigned)r);
        }
      }
      if (tid == 0) wait_word(go + (size_t)w * kProbeLine, (unsigned)r);
    }
    __syncthreads();
  }
  if (tid == 0 && dead) atomicAdd(out + 1, 1ull);
  if (tid == 0 && w == 0) out[0] = wall_clock64() - t0;
}

}  // namespace crl
