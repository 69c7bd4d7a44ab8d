// Deterministic ordered reduction of TD deltas that hit the same (s,a) key of
// one table - the replacement for float atomics.  Samples (envs) are taken in
// index order through a fixed three-level tree:
//
//   block  = 256 consecutive samples, added left to right from +0.0f
//   group  = 16 consecutive blocks, block sums added left to right from +0.0f
//   total  = group sums added left to right from +0.0f;   Q[k] = Q[k] + total[k]
//
// Two passes over the chip:
//   1. one workgroup per block walks its 256 samples in order (wave after wave;
//      inside a wave the lanes that share a key are found with ballots and
//      folded in lane order) keeping the running sums in a dense LDS table, and
//      hands every distinct key's block sum to the workgroup that owns the key;
//   2. one workgroup per 64 keys lays the block sums it was handed out as a
//      dense [block][key] tile in LDS and adds the columns in the tree order.
// Empty blocks add +0.0f, which changes nothing, so the result is a pure
// function of (keys, deltas) whatever the occupancy.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace crl {

constexpr int kBlockSamples = 256;   // level 0
constexpr int kGroupBlocks = 16;     // level 1
constexpr int kOwnKeys = 64;         // keys per owner workgroup
constexpr int kSlotCap = 8;          // block sums one block can hand one owner
constexpr int kHandoffRecs = 8;      // one 64-byte hand-off cell of 8 records {key slot | count << 8, sum}
constexpr int kSlotOverflow = 255;   // count value: read the block's raw samples instead
constexpr int kDenseKeys = 16384;    // keys the dense LDS table of pass 1 can hold
constexpr int kTileBlocks = 256;     // blocks per LDS tile of pass 2
constexpr uint32_t kOwnerMix = 37;   // odd: spreads neighbouring keys over owners

struct ReduceGeom {
  int K;          // keys of the table
  int key_bits;   // ceil(log2 K)
  int own_shift;  // log2(number of owners); owners = 1 << own_shift, (K >> own_shift) <= 64
  int n_blocks;   // ceil(n / 256)
};

// key <-> (owner, slot in the owner's 64): slot = key >> own_shift,
// owner = (low bits + 37 * slot) mod owners
__device__ __forceinline__ int owner_of(int key, int own_shift) {
  const uint32_t mask = (1u << own_shift) - 1u;
  const uint32_t hi = (uint32_t)key >> own_shift;
  return (int)(((uint32_t)key + kOwnerMix * hi) & mask);
}
__device__ __forceinline__ int key_of(int owner, int slot, int own_shift) {
  const uint32_t mask = (1u << own_shift) - 1u;
  const uint32_t lo = ((uint32_t)owner - kOwnerMix * (uint32_t)slot) & mask;
  return (int)(((uint32_t)slot << own_shift) | lo);
}

struct ReduceLds {
  float run[kDenseKeys];      // running sum of the block, per key
  uint8_t seen[kDenseKeys];   // key touched by this block
  int handed[256];            // block sums handed to each owner so far
};

// Clears the block's LDS state.  Needs no sample, so a kernel calls it first and
// lets it overlap with the loads that produce the samples; reduce_block() has the
// barrier that orders it before the first use.
__device__ __forceinline__ void reduce_block_clear(ReduceLds& L, const ReduceGeom G) {
  const int tid = threadIdx.x;
  uint4* seen4 = reinterpret_cast<uint4*>(L.seen);
  for (int i = tid; i < kDenseKeys / 16; i += kBlockSamples) seen4[i] = make_uint4(0, 0, 0, 0);
  if (tid < (1 << G.own_shift)) L.handed[tid] = 0;
}

// Pass 1 for one block, after reduce_block_clear().  All 256 threads of the
// workgroup call it with their sample (valid = false: no sample / no delta).
// key < K <= kDenseKeys.
__device__ __forceinline__ void reduce_block(ReduceLds& L, const ReduceGeom G, const int block,
                                             const int key, const float delta, const bool valid,
                                             uint2* __restrict__ handoff) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int n_own = 1 << G.own_shift;

  // lanes of this wave that hold the same key
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
  // The waves take turns below (a key's running sum passes from wave to wave), so
  // what can be done before a wave's turn is done here, by all waves at once: a
  // leader fetches the deltas of its first eight samples, itself included.  Absent
  // ones are +0.0f, which leaves a sum that started from +0.0f unchanged.
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
      while (__ballot(rest != 0ull) != 0ull) {  // the rare key with more than eight samples in a wave
        const int j = rest ? __builtin_ctzll(rest) : lane;
        const float dj = __shfl(delta, j);
        if (rest) acc = acc + dj;  // lane order = sample order
        rest &= rest - 1ull;
      }
      if (leader) {
        L.run[key] = acc;
        L.seen[key] = 1;
        if (first) slot = atomicAdd(&L.handed[owner], 1);  // slot order is free: records carry the key
      }
    }
    __syncthreads();
  }

  // hand-off cell of (owner, block): 64 bytes that the owner gets with one
  // independent read; record 0 also carries the count (0: nothing for this owner)
  if (leader && first && slot < kSlotCap) {
    const size_t at = ((size_t)owner * G.n_blocks + block) * kHandoffRecs + slot;
    uint32_t tag = (uint32_t)(key >> G.own_shift);
    if (slot == 0) {
      const int c = L.handed[owner];  // final: every wave has had its turn
      tag |= (uint32_t)(c > kSlotCap ? kSlotOverflow : c) << 8;
    }
    handoff[at] = make_uint2(tag, __float_as_uint(L.run[key]));
  }
  if (tid < n_own && L.handed[tid] == 0)
    handoff[((size_t)tid * G.n_blocks + block) * kHandoffRecs] = make_uint2(0u, 0u);
}

// Pass 1 over (key, delta) arrays already in memory.
__global__ __launch_bounds__(kBlockSamples) void k_reduce_blocks(const ReduceGeom G,
                                                                 const int32_t* __restrict__ key,
                                                                 const float* __restrict__ delta,
                                                                 const int n,
                                                                 uint2* __restrict__ handoff) {
  extern __shared__ unsigned char lds_raw[];
  ReduceLds& L = *reinterpret_cast<ReduceLds*>(lds_raw);
  reduce_block_clear(L, G);
  const int i = blockIdx.x * kBlockSamples + threadIdx.x;
  const int k = i < n ? key[i] : -1;
  const bool valid = k >= 0;
  const float d = valid ? delta[i] : 0.0f;
  reduce_block(L, G, blockIdx.x, valid ? k : 0, d, valid, handoff);
}

// Pass 2: one workgroup per owner (64 keys).
__global__ __launch_bounds__(256) void k_reduce_owners(const ReduceGeom G, float* __restrict__ Q,
                                                        const int32_t* __restrict__ key,
                                                        const float* __restrict__ delta, const int n,
                                                        const uint2* __restrict__ handoff) {
  extern __shared__ float tile[];  // [kTileBlocks][64] block sums, then [16][64] group sums
  float* gsum = tile + kTileBlocks * kOwnKeys;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int owner = blockIdx.x;
  float total = 0.0f;
  // the table entry this lane will update: fetched now, needed last
  const int my_key = key_of(owner, lane, G.own_shift);
  const float q_old = (wave == 0 && my_key < G.K) ? Q[my_key] : 0.0f;

  for (int b0 = 0; b0 < G.n_blocks; b0 += kTileBlocks) {
    const int b = b0 + tid;
    // the whole hand-off cell in one go: no load depends on another
    uint4 cell[kHandoffRecs / 2];
    if (b < G.n_blocks) {
      const uint4* src = reinterpret_cast<const uint4*>(handoff + ((size_t)owner * G.n_blocks + b) * kHandoffRecs);
#pragma unroll
      for (int i = 0; i < kHandoffRecs / 2; ++i) cell[i] = src[i];
    } else {
#pragma unroll
      for (int i = 0; i < kHandoffRecs / 2; ++i) cell[i] = make_uint4(0, 0, 0, 0);
    }
    float4* my_row = reinterpret_cast<float4*>(tile + tid * kOwnKeys);
#pragma unroll
    for (int i = 0; i < kOwnKeys / 4; ++i) my_row[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    const int c = (int)((cell[0].x >> 8) & 0xFFu);
    if (c != kSlotOverflow) {
      float* row = tile + tid * kOwnKeys;
#pragma unroll
      for (int i = 0; i < kHandoffRecs / 2; ++i) {
        if (c > 2 * i) row[cell[i].x & 0xFFu] = __uint_as_float(cell[i].y);
        if (c > 2 * i + 1) row[cell[i].z & 0xFFu] = __uint_as_float(cell[i].w);
      }
    } else {
      // more distinct keys than slots: redo the block's part from its samples, in order
      const int lo = b * kBlockSamples, hi = min(n, lo + kBlockSamples);
      for (int i = lo; i < hi; ++i) {
        const int k = key[i];
        if (k >= 0 && owner_of(k, G.own_shift) == owner) {
          float& acc = tile[tid * kOwnKeys + (k >> G.own_shift)];
          acc = acc + delta[i];
        }
      }
    }
    __syncthreads();
    // group sums: 16 groups of 16 blocks in this tile, four per wave; lane = key slot
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
#pragma unroll
      for (int grp = 0; grp < kTileBlocks / kGroupBlocks; ++grp) total = total + gsum[grp * kOwnKeys + lane];
    }
    __syncthreads();
  }
  if (wave == 0 && my_key < G.K) Q[my_key] = q_old + total;
}

// Fallback for tables with more than kDenseKeys keys (or too many blocks for the
// hand-off buffer): one workgroup per 64 consecutive keys scans all samples,
// group by group (4096 samples), compacting its matches in order, and wave 0
// then folds them through the same tree.  Slow, same result.
__global__ __launch_bounds__(256) void k_reduce_scan(float* __restrict__ Q, const int K,
                                                      const int32_t* __restrict__ key,
                                                      const float* __restrict__ delta, const int n) {
  constexpr int kSpan = 1024;  // samples one wave scans per group: 4 blocks
  __shared__ float l_d[4][kSpan];
  __shared__ uint8_t l_k[4][kSpan];
  __shared__ uint16_t l_o[4][kSpan];  // sample offset inside the wave's span
  __shared__ int l_cnt[4];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int owner = blockIdx.x;
  float total = 0.0f;

  for (int g0 = 0; g0 < n; g0 += 4 * kSpan) {
    int cnt = 0;
    const int base = g0 + wave * kSpan;
    for (int it = 0; it < kSpan / 64; ++it) {
      const int i = base + it * 64 + lane;
      const int k = (i < n) ? key[i] : -1;
      const bool match = (k >= 0) && ((k / kOwnKeys) == owner);
      const unsigned long long bal = __ballot(match);
      if (bal != 0ull) {
        if (match) {
          const int pos = cnt + __popcll(bal & ((1ull << lane) - 1ull));
          l_d[wave][pos] = delta[i];
          l_k[wave][pos] = (uint8_t)(k - owner * kOwnKeys);
          l_o[wave][pos] = (uint16_t)(it * 64 + lane);
        }
        cnt += __popcll(bal);
      }
    }
    if (lane == 0) l_cnt[wave] = cnt;
    __syncthreads();
    if (wave == 0) {
      float gs = 0.0f;
      for (int w = 0; w < 4; ++w) {
        const int c = l_cnt[w];
        float bs = 0.0f;
        int cur = 0;  // block inside the wave's span
        for (int e = 0; e < c; ++e) {
          const int blk = l_o[w][e] >> 8;
          if (blk != cur) {
            gs = gs + bs;
            bs = 0.0f;
            cur = blk;
          }
          const float dv = l_d[w][e];
          if (l_k[w][e] == lane) bs = bs + dv;
        }
        gs = gs + bs;
      }
      total = total + gs;
    }
    __syncthreads();
  }
  const int k = owner * kOwnKeys + lane;
  if (wave == 0 && k < K) Q[k] = Q[k] + total;
}

}  // namespace crl
