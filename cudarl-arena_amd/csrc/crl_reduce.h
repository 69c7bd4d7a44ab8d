// Deterministic ordered reduction of TD deltas that hit the same (s,a) key of
// one table - the replacement for float atomics.  Samples (envs) are taken in
// index order through a fixed three-level tree:
//
//   block  = 256 consecutive samples, added left to right from +0.0f
//   group  = 16 consecutive blocks, block sums added left to right from +0.0f
//   total  = group sums added left to right from +0.0f;   Q[k] = Q[k] + total[k]
//
// Two passes over the chip:
//   1. one workgroup per block: the lowest thread that holds a key becomes the
//      key's leader (LDS atomic min on a dense table), the other holders mark
//      themselves in the leader's 256-bit member set (LDS atomic or) and line
//      their deltas up by their place in it, and the leader adds them in that
//      order = thread order = sample order; every distinct key's block sum goes
//      to the workgroup that owns the key;
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
constexpr int kOwnKeys = 64;         // keys per owner workgroup: 64 / A whole table rows
constexpr int kMinCellRecs = 8;      // records of a hand-off cell: 8 ... 64, see cell_shift_for()
constexpr int kSlotOverflow = 127;   // count value: more distinct keys than records, read the block's raw samples instead
constexpr int kStagePieces = 512;    // 16-byte pieces of the main halves of one block's cells in the one-launch kernel
constexpr int kDenseKeys = 16384;    // keys the dense LDS table of pass 1 can hold
constexpr int kTileBlocks = 256;     // blocks per LDS tile of pass 2
constexpr uint32_t kOwnerMix = 37;   // odd: spreads cells a power of two apart over owners
constexpr uint32_t kNoLead = 0xFFFFFFFFu;

// A hand-off record is 64 bits, written and read as one unit:
//   bits  0..5   slot of the key among its owner's 64
//   bits  6..12  record 0 of a cell only: how many records the cell holds
//                (0: none, kSlotOverflow: more distinct keys than the cell has records)
//   bits 13..31  step tag (the one-launch kernel: a record is valid once its tag is
//                the step's; 0 where launches separate the steps)
//   bits 32..63  the block sum, fp32
constexpr int kRecCountShift = 6, kRecTagShift = 13;
constexpr uint32_t kRecTagMask = (1u << (32 - kRecTagShift)) - 1u;
__device__ __forceinline__ unsigned long long make_rec(uint32_t slot, uint32_t count, uint32_t tag, float v) {
  const uint32_t meta = slot | (count << kRecCountShift) | (tag << kRecTagShift);
  return (unsigned long long)meta | ((unsigned long long)__float_as_uint(v) << 32);
}
__device__ __forceinline__ int rec_slot(uint32_t meta) { return (int)(meta & 63u); }
__device__ __forceinline__ int rec_count(uint32_t meta) { return (int)((meta >> kRecCountShift) & 127u); }
__device__ __forceinline__ uint32_t rec_tag(uint32_t meta) { return meta >> kRecTagShift; }

struct ReduceGeom {
  int K;          // keys of the table, key = cell * A + action
  int a_shift;    // log2(A)
  int own_shift;  // log2(number of owners); owners = 1 << own_shift, (K >> own_shift) <= 64
  int n_blocks;   // ceil(n / 256)
  int cell_shift; // log2(records of a hand-off cell), cell_shift_for(own_shift)
  int main_shift; // one-launch kernel: log2(records in the part of a cell that is written every step), main_shift_for()
};

// Records per hand-off cell.  A block's 256 samples spread over the owners, so a cell
// sees about 256 / owners distinct keys: eight records for 256 owners (more than eight
// keys once in a million cells), more where fewer owners share the samples, and all 64
// keys an owner has from 16 owners down, where a cell cannot overflow at all.  A block's
// cells together stay within 16 KB.
__host__ __device__ constexpr int cell_shift_for(int own_shift) {
  return own_shift >= 8 ? 3 : own_shift >= 6 ? 4 : own_shift == 5 ? 5 : 6;
}

// One-launch kernel: what a block's cell stores cost grows with their bytes (16 KB of
// cells of eight records for 256 owners, seven eighths of them padding, need 1.4 us to be
// acknowledged, 8 KB half of that).  So with more than 64 owners a cell is two halves:
// the main half, written whole every step with all the others of the block (8 KB), and
// an extension of as many records that only a block with more distinct keys for that
// owner than the main half holds writes into (one cell in 270 with 256 owners), record by
// record.  Record 0 of the main half says how many records there are in all.  The
// extensions lie [owner][block]: an owner asks for all of them with its main halves,
// 8 KB in one piece, and looks at those the counts point to.
__host__ __device__ constexpr int main_shift_for(int own_shift) {
  const int c = cell_shift_for(own_shift), m = 10 - own_shift;
  return m < c ? (m < 2 ? 2 : m) : c;
}

// key <-> (owner, slot in the owner's 64).  An owner holds whole table rows:
// hi = cell >> own_shift, owner = (cell + 37 * hi) mod owners, slot = hi * A + action
__device__ __forceinline__ int owner_of(int key, const ReduceGeom& G) {
  const uint32_t mask = (1u << G.own_shift) - 1u;
  const uint32_t cell = (uint32_t)key >> G.a_shift;
  return (int)((cell + kOwnerMix * (cell >> G.own_shift)) & mask);
}
__device__ __forceinline__ int slot_of(int key, const ReduceGeom& G) {
  const uint32_t cell = (uint32_t)key >> G.a_shift;
  return (int)(((cell >> G.own_shift) << G.a_shift) | ((uint32_t)key & ((1u << G.a_shift) - 1u)));
}
__device__ __forceinline__ int key_of(int owner, int slot, const ReduceGeom& G) {
  const uint32_t mask = (1u << G.own_shift) - 1u;
  const uint32_t hi = (uint32_t)slot >> G.a_shift;
  const uint32_t lo = ((uint32_t)owner - kOwnerMix * hi) & mask;
  const uint32_t cell = (hi << G.own_shift) | lo;
  return (int)((cell << G.a_shift) | ((uint32_t)slot & ((1u << G.a_shift) - 1u)));
}

// ---- device-scope accesses --------------------------------------------------------
// gfx950 has eight XCDs, each with its own L2; plain loads and stores are coherent
// inside one XCD only.  Relaxed atomic loads and stores at agent scope compile to
// accesses that carry the sc1 bit and are served past the L2: a value stored that
// way by one workgroup is seen by the next such load of any other, without the
// whole-L2 write-back / invalidate of a release / acquire fence.  64 bits is the
// unit: every exchanged datum carries its own step tag in the same 64 bits, so no
// ordering between two stores is ever relied on.
__device__ __forceinline__ void st_dev64(unsigned long long* p, unsigned long long v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long ld_dev64(const unsigned long long* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_dev32(unsigned* p, unsigned v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned ld_dev32(const unsigned* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Aligned 16-byte device-scope loads: a buffer load with the sc1 bit, through a window
// (buffer descriptor) that starts at `base` and spans 2 GB.  Each aligned 64-bit half is
// one of the tagged units above; nothing is assumed about the two halves of a load
// belonging together.  To the compiler this is an ordinary read of memory: a loop that
// asks again and again must call poll_fence() in every round, or the load is taken out
// of the loop as invariant.
typedef unsigned int crl_u4 __attribute__((ext_vector_type(4)));
using DevWindow = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ DevWindow dev_window(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ uint4 ld_dev128(DevWindow w, uint32_t byte_offset) {
  const crl_u4 v = __builtin_amdgcn_raw_buffer_load_b128(w, (int)byte_offset, 0, 16 /* sc1 */);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st_dev128(DevWindow w, uint32_t byte_offset, const uint4 v) {
  crl_u4 t;
  t.x = v.x;
  t.y = v.y;
  t.z = v.z;
  t.w = v.w;
  __builtin_amdgcn_raw_buffer_store_b128(t, w, (int)byte_offset, 0, 16 /* sc1 */);
}
__device__ __forceinline__ void poll_fence() { asm volatile("" ::: "memory"); }

struct alignas(16) ReduceLds {  // (lead and members are also accessed 16 bytes at a time)
  alignas(16) uint32_t lead[kDenseKeys];                     // lowest thread of the block that holds the key; kNoLead between uses
  alignas(16) unsigned long long members[kBlockSamples][4];  // per leader: the threads that hold its key; zero between uses
  float delta[kBlockSamples];
  int handed[256];                               // block sums handed to each owner
  int over;                                      // some owner was handed more than a cell holds
};

// Besides ReduceLds, reduce_block() needs kSortBytes of LDS for `sorted`: the deltas of a
// key's further holders, lined up for its leader ([place among the holders][leader]).
constexpr int kSortRows = 32;
constexpr size_t kSortBytes = (size_t)kSortRows * kBlockSamples * sizeof(float);
constexpr size_t kReduceLdsBytes = sizeof(ReduceLds) + kSortBytes;  // ReduceLds, then `sorted`

// Once per kernel, before the first reduce_block() and separated from it by a barrier.
__device__ __forceinline__ void reduce_block_init(ReduceLds& L) {
  const int tid = threadIdx.x;
  uint4* lead4 = reinterpret_cast<uint4*>(L.lead);
  for (int i = tid; i < kDenseKeys / 4; i += kBlockSamples) lead4[i] = make_uint4(kNoLead, kNoLead, kNoLead, kNoLead);
  L.members[tid][0] = 0ull;
  L.members[tid][1] = 0ull;
  L.members[tid][2] = 0ull;
  L.members[tid][3] = 0ull;
  if (tid == 0) L.over = 0;
}

// Pass 1 for one block.  All 256 threads of the workgroup call it with their
// sample (valid = false: no sample / no delta); key < K <= kDenseKeys.  Leaves the
// LDS state as reduce_block_init() did, so it can be called again and again.
// DEV = false: the records go straight to memory with plain stores, for a reader in a
// later launch; the cell of (owner, block) is at handoff[(owner * blocks + block) << cell_shift],
// so that an owner reads its cells side by side.
// DEV = true: for readers on other XCDs in the same launch.  All cells of the block
// main halves are put together in LDS (`stage`, owners << main_shift records, free again
// on return) and go out as whole lines (that of (block, owner) at (block * owners + owner)
// << main_shift behind `window_offset`), 16 bytes to a store and lane, every record
// carrying `tag`; a record beyond the main half goes straight to
// ext[(owner * blocks + block) << main_shift]:
// scattered 8-byte stores are partial line writes, and some 350 of them per workgroup
// took 1.6 us to be acknowledged.  `window` is a buffer window on `handoff`.
// Returns (to every thread) whether some owner was handed more distinct keys than a
// cell has records: its cell then says kSlotOverflow and the owner needs the block's
// raw samples.
// DEV = true: before each reduce_block(), separated from it by a barrier (and from the
// one before by another): every record of every cell starts as "nothing, of this step".
// Thread t touches the 16-byte pieces t, t + 256, ... of `stage` here and on the way out
// of reduce_block(), and no others.
__device__ __forceinline__ void reduce_stage_init(unsigned long long* stage, const ReduceGeom G, const uint32_t tag) {
  const unsigned long long none = make_rec(0u, 0u, tag, 0.0f);
  ulonglong2* stage2 = reinterpret_cast<ulonglong2*>(stage);
  for (int i = threadIdx.x; i < 1 << (G.main_shift - 1 + G.own_shift); i += kBlockSamples) stage2[i] = make_ulonglong2(none, none);
}

template <bool DEV>
__device__ __forceinline__ bool reduce_block(ReduceLds& L, const ReduceGeom G, const int block,
                                             const int key, const float delta, const bool valid,
                                             unsigned long long* handoff, const uint32_t tag, float* sorted,
                                             unsigned long long* stage = nullptr, const DevWindow* window = nullptr,
                                             const uint32_t window_offset = 0, unsigned long long* ext = nullptr,
                                             const bool elected = false) {
  const int tid = threadIdx.x;
  const int n_own = 1 << G.own_shift;
  const int cap = 1 << G.cell_shift;  // records of a cell
  const int cap_main = 1 << G.main_shift;  // DEV: of its main half
  if (valid && !elected) atomicMin(&L.lead[key], (uint32_t)tid);  // (elected: the caller has done this already)
  L.delta[tid] = delta;
  __syncthreads();
  L.handed[tid] = 0;  // (256 >= owners; the last call's readers are past the barrier above)
  if (tid == 0) L.over = 0;
  uint32_t ld = (uint32_t)tid;
  if (valid) {
    ld = L.lead[key];
    if (ld != (uint32_t)tid) atomicOr(&L.members[ld][tid >> 6], 1ull << (tid & 63));
  }
  __syncthreads();
  // A key's sum is its samples' deltas added in thread order, one after the other: the
  // leader has to walk through them.  Every further holder finds its place among them
  // (the set bits below its own) and puts its delta there, all at once, so that the
  // leader's walk is loads from known addresses, several in flight, instead of one bit
  // scan, load and add after the other (envs that crowd on a few cells: 14 holders of
  // one key in most blocks, 1 us of such a walk).
  // (Written without branches: one wave to a SIMD has nothing to hide them behind.  A thread
  // without a sample reads its own, empty member set; a thread that has nothing to line up
  // writes its delta where it already is.)
  const bool leader = valid && ld == (uint32_t)tid;
  unsigned long long mw[4];
  int holders;  // leader: the key's further holders
  {
    const ulonglong2 lo = *reinterpret_cast<const ulonglong2*>(&L.members[ld][0]);
    const ulonglong2 hi = *reinterpret_cast<const ulonglong2*>(&L.members[ld][2]);
    mw[0] = lo.x;
    mw[1] = lo.y;
    mw[2] = hi.x;
    mw[3] = hi.y;
    const int p0 = __popcll(mw[0]), p1 = __popcll(mw[1]), p2 = __popcll(mw[2]), p3 = __popcll(mw[3]);
    holders = leader ? p0 + p1 + p2 + p3 : 0;
    const int w = tid >> 6;
    const unsigned long long mine = w == 0 ? mw[0] : w == 1 ? mw[1] : w == 2 ? mw[2] : mw[3];
    const int place = (w > 0 ? p0 : 0) + (w > 1 ? p1 : 0) + (w > 2 ? p2 : 0) + __popcll(mine & ((1ull << (tid & 63)) - 1ull));
    const bool lines_up = valid && !leader && place < kSortRows;
    *(lines_up ? &sorted[place * kBlockSamples + (int)ld] : &L.delta[tid]) = delta;
  }
  __syncthreads();
  float acc = 0.0f;
  int slot = 0, owner = 0;
  if (leader) {
    acc = acc + delta;  // the leader is the key's first sample; the other holders come after it
    if (holders != 0) {
      *reinterpret_cast<ulonglong2*>(&L.members[tid][0]) = make_ulonglong2(0ull, 0ull);
      *reinterpret_cast<ulonglong2*>(&L.members[tid][2]) = make_ulonglong2(0ull, 0ull);
      const int lined = holders < kSortRows ? holders : kSortRows;
      for (int r0 = 0; r0 < lined; r0 += 4) {
        float d[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) d[i] = sorted[(r0 + i < kSortRows ? r0 + i : kSortRows - 1) * kBlockSamples + tid];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (r0 + i < lined) acc = acc + d[i];  // thread order = sample order
      }
      if (holders > kSortRows) {  // more holders than places: the rest one by one
        int seen = 0;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
          unsigned long long m = mw[w];
          while (m != 0ull) {
            const int j = __builtin_ctzll(m);
            if (seen >= kSortRows) acc = acc + L.delta[w * 64 + j];
            ++seen;
            m &= m - 1ull;
          }
        }
      }
    }
    L.lead[key] = kNoLead;
    owner = owner_of(key, G);
    slot = atomicAdd(&L.handed[owner], 1);  // slot order is free: records carry the key
    if (slot >= cap) L.over = 1;
    // (record 0's count is added on the way out, when every leader has drawn its slot)
    if (DEV && slot < cap_main) stage[(owner << G.main_shift) + slot] = make_rec((uint32_t)slot_of(key, G), 0u, tag, acc);
  }
  __syncthreads();
  const bool over = L.over != 0;
  // (behind the barrier: a barrier waits for the stores before it to be acknowledged)
  if (DEV && leader && slot >= cap_main && slot < cap)
    st_dev64(ext + ((((size_t)owner * G.n_blocks + block) << G.main_shift) + (slot - cap_main)),
             make_rec((uint32_t)slot_of(key, G), 0u, tag, acc));

  if (DEV) {
    // (the one-launch kernel always has 256 owners and main halves of 4 records: 512 pieces,
    // two to a thread, both asked for before the first is used)
    const ulonglong2* stage2 = reinterpret_cast<const ulonglong2*>(stage);
    const int piece_shift = G.main_shift - 1;  // log2(pieces of a cell's main half)
    const int pieces = n_own << piece_shift;
    constexpr int kPer = kStagePieces / kBlockSamples;
    static_assert(kPer == 2, "two pieces of the stage to a thread");
    ulonglong2 v[kPer];
    int c[kPer];
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int i = tid + j * kBlockSamples;
      v[j] = i < pieces ? stage2[i] : make_ulonglong2(0ull, 0ull);
      c[j] = (i < pieces && (i & ((1 << piece_shift) - 1)) == 0) ? L.handed[i >> piece_shift] : 0;
    }
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int i = tid + j * kBlockSamples;
      v[j].x |= (unsigned long long)(uint32_t)(c[j] > cap ? kSlotOverflow : c[j]) << kRecCountShift;
      if (i < pieces)
        st_dev128(*window, window_offset + (uint32_t)((((size_t)block * n_own) << (G.main_shift + 3)) + (size_t)i * 16),
                  make_uint4((uint32_t)v[j].x, (uint32_t)(v[j].x >> 32), (uint32_t)v[j].y, (uint32_t)(v[j].y >> 32)));
    }
  } else {
    if (leader && slot < cap) {
      uint32_t count = 0;
      if (slot == 0) {
        const int c = L.handed[owner];  // final: every leader has drawn its slot
        count = (uint32_t)(c > cap ? kSlotOverflow : c);
      }
      handoff[((((size_t)owner * G.n_blocks) + block) << G.cell_shift) + slot] = make_rec((uint32_t)slot_of(key, G), count, tag, acc);
    }
    if (tid < n_own && L.handed[tid] == 0) handoff[(((size_t)tid * G.n_blocks) + block) << G.cell_shift] = make_rec(0u, 0u, tag, 0.0f);
  }
  return over;
}

// Pass 1 over (key, delta) arrays already in memory.
__global__ __launch_bounds__(kBlockSamples) void k_reduce_blocks(const ReduceGeom G,
                                                                 const int32_t* __restrict__ key,
                                                                 const float* __restrict__ delta,
                                                                 const int n,
                                                                 unsigned long long* __restrict__ handoff) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  ReduceLds& L = *reinterpret_cast<ReduceLds*>(lds_raw);
  reduce_block_init(L);
  const int i = blockIdx.x * kBlockSamples + threadIdx.x;
  const int k = i < n ? key[i] : -1;
  const bool valid = k >= 0;
  const float d = valid ? delta[i] : 0.0f;
  __syncthreads();
  reduce_block<false>(L, G, blockIdx.x, valid ? k : 0, d, valid, handoff, 0u, reinterpret_cast<float*>(lds_raw + sizeof(ReduceLds)));
}

// Pass 2: one workgroup per owner (64 keys).
__global__ __launch_bounds__(256) void k_reduce_owners(const ReduceGeom G, float* __restrict__ Q,
                                                        const int32_t* __restrict__ key,
                                                        const float* __restrict__ delta, const int n,
                                                        const unsigned long long* __restrict__ handoff) {
  extern __shared__ __align__(16) float tile[];  // [kTileBlocks][64] block sums, then [16][64] group sums, then a word per thread
  float* gsum = tile + kTileBlocks * kOwnKeys;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int owner = blockIdx.x;
  float total = 0.0f;
  // the table entry this lane will update: fetched now, needed last
  const int my_key = key_of(owner, lane, G);
  const float q_old = (wave == 0 && my_key < G.K) ? Q[my_key] : 0.0f;

  for (int b0 = 0; b0 < G.n_blocks; b0 += kTileBlocks) {
    const int b = b0 + tid;
    // the first eight records of the hand-off cell in one go: no load depends on
    // another (a cell with more records has the rest fetched below, when it holds them)
    uint4 cell[kMinCellRecs / 2];
    const uint4* src = reinterpret_cast<const uint4*>(handoff + ((((size_t)owner * G.n_blocks) + b) << G.cell_shift));
    if (b < G.n_blocks) {
#pragma unroll
      for (int i = 0; i < kMinCellRecs / 2; ++i) cell[i] = src[i];
    } else {
#pragma unroll
      for (int i = 0; i < kMinCellRecs / 2; ++i) cell[i] = make_uint4(0, 0, 0, 0);
    }
    // the tile is cleared by all threads side by side (a thread clearing its own row
    // would put all 64 lanes of a store on the same LDS banks)
    float4* tile4 = reinterpret_cast<float4*>(tile);
#pragma unroll
    for (int i = 0; i < kTileBlocks * kOwnKeys / 4 / 256; ++i) tile4[i * 256 + tid] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    __syncthreads();
    const int c = rec_count(cell[0].x);
    if (c != kSlotOverflow) {
      float* row = tile + tid * kOwnKeys;
      // (no branches: a record that is not there goes to a word that nobody reads)
      float* none = gsum + 16 * kOwnKeys + tid;
#pragma unroll
      for (int i = 0; i < kMinCellRecs / 2; ++i) {
        *(c > 2 * i ? &row[rec_slot(cell[i].x)] : none) = __uint_as_float(cell[i].y);
        *(c > 2 * i + 1 ? &row[rec_slot(cell[i].z)] : none) = __uint_as_float(cell[i].w);
      }
      for (int i = kMinCellRecs / 2; 2 * i < c; ++i) {
        const uint4 more = src[i];
        row[rec_slot(more.x)] = __uint_as_float(more.y);
        if (c > 2 * i + 1) row[rec_slot(more.z)] = __uint_as_float(more.w);
      }
    } else {
      // more distinct keys than slots: redo the block's part from its samples, in order
      const int lo = b * kBlockSamples, hi = min(n, lo + kBlockSamples);
      for (int i = lo; i < hi; ++i) {
        const int k = key[i];
        if (k >= 0 && owner_of(k, G) == owner) {
          float& acc = tile[tid * kOwnKeys + slot_of(k, G)];
          acc = acc + delta[i];
        }
      }
    }
    __syncthreads();
    // group sums: 16 groups of 16 blocks in this tile, four per wave; a lane takes four
    // keys of one group (16 LDS loads of 16 bytes instead of 64 of 4)
    {
      const int grp = wave * 4 + (lane >> 4);
      const float4* rows = reinterpret_cast<const float4*>(tile + grp * kGroupBlocks * kOwnKeys) + (lane & 15);
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
      reinterpret_cast<float4*>(gsum + grp * kOwnKeys)[lane & 15] = acc;
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
