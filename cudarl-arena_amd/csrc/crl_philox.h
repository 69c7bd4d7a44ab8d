// Philox4x32-10 counter-based generator (Salmon, Moraes, Dror, Shaw, SC'11),
// usable from host code and from gfx950 device code.  The reference has no
// reproducible generator (np.random / rand() / time-seeded mt19937:
// src/train.py:101-102, src/main.cu:51, src/environment.cu:140-142); the
// engine's exploration stream is this one, keyed by (seed; env, step).
#pragma once
#include <stdint.h>

#if defined(__HIP__)
#define CRL_HD __host__ __device__ inline __attribute__((always_inline))
#else
#define CRL_HD inline
#endif

namespace crl {

// four named words, not an array: a select between two array elements would be
// folded into an indexed load and push the block into scratch memory on the GPU
struct Philox4 {
  uint32_t w0, w1, w2, w3;
};

CRL_HD Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                             uint32_t k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  Philox4 r;
  r.w0 = c0;
  r.w1 = c1;
  r.w2 = c2;
  r.w3 = c3;
  return r;
}

// stream ids: second counter word
enum : uint32_t {
  kStreamExplore = 0,
  kStreamMap = 1,
  kStreamStartGoal = 2,
  kStreamTrap = 3,
  kStreamReward = 4,
  kStreamLattice = 5
};

// One block serves two consecutive steps: block = t >> 1, even t uses words
// 0,1 and odd t words 2,3.
CRL_HD Philox4 explore_block(uint64_t seed, uint32_t env, uint64_t block) {
  return philox4x32_10(env, kStreamExplore, (uint32_t)block, (uint32_t)(block >> 32),
                       (uint32_t)seed, (uint32_t)(seed >> 32));
}

// uniform in [0,1) from the top 24 bits: exact in fp32
CRL_HD float u01(uint32_t w) { return (float)(w >> 8) * (1.0f / 16777216.0f); }

// integer in [0, n) by multiply-shift
CRL_HD uint32_t below(uint32_t w, uint32_t n) { return (uint32_t)(((uint64_t)w * n) >> 32); }

}  // namespace crl
