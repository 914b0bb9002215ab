// Device-side helpers shared by the kernel translation units (gfx950 only).
#pragma once

#include "scn_kernels.hpp"

namespace scn {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// --------------------------------------------------------------------------------------------
// device helpers
// --------------------------------------------------------------------------------------------
// murmur3 finaliser evaluated in 64 bits (libraries/3DSparseConvolution/src/voxelization.cu:41-48)
__host__ __device__ __forceinline__ uint64_t hash64(uint64_t k) {
  k ^= k >> 16;
  k *= 0x85ebca6bull;
  k ^= k >> 13;
  k *= 0xc2b2ae35ull;
  k ^= k >> 16;
  return k;
}

__device__ __forceinline__ void table_insert(uint64_t* slots, uint32_t mask, uint32_t key, uint32_t row) {
  const uint64_t packed = ((uint64_t)key << 32) | row;
  uint32_t slot = (uint32_t)hash64(key) & mask;
  for (uint32_t probe = 0; probe <= mask; ++probe) {
    unsigned long long prev = atomicCAS((unsigned long long*)&slots[slot], (unsigned long long)kEmptySlot,
                                        (unsigned long long)packed);
    if (prev == kEmptySlot) return;
    if ((uint32_t)(prev >> 32) == key) {  // duplicate coordinate: the lowest row wins, deterministically
      atomicMin((unsigned long long*)&slots[slot], (unsigned long long)packed);
      return;
    }
    slot = (slot + 1) & mask;
  }
}

__device__ __forceinline__ int32_t table_lookup(const uint64_t* __restrict__ slots, uint32_t mask, uint32_t key) {
  uint32_t slot = (uint32_t)hash64(key) & mask;
  for (uint32_t probe = 0; probe <= mask; ++probe) {
    const uint64_t v = slots[slot];
    if (v == kEmptySlot) return -1;
    if ((uint32_t)(v >> 32) == key) return (int32_t)(uint32_t)v;
    slot = (slot + 1) & mask;
  }
  return -1;
}

__device__ __forceinline__ uint32_t eff_n(const uint32_t* n_dev, uint32_t n_bound) {
  if (n_dev == nullptr) return n_bound;
  const uint32_t n = *n_dev;
  return n < n_bound ? n : n_bound;
}

struct Int3 {
  int v[3];
};

// Block-wide exclusive scan of one value per thread (blockDim.x multiple of 64, <= 1024).
// Returns the exclusive prefix; *total receives the block sum.  scratch: >= 17 uint32 in LDS.
__device__ __forceinline__ uint32_t block_exclusive_scan(uint32_t x, uint32_t* scratch, uint32_t* total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  uint32_t incl = x;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    uint32_t y = __shfl_up(incl, d, 64);
    if (lane >= d) incl += y;
  }
  __syncthreads();  // scratch may still be read from a previous call
  if (lane == 63) scratch[wave] = incl;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t s = 0;
    for (int w = 0; w < nw; ++w) {
      uint32_t t = scratch[w];
      scratch[w] = s;
      s += t;
    }
    scratch[16] = s;
  }
  __syncthreads();
  *total = scratch[16];
  return scratch[wave] + incl - x;
}

// --------------------------------------------------------------------------------------------
// Workgroup-level aggregation of bitmap ORs.  Atomics on a bitmap shared by all XCDs are resolved
// outside the XCD-local L2 and are slow; rows arrive in (nearly) sorted order, so the rows of one
// workgroup hit few distinct words.  The ORs are first combined in a small LDS hash of
// (word index -> bits) and each distinct word then costs one global atomic.
// --------------------------------------------------------------------------------------------
constexpr uint32_t kAggSlots = 2048;  // power of two
constexpr uint32_t kAggEmpty = 0xFFFFFFFFu;

__device__ __forceinline__ void agg_init(uint32_t* keys, uint32_t* vals) {
  for (uint32_t i = threadIdx.x; i < kAggSlots; i += blockDim.x) {
    keys[i] = kAggEmpty;
    vals[i] = 0;
  }
  __syncthreads();
}

__device__ __forceinline__ void agg_or(uint32_t* keys, uint32_t* vals, uint32_t* bitmap, uint32_t word, uint32_t bits) {
  uint32_t slot = (word * 2654435761u) >> (32 - 11);
  for (int probe = 0; probe < 16; ++probe) {
    const uint32_t prev = atomicCAS(&keys[slot], kAggEmpty, word);
    if (prev == kAggEmpty || prev == word) {
      atomicOr(&vals[slot], bits);
      return;
    }
    slot = (slot + 1) & (kAggSlots - 1);
  }
  atomicOr(&bitmap[word], bits);  // crowded table: straight to memory
}

__device__ __forceinline__ void agg_flush(const uint32_t* keys, const uint32_t* vals, uint32_t* bitmap) {
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < kAggSlots; i += blockDim.x) {
    const uint32_t w = keys[i];
    if (w != kAggEmpty) atomicOr(&bitmap[w], vals[i]);
  }
}

// int8 store of the fake-quant form: round(y * (127/amax)), saturated to +-127
__device__ __forceinline__ float quant_f(float y, float r) {
  float q = rintf(y * r);
  q = fminf(fmaxf(q, -127.f), 127.f);  // NaN -> -127 (fmaxf returns the non-NaN operand)
  return q;
}

__device__ __forceinline__ float half_round(float y) { return (float)(_Float16)y; }

}  // namespace scn
