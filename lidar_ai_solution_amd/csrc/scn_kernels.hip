// Hand-written gfx950 kernels of the SCN path and their launchers.
//
//   coordinate hash        atomicCAS open addressing over 64-bit {key,row} slots
//   bitmap rank            occupancy bitmap + popcount scan: de-duplicates and orders keys
//   rulebooks              output-stationary neighbour tables nbr[k][out] (+ pair compaction)
//   gather-GEMM            MFMA 16x16x64 i8 / 16x16x32 f16, operands gathered straight into the
//                          MFMA register layout, fused bias/requant/ReLU/residual epilogue
//   elementwise            quantise / dequantise / pad, add(+relu)
//   sparse -> dense        zero fill + strided scatter (covers the fused Transpose)
//   voxelization           bitmap rank for voxel ids + atomicMin cascade for the kept points
//
// All kernels read row counts from device memory so that a forward pass never needs the host.
#include "scn_kernels.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <type_traits>
#include <vector>

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

// --------------------------------------------------------------------------------------------
// fill
// --------------------------------------------------------------------------------------------
__global__ void k_fill_u32(uint32_t* __restrict__ p, uint32_t value, size_t count) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  // 16-byte stores over the aligned body
  const size_t n4 = count / 4;
  uint4 v4 = make_uint4(value, value, value, value);
  for (size_t j = i; j < n4; j += stride) reinterpret_cast<uint4*>(p)[j] = v4;
  for (size_t j = n4 * 4 + i; j < count; j += stride) p[j] = value;
}

// Several fills (and the publication of a clamped row count) in one launch: grid.y = job.
struct FillJobs {
  FillJob j[kMaxFillJobs];
};

__global__ __launch_bounds__(256) void k_fill_multi(FillJobs jobs, uint32_t* count_dst, const uint32_t* n_dev,
                                                    uint32_t n_bound) {
  if (count_dst && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    const uint32_t n = eff_n(n_dev, n_bound);
    count_dst[0] = n;
    count_dst[1] = n;
  }
  const FillJob job = jobs.j[blockIdx.y];
  uint32_t* p = reinterpret_cast<uint32_t*>(job.p);
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t n4 = job.count / 4;
  const uint4 v4 = make_uint4(job.value, job.value, job.value, job.value);
  for (size_t k = i; k < n4; k += stride) reinterpret_cast<uint4*>(p)[k] = v4;
  for (size_t k = n4 * 4 + i; k < job.count; k += stride) p[k] = job.value;
}

int fill_multi(const FillJob* jobs, int n_jobs, uint32_t* count_dst, const uint32_t* n_dev, uint32_t n_bound,
               hipStream_t stream) {
  SCN_REQUIRE(n_jobs >= 0 && n_jobs <= kMaxFillJobs, SCN_ERR_INVALID, "fill_multi: too many jobs");
  FillJobs fj;
  memset(&fj, 0, sizeof(fj));
  for (int i = 0; i < n_jobs; ++i) {
    SCN_REQUIRE(((uintptr_t)jobs[i].p & 15) == 0, SCN_ERR_INVALID, "fill_multi: pointer not 16-byte aligned");
    fj.j[i] = jobs[i];
  }
  hipLaunchKernelGGL(k_fill_multi, dim3(1024, n_jobs > 0 ? n_jobs : 1), dim3(256), 0, stream, fj, count_dst, n_dev,
                     n_bound);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

int fill_u32(void* p, uint32_t value, size_t count, hipStream_t stream) {
  if (count == 0) return SCN_OK;
  SCN_REQUIRE(((uintptr_t)p & 15) == 0, SCN_ERR_INVALID, "fill_u32: pointer not 16-byte aligned");
  size_t blocks = (count / 4 + 255) / 256;
  if (blocks < 1) blocks = 1;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)blocks), dim3(256), 0, stream, (uint32_t*)p, value, count);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// coordinate hash build / query
// --------------------------------------------------------------------------------------------
__device__ __forceinline__ bool coord_key(const int4 c, const Int3 g, uint32_t* key) {
  if (c.x != 0 || c.y < 0 || c.y >= g.v[0] || c.z < 0 || c.z >= g.v[1] || c.w < 0 || c.w >= g.v[2]) return false;
  *key = ((uint32_t)c.y * (uint32_t)g.v[1] + (uint32_t)c.z) * (uint32_t)g.v[2] + (uint32_t)c.w;
  return true;
}

// filter (nullable): occupancy bitmap of the grid, set for every inserted coordinate; lookups test it
// before probing the table (most neighbour lookups of a sparse tensor miss).
__global__ __launch_bounds__(256) void k_hash_insert(uint64_t* slots, uint32_t mask, const int4* __restrict__ coords,
                                                     uint32_t n_bound, const uint32_t* n_dev, Int3 grid,
                                                     uint32_t* n_eff_out, uint32_t* filter) {
  __shared__ uint32_t akeys[kAggSlots], avals[kAggSlots];
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r == 0 && n_eff_out) {
    n_eff_out[0] = n;
    n_eff_out[1] = n;
  }
  if (filter) agg_init(akeys, avals);
  uint32_t key;
  if (r < n && coord_key(coords[r], grid, &key)) {
    table_insert(slots, mask, key, r);
    if (filter) agg_or(akeys, avals, filter, key >> 5, 1u << (key & 31));
  }
  if (filter) agg_flush(akeys, avals, filter);
}

__global__ void k_hash_query(const uint64_t* __restrict__ slots, uint32_t mask, const int4* __restrict__ coords,
                             uint32_t n, Int3 grid, int32_t* rows) {
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= n) return;
  uint32_t key;
  rows[r] = coord_key(coords[r], grid, &key) ? table_lookup(slots, mask, key) : -1;
}

size_t hash_capacity_for(uint32_t n) {
  size_t cap = 1024;
  while (cap < (size_t)n * 2) cap <<= 1;
  return cap;
}

bool CoordTable::alloc_for(uint32_t max_rows) {
  cap = hash_capacity_for(max_rows);
  mask = (uint32_t)(cap - 1);
  return buf.alloc(cap * sizeof(uint64_t));
}

// Occupancy filter of the whole grid, one bit per cell; skipped (lookups then go straight to the
// table) for grids above 2^29 cells = 64 MB of bitmap.
bool CoordTable::alloc_filter(const int grid[3]) {
  const uint64_t cells = (uint64_t)grid[0] * (uint64_t)grid[1] * (uint64_t)grid[2];
  if (cells == 0 || cells > (1ull << 29)) {
    filter_words = 0;
    return true;
  }
  const size_t words = (size_t)((cells + 31) / 32 + 3) & ~(size_t)3;
  if (words > filter.bytes / 4 && !filter.alloc(words * 4)) return false;
  filter_words = words;
  return true;
}

static bool grid_fits_u32(const int g[3]) {
  if (g[0] <= 0 || g[1] <= 0 || g[2] <= 0) return false;
  const uint64_t vol = (uint64_t)g[0] * (uint64_t)g[1] * (uint64_t)g[2];
  return vol < 0xFFFFFFFFull;
}

int hash_build(const CoordTable& t, const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3],
               uint32_t* n_eff_out, hipStream_t stream) {
  SCN_REQUIRE(t.cap >= hash_capacity_for(n), SCN_ERR_CAPACITY, "hash table capacity %zu too small for %u rows",
              t.cap, n);
  SCN_REQUIRE(grid_fits_u32(grid), SCN_ERR_UNSUPPORTED, "grid %dx%dx%d does not fit 32-bit keys", grid[0], grid[1],
              grid[2]);
  const_cast<CoordTable&>(t).mask = (uint32_t)(hash_capacity_for(n) - 1);
  int rc = SCN_OK;
  if (t.precleared_for != n) {  // not already cleared (for exactly this size) by the caller's batched fill
    rc = fill_u32(t.slots(), 0xFFFFFFFFu, ((size_t)t.mask + 1) * 2, stream);
    if (rc) return rc;
    if (t.filter_words) {
      rc = fill_u32(t.filter.p, 0u, t.filter_words, stream);
      if (rc) return rc;
    }
  }
  const_cast<CoordTable&>(t).precleared_for = 0xFFFFFFFFu;
  Int3 g{{grid[0], grid[1], grid[2]}};
  const uint32_t blocks = n ? ceil_div(n, 256) : 1;
  hipLaunchKernelGGL(k_hash_insert, dim3(blocks), dim3(256), 0, stream, t.slots(), t.mask,
                     (const int4*)idx, n, n_dev, g, n_eff_out, t.filter_words ? t.filter.as<uint32_t>() : nullptr);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

int hash_query(const CoordTable& t, const int32_t* coords, uint32_t n, const int grid[3], int32_t* rows,
               hipStream_t stream) {
  if (n == 0) return SCN_OK;
  Int3 g{{grid[0], grid[1], grid[2]}};
  hipLaunchKernelGGL(k_hash_query, dim3(ceil_div(n, 256)), dim3(256), 0, stream, t.slots(), t.mask,
                     (const int4*)coords, n, g, rows);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// bitmap rank: block sums, scan of block sums, expansion
// one block = 256 threads x 4 words = 1024 bitmap words
// --------------------------------------------------------------------------------------------
constexpr uint32_t kWordsPerBlock = 1024;

__global__ __launch_bounds__(256) void k_bitmap_blocksum(const uint32_t* __restrict__ bitmap, uint32_t* blocksum) {
  __shared__ uint32_t scratch[17];
  const uint4 w = reinterpret_cast<const uint4*>(bitmap)[(size_t)blockIdx.x * 256 + threadIdx.x];
  uint32_t c = __popc(w.x) + __popc(w.y) + __popc(w.z) + __popc(w.w);
  uint32_t total;
  (void)block_exclusive_scan(c, scratch, &total);
  if (threadIdx.x == 0) blocksum[blockIdx.x] = total;
}

// Single block: in-place exclusive scan of `count` values; counters[1] = total, counters[0] = min(total, cap).
__global__ __launch_bounds__(1024) void k_scan_blocksums(uint32_t* vals, uint32_t count, uint32_t* counters,
                                                        uint32_t cap) {
  __shared__ uint32_t scratch[17];
  uint32_t carry = 0;
  for (uint32_t base = 0; base < count; base += 1024) {
    const uint32_t i = base + threadIdx.x;
    const uint32_t x = i < count ? vals[i] : 0;
    uint32_t total;
    const uint32_t ex = block_exclusive_scan(x, scratch, &total);
    if (i < count) vals[i] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0 && counters) {
    counters[1] = carry;
    counters[0] = carry < cap ? carry : cap;
  }
}

// Sparse bitmaps (fewer set bits than words): one thread per word expands its bits in rank order.
// Optional outputs: coordinate rows and the per-word exclusive prefix (rank of the word's first bit),
// which together with the bitmap answers "row of this cell" (see coord_row).
// Block = 1024 threads = 1024 words.  blockoff holds either the exclusive scan of the per-block counts
// (raw_sums = 0) or the counts themselves (raw_sums = 1: every block adds up the counts before it, and
// the last block publishes the totals in counters -- one launch less than a separate scan).
__global__ __launch_bounds__(1024) void k_bitmap_expand(const uint32_t* __restrict__ bitmap,
                                                        const uint32_t* __restrict__ blockoff, Int3 grid, uint32_t cap,
                                                        int4* coords_out, uint32_t* prefix_out, int raw_sums,
                                                        uint32_t* counters) {
  __shared__ uint32_t scratch[17];
  const size_t t = (size_t)blockIdx.x * 1024 + threadIdx.x;
  uint32_t bits = bitmap[t];
  const uint32_t c = __popc(bits);
  uint32_t base;
  if (raw_sums) {
    uint32_t part = 0;
    for (uint32_t i = threadIdx.x; i < blockIdx.x; i += 1024) part += blockoff[i];
    (void)block_exclusive_scan(part, scratch, &base);
  } else {
    base = blockoff[blockIdx.x];
  }
  uint32_t total;
  uint32_t rank = base + block_exclusive_scan(c, scratch, &total);
  if (raw_sums && counters && blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
    const uint32_t all = base + total;
    counters[1] = all;
    counters[0] = all < cap ? all : cap;
  }
  if (prefix_out) prefix_out[t] = rank;
  if (c == 0 || coords_out == nullptr) return;
  const uint32_t g12 = (uint32_t)grid.v[1] * (uint32_t)grid.v[2];
  while (bits) {
    const int b = __ffs(bits) - 1;
    bits &= bits - 1;
    if (rank < cap) {
      const uint32_t key = (uint32_t)t * 32u + (uint32_t)b;
      const uint32_t i0 = key / g12, rem = key - i0 * g12;
      const uint32_t i1 = rem / (uint32_t)grid.v[2], i2 = rem - i1 * (uint32_t)grid.v[2];
      coords_out[rank] = make_int4(0, (int)i0, (int)i1, (int)i2);
    }
    rank++;
  }
}

// Dense bitmaps: one thread per cell, rank = prefix of its word + set bits below it.
__global__ __launch_bounds__(256) void k_expand_cells(const uint32_t* __restrict__ bitmap,
                                                      const uint32_t* __restrict__ prefix, uint32_t cells, Int3 grid,
                                                      uint32_t cap, int4* coords_out) {
  const uint32_t key = blockIdx.x * 256 + threadIdx.x;
  if (key >= cells) return;
  const uint32_t w = bitmap[key >> 5], b = key & 31;
  if (!((w >> b) & 1u)) return;
  const uint32_t rank = prefix[key >> 5] + __popc(w & ((1u << b) - 1u));
  if (rank >= cap) return;
  const uint32_t g12 = (uint32_t)grid.v[1] * (uint32_t)grid.v[2];
  const uint32_t i0 = key / g12, rem = key - i0 * g12;
  const uint32_t i1 = rem / (uint32_t)grid.v[2], i2 = rem - i1 * (uint32_t)grid.v[2];
  coords_out[rank] = make_int4(0, (int)i0, (int)i1, (int)i2);
}

static size_t bitmap_words_for(const int g[3]) {
  const uint64_t vol = (uint64_t)g[0] * g[1] * g[2];
  const uint64_t words = (vol + 31) / 32;
  return (size_t)((words + kWordsPerBlock - 1) / kWordsPerBlock * kWordsPerBlock);
}

// --------------------------------------------------------------------------------------------
// rulebooks
// --------------------------------------------------------------------------------------------
struct GeomDev {
  int gi[3], go[3], ks[3], st[3], pd[3], dl[3];
};

static GeomDev to_dev(const ConvGeom& g) {
  GeomDev d;
  for (int a = 0; a < 3; ++a) {
    d.gi[a] = g.grid_in[a];
    d.go[a] = g.grid_out[a];
    d.ks[a] = g.ks[a];
    d.st[a] = g.stride[a];
    d.pd[a] = g.pad[a];
    d.dl[a] = g.dil[a];
  }
  return d;
}

// Row of the voxel with linear index `key` in a tensor described by `lk`: a probe of the coordinate
// hash (tensors in caller order), or rank = prefix[word] + popcount(bits below) in the occupancy
// bitmap of a tensor whose rows are in canonical order (outputs of strided convolutions): two
// independent loads, no probing loop.
__device__ __forceinline__ int32_t coord_row(const CoordLookup& lk, uint32_t key) {
  if (lk.bitmap) {
    const uint32_t w = lk.bitmap[key >> 5], b = key & 31;
    if (!((w >> b) & 1u)) return -1;
    const uint32_t r = lk.prefix[key >> 5] + __popc(w & ((1u << b) - 1u));
    return r < lk.rank_cap ? (int32_t)r : -1;
  }
  if (lk.filter && !((lk.filter[key >> 5] >> (key & 31)) & 1u)) return -1;
  return table_lookup(lk.slots, lk.mask, key);
}

// nbr[k][o] = row of the input at  o*stride - pad + k*dilation  (or -1).  grid.y = k0; a thread
// walks the K1*K2 offsets of its k0 plane (independent lookups, coalesced stores per offset).
// Used for both kinds: submanifold passes stride 1 and pad = floor(K/2)*dilation.
// Thread (0,0) also publishes the row count for the kernels that follow (n_publish, nullable).
__global__ __launch_bounds__(256) void k_build_nbr(const int4* __restrict__ out_coords, const uint32_t* n_out_dev,
                                                   uint32_t n_bound, GeomDev g, CoordLookup lk, int32_t* nbr,
                                                   uint32_t ld, int identity_center, uint32_t* n_publish,
                                                   uint32_t* n_host) {
  const uint32_t n = eff_n(n_out_dev, n_bound);
  const uint32_t o = blockIdx.x * 256 + threadIdx.x;
  if (o == 0 && blockIdx.y == 0) {
    if (n_publish) {
      n_publish[0] = n;
      n_publish[1] = n;
    }
    if (n_host) *n_host = n;  // pinned host word: the row count as a launch hint for the next forward
  }
  if (o >= n) return;
  const int k0 = blockIdx.y;
  const int4 c = out_coords[o];
  const int i0 = c.y * g.st[0] - g.pd[0] + k0 * g.dl[0];
  const bool ok0 = c.x == 0 && i0 >= 0 && i0 < g.gi[0];
  const bool centre0 = identity_center && k0 == g.ks[0] / 2;
  for (int k1 = 0; k1 < g.ks[1]; ++k1) {
    const int i1 = c.z * g.st[1] - g.pd[1] + k1 * g.dl[1];
    const bool ok1 = ok0 && i1 >= 0 && i1 < g.gi[1];
    const uint32_t line = ((uint32_t)i0 * (uint32_t)g.gi[1] + (uint32_t)i1) * (uint32_t)g.gi[2];
#pragma unroll 3
    for (int k2 = 0; k2 < g.ks[2]; ++k2) {
      const int i2 = c.w * g.st[2] - g.pd[2] + k2 * g.dl[2];
      int32_t res = -1;
      if (centre0 && k1 == g.ks[1] / 2 && k2 == g.ks[2] / 2) {
        res = (int32_t)o;
      } else if (ok1 && i2 >= 0 && i2 < g.gi[2]) {
        res = coord_row(lk, line + (uint32_t)i2);
      }
      nbr[(size_t)((k0 * g.ks[1] + k1) * g.ks[2] + k2) * ld + o] = res;
    }
  }
}

// Marks every output cell reached by an input row through some kernel offset.  One thread per
// input row; per axis the (at most K) reachable output coordinates are found first, then their
// combinations are marked -- the bits of one output line that fall into the same word in one
// operation, through the workgroup's LDS aggregation (see agg_or).
__global__ __launch_bounds__(256) void k_mark_outputs(const int4* __restrict__ in_coords, const uint32_t* n_dev,
                                                      uint32_t n_bound, GeomDev g, uint32_t* bitmap) {
  __shared__ uint32_t akeys[kAggSlots], avals[kAggSlots];
  agg_init(akeys, avals);
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t r = blockIdx.x * 256 + threadIdx.x;
  int4 c = make_int4(-1, 0, 0, 0);
  if (r < n) c = in_coords[r];
  if (c.x == 0 && c.y >= 0 && c.y < g.gi[0] && c.z >= 0 && c.z < g.gi[1] && c.w >= 0 && c.w < g.gi[2]) {
    const int cc[3] = {c.y, c.z, c.w};
    constexpr int kMaxK = 8;  // per-axis kernel sizes are limited to 8 by the host checks
    int o[3][kMaxK];
    int cnt[3] = {0, 0, 0};
#pragma unroll
    for (int a = 0; a < 3; ++a) {
      const int ks = g.ks[a] < kMaxK ? g.ks[a] : kMaxK;
      for (int k = 0; k < ks; ++k) {
        const int t = cc[a] + g.pd[a] - k * g.dl[a];
        if (t < 0) continue;
        const int q = t / g.st[a];
        if (q * g.st[a] != t || q >= g.go[a]) continue;
        o[a][cnt[a]++] = q;
      }
    }
    for (int a0 = 0; a0 < cnt[0]; ++a0)
      for (int a1 = 0; a1 < cnt[1]; ++a1) {
        const uint32_t line = ((uint32_t)o[0][a0] * (uint32_t)g.go[1] + (uint32_t)o[1][a1]) * (uint32_t)g.go[2];
        uint32_t word = kAggEmpty, bits = 0;
        for (int a2 = 0; a2 < cnt[2]; ++a2) {
          const uint32_t key = line + (uint32_t)o[2][a2];
          if ((key >> 5) != word) {
            if (bits) agg_or(akeys, avals, bitmap, word, bits);
            word = key >> 5;
            bits = 0;
          }
          bits |= 1u << (key & 31);
        }
        if (bits) agg_or(akeys, avals, bitmap, word, bits);
      }
  }
  agg_flush(akeys, avals, bitmap);
}

// Row count of the previous build as seen by the host (0 before the first one has run): a hint for
// launch configuration only, never used for bounds.
uint32_t Rulebook::n_out_hint() const {
  if (!host_count.p) return n_bound_out;
  const uint32_t v = *reinterpret_cast<const volatile uint32_t*>(host_count.p);
  return v == 0 || v > n_bound_out ? n_bound_out : v;
}

bool Rulebook::init(uint32_t max_in_, uint32_t max_out_, int kvol) {
  if (!host_count.alloc(16)) return false;
  memset(host_count.p, 0, 16);
  max_in = max_in_;
  max_out = max_out_;
  kvol_cap = kvol;
  ld = (std::max(max_in, max_out) + 63u) & ~63u;
  if (ld == 0) ld = 64;
  if (!nbr.alloc((size_t)kvol * ld * sizeof(int32_t))) return false;
  if (!counters.alloc(64 * sizeof(uint32_t))) return false;
  if (hipMemset(counters.p, 0, 64 * sizeof(uint32_t)) != hipSuccess) return false;
  return true;
}

static int check_geom(const int ks[3], const int st[3], const int dl[3], int kvol_cap) {
  for (int a = 0; a < 3; ++a)
    SCN_REQUIRE(ks[a] >= 1 && ks[a] <= 8 && st[a] >= 1 && dl[a] >= 1, SCN_ERR_INVALID,
                "kernel size must be 1..8, stride and dilation >= 1");
  SCN_REQUIRE(ks[0] * ks[1] * ks[2] <= kvol_cap, SCN_ERR_CAPACITY, "kernel volume %d exceeds the rulebook's %d",
              ks[0] * ks[1] * ks[2], kvol_cap);
  return SCN_OK;
}

__global__ void k_set_count(uint32_t* dst, const uint32_t* n_dev, uint32_t n_bound) {
  if (threadIdx.x == 0 && blockIdx.x == 0) {
    const uint32_t n = eff_n(n_dev, n_bound);
    dst[0] = n;
    dst[1] = n;
  }
}

int set_count(uint32_t* dst, const uint32_t* n_dev, uint32_t n_bound, hipStream_t stream) {
  hipLaunchKernelGGL(k_set_count, dim3(1), dim3(64), 0, stream, dst, n_dev, n_bound);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

static int launch_build_nbr(const Rulebook& rb, const int32_t* out_coords, const uint32_t* n_dev, uint32_t n_bound,
                            bool identity_center, uint32_t* n_publish, hipStream_t stream) {
  const uint32_t blocks = n_bound ? ceil_div(n_bound, 256) : 1;  // one block even when empty: it publishes the count
  hipLaunchKernelGGL(k_build_nbr, dim3(blocks, rb.geom.ks[0]), dim3(256), 0, stream, (const int4*)out_coords, n_dev,
                     n_bound, to_dev(rb.geom), rb.in_lookup, rb.nbr.as<int32_t>(), rb.ld, identity_center ? 1 : 0,
                     n_publish, rb.host_count.as<uint32_t>());
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

CoordLookup CoordTable::lookup() const {
  CoordLookup lk;
  lk.slots = slots();
  lk.mask = mask;
  lk.filter = filter_words ? filter.as<uint32_t>() : nullptr;
  return lk;
}

CoordLookup Rulebook::out_lookup() const {
  CoordLookup lk;
  lk.bitmap = bitmap.as<uint32_t>();
  lk.prefix = prefix.as<uint32_t>();
  lk.rank_cap = n_bound_out;
  return lk;
}

int Rulebook::build_subm(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3], const int ks[3],
                         const int dil[3], const CoordLookup* shared_lookup, hipStream_t stream) {
  const int one[3] = {1, 1, 1};
  int rc = check_geom(ks, one, dil, kvol_cap);
  if (rc) return rc;
  SCN_REQUIRE(n <= max_in && n <= ld, SCN_ERR_CAPACITY, "submanifold rulebook: %u rows exceed capacity %u", n, max_in);
  SCN_REQUIRE(grid_fits_u32(grid), SCN_ERR_UNSUPPORTED, "grid %dx%dx%d does not fit 32-bit keys", grid[0], grid[1],
              grid[2]);
  subm = true;
  for (int a = 0; a < 3; ++a) {
    geom.grid_in[a] = geom.grid_out[a] = grid[a];
    geom.ks[a] = ks[a];
    geom.stride[a] = 1;
    geom.dil[a] = dil[a];
    geom.pad[a] = (ks[a] / 2) * dil[a];
  }
  geom.kvol = ks[0] * ks[1] * ks[2];
  in_indices = out_indices = idx;
  n_bound_in = n_bound_out = n;
  uint32_t* cnt = counters.as<uint32_t>();
  if (shared_lookup) {
    in_lookup = *shared_lookup;
  } else {
    rc = reserve_subm(true);
    if (rc) return rc;
    if (!own_in_table.alloc_filter(grid)) return SCN_ERR_HIP;
    rc = hash_build(own_in_table, idx, n, n_dev, grid, nullptr, stream);
    if (rc) return rc;
    in_lookup = own_in_table.lookup();
  }
  const bool odd = (ks[0] & 1) && (ks[1] & 1) && (ks[2] & 1);
  rc = launch_build_nbr(*this, idx, n_dev, n, odd, cnt, stream);
  if (rc) return rc;
  built = true;
  return SCN_OK;
}

// Allocates what a strided build needs for the given output grid (no-op when already large enough),
// so that a later build only launches kernels.
int Rulebook::reserve_sparse(const int out_grid[3], bool need_own_in_table) {
  const size_t words = bitmap_words_for(out_grid);
  if (words > bitmap_cap_words) {
    if (!bitmap.alloc(words * 4)) return SCN_ERR_HIP;
    if (!blocksum.alloc((words / kWordsPerBlock + 2) * 4)) return SCN_ERR_HIP;
    if (!prefix.alloc(words * 4)) return SCN_ERR_HIP;
    bitmap_cap_words = words;
  }
  bitmap_words = words;
  if (out_idx.bytes < (size_t)std::max(max_out, 1u) * 16 && !out_idx.alloc((size_t)std::max(max_out, 1u) * 16))
    return SCN_ERR_HIP;
  if (need_own_in_table && own_in_table.cap < hash_capacity_for(max_in) && !own_in_table.alloc_for(max_in))
    return SCN_ERR_HIP;
  return SCN_OK;
}

int Rulebook::reserve_subm(bool need_own_in_table) {
  if (need_own_in_table && own_in_table.cap < hash_capacity_for(max_in) && !own_in_table.alloc_for(max_in))
    return SCN_ERR_HIP;
  return SCN_OK;
}

int Rulebook::build_sparse(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3], const int ks[3],
                           const int stride[3], const int pad[3], const int dil[3],
                           const CoordLookup* shared_lookup, hipStream_t stream) {
  int rc = check_geom(ks, stride, dil, kvol_cap);
  if (rc) return rc;
  SCN_REQUIRE(n <= max_in, SCN_ERR_CAPACITY, "sparse rulebook: %u rows exceed capacity %u", n, max_in);
  SCN_REQUIRE(grid_fits_u32(grid), SCN_ERR_UNSUPPORTED, "grid %dx%dx%d does not fit 32-bit keys", grid[0], grid[1],
              grid[2]);
  subm = false;
  for (int a = 0; a < 3; ++a) {
    SCN_REQUIRE(pad[a] >= 0, SCN_ERR_INVALID, "negative padding");
    geom.grid_in[a] = grid[a];
    geom.ks[a] = ks[a];
    geom.stride[a] = stride[a];
    geom.dil[a] = dil[a];
    geom.pad[a] = pad[a];
    geom.grid_out[a] = (grid[a] + 2 * pad[a] - dil[a] * (ks[a] - 1) - 1) / stride[a] + 1;
    SCN_REQUIRE(geom.grid_out[a] >= 1, SCN_ERR_INVALID, "convolution output size < 1 on axis %d", a);
  }
  SCN_REQUIRE(grid_fits_u32(geom.grid_out), SCN_ERR_UNSUPPORTED, "output grid does not fit 32-bit keys");
  geom.kvol = ks[0] * ks[1] * ks[2];
  in_indices = idx;
  n_bound_in = n;
  // host-side bound of the number of outputs
  {
    const uint64_t vol = (uint64_t)geom.grid_out[0] * geom.grid_out[1] * geom.grid_out[2];
    uint64_t b = std::min<uint64_t>((uint64_t)n * (uint64_t)geom.kvol, vol);
    n_bound_out = (uint32_t)std::min<uint64_t>(b, max_out);
  }
  rc = reserve_sparse(geom.grid_out, shared_lookup == nullptr);
  if (rc) return rc;
  const size_t words = bitmap_words;
  out_indices = out_idx.as<int32_t>();
  uint32_t* cnt = counters.as<uint32_t>();
  if (shared_lookup) {
    in_lookup = *shared_lookup;
  } else {
    if (!own_in_table.alloc_filter(grid)) return SCN_ERR_HIP;
    rc = hash_build(own_in_table, idx, n, n_dev, grid, nullptr, stream);
    if (rc) return rc;
    in_lookup = own_in_table.lookup();
  }
  // occupancy bitmap of the outputs -> ordered unique output coordinates + per-word ranks
  if (!bitmap_precleared) {
    rc = fill_u32(bitmap.p, 0u, words, stream);
    if (rc) return rc;
  }
  bitmap_precleared = false;
  const GeomDev gd = to_dev(geom);
  if (n) {
    hipLaunchKernelGGL(k_mark_outputs, dim3(ceil_div(n, 256)), dim3(256), 0, stream, (const int4*)idx, n_dev, n, gd,
                       bitmap.as<uint32_t>());
  }
  const uint32_t nblocks = (uint32_t)(words / kWordsPerBlock);
  hipLaunchKernelGGL(k_bitmap_blocksum, dim3(nblocks), dim3(256), 0, stream, bitmap.as<uint32_t>(),
                     blocksum.as<uint32_t>());
  // up to a few thousand blocks every expand block adds up the counts before it itself
  const int raw = nblocks <= 8192 ? 1 : 0;
  if (!raw)
    hipLaunchKernelGGL(k_scan_blocksums, dim3(1), dim3(1024), 0, stream, blocksum.as<uint32_t>(), nblocks, cnt,
                       n_bound_out);
  const Int3 og{{geom.grid_out[0], geom.grid_out[1], geom.grid_out[2]}};
  const uint64_t cells = (uint64_t)geom.grid_out[0] * geom.grid_out[1] * geom.grid_out[2];
  if (cells <= 32ull * std::max(n_bound_out, 1u)) {
    // dense output grid: per-word ranks, then one thread per cell
    hipLaunchKernelGGL(k_bitmap_expand, dim3(nblocks), dim3(1024), 0, stream, bitmap.as<uint32_t>(),
                       blocksum.as<uint32_t>(), og, n_bound_out, (int4*)nullptr, prefix.as<uint32_t>(), raw, cnt);
    hipLaunchKernelGGL(k_expand_cells, dim3((unsigned)((cells + 255) / 256)), dim3(256), 0, stream,
                       bitmap.as<uint32_t>(), prefix.as<uint32_t>(), (uint32_t)cells, og, n_bound_out, (int4*)out_idx.p);
  } else {
    hipLaunchKernelGGL(k_bitmap_expand, dim3(nblocks), dim3(1024), 0, stream, bitmap.as<uint32_t>(),
                       blocksum.as<uint32_t>(), og, n_bound_out, (int4*)out_idx.p, prefix.as<uint32_t>(), raw, cnt);
  }
  SCN_HIP(hipGetLastError());
  rc = launch_build_nbr(*this, out_indices, cnt, n_bound_out, false, nullptr, stream);
  if (rc) return rc;
  built = true;
  return SCN_OK;
}

// ---- inverse rulebook ---------------------------------------------------------------------------
// SparseInverseConvolution runs on the rulebook of an earlier strided convolution with the roles
// swapped: its outputs are that convolution's inputs.  For a fixed kernel offset an input row has at
// most one output row (o = (i + pad - k dil) / stride), so the swapped rulebook is again a neighbour
// table: inv[k][i] = o where fwd[k][o] = i.  grid.y = kernel offset.
__global__ __launch_bounds__(256) void k_invert_nbr(const int32_t* __restrict__ fwd, uint32_t fwd_ld,
                                                    const uint32_t* n_fwd_out_dev, uint32_t n_fwd_out_bound,
                                                    int32_t* inv, uint32_t inv_ld, const uint32_t* n_in_dev,
                                                    uint32_t n_in_bound, uint32_t* n_publish, uint32_t* n_host) {
  const uint32_t n_out = eff_n(n_fwd_out_dev, n_fwd_out_bound);
  const uint32_t n_in = eff_n(n_in_dev, n_in_bound);
  const uint32_t o = blockIdx.x * 256 + threadIdx.x;
  if (o == 0 && blockIdx.y == 0) {
    n_publish[0] = n_in;
    n_publish[1] = n_in;
    if (n_host) *n_host = n_in;
  }
  if (o >= n_out) return;
  const int32_t i = fwd[(size_t)blockIdx.y * fwd_ld + o];
  if (i >= 0 && (uint32_t)i < n_in) inv[(size_t)blockIdx.y * inv_ld + (uint32_t)i] = (int32_t)o;
}

__global__ __launch_bounds__(256) void k_fill_table_rows(int32_t* table, uint32_t ld, uint32_t n, int32_t value) {
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) table[(size_t)blockIdx.y * ld + i] = value;
}

int Rulebook::build_inverse(const Rulebook& fwd, const uint32_t* n_in_dev, hipStream_t stream) {
  SCN_REQUIRE(fwd.built && !fwd.subm, SCN_ERR_INVALID, "inverse rulebook: needs a built strided rulebook");
  SCN_REQUIRE(fwd.geom.kvol <= kvol_cap, SCN_ERR_CAPACITY, "inverse rulebook: kernel volume %d exceeds %d",
              fwd.geom.kvol, kvol_cap);
  SCN_REQUIRE(fwd.n_bound_in <= max_out && fwd.n_bound_in <= ld && fwd.n_bound_out <= max_in, SCN_ERR_CAPACITY,
              "inverse rulebook: %u x %u rows exceed capacity %u x %u", fwd.n_bound_out, fwd.n_bound_in, max_in, max_out);
  subm = false;
  geom = fwd.geom;
  for (int a = 0; a < 3; ++a) {
    geom.grid_in[a] = fwd.geom.grid_out[a];
    geom.grid_out[a] = fwd.geom.grid_in[a];
  }
  in_indices = fwd.out_indices;
  out_indices = fwd.in_indices;
  n_bound_in = fwd.n_bound_out;
  n_bound_out = fwd.n_bound_in;
  // every offset's row of the table, up to the row bound, starts as "no neighbour"
  if (n_bound_out)
    hipLaunchKernelGGL(k_fill_table_rows, dim3(ceil_div(n_bound_out, 256), geom.kvol), dim3(256), 0, stream,
                       nbr.as<int32_t>(), ld, n_bound_out, -1);
  const uint32_t blocks = n_bound_in ? ceil_div(n_bound_in, 256) : 1;  // one block even when empty: it publishes the count
  hipLaunchKernelGGL(k_invert_nbr, dim3(blocks, geom.kvol), dim3(256), 0, stream, fwd.nbr.as<int32_t>(), fwd.ld,
                     fwd.n_out_dev(), fwd.n_bound_out, nbr.as<int32_t>(), ld, n_in_dev, n_bound_out,
                     counters.as<uint32_t>(), host_count.as<uint32_t>());
  SCN_HIP(hipGetLastError());
  built = true;
  return SCN_OK;
}

// ---- pair compaction: nbr[k][o] -> (in,out) lists per offset, ordered by (k, out) -------------
__global__ __launch_bounds__(256) void k_pair_count(const int32_t* __restrict__ nbr, uint32_t ld,
                                                    const uint32_t* n_out_dev, uint32_t n_bound, uint32_t* counts) {
  __shared__ uint32_t wsum[4];
  const uint32_t n = eff_n(n_out_dev, n_bound);
  const uint32_t o = blockIdx.x * 256 + threadIdx.x;
  const bool valid = o < n && nbr[(size_t)blockIdx.y * ld + o] >= 0;
  const uint64_t m = __ballot(valid);
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = (uint32_t)__popcll(m);
  __syncthreads();
  if (threadIdx.x == 0) counts[blockIdx.y * gridDim.x + blockIdx.x] = wsum[0] + wsum[1] + wsum[2] + wsum[3];
}

__global__ __launch_bounds__(256) void k_pair_write(const int32_t* __restrict__ nbr, uint32_t ld,
                                                    const uint32_t* n_out_dev, uint32_t n_bound,
                                                    const uint32_t* __restrict__ block_off, const uint32_t* total,
                                                    int32_t* pair_in, int32_t* pair_out, int64_t* offsets,
                                                    uint64_t capacity) {
  __shared__ uint32_t wsum[4];
  const uint32_t n = eff_n(n_out_dev, n_bound);
  const uint32_t o = blockIdx.x * 256 + threadIdx.x;
  int32_t in = -1;
  if (o < n) in = nbr[(size_t)blockIdx.y * ld + o];
  const bool valid = in >= 0;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint64_t m = __ballot(valid);  // wavefront ballot
  const uint32_t below = (uint32_t)__popcll(m & ((1ull << lane) - 1ull));  // prefix inside the wavefront
  if (lane == 0) wsum[wave] = (uint32_t)__popcll(m);
  __syncthreads();
  uint32_t wbase = 0;
  for (int w = 0; w < wave; ++w) wbase += wsum[w];
  const uint32_t base = block_off[blockIdx.y * gridDim.x + blockIdx.x];
  if (valid) {
    const uint64_t pos = (uint64_t)base + wbase + below;
    if (pos < capacity) {
      pair_in[pos] = in;
      pair_out[pos] = (int32_t)o;
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    offsets[blockIdx.y] = base;
    if (blockIdx.y == gridDim.y - 1) offsets[gridDim.y] = total[1];
  }
}

int Rulebook::pairs(int32_t* pair_in, int32_t* pair_out, int64_t* offsets, uint64_t capacity, hipStream_t stream) {
  SCN_REQUIRE(built, SCN_ERR_INVALID, "rulebook has not been built");
  const uint32_t nb = std::max(1u, ceil_div(n_bound_out, 256));
  const size_t need = ((size_t)nb * geom.kvol + 8) * 4;
  if (pair_scratch.bytes < need && !pair_scratch.alloc(need)) return SCN_ERR_HIP;
  uint32_t* counts = pair_scratch.as<uint32_t>();
  uint32_t* total = counters.as<uint32_t>() + 8;
  hipLaunchKernelGGL(k_pair_count, dim3(nb, geom.kvol), dim3(256), 0, stream, nbr.as<int32_t>(), ld, n_out_dev(),
                     n_bound_out, counts);
  hipLaunchKernelGGL(k_scan_blocksums, dim3(1), dim3(1024), 0, stream, counts, nb * (uint32_t)geom.kvol, total,
                     0xFFFFFFFFu);
  hipLaunchKernelGGL(k_pair_write, dim3(nb, geom.kvol), dim3(256), 0, stream, nbr.as<int32_t>(), ld, n_out_dev(),
                     n_bound_out, counts, total, pair_in, pair_out, offsets, capacity);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// gather-GEMM convolution
// --------------------------------------------------------------------------------------------
// Operand mapping of v_mfma_i32_16x16x64_i8 / v_mfma_f32_16x16x32_f16 (D = A x B + C, wave64):
//   A (16 x K): lane l supplies row  m = l % 16, the 16 bytes of K-block l / 16
//   B (K x 16): lane l supplies col  n = l % 16, the 16 bytes of K-block l / 16
//   D (16 x 16): lane l holds col n = l % 16, rows m = 4 * (l / 16) + {0,1,2,3}
// Rows of A are output channels (weights, pre-packed on the host in exactly this order), columns of
// B are voxels: the 16 bytes a lane needs are 16 contiguous input channels of one gathered row, so
// a gathered row goes from memory straight into the MFMA operand with one 16-byte load, and each
// lane ends up with 4 consecutive output channels of one voxel, stored with one 4/8-byte store.
// One 16-byte "chunk" = 16 int8 or 8 fp16 input channels; K-step s consumes chunks 4s..4s+3 of the
// sequence (offset 0 chunk 0, offset 0 chunk 1, ..., offset kvol-1 chunk CHUNKS-1).
struct ConvArgs {
  const char* x;
  uint32_t x_ld_bytes;
  const int32_t* nbr;
  uint32_t nbr_ld;
  int kvol;
  const uint32_t* n_out_dev;
  uint32_t n_bound;
  const uint4* wfrag;
  int steps;
  const float* wscale;
  const float* bias;
  int cout;
  float x_scale;            // amax_x / 127
  int relu;
  int out_dtype;
  float out_r;              // 127 / amax_out
  char* out;
  uint32_t out_ld;
  void* acc;
  const char* res;
  int res_dtype;
  float res_scale;          // amax_res / 127
  uint32_t res_ld;
  int mid_dtype;
  float mid_s, mid_r;       // amax_mid / 127, 127 / amax_mid
  float a_rq_s, a_rq_r;     // re-quantisation of an fp16 operand by an int8 Add (0 = none)
  float b_rq_s, b_rq_r;
  int relu2;
  int out_vec16;     // output rows are 16-byte aligned and a multiple of 16 bytes: 16-byte stores allowed
  const char* zrow;  // 512 bytes of zeros (gather source of lanes without a neighbour), then 64 words of -1
};

// int8 store of the fake-quant form: round(y * (127/amax)), saturated to +-127
__device__ __forceinline__ float quant_f(float y, float r) {
  float q = rintf(y * r);
  q = fminf(fmaxf(q, -127.f), 127.f);  // NaN -> -127 (fmaxf returns the non-NaN operand)
  return q;
}

__device__ __forceinline__ float half_round(float y) { return (float)(_Float16)y; }

template <int EL>
struct Mma;
template <>
struct Mma<0> {
  using Acc = v4i;
  static __device__ __forceinline__ Acc run(const v4i a, const v4i b, Acc c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ Acc run(const uint4& a, const uint4& b, Acc c) {
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(__builtin_bit_cast(v4i, a), __builtin_bit_cast(v4i, b), c, 0, 0, 0);
  }
};
template <>
struct Mma<1> {
  using Acc = v4f;
  static __device__ __forceinline__ Acc run(const v4i a, const v4i b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ Acc run(const uint4& a, const uint4& b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};

// Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2.  Giving XCD x the
// x-th contiguous eighth of the row tiles keeps the rows a tile gathers (spatial neighbours, i.e.
// nearby rows in canonical order) inside one L2 instead of spreading every row over all eight.
// Returns false when this workgroup has no tile.
__device__ __forceinline__ bool xcd_tile(uint32_t n, uint32_t rows_per_block, uint32_t* tile) {
  const uint32_t tiles = (n + rows_per_block - 1) / rows_per_block;
  const uint32_t per = (tiles + 7) >> 3;
  const uint32_t xcd = blockIdx.x & 7, j = blockIdx.x >> 3;
  *tile = xcd * per + j;
  return j < per && *tile < tiles;
}

// Fused epilogue of 4 consecutive channels of one row: bias, requantisation scale, ReLU, residual add
// (with the mid-quantisation the un-fused graph would have applied), second ReLU.  Also dumps the raw
// accumulators when asked to.  y[] receives the values to store.
template <int EL>
__device__ __forceinline__ void epilogue_values(const ConvArgs& a, uint32_t row, int co,
                                                const typename Mma<EL>::Acc& acc, float y[4]) {
  const float4 bs = *reinterpret_cast<const float4*>(a.bias + co);
  const float b4[4] = {bs.x, bs.y, bs.z, bs.w};
  if (EL == 0) {
    const float4 ws = *reinterpret_cast<const float4*>(a.wscale + co);
    const float w4[4] = {ws.x, ws.y, ws.z, ws.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float sc = a.x_scale * w4[j];         // s_x * s_w[c], one fp32 rounding
      const float m = (float)acc[j] * sc;          // fp32 multiply
      y[j] = m + b4[j];                            // fp32 add (the library is built with -ffp-contract=off)
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) y[j] = (float)acc[j] + b4[j];
  }
  if (a.acc) {
    if (EL == 0)
      *reinterpret_cast<v4i*>((int32_t*)a.acc + (size_t)row * a.cout + co) = __builtin_bit_cast(v4i, acc);
    else
      *reinterpret_cast<v4f*>((float*)a.acc + (size_t)row * a.cout + co) = __builtin_bit_cast(v4f, acc);
  }
  if (a.relu) {
#pragma unroll
    for (int j = 0; j < 4; ++j) y[j] = y[j] > 0.f ? y[j] : 0.f;
  }
  if (a.res) {
    // value of the un-fused conv output as its consumer (the Add) would have read it
    float rv[4];
    if (a.res_dtype == SCN_DTYPE_INT8) {
      const char4 r = *reinterpret_cast<const char4*>(a.res + (size_t)row * a.res_ld + co);
      rv[0] = (float)r.x * a.res_scale;
      rv[1] = (float)r.y * a.res_scale;
      rv[2] = (float)r.z * a.res_scale;
      rv[3] = (float)r.w * a.res_scale;
    } else {
      const _Float16* r = reinterpret_cast<const _Float16*>(a.res) + (size_t)row * a.res_ld + co;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rv[j] = (float)r[j];
        if (a.b_rq_r > 0.f) rv[j] = quant_f(rv[j], a.b_rq_r) * a.b_rq_s;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v;
      if (a.mid_dtype == SCN_DTYPE_INT8) {
        v = quant_f(y[j], a.mid_r) * a.mid_s;
      } else {
        v = half_round(y[j]);
        if (a.a_rq_r > 0.f) v = quant_f(v, a.a_rq_r) * a.a_rq_s;
      }
      v = v + rv[j];
      if (a.relu2) v = v > 0.f ? v : 0.f;
      y[j] = v;
    }
  }
}

typedef _Float16 v4h __attribute__((ext_vector_type(4)));

__device__ __forceinline__ char4 pack_int8(const ConvArgs& a, const float y[4]) {
  char4 q;
  q.x = (signed char)quant_f(y[0], a.out_r);
  q.y = (signed char)quant_f(y[1], a.out_r);
  q.z = (signed char)quant_f(y[2], a.out_r);
  q.w = (signed char)quant_f(y[3], a.out_r);
  return q;
}

__device__ __forceinline__ v4h pack_fp16(const float y[4]) {
  return v4h{(_Float16)y[0], (_Float16)y[1], (_Float16)y[2], (_Float16)y[3]};
}

// Stores 4 consecutive channels of one row after the fused epilogue.
template <int EL>
__device__ __forceinline__ void epilogue_store(const ConvArgs& a, uint32_t row, int co, const typename Mma<EL>::Acc& acc) {
  float y[4];
  epilogue_values<EL>(a, row, co, acc, y);
  if (a.out_dtype == SCN_DTYPE_INT8)
    *reinterpret_cast<char4*>(a.out + (size_t)row * a.out_ld + co) = pack_int8(a, y);
  else
    *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(a.out) + (size_t)row * a.out_ld + co) = pack_fp16(y);
}

// Row-split kernel: each wave owns 16*NT output rows and all MT*16 output channels; both operands
// come straight from global memory / L2 (weights: coalesced 1 KB fragments; features: gathered rows).
template <int EL, int CHUNKS, int MT, int NT>
__global__ __launch_bounds__(256) void k_conv_rows(const ConvArgs a) {
  using Acc = typename Mma<EL>::Acc;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const uint32_t n = eff_n(a.n_out_dev, a.n_bound);
  uint32_t tile;
  if (!xcd_tile(n, 64u * NT, &tile)) return;
  const uint32_t row0 = (tile * 4 + wave) * (16 * NT);
  if (row0 >= n) return;
  Acc acc[MT][NT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int u = 0; u < NT; ++u) acc[t][u] = Acc{0, 0, 0, 0};
  const uint4* wf = a.wfrag + lane;
  const uint4 zero = make_uint4(0, 0, 0, 0);
  uint32_t rows[NT];
#pragma unroll
  for (int u = 0; u < NT; ++u) rows[u] = row0 + u * 16 + lr;

  if constexpr (CHUNKS >= 4) {
    constexpr int SPK = CHUNKS / 4;  // K-steps per kernel offset
    for (int k = 0; k < a.kvol; ++k) {
      int32_t idx[NT];
      bool any = false;
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        idx[u] = rows[u] < n ? a.nbr[(size_t)k * a.nbr_ld + rows[u]] : -1;
        any |= idx[u] >= 0;
      }
      if (!__any(any)) continue;  // no row of this wave has a neighbour at this offset
#pragma unroll
      for (int ss = 0; ss < SPK; ++ss) {
        uint4 b[NT];
#pragma unroll
        for (int u = 0; u < NT; ++u) {
          b[u] = *reinterpret_cast<const uint4*>(a.x + (size_t)(idx[u] >= 0 ? idx[u] : 0) * a.x_ld_bytes +
                                                 (ss * 4 + lg) * 16);
          if (idx[u] < 0) b[u] = zero;
        }
        const int s = k * SPK + ss;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const uint4 av = wf[(size_t)(s * MT + t) * 64];
#pragma unroll
          for (int u = 0; u < NT; ++u) acc[t][u] = Mma<EL>::run(av, b[u], acc[t][u]);
        }
      }
    }
  } else {
    const int total_chunks = a.kvol * CHUNKS;
    for (int s = 0; s < a.steps; ++s) {
      const int g = 4 * s + lg;
      const int k = g / CHUNKS, c = g % CHUNKS;
      const bool gv = g < total_chunks;
      uint4 b[NT];
      bool any = false;
#pragma unroll
      for (int u = 0; u < NT; ++u) {
        int32_t idx = -1;
        if (gv && rows[u] < n) idx = a.nbr[(size_t)k * a.nbr_ld + rows[u]];
        any |= idx >= 0;
        b[u] = *reinterpret_cast<const uint4*>(a.x + (size_t)(idx >= 0 ? idx : 0) * a.x_ld_bytes + c * 16);
        if (idx < 0) b[u] = zero;
      }
      if (!__any(any)) continue;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const uint4 av = wf[(size_t)(s * MT + t) * 64];
#pragma unroll
        for (int u = 0; u < NT; ++u) acc[t][u] = Mma<EL>::run(av, b[u], acc[t][u]);
      }
    }
  }
#pragma unroll
  for (int u = 0; u < NT; ++u) {
    if (rows[u] >= n) continue;
#pragma unroll
    for (int t = 0; t < MT; ++t) epilogue_store<EL>(a, rows[u], t * 16 + lg * 4, acc[t][u]);
  }
}

// --------------------------------------------------------------------------------------------
// 32x32 MFMA variant (output channels >= 32).
// Measured issue rates on MI355X (independent accumulators, 4 waves per SIMD): v_mfma_i32_32x32x32_i8
// 4.77 POP/s and v_mfma_f32_32x32x16_f16 2.39 PFLOP/s, against 2.7 POP/s / 1.35 PFLOP/s for the
// 16x16x64 / 16x16x32 forms: only the 32x32 forms reach the matrix peak, so wide layers use them.
// Operand mapping (wave64):  A (32 x K): lane l supplies row m = l % 32, the 16 bytes of K-half l / 32
//                            B (K x 32): lane l supplies col n = l % 32, the 16 bytes of K-half l / 32
//                            D (32 x 32): lane l holds col n = l % 32, rows 8 * (j / 4) + 4 * (l / 32) + j % 4
// Rows of A are output channels, columns of B voxels; K-step s consumes chunks 2s and 2s+1 of the
// (offset, chunk) sequence.
template <int EL>
struct Mma32;
template <>
struct Mma32<0> {
  using Acc = v16i;
  using Acc4 = v4i;
  static __device__ __forceinline__ Acc run(const v4i a, const v4i b, Acc c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma32<1> {
  using Acc = v16f;
  using Acc4 = v4f;
  static __device__ __forceinline__ Acc run(const v4i a, const v4i b, Acc c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(v8h, a), __builtin_bit_cast(v8h, b), c, 0, 0, 0);
  }
};

// --------------------------------------------------------------------------------------------
// LDS-staged gather kernel (32x32 MFMA, output channels >= 32).
// What bounds the register-gather kernels above is the vector-memory path, not the matrix cores: a
// gather in MFMA operand order (32 rows x 2 lanes x 16 B) costs ~97 cycles of a CU's texture pipe per
// instruction, one whose 8 adjacent lanes read one row's 128 contiguous bytes ~35 (both measured,
// cache-resident table).  So everything that comes from global memory -- gathered rows, weight slabs,
// neighbour indices -- is loaded in memory-friendly order straight into LDS (global_load_lds: no
// registers, no masking; lanes without a neighbour read a row of zeros) and the MFMA operands are read
// back from LDS.  With no staging registers the kernel fits 128 VGPRs, so two 8-wave workgroups (four
// waves per SIMD, 512 output rows) share a CU and hide each other's latencies.
// Hardware places lane l's bytes at base + 16 l, so the bank-conflict-free read order of the B operand is
// obtained by permuting which chunk of its row a lane fetches: position p of a row holds chunk p ^ swz(row).
//   iteration     = 4 K-steps = 4 KB of gathered rows per wave (32 rows x 8 chunks, or G = 8 / SEG
//                   kernel offsets of SEG-chunk rows) and a weight slab of 4 * MT fragments
//   LDS           = 2 weight slabs (iteration i, i+1), one 4 KB stage of gathered rows per wave, and a
//                   4-deep ring of neighbour indices per wave (they always miss the caches)
//   per iteration = one barrier for the slab; a wave consumes only rows and indices it fetched itself,
//                   so those need a wait on the wave's own memory counter only
// The memory counter retires loads in order, so "at most N outstanding" names exactly which older load
// has landed.  Issue order per iteration i: slab S(i+1), indices I(i+4), gathers G(i+1).
// waves per SIMD the kernel is compiled for: two 8-wave workgroups per CU, or one of 10 / 12 waves
constexpr int conv_lds_min_waves(int waves) { return waves <= 8 ? 4 : 3; }

template <int EL, int CHUNKS, int MT, int WAVES>
__global__ __launch_bounds__(64 * WAVES, conv_lds_min_waves(WAVES)) void k_conv_lds(const ConvArgs a) {
  using Acc = typename Mma32<EL>::Acc;
  using Acc4 = typename Mma32<EL>::Acc4;
  constexpr int THREADS = 64 * WAVES;
  constexpr int SEG = CHUNKS < 8 ? CHUNKS : 8;   // chunks gathered per row and iteration
  constexpr int IPO = CHUNKS / SEG;              // iterations per kernel offset (rows wider than 128 B)
  constexpr int G = 8 / SEG;                     // kernel offsets per iteration
  constexpr int RP = 8 / SEG;                    // rows per 128 bytes of the gathered stage
  constexpr int SLAB = 4 * MT * 64;              // 16-byte weight fragments per iteration
  constexpr int NL = SLAB / 64;                  // 1 KB wave-loads per slab
  constexpr int WPT = (NL + WAVES - 1) / WAVES;  // slab loads per wave and iteration (the same for every wave:
                                                 // the waits below count loads; surplus ones go to `spare`)
  constexpr int IDXI = G >= 2 ? G / 2 : 1;       // index loads per wave and iteration (64 entries each)
  constexpr int R = 32 * WAVES;                  // output rows per workgroup
  __shared__ v4i lds[2][SLAB];
  __shared__ v4i ring[WAVES][256];
  __shared__ int32_t iring[4][WAVES][64 * IDXI];
  __shared__ v4i spare[NL % WAVES ? 64 : 1];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int ln = lane & 31, lh = lane >> 5;
  const uint32_t n = eff_n(a.n_out_dev, a.n_bound);
  uint32_t tile;
  if (!xcd_tile(n, R, &tile)) return;
  const uint32_t row0 = (tile * WAVES + wave) * 32;
  const int iters = IPO > 1 ? a.kvol * IPO : (a.kvol + G - 1) / G;
  const char* __restrict__ xb = a.x;
  const char* __restrict__ zrow = a.zrow;
  const v4i* __restrict__ wsrc = reinterpret_cast<const v4i*>(a.wfrag);
  const uint32_t ldb = a.x_ld_bytes;
  const int32_t* __restrict__ minus1 = reinterpret_cast<const int32_t*>(a.zrow + 512);  // words of -1

  Acc acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[t][j] = 0;

  typedef const __attribute__((address_space(1))) void* gptr_t;
  typedef __attribute__((address_space(3))) void* lptr_t;
#define SCN_WAIT_VM(N) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory")
// LDS reads of what global_load_lds wrote are written in assembly: the compiler orders a visible LDS read
// after EVERY outstanding global_load_lds (vmcnt(0)), which would drain the loads issued for the next
// iterations.  The waits that are really needed are the explicit ones below.
// weight slab of iteration IT -> LDS buffer IT % 2 (iterations past the end re-load the last slab)
#define SCN_SLAB(IT)                                                                            \
  {                                                                                             \
    const int it_ = (IT) < iters ? (IT) : iters - 1;                                            \
    _Pragma("unroll") for (int j = 0; j < WPT; ++j) {                                           \
      const int f_ = j * WAVES + wave; /* wave-uniform */                                       \
      if (NL % WAVES == 0 || f_ < NL)                                                           \
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + (size_t)it_ * SLAB + f_ * 64 + lane),  \
                                         (lptr_t)&lds[(IT) & 1][f_ * 64], 16, 0, 0);            \
      else                                                                                      \
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + (size_t)it_ * SLAB + lane),            \
                                         (lptr_t)&spare[0], 16, 0, 0);                          \
    }                                                                                           \
  }
// neighbour rows of iteration IT -> index ring stage IT % 4: entry e = 64 q + lane is kernel offset
// e / 32 of the iteration, tile row e % 32; slots outside the volume or beyond row n read -1
#define SCN_INDEX(IT)                                                                           \
  {                                                                                             \
    _Pragma("unroll") for (int q = 0; q < IDXI; ++q) {                                          \
      const int e_ = q * 64 + lane;                                                             \
      const int k_ = IPO > 1 ? (IT) / IPO + e_ / 32 : (IT) * G + e_ / 32;                       \
      const uint32_t r_ = row0 + (e_ & 31);                                                     \
      const bool ok_ = (IT) < iters && k_ < a.kvol && r_ < n;                                   \
      const int32_t* p_ = ok_ ? a.nbr + (size_t)k_ * a.nbr_ld + r_ : minus1 + lane;             \
      __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&iring[(IT) & 3][wave][q * 64], 4, 0, 0); \
    }                                                                                           \
  }
// gathers of iteration IT (neighbour rows GI[4] of this lane's slots) into the wave's stage; element
// e = 64 q + lane of its [G][32 rows][SEG] array
#define SCN_GATHER(IT, GI)                                                                      \
  {                                                                                             \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                             \
      const int e_ = q * 64 + lane;                                                             \
      const int row_ = (e_ / SEG) % 32;                                                         \
      const int cg_ = (IPO > 1 ? ((IT) % IPO) * 8 : 0) + ((e_ % SEG) ^ ((row_ / RP) % SEG));    \
      const char* p_ = GI[q] >= 0 ? xb + (size_t)(uint32_t)GI[q] * ldb + cg_ * 16 : zrow + cg_ * 16; \
      __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&ring[wave][q * 64], 16, 0, 0);      \
    }                                                                                           \
  }
// this lane's four index slots of ring stage STG -> GI[4], waited for.  Slot q of lane l is entry
// e / SEG of the stage (e = 64 q + l), i.e. a fixed stride of 64 / SEG entries between slots.
#define SCN_READ_INDEX(STG, GI)                                                                 \
  {                                                                                             \
    const uint32_t base_ = iring_addr + (uint32_t)(STG) * (WAVES * 64 * IDXI * 4);              \
    asm volatile("ds_read_b32 %0, %4\n\tds_read_b32 %1, %4 offset:%5\n\tds_read_b32 %2, %4 offset:%6\n\t" \
                 "ds_read_b32 %3, %4 offset:%7\n\ts_waitcnt lgkmcnt(0)"                         \
                 : "=&v"(GI[0]), "=&v"(GI[1]), "=&v"(GI[2]), "=&v"(GI[3])                       \
                 : "v"(base_), "n"(256 / SEG), "n"(2 * 256 / SEG), "n"(3 * 256 / SEG)           \
                 : "memory");                                                                   \
  }
// A fragments of K-step SS from the slab at LDS byte address LA (+ lane * 16 already included)
#define SCN_READ_A(SS, LA, AF)                                                                  \
  {                                                                                             \
    if constexpr (MT == 4)                                                                      \
      asm volatile("ds_read_b128 %0, %4 offset:%5\n\tds_read_b128 %1, %4 offset:%6\n\t"         \
                   "ds_read_b128 %2, %4 offset:%7\n\tds_read_b128 %3, %4 offset:%8"             \
                   : "=&v"(AF[0]), "=&v"(AF[1]), "=&v"(AF[2]), "=&v"(AF[3])                     \
                   : "v"(LA), "n"(((SS) * 4 + 0) * 1024), "n"(((SS) * 4 + 1) * 1024),           \
                     "n"(((SS) * 4 + 2) * 1024), "n"(((SS) * 4 + 3) * 1024)                     \
                   : "memory");                                                                 \
    else if constexpr (MT == 2)                                                                 \
      asm volatile("ds_read_b128 %0, %2 offset:%3\n\tds_read_b128 %1, %2 offset:%4"             \
                   : "=&v"(AF[0]), "=&v"(AF[1])                                                 \
                   : "v"(LA), "n"(((SS) * 2 + 0) * 1024), "n"(((SS) * 2 + 1) * 1024)            \
                   : "memory");                                                                 \
    else                                                                                        \
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=&v"(AF[0]) : "v"(LA), "n"((SS) * 1024) : "memory"); \
  }
// wait until at most KEEP LDS operations are outstanding; AF is named as in/out so that its MFMAs stay below
#define SCN_WAIT_A(KEEP, AF)                                                                    \
  {                                                                                             \
    if constexpr (MT == 4)                                                                      \
      asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(AF[0]), "+v"(AF[1]), "+v"(AF[2]), "+v"(AF[3]) : "n"(KEEP) : "memory"); \
    else if constexpr (MT == 2)                                                                 \
      asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(AF[0]), "+v"(AF[1]) : "n"(KEEP) : "memory");  \
    else                                                                                        \
      asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(AF[0]) : "n"(KEEP) : "memory");               \
  }

  const uint32_t ring_addr = (uint32_t)(uintptr_t)(lptr_t)&ring[wave][0];
  const uint32_t iring_addr = (uint32_t)(uintptr_t)(lptr_t)&iring[0][wave][0] + (uint32_t)(lane / SEG) * 4;
  const uint32_t lds_a_addr = (uint32_t)(uintptr_t)(lptr_t)&lds[0][lane];
  // B-operand read address of K-step ss inside the wave's stage: row ln, chunk 2 ss' + lh at its swizzled
  // position.  Recomputed per iteration from two values (registers are what limits occupancy here).
  const uint32_t b_base = ring_addr + (uint32_t)(SEG >= 2 ? ln * SEG : lh * 32 + ln) * 16;
  const uint32_t b_swz = SEG >= 2 ? (uint32_t)(lh ^ ((ln / RP) % SEG)) : 0u;
#define SCN_B_ADDR(SS, BB, SW)                                                                  \
  (SEG >= 2 ? (BB) + (uint32_t)((((SS) / (SEG / 2 > 0 ? SEG / 2 : 1)) * 32 * SEG) +             \
                                ((2 * ((SS) % (SEG / 2 > 0 ? SEG / 2 : 1))) ^ (SW))) * 16       \
            : (BB) + (uint32_t)(2 * (SS) * 32) * 16)

  // prologue: indices of iterations 0..3, slab 0, then the gathers of iteration 0
  SCN_INDEX(0);
  SCN_INDEX(1);
  SCN_INDEX(2);
  SCN_INDEX(3);
  SCN_SLAB(0);
  SCN_WAIT_VM(0);
  {
    int32_t gi[4];
    SCN_READ_INDEX(0, gi);
    SCN_GATHER(0, gi);
  }
  asm volatile("s_barrier" ::: "memory");

  for (int it = 0; it < iters; ++it) {
    SCN_SLAB(it + 1);
    SCN_INDEX(it + 4);
    SCN_WAIT_VM(WPT + IDXI);  // G(it), I(it+1) and everything older have landed
    v4i bf[4];
    int32_t gi[4];
    {
      uint32_t bb = b_base, sw = b_swz;
      asm volatile("" : "+v"(bb), "+v"(sw));  // keeps the four addresses out of loop-carried registers
      asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\tds_read_b128 %3, %7"
                   : "=&v"(bf[0]), "=&v"(bf[1]), "=&v"(bf[2]), "=&v"(bf[3])
                   : "v"(SCN_B_ADDR(0, bb, sw)), "v"(SCN_B_ADDR(1, bb, sw)), "v"(SCN_B_ADDR(2, bb, sw)),
                     "v"(SCN_B_ADDR(3, bb, sw))
                   : "memory");
    }
    // waits for the index reads and, LDS returning in order, for bf[]: the stage may be overwritten
    SCN_READ_INDEX((it + 1) & 3, gi);
    SCN_GATHER(it + 1, gi);
    const uint32_t la = lds_a_addr + (uint32_t)(it & 1) * (SLAB * 16);
    if constexpr (MT >= 4 && conv_lds_min_waves(WAVES) >= 4) {
      // 64 accumulator registers leave room for one set of fragments under the 128-register budget of
      // four waves per SIMD (a spill would also put scratch loads into the memory counter and break the
      // counts above); the other three waves of the SIMD cover the LDS latency instead
      v4i af[MT];
#pragma unroll
      for (int ss = 0; ss < 4; ++ss) {
        SCN_READ_A(ss, la, af);
        SCN_WAIT_A(0, af);
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = Mma32<EL>::run(af[t], bf[ss], acc[t]);
      }
    } else {
      v4i afA[MT], afB[MT];
      SCN_READ_A(0, la, afA);
      SCN_READ_A(1, la, afB);
      SCN_WAIT_A(MT, afA);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = Mma32<EL>::run(afA[t], bf[0], acc[t]);
      SCN_READ_A(2, la, afA);
      SCN_WAIT_A(MT, afB);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = Mma32<EL>::run(afB[t], bf[1], acc[t]);
      SCN_READ_A(3, la, afB);
      SCN_WAIT_A(MT, afA);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = Mma32<EL>::run(afA[t], bf[2], acc[t]);
      SCN_WAIT_A(0, afB);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = Mma32<EL>::run(afB[t], bf[3], acc[t]);
    }
    SCN_WAIT_VM(4);  // this wave's part of S(it+1) has landed (younger: G(it+1))
    // every wave has read slab it (its fragments are in registers) and written its part of slab it+1
    asm volatile("s_barrier" ::: "memory");
  }
#undef SCN_READ_INDEX
#undef SCN_B_ADDR
#undef SCN_READ_A
#undef SCN_WAIT_A
#undef SCN_WAIT_VM
#undef SCN_SLAB
#undef SCN_INDEX
#undef SCN_GATHER
  // Epilogue.  Each lane holds 4-channel pieces of one row; writing them directly would touch every
  // 128-byte line of the tile 16 times.  The pieces go through the wave's LDS stage instead (same XOR
  // placement as the gathers) and leave as 16 bytes per lane, 8 lanes per row.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stage still receives the gathers issued past the end
  const uint32_t row = row0 + ln;
  const int cout_pad = (a.cout + 15) & ~15;
  if (!a.out_vec16) {
    if (row >= n) return;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int co = t * 32 + g * 8 + lh * 4;
        if (co >= cout_pad) continue;
        const Acc4 piece = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
        epilogue_store<EL>(a, row, co, piece);
      }
    return;
  }
  char* stage = reinterpret_cast<char*>(&ring[wave][0]);
  const bool out8 = a.out_dtype == SCN_DTYPE_INT8;
  constexpr int PASSES = MT >= 4 ? 2 : 1;          // fp16 rows of 128 channels take two 128-byte passes
  constexpr int TPP = MT >= 4 ? 2 : MT;            // 32-channel tiles per fp16 pass
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    if (out8 && p > 0) break;
    const int t_lo = out8 ? 0 : p * TPP, t_hi = out8 ? MT : p * TPP + TPP;
    const int c0 = t_lo * 32;                      // first channel of the pass
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      if (t < t_lo || t >= t_hi) continue;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int co = t * 32 + g * 8 + lh * 4;
        if (co >= cout_pad || row >= n) continue;
        const Acc4 piece = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
        float y[4];
        epilogue_values<EL>(a, row, co, piece, y);
        const int off = (co - c0) * (out8 ? 1 : 2);  // byte offset inside the 128-byte pass row
        char* dst = stage + ln * 128 + (((off >> 4) ^ (ln & 7)) << 4) + (off & 15);
        if (out8)
          *reinterpret_cast<char4*>(dst) = pack_int8(a, y);
        else
          *reinterpret_cast<v4h*>(dst) = pack_fp16(y);
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int osz = out8 ? 1 : 2;
    const int valid = (cout_pad - c0) * osz;       // bytes of the pass row that exist
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = (lane >> 3) + 8 * j, c = lane & 7;
      const uint32_t grow = row0 + r;
      if (grow < n && c * 16 < valid) {
        const v4i v = *reinterpret_cast<const v4i*>(stage + r * 128 + ((c ^ (r & 7)) << 4));
        *reinterpret_cast<v4i*>(a.out + ((size_t)grow * a.out_ld + c0) * osz + c * 16) = v;
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
}

bool ConvWeights::init(const uint16_t* w_fp16, const int shape[5], const float* ranges, const uint16_t* bias_fp16,
                       int prec) {
  cout = shape[0];
  ks[0] = shape[1];
  ks[1] = shape[2];
  ks[2] = shape[3];
  cin = shape[4];
  kvol = ks[0] * ks[1] * ks[2];
  precision = prec;
  if (cout <= 0 || cin <= 0 || kvol <= 0) {
    set_error("invalid weight shape");
    return false;
  }
  if (prec == SCN_PRECISION_INT8 && ranges == nullptr) {
    set_error("int8 convolution needs weight_dynamic_ranges");
    return false;
  }
  const int epc = prec == SCN_PRECISION_INT8 ? 16 : 8;  // elements per 16-byte chunk
  int ch = (cin + epc - 1) / epc;
  int p2 = 1;
  while (p2 < ch) p2 <<= 1;  // chunks per row rounded to a power of two (rows are padded to it)
  chunks = p2;
  cin_pad = (uint32_t)(chunks * epc);
  mtiles = (cout + 15) / 16;
  steps = (kvol * chunks + 3) / 4;
  const int cout_pad = mtiles * 16;
  std::vector<float> ws(cout_pad, 1.f), bs(cout_pad, 0.f);
  for (int c = 0; c < cout; ++c) {
    if (prec == SCN_PRECISION_INT8) ws[c] = ranges[c] / 127.f;
    if (bias_fp16) bs[c] = half_bits_to_float(bias_fp16[c]);
  }
  std::vector<uint8_t> frag((size_t)steps * mtiles * 64 * 16, 0);
  for (int s = 0; s < steps; ++s)
    for (int t = 0; t < mtiles; ++t)
      for (int l = 0; l < 64; ++l) {
        const int g = 4 * s + l / 16;
        if (g >= kvol * chunks) continue;
        const int k = g / chunks, c = g % chunks;
        const int co = 16 * t + l % 16;
        if (co >= cout) continue;
        uint8_t* dst = &frag[((size_t)(s * mtiles + t) * 64 + l) * 16];
        for (int e = 0; e < epc; ++e) {
          const int ci = c * epc + e;
          if (ci >= cin) break;
          const uint16_t hb = w_fp16[((size_t)co * kvol + k) * cin + ci];
          if (prec == SCN_PRECISION_INT8) {
            float q = rintf(half_bits_to_float(hb) * (127.f / ranges[co]));
            if (!(q >= -127.f)) q = -127.f;
            if (q > 127.f) q = 127.f;
            dst[e] = (uint8_t)(int8_t)q;
          } else {
            memcpy(dst + 2 * e, &hb, 2);
          }
        }
      }
  // 32x32 MFMA order for layers with more than 16 output channels: [step][mtile32][lane] x 16 bytes,
  // lane l = channel 32 t + l % 32, K-half l / 32; K-step s holds chunks 2s, 2s+1 of the sequence
  if (mtiles >= 1) {
    mtiles32 = (cout + 31) / 32;
    if (mtiles32 == 3) mtiles32 = 4;  // kernels exist for 1, 2 and 4 tiles; the fourth is zero weights
    steps32 = 4 * ((kvol * chunks + 7) / 8);  // whole iterations of 4 K-steps, zero weights beyond the volume
    std::vector<uint8_t> f32((size_t)steps32 * mtiles32 * 64 * 16, 0);
    for (int s = 0; s < steps32; ++s)
      for (int t = 0; t < mtiles32; ++t)
        for (int l = 0; l < 64; ++l) {
          const int g = 2 * s + l / 32;
          if (g >= kvol * chunks) continue;
          const int k = g / chunks, c = g % chunks;
          const int co = 32 * t + l % 32;
          if (co >= cout) continue;
          uint8_t* dst = &f32[((size_t)(s * mtiles32 + t) * 64 + l) * 16];
          for (int e = 0; e < epc; ++e) {
            const int ci = c * epc + e;
            if (ci >= cin) break;
            const uint16_t hb = w_fp16[((size_t)co * kvol + k) * cin + ci];
            if (prec == SCN_PRECISION_INT8) {
              float q = rintf(half_bits_to_float(hb) * (127.f / ranges[co]));
              if (!(q >= -127.f)) q = -127.f;
              if (q > 127.f) q = 127.f;
              dst[e] = (uint8_t)(int8_t)q;
            } else {
              memcpy(dst + 2 * e, &hb, 2);
            }
          }
        }
    if (!zrow.alloc(768) || hipMemset(zrow.p, 0, 512) != hipSuccess ||
        hipMemset(zrow.as<char>() + 512, 0xFF, 256) != hipSuccess ||  // 64 words of -1 ("no neighbour")
        !wfrag32.alloc(f32.size()) || hipMemcpy(wfrag32.p, f32.data(), f32.size(), hipMemcpyHostToDevice) != hipSuccess) {
      set_error("weight upload failed");
      return false;
    }
  }
  if (!wfrag.alloc(frag.size()) || !wscale.alloc(ws.size() * 4) || !bias.alloc(bs.size() * 4)) return false;
  if (hipMemcpy(wfrag.p, frag.data(), frag.size(), hipMemcpyHostToDevice) != hipSuccess ||
      hipMemcpy(wscale.p, ws.data(), ws.size() * 4, hipMemcpyHostToDevice) != hipSuccess ||
      hipMemcpy(bias.p, bs.data(), bs.size() * 4, hipMemcpyHostToDevice) != hipSuccess) {
    set_error("weight upload failed");
    return false;
  }
  return true;
}

// SCN_CONV_IMPL=rows forces the plain row-split kernel (A/B measurements; it is also the fallback for
// more than 128 output channels).
static int conv_impl() {
  static const int impl = [] {
    const char* e = getenv("SCN_CONV_IMPL");
    return (e && !strcmp(e, "rows")) ? 1 : 0;
  }();
  return impl;
}

template <int EL, int CHUNKS, int MT>
static void launch_conv_rows(const ConvArgs& a, hipStream_t stream) {
  constexpr int NT = MT >= 8 ? 2 : 4;
  const uint32_t rows_per_block = 4 * 16 * NT;
  const uint32_t blocks = 8 * ceil_div(ceil_div(a.n_bound, rows_per_block), 8);  // see xcd_tile()
  hipLaunchKernelGGL((k_conv_rows<EL, CHUNKS, MT, NT>), dim3(blocks), dim3(256), 0, stream, a);
}

template <int EL, int CHUNKS, int MT, int WAVES>
static void launch_conv_lds(const ConvArgs& a, hipStream_t stream) {
  constexpr uint32_t R = 32 * WAVES;
  const uint32_t blocks = 8 * ceil_div(ceil_div(a.n_bound, R), 8);  // see xcd_tile()
  hipLaunchKernelGGL((k_conv_lds<EL, CHUNKS, MT, WAVES>), dim3(blocks), dim3(64 * WAVES), 0, stream, a);
}

// Workgroup size of the 128-channel kernel.  A layer of a lidar backbone's deep stages is about one
// workgroup per CU, so its duration is that of the busiest CU: 257 tiles of 256 rows on 256 CUs take
// as long as 512.  With the expected row count (the count of the previous forward, see
// Rulebook::n_out_hint) the tile height is chosen so that all rows fit one workgroup per CU when they
// can: 8 to 12 waves of 32 rows; beyond 384 rows per CU it is 8 waves and two workgroups per CU.
static int conv_lds_waves(uint32_t n_hint) {
  static const int forced = [] {
    const char* e = getenv("SCN_CONV_WAVES");
    return e ? atoi(e) : 0;
  }();
  if (forced >= 8 && forced <= 12) return forced;
  constexpr uint32_t kCus = 256;
  const uint32_t waves = ceil_div(n_hint, kCus * 32u);  // 32-row tiles per CU
  if (waves <= 8) return 8;
  if (waves <= 12) return (int)waves;
  return 8;
}

template <int EL, int CHUNKS>
static bool dispatch_mt32(int mt, uint32_t n_hint, const ConvArgs& a, hipStream_t stream) {
  switch (mt) {
    case 1: launch_conv_lds<EL, CHUNKS, 1, 4>(a, stream); return true;
    case 2: launch_conv_lds<EL, CHUNKS, 2, 8>(a, stream); return true;
    case 4:
      switch (conv_lds_waves(n_hint)) {
        case 9: launch_conv_lds<EL, CHUNKS, 4, 9>(a, stream); return true;
        case 10: launch_conv_lds<EL, CHUNKS, 4, 10>(a, stream); return true;
        case 11: launch_conv_lds<EL, CHUNKS, 4, 11>(a, stream); return true;
        case 12: launch_conv_lds<EL, CHUNKS, 4, 12>(a, stream); return true;
        default: launch_conv_lds<EL, CHUNKS, 4, 8>(a, stream); return true;
      }
    default: return false;
  }
}

template <int EL>
static bool dispatch_chunks32(int chunks, int mt, uint32_t n_hint, const ConvArgs& a, hipStream_t stream) {
  switch (chunks) {
    case 1: return dispatch_mt32<EL, 1>(mt, n_hint, a, stream);
    case 2: return dispatch_mt32<EL, 2>(mt, n_hint, a, stream);
    case 4: return dispatch_mt32<EL, 4>(mt, n_hint, a, stream);
    case 8: return dispatch_mt32<EL, 8>(mt, n_hint, a, stream);
    case 16: return dispatch_mt32<EL, 16>(mt, n_hint, a, stream);
    default: return false;
  }
}

template <int EL, int CHUNKS>
static bool dispatch_mt(int mt, const ConvArgs& a, hipStream_t stream) {
  switch (mt) {
    case 1: launch_conv_rows<EL, CHUNKS, 1>(a, stream); return true;
    case 2: launch_conv_rows<EL, CHUNKS, 2>(a, stream); return true;
    case 4: launch_conv_rows<EL, CHUNKS, 4>(a, stream); return true;
    case 8: launch_conv_rows<EL, CHUNKS, 8>(a, stream); return true;
    default: return false;
  }
}

template <int EL>
static bool dispatch_chunks(int chunks, int mt, const ConvArgs& a, hipStream_t stream) {
  switch (chunks) {
    case 1: return dispatch_mt<EL, 1>(mt, a, stream);
    case 2: return dispatch_mt<EL, 2>(mt, a, stream);
    case 4: return dispatch_mt<EL, 4>(mt, a, stream);
    case 8: return dispatch_mt<EL, 8>(mt, a, stream);
    case 16: return dispatch_mt<EL, 16>(mt, a, stream);
    default: return false;
  }
}

int conv_forward(const ConvWeights& w, const int32_t* nbr, uint32_t nbr_ld, const uint32_t* n_out_dev,
                 uint32_t n_bound, uint32_t n_hint, const scn_conv_io& io, hipStream_t stream) {
  if (n_bound == 0) return SCN_OK;
  const int esz = w.precision == SCN_PRECISION_INT8 ? 1 : 2;
  SCN_REQUIRE(io.x_dev && io.out_dev, SCN_ERR_INVALID, "conv: null input or output");
  SCN_REQUIRE(io.x_ld >= w.cin_pad, SCN_ERR_INVALID, "conv: input row stride %u < padded channels %u", io.x_ld,
              w.cin_pad);
  SCN_REQUIRE(((size_t)io.x_ld * esz) % 16 == 0 && ((uintptr_t)io.x_dev & 15) == 0, SCN_ERR_INVALID,
              "conv: input rows must be 16-byte aligned");
  SCN_REQUIRE(io.out_dtype == SCN_DTYPE_INT8 || io.out_dtype == SCN_DTYPE_FP16, SCN_ERR_INVALID, "conv: bad out dtype");
  SCN_REQUIRE(io.out_ld >= (uint32_t)w.mtiles * 16, SCN_ERR_INVALID, "conv: output row stride %u < %d", io.out_ld,
              w.mtiles * 16);
  const int osz = io.out_dtype == SCN_DTYPE_INT8 ? 1 : 2;
  SCN_REQUIRE(((size_t)io.out_ld * osz) % (4 * osz) == 0 && ((uintptr_t)io.out_dev & 7) == 0, SCN_ERR_INVALID,
              "conv: output rows must be 8-byte aligned");
  if (io.res_dev) {
    SCN_REQUIRE(io.res_dtype == SCN_DTYPE_INT8 || io.res_dtype == SCN_DTYPE_FP16, SCN_ERR_INVALID, "conv: bad residual dtype");
    SCN_REQUIRE(io.mid_dtype == SCN_DTYPE_INT8 || io.mid_dtype == SCN_DTYPE_FP16, SCN_ERR_INVALID, "conv: bad mid dtype");
    SCN_REQUIRE(io.res_ld >= (uint32_t)w.mtiles * 16 && io.res_ld % 4 == 0 && ((uintptr_t)io.res_dev & 7) == 0,
                SCN_ERR_INVALID, "conv: residual rows misaligned or too short");
  }
  SCN_REQUIRE(!io.acc_dev || w.cout % 16 == 0, SCN_ERR_UNSUPPORTED, "accumulator dump needs Cout %% 16 == 0");
  ConvArgs a;
  a.x = (const char*)io.x_dev;
  a.x_ld_bytes = io.x_ld * esz;
  a.nbr = nbr;
  a.nbr_ld = nbr_ld;
  a.kvol = w.kvol;
  a.n_out_dev = n_out_dev;
  a.n_bound = n_bound;
  a.wfrag = w.wfrag.as<uint4>();
  a.zrow = w.zrow.as<char>();
  a.steps = w.steps;
  a.wscale = w.wscale.as<float>();
  a.bias = w.bias.as<float>();
  a.cout = w.cout;
  auto s_of = [](float range) { return range > 0.f ? range / 127.f : 0.f; };
  auto r_of = [](float range) { return range > 0.f ? 127.f / range : 0.f; };
  a.x_scale = s_of(io.x_dynamic_range);
  a.relu = io.relu;
  a.out_dtype = io.out_dtype;
  a.out_r = r_of(io.out_dynamic_range);
  a.out = (char*)io.out_dev;
  a.out_ld = io.out_ld;
  a.acc = io.acc_dev;
  a.res = (const char*)io.res_dev;
  a.res_dtype = io.res_dtype;
  a.res_scale = s_of(io.res_dynamic_range);
  a.res_ld = io.res_ld;
  a.mid_dtype = io.mid_dtype;
  a.mid_s = s_of(io.mid_dynamic_range);
  a.mid_r = r_of(io.mid_dynamic_range);
  a.a_rq_s = s_of(io.a_requant_range);
  a.a_rq_r = r_of(io.a_requant_range);
  a.b_rq_s = s_of(io.b_requant_range);
  a.b_rq_r = r_of(io.b_requant_range);
  a.relu2 = io.relu_after_add;
  a.out_vec16 = (((size_t)io.out_ld * osz) % 16 == 0 && ((uintptr_t)io.out_dev & 15) == 0 &&
                 ((size_t)((w.cout + 15) & ~15) * osz) % 16 == 0) ? 1 : 0;
  if (io.out_dtype == SCN_DTYPE_INT8)
    SCN_REQUIRE(io.out_dynamic_range > 0.f, SCN_ERR_INVALID, "conv: int8 output needs out_dynamic_range > 0");
  if (w.precision == SCN_PRECISION_INT8)
    SCN_REQUIRE(io.x_dynamic_range > 0.f, SCN_ERR_INVALID, "conv: int8 input needs x_dynamic_range > 0");
  bool ok = false;
  const int mt32 = w.mtiles32;
  if (mt32 >= 1 && mt32 <= 4 && conv_impl() == 0) {
    a.wfrag = w.wfrag32.as<uint4>();
    if (n_hint == 0 || n_hint > n_bound) n_hint = n_bound;
    ok = w.precision == SCN_PRECISION_INT8 ? dispatch_chunks32<0>(w.chunks, mt32, n_hint, a, stream)
                                           : dispatch_chunks32<1>(w.chunks, mt32, n_hint, a, stream);
  }
  if (!ok) {
    a.wfrag = w.wfrag.as<uint4>();
    ok = w.precision == SCN_PRECISION_INT8 ? dispatch_chunks<0>(w.chunks, w.mtiles, a, stream)
                                           : dispatch_chunks<1>(w.chunks, w.mtiles, a, stream);
  }
  SCN_REQUIRE(ok, SCN_ERR_UNSUPPORTED, "conv: no kernel for Cin=%d Cout=%d (chunks %d, m-tiles %d)", w.cin, w.cout,
              w.chunks, w.mtiles);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// elementwise glue
// --------------------------------------------------------------------------------------------
// scale = amax/127 of an int8 operand; rq_s / rq_r = amax/127 and 127/amax of the re-quantisation an
// int8 Add applies to an fp16 operand (0 = none)
__device__ __forceinline__ float load_value(const void* p, int dtype, size_t i, float scale, float rq_s, float rq_r) {
  if (dtype == SCN_DTYPE_INT8) return (float)reinterpret_cast<const signed char*>(p)[i] * scale;
  float v = (float)reinterpret_cast<const _Float16*>(p)[i];
  if (rq_r > 0.f) v = quant_f(v, rq_r) * rq_s;
  return v;
}

// r = 127/amax of an int8 destination
__device__ __forceinline__ void store_value(void* p, int dtype, size_t i, float v, float r) {
  if (dtype == SCN_DTYPE_INT8)
    reinterpret_cast<signed char*>(p)[i] = (signed char)quant_f(v, r);
  else
    reinterpret_cast<_Float16*>(p)[i] = (_Float16)v;
}

__global__ __launch_bounds__(256) void k_convert_rows(const void* in, int in_dtype, uint32_t in_c, uint32_t in_ld,
                                                      float in_scale, void* out, int out_dtype, uint32_t out_c,
                                                      uint32_t out_ld, float out_r, int relu, uint32_t n_bound,
                                                      const uint32_t* n_dev) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  const uint32_t row = (uint32_t)(t / out_c), c = (uint32_t)(t % out_c);
  if (row >= n) return;
  float v = 0.f;
  if (c < in_c) v = load_value(in, in_dtype, (size_t)row * in_ld + c, in_scale, 0.f, 0.f);
  if (relu) v = v > 0.f ? v : 0.f;
  store_value(out, out_dtype, (size_t)row * out_ld + c, v, out_r);
}

// in_range / out_range: dynamic ranges (amax) of int8 operands; a range of 127 makes q <-> value the identity
int convert_rows(const void* in, int in_dtype, uint32_t in_c, uint32_t in_ld, float in_range, void* out,
                 int out_dtype, uint32_t out_c, uint32_t out_ld, float out_range, int relu, uint32_t n,
                 const uint32_t* n_dev, hipStream_t stream) {
  const float in_scale = in_range > 0.f ? in_range / 127.f : 1.f;
  const float out_scale = out_range > 0.f ? 127.f / out_range : 1.f;
  if (n == 0) return SCN_OK;
  SCN_REQUIRE(in && out && out_c > 0 && out_ld >= out_c && in_ld >= in_c, SCN_ERR_INVALID, "convert_rows: bad arguments");
  const size_t total = (size_t)n * out_c;
  hipLaunchKernelGGL(k_convert_rows, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, in, in_dtype, in_c,
                     in_ld, in_scale, out, out_dtype, out_c, out_ld, out_scale, relu, n, n_dev);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

struct AddOperand {
  const void* p;
  int dtype;
  float scale, rq_s, rq_r;
};

__global__ __launch_bounds__(256) void k_add_relu(AddOperand a, AddOperand b, void* out, int out_dtype, float out_r,
                                                  int relu, uint32_t c, uint32_t n_bound, const uint32_t* n_dev) {
  const size_t total = (size_t)eff_n(n_dev, n_bound) * c;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  float v = load_value(a.p, a.dtype, i, a.scale, a.rq_s, a.rq_r) + load_value(b.p, b.dtype, i, b.scale, b.rq_s, b.rq_r);
  if (relu) v = v > 0.f ? v : 0.f;
  store_value(out, out_dtype, i, v, out_r);
}

// *_range: dynamic range (amax) of an int8 operand; *_rq: range an int8 Add re-quantises an fp16 operand with
int add_relu(const void* a, int a_dtype, float a_range, float a_rq, const void* b, int b_dtype, float b_range,
             float b_rq, void* out, int out_dtype, float out_range, int relu, uint32_t c, uint32_t n,
             const uint32_t* n_dev, hipStream_t stream) {
  if (n == 0 || c == 0) return SCN_OK;
  SCN_REQUIRE(a && b && out, SCN_ERR_INVALID, "add_relu: null pointer");
  const size_t total = (size_t)n * c;
  auto s_of = [](float r) { return r > 0.f ? r / 127.f : 0.f; };
  auto r_of = [](float r) { return r > 0.f ? 127.f / r : 0.f; };
  const AddOperand oa{a, a_dtype, s_of(a_range), s_of(a_rq), r_of(a_rq)};
  const AddOperand ob{b, b_dtype, s_of(b_range), s_of(b_rq), r_of(b_rq)};
  hipLaunchKernelGGL(k_add_relu, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, oa, ob, out, out_dtype,
                     r_of(out_range), relu, c, n, n_dev);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// sparse -> dense.  strides are those of the final (possibly transposed) layout, in elements.
// --------------------------------------------------------------------------------------------
struct DenseStrides {
  int64_t sc, s0, s1, s2;
  int d0, d1, d2;
};

// One thread per (row, group of 8 channels): the coordinate row and 8 channels are read with one
// vector load each; consecutive threads are consecutive rows, i.e. mostly adjacent cells of the
// innermost dense axis, so the 8 strided stores of a wave land in 8 short contiguous runs.
__global__ __launch_bounds__(256) void k_scatter_dense(const void* feat, int dtype, float scale, uint32_t c_total,
                                                       uint32_t ld, const int4* __restrict__ coords, uint32_t n_bound,
                                                       const uint32_t* n_dev, DenseStrides st, _Float16* out) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t row = blockIdx.x * 256 + threadIdx.x;
  if (row >= n) return;
  const uint32_t c0 = blockIdx.y * 8;
  const int4 p = coords[row];
  if (p.x != 0 || p.y < 0 || p.y >= st.d0 || p.z < 0 || p.z >= st.d1 || p.w < 0 || p.w >= st.d2) return;
  _Float16* dst = out + p.y * st.s0 + p.z * st.s1 + p.w * st.s2;
  float v[8];
  const bool full = c0 + 8 <= c_total;
  if (full && dtype == SCN_DTYPE_FP16 && (ld & 7) == 0) {
    typedef _Float16 v8hh __attribute__((ext_vector_type(8)));
    const v8hh h = *reinterpret_cast<const v8hh*>(reinterpret_cast<const _Float16*>(feat) + (size_t)row * ld + c0);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (float)h[j];
  } else if (full && dtype == SCN_DTYPE_INT8 && (ld & 7) == 0) {
    typedef signed char v8c __attribute__((ext_vector_type(8)));
    const v8c q = *reinterpret_cast<const v8c*>(reinterpret_cast<const signed char*>(feat) + (size_t)row * ld + c0);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (float)q[j] * scale;
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j)
      v[j] = c0 + j < c_total ? load_value(feat, dtype, (size_t)row * ld + c0 + j, scale, 0.f, 0.f) : 0.f;
  }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (c0 + j < c_total) dst[(c0 + j) * st.sc] = (_Float16)v[j];
}

// Dense-major variant for layouts whose channel axis is outermost (the reference's
// [1, C, D0, D1, D2] after its Transpose): cell_map[cell] holds the row that occupies a cell or -1,
// where "cell" is the element offset inside one channel plane.  Pass 1 writes the row numbers,
// pass 2 walks the dense tensor in memory order and writes every element exactly once (value or
// zero) in whole 16-byte vectors, so the tensor needs no clear and no partial-line stores.
__global__ __launch_bounds__(256) void k_cell_map(const int4* __restrict__ coords, uint32_t n_bound,
                                                  const uint32_t* n_dev, DenseStrides st, int32_t* cell_map) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t row = blockIdx.x * 256 + threadIdx.x;
  if (row >= n) return;
  const int4 p = coords[row];
  if (p.x != 0 || p.y < 0 || p.y >= st.d0 || p.z < 0 || p.z >= st.d1 || p.w < 0 || p.w >= st.d2) return;
  cell_map[p.y * st.s0 + p.z * st.s1 + p.w * st.s2] = (int32_t)row;
}

// One thread per (8 consecutive cells, 8 channels): 8 map entries, up to 8 gathered 8-channel
// vectors, transposed in registers into 8 stores of 16 bytes (one per channel plane); consecutive
// lanes own consecutive cell groups, so every store instruction of a wave writes 1 KiB contiguously.
__global__ __launch_bounds__(128) void k_dense_from_map(const void* feat, int dtype, float scale, uint32_t c_total,
                                                        uint32_t ld, const int32_t* __restrict__ cell_map,
                                                        uint32_t cell_groups, uint32_t plane, _Float16* out) {
  typedef _Float16 v8hh __attribute__((ext_vector_type(8)));
  const uint32_t g = blockIdx.x * 128 + threadIdx.x;
  if (g >= cell_groups) return;
  const uint32_t c0 = blockIdx.y * 8;
  const int4 ma = *reinterpret_cast<const int4*>(cell_map + (size_t)g * 8);
  const int4 mb = *reinterpret_cast<const int4*>(cell_map + (size_t)g * 8 + 4);
  const int m[8] = {ma.x, ma.y, ma.z, ma.w, mb.x, mb.y, mb.z, mb.w};
  v8hh o[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) o[j] = v8hh{0, 0, 0, 0, 0, 0, 0, 0};
  if ((ma.x & ma.y & ma.z & ma.w & mb.x & mb.y & mb.z & mb.w) >= 0) {   // some entry is a row
    // all eight gathers are issued before the first is used; empty cells read row 0 and are masked
    const bool full = c0 + 8 <= c_total && (ld & 7) == 0;
    size_t base[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) base[i] = (size_t)(m[i] < 0 ? 0 : m[i]) * ld + c0;
    if (full && dtype == SCN_DTYPE_FP16) {
      v8hh h[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = *reinterpret_cast<const v8hh*>(reinterpret_cast<const _Float16*>(feat) + base[i]);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j][i] = m[i] < 0 ? (_Float16)0 : h[i][j];
    } else if (full && dtype == SCN_DTYPE_INT8) {
      typedef signed char v8c __attribute__((ext_vector_type(8)));
      v8c q[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) q[i] = *reinterpret_cast<const v8c*>(reinterpret_cast<const signed char*>(feat) + base[i]);
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j][i] = m[i] < 0 ? (_Float16)0 : (_Float16)((float)q[i][j] * scale);
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (m[i] < 0) continue;
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (c0 + j < c_total) o[j][i] = (_Float16)load_value(feat, dtype, base[i] + j, scale, 0.f, 0.f);
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (c0 + j < c_total) *reinterpret_cast<v8hh*>(out + (size_t)(c0 + j) * plane + (size_t)g * 8) = o[j];
}

// strides (in elements) of dense_shape's five axes inside the (possibly transposed) output
static bool dense_layout(const int dense_shape[5], const int perm[5], int64_t dstride[5], size_t* numel) {
  int p[5] = {0, 1, 2, 3, 4};
  if (perm) {
    bool seen[5] = {false, false, false, false, false};
    for (int j = 0; j < 5; ++j) {
      if (perm[j] < 0 || perm[j] >= 5 || seen[perm[j]]) return false;
      seen[perm[j]] = true;
      p[j] = perm[j];
    }
  }
  int64_t tstride[5];
  int64_t s = 1;
  for (int j = 4; j >= 0; --j) {
    tstride[j] = s;
    s *= dense_shape[p[j]];
  }
  for (int j = 0; j < 5; ++j) dstride[p[j]] = tstride[j];
  *numel = (size_t)s;
  return true;
}

size_t scatter_dense_map_cells(const int dense_shape[5], const int perm[5]) {
  int64_t dstride[5];
  size_t numel = 0;
  if (!dense_shape || dense_shape[0] != 1 || !dense_layout(dense_shape, perm, dstride, &numel)) return 0;
  const size_t plane = (size_t)dense_shape[2] * dense_shape[3] * dense_shape[4];
  if (plane == 0 || plane % 8 != 0 || plane > 0x7fffffffu) return 0;
  return dstride[1] == (int64_t)plane ? plane : 0;   // channel axis outermost
}

int scatter_dense_build_map(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                            const int perm[5], int32_t* cell_map, bool map_precleared, hipStream_t stream) {
  const size_t plane = scatter_dense_map_cells(dense_shape, perm);
  SCN_REQUIRE(plane && cell_map, SCN_ERR_INVALID, "scatter_dense: this layout takes no row map");
  SCN_REQUIRE(n == 0 || idx, SCN_ERR_INVALID, "scatter_dense: null input");
  int64_t dstride[5];
  size_t numel = 0;
  dense_layout(dense_shape, perm, dstride, &numel);
  DenseStrides st{dstride[1], dstride[2], dstride[3], dstride[4], dense_shape[2], dense_shape[3], dense_shape[4]};
  if (!map_precleared) {
    int rc = fill_u32(cell_map, 0xFFFFFFFFu, plane, stream);
    if (rc) return rc;
  }
  if (n)
    hipLaunchKernelGGL(k_cell_map, dim3(ceil_div(n, 256)), dim3(256), 0, stream, (const int4*)idx, n, n_dev, st, cell_map);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

int scatter_dense(const void* feat, int dtype, float range, uint32_t c, uint32_t ld, const int32_t* idx, uint32_t n,
                  const uint32_t* n_dev, const int dense_shape[5], const int perm[5], void* out, hipStream_t stream,
                  bool precleared, int32_t* cell_map, bool map_precleared, bool map_built) {
  SCN_REQUIRE(out && dense_shape, SCN_ERR_INVALID, "scatter_dense: null pointer");
  const float scale = range > 0.f ? range / 127.f : 1.f;
  SCN_REQUIRE(dense_shape[0] == 1 && (uint32_t)dense_shape[1] == c, SCN_ERR_INVALID,
              "scatter_dense: output_shape must be [1, C=%u, D0, D1, D2]", c);
  int64_t dstride[5];
  size_t numel = 0;
  SCN_REQUIRE(dense_layout(dense_shape, perm, dstride, &numel), SCN_ERR_INVALID, "scatter_dense: bad permutation");
  SCN_REQUIRE(numel % 2 == 0, SCN_ERR_UNSUPPORTED, "scatter_dense: odd element count");
  DenseStrides st{dstride[1], dstride[2], dstride[3], dstride[4], dense_shape[2], dense_shape[3], dense_shape[4]};
  const size_t plane = cell_map ? scatter_dense_map_cells(dense_shape, perm) : 0;
  if (plane) {
    SCN_REQUIRE(n == 0 || (feat && idx), SCN_ERR_INVALID, "scatter_dense: null input");
    if (!map_built) {
      int rc = scatter_dense_build_map(idx, n, n_dev, dense_shape, perm, cell_map, map_precleared, stream);
      if (rc) return rc;
    }
    const uint32_t groups = (uint32_t)(plane / 8);
    hipLaunchKernelGGL(k_dense_from_map, dim3(ceil_div(groups, 128), ceil_div(c, 8)), dim3(128), 0, stream, feat, dtype,
                       scale, c, ld, cell_map, groups, (uint32_t)plane, (_Float16*)out);
    SCN_HIP(hipGetLastError());
    return SCN_OK;
  }
  if (!precleared) {
    int rc = fill_u32(out, 0u, numel / 2, stream);
    if (rc) return rc;
  }
  if (n == 0) return SCN_OK;
  SCN_REQUIRE(feat && idx, SCN_ERR_INVALID, "scatter_dense: null input");
  hipLaunchKernelGGL(k_scatter_dense, dim3(ceil_div(n, 256), ceil_div(c, 8)), dim3(256), 0, stream, feat, dtype, scale, c,
                     ld, (const int4*)idx, n, n_dev, st, (_Float16*)out);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// Stand-alone dense permute of a 5-D fp16 tensor (used only when the Transpose is not fused into
// the scatter): out[o0..o4] = in[index with dim perm[j] = o_j].
struct Permute5 {
  int64_t in_stride[5];   // input stride of the dimension that output dim j walks
  int64_t out_shape[5];
};

__global__ __launch_bounds__(256) void k_permute5(const _Float16* __restrict__ in, _Float16* out, Permute5 p,
                                                  size_t numel) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= numel) return;
  size_t rem = i, src = 0;
#pragma unroll
  for (int j = 4; j >= 0; --j) {
    const size_t c = rem % (size_t)p.out_shape[j];
    rem /= (size_t)p.out_shape[j];
    src += c * (size_t)p.in_stride[j];
  }
  out[i] = in[src];
}

int permute_dense(const void* in, const int64_t in_shape[5], const int perm[5], void* out, hipStream_t stream) {
  Permute5 p;
  int64_t istride[5];
  int64_t s = 1;
  for (int j = 4; j >= 0; --j) {
    istride[j] = s;
    s *= in_shape[j];
  }
  for (int j = 0; j < 5; ++j) {
    SCN_REQUIRE(perm[j] >= 0 && perm[j] < 5, SCN_ERR_INVALID, "permute: bad permutation");
    p.in_stride[j] = istride[perm[j]];
    p.out_shape[j] = in_shape[perm[j]];
  }
  const size_t numel = (size_t)s;
  if (numel == 0) return SCN_OK;
  hipLaunchKernelGGL(k_permute5, dim3((unsigned)((numel + 255) / 256)), dim3(256), 0, stream, (const _Float16*)in,
                     (_Float16*)out, p, numel);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// --------------------------------------------------------------------------------------------
// voxelization
// --------------------------------------------------------------------------------------------
struct VoxGeom {
  float mn[3], mx[3], vs[3];
  int g[3];     // x, y, z cells
  int og[3];    // grid in output coordinate order (zyx: z,y,x / xyz: x,y,z)
  int order;
  int nf;
  int max_voxels, max_pts;
};

// Pass 1 over the point stream: cell key per point + occupancy bit.
__global__ __launch_bounds__(256) void k_vox_mark(const _Float16* __restrict__ pts, uint32_t n, VoxGeom g,
                                                  uint32_t* pkey, uint32_t* bitmap) {
  const uint32_t p = blockIdx.x * 256 + threadIdx.x;
  if (p >= n) return;
  const float px = (float)pts[(size_t)p * g.nf + 0];
  const float py = (float)pts[(size_t)p * g.nf + 1];
  const float pz = (float)pts[(size_t)p * g.nf + 2];
  uint32_t key = 0xFFFFFFFFu;
  if (px >= g.mn[0] && px < g.mx[0] && py >= g.mn[1] && py < g.mx[1] && pz >= g.mn[2] && pz < g.mx[2]) {
    const int ix = (int)floorf((px - g.mn[0]) / g.vs[0]);
    const int iy = (int)floorf((py - g.mn[1]) / g.vs[1]);
    const int iz = (int)floorf((pz - g.mn[2]) / g.vs[2]);
    if (ix >= 0 && ix < g.g[0] && iy >= 0 && iy < g.g[1] && iz >= 0 && iz < g.g[2]) {
      key = g.order == SCN_ORDER_ZYX ? ((uint32_t)iz * g.g[1] + iy) * g.g[0] + ix
                                     : ((uint32_t)ix * g.g[1] + iy) * g.g[2] + iz;
      atomicOr(&bitmap[key >> 5], 1u << (key & 31));
    }
  }
  pkey[p] = key;
}

// Pass 2: voxel id = rank of the cell; count the point and keep the max_pts lowest point indices
// of the voxel, sorted, with an atomicMin cascade (slot j ends up holding the j-th smallest index
// whatever the arrival order).
__global__ __launch_bounds__(256) void k_vox_assign(const uint32_t* __restrict__ pkey, uint32_t n,
                                                    const uint32_t* __restrict__ bitmap,
                                                    const uint32_t* __restrict__ prefix, int max_voxels, int max_pts,
                                                    uint32_t* counts, uint32_t* mins) {
  const uint32_t p = blockIdx.x * 256 + threadIdx.x;
  if (p >= n) return;
  const uint32_t key = pkey[p];
  if (key == 0xFFFFFFFFu) return;
  const uint32_t w = key >> 5, b = key & 31;
  const uint32_t id = prefix[w] + __popc(bitmap[w] & ((1u << b) - 1u));
  if (id >= (uint32_t)max_voxels) return;
  atomicAdd(&counts[id], 1u);
  uint32_t x = p;
  uint32_t* slot = mins + (size_t)id * max_pts;
  for (int j = 0; j < max_pts; ++j) {
    const uint32_t old = atomicMin(&slot[j], x);
    if (old == 0xFFFFFFFFu) break;  // slot was empty: nothing is displaced
    x = old > x ? old : x;
  }
}

// Pass 3: per voxel mean of the kept points, summed in point-index order in fp32.
__global__ __launch_bounds__(256) void k_vox_mean(const _Float16* __restrict__ pts, const uint32_t* n_vox_dev,
                                                  int max_voxels, int max_pts, int nf,
                                                  const uint32_t* __restrict__ counts,
                                                  const uint32_t* __restrict__ mins, _Float16* feats) {
  const uint32_t nv = eff_n(n_vox_dev, (uint32_t)max_voxels);
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  const uint32_t v = t / nf, f = t % nf;
  if (v >= nv) return;
  uint32_t cnt = counts[v];
  if (cnt > (uint32_t)max_pts) cnt = max_pts;
  const uint32_t* slot = mins + (size_t)v * max_pts;
  float s = 0.f;
  for (uint32_t j = 0; j < cnt; ++j) {
    const float x = (float)pts[(size_t)slot[j] * nf + f];
    s = j == 0 ? x : s + x;
  }
  s = s / (float)cnt;
  feats[(size_t)v * nf + f] = (_Float16)s;
}

}  // namespace scn

// ============================================================================================
// C ABI: stage-level entry points
// ============================================================================================
using namespace scn;

extern "C" {

uint64_t scn_hash_u64(uint64_t key) { return hash64(key); }
size_t scn_hash_capacity_for(uint32_t n) { return hash_capacity_for(n); }

int scn_hash_build(uint64_t* table_dev, size_t capacity, const int32_t* indices_dev, uint32_t n,
                   const uint32_t* n_dev, const int grid[3], void* stream) {
  SCN_REQUIRE(table_dev && grid && (indices_dev || n == 0), SCN_ERR_INVALID, "scn_hash_build: null pointer");
  SCN_REQUIRE(capacity >= hash_capacity_for(n) && (capacity & (capacity - 1)) == 0, SCN_ERR_CAPACITY,
              "scn_hash_build: capacity %zu must be a power of two >= %zu", capacity, hash_capacity_for(n));
  SCN_REQUIRE(grid_fits_u32(grid), SCN_ERR_UNSUPPORTED, "grid does not fit 32-bit keys");
  // the whole caller-provided table is used so that scn_hash_query can be given the same capacity
  int rc = fill_u32(table_dev, 0xFFFFFFFFu, capacity * 2, (hipStream_t)stream);
  if (rc) return rc;
  Int3 g{{grid[0], grid[1], grid[2]}};
  if (n) {
    hipLaunchKernelGGL(k_hash_insert, dim3(ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, table_dev,
                       (uint32_t)(capacity - 1), (const int4*)indices_dev, n, n_dev, g, (uint32_t*)nullptr,
                       (uint32_t*)nullptr);
    SCN_HIP(hipGetLastError());
  }
  return SCN_OK;
}

int scn_hash_query(const uint64_t* table_dev, size_t capacity, const int32_t* coords_dev, uint32_t n,
                   const int grid[3], int32_t* rows_out_dev, void* stream) {
  SCN_REQUIRE(table_dev && grid && rows_out_dev && (coords_dev || n == 0), SCN_ERR_INVALID, "scn_hash_query: null pointer");
  SCN_REQUIRE(capacity && (capacity & (capacity - 1)) == 0, SCN_ERR_INVALID, "capacity must be a power of two");
  if (n == 0) return SCN_OK;
  Int3 g{{grid[0], grid[1], grid[2]}};
  hipLaunchKernelGGL(k_hash_query, dim3(ceil_div(n, 256)), dim3(256), 0, (hipStream_t)stream, table_dev,
                     (uint32_t)(capacity - 1), (const int4*)coords_dev, n, g, rows_out_dev);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

// ---- voxelizer ------------------------------------------------------------------------------
scn_voxelizer* scn_voxelizer_create(const scn_voxelization_param* param) {
  if (!param || param->num_feature < 3 || param->max_voxels <= 0 || param->max_points_per_voxel <= 0 ||
      param->max_points <= 0) {
    set_error("scn_voxelizer_create: invalid parameter");
    return nullptr;
  }
  const int g[3] = {param->grid_size[0], param->grid_size[1], param->grid_size[2]};
  if (!grid_fits_u32(g)) {
    set_error("scn_voxelizer_create: grid does not fit 32-bit keys");
    return nullptr;
  }
  auto* v = new scn_voxelizer();
  v->p = *param;
  v->words = bitmap_words_for(g);
  const size_t mv = (size_t)param->max_voxels;
  bool ok = v->bitmap.alloc(v->words * 4) && v->prefix.alloc(v->words * 4) &&
            v->blocksum.alloc((v->words / kWordsPerBlock + 1) * 4) && v->pkey.alloc((size_t)param->max_points * 4) &&
            v->mins.alloc(mv * param->max_points_per_voxel * 4) && v->counts.alloc(mv * 4) &&
            v->feats.alloc(mv * param->num_feature * 2) && v->idx.alloc(mv * 16) && v->counters.alloc(64);
  if (ok) ok = hipMemset(v->counters.p, 0, 64) == hipSuccess && hipMemset(v->idx.p, 0, mv * 16) == hipSuccess &&
               hipMemset(v->feats.p, 0, mv * param->num_feature * 2) == hipSuccess &&
               hipHostMalloc((void**)&v->host_count, sizeof(uint32_t), hipHostMallocDefault) == hipSuccess;
  if (!ok) {
    delete v;
    return nullptr;
  }
  *v->host_count = 0;
  return v;
}

void scn_voxelizer_destroy(scn_voxelizer* v) {
  if (!v) return;
  if (v->host_count) (void)hipHostFree(v->host_count);
  delete v;
}

int scn_voxelizer_forward(scn_voxelizer* v, const void* points_fp16_dev, uint32_t num_points, int order,
                          void* stream_) {
  SCN_REQUIRE(v, SCN_ERR_INVALID, "scn_voxelizer_forward: null voxelizer");
  SCN_REQUIRE(order == SCN_ORDER_XYZ || order == SCN_ORDER_ZYX, SCN_ERR_INVALID, "Invalid output_order: %d", order);
  SCN_REQUIRE(points_fp16_dev || num_points == 0, SCN_ERR_INVALID, "scn_voxelizer_forward: null points");
  hipStream_t stream = (hipStream_t)stream_;
  if (num_points > (uint32_t)v->p.max_points) {
    SCN_LOGW("voxelization: %u points exceed max_points %d, the frame is cropped", num_points, v->p.max_points);
    num_points = (uint32_t)v->p.max_points;
  }
  const auto& p = v->p;
  VoxGeom g;
  for (int a = 0; a < 3; ++a) {
    g.mn[a] = p.min_range[a];
    g.mx[a] = p.max_range[a];
    g.vs[a] = p.voxel_size[a];
    g.g[a] = p.grid_size[a];
  }
  g.order = order;
  if (order == SCN_ORDER_ZYX) {
    g.og[0] = p.grid_size[2]; g.og[1] = p.grid_size[1]; g.og[2] = p.grid_size[0];
  } else {
    g.og[0] = p.grid_size[0]; g.og[1] = p.grid_size[1]; g.og[2] = p.grid_size[2];
  }
  g.nf = p.num_feature;
  g.max_voxels = p.max_voxels;
  g.max_pts = p.max_points_per_voxel;
  v->last_order = order;
  int rc = fill_u32(v->bitmap.p, 0u, v->words, stream);
  if (rc) return rc;
  rc = fill_u32(v->mins.p, 0xFFFFFFFFu, (size_t)p.max_voxels * p.max_points_per_voxel, stream);
  if (rc) return rc;
  rc = fill_u32(v->counts.p, 0u, (size_t)p.max_voxels, stream);
  if (rc) return rc;
  uint32_t* cnt = v->counters.as<uint32_t>();
  const uint32_t nblocks = (uint32_t)(v->words / kWordsPerBlock);
  if (num_points)
    hipLaunchKernelGGL(k_vox_mark, dim3(ceil_div(num_points, 256)), dim3(256), 0, stream,
                       (const _Float16*)points_fp16_dev, num_points, g, v->pkey.as<uint32_t>(), v->bitmap.as<uint32_t>());
  hipLaunchKernelGGL(k_bitmap_blocksum, dim3(nblocks), dim3(256), 0, stream, v->bitmap.as<uint32_t>(),
                     v->blocksum.as<uint32_t>());
  hipLaunchKernelGGL(k_scan_blocksums, dim3(1), dim3(1024), 0, stream, v->blocksum.as<uint32_t>(), nblocks, cnt,
                     (uint32_t)p.max_voxels);
  hipLaunchKernelGGL(k_bitmap_expand, dim3(nblocks), dim3(1024), 0, stream, v->bitmap.as<uint32_t>(),
                     v->blocksum.as<uint32_t>(), Int3{{g.og[0], g.og[1], g.og[2]}}, (uint32_t)p.max_voxels,
                     (int4*)v->idx.p, v->prefix.as<uint32_t>(), 0, (uint32_t*)nullptr);
  if (num_points) {
    hipLaunchKernelGGL(k_vox_assign, dim3(ceil_div(num_points, 256)), dim3(256), 0, stream, v->pkey.as<uint32_t>(),
                       num_points, v->bitmap.as<uint32_t>(), v->prefix.as<uint32_t>(), p.max_voxels,
                       p.max_points_per_voxel, v->counts.as<uint32_t>(), v->mins.as<uint32_t>());
    const uint32_t bound = (uint32_t)std::min<uint64_t>((uint64_t)p.max_voxels, num_points);
    hipLaunchKernelGGL(k_vox_mean, dim3(ceil_div(bound * p.num_feature, 256)), dim3(256), 0, stream,
                       (const _Float16*)points_fp16_dev, cnt, p.max_voxels, p.max_points_per_voxel, p.num_feature,
                       v->counts.as<uint32_t>(), v->mins.as<uint32_t>(), (_Float16*)v->feats.p);
  }
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

const void* scn_voxelizer_features(const scn_voxelizer* v) { return v ? v->feats.p : nullptr; }
const int32_t* scn_voxelizer_indices(const scn_voxelizer* v) { return v ? v->idx.as<int32_t>() : nullptr; }
const uint32_t* scn_voxelizer_num_voxels_dev(const scn_voxelizer* v) { return v ? v->counters.as<uint32_t>() : nullptr; }
const uint32_t* scn_voxelizer_points_per_voxel(const scn_voxelizer* v) { return v ? v->counts.as<uint32_t>() : nullptr; }

uint32_t scn_voxelizer_num_voxels(scn_voxelizer* v, void* stream) {
  if (!v) return 0;
  if (hipMemcpyAsync(v->host_count, v->counters.p, 4, hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess) return 0;
  if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) return 0;
  return *v->host_count;
}

void scn_voxelizer_grid_size(const scn_voxelizer* v, int order, int grid[3]) {
  if (!v || !grid) return;
  if (order == SCN_ORDER_ZYX) {
    grid[0] = v->p.grid_size[2] + 1; grid[1] = v->p.grid_size[1]; grid[2] = v->p.grid_size[0];
  } else {
    grid[0] = v->p.grid_size[0]; grid[1] = v->p.grid_size[1]; grid[2] = v->p.grid_size[2] + 1;
  }
}

// ---- rulebook -------------------------------------------------------------------------------
struct scn_rulebook {
  Rulebook rb;
};

scn_rulebook* scn_rulebook_create(uint32_t max_in, uint32_t max_out, int kernel_volume) {
  if (kernel_volume <= 0 || (max_in == 0 && max_out == 0)) {
    set_error("scn_rulebook_create: invalid arguments");
    return nullptr;
  }
  auto* r = new scn_rulebook();
  if (!r->rb.init(max_in, max_out, kernel_volume)) {
    delete r;
    return nullptr;
  }
  return r;
}
void scn_rulebook_destroy(scn_rulebook* rb) { delete rb; }

int scn_rulebook_build_subm(scn_rulebook* rb, const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev,
                            const int grid[3], const int ksize[3], const int dilation[3], void* stream) {
  SCN_REQUIRE(rb && grid && ksize && dilation && (indices_dev || n == 0), SCN_ERR_INVALID, "null pointer");
  return rb->rb.build_subm(indices_dev, n, n_dev, grid, ksize, dilation, nullptr, (hipStream_t)stream);
}
int scn_rulebook_build_sparse(scn_rulebook* rb, const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev,
                              const int grid[3], const int ksize[3], const int stride[3], const int padding[3],
                              const int dilation[3], void* stream) {
  SCN_REQUIRE(rb && grid && ksize && stride && padding && dilation && (indices_dev || n == 0), SCN_ERR_INVALID,
              "null pointer");
  return rb->rb.build_sparse(indices_dev, n, n_dev, grid, ksize, stride, padding, dilation, nullptr,
                             (hipStream_t)stream);
}
int scn_rulebook_build_inverse(scn_rulebook* rb, const scn_rulebook* forward, const uint32_t* n_in_dev, void* stream) {
  SCN_REQUIRE(rb && forward, SCN_ERR_INVALID, "null pointer");
  return rb->rb.build_inverse(forward->rb, n_in_dev, (hipStream_t)stream);
}
const int32_t* scn_rulebook_nbr(const scn_rulebook* rb) { return rb ? rb->rb.nbr.as<int32_t>() : nullptr; }
uint32_t scn_rulebook_nbr_ld(const scn_rulebook* rb) { return rb ? rb->rb.ld : 0; }
const int32_t* scn_rulebook_out_indices(const scn_rulebook* rb) { return rb ? rb->rb.out_indices : nullptr; }
const uint32_t* scn_rulebook_num_out_dev(const scn_rulebook* rb) { return rb ? rb->rb.counters.as<uint32_t>() : nullptr; }
const uint32_t* scn_rulebook_num_out_total_dev(const scn_rulebook* rb) {
  return rb ? rb->rb.counters.as<uint32_t>() + 1 : nullptr;
}
void scn_rulebook_out_grid(const scn_rulebook* rb, int grid[3]) {
  if (rb && grid)
    for (int a = 0; a < 3; ++a) grid[a] = rb->rb.geom.grid_out[a];
}
int scn_rulebook_pairs(scn_rulebook* rb, int32_t* pair_in_dev, int32_t* pair_out_dev, int64_t* offsets_dev,
                       uint64_t capacity, void* stream) {
  SCN_REQUIRE(rb && pair_in_dev && pair_out_dev && offsets_dev, SCN_ERR_INVALID, "null pointer");
  return rb->rb.pairs(pair_in_dev, pair_out_dev, offsets_dev, capacity, (hipStream_t)stream);
}

// ---- convolution ----------------------------------------------------------------------------
struct scn_conv {
  ConvWeights w;
};

scn_conv* scn_conv_create(const uint16_t* weight_fp16, const int weight_shape[5], const float* weight_dynamic_ranges,
                          const uint16_t* bias_fp16, int precision) {
  if (!weight_fp16 || !weight_shape || (precision != SCN_PRECISION_FP16 && precision != SCN_PRECISION_INT8)) {
    set_error("scn_conv_create: invalid arguments");
    return nullptr;
  }
  auto* c = new scn_conv();
  if (!c->w.init(weight_fp16, weight_shape, weight_dynamic_ranges, bias_fp16, precision)) {
    delete c;
    return nullptr;
  }
  return c;
}
void scn_conv_destroy(scn_conv* c) { delete c; }

int scn_conv_forward(const scn_conv* c, const scn_rulebook* rb, const scn_conv_io* io, void* stream) {
  SCN_REQUIRE(c && rb && io, SCN_ERR_INVALID, "scn_conv_forward: null pointer");
  SCN_REQUIRE(rb->rb.built, SCN_ERR_INVALID, "scn_conv_forward: rulebook not built");
  SCN_REQUIRE(rb->rb.geom.kvol == c->w.kvol, SCN_ERR_INVALID, "scn_conv_forward: kernel volume mismatch (%d vs %d)",
              rb->rb.geom.kvol, c->w.kvol);
  return conv_forward(c->w, rb->rb.nbr.as<int32_t>(), rb->rb.ld, rb->rb.n_out_dev(), rb->rb.n_bound_out,
                      rb->rb.n_out_hint(), *io,
                      (hipStream_t)stream);
}

// ---- elementwise / dense --------------------------------------------------------------------
int scn_convert_rows(const void* in_dev, int in_dtype, uint32_t in_c, uint32_t in_ld, float in_range, void* out_dev,
                     int out_dtype, uint32_t out_c, uint32_t out_ld, float out_range, int relu, uint32_t n,
                     const uint32_t* n_dev, void* stream) {
  return convert_rows(in_dev, in_dtype, in_c, in_ld, in_range, out_dev, out_dtype, out_c, out_ld, out_range, relu, n,
                      n_dev, (hipStream_t)stream);
}
int scn_add_relu(const void* a_dev, int a_dtype, float a_range, float a_requant_range, const void* b_dev, int b_dtype,
                 float b_range, float b_requant_range, void* out_dev, int out_dtype, float out_range, int relu,
                 uint32_t c, uint32_t n, const uint32_t* n_dev, void* stream) {
  return add_relu(a_dev, a_dtype, a_range, a_requant_range, b_dev, b_dtype, b_range, b_requant_range, out_dev,
                  out_dtype, out_range, relu, c, n, n_dev, (hipStream_t)stream);
}
int scn_scatter_dense(const void* feat_dev, int dtype, float dynamic_range, uint32_t c, uint32_t ld,
                      const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                      const int perm[5], void* out_fp16_dev, void* stream) {
  return scatter_dense(feat_dev, dtype, dynamic_range, c, ld, indices_dev, n, n_dev, dense_shape, perm, out_fp16_dev,
                       (hipStream_t)stream);
}

size_t scn_scatter_dense_map_cells(const int dense_shape[5], const int perm[5]) {
  return scatter_dense_map_cells(dense_shape, perm);
}

int scn_scatter_dense_with_map(const void* feat_dev, int dtype, float dynamic_range, uint32_t c, uint32_t ld,
                               const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                               const int perm[5], void* out_fp16_dev, int32_t* cell_map_dev, void* stream) {
  return scatter_dense(feat_dev, dtype, dynamic_range, c, ld, indices_dev, n, n_dev, dense_shape, perm, out_fp16_dev,
                       (hipStream_t)stream, false, cell_map_dev, false);
}

}  // extern "C"
