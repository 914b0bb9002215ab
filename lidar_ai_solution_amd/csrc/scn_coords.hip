// Coordinate side of the SCN path (gfx950): fills, the coordinate hash, bitmap rank (de-duplicates and
// orders keys), rulebooks as output-stationary neighbour tables nbr[k][out] with their pair compaction and
// inverse, and voxelization (bitmap rank for voxel ids + atomicMin cascade for the kept points).
// All kernels read row counts from device memory so that a forward pass never needs the host.
#include "scn_device.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace scn {

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

// Byte fill of an arbitrary range: the 16-byte aligned body in whole vectors, head and tail byte by byte.
__global__ __launch_bounds__(256) void k_fill_bytes(unsigned char* __restrict__ p, unsigned char value, size_t bytes) {
  const size_t head = min(bytes, (size_t)((16 - ((uintptr_t)p & 15)) & 15));
  const size_t body = (bytes - head) / 16;
  const size_t stride = (size_t)gridDim.x * 256;
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  const uint32_t v = value * 0x01010101u;
  const uint4 v4 = make_uint4(v, v, v, v);
  uint4* b = reinterpret_cast<uint4*>(p + head);
  for (size_t k = i; k < body; k += stride) b[k] = v4;
  if (i < head) p[i] = value;
  const size_t tail0 = head + body * 16;
  if (tail0 + i < bytes && i < 16) p[tail0 + i] = value;
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
// skip_if_zero (nullable): the "not in canonical order" flag of k_index_sorted_rows, which ran just before; while
// it is 0 the rows need no hash and the whole grid leaves at once.
__global__ __launch_bounds__(256) void k_hash_insert(uint64_t* slots, uint32_t mask, const int4* __restrict__ coords,
                                                     uint32_t n_bound, const uint32_t* n_dev, Int3 grid,
                                                     uint32_t* n_eff_out, uint32_t* filter,
                                                     const uint32_t* skip_if_zero, uint32_t* sorted_hint_host) {
  __shared__ uint32_t akeys[kAggSlots], avals[kAggSlots];
  const uint32_t r = blockIdx.x * blockDim.x + threadIdx.x;
  // (the flag first: a grid that only has to leave should not wait for the row count as well)
  const bool skip = skip_if_zero && *skip_if_zero == 0;
  // pinned host word: 1 when this build found the rows in canonical order, 0 when it did not or did not look.  The host
  // reads it when it enqueues a later build (a launch hint only, possibly one build behind).
  if (r == 0 && sorted_hint_host) *sorted_hint_host = skip ? 1u : 0u;
  if (skip && !(r == 0 && n_eff_out)) return;
  const uint32_t n = eff_n(n_dev, n_bound);
  if (r == 0 && n_eff_out) {
    n_eff_out[0] = n;
    n_eff_out[1] = n;
  }
  if (skip) return;
  if (filter) agg_init(akeys, avals);
  uint32_t key;
  if (r < n && coord_key(coords[r], grid, &key)) {
    table_insert(slots, mask, key, r);
    if (filter) agg_or(akeys, avals, filter, key >> 5, 1u << (key & 31));
  }
  if (filter) agg_flush(akeys, avals, filter);
}

// Rows in canonical order (strictly ascending linear index, every coordinate inside the grid): the first row of
// every occupied 32-cell word writes the word's occupancy bits and its own row number.  The bits of a word's run of
// rows (at most 32, consecutive) are combined inside the wavefront by a segmented suffix OR over lane shuffles; a run
// that is whole inside one wavefront is written with a plain store, the two parts of one that crosses into the next
// wavefront with an atomic OR each (the bitmap is cleared beforehand).  Any row that breaks the order raises
// *unsorted; what was written by then is a subset of the true occupancy, which the hash insert that follows
// completes with its atomics.
__global__ __launch_bounds__(256) void k_index_sorted_rows(const int4* __restrict__ coords, uint32_t n_bound,
                                                           const uint32_t* n_dev, Int3 grid, uint32_t* bitmap,
                                                           uint32_t* first_row, uint32_t* unsorted) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t r = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  const bool have = r < n;
  uint32_t key = 0;
  const bool ok = have && coord_key(coords[r], grid, &key);
  // the row before: the neighbouring lane's, or a load for the first lane of a wavefront
  uint32_t kp = (uint32_t)__shfl_up((int)key, 1, 64);
  bool okp = __shfl_up((int)ok, 1, 64) != 0;
  if (lane == 0 && have && r > 0) okp = coord_key(coords[r - 1], grid, &kp);
  if (have && (!ok || (r > 0 && (!okp || kp >= key)))) *unsorted = 1u;
  const uint32_t word = ok ? key >> 5 : 0xFFFFFF00u + (uint32_t)lane;   // (rows without a cell never share a word)
  const bool leader = ok && (r == 0 || !okp || (kp >> 5) != word);
  uint32_t bits = ok ? 1u << (key & 31) : 0u;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const uint32_t ob = (uint32_t)__shfl_down((int)bits, d, 64);
    const uint32_t ow = (uint32_t)__shfl_down((int)word, d, 64);
    if (lane + d < 64 && ow == word) bits |= ob;   // equal words are contiguous, so the doubling covers the run
  }
  const bool reaches_end = (uint32_t)__shfl((int)word, 63, 64) == word;   // the run may go on in the next wavefront
  if (leader) {
    if (reaches_end)
      atomicOr(&bitmap[word], bits);
    else
      bitmap[word] = bits;
    first_row[word] = r;
  } else if (lane == 0 && ok) {
    atomicOr(&bitmap[word], bits);   // the part of a run that began in the wavefront before
  }
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
  if ((words + 4) > filter.bytes / 4 && !filter.alloc((words + 4) * 4)) return false;
  filter_words = words;
  static const bool no_rank = [] {
    const char* e = getenv("SCN_INPUT_INDEX");   // "hash": never try the canonical-order index (A/B measurements)
    return e && !strcmp(e, "hash");
  }();
  if (!no_rank) {
    if (words > first_row.bytes / 4 && !first_row.alloc(words * 4)) return false;
    if (!sorted_hint.p) {
      if (!sorted_hint.alloc(16)) return false;
      *sorted_hint.as<uint32_t>() = 0;
    }
  }
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
      rc = fill_u32(t.filter.p, 0u, t.filter_fill_words(), stream);   // (with the order flag behind the words)
      if (rc) return rc;
    }
  }
  CoordTable& tm = const_cast<CoordTable&>(t);
  tm.precleared_for = 0xFFFFFFFFu;
  Int3 g{{grid[0], grid[1], grid[2]}};
  const uint32_t blocks = n ? ceil_div(n, 256) : 1;
  // the canonical-order index first, when the previous build found that order (or nothing is known yet, or it is
  // time to look again); the hash insert then runs only if the order does not hold
  tm.probed = t.filter_words && t.first_row.p && t.sorted_hint.p &&
              (t.builds == 0 || *t.sorted_hint.as<uint32_t>() != 0 || t.builds % 16 == 0);
  tm.builds++;
  if (tm.probed)
    hipLaunchKernelGGL(k_index_sorted_rows, dim3(blocks), dim3(256), 0, stream, (const int4*)idx, n, n_dev, g,
                       t.filter.as<uint32_t>(), t.first_row.as<uint32_t>(), t.unsorted_flag());
  hipLaunchKernelGGL(k_hash_insert, dim3(blocks), dim3(256), 0, stream, t.slots(), t.mask,
                     (const int4*)idx, n, n_dev, g, n_eff_out, t.filter_words ? t.filter.as<uint32_t>() : nullptr,
                     tm.probed ? (const uint32_t*)t.unsorted_flag() : (const uint32_t*)nullptr,
                     t.sorted_hint.as<uint32_t>());
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

// nbr[k][o] = row of the input at  o*stride - pad + k*dilation  (or -1).  grid.y = (k0, k1); a thread
// walks the K2 offsets of its line (independent lookups, coalesced stores per offset): short chains and
// K0*K1 times the rows in threads, because the first table of a frame is on the critical path.
// Used for both kinds: submanifold passes stride 1 and pad = floor(K/2)*dilation.
// Thread (0,0) also publishes the row count for the kernels that follow (n_publish, nullable).
__global__ __launch_bounds__(256) void k_build_nbr(const int4* __restrict__ out_coords, const uint32_t* n_out_dev,
                                                   uint32_t n_bound, GeomDev g, CoordLookup lk, int32_t* nbr,
                                                   uint32_t ld, int identity_center, uint32_t* n_publish,
                                                   uint32_t* n_host) {
  const uint32_t n = eff_n(n_out_dev, n_bound);
  const uint32_t o = blockIdx.x * 256 + threadIdx.x;
  // a hash table whose build found the rows in canonical order answers by rank
  const bool by_rank = lk.unsorted != nullptr && *lk.unsorted == 0;
  if (by_rank) {
    lk.bitmap = lk.filter;
    lk.prefix = lk.first_row;
    lk.rank_cap = 0xFFFFFFFFu;
  }
  if (o == 0 && blockIdx.y == 0) {
    if (n_publish) {
      n_publish[0] = n;
      n_publish[1] = n;
    }
    if (n_host) *n_host = n;  // pinned host word: the row count as a launch hint for the next forward
  }
  const int k01 = blockIdx.y;  // k0 * K1 + k1
  if (o >= n) {
    // the convolution kernels fetch table entries four rows at a time within a 32-row tile: the rows
    // between the count and the next multiple of 32 read as "no neighbour"
    if (o < ((n + 31u) & ~31u))
      for (int k = 0; k < g.ks[2]; ++k) nbr[(size_t)(k01 * g.ks[2] + k) * ld + o] = -1;
    return;
  }
  const int k0 = k01 / g.ks[1], k1 = k01 - k0 * g.ks[1];
  const int4 c = out_coords[o];
  const int i0 = c.y * g.st[0] - g.pd[0] + k0 * g.dl[0];
  const int i1 = c.z * g.st[1] - g.pd[1] + k1 * g.dl[1];
  const bool ok1 = c.x == 0 && i0 >= 0 && i0 < g.gi[0] && i1 >= 0 && i1 < g.gi[1];
  const bool centre01 = identity_center && k0 == g.ks[0] / 2 && k1 == g.ks[1] / 2;
  const uint32_t line = ((uint32_t)i0 * (uint32_t)g.gi[1] + (uint32_t)i1) * (uint32_t)g.gi[2];
#pragma unroll 3
  for (int k2 = 0; k2 < g.ks[2]; ++k2) {
    const int i2 = c.w * g.st[2] - g.pd[2] + k2 * g.dl[2];
    int32_t res = -1;
    if (centre01 && k2 == g.ks[2] / 2) {
      res = (int32_t)o;
    } else if (ok1 && i2 >= 0 && i2 < g.gi[2]) {
      res = coord_row(lk, line + (uint32_t)i2);
    }
    nbr[(size_t)(k01 * g.ks[2] + k2) * ld + o] = res;
  }
}

// Strided rulebooks build their table from the input side: an output row has 27 candidate inputs of which a
// lidar frame fills 1 .. 5, an input row has at most 27 outputs that all exist.  Two kernels: every entry of the
// rows in use becomes -1 (16-byte stores; rows up to the next multiple of 32, see Rulebook::nbr), then one thread
// per (input row, k0, k1) walks k2, finds the output cell o = (i + pad - k dil) / stride where that division is
// exact, its row by bitmap rank, and enters itself.  For a fixed offset an output has one input cell, so entries
// have one writer unless the caller's coordinates repeat; the smallest row then wins, as in the coordinate hash.
__global__ __launch_bounds__(256) void k_clear_table(int32_t* nbr, uint32_t ld, const uint32_t* n_out_dev,
                                                     uint32_t n_bound, uint32_t* n_host) {
  const uint32_t n = eff_n(n_out_dev, n_bound);
  if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0 && n_host) *n_host = n;
  const uint32_t j = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (j >= ((n + 31u) & ~31u)) return;
  *reinterpret_cast<int4*>(nbr + (size_t)blockIdx.y * ld + j) = make_int4(-1, -1, -1, -1);
}

__global__ __launch_bounds__(256) void k_scatter_nbr(const int4* __restrict__ in_coords, const uint32_t* n_in_dev,
                                                     uint32_t n_in_bound, GeomDev g, CoordLookup out_lk, int32_t* nbr,
                                                     uint32_t ld) {
  const uint32_t n = eff_n(n_in_dev, n_in_bound);
  const uint32_t i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int4 c = in_coords[i];
  if (c.x != 0 || c.y < 0 || c.y >= g.gi[0] || c.z < 0 || c.z >= g.gi[1] || c.w < 0 || c.w >= g.gi[2]) return;
  const int k01 = blockIdx.y;
  const int k0 = k01 / g.ks[1], k1 = k01 - k0 * g.ks[1];
  const int t0 = c.y + g.pd[0] - k0 * g.dl[0], t1 = c.z + g.pd[1] - k1 * g.dl[1];
  if (t0 < 0 || t1 < 0) return;
  const int o0 = t0 / g.st[0], o1 = t1 / g.st[1];
  if (o0 * g.st[0] != t0 || o1 * g.st[1] != t1 || o0 >= g.go[0] || o1 >= g.go[1]) return;
  const uint32_t line = ((uint32_t)o0 * (uint32_t)g.go[1] + (uint32_t)o1) * (uint32_t)g.go[2];
  for (int k2 = 0; k2 < g.ks[2]; ++k2) {
    const int t2 = c.w + g.pd[2] - k2 * g.dl[2];
    if (t2 < 0) continue;
    const int o2 = t2 / g.st[2];
    if (o2 * g.st[2] != t2 || o2 >= g.go[2]) continue;
    const int32_t o = coord_row(out_lk, line + (uint32_t)o2);
    if (o < 0) continue;   // (an output beyond the row bound)
    atomicMin(reinterpret_cast<uint32_t*>(nbr) + (size_t)(k01 * g.ks[2] + k2) * ld + (uint32_t)o, i);
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
  hipLaunchKernelGGL(k_build_nbr, dim3(blocks, rb.geom.ks[0] * rb.geom.ks[1]), dim3(256), 0, stream, (const int4*)out_coords, n_dev,
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
  if (probed) {
    lk.unsorted = unsorted_flag();
    lk.first_row = first_row.as<uint32_t>();
  }
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
  plan.built = false;   // a tile plan describes the table of one build
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
  plan.built = false;   // a tile plan describes the table of one build
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
  // The table: from the output side (every output row looks up its candidate inputs) or from the input side (see
  // k_scatter_nbr).  The first costs rows_out x volume look-ups, the second a clear of as many entries plus two
  // dependent loads and an atomic per pair: measured on a 123 k -> 322 k-row stage (1.3 pairs per output) 37 -> 21 us
  // from the input side, on 322 k -> 215 k rows (4.7 pairs per output) 13 us slower.  So: the input side when the
  // outputs expected (the previous forward's count) are at least twice the inputs.  SCN_RULEBOOK_TABLE=gather /
  // scatter forces one.
  static const int forced = [] {
    const char* e = getenv("SCN_RULEBOOK_TABLE");
    return !e ? 0 : !strcmp(e, "gather") ? 1 : !strcmp(e, "scatter") ? 2 : 0;
  }();
  const bool gather_build = forced == 1 || (forced == 0 && (uint64_t)n_out_hint() < 2ull * n);
  if (gather_build) {
    rc = launch_build_nbr(*this, out_indices, cnt, n_bound_out, false, nullptr, stream);
    if (rc) return rc;
  } else {
    const uint32_t pos = (n_bound_out + 31u) & ~31u;
    if (pos)
      hipLaunchKernelGGL(k_clear_table, dim3(ceil_div(pos / 4, 256), geom.kvol), dim3(256), 0, stream, nbr.as<int32_t>(), ld,
                         cnt, n_bound_out, host_count.as<uint32_t>());
    else
      *host_count.as<uint32_t>() = 0;
    if (n && pos)
      hipLaunchKernelGGL(k_scatter_nbr, dim3(ceil_div(n, 256), geom.ks[0] * geom.ks[1]), dim3(256), 0, stream,
                         (const int4*)idx, n_dev, n, gd, out_lookup(), nbr.as<int32_t>(), ld);
    SCN_HIP(hipGetLastError());
  }
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
  plan.built = false;   // a tile plan describes the table of one build
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
  // (and the rows up to the next multiple of 32, which the convolution kernels may fetch)
  const uint32_t fill_rows = std::min((n_bound_out + 31u) & ~31u, ld);
  if (fill_rows)
    hipLaunchKernelGGL(k_fill_table_rows, dim3(ceil_div(fill_rows, 256), geom.kvol), dim3(256), 0, stream,
                       nbr.as<int32_t>(), ld, fill_rows, -1);
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

// The voxelizer keeps its working memory clean between calls instead of clearing it at the start of each:
//   cells     uint2 per 32 cells: .x occupancy bits, .y rank of the word's first bit.  Bits are cleared at the end of
//             the forward that set them, one store per point (k_vox_mean).
//   flags     one word per block of 1024 words: some cell of the block is occupied; cleared the same way.  (Walking
//             a second-level bitmap of the occupied words instead -- one thread per 32 words, 82 workgroups -- was
//             measured at 16 + 46 us for the two rank passes against 5 + 17 us: few threads with dependent loads.)
//   slots     [max_voxels][max_points] point indices with a phase bit above them: 1 for the slots filled in arrival
//             order, 0 for the cascade of the voxels that overflow, so that to the cascade (atomicMin) a slot of the
//             arrival phase is an empty one.  Never cleared: a forward writes every slot that it reads or that its
//             cascade can reach (the first min(count, max_points) of a voxel), so what earlier forwards left
//             behind them is never looked at.  No state on the host either: a captured forward replays as it is.
// Atomics that every XCD must see are the cost of this stage (they are served by the memory side, not by an XCD's L2),
// so a point costs two: the occupancy bit, and its voxel's counter, whose old value is its slot.  A voxel that
// receives more than max_points points needs the lowest indices among them, which arrival order does not give: those
// voxels' points (none in most frames: the pass leaves at once when no counter overflowed) go through a cascade.
// One forward = mark, block sums, rank, assign, overflow, mean.
constexpr uint32_t kVoxTagShift = 24;     // point indices stay below 2^24
constexpr uint32_t kVoxTagArrival = 1, kVoxTagCascade = 0;

// Pass 1 over the point stream (PT: fp16 points, or the fp32 points of CUDA-CenterPoint's preprocessing,
// src/preprocess_kernels.cu:70-98): cell key per point, occupancy bit, and the flag of the cell's block.
template <typename PT>
__global__ __launch_bounds__(256) void k_vox_mark(const PT* __restrict__ pts, uint32_t n, VoxGeom g,
                                                  uint32_t* pkey, uint2* cells, uint32_t* flags) {
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
      const uint32_t bit = 1u << (key & 31);
      const uint32_t old = atomicOr(&cells[key >> 5].x, bit);
      if (!(old & bit)) flags[key >> 15] = 1u;   // (1024 words of 32 cells per block)
    }
  }
  pkey[p] = key;
}

// Pass 2a: occupied cells per block of 1024 words; a block whose flag is down is not read.
__global__ __launch_bounds__(256) void k_vox_blocksum(const uint2* __restrict__ cells, const uint32_t* __restrict__ flags,
                                                      uint32_t* blocksum) {
  __shared__ uint32_t scratch[17];
  if (flags[blockIdx.x] == 0) {   // (the whole workgroup)
    if (threadIdx.x == 0) blocksum[blockIdx.x] = 0;
    return;
  }
  const uint4* w = reinterpret_cast<const uint4*>(cells + (size_t)blockIdx.x * 1024);   // two words' (bits, rank) each
  uint32_t c = 0;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const uint4 v = w[j * 256 + threadIdx.x];
    c += __popc(v.x) + __popc(v.z);
  }
  uint32_t total;
  (void)block_exclusive_scan(c, scratch, &total);
  if (threadIdx.x == 0) blocksum[blockIdx.x] = total;
}

// Pass 2b, one workgroup per block of 1024 words (four per thread): ranks.  Every block with an occupied cell adds up
// the counts of the blocks before it, writes the rank of each occupied word's first bit next to its bits and the
// coordinate rows of its cells; the last block publishes the totals; all of them zero the per-voxel point counts.
__global__ __launch_bounds__(256) void k_vox_rank(uint2* cells, const uint32_t* __restrict__ blocksum, Int3 grid,
                                                  uint32_t cap, int4* coords_out, uint32_t* counters,
                                                  uint32_t* counts) {
  __shared__ uint32_t scratch[17];
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < cap; i += (size_t)gridDim.x * 256) counts[i] = 0;
  const uint32_t own = blocksum[blockIdx.x];
  if (own == 0 && blockIdx.x != gridDim.x - 1) return;   // (the whole workgroup; the last block publishes the totals)
  uint32_t part = 0;
  for (uint32_t i = threadIdx.x; i < blockIdx.x; i += 256) part += blocksum[i];
  uint32_t base;
  (void)block_exclusive_scan(part, scratch, &base);
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == 0) {
    const uint32_t all = base + own;
    counters[1] = all;
    counters[0] = all < cap ? all : cap;
  }
  if (own == 0) return;   // (the whole workgroup)
  const size_t w0 = (size_t)blockIdx.x * 1024 + (size_t)threadIdx.x * 4;
  uint32_t bits[4];
  uint32_t c = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    bits[j] = cells[w0 + j].x;
    c += __popc(bits[j]);
  }
  uint32_t total;
  uint32_t rank = base + block_exclusive_scan(c, scratch, &total);
  if (c == 0) return;
  const uint32_t g12 = (uint32_t)grid.v[1] * (uint32_t)grid.v[2];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    uint32_t bj = bits[j];
    if (bj == 0) continue;
    cells[w0 + j].y = rank;
    while (bj) {
      const int b = __ffs(bj) - 1;
      bj &= bj - 1;
      if (rank < cap) {
        const uint32_t key = (uint32_t)(w0 + j) * 32u + (uint32_t)b;
        const uint32_t i0 = key / g12, rem = key - i0 * g12;
        const uint32_t i1 = rem / (uint32_t)grid.v[2], i2 = rem - i1 * (uint32_t)grid.v[2];
        coords_out[rank] = make_int4(0, (int)i0, (int)i1, (int)i2);
      }
      rank++;
    }
  }
}

// Lanes of a wave that follow each other with the same cell (a real sweep lists its points ring by ring): the run's
// first lane, its length, and this lane's place in it.  All 64 lanes call this.
struct VoxRun {
  int start, len, pos;
};
__device__ __forceinline__ VoxRun vox_run(uint32_t key, int lane) {
  const uint32_t prev = (uint32_t)__shfl_up((int)key, 1, 64);
  const bool head = lane == 0 || key != prev;
  const uint64_t heads = __ballot(head);
  const uint64_t upto = heads & (lane == 63 ? ~0ull : ((2ull << lane) - 1ull));   // heads at or below this lane
  const int start = 63 - __clzll((long long)upto);
  const uint64_t above = lane == 63 ? 0ull : heads & ~((2ull << lane) - 1ull);
  const int end = above ? __ffsll((long long)above) - 1 : 64;
  VoxRun r;
  r.start = start;
  r.len = end - start;
  r.pos = lane - start;
  return r;
}

// Pass 3: voxel id = rank of the cell; the voxel's counter gives the point its slot (arrival order; a run of lanes
// with one cell adds its length once and takes consecutive slots).  Raises *overflow when a voxel receives more
// points than it has slots.
__global__ __launch_bounds__(256) void k_vox_assign(const uint32_t* __restrict__ pkey, uint32_t n,
                                                    const uint2* __restrict__ cells, int max_voxels, int max_pts,
                                                    uint32_t tag, uint32_t* counts, uint32_t* slots, uint32_t* overflow,
                                                    int always) {
  const uint32_t p = blockIdx.x * 256 + threadIdx.x;
  const int lane = threadIdx.x & 63;
  if (always && p == 0) *overflow = 1u;   // (more slots than pass 4 puts in order: every voxel goes through pass 3b)
  const uint32_t key = p < n ? pkey[p] : 0xFFFFFFFFu;
  const VoxRun r = vox_run(key, lane);
  uint32_t id = 0xFFFFFFFFu;
  if (key != 0xFFFFFFFFu) {
    const uint2 ci = cells[key >> 5];
    id = ci.y + __popc(ci.x & ((1u << (key & 31)) - 1u));
  }
  const bool take = id < (uint32_t)max_voxels;
  uint32_t base = 0;
  if (take && r.pos == 0) base = atomicAdd(&counts[id], (uint32_t)r.len);
  base = (uint32_t)__shfl((int)base, r.start, 64);
  if (!take) return;
  const uint32_t at = base + (uint32_t)r.pos;
  if (at < (uint32_t)max_pts)
    slots[(size_t)id * max_pts + at] = (tag << kVoxTagShift) | p;
  else if (at == (uint32_t)max_pts)
    *overflow = 1u;
}

// Pass 3b, only for frames in which some voxel overflowed: every point of such a voxel enters an atomicMin cascade
// over the voxel's slots (slot j ends up holding the j-th smallest index whatever the arrival order; the slots that
// pass 3 filled carry the larger tag and count as empty).  Of a run of lanes only the first max_pts can be among the
// max_pts lowest.  Two launches: the first lanes of the runs (phase 0), then the others (phase 1).  A voxel next to
// the sensor holds a thousand points in a hundred runs, and read-modify-writes on one 64-byte line are carried out one
// after the other by the memory side, about ten per microsecond: all candidates at once are over a thousand of them
// (135 us on the reference's demo sweep), while after phase 0 the slots hold ten low indices and nearly every
// other candidate leaves on the reads in front of the cascade (86 us for the two launches).  (A bound per voxel from
// the indices that pass 3 happened to store -- the lowest max_pts cannot lie above the largest of any max_pts -- in
// place of phase 0: 113 us; arrival order follows index order too loosely for it.)
__global__ __launch_bounds__(256) void k_vox_overflow(const uint32_t* __restrict__ pkey, uint32_t n,
                                                      const uint2* __restrict__ cells, int max_voxels, int max_pts,
                                                      uint32_t tag, const uint32_t* __restrict__ counts, uint32_t* slots,
                                                      const uint32_t* __restrict__ overflow, int always, int phase) {
  if (*overflow == 0) return;
  const int lane = threadIdx.x & 63;
  // (whole waves run every round of the loop: the run bookkeeping is wave-wide)
  for (uint32_t p0 = blockIdx.x * 256; p0 < n; p0 += gridDim.x * 256) {
    const uint32_t p = p0 + threadIdx.x;
    const uint32_t key = p < n ? pkey[p] : 0xFFFFFFFFu;
    const VoxRun r = vox_run(key, lane);
    if (key == 0xFFFFFFFFu || r.pos >= max_pts || (phase == 0) != (r.pos == 0)) continue;
    const uint2 ci = cells[key >> 5];
    const uint32_t id = ci.y + __popc(ci.x & ((1u << (key & 31)) - 1u));
    if (id >= (uint32_t)max_voxels || (!always && counts[id] <= (uint32_t)max_pts)) continue;
    uint32_t x = (tag << kVoxTagShift) | p;
    uint32_t* slot = slots + (size_t)id * max_pts;
    // A voxel of hundreds of points (next to the sensor) would send every one of them down the same ten addresses,
    // starting with the first.  Slot values only fall and stay in ascending order, so the slots that hold less than
    // this point now (plain loads) will always do: the point enters the cascade behind them, and not at all when
    // that is every slot.
    // (Loads at device scope: the atomics are carried out by the memory side, and an ordinary load could be served
    // from a copy that never sees them.  Read-modify-writes on one 64-byte line run one after the other, at about ten
    // per microsecond: without these reads the frame's fullest voxel alone sets the time of the pass.)
    // (Not when every voxel takes this pass: a voxel with fewer points than slots then keeps, in the slots behind them,
    // what an earlier forward's cascade left there, and those must not be read.)
    int j0 = 0;
    if (!always) {
      const uint32_t last = __hip_atomic_load(&slot[max_pts - 1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((last >> kVoxTagShift) == tag && last < x) continue;
    }
    for (; !always && j0 < max_pts; ++j0) {
      const uint32_t cur = __hip_atomic_load(&slot[j0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((cur >> kVoxTagShift) != tag || cur > x) break;
    }
    for (int j = j0; j < max_pts; ++j) {
      const uint32_t old = atomicMin(&slot[j], x);
      if ((old >> kVoxTagShift) != tag) break;  // the slot was empty (cleared, an earlier call's, or pass 3's): nothing is displaced
      x = old > x ? old : x;
    }
  }
}

// Mean of cnt <= N points whose indices stand in slot[] in any order: indices through a bitonic network (ascending,
// padding last), values added in that order in fp32.  N a power of two; nf <= kVoxMaxFeatures.
constexpr int kVoxMaxSlots = 16;
constexpr int kVoxMaxFeatures = 8;
template <typename PT, int N>
__device__ __forceinline__ void vox_ordered_mean(const PT* __restrict__ pts, const uint32_t* __restrict__ slot, uint32_t cnt,
                                                 int nf, _Float16* out) {
  const uint32_t pmask = (1u << kVoxTagShift) - 1u;
  uint32_t idx[N];
#pragma unroll
  for (int j = 0; j < N; ++j) idx[j] = (uint32_t)j < cnt ? slot[j] & pmask : 0xFFFFFFFFu;
#pragma unroll
  for (int k = 2; k <= N; k <<= 1)
#pragma unroll
    for (int d = k >> 1; d > 0; d >>= 1)
#pragma unroll
      for (int i = 0; i < N; ++i) {
        const int l = i ^ d;
        if (l > i) {
          const bool up = (i & k) == 0;
          const uint32_t a = idx[i], b = idx[l];
          const bool sw = (a > b) == up;
          idx[i] = sw ? b : a;
          idx[l] = sw ? a : b;
        }
      }
  float s[kVoxMaxFeatures];
#pragma unroll
  for (int f = 0; f < kVoxMaxFeatures; ++f) s[f] = 0.f;
#pragma unroll
  for (int r = 0; r < N; ++r) {
    if ((uint32_t)r < cnt) {
      const PT* q = pts + (size_t)idx[r] * nf;
#pragma unroll
      for (int f = 0; f < kVoxMaxFeatures; ++f)
        if (f < nf) {
          const float x = (float)q[f];
          s[f] = r == 0 ? x : s[f] + x;
        }
    }
  }
#pragma unroll
  for (int f = 0; f < kVoxMaxFeatures; ++f)
    if (f < nf) out[f] = (_Float16)(s[f] / (float)cnt);
}

// Pass 4, one thread per voxel: mean of the kept points, summed in point-index order in fp32 (slots in arrival order
// are put in order first, by a sorting network over at most 16 of them); and, one thread per point, the occupancy bits
// and block flags of this frame back to zero for the next one.
template <typename PT>
__global__ __launch_bounds__(256) void k_vox_mean(const PT* __restrict__ pts, const uint32_t* n_vox_dev,
                                                  int max_voxels, int max_pts, int nf,
                                                  const uint32_t* __restrict__ counts,
                                                  const uint32_t* __restrict__ slots, _Float16* feats,
                                                  const uint32_t* __restrict__ pkey, uint32_t n_points, uint2* cells,
                                                  uint32_t* flags, uint32_t* overflow) {
  const uint32_t t = blockIdx.x * 256 + threadIdx.x;
  if (t == 0) *overflow = 0;   // (pass 3b of this forward has run)
  if (t < n_points) {
    const uint32_t key = pkey[t];
    if (key != 0xFFFFFFFFu) {
      cells[key >> 5].x = 0;
      flags[key >> 15] = 0;
    }
  }
  const uint32_t nv = eff_n(n_vox_dev, (uint32_t)max_voxels);
  const uint32_t v = t;
  if (v >= nv) return;
  const uint32_t all = counts[v];
  const uint32_t cnt = all > (uint32_t)max_pts ? (uint32_t)max_pts : all;
  const uint32_t* slot = slots + (size_t)v * max_pts;
  const uint32_t pmask = (1u << kVoxTagShift) - 1u;
  _Float16* out = feats + (size_t)v * nf;
  if (max_pts > kVoxMaxSlots || nf > kVoxMaxFeatures) {
    // more slots or features than the registers below hold: every voxel went through the cascade (see the host
    // side), its slots are in order
    for (int f = 0; f < nf; ++f) {
      float s = 0.f;
      for (uint32_t j = 0; j < cnt; ++j) {
        const float x = (float)pts[(size_t)(slot[j] & pmask) * nf + f];
        s = j == 0 ? x : s + x;
      }
      out[f] = (_Float16)(s / (float)cnt);
    }
    return;
  }
  if (cnt <= 2)
    vox_ordered_mean<PT, 2>(pts, slot, cnt, nf, out);
  else if (cnt <= 4)
    vox_ordered_mean<PT, 4>(pts, slot, cnt, nf, out);
  else if (cnt <= 8)
    vox_ordered_mean<PT, 8>(pts, slot, cnt, nf, out);
  else
    vox_ordered_mean<PT, kVoxMaxSlots>(pts, slot, cnt, nf, out);
}

}  // namespace scn

// ============================================================================================
// C ABI: stage-level entry points (hash, voxelizer, rulebook)
// ============================================================================================
using namespace scn;

extern "C" {

int scn_memset_async(void* dev, unsigned char value, size_t bytes, void* stream) {
  if (bytes == 0) return SCN_OK;
  SCN_REQUIRE(dev, SCN_ERR_INVALID, "scn_memset_async: null pointer");
  size_t blocks = (bytes / 16 + 255) / 256;
  blocks = blocks < 1 ? 1 : blocks > 4096 ? 4096 : blocks;
  hipLaunchKernelGGL(k_fill_bytes, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (unsigned char*)dev, value,
                     bytes);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

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
                       (uint32_t*)nullptr, (const uint32_t*)nullptr, (uint32_t*)nullptr);
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
  if ((uint64_t)param->max_points >= (1ull << kVoxTagShift)) {
    set_error("scn_voxelizer_create: max_points must be below 2^24");
    delete v;
    return nullptr;
  }
  // bitmap: uint2 per word (bits, rank of the first bit); clean = zero bits, zero block counts, cleared slots
  bool ok = v->bitmap.alloc(v->words * 8) && v->blocksum.alloc((v->words / kWordsPerBlock + 1) * 4) &&
            v->flags.alloc((v->words / kWordsPerBlock + 1) * 4) &&
            v->pkey.alloc((size_t)param->max_points * 4) &&
            v->mins.alloc(mv * param->max_points_per_voxel * 4) && v->counts.alloc(mv * 4) &&
            v->feats.alloc(mv * param->num_feature * 2) && v->idx.alloc(mv * 16) && v->counters.alloc(64);
  if (ok) ok = hipMemset(v->bitmap.p, 0, v->words * 8) == hipSuccess &&
               hipMemset(v->blocksum.p, 0, (v->words / kWordsPerBlock + 1) * 4) == hipSuccess &&
               hipMemset(v->flags.p, 0, (v->words / kWordsPerBlock + 1) * 4) == hipSuccess &&
               hipMemset(v->mins.p, 0xFF, mv * param->max_points_per_voxel * 4) == hipSuccess &&
               hipMemset(v->counts.p, 0, mv * 4) == hipSuccess &&
               hipMemset(v->counters.p, 0, 64) == hipSuccess && hipMemset(v->idx.p, 0, mv * 16) == hipSuccess &&
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
  return scn_voxelizer_forward_points(v, points_fp16_dev, SCN_DTYPE_FP16, num_points, order, stream_);
}

int scn_voxelizer_forward_points(scn_voxelizer* v, const void* points_fp16_dev, int points_dtype, uint32_t num_points,
                                 int order, void* stream_) {
  SCN_REQUIRE(v, SCN_ERR_INVALID, "scn_voxelizer_forward: null voxelizer");
  SCN_REQUIRE(order == SCN_ORDER_XYZ || order == SCN_ORDER_ZYX, SCN_ERR_INVALID, "Invalid output_order: %d", order);
  SCN_REQUIRE(points_fp16_dev || num_points == 0, SCN_ERR_INVALID, "scn_voxelizer_forward: null points");
  SCN_REQUIRE(points_dtype == SCN_DTYPE_FP16 || points_dtype == SCN_DTYPE_FP32, SCN_ERR_INVALID,
              "scn_voxelizer_forward: points must be fp16 or fp32 (dtype %d)", points_dtype);
  const bool p32 = points_dtype == SCN_DTYPE_FP32;
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
  const uint32_t tag_arrival = kVoxTagArrival, tag_cascade = kVoxTagCascade;   // (the working memory is clean: see the kernels)
  // (more slots or features than pass 4 puts in order in registers: every voxel goes through the cascade of pass 3b)
  const int always = (p.max_points_per_voxel > kVoxMaxSlots || p.num_feature > kVoxMaxFeatures) ? 1 : 0;
  uint32_t* cnt = v->counters.as<uint32_t>();
  uint32_t* overflow = cnt + 4;
  uint2* cells = reinterpret_cast<uint2*>(v->bitmap.p);
  uint32_t* flags = v->flags.as<uint32_t>();
  const uint32_t nblocks = (uint32_t)(v->words / kWordsPerBlock);
  if (num_points && p32)
    hipLaunchKernelGGL(k_vox_mark<float>, dim3(ceil_div(num_points, 256)), dim3(256), 0, stream,
                       (const float*)points_fp16_dev, num_points, g, v->pkey.as<uint32_t>(), cells, flags);
  else if (num_points)
    hipLaunchKernelGGL(k_vox_mark<_Float16>, dim3(ceil_div(num_points, 256)), dim3(256), 0, stream,
                       (const _Float16*)points_fp16_dev, num_points, g, v->pkey.as<uint32_t>(), cells, flags);
  hipLaunchKernelGGL(k_vox_blocksum, dim3(nblocks), dim3(256), 0, stream, cells, flags, v->blocksum.as<uint32_t>());
  hipLaunchKernelGGL(k_vox_rank, dim3(nblocks), dim3(256), 0, stream, cells, v->blocksum.as<uint32_t>(),
                     Int3{{g.og[0], g.og[1], g.og[2]}}, (uint32_t)p.max_voxels, (int4*)v->idx.p, cnt, v->counts.as<uint32_t>());
  if (num_points) {
    const dim3 pgrid(ceil_div(num_points, 256));
    hipLaunchKernelGGL(k_vox_assign, pgrid, dim3(256), 0, stream, v->pkey.as<uint32_t>(), num_points, cells, p.max_voxels,
                       p.max_points_per_voxel, tag_arrival, v->counts.as<uint32_t>(), v->mins.as<uint32_t>(), overflow, always);
    for (int phase = 0; phase < 2; ++phase)
      hipLaunchKernelGGL(k_vox_overflow, dim3(std::min(pgrid.x, 512u)), dim3(256), 0, stream, v->pkey.as<uint32_t>(),
                         num_points, cells, p.max_voxels, p.max_points_per_voxel, tag_cascade, v->counts.as<uint32_t>(),
                         v->mins.as<uint32_t>(), overflow, always, phase);
    const uint32_t bound = (uint32_t)std::min<uint64_t>((uint64_t)p.max_voxels, num_points);
    const uint32_t threads = std::max(bound, num_points);
    if (p32)
      hipLaunchKernelGGL(k_vox_mean<float>, dim3(ceil_div(threads, 256)), dim3(256), 0, stream,
                         (const float*)points_fp16_dev, cnt, p.max_voxels, p.max_points_per_voxel, p.num_feature,
                         v->counts.as<uint32_t>(), v->mins.as<uint32_t>(), (_Float16*)v->feats.p, v->pkey.as<uint32_t>(),
                         num_points, cells, flags, overflow);
    else
      hipLaunchKernelGGL(k_vox_mean<_Float16>, dim3(ceil_div(threads, 256)), dim3(256), 0, stream,
                         (const _Float16*)points_fp16_dev, cnt, p.max_voxels, p.max_points_per_voxel, p.num_feature,
                         v->counts.as<uint32_t>(), v->mins.as<uint32_t>(), (_Float16*)v->feats.p, v->pkey.as<uint32_t>(),
                         num_points, cells, flags, overflow);
  }
  SCN_HIP(hipGetLastError());
  if (debug_sync_enabled()) return debug_sync_check(stream, "scn_voxelizer_forward");
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
  int rc = rb->rb.build_subm(indices_dev, n, n_dev, grid, ksize, dilation, nullptr, (hipStream_t)stream);
  if (rc == SCN_OK && debug_sync_enabled()) rc = debug_sync_check((hipStream_t)stream, "scn_rulebook_build_subm");
  return rc;
}
int scn_rulebook_build_sparse(scn_rulebook* rb, const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev,
                              const int grid[3], const int ksize[3], const int stride[3], const int padding[3],
                              const int dilation[3], void* stream) {
  SCN_REQUIRE(rb && grid && ksize && stride && padding && dilation && (indices_dev || n == 0), SCN_ERR_INVALID,
              "null pointer");
  int rc = rb->rb.build_sparse(indices_dev, n, n_dev, grid, ksize, stride, padding, dilation, nullptr,
                               (hipStream_t)stream);
  if (rc == SCN_OK && debug_sync_enabled()) rc = debug_sync_check((hipStream_t)stream, "scn_rulebook_build_sparse");
  return rc;
}
int scn_rulebook_build_inverse(scn_rulebook* rb, const scn_rulebook* forward, const uint32_t* n_in_dev, void* stream) {
  SCN_REQUIRE(rb && forward, SCN_ERR_INVALID, "null pointer");
  int rc = rb->rb.build_inverse(forward->rb, n_in_dev, (hipStream_t)stream);
  if (rc == SCN_OK && debug_sync_enabled()) rc = debug_sync_check((hipStream_t)stream, "scn_rulebook_build_inverse");
  return rc;
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

}  // extern "C"
