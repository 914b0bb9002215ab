// Tile plan of a rulebook (gfx950): per 32-row tile the set of kernel offsets at which any of its rows has a
// neighbour, and optionally the rows re-ordered so that rows with equal or similar offset sets share a tile.
// This is what the reference's loader calls `sortmask` ("skip more insignificance computations",
// libraries/3DSparseConvolution/src/onnx-parser.hpp:35-37, src/infer.cpp:477): in a lidar frame's first stages a
// row has 2 .. 10 of 27 neighbours, so a tile of 32 rows in coordinate order touches 14 .. 21 offsets.
// The re-ordering is local: rows are sorted by offset set inside windows of 1024 consecutive rows, in LDS, one
// workgroup per window.  Rows in coordinate order gather neighbouring rows, which share cache lines and L2; a sort of
// the whole tensor (measured with a device-wide radix sort: 70 .. 190 us per rulebook, and the 32-channel layers went
// from 27 to 41 .. 55 us although their tiles touched 13 instead of 21 offsets) gives that locality away, a window
// keeps it to within 1024 rows.
#include "scn_device.hpp"

namespace scn {

// OR over the 32 lanes of a half wave (the lanes of one tile)
__device__ __forceinline__ uint32_t half_wave_or(uint32_t v) {
#pragma unroll
  for (int d = 16; d >= 1; d >>= 1) v |= (uint32_t)__shfl_xor((int)v, d, 64);
  return v;
}

// One thread per position j < positions (a multiple of 32): the offset set of row j from the table.  Rows
// beyond the count get an empty set and, as a sort key, the flag bit above the kernel volume, which puts them
// behind every real row.  tmask (nullable: only for plans in row order) receives the tiles' ORs.
__global__ __launch_bounds__(256) void k_row_masks(const int32_t* __restrict__ nbr, uint32_t ld, int kvol,
                                                   const uint32_t* n_dev, uint32_t n_bound, uint32_t positions,
                                                   uint32_t* keys, uint32_t* tmask) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const uint32_t j = blockIdx.x * 256 + threadIdx.x;
  if (j >= positions) return;   // (whole half waves: positions is a multiple of 32)
  uint32_t m = 0;
  if (j < n)
    for (int k = 0; k < kvol; ++k) m |= (nbr[(size_t)k * ld + j] >= 0 ? 1u : 0u) << k;
  if (keys) keys[j] = j < n ? m : (1u << kvol);
  if (tmask) {
    const uint32_t t = half_wave_or(m);
    if ((threadIdx.x & 31) == 0) tmask[j >> 5] = t;
  }
}

// One workgroup per window of 1024 positions: bitonic sort of (offset set, position) in LDS, ascending; equal sets
// keep their row order.  keys_sorted / perm receive the window in sorted order (perm: the row a position stands for).
constexpr uint32_t kPlanWindow = 1024;
__global__ __launch_bounds__(1024) void k_window_sort(const uint32_t* __restrict__ keys, uint32_t positions,
                                                      uint32_t* keys_sorted, uint32_t* perm) {
  __shared__ uint64_t v[kPlanWindow];
  const uint32_t i = threadIdx.x, base = blockIdx.x * kPlanWindow;
  const uint32_t j = base + i;
  v[i] = j < positions ? ((uint64_t)keys[j] << 10) | i : ~0ull;
  __syncthreads();
  for (uint32_t k = 2; k <= kPlanWindow; k <<= 1)
    for (uint32_t d = k >> 1; d > 0; d >>= 1) {
      const uint32_t p = i ^ d;
      if (p > i) {
        const uint64_t a = v[i], b = v[p];
        const bool up = (i & k) == 0;
        if ((a > b) == up) {
          v[i] = b;
          v[p] = a;
        }
      }
      __syncthreads();
    }
  if (j < positions) {
    const uint64_t x = v[i];
    keys_sorted[j] = (uint32_t)(x >> 10);
    perm[j] = base + (uint32_t)(x & 1023u);
  }
}

// The table in plan order: out[k][j] = nbr[k][perm[j]] (-1 for positions that hold no row); grid.y = kernel
// offset.  The blocks of offset 0 also reduce the sorted offset sets to the tiles' masks.
__global__ __launch_bounds__(256) void k_plan_table(const int32_t* __restrict__ nbr, uint32_t ld, int kvol,
                                                    const uint32_t* __restrict__ keys_sorted,
                                                    const uint32_t* __restrict__ perm, uint32_t positions,
                                                    int32_t* out, uint32_t* tmask) {
  const uint32_t j = blockIdx.x * 256 + threadIdx.x;
  if (j >= positions) return;
  const uint32_t key = keys_sorted[j];
  const bool real = (key >> kvol) == 0;
  const int k = blockIdx.y;
  out[(size_t)k * ld + j] = real && ((key >> k) & 1u) ? nbr[(size_t)k * ld + perm[j]] : -1;
  if (k == 0) {
    const uint32_t t = half_wave_or(real ? key : 0u);
    if ((threadIdx.x & 31) == 0) tmask[j >> 5] = t;
  }
}

int Rulebook::reserve_plan(bool sorted) {
  SCN_REQUIRE(kvol_cap <= 31, SCN_ERR_UNSUPPORTED, "tile plan: kernel volume %d > 31", kvol_cap);
  const uint32_t cap = (std::max(max_out, 1u) + 31u) & ~31u;
  SCN_REQUIRE(cap <= ld, SCN_ERR_CAPACITY, "tile plan: %u positions exceed the table's leading dimension %u", cap, ld);
  TilePlan& p = plan;
  if (p.cap_rows < cap || (sorted && !p.reserved_sorted)) {
    if (!p.tmask.alloc((size_t)cap / 32 * 4)) return SCN_ERR_HIP;
    if (sorted) {
      if (!p.keys.alloc((size_t)cap * 4) || !p.keys_sorted.alloc((size_t)cap * 4) || !p.perm.alloc((size_t)cap * 4) ||
          !p.nbr.alloc((size_t)kvol_cap * ld * 4))
        return SCN_ERR_HIP;
      p.reserved_sorted = true;
    }
    p.cap_rows = cap;
  }
  return SCN_OK;
}

int Rulebook::build_plan(bool sorted, hipStream_t stream) {
  SCN_REQUIRE(built, SCN_ERR_INVALID, "tile plan: the rulebook has not been built");
  SCN_REQUIRE(geom.kvol <= 31, SCN_ERR_UNSUPPORTED, "tile plan: kernel volume %d > 31", geom.kvol);
  TilePlan& p = plan;
  const uint32_t positions = (n_bound_out + 31u) & ~31u;
  if (p.cap_rows < positions || (sorted && !p.reserved_sorted)) {
    int rc = reserve_plan(sorted);   // (the engine reserves up front; the stage-level entry point lands here)
    if (rc) return rc;
  }
  p.built = false;
  p.sorted = sorted;
  if (positions == 0) {
    p.built = true;
    return SCN_OK;
  }
  SCN_REQUIRE(positions <= ld && positions <= p.cap_rows, SCN_ERR_CAPACITY, "tile plan: %u positions exceed capacity", positions);
  const uint32_t blocks = ceil_div(positions, 256);
  if (!sorted) {
    hipLaunchKernelGGL(k_row_masks, dim3(blocks), dim3(256), 0, stream, nbr.as<int32_t>(), ld, geom.kvol, n_out_dev(),
                       n_bound_out, positions, (uint32_t*)nullptr, p.tmask.as<uint32_t>());
    SCN_HIP(hipGetLastError());
    p.built = true;
    return SCN_OK;
  }
  hipLaunchKernelGGL(k_row_masks, dim3(blocks), dim3(256), 0, stream, nbr.as<int32_t>(), ld, geom.kvol, n_out_dev(),
                     n_bound_out, positions, p.keys.as<uint32_t>(), (uint32_t*)nullptr);
  hipLaunchKernelGGL(k_window_sort, dim3(ceil_div(positions, kPlanWindow)), dim3(1024), 0, stream, p.keys.as<uint32_t>(),
                     positions, p.keys_sorted.as<uint32_t>(), p.perm.as<uint32_t>());
  hipLaunchKernelGGL(k_plan_table, dim3(blocks, geom.kvol), dim3(256), 0, stream, nbr.as<int32_t>(), ld, geom.kvol,
                     p.keys_sorted.as<uint32_t>(), p.perm.as<uint32_t>(), positions, p.nbr.as<int32_t>(),
                     p.tmask.as<uint32_t>());
  SCN_HIP(hipGetLastError());
  p.built = true;
  return SCN_OK;
}

}  // namespace scn

using namespace scn;

extern "C" {

int scn_rulebook_build_plan(scn_rulebook* rb, int sorted, void* stream) {
  SCN_REQUIRE(rb, SCN_ERR_INVALID, "scn_rulebook_build_plan: null rulebook");
  return rb->rb.build_plan(sorted != 0, (hipStream_t)stream);
}

int scn_rulebook_plan(const scn_rulebook* rb, const uint32_t** tile_masks_dev, const uint32_t** perm_dev,
                      const int32_t** nbr_plan_dev) {
  SCN_REQUIRE(rb && rb->rb.plan.built, SCN_ERR_INVALID, "scn_rulebook_plan: no plan has been built");
  const TilePlan& p = rb->rb.plan;
  if (tile_masks_dev) *tile_masks_dev = p.tmask.as<uint32_t>();
  if (perm_dev) *perm_dev = p.sorted ? p.perm.as<uint32_t>() : nullptr;
  if (nbr_plan_dev) *nbr_plan_dev = p.sorted ? p.nbr.as<int32_t>() : nullptr;
  return SCN_OK;
}

}  // extern "C"
