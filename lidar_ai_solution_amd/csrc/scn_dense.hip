// Elementwise glue (quantise / dequantise / pad, add + relu) and sparse -> dense of the SCN path (gfx950).
#include "scn_device.hpp"
#include <mutex>

#include <algorithm>
#include <cstdlib>
#include <cstring>

namespace scn {

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

// max |value| over the first n rows x c channels of a row-major tensor (calibration: the dynamic range of a
// tensor is the largest magnitude seen).  Non-negative floats order like their bit patterns, so the
// reduction is an integer atomicMax; *result must be zero on entry.
__global__ __launch_bounds__(256) void k_absmax(const void* x, int dtype, float scale, uint32_t c, uint32_t ld,
                                               uint32_t n_bound, const uint32_t* n_dev, uint32_t* result) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const size_t total = (size_t)n * c;
  float m = 0.f;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (size_t)gridDim.x * 256) {
    const size_t row = i / c, col = i % c;
    const float v = fabsf(load_value(x, dtype, row * ld + col, scale, 0.f, 0.f));
    m = v > m ? v : m;   // NaN never wins
  }
#pragma unroll
  for (int d = 32; d >= 1; d >>= 1) m = fmaxf(m, __shfl_xor(m, d, 64));
  if ((threadIdx.x & 63) == 0 && m > 0.f) atomicMax(result, __float_as_uint(m));
}

int absmax_rows(const void* x, int dtype, float range, uint32_t c, uint32_t ld, uint32_t n, const uint32_t* n_dev,
                float* result_dev, hipStream_t stream) {
  SCN_REQUIRE(result_dev, SCN_ERR_INVALID, "absmax: null result");
  int rc = fill_u32(result_dev, 0u, 1, stream);   // one word; the pointer must be 16-byte aligned
  if (rc) return rc;
  if (n == 0 || c == 0) return SCN_OK;
  SCN_REQUIRE(x, SCN_ERR_INVALID, "absmax: null tensor");
  const size_t total = (size_t)n * c;
  const unsigned blocks = (unsigned)std::min<size_t>((total + 255) / 256, 2048);
  hipLaunchKernelGGL(k_absmax, dim3(blocks), dim3(256), 0, stream, x, dtype, range > 0.f ? range / 127.f : 1.f, c, ld, n,
                     n_dev, reinterpret_cast<uint32_t*>(result_dev));
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

// The remaining dense forms of push_dense (libraries/3DSparseConvolution/libspconv/include/spconv/engine.hpp:26,
// 114-123): int8 output and the vectorised layouts.  The sparse tensor [N, C] on the grid (D0, D1, D2), one of whose
// axes is z (the first for "zyx" tensors, the last for "xyz" ones; the other two are H and W in their order), is the
// 4-D tensor [1, C * Z, H, W] with channel c * Z + z (what the exporters' dense().view() / permute().reshape() tails
// build).  NCHW32 stores it as [1, ceil(C Z / 32), H, W, 32] (groups of 32 channels innermost, zero padded),
// NHWzC as [1, H, W, Z, C].  The closed engine's own definition of the two layouts is not in the reference's
// sources; these follow the layout names.  One thread per (row, channel); the tensor is cleared first.
struct DenseForm {
  int layout;      // 1 strides (NCHW and its transposes), 2 NCHW32, 3 NHWzC
  int zaxis;       // 0 or 2: which spatial axis is z
  int C, Z, H, W;
  DenseStrides st; // layout 1
};

__global__ __launch_bounds__(256) void k_scatter_form(const void* feat, int dtype, float scale, uint32_t ld,
                                                      const int4* __restrict__ coords, uint32_t n_bound,
                                                      const uint32_t* n_dev, DenseForm f, void* out, int out_dtype,
                                                      float out_r) {
  const uint32_t n = eff_n(n_dev, n_bound);
  const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
  const uint32_t row = (uint32_t)(t / (uint32_t)f.C), c = (uint32_t)(t % (uint32_t)f.C);
  if (row >= n) return;
  const int4 p = coords[row];
  if (p.x != 0 || p.y < 0 || p.y >= f.st.d0 || p.z < 0 || p.z >= f.st.d1 || p.w < 0 || p.w >= f.st.d2) return;
  const float v = load_value(feat, dtype, (size_t)row * ld + c, scale, 0.f, 0.f);
  size_t off;
  if (f.layout == 1) {
    off = (size_t)(c * f.st.sc + p.y * f.st.s0 + p.z * f.st.s1 + p.w * f.st.s2);
  } else {
    const int z = f.zaxis == 0 ? p.y : p.w;
    const int h = f.zaxis == 0 ? p.z : p.y;
    const int w = f.zaxis == 0 ? p.w : p.z;
    if (f.layout == 2) {
      const uint32_t cz = c * (uint32_t)f.Z + (uint32_t)z;
      off = ((((size_t)(cz >> 5) * f.H + h) * f.W + w) << 5) + (cz & 31u);
    } else {
      off = (((size_t)h * f.W + w) * f.Z + z) * f.C + c;
    }
  }
  store_value(out, out_dtype, off, v, out_r);
}

size_t scatter_dense_form_elements(const int dense_shape[5], int zaxis, int layout) {
  const size_t C = dense_shape[1];
  const size_t Z = dense_shape[2 + zaxis], H = dense_shape[zaxis == 0 ? 3 : 2], W = dense_shape[zaxis == 0 ? 4 : 3];
  if (layout == 2) return (C * Z + 31) / 32 * 32 * H * W;
  return C * Z * H * W;
}

int scatter_dense_form(const void* feat, int dtype, float range, uint32_t c, uint32_t ld, const int32_t* idx, uint32_t n,
                       const uint32_t* n_dev, const int dense_shape[5], const int perm[5], int zaxis, int layout,
                       int out_dtype, float out_range, void* out, hipStream_t stream) {
  SCN_REQUIRE(out && dense_shape, SCN_ERR_INVALID, "scatter_dense: null pointer");
  SCN_REQUIRE(dense_shape[0] == 1 && (uint32_t)dense_shape[1] == c && c > 0, SCN_ERR_INVALID,
              "scatter_dense: output_shape must be [1, C=%u, D0, D1, D2]", c);
  SCN_REQUIRE(layout >= 1 && layout <= 3 && (zaxis == 0 || zaxis == 2), SCN_ERR_INVALID, "scatter_dense: bad layout");
  SCN_REQUIRE(out_dtype == SCN_DTYPE_FP16 || (out_dtype == SCN_DTYPE_INT8 && out_range > 0.f), SCN_ERR_INVALID,
              "scatter_dense: the output is fp16, or int8 with a dynamic range");
  DenseForm f{};
  f.layout = layout;
  f.zaxis = zaxis;
  f.C = (int)c;
  f.Z = dense_shape[2 + zaxis];
  f.H = dense_shape[zaxis == 0 ? 3 : 2];
  f.W = dense_shape[zaxis == 0 ? 4 : 3];
  int64_t dstride[5] = {0, 0, 0, 0, 0};
  size_t numel = 0;
  if (layout == 1) {
    SCN_REQUIRE(dense_layout(dense_shape, perm, dstride, &numel), SCN_ERR_INVALID, "scatter_dense: bad permutation");
  } else {
    SCN_REQUIRE(perm == nullptr, SCN_ERR_INVALID, "scatter_dense: a vectorised layout takes no Transpose");
    numel = scatter_dense_form_elements(dense_shape, zaxis, layout);
  }
  f.st = DenseStrides{dstride[1], dstride[2], dstride[3], dstride[4], dense_shape[2], dense_shape[3], dense_shape[4]};
  const size_t bytes = numel * (out_dtype == SCN_DTYPE_INT8 ? 1 : 2);
  SCN_REQUIRE(bytes % 4 == 0, SCN_ERR_UNSUPPORTED, "scatter_dense: tensor size %zu is not a multiple of 4 bytes", bytes);
  int rc = fill_u32(out, 0u, bytes / 4, stream);
  if (rc || n == 0) return rc;
  SCN_REQUIRE(feat && idx, SCN_ERR_INVALID, "scatter_dense: null input");
  const size_t total = (size_t)n * c;
  hipLaunchKernelGGL(k_scatter_form, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, feat, dtype,
                     range > 0.f ? range / 127.f : 1.f, ld, (const int4*)idx, n, n_dev, f, out, out_dtype,
                     out_range > 0.f ? 127.f / out_range : 1.f);
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

}  // namespace scn

using namespace scn;

// ---------------------------------------------------------------- allocation-free sparse -> dense
// scn_scatter_dense_with_map with the row map in a static device array instead of a caller's workspace: for
// callers that cannot allocate (HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The array
// exists once per GPU for the life of the process; its device address is looked up once per device, with that
// device current, and only that address -- never the array's name, which in host code is a stand-in and not a
// device address -- is passed to kernels.  Every call on a GPU uses that GPU's one array, so calls that overlap
// on one GPU (two streams, two threads) race; the map is cleared by a fill kernel at the start of every call.
#define SCN_NOALLOC_MAX_CELLS (1u << 18)
static __device__ __align__(256) int32_t scratch[SCN_NOALLOC_MAX_CELLS];

namespace {
constexpr int kMaxDevices = 64;
int32_t* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

int scratch_of_current_device(int32_t** out) {
  int dev = -1;
  SCN_HIP(hipGetDevice(&dev));
  SCN_REQUIRE(dev >= 0 && dev < kMaxDevices, SCN_ERR_UNSUPPORTED, "device ordinal %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    SCN_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SCN_REQUIRE(p != nullptr, SCN_ERR_HIP, "hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = static_cast<int32_t*>(p);
  }
  *out = g_scratch_ptr[dev];
  return SCN_OK;
}
}  // namespace


extern "C" {
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

int scn_scatter_dense_layout(const void* feat_dev, int dtype, float dynamic_range, uint32_t c, uint32_t ld,
                             const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                             const int perm[5], int z_axis, int output_layout, int out_dtype, float out_dynamic_range,
                             void* out_dev, void* stream) {
  return scatter_dense_form(feat_dev, dtype, dynamic_range, c, ld, indices_dev, n, n_dev, dense_shape, perm, z_axis,
                            output_layout, out_dtype, out_dynamic_range, out_dev, (hipStream_t)stream);
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


size_t scn_scatter_dense_noalloc_max_cells(void) { return SCN_NOALLOC_MAX_CELLS; }

int scn_scatter_dense_noalloc(const void* feat_dev, int dtype, float dynamic_range, uint32_t c, uint32_t ld,
                              const int32_t* indices_dev, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                              const int perm[5], void* out_fp16_dev, void* stream) {
  SCN_REQUIRE(dense_shape, SCN_ERR_INVALID, "scatter_dense: null pointer");
  const size_t cells = scatter_dense_map_cells(dense_shape, perm);
  SCN_REQUIRE(cells != 0, SCN_ERR_UNSUPPORTED,
              "scn_scatter_dense_noalloc: the layout takes no row map (channel axis must be outermost after the "
              "Transpose and D0*D1*D2 a multiple of 8)");
  SCN_REQUIRE(cells <= SCN_NOALLOC_MAX_CELLS, SCN_ERR_CAPACITY,
              "scn_scatter_dense_noalloc: D0*D1*D2 = %zu cells exceed the static row map of %u cells", cells,
              (unsigned)SCN_NOALLOC_MAX_CELLS);
  int32_t* map = nullptr;
  int rc = scratch_of_current_device(&map);
  if (rc) return rc;
  return scatter_dense(feat_dev, dtype, dynamic_range, c, ld, indices_dev, n, n_dev, dense_shape, perm, out_fp16_dev,
                       (hipStream_t)stream, false, map, false);
}

}  // extern "C"
