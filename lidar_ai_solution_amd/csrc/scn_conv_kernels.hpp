// Convolution kernels of the SCN path (gfx950) and their launch dispatch, as templates over the element
// type: included by one translation unit per element type so that the two sets of instantiations
// compile side by side.
#pragma once

#include <type_traits>

#include "scn_conv_args.hpp"
#include "scn_device.hpp"

#include <cstdlib>
#include <cstring>

namespace scn {

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
//   b4   bias of the 4 channels
//   sc4  int8: s_x * s_w[c] of the 4 channels (one fp32 rounding); unused for fp16
//   resp the 4 residual values of this row (a.res_dtype), in global memory or staged in LDS; unused
//        without a residual
//   MODE 0: every switch is read from the arguments.  The others fix the combinations the backbones use
//        at compile time, because 16 unrolled pieces of the general code are ~11,000 instructions, more
//        than the instruction cache holds, and the epilogue then runs at the speed of its fetches:
//        1 / 2: no accumulator dump, no residual, int8 / fp16 output
//        3 / 4: no dump, residual and un-fused intermediate both int8 / both fp16 (same type as the output)
template <int EL, int MODE = 0>
__device__ __forceinline__ void epilogue_values(const ConvArgs& a, uint32_t row, int co,
                                                const typename Mma<EL>::Acc& acc, const float4 b4v, const float4 sc4v,
                                                const void* resp, float y[4]) {
  const bool dump = MODE == 0 && a.acc != nullptr;
  const bool has_res = MODE == 0 ? a.res != nullptr : MODE >= 3;
  const bool res8 = MODE == 0 ? a.res_dtype == SCN_DTYPE_INT8 : MODE == 3;
  const bool mid8 = MODE == 0 ? a.mid_dtype == SCN_DTYPE_INT8 : MODE == 3;
  const float b4[4] = {b4v.x, b4v.y, b4v.z, b4v.w};
  if (EL == 0) {
    const float sc4[4] = {sc4v.x, sc4v.y, sc4v.z, sc4v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float m = (float)acc[j] * sc4[j];      // fp32 multiply
      y[j] = m + b4[j];                            // fp32 add (the library is built with -ffp-contract=off)
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) y[j] = (float)acc[j] + b4[j];
  }
  if (dump) {
    if (EL == 0)
      *reinterpret_cast<v4i*>((int32_t*)a.acc + (size_t)row * a.cout + co) = __builtin_bit_cast(v4i, acc);
    else
      *reinterpret_cast<v4f*>((float*)a.acc + (size_t)row * a.cout + co) = __builtin_bit_cast(v4f, acc);
  }
  if (a.relu) {
#pragma unroll
    for (int j = 0; j < 4; ++j) y[j] = y[j] > 0.f ? y[j] : 0.f;
  }
  if (has_res) {
    // value of the un-fused conv output as its consumer (the Add) would have read it
    float rv[4];
    if (res8) {
      const char4 r = *reinterpret_cast<const char4*>(resp);
      rv[0] = (float)r.x * a.res_scale;
      rv[1] = (float)r.y * a.res_scale;
      rv[2] = (float)r.z * a.res_scale;
      rv[3] = (float)r.w * a.res_scale;
    } else {
      const _Float16* r = reinterpret_cast<const _Float16*>(resp);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        rv[j] = (float)r[j];
        if (a.b_rq_r > 0.f) rv[j] = quant_f(rv[j], a.b_rq_r) * a.b_rq_s;
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v;
      if (mid8) {
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

// Address of the 4 residual values of (row, co) in global memory.
__device__ __forceinline__ const void* residual_ptr(const ConvArgs& a, uint32_t row, int co) {
  return a.res + ((size_t)row * a.res_ld + co) * (a.res_dtype == SCN_DTYPE_INT8 ? 1 : 2);
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

// One rounded, clamped value -> byte BYTE of the packed word (the conversion writes the byte itself,
// so no shifts and masks are needed to pack four of them).
#define SCN_CVT_BYTE(BYTE, PACKED, Q) \
  asm("v_cvt_i32_f32_sdwa %0, %1 dst_sel:BYTE_" #BYTE " dst_unused:UNUSED_PRESERVE src0_sel:DWORD" : "+v"(PACKED) : "v"(Q))

// The int8-output modes 1 and 3 of epilogue_values() without a branch: the same operations in the same
// order, except that a ReLU directly in front of a quantiser is the quantiser's lower clamp (0 instead
// of -127: rounding a negative product gives a value <= -0, which clamps to 0 either way).
//   lo1  lower clamp of the first quantiser after the convolution's own ReLU switch (a.relu ? 0 : -127):
//        the output quantiser (mode 1) or the un-fused intermediate's (mode 3)
//   lo2  mode 3: lower clamp of the output quantiser (a.relu2 ? 0 : -127)
//   r4   mode 3: the 4 residual bytes
template <int EL, int MODE>
__device__ __forceinline__ uint32_t epilogue_pack8(const ConvArgs& a, const typename Mma<EL>::Acc& acc, const float4 b4v,
                                                   const float4 sc4v, float lo1, float lo2, uint32_t r4) {
  static_assert(MODE == 1 || MODE == 3, "int8-output modes only");
  const float b4[4] = {b4v.x, b4v.y, b4v.z, b4v.w};
  const float sc4[4] = {sc4v.x, sc4v.y, sc4v.z, sc4v.w};
  float q[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    float y;
    if (EL == 0) {
      const float m = (float)acc[j] * sc4[j];
      y = m + b4[j];
    } else {
      y = (float)acc[j] + b4[j];
    }
    if (MODE == 1) {
      q[j] = __builtin_amdgcn_fmed3f(rintf(y * a.out_r), lo1, 127.f);
    } else {
      const float mid = __builtin_amdgcn_fmed3f(rintf(y * a.mid_r), lo1, 127.f) * a.mid_s;
      const float rv = (float)(int)(signed char)(r4 >> (8 * j)) * a.res_scale;
      const float v = mid + rv;
      q[j] = __builtin_amdgcn_fmed3f(rintf(v * a.out_r), lo2, 127.f);
    }
  }
  uint32_t packed = 0;
  SCN_CVT_BYTE(0, packed, q[0]);
  SCN_CVT_BYTE(1, packed, q[1]);
  SCN_CVT_BYTE(2, packed, q[2]);
  SCN_CVT_BYTE(3, packed, q[3]);
  return packed;
}
#undef SCN_CVT_BYTE

// The fp16-output modes 2 and 4 of epilogue_values() without a branch (mode 4 is only chosen when neither
// operand of the fused Add is re-quantised).  lo1 / lo2: 0 where the ReLU switch is on, -inf where it is off.
template <int EL, int MODE>
__device__ __forceinline__ v4h epilogue_pack16(const typename Mma<EL>::Acc& acc, const float4 b4v, const float4 sc4v,
                                               float lo1, float lo2, v4h r4) {
  static_assert(MODE == 2 || MODE == 4, "fp16-output modes only");
  const float b4[4] = {b4v.x, b4v.y, b4v.z, b4v.w};
  const float sc4[4] = {sc4v.x, sc4v.y, sc4v.z, sc4v.w};
  float y[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (EL == 0) {
      const float m = (float)acc[j] * sc4[j];
      y[j] = m + b4[j];
    } else {
      y[j] = (float)acc[j] + b4[j];
    }
    y[j] = y[j] > lo1 ? y[j] : lo1;
    if (MODE == 4) {
      const float v = half_round(y[j]) + (float)r4[j];
      y[j] = v > lo2 ? v : lo2;
    }
  }
  return pack_fp16(y);
}

// Stores 4 consecutive channels of one row after the fused epilogue.
template <int EL>
__device__ __forceinline__ void epilogue_store(const ConvArgs& a, uint32_t row, int co, const typename Mma<EL>::Acc& acc,
                                               const float4 b4, const float4 sc4) {
  float y[4];
  epilogue_values<EL>(a, row, co, acc, b4, sc4, a.res ? residual_ptr(a, row, co) : nullptr, y);
  if (a.out_dtype == SCN_DTYPE_INT8)
    *reinterpret_cast<char4*>(a.out + (size_t)row * a.out_ld + co) = pack_int8(a, y);
  else
    *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(a.out) + (size_t)row * a.out_ld + co) = pack_fp16(y);
}

// Bias and (int8) full requantisation scale of 4 channels from global memory.
template <int EL>
__device__ __forceinline__ void epilogue_consts(const ConvArgs& a, int co, float4* b4, float4* sc4) {
  *b4 = *reinterpret_cast<const float4*>(a.bias + co);
  *sc4 = make_float4(0.f, 0.f, 0.f, 0.f);
  if (EL == 0) {
    const float4 ws = *reinterpret_cast<const float4*>(a.wscale + co);
    *sc4 = make_float4(a.x_scale * ws.x, a.x_scale * ws.y, a.x_scale * ws.z, a.x_scale * ws.w);  // s_x * s_w[c]
  }
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
    for (int t = 0; t < MT; ++t) {
      float4 b4, sc4;
      epilogue_consts<EL>(a, t * 16 + lg * 4, &b4, &sc4);
      epilogue_store<EL>(a, rows[u], t * 16 + lg * 4, acc[t][u], b4, sc4);
    }
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
// obtained by permuting which chunk of its row a lane fetches: position p of a row holds chunk p ^ swz(row),
// swz(row) = (row / rows per 256 bytes) % chunks per row.
//   iteration     = 4 K-steps = 4 KB of gathered rows per wave (32 rows x 8 chunks, or G = 8 / SEG
//                   kernel offsets of SEG-chunk rows) and a weight slab of 4 * MT fragments
//   LDS           = 2 weight slabs (iteration i, i+1), one 4 KB stage of gathered rows per wave, and a
//                   ring of neighbour indices per wave, DEPTH = 4 or 2 iterations deep (they always miss the caches)
//   per iteration = one barrier for the slab; a wave consumes only rows and indices it fetched itself,
//                   so those need a wait on the wave's own memory counter only
// The memory counter retires loads in order, so "at most N outstanding" names exactly which older load
// has landed.  Issue order per iteration i: slab S(i+1), indices I(i+DEPTH), gathers G(i+1).
// Waves per SIMD the kernel is compiled for: two 8-wave workgroups per CU (128 registers), or one of
// 9 .. 12 waves.  The 64-channel kernels with 64- and 128-byte input rows take three 8-wave workgroups per
// CU instead (80 registers without spilling, with a two-stage index ring and one set of A fragments): a
// lidar frame's 64-channel stage is more tiles than two workgroups per CU hold in one round.  Workgroups of
// 2 or 4 waves (64 and 128 output channels, launches of few rows) are alone on their SIMDs: 256 registers.
constexpr bool conv_lds_three_groups(int chunks, int mt, int waves) {
  return mt == 2 && waves == 8 && (chunks == 4 || chunks == 8);
}
constexpr int conv_lds_min_waves(int chunks, int mt, int waves) {
  return conv_lds_three_groups(chunks, mt, waves) ? 6 : (mt >= 2 && waves <= 4) ? 2 : waves <= 8 ? 4 : 3;
}

template <int EL, int CHUNKS, int MT, int WAVES>
__global__ __launch_bounds__(64 * WAVES, conv_lds_min_waves(CHUNKS, MT, WAVES)) void k_conv_lds(const ConvArgs a) {
  using Acc = typename Mma32<EL>::Acc;
  using Acc4 = typename Mma32<EL>::Acc4;
  constexpr int THREADS = 64 * WAVES;
  constexpr int SEG = CHUNKS < 8 ? CHUNKS : 8;   // chunks gathered per row and iteration
  constexpr int IPO = CHUNKS / SEG;              // iterations per kernel offset (rows wider than 128 B)
  constexpr int G = 8 / SEG;                     // kernel offsets per iteration
  // Rows per rotation period of the gathered stage.  The LDS of gfx950 reads 256 bytes per clock (64 banks), so
  // the chunk a position holds rotates over runs of 256 bytes: a stand-alone probe of ds_read_b128 of the B operand
  // takes 1.36 times as long with the rotation over 128 bytes (the one for 32 banks) as a conflict-free read, and
  // is level over 256.  The kernels of 128-byte rows at three workgroups per CU keep the 128-byte period: the extra
  // shift of the longer one costs them a register they do not have (80 without scratch).
  constexpr int RP = (CHUNKS == 8 && conv_lds_three_groups(CHUNKS, MT, WAVES) ? 8 : 16) / SEG;
  constexpr int SLAB = 4 * MT * 64;              // 16-byte weight fragments per iteration
  constexpr int NL = SLAB / 64;                  // 1 KB wave-loads per slab
  constexpr int WPT = (NL + WAVES - 1) / WAVES;  // slab loads per wave and iteration (the same for every wave:
                                                 // the waits below count loads; surplus ones go to `spare`)
  constexpr int IDXE = G >= 2 ? G / 2 : 1;       // index entries per wave and iteration, in units of 64
  constexpr bool IDX4 = G >= 8;                  // 16-byte index loads (all 64 lanes busy; measured slower for G = 2, equal for 4)
  constexpr int IDXI = IDX4 ? 1 : IDXE;          // index loads per wave and iteration
  constexpr int R = 32 * WAVES;                  // output rows per workgroup
  __shared__ v4i lds[2][SLAB];                   // weight slabs of iterations i and i+1
  __shared__ v4i ring[WAVES][1][256];            // one stage of gathered rows per wave
  constexpr int DEPTH = ((MT == 1 && CHUNKS <= 2) || conv_lds_three_groups(CHUNKS, MT, WAVES)) ? 2 : 4;   // index ring stages (LDS is what limits the narrow layers' occupancy)
  __shared__ int32_t iring[DEPTH][WAVES][64 * IDXE];
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
#define SCN_SLAB(IT, BUF)                                                                       \
  {                                                                                             \
    const int it_ = (IT) < iters ? (IT) : iters - 1;                                            \
    _Pragma("unroll") for (int j = 0; j < WPT; ++j) {                                           \
      const int f_ = j * WAVES + wave; /* wave-uniform */                                       \
      if (NL % WAVES == 0 || f_ < NL)                                                           \
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + (size_t)it_ * SLAB + f_ * 64 + lane),  \
                                         (lptr_t)&lds[BUF][f_ * 64], 16, 0, 0);                 \
      else                                                                                      \
        __builtin_amdgcn_global_load_lds((gptr_t)(wsrc + (size_t)it_ * SLAB + lane),            \
                                         (lptr_t)&spare[0], 16, 0, 0);                          \
    }                                                                                           \
  }
// neighbour rows of iteration IT -> index ring stage IT % DEPTH: entry e is kernel offset e / 32 of the
// iteration, tile row e % 32; slots outside the volume or beyond row n read -1.  Lane l of load q fetches
// entry 64 q + l; with 8 offsets per iteration (16-byte rows) one load fetches all 256 entries instead,
// lane l the 16 bytes of rows 4 (l % 8) .. + 3 of offset l / 8, which relies on the rulebooks' guarantee
// that the table holds -1 for the rows between the count and the next multiple of 32.
#define SCN_INDEX(IT)                                                                           \
  {                                                                                             \
    if constexpr (IDX4) {                                                                       \
      const int k_ = (IT) * G + lane / 8;                                                       \
      const bool ok_ = (IT) < iters && k_ < a.kvol && row0 < n;                                 \
      const int32_t* p_ = ok_ ? a.nbr + (size_t)k_ * a.nbr_ld + row0 + 4 * (lane & 7) : minus1 + 4 * lane; \
      __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&iring[(IT) & (DEPTH - 1)][wave][0], 16, 0, 0); \
    } else {                                                                                    \
      _Pragma("unroll") for (int q = 0; q < IDXI; ++q) {                                        \
        const int e_ = q * 64 + lane;                                                           \
        const int k_ = IPO > 1 ? (IT) / IPO + e_ / 32 : (IT) * G + e_ / 32;                     \
        const uint32_t r_ = row0 + (e_ & 31);                                                   \
        const bool ok_ = (IT) < iters && k_ < a.kvol && r_ < n;                                 \
        const int32_t* p_ = ok_ ? a.nbr + (size_t)k_ * a.nbr_ld + r_ : minus1 + lane;           \
        __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&iring[(IT) & (DEPTH - 1)][wave][q * 64], 4, 0, 0); \
      }                                                                                         \
    }                                                                                           \
  }
// gathers of iteration IT (neighbour rows GI[4] of this lane's slots) into the wave's stage; element
// e = 64 q + lane of its [G][32 rows][SEG] array
#define SCN_GATHER(IT, GI, STG)                                                                 \
  {                                                                                             \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                             \
      const int e_ = q * 64 + lane;                                                             \
      const int row_ = (e_ / SEG) % 32;                                                         \
      const int cg_ = (IPO > 1 ? ((IT) % IPO) * 8 : 0) + ((e_ % SEG) ^ ((row_ / RP) % SEG));    \
      const char* p_ = GI[q] >= 0 ? xb + (size_t)(uint32_t)GI[q] * ldb + cg_ * 16 : zrow + cg_ * 16; \
      __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&ring[wave][STG][q * 64], 16, 0, 0); \
    }                                                                                           \
  }
// this lane's four index slots of ring stage STG -> GI[4], waited for.  Slot q of lane l is entry
// e / SEG of the stage (e = 64 q + l), i.e. a fixed stride of 64 / SEG entries between slots.
#define SCN_READ_INDEX(STG, GI)                                                                 \
  {                                                                                             \
    const uint32_t base_ = iring_addr + (uint32_t)(STG) * (WAVES * 64 * IDXE * 4);              \
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

  const uint32_t ring_addr = (uint32_t)(uintptr_t)(lptr_t)&ring[wave][0][0];
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

  // B fragments of the wave's stage STG (the four K-steps of an iteration)
#define SCN_READ_B(STG, BF)                                                                     \
  {                                                                                             \
    uint32_t bb = b_base + (uint32_t)(STG) * 4096u, sw = b_swz;                                 \
    asm volatile("" : "+v"(bb), "+v"(sw)); /* keeps the four addresses out of loop-carried registers */ \
    asm volatile("ds_read_b128 %0, %4\n\tds_read_b128 %1, %5\n\tds_read_b128 %2, %6\n\tds_read_b128 %3, %7" \
                 : "=&v"(BF[0]), "=&v"(BF[1]), "=&v"(BF[2]), "=&v"(BF[3])                       \
                 : "v"(SCN_B_ADDR(0, bb, sw)), "v"(SCN_B_ADDR(1, bb, sw)), "v"(SCN_B_ADDR(2, bb, sw)), \
                   "v"(SCN_B_ADDR(3, bb, sw))                                                   \
                 : "memory");                                                                   \
  }
  // the 4 * MT MFMAs of an iteration: A fragments from the slab at LDS address la, B fragments bf[]
  auto multiply = [&](const uint32_t la, const v4i (&bf)[4]) {
    if constexpr (WAVES >= 8 && ((MT >= 4 && conv_lds_min_waves(CHUNKS, MT, WAVES) >= 4) || conv_lds_three_groups(CHUNKS, MT, WAVES))) {
      // 64 accumulator registers leave room for one set of fragments under the 128-register budget of
      // four waves per SIMD (a spill would also put scratch loads into the memory counter and break the
      // counts below); the other three waves of the SIMD cover the LDS latency instead.  (Workgroups of 2 or 4
      // waves are alone on their SIMD and have the registers: they take the other path.)
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
  };

  // Residual tile of a fused Add (same element type as the output, see the epilogue): fetched into the wave's stage
  // by the last iteration, once that iteration's B fragments are in registers, so that its latency passes behind the
  // last MFMAs instead of in front of the epilogue.  Same placement as the epilogue's own staging: lane l of load q
  // holds position l % 8 of tile row l / 8 + 8 q, i.e. chunk (l % 8) ^ (row % 8) of that row (first 128-byte pass).
  // (Everything it needs is re-derived from the kernel arguments where it is used: a value kept across the loop
  // costs a register, and these kernels have none to spare.)
  // Not in the kernels compiled for 80 registers (three workgroups per CU) nor in the 8-wave kernels with 128 output
  // channels (128 registers): there the few extra address registers of the last iteration spill, and spills are loads
  // the counted waits do not know about.
  constexpr bool RES_EARLY = !conv_lds_three_groups(CHUNKS, MT, WAVES) && !(MT >= 4 && WAVES == 8);
#define SCN_RES_DMA() (RES_EARLY && a.res && a.res_vec16 && a.res_dtype == a.out_dtype && a.cout > 16 && a.out_vec16)
#define SCN_RESIDUAL()                                                                          \
  {                                                                                             \
    const int res_esz = a.out_dtype == SCN_DTYPE_INT8 ? 1 : 2;                                  \
    const int res_valid = ((a.cout + 15) & ~15) * res_esz;                                      \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                             \
      const int r_ = (lane >> 3) + 8 * q, c_ = (lane & 7) ^ (r_ & 7);                           \
      const uint32_t grow_ = row0 + (uint32_t)r_;                                               \
      const char* p_ = (grow_ < n && c_ * 16 < res_valid)                                       \
                           ? a.res + (size_t)grow_ * a.res_ld * res_esz + c_ * 16               \
                           : zrow + c_ * 16;                                                    \
      __builtin_amdgcn_global_load_lds((gptr_t)p_, (lptr_t)&ring[wave][0][q * 64], 16, 0, 0);   \
    }                                                                                           \
  }

  // A wave whose 32 rows have no neighbour at any kernel offset of an iteration (rows of one z slice and
  // the offsets that leave it, tiles next to empty space: a third to a half of all (tile, offset)
  // combinations of a synthetic frame, a tenth of a real one's) skips that iteration's operand reads and
  // MFMAs -- they would add zeros -- and, where the waits below can follow it, its gathers.
  {
    // prologue: indices of iterations 0 .. DEPTH-1, slab 0, then the gathers of iteration 0
    SCN_INDEX(0);
    SCN_INDEX(1);
    if constexpr (DEPTH == 4) {
      SCN_INDEX(2);
      SCN_INDEX(3);
    }
    SCN_SLAB(0, 0);
    SCN_WAIT_VM((DEPTH - 1) * IDXI + WPT);  // I(0), the oldest, has landed
    bool work;  // wave-uniform: the current iteration has at least one neighbour row
    {
      int32_t gi[4];
      SCN_READ_INDEX(0, gi);
      work = __builtin_amdgcn_ballot_w64((gi[0] & gi[1] & gi[2] & gi[3]) >= 0) != 0;
      if (work) {
        SCN_GATHER(0, gi, 0);
        SCN_WAIT_VM(4);  // ... and this wave's part of S(0) (younger: G(0))
      } else {
        SCN_WAIT_VM(0);
      }
    }
    asm volatile("s_barrier" ::: "memory");

    for (int it = 0; it < iters; ++it) {
      SCN_SLAB(it + 1, (it + 1) & 1);
      SCN_INDEX(it + DEPTH);
      SCN_WAIT_VM(WPT + IDXI);  // G(it), I(it+1) and everything older have landed
      v4i bf[4];
      int32_t gi[4];
      if (work) SCN_READ_B(0, bf);
      // waits for the index reads and, LDS returning in order, for bf[]: the stage may be overwritten
      SCN_READ_INDEX((it + 1) & (DEPTH - 1), gi);
      // (iterations past the end read -1 everywhere)
      const bool work_next = __builtin_amdgcn_ballot_w64((gi[0] & gi[1] & gi[2] & gi[3]) >= 0) != 0;
      const bool res_now = it + 1 == iters && SCN_RES_DMA();   // (the last iteration has no next gathers: work_next is false)
      if (work_next) {
        SCN_GATHER(it + 1, gi, 0);
      } else if (res_now) {
        SCN_RESIDUAL();
      }
      if (work) multiply(lds_a_addr + (uint32_t)(it & 1) * (SLAB * 16), bf);
      // this wave's part of S(it+1) has landed (younger: G(it+1) or the residual tile, when issued)
      if (work_next || res_now) {
        SCN_WAIT_VM(4);
      } else {
        SCN_WAIT_VM(0);
      }
      work = work_next;
      // every wave has read slab it (its fragments are in registers) and written its part of slab it+1
      asm volatile("s_barrier" ::: "memory");
    }
  }
#undef SCN_READ_B
#undef SCN_READ_INDEX
#undef SCN_B_ADDR
#undef SCN_READ_A
#undef SCN_WAIT_A
#undef SCN_WAIT_VM
#undef SCN_SLAB
#undef SCN_INDEX
#undef SCN_GATHER
#undef SCN_RESIDUAL
  // Epilogue.  Nothing in it may wait for global memory once per 4-channel piece (16 pieces per lane
  // for 128 channels, each a cache round trip): the per-channel constants are staged in LDS once per
  // workgroup, in the weight slab's space, and a residual tile is staged per wave like the output.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stage still receives what the last iteration issued
  const int cout_pad = (a.cout + 15) & ~15;
  const bool res_dma = SCN_RES_DMA();
#undef SCN_RES_DMA
  float* ep = reinterpret_cast<float*>(&lds[0][0]);  // [0, 128): bias, [128, 256): s_x * s_w[c]
  float4 cb[MT == 1 ? 4 : 1], cs[MT == 1 ? 4 : 1];
  if constexpr (MT == 1) {
    // 32 output channels are 4 pieces per lane: their constants fit registers and arrive in one round
    // trip, without the two barriers below (these layers are short; a barrier is a visible part of them)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int co = g * 8 + lh * 4;
      const int cc = co < cout_pad ? co : 0;
      cb[g] = *reinterpret_cast<const float4*>(a.bias + cc);
      cs[g] = make_float4(0.f, 0.f, 0.f, 0.f);
      if (EL == 0) {
        const float4 ws = *reinterpret_cast<const float4*>(a.wscale + cc);
        cs[g] = make_float4(a.x_scale * ws.x, a.x_scale * ws.y, a.x_scale * ws.z, a.x_scale * ws.w);
      }
    }
  } else {
    asm volatile("s_barrier" ::: "memory");         // the slab buffers received every wave's re-loads of the last slab
    if (tid < MT * 32) {
      const bool okc = tid < cout_pad;
      ep[tid] = okc ? a.bias[tid] : 0.f;
      if (EL == 0) ep[128 + tid] = okc ? a.x_scale * a.wscale[tid] : 0.f;
    }
    __syncthreads();
  }
  // constants of piece g of tile t (channels co .. co + 3)
  auto consts = [&](int g, int co, float4* b4, float4* sc4) {
    if constexpr (MT == 1) {
      *b4 = cb[g];
      *sc4 = cs[g];
    } else {
      *b4 = *reinterpret_cast<const float4*>(ep + co);
      *sc4 = *reinterpret_cast<const float4*>(ep + 128 + co);
    }
  };
  const uint32_t row = row0 + ln;
  if (!a.out_vec16) {
    if (row >= n) return;
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int co = t * 32 + g * 8 + lh * 4;
        if (co >= cout_pad) continue;
        const Acc4 piece = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
        float4 b4, sc4;
        consts(g, co, &b4, &sc4);
        epilogue_store<EL>(a, row, co, piece, b4, sc4);
      }
    return;
  }
  // Each lane holds 4-channel pieces of one row; writing them directly would touch every 128-byte line
  // of the tile 16 times.  The pieces go through the wave's LDS stage instead (same XOR placement as the
  // gathers) and leave as 16 bytes per lane, 8 lanes per row.  A residual of the output's element size
  // comes in the same way first: each piece finds its 4 residual values in the slot it then overwrites.
  char* stage = reinterpret_cast<char*>(&ring[wave][0][0]);
  const bool out8 = a.out_dtype == SCN_DTYPE_INT8;
  // (16-channel rows are one 16-byte chunk: staging them costs more than the two 4-byte reads it replaces)
  const bool res_staged = a.res && a.res_vec16 && a.res_dtype == a.out_dtype && cout_pad >= 32;
  constexpr int PASSES = MT >= 4 ? 2 : 1;          // fp16 rows of 128 channels take two 128-byte passes
  constexpr int TPP = MT >= 4 ? 2 : MT;            // 32-channel tiles per fp16 pass
  auto run = [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
    const bool o8 = MODE == 0 ? out8 : (MODE == 1 || MODE == 3);
    const bool staged = MODE == 0 ? res_staged : MODE >= 3;
    const float lo1 = a.relu ? 0.f : -127.f, lo2 = a.relu2 ? 0.f : -127.f;          // int8 clamps
    const float lo1h = a.relu ? 0.f : -__builtin_inff(), lo2h = a.relu2 ? 0.f : -__builtin_inff();
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
      if (o8 && p > 0) break;
      const int t_lo = o8 ? 0 : p * TPP, t_hi = o8 ? MT : p * TPP + TPP;
      const int c0 = t_lo * 32;                      // first channel of the pass
      const int osz = o8 ? 1 : 2;
      const int valid = (cout_pad - c0) * osz;       // bytes of the pass row that exist
      if (staged && !(p == 0 && res_dma)) {   // (the first pass's residual tile is in the stage already)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int r = (lane >> 3) + 8 * j, c = lane & 7;
          const uint32_t grow = row0 + r;
          v4i v = {0, 0, 0, 0};
          if (grow < n && c * 16 < valid)
            v = *reinterpret_cast<const v4i*>(a.res + ((size_t)grow * a.res_ld + c0) * osz + c * 16);
          *reinterpret_cast<v4i*>(stage + r * 128 + ((c ^ (r & 7)) << 4)) = v;
        }
      }
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        if (t < t_lo || t >= t_hi) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int co = t * 32 + g * 8 + lh * 4;
          // (the specialised modes touch nothing but LDS here: lanes without a row or channel run along)
          if (MODE == 0 && (co >= cout_pad || row >= n)) continue;
          if (MT == 1 && t * 32 + g * 8 >= cout_pad) continue;  // narrow layers: skip the padding pieces (uniform)
          const Acc4 piece = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
          const int off = (co - c0) * osz;           // byte offset inside the 128-byte pass row
          char* dst = stage + ln * 128 + (((off >> 4) ^ (ln & 7)) << 4) + (off & 15);
          float4 b4, sc4;
          consts(g, co, &b4, &sc4);
          if constexpr (MODE == 1 || MODE == 3) {
            const uint32_t r4 = MODE == 3 ? *reinterpret_cast<const uint32_t*>(dst) : 0u;
            *reinterpret_cast<uint32_t*>(dst) = epilogue_pack8<EL, MODE>(a, piece, b4, sc4, lo1, lo2, r4);
            continue;
          }
          if constexpr (MODE == 2 || MODE == 4) {
            const v4h r4 = MODE == 4 ? *reinterpret_cast<const v4h*>(dst) : v4h{0, 0, 0, 0};
            *reinterpret_cast<v4h*>(dst) = epilogue_pack16<EL, MODE>(piece, b4, sc4, lo1h, lo2h, r4);
            continue;
          }
          float y[4];
          epilogue_values<EL, MODE>(a, row, co, piece, b4, sc4,
                              staged ? (const void*)dst : (a.res ? residual_ptr(a, row, co) : nullptr), y);
          if (o8)
            *reinterpret_cast<char4*>(dst) = pack_int8(a, y);
          else
            *reinterpret_cast<v4h*>(dst) = pack_fp16(y);
        }
      }
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
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
  };
  int mode = 0;
  if (!a.acc) {
    if (!a.res)
      mode = out8 ? 1 : 2;
    else if (res_staged && a.mid_dtype == a.out_dtype && (out8 || (a.a_rq_r <= 0.f && a.b_rq_r <= 0.f)))
      mode = out8 ? 3 : 4;
  }
  switch (mode) {
    case 1: run(std::integral_constant<int, 1>{}); break;
    case 2: run(std::integral_constant<int, 2>{}); break;
    case 3: run(std::integral_constant<int, 3>{}); break;
    case 4: run(std::integral_constant<int, 4>{}); break;
    default: run(std::integral_constant<int, 0>{}); break;
  }
}

// --------------------------------------------------------------------------------------------
// Tile-plan kernel for the narrow layers (input rows of 16 .. 64 bytes, at most 64 output channels).
// In a lidar frame's first stages a row has 2 .. 10 of its 27 neighbours, so what such a layer costs is not
// arithmetic but the slots it visits: this kernel visits, per 32-row tile, only the kernel offsets named in the
// tile's mask (see TilePlan), and with a sorted plan the rows of a tile share most of theirs.
//   * persistent workgroups of 8 waves: the whole weight tensor (14 .. 56 KB) is copied to LDS once, after that
//     the waves never synchronise again; wave w of workgroup g takes tiles 8 g + w, + 8 * gridDim.x, ...
//   * a wave's step: up to UNR offsets of the mask -> their table entries (one coalesced 128-byte load per
//     offset) -> the neighbour rows straight into the B operand (16 bytes per lane; rows of 16 bytes pair two
//     offsets in one MFMA, K-half = offset) -> A fragments from LDS -> MFMA.  No LDS staging of rows: with one
//     16-byte chunk per lane there is nothing to coalesce.
//   * positions of a sorted plan are not rows: the epilogue stores (and reads the residual of) row perm[pos].
// Results are bit-identical to the other kernels: a row's products are added in offset order, integers exactly,
// fp16 products in fp32 with zero terms left out.
// waves per SIMD the tile-plan kernel is compiled for: eight (64 registers, four workgroups per CU) where the
// weights leave room for four workgroups' copies in LDS, four otherwise
constexpr int conv_tile_min_waves(int chunks, int mt) { return (mt == 1 && chunks <= 2) ? 8 : 4; }

template <int EL, int CHUNKS, int MT>
__global__ __launch_bounds__(512, conv_tile_min_waves(CHUNKS, MT)) void k_conv_tile(const ConvArgs a) {
  using Acc = typename Mma32<EL>::Acc;
  using Acc4 = typename Mma32<EL>::Acc4;
  constexpr int WAVES = 8;
  constexpr int KS = CHUNKS >= 2 ? CHUNKS / 2 : 1;   // MFMAs per offset and output tile (16-byte rows: half of one)
  constexpr int UNR = (CHUNKS >= 4 || conv_tile_min_waves(CHUNKS, MT) >= 8) ? 2 : 4;   // offsets (16-byte rows: offset pairs) in flight per step
  extern __shared__ v4i wl[];                        // [steps32][MT][64] A fragments, then bias[MT*32], scale[MT*32]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, ln = lane & 31, lh = lane >> 5;
  const int nfrag = a.steps32 * MT * 64;
  const uint32_t n = eff_n(a.n_out_dev, a.n_bound);
  const uint32_t tiles = (n + 31u) >> 5;
  // the first tile's mask is on its way while the weights are copied
  uint32_t tile = blockIdx.x * WAVES + wave;
  uint32_t m_next = tile < tiles ? a.tmask[tile] : 0u;
  {
    const v4i* __restrict__ src = reinterpret_cast<const v4i*>(a.wfrag32);
    for (int i = tid; i < nfrag; i += 64 * WAVES) wl[i] = src[i];
  }
  float* ep = reinterpret_cast<float*>(wl + nfrag);
  const int cout_pad = (a.cout + 15) & ~15;
  if (tid < MT * 32) {
    const bool okc = tid < cout_pad;
    ep[tid] = okc ? a.bias[tid] : 0.f;
    ep[MT * 32 + tid] = (EL == 0 && okc) ? a.x_scale * a.wscale[tid] : 0.f;
  }
  __syncthreads();

  const uint32_t ldb = a.x_ld_bytes;
  const char* __restrict__ xb = a.x;
  const char* __restrict__ zrow = a.zrow;
  const bool out8 = a.out_dtype == SCN_DTYPE_INT8;
  int mode = 0;
  if (!a.acc) {
    if (!a.res)
      mode = out8 ? 1 : 2;
    else if (a.res_dtype == a.out_dtype && a.mid_dtype == a.out_dtype && (out8 || (a.a_rq_r <= 0.f && a.b_rq_r <= 0.f)))
      mode = out8 ? 3 : 4;
  }
  const float lo1 = a.relu ? 0.f : -127.f, lo2 = a.relu2 ? 0.f : -127.f;
  const float lo1h = a.relu ? 0.f : -__builtin_inff(), lo2h = a.relu2 ? 0.f : -__builtin_inff();

  for (; tile < tiles; tile += gridDim.x * WAVES) {
    uint32_t m = __builtin_amdgcn_readfirstlane(m_next);
    {
      const uint32_t nt = tile + gridDim.x * WAVES;   // the next tile's mask arrives during this tile
      m_next = nt < tiles ? a.tmask[nt] : 0u;
    }
    const uint32_t pos = tile * 32u + ln;
    const uint32_t row = a.perm ? a.perm[pos] : pos;
    const int32_t* __restrict__ nb = a.nbr + pos;
    Acc acc[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[t][j] = 0;
    while (m) {
      int32_t idx[UNR];
      int kk[UNR];     // this lane's offset of step u (16-byte rows: K-half 1 takes the pair's second offset)
      int cnt = 0;
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        idx[u] = -1;
        kk[u] = 0;
        if (m) {   // wave-uniform
          const int ka = __builtin_ctz(m);
          m &= m - 1;
          int k = ka;
          bool have = true;
          if (CHUNKS == 1) {
            const int kb = m ? __builtin_ctz(m) : -1;
            if (m) m &= m - 1;
            have = lh == 0 || kb >= 0;
            k = (lh && kb >= 0) ? kb : ka;
          }
          kk[u] = k;
          if (have) idx[u] = nb[(size_t)k * a.nbr_ld];
          cnt = u + 1;
        }
      }
      v4i bf[UNR][KS];
#pragma unroll
      for (int u = 0; u < UNR; ++u)
#pragma unroll
        for (int ss = 0; ss < KS; ++ss) {
          const int chunk = CHUNKS == 1 ? 0 : 2 * ss + lh;
          const char* p = idx[u] >= 0 ? xb + (size_t)(uint32_t)idx[u] * ldb + chunk * 16 : zrow;
          bf[u][ss] = u < cnt ? *reinterpret_cast<const v4i*>(p) : v4i{0, 0, 0, 0};
        }
#pragma unroll
      for (int u = 0; u < UNR; ++u) {
        if (u >= cnt) break;   // wave-uniform
#pragma unroll
        for (int ss = 0; ss < KS; ++ss) {
          const int g = kk[u] * CHUNKS + (CHUNKS == 1 ? 0 : 2 * ss + lh);   // this lane's chunk of the weight sequence
#pragma unroll
          for (int t = 0; t < MT; ++t) {
            const v4i af = wl[((g >> 1) * MT + t) * 64 + (g & 1) * 32 + ln];
            acc[t] = Mma32<EL>::run(af, bf[u][ss], acc[t]);
          }
        }
      }
    }
    // epilogue: lane (ln, lh) holds channels 32 t + 8 g + 4 lh .. + 3 of row `row`
    if (row >= n) continue;
    auto store_tile = [&](auto mode_c) {
      constexpr int MODE = decltype(mode_c)::value;
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int co = t * 32 + g * 8 + lh * 4;
          if (co >= cout_pad) continue;
          const Acc4 piece = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
          const float4 b4 = *reinterpret_cast<const float4*>(ep + co);
          const float4 sc4 = *reinterpret_cast<const float4*>(ep + MT * 32 + co);
          if constexpr (MODE == 1 || MODE == 3) {
            uint32_t r4 = 0;
            if constexpr (MODE == 3) r4 = *reinterpret_cast<const uint32_t*>(a.res + (size_t)row * a.res_ld + co);
            *reinterpret_cast<uint32_t*>(a.out + (size_t)row * a.out_ld + co) =
                epilogue_pack8<EL, MODE>(a, piece, b4, sc4, lo1, lo2, r4);
          } else if constexpr (MODE == 2 || MODE == 4) {
            v4h r4 = {0, 0, 0, 0};
            if constexpr (MODE == 4)
              r4 = *reinterpret_cast<const v4h*>(reinterpret_cast<const _Float16*>(a.res) + (size_t)row * a.res_ld + co);
            *reinterpret_cast<v4h*>(reinterpret_cast<_Float16*>(a.out) + (size_t)row * a.out_ld + co) =
                epilogue_pack16<EL, MODE>(piece, b4, sc4, lo1h, lo2h, r4);
          } else {
            epilogue_store<EL>(a, row, co, piece, b4, sc4);
          }
        }
    };
    switch (mode) {
      case 1: store_tile(std::integral_constant<int, 1>{}); break;
      case 2: store_tile(std::integral_constant<int, 2>{}); break;
      case 3: store_tile(std::integral_constant<int, 3>{}); break;
      case 4: store_tile(std::integral_constant<int, 4>{}); break;
      default: store_tile(std::integral_constant<int, 0>{}); break;
    }
  }
}

template <int EL, int CHUNKS, int MT>
static void launch_conv_tile(const ConvArgs& a, uint32_t n_hint, hipStream_t stream) {
  // as many workgroups of 8 waves as fit the GPU at once (two or four per CU); fewer when the expected rows
  // are fewer than that many tiles
  (void)n_hint;
  const uint32_t tiles = ceil_div(a.launch_rows, 32u);
  const uint32_t resident = 256u * (conv_tile_min_waves(CHUNKS, MT) / 2);
  uint32_t blocks = ceil_div(tiles, 8u);
  blocks = blocks < 1 ? 1 : blocks > resident ? resident : blocks;
  const size_t lds = (size_t)a.steps32 * MT * 1024 + (size_t)MT * 32 * 8;
  hipLaunchKernelGGL((k_conv_tile<EL, CHUNKS, MT>), dim3(blocks), dim3(512), lds, stream, a);
}

template <int EL>
static bool dispatch_tile(int chunks, int mt, uint32_t n_hint, const ConvArgs& a, hipStream_t stream) {
  if (mt == 1) {
    switch (chunks) {
      case 1: launch_conv_tile<EL, 1, 1>(a, n_hint, stream); return true;
      case 2: launch_conv_tile<EL, 2, 1>(a, n_hint, stream); return true;
      case 4: launch_conv_tile<EL, 4, 1>(a, n_hint, stream); return true;
    }
  } else if (mt == 2) {
    switch (chunks) {
      case 1: launch_conv_tile<EL, 1, 2>(a, n_hint, stream); return true;
      case 2: launch_conv_tile<EL, 2, 2>(a, n_hint, stream); return true;
    }
  }
  return false;
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
  if (forced == 2 || forced == 4 || (forced >= 8 && forced <= 12)) return forced;
  constexpr uint32_t kCus = 256;
  const uint32_t waves = ceil_div(n_hint, kCus * 32u);  // 32-row tiles per CU
  // Few rows (a real frame's deep stages are 10,000 .. 30,000 rows): a workgroup's kernel offsets are a
  // dependent chain whose step grows with the loads its waves issue together, and 8-wave workgroups
  // would leave most CUs idle, so the tiles are spread over more, smaller workgroups.
  if (waves <= 2) return 2;
  if (waves <= 4) return 4;
  if (waves <= 8) return 8;
  if (waves <= 12) return (int)waves;
  return 8;
}

template <int EL, int CHUNKS>
static bool dispatch_mt32(int mt, uint32_t n_hint, const ConvArgs& a, hipStream_t stream) {
  switch (mt) {
    case 1: launch_conv_lds<EL, CHUNKS, 1, 4>(a, stream); return true;
    case 2:
      if (conv_lds_waves(n_hint) <= 4)
        launch_conv_lds<EL, CHUNKS, 2, 4>(a, stream);
      else
        launch_conv_lds<EL, CHUNKS, 2, 8>(a, stream);
      return true;
    case 4:
      switch (conv_lds_waves(n_hint)) {
        case 2: launch_conv_lds<EL, CHUNKS, 4, 2>(a, stream); return true;
        case 4: launch_conv_lds<EL, CHUNKS, 4, 4>(a, stream); return true;
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

}  // namespace scn
