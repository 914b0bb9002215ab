// Arguments of the convolution kernels and the per-element-type launchers.
#pragma once

#include "scn_kernels.hpp"

namespace scn {

struct ConvArgs {
  const char* x;
  uint32_t x_ld_bytes;
  const int32_t* nbr;
  uint32_t nbr_ld;
  int kvol;
  const uint32_t* n_out_dev;
  uint32_t n_bound;
  // rows the persistent grid of the tile-plan kernel is sized for, 1 .. n_bound: the larger of the caller's
  // fixed_launch_points and the row count of the previous forward.  Never a limit: its waves loop over all tiles.
  // (The LDS-staged kernels launch one workgroup per tile of the bound; workgroups beyond the count leave at once.
  // A loop over tiles in those kernels was built and measured: the compiler then spills 100 .. 680 bytes of registers
  // per lane and every layer takes 1.3 .. 2.4 times as long, while the surplus workgroups it saves cost under 1 us.)
  uint32_t launch_rows;
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
  int res_vec16;            // residual rows are 16-byte aligned and a multiple of 16 bytes
  int mid_dtype;
  float mid_s, mid_r;       // amax_mid / 127, 127 / amax_mid
  float a_rq_s, a_rq_r;     // re-quantisation of an fp16 operand by an int8 Add (0 = none)
  float b_rq_s, b_rq_r;
  int relu2;
  int out_vec16;     // output rows are 16-byte aligned and a multiple of 16 bytes: 16-byte stores allowed
  const char* zrow;  // 512 bytes of zeros (gather source of lanes without a neighbour), then 256 words of -1
  // tile plan of the rulebook (k_conv_tile only; see TilePlan): one word per 32-row tile with the kernel offsets
  // at which some row of the tile has a neighbour, and, when the rows were sorted by their offset sets, the row
  // that each position of the plan order stands for (nbr is then the table in plan order)
  const uint32_t* tmask = nullptr;
  const uint32_t* perm = nullptr;
  const uint4* wfrag32 = nullptr;  // weights in 32x32 MFMA fragment order, steps32 K-steps
  int steps32 = 0;
};

// What a convolution launch may use of a rulebook's tile plan.
struct PlanView {
  const uint32_t* tmask = nullptr;
  const uint32_t* perm = nullptr;   // nullptr: plan order = row order
  const int32_t* nbr = nullptr;     // table in plan order (sorted plans), else nullptr
};

// Launch the kernel for these weights (one definition per element type, each in its own translation unit).
// n_hint: expected number of output rows.  Returns false when no kernel covers the shape.
bool conv_dispatch_int8(const ConvWeights& w, uint32_t n_hint, ConvArgs& a, hipStream_t stream);
bool conv_dispatch_fp16(const ConvWeights& w, uint32_t n_hint, ConvArgs& a, hipStream_t stream);
// Shapes the tile-plan kernel covers (narrow layers: input rows of at most 64 bytes, at most 64 output channels).
bool conv_tile_covers(const ConvWeights& w);

}  // namespace scn
