// Host side of the convolution: weight packing into MFMA operand order, argument checks and the
// choice of kernel; C ABI of the convolution stage.
#include "scn_conv_args.hpp"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <vector>

namespace scn {

bool ConvWeights::init(const uint16_t* w_fp16, const int shape[5], const float* ranges, const uint16_t* bias_fp16,
                       int prec) {
  if (!set_geometry(shape, prec)) {
    set_error("invalid weight shape");
    return false;
  }
  if (prec == SCN_PRECISION_INT8 && ranges == nullptr) {
    set_error("int8 convolution needs weight_dynamic_ranges");
    return false;
  }
  const int epc = prec == SCN_PRECISION_INT8 ? 16 : 8;  // elements per 16-byte chunk
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
    if (!zrow.alloc(1536) || hipMemset(zrow.p, 0, 512) != hipSuccess ||
        hipMemset(zrow.as<char>() + 512, 0xFF, 1024) != hipSuccess ||  // 256 words of -1 ("no neighbour")
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

bool conv_tile_covers(const ConvWeights& w) {
  static const bool off = [] {
    const char* e = getenv("SCN_CONV_IMPL");
    return e && (!strcmp(e, "lds") || !strcmp(e, "rows"));
  }();
  if (off || w.kvol > 31 || w.mtiles32 < 1 || w.mtiles32 > 2) return false;
  if (w.chunks != 1 && w.chunks != 2 && w.chunks != 4) return false;
  // the whole weight tensor stays in LDS: [steps32][mtiles32] fragments of 1 KB
  return (size_t)w.steps32 * w.mtiles32 * 1024 + 512 <= 60 * 1024;
}

int conv_forward(const ConvWeights& w, const int32_t* nbr, uint32_t nbr_ld, const uint32_t* n_out_dev,
                 uint32_t n_bound, uint32_t n_hint, const scn_conv_io& io, hipStream_t stream, const PlanView* plan) {
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
  a.wfrag32 = w.wfrag32.as<uint4>();
  a.steps32 = w.steps32;
  if (plan && plan->tmask && conv_tile_covers(w)) {
    a.tmask = plan->tmask;
    a.perm = plan->perm;
    if (plan->nbr) a.nbr = plan->nbr;
  }
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
  {
    const size_t rsz = io.res_dtype == SCN_DTYPE_INT8 ? 1 : 2;
    a.res_vec16 = (io.res_dev && ((size_t)io.res_ld * rsz) % 16 == 0 && ((uintptr_t)io.res_dev & 15) == 0) ? 1 : 0;
  }
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
  if (n_hint == 0 || n_hint > n_bound) n_hint = n_bound;
  // fixed_launch_points (engine.hpp:107,150; src/infer.cpp:380-398): 0 sizes the grid for the bound, as a caller
  // that knows nothing about its inputs must; otherwise for that many rows or for what the previous forward had,
  // whichever is more
  a.launch_rows = io.fixed_launch_points ? std::min(n_bound, std::max(io.fixed_launch_points, n_hint)) : n_bound;
  if (a.launch_rows == 0) a.launch_rows = 1;
  const bool ok = w.precision == SCN_PRECISION_INT8 ? conv_dispatch_int8(w, n_hint, a, stream)
                                                    : conv_dispatch_fp16(w, n_hint, a, stream);
  SCN_REQUIRE(ok, SCN_ERR_UNSUPPORTED, "conv: no kernel for Cin=%d Cout=%d (chunks %d, m-tiles %d)", w.cin, w.cout,
              w.chunks, w.mtiles);
  SCN_HIP(hipGetLastError());
  return SCN_OK;
}

}  // namespace scn

using namespace scn;

extern "C" {
// ---- convolution ----------------------------------------------------------------------------

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
  PlanView pv;
  const TilePlan& tp = rb->rb.plan;
  if (tp.built) {
    pv.tmask = tp.tmask.as<uint32_t>();
    if (tp.sorted) {
      pv.perm = tp.perm.as<uint32_t>();
      pv.nbr = tp.nbr.as<int32_t>();
    }
  }
  int rc = conv_forward(c->w, rb->rb.nbr.as<int32_t>(), rb->rb.ld, rb->rb.n_out_dev(), rb->rb.n_bound_out,
                        rb->rb.n_out_hint(), *io, (hipStream_t)stream, tp.built ? &pv : nullptr);
  if (rc == SCN_OK && debug_sync_enabled()) rc = debug_sync_check((hipStream_t)stream, "scn_conv_forward");
  return rc;
}

}  // extern "C"
