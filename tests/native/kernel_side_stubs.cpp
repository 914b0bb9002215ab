// Host-only stand-ins for the kernel side of libscn_hip (the .hip translation units), so that the engine's host
// code -- ONNX reader, loader, builder checks, graph planning and fusion -- links into a plain g++ program that is
// built with AddressSanitizer and UndefinedBehaviorSanitizer and runs without a GPU.  Test infrastructure only:
// nothing here computes; whatever would launch a kernel reports SCN_ERR_UNSUPPORTED.  Weight and rulebook objects
// "initialise" successfully without touching a device, so that a well-formed model gets through the whole build and
// only fails, if at all, at the first device allocation.
#include "../../lidar_ai_solution_amd/csrc/scn_conv_args.hpp"
#include "../../lidar_ai_solution_amd/csrc/scn_kernels.hpp"

namespace scn {

static int no_device(const char* what) {
  set_error("%s: not available in the host-only build", what);
  return SCN_ERR_UNSUPPORTED;
}

bool CoordTable::alloc_filter(const int*) { return true; }
bool CoordTable::alloc_for(uint32_t) { return true; }
CoordLookup CoordTable::lookup() const { return CoordLookup{}; }
size_t hash_capacity_for(uint32_t n) {
  size_t cap = 1024;
  while (cap < (size_t)n * 2) cap <<= 1;
  return cap;
}
int fill_multi(const FillJob*, int, uint32_t*, const uint32_t*, uint32_t, hipStream_t) { return no_device("fill_multi"); }
int hash_build(const CoordTable&, const int32_t*, uint32_t, const uint32_t*, const int*, uint32_t*, hipStream_t) {
  return no_device("hash_build");
}
bool ConvWeights::init(const uint16_t* w, const int shape[5], const float* ranges, const uint16_t*, int prec) {
  if (!set_geometry(shape, prec)) {
    set_error("invalid weight shape");
    return false;
  }
  if (prec == SCN_PRECISION_INT8 && ranges == nullptr) {
    set_error("int8 convolution needs weight_dynamic_ranges");
    return false;
  }
  // touch every weight and range the real packing reads, so that a short buffer shows under the sanitizer
  unsigned sum = 0;
  for (size_t i = 0; i < (size_t)cout * kvol * cin; ++i) sum += w[i];
  if (ranges)
    for (int c = 0; c < cout; ++c) sum += ranges[c] > 0.f;
  return sum != 0xFFFFFFFFu || true;
}
bool conv_tile_covers(const ConvWeights& w) { return w.kvol <= 31 && w.mtiles32 <= 2 && w.chunks <= 4; }
int conv_forward(const ConvWeights&, const int32_t*, uint32_t, const uint32_t*, uint32_t, uint32_t, const scn_conv_io&,
                 hipStream_t, const PlanView*) {
  return no_device("conv_forward");
}
int absmax_rows(const void*, int, float, uint32_t, uint32_t, uint32_t, const uint32_t*, float*, hipStream_t) {
  return no_device("absmax_rows");
}
int convert_rows(const void*, int, uint32_t, uint32_t, float, void*, int, uint32_t, uint32_t, float, int, uint32_t,
                 const uint32_t*, hipStream_t) {
  return no_device("convert_rows");
}
int add_relu(const void*, int, float, float, const void*, int, float, float, void*, int, float, int, uint32_t, uint32_t,
             const uint32_t*, hipStream_t) {
  return no_device("add_relu");
}
int permute_dense(const void*, const int64_t*, const int*, void*, hipStream_t) { return no_device("permute_dense"); }
int scatter_dense(const void*, int, float, uint32_t, uint32_t, const int32_t*, uint32_t, const uint32_t*, const int*,
                  const int*, void*, hipStream_t, bool, int32_t*, bool, bool) {
  return no_device("scatter_dense");
}
int scatter_dense_form(const void*, int, float, uint32_t, uint32_t, const int32_t*, uint32_t, const uint32_t*, const int*,
                       const int*, int, int, int, float, void*, hipStream_t) {
  return no_device("scatter_dense_form");
}
int scatter_dense_build_map(const int32_t*, uint32_t, const uint32_t*, const int*, const int*, int32_t*, bool, hipStream_t) {
  return no_device("scatter_dense_build_map");
}
size_t scatter_dense_map_cells(const int*, const int*) { return 0; }
size_t scatter_dense_form_elements(const int*, int, int) { return 0; }

bool Rulebook::init(uint32_t max_in_, uint32_t max_out_, int kvol) {
  max_in = max_in_;
  max_out = max_out_;
  kvol_cap = kvol;
  ld = (std::max(max_in, max_out) + 63u) & ~63u;
  return true;
}
int Rulebook::reserve_sparse(const int*, bool) { return SCN_OK; }
int Rulebook::reserve_subm(bool) { return SCN_OK; }
int Rulebook::reserve_plan(bool) { return SCN_OK; }
int Rulebook::build_plan(bool, hipStream_t) { return no_device("build_plan"); }
int Rulebook::build_subm(const int32_t*, uint32_t, const uint32_t*, const int*, const int*, const int*, const CoordLookup*,
                         hipStream_t) {
  return no_device("build_subm");
}
int Rulebook::build_sparse(const int32_t*, uint32_t, const uint32_t*, const int*, const int*, const int*, const int*,
                           const int*, const CoordLookup*, hipStream_t) {
  return no_device("build_sparse");
}
int Rulebook::build_inverse(const Rulebook&, const uint32_t*, hipStream_t) { return no_device("build_inverse"); }
CoordLookup Rulebook::out_lookup() const { return CoordLookup{}; }
uint32_t Rulebook::n_out_hint() const { return n_bound_out; }

}  // namespace scn
