// Internal C++ interface between the kernel translation unit and the engine / C-ABI layers.
#pragma once

#include "scn_common.hpp"

namespace scn {

// Open-addressing coordinate hash: 64-bit slots {key (linear voxel index) << 32 | row}.
constexpr uint64_t kEmptySlot = ~0ull;

// How a kernel turns a voxel's linear index into its row: either a coordinate hash (tensors whose rows
// are in caller order) or the occupancy bitmap + per-word ranks of a tensor in canonical order.
struct CoordLookup {
  const uint64_t* slots = nullptr;
  uint32_t mask = 0;
  const uint32_t* bitmap = nullptr;
  const uint32_t* prefix = nullptr;
  uint32_t rank_cap = 0;  // ranks >= rank_cap were truncated away
  const uint32_t* filter = nullptr;  // hash lookups: occupancy bitmap tested before probing (nullable)
  // Hash tables whose build also indexed the rows as a canonical-order tensor (see CoordTable): when *unsorted is 0
  // the rows were strictly ascending in linear index, the filter is their occupancy bitmap and first_row[word] the row
  // of the word's lowest set bit, so a look-up is a rank (two loads) and the hash table was not filled at all.
  const uint32_t* unsorted = nullptr;
  const uint32_t* first_row = nullptr;
};

struct CoordTable {
  DevBuf buf;
  size_t cap = 0;     // allocated slots, power of two
  uint32_t mask = 0;  // slots in use - 1 (power of two <= cap), set by the last build
  DevBuf filter;             // occupancy bitmap of the grid (optional, see alloc_filter); four more words follow it,
                             // the first of which is the "rows are not in canonical order" flag of the last build
  size_t filter_words = 0;
  // Canonical-order inputs (rows strictly ascending in linear voxel index: what a voxelizer that ranks cells emits)
  // need no hash: one kernel without atomics writes each occupied word of the filter and the row of its first
  // voxel, and look-ups become ranks.  The kernel also checks the order; when it does not hold, the hash insert
  // that follows (and skips itself otherwise) fills table and filter as for any caller order.  Whether the check
  // is launched at all follows the previous build's finding (a pinned host word), re-examined every 16th build.
  DevBuf first_row;
  HostBuf sorted_hint;
  uint32_t builds = 0;
  bool probed = false;       // the last build launched the canonical-order kernel
  size_t filter_fill_words() const { return filter_words ? filter_words + 4 : 0; }
  uint32_t* unsorted_flag() const { return filter.as<uint32_t>() + filter_words; }
  uint32_t precleared_for = 0xFFFFFFFFu;  // row count for which slots + filter were cleared by a batched fill
  bool alloc_for(uint32_t max_rows);
  bool alloc_filter(const int grid[3]);
  uint64_t* slots() const { return buf.as<uint64_t>(); }
  CoordLookup lookup() const;
};

size_t hash_capacity_for(uint32_t n);

struct ConvGeom {
  int grid_in[3];
  int grid_out[3];
  int ks[3];
  int stride[3];
  int pad[3];
  int dil[3];
  int kvol;
};

// Tile plan of a rulebook: what lets a convolution skip the kernel offsets at which none of a 32-row tile's rows
// has a neighbour (`sortmask` of the reference's loader, libraries/3DSparseConvolution/src/onnx-parser.hpp:35-37:
// "skip more insignificance computations").  tmask[t] = OR of the rows' offset sets (bit k: nbr[k][row] >= 0).
// A sorted plan also orders the rows by their offset set (stable, the sets as numbers, inside windows of 1024
// consecutive rows), so that the rows of a tile share most offsets: perm[j] = row at position j, nbr = the table in that order.  Results do not
// depend on the plan: every row still adds its own products in offset order.
struct TilePlan {
  DevBuf keys, keys_sorted, perm, tmask, nbr;
  uint32_t cap_rows = 0;   // positions allocated (multiple of 32)
  bool reserved_sorted = false;
  bool sorted = false;     // what the last build produced
  bool built = false;
};

// Rulebook object (= scn_rulebook of the C ABI).
struct Rulebook {
  uint32_t max_in = 0, max_out = 0;
  int kvol_cap = 0;
  bool subm = false;
  ConvGeom geom{};
  CoordTable own_in_table;    // hash of the input rows when no shared lookup is passed
  CoordLookup in_lookup;      // what the last build used to find input rows
  DevBuf nbr;                 // int32 [kvol_cap][ld]; every build leaves -1 in the rows from the count up to the
                              // next multiple of 32 (the convolution kernels fetch whole 32-row tiles of entries)
  uint32_t ld = 0;
  DevBuf out_idx;             // int32 [max_out][4] (strided)
  DevBuf counters;            // uint32: [0] n_out kept, [1] n_out before truncation, [2..] scratch
  HostBuf host_count;         // pinned: [0] n_out kept of the last build that has run (launch hint)
  DevBuf bitmap, blocksum, prefix;  // strided: occupancy bitmap of the output grid, per-block popcounts, per-word ranks
  size_t bitmap_words = 0, bitmap_cap_words = 0;
  DevBuf pair_scratch;        // pair compaction: per (k, block) counts
  const int32_t* in_indices = nullptr;
  const int32_t* out_indices = nullptr;  // subm: aliases in_indices
  uint32_t n_bound_in = 0, n_bound_out = 0;
  bool built = false;
  bool bitmap_precleared = false;  // the next build_sparse finds its output bitmap already zeroed
  TilePlan plan;

  bool init(uint32_t max_in_, uint32_t max_out_, int kvol);
  int reserve_sparse(const int out_grid[3], bool need_own_in_table);
  int reserve_subm(bool need_own_in_table);
  int build_subm(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3], const int ks[3],
                 const int dil[3], const CoordLookup* shared_lookup, hipStream_t stream);
  int build_sparse(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3], const int ks[3],
                   const int stride[3], const int pad[3], const int dil[3], const CoordLookup* shared_lookup,
                   hipStream_t stream);
  // the rulebook of SparseInverseConvolution: fwd (strided, built) with inputs and outputs swapped; n_in_dev
  // (nullable) is the device-side row count of fwd's input, which becomes this rulebook's output count
  int build_inverse(const Rulebook& fwd, const uint32_t* n_in_dev, hipStream_t stream);
  // tile plan of the table built last (kernel volumes up to 31); reserve_plan allocates, build_plan only launches
  int reserve_plan(bool sorted);
  int build_plan(bool sorted, hipStream_t stream);
  CoordLookup out_lookup() const;  // strided: rows of the output tensor from bitmap ranks
  int pairs(int32_t* pair_in, int32_t* pair_out, int64_t* offsets, uint64_t capacity, hipStream_t stream);
  const uint32_t* n_out_dev() const { return counters.as<uint32_t>(); }
  uint32_t n_out_hint() const;
};

// Packed weights of one convolution (= scn_conv of the C ABI).
struct ConvWeights {
  int cin = 0, cout = 0, kvol = 0, ks[3] = {1, 1, 1};
  int precision = SCN_PRECISION_FP16;  // compute precision
  int chunks = 0;   // 16-byte chunks per (padded) input row
  int mtiles = 0;   // ceil(cout / 16)
  int steps = 0;    // MFMA K-steps = ceil(kvol * chunks / 4)
  uint32_t cin_pad = 0;  // padded input channels the kernel expects (elements)
  DevBuf wfrag;     // [steps][mtiles][64] x 16 bytes, MFMA A-operand order
  int mtiles32 = 0, steps32 = 0;
  DevBuf zrow;      // 512 bytes of zeros, then 64 words of -1
  DevBuf wfrag32;   // cout > 16: [steps32][mtiles32][64] x 16 bytes, A-operand order of the 32x32 MFMA
  DevBuf wscale;    // fp32 [cout_pad]: s_w[c] (int8) or 1
  DevBuf bias;      // fp32 [cout_pad]
  bool init(const uint16_t* w_fp16, const int shape[5], const float* ranges, const uint16_t* bias_fp16, int prec);
  // the sizes above from a weight shape [Cout, K0, K1, K2, Cin] (host only; false for a shape with a dimension < 1)
  bool set_geometry(const int shape[5], int prec) {
    cout = shape[0];
    ks[0] = shape[1];
    ks[1] = shape[2];
    ks[2] = shape[3];
    cin = shape[4];
    if (cout <= 0 || cin <= 0 || ks[0] <= 0 || ks[1] <= 0 || ks[2] <= 0) return false;
    kvol = ks[0] * ks[1] * ks[2];
    precision = prec;
    const int epc = prec == SCN_PRECISION_INT8 ? 16 : 8;  // elements per 16-byte chunk
    const int ch = (cin + epc - 1) / epc;
    int p2 = 1;
    while (p2 < ch) p2 <<= 1;  // chunks per row rounded to a power of two (rows are padded to it)
    chunks = p2;
    cin_pad = (uint32_t)(chunks * epc);
    mtiles = (cout + 15) / 16;
    steps = (kvol * chunks + 3) / 4;
    mtiles32 = (cout + 31) / 32;
    if (mtiles32 == 3) mtiles32 = 4;  // kernels exist for 1, 2 and 4 tiles; the fourth is zero weights
    steps32 = 4 * ((kvol * chunks + 7) / 8);  // whole iterations of 4 K-steps, zero weights beyond the volume
    return true;
  }
};

// n_hint: expected row count (0 = unknown), only used to choose the launch configuration
struct PlanView;
int conv_forward(const ConvWeights& w, const int32_t* nbr, uint32_t nbr_ld, const uint32_t* n_out_dev,
                 uint32_t n_bound, uint32_t n_hint, const scn_conv_io& io, hipStream_t stream,
                 const PlanView* plan = nullptr);

int set_count(uint32_t* dst, const uint32_t* n_dev, uint32_t n_bound, hipStream_t stream);
int fill_u32(void* p, uint32_t value, size_t count, hipStream_t stream);
// several fills and (count_dst != nullptr) the publication of min(*n_dev, n_bound) in one launch
struct FillJob {
  void* p;
  size_t count;  // 32-bit words
  uint32_t value;
};
constexpr int kMaxFillJobs = 12;
int fill_multi(const FillJob* jobs, int n_jobs, uint32_t* count_dst, const uint32_t* n_dev, uint32_t n_bound,
               hipStream_t stream);
int hash_build(const CoordTable& t, const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int grid[3],
               uint32_t* n_eff_out, hipStream_t stream);
int hash_query(const CoordTable& t, const int32_t* coords, uint32_t n, const int grid[3], int32_t* rows,
               hipStream_t stream);

// the float arguments below are dynamic ranges (amax) of int8 operands, see scn_c_api.h
int convert_rows(const void* in, int in_dtype, uint32_t in_c, uint32_t in_ld, float in_range, void* out,
                 int out_dtype, uint32_t out_c, uint32_t out_ld, float out_range, int relu, uint32_t n,
                 const uint32_t* n_dev, hipStream_t stream);
int add_relu(const void* a, int a_dtype, float a_range, float a_rq, const void* b, int b_dtype, float b_range,
             float b_rq, void* out, int out_dtype, float out_range, int relu, uint32_t c, uint32_t n,
             const uint32_t* n_dev, hipStream_t stream);
// max |value| of the first min(*n_dev, n) rows x c channels -> *result_dev (a 16-byte aligned device float)
int absmax_rows(const void* x, int dtype, float range, uint32_t c, uint32_t ld, uint32_t n, const uint32_t* n_dev,
                float* result_dev, hipStream_t stream);
int scatter_dense(const void* feat, int dtype, float range, uint32_t c, uint32_t ld, const int32_t* idx, uint32_t n,
                  const uint32_t* n_dev, const int dense_shape[5], const int perm[5], void* out, hipStream_t stream,
                  bool precleared = false, int32_t* cell_map = nullptr, bool map_precleared = false,
                  bool map_built = false);
// first half of the map variant on its own (it needs only the coordinates): scatter_dense(..., map_built = true)
// may then follow on another stream once this one is done
int scatter_dense_build_map(const int32_t* idx, uint32_t n, const uint32_t* n_dev, const int dense_shape[5],
                            const int perm[5], int32_t* cell_map, bool map_precleared, hipStream_t stream);
// Cells of the row map that lets scatter_dense write the dense tensor in memory order (no clear, whole
// 16-byte stores); 0 when the layout does not qualify (channel axis not outermost, plane not a multiple of 8).
size_t scatter_dense_map_cells(const int dense_shape[5], const int perm[5]);

// the other forms of the dense output: layout 1 NCHW (with an optional Transpose), 2 NCHW32, 3 NHWzC of the
// [1, C * Z, H, W] view (zaxis 0: "zyx" tensors, 2: "xyz"), fp16 or int8 (out_range = its dynamic range)
size_t scatter_dense_form_elements(const int dense_shape[5], int zaxis, int layout);
int scatter_dense_form(const void* feat, int dtype, float range, uint32_t c, uint32_t ld, const int32_t* idx, uint32_t n,
                       const uint32_t* n_dev, const int dense_shape[5], const int perm[5], int zaxis, int layout,
                       int out_dtype, float out_range, void* out, hipStream_t stream);

int permute_dense(const void* in, const int64_t in_shape[5], const int perm[5], void* out, hipStream_t stream);

}  // namespace scn

// Rulebook and convolution objects of the C ABI.
struct scn_rulebook {
  scn::Rulebook rb;
};
struct scn_conv {
  scn::ConvWeights w;
};

// Voxelizer object of the C ABI.
struct scn_voxelizer {
  scn_voxelization_param p{};
  scn::DevBuf bitmap, blocksum, flags, pkey, mins, counts, feats, idx, counters;
  size_t words = 0;
  uint32_t* host_count = nullptr;  // pinned
  int last_order = SCN_ORDER_XYZ;
};
