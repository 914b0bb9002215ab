// PreProcessCuda of CUDA-CenterPoint over the C ABI of libscn_hip.so (header-only).
//
// Same class, method and parameter names as the reference's CUDA-CenterPoint/include/preprocess.h:25-52 (with the
// voxelization part of `Params`, include/common.h:71-96), so that CenterPoint::doinfer (src/centerpoint.cpp:136-150)
//     pre_->generateVoxels((float*)points, point_num, stream);
//     valid_num = pre_->getOutput(&d_voxel_features, &d_voxel_indices, sparse_shape);
// compiles unchanged apart from cudaStream_t -> hipStream_t: the raw fp32 sweep [N, feature_num] on the device ->
// fp16 voxel means and int32 (batch, z, y, x) indices, sparse_shape = {Z + 1, Y, X}.  Differences a caller can
// observe: rows come out in ascending linear-index order and a crowded voxel keeps its lowest point indices
// (the reference's order and choice depend on thread timing); generateVoxels() does not wait for the GPU -- the
// one host synchronisation is in getOutput(), which needs the voxel count on the host as the reference's does.
#ifndef SCN_LEGACY_PREPROCESS_H
#define SCN_LEGACY_PREPROCESS_H

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <vector>

#include "../scn_c_api.h"

#ifndef MAX_POINTS_NUM
#define MAX_POINTS_NUM 300000
#endif

class Params {
 public:
  float min_x_range = -54, max_x_range = 54;
  float min_y_range = -54, max_y_range = 54;
  float min_z_range = -5.0f, max_z_range = 3.0f;
  float pillar_x_size = 0.075f, pillar_y_size = 0.075f, pillar_z_size = 0.2f;   // the size of a voxel
  int max_points_per_voxel = 10;
  unsigned int max_voxels = 160000;
  unsigned int feature_num = 5;

  int getGridXSize() const { return (int)std::round((max_x_range - min_x_range) / pillar_x_size); }
  int getGridYSize() const { return (int)std::round((max_y_range - min_y_range) / pillar_y_size); }
  int getGridZSize() const { return (int)std::round((max_z_range - min_z_range) / pillar_z_size); }
};

class PreProcessCuda {
 public:
  PreProcessCuda() = default;
  explicit PreProcessCuda(const Params& params) : params_(params) {}
  PreProcessCuda(const PreProcessCuda&) = delete;
  PreProcessCuda& operator=(const PreProcessCuda&) = delete;
  ~PreProcessCuda() {
    if (vox_) scn_voxelizer_destroy(vox_);
  }

  // allocates everything generateVoxels needs; 0 on success
  int alloc_resource() {
    if (vox_) return 0;
    scn_voxelization_param p{};
    p.min_range[0] = params_.min_x_range; p.min_range[1] = params_.min_y_range; p.min_range[2] = params_.min_z_range;
    p.max_range[0] = params_.max_x_range; p.max_range[1] = params_.max_y_range; p.max_range[2] = params_.max_z_range;
    p.voxel_size[0] = params_.pillar_x_size; p.voxel_size[1] = params_.pillar_y_size; p.voxel_size[2] = params_.pillar_z_size;
    p.grid_size[0] = params_.getGridXSize(); p.grid_size[1] = params_.getGridYSize(); p.grid_size[2] = params_.getGridZSize();
    p.num_feature = (int)params_.feature_num;
    p.max_voxels = (int)params_.max_voxels;
    p.max_points_per_voxel = params_.max_points_per_voxel;
    p.max_points = MAX_POINTS_NUM;
    vox_ = scn_voxelizer_create(&p);
    if (!vox_) {
      fprintf(stderr, "PreProcessCuda: %s\n", scn_last_error());
      return -1;
    }
    return 0;
  }

  // points: fp32 [points_size, feature_num] on the device; enqueues only
  int generateVoxels(const float* points, size_t points_size, hipStream_t stream) {
    if (alloc_resource() != 0) return -1;
    stream_ = stream;
    const int rc = scn_voxelizer_forward_points(vox_, points, SCN_DTYPE_FP32, (uint32_t)points_size, SCN_ORDER_ZYX, stream);
    if (rc != 0) fprintf(stderr, "PreProcessCuda::generateVoxels: %s\n", scn_last_error());
    last_rc_ = rc;
    return rc;
  }

  // device pointers of the voxel features ([n, feature_num] fp16) and indices ([n, 4] int32) of the last call,
  // the sparse shape {Z + 1, Y, X}, and n (this waits for the stream of the last generateVoxels)
  unsigned int getOutput(half** d_voxel_features, unsigned int** d_voxel_indices, std::vector<int>& sparse_shape) {
    sparse_shape.clear();
    if (!vox_ || last_rc_ != 0) return 0;   // (after a failed call the buffers still hold the previous frame)
    *d_voxel_features = (half*)scn_voxelizer_features(vox_);
    *d_voxel_indices = (unsigned int*)scn_voxelizer_indices(vox_);
    int g[3];
    scn_voxelizer_grid_size(vox_, SCN_ORDER_ZYX, g);
    sparse_shape.assign(g, g + 3);
    return scn_voxelizer_num_voxels(vox_, stream_);
  }

  // the voxel count of the last call where it is, for callers that hand it to the engine without a host round trip
  const unsigned int* num_voxels_device() const { return vox_ ? scn_voxelizer_num_voxels_dev(vox_) : nullptr; }

 private:
  Params params_;
  scn_voxelizer* vox_ = nullptr;
  hipStream_t stream_ = nullptr;
  int last_rc_ = 0;
};

#endif  // SCN_LEGACY_PREPROCESS_H
