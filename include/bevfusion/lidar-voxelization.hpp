// bevfusion::lidar::Voxelization over the C ABI of libscn_hip.so (header-only).
//
// Same names as the reference's CUDA-BEVFusion/src/bevfusion/lidar-voxelization.hpp:36-75: points
// (x, y, z, features...) in fp16 on the device -> mean features per voxel (fp16) and int32 indices
// (batch, then x,y,z or z,y,x).  Differences a caller can observe: rows come out in ascending linear-index
// order and a crowded voxel keeps its lowest point indices (the reference's order and choice depend on thread
// timing); forward() never waits for the GPU -- the voxel count stays on the device (num_voxels_device())
// until num_voxels() is called, which synchronises the stream of the last forward().
#ifndef SCN_BEVFUSION_LIDAR_VOXELIZATION_HPP
#define SCN_BEVFUSION_LIDAR_VOXELIZATION_HPP

#include <cmath>
#include <memory>
#include <vector>

#include "../common/dtype.hpp"
#include "../scn_c_api.h"
#include "../spconv/engine.hpp"

namespace bevfusion {
namespace lidar {

enum class CoordinateOrder : int {
  NoneOrder = 0,
  XYZ = 1,  // BEVFusion
  ZYX = 2   // CenterPoint
};

struct VoxelizationParameter {
  nvtype::Float3 min_range;
  nvtype::Float3 max_range;
  nvtype::Float3 voxel_size;
  nvtype::Int3 grid_size;
  int num_feature = 5;
  int max_voxels = 160000;
  int max_points_per_voxel = 10;
  int max_points = 300000;

  static nvtype::Int3 compute_grid_size(const nvtype::Float3& max_range, const nvtype::Float3& min_range,
                                        const nvtype::Float3& voxel_size) {
    return nvtype::Int3((int)std::round((max_range.x - min_range.x) / voxel_size.x),
                        (int)std::round((max_range.y - min_range.y) / voxel_size.y),
                        (int)std::round((max_range.z - min_range.z) / voxel_size.z));
  }
};

class Voxelization {
 public:
  virtual ~Voxelization() = default;
  // points: device pointer to num_points x num_feature fp16 values
  virtual void forward(const nvtype::half* points, int num_points, void* stream = nullptr,
                       CoordinateOrder output_order = CoordinateOrder::XYZ) = 0;
  virtual unsigned int num_voxels() = 0;   // waits for the last forward()
  virtual unsigned int voxel_dim() = 0;
  virtual unsigned int indices_dim() = 0;
  virtual std::vector<int> grid_size() = 0;
  virtual const void* indices() = 0;
  virtual const void* features() = 0;
  virtual CoordinateOrder order() = 0;
  // not in the reference: what a caller needs to hand the result on without a host round trip
  virtual const unsigned int* num_voxels_device() = 0;
  virtual unsigned int max_voxels() = 0;
  // false after a forward() that failed (invalid order, null points, launch error): the buffers then still hold the
  // previous frame and num_voxels() reports 0.  (forward() itself returns nothing, as in the reference.)
  virtual bool last_forward_ok() { return true; }
};

namespace detail {
class VoxelizationImplement : public Voxelization {
 public:
  ~VoxelizationImplement() override {
    if (v_) scn_voxelizer_destroy(v_);
  }
  bool init(const VoxelizationParameter& p) {
    param_ = p;
    scn_voxelization_param c{};
    c.min_range[0] = p.min_range.x, c.min_range[1] = p.min_range.y, c.min_range[2] = p.min_range.z;
    c.max_range[0] = p.max_range.x, c.max_range[1] = p.max_range.y, c.max_range[2] = p.max_range.z;
    c.voxel_size[0] = p.voxel_size.x, c.voxel_size[1] = p.voxel_size.y, c.voxel_size[2] = p.voxel_size.z;
    c.grid_size[0] = p.grid_size.x, c.grid_size[1] = p.grid_size.y, c.grid_size[2] = p.grid_size.z;
    c.num_feature = p.num_feature;
    c.max_voxels = p.max_voxels;
    c.max_points_per_voxel = p.max_points_per_voxel;
    c.max_points = p.max_points;
    v_ = scn_voxelizer_create(&c);
    return v_ != nullptr;
  }
  void forward(const nvtype::half* points, int num_points, void* stream, CoordinateOrder output_order) override {
    order_ = output_order;
    stream_ = stream;
    rc_ = scn_voxelizer_forward(v_, points, (uint32_t)(num_points < 0 ? 0 : num_points), (int)output_order, stream);
    if (rc_ != SCN_OK)
      spconv::logger_output(__FILE__, __LINE__, spconv::LoggerLevel::Error, "voxelization failed (%d): %s", rc_, scn_last_error());
  }
  bool last_forward_ok() override { return rc_ == SCN_OK; }
  unsigned int num_voxels() override { return rc_ == SCN_OK ? scn_voxelizer_num_voxels(v_, stream_) : 0u; }
  unsigned int voxel_dim() override { return (unsigned int)param_.num_feature; }
  unsigned int indices_dim() override { return 4; }
  std::vector<int> grid_size() override {
    int g[3];
    scn_voxelizer_grid_size(v_, (int)order_, g);
    return {g[0], g[1], g[2]};
  }
  const void* indices() override { return scn_voxelizer_indices(v_); }
  const void* features() override { return scn_voxelizer_features(v_); }
  CoordinateOrder order() override { return order_; }
  const unsigned int* num_voxels_device() override { return scn_voxelizer_num_voxels_dev(v_); }
  unsigned int max_voxels() override { return (unsigned int)param_.max_voxels; }

 private:
  VoxelizationParameter param_;
  scn_voxelizer* v_ = nullptr;
  CoordinateOrder order_ = CoordinateOrder::XYZ;
  void* stream_ = nullptr;
  int rc_ = SCN_OK;
};
}  // namespace detail

inline std::shared_ptr<Voxelization> create_voxelization(VoxelizationParameter parameter) {
  auto impl = std::make_shared<detail::VoxelizationImplement>();
  if (!impl->init(parameter)) return nullptr;
  return impl;
}

}  // namespace lidar
}  // namespace bevfusion

#endif  // SCN_BEVFUSION_LIDAR_VOXELIZATION_HPP
