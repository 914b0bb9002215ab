// bevfusion::lidar::SCN: points -> voxels -> sparse backbone -> dense BEV tensor, over the C ABI (header-only).
//
// Same names as the reference's CUDA-BEVFusion/src/bevfusion/lidar-scn.hpp:33-56 and what its implementation
// does in lidar-scn.cpp:34-50.  The hand-off differs in one way: the reference reads the voxel count back to
// the host between the two stages; here the engine's input is bound once to the voxelizer's buffers at their
// capacity, with the voxelizer's device-side counter as the row count, so forward() only enqueues kernels and
// the whole points -> BEV pass can be captured into one HIP graph and replayed on frames of any size.
#ifndef SCN_BEVFUSION_LIDAR_SCN_HPP
#define SCN_BEVFUSION_LIDAR_SCN_HPP

#include <memory>
#include <string>
#include <vector>

#include "../spconv/engine.hpp"
#include "../spconv/onnx-parser.hpp"
#include "lidar-voxelization.hpp"

namespace bevfusion {
namespace lidar {

enum class Precision : int { NonePrecision = 0, Float16 = 1, Int8 = 2 };

struct SCNParameter {
  VoxelizationParameter voxelization;
  std::string model;
  CoordinateOrder order = CoordinateOrder::XYZ;
  Precision precision = Precision::Float16;
  // engine options of spconv::load_engine_from_onnx (not in the reference's struct, which takes the defaults)
  bool sortmask = false;
  bool with_auxiliary_stream = false;
  unsigned int fixed_launch_points = 10000;
};

class SCN {
 public:
  virtual ~SCN() = default;
  // points: device pointer to num_points x num_feature fp16 values; returns the dense fp16 output on the device
  virtual const nvtype::half* forward(const nvtype::half* points, unsigned int num_points, void* stream = nullptr) = 0;
  virtual std::vector<int64_t> shape() = 0;
};

namespace detail {
class SCNImplement : public SCN {
 public:
  bool init(const SCNParameter& param) {
    param_ = param;
    voxelization_ = create_voxelization(param_.voxelization);
    if (!voxelization_) return false;
    native_scn_ = spconv::load_engine_from_onnx(param_.model, static_cast<spconv::Precision>(param_.precision), param_.sortmask,
                                                false, param_.with_auxiliary_stream, param_.fixed_launch_points);
    return native_scn_ != nullptr;
  }
  const nvtype::half* forward(const nvtype::half* points, unsigned int num_points, void* stream) override {
    voxelization_->forward(points, (int)num_points, stream, param_.order);
    if (!voxelization_->last_forward_ok()) return nullptr;   // (logged there; the backbone must not run on stale voxels)
    auto* in = native_scn_->input(0);
    const int64_t cap = voxelization_->max_voxels();
    in->features().reference(const_cast<void*>(voxelization_->features()), {cap, (int64_t)voxelization_->voxel_dim()},
                             spconv::DataType::Float16, true);
    in->indices().reference(const_cast<void*>(voxelization_->indices()), {cap, (int64_t)voxelization_->indices_dim()},
                            spconv::DataType::Int32, true);
    in->set_dds_num_of_points_pointer(const_cast<uint32_t*>(voxelization_->num_voxels_device()));
    in->set_grid_size(voxelization_->grid_size());
    native_scn_->forward(stream);
    return native_scn_->output(0)->features().ptr<nvtype::half>();
  }
  std::vector<int64_t> shape() override { return native_scn_->output(0)->features().shape; }
  Voxelization* voxelization() { return voxelization_.get(); }
  spconv::Engine* engine() { return native_scn_.get(); }

 private:
  SCNParameter param_;
  std::shared_ptr<Voxelization> voxelization_;
  std::shared_ptr<spconv::Engine> native_scn_;
};
}  // namespace detail

inline std::shared_ptr<SCN> create_scn(const SCNParameter& param) {
  auto impl = std::make_shared<detail::SCNImplement>();
  if (!impl->init(param)) return nullptr;
  return impl;
}

}  // namespace lidar
}  // namespace bevfusion

#endif  // SCN_BEVFUSION_LIDAR_SCN_HPP
