// The lidar half of CUDA-CenterPoint's CenterPoint::doinfer (src/centerpoint.cpp:136-150) on this library:
// raw fp32 sweep -> PreProcessCuda::generateVoxels / getOutput (include/legacy/preprocess.h) -> the older
// single-call engine interface (include/legacy/spconv/engine.hpp) -> dense BEV tensor.
//
//   centerpoint_pre <model.scn.onnx> <points.bin: fp32 [N, 5]> [fp16|int8] [output prefix]
// writes <prefix>.features.tensor / <prefix>.indices.tensor (the voxels) and <prefix>.bev.tensor
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <preprocess.h>       // compiled with -Iinclude/legacy first
#include <spconv/engine.hpp>  // the legacy header
#include <spconv/tensor.hpp>

int main(int argc, char** argv) {
  if (argc < 3) {
    printf("usage: %s model.onnx points.bin [fp16|int8] [output prefix]\n", argv[0]);
    return 1;
  }
  const auto precision = (argc > 3 && !strcmp(argv[3], "int8")) ? spconv::Precision::Int8 : spconv::Precision::Float16;
  const std::string prefix = argc > 4 ? argv[4] : "centerpoint";
  FILE* f = fopen(argv[2], "rb");
  if (!f) {
    printf("Failed to open %s\n", argv[2]);
    return 2;
  }
  fseek(f, 0, SEEK_END);
  const long bytes = ftell(f);
  fseek(f, 0, SEEK_SET);
  std::vector<float> host((size_t)bytes / sizeof(float));
  if (fread(host.data(), 1, (size_t)bytes, f) != (size_t)bytes) return 2;
  fclose(f);
  const unsigned int point_num = (unsigned int)(host.size() / 5);

  hipStream_t stream;
  if (hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) != hipSuccess) return 3;
  float* points = nullptr;
  if (hipMalloc((void**)&points, (size_t)bytes ? (size_t)bytes : 16) != hipSuccess) return 3;
  if (hipMemcpyAsync(points, host.data(), (size_t)bytes, hipMemcpyHostToDevice, stream) != hipSuccess) return 3;

  auto engine = spconv::load_engine_from_onnx(argv[1], precision);
  if (engine == nullptr) {
    printf("Failed to load the model %s\n", argv[1]);
    return 4;
  }
  PreProcessCuda pre;
  if (pre.alloc_resource() != 0) return 5;

  half* d_voxel_features = nullptr;
  unsigned int* d_voxel_indices = nullptr;
  std::vector<int> sparse_shape;
  spconv::DTensor* result = nullptr;
  unsigned int valid_num = 0;
  for (int rep = 0; rep < 2; ++rep) {   // the second frame re-uses everything the first one allocated
    if (pre.generateVoxels(points, point_num, stream) != 0) return 6;
    valid_num = pre.getOutput(&d_voxel_features, &d_voxel_indices, sparse_shape);
    result = engine->forward({valid_num, 5}, spconv::DType::Float16, d_voxel_features, {valid_num, 4},
                             spconv::DType::Int32, d_voxel_indices, 1, sparse_shape, stream);
    if (result == nullptr) return 7;
  }
  if (hipStreamSynchronize(stream) != hipSuccess) return 8;
  printf("points: %u  valid_num: %u  sparse_shape: %d x %d x %d\n", point_num, valid_num, sparse_shape[0], sparse_shape[1],
         sparse_shape[2]);
  spconv::Tensor::from_data_reference(d_voxel_features, {valid_num, 5}, spconv::DataType::Float16)
      .save((prefix + ".features.tensor").c_str(), stream);
  spconv::Tensor::from_data_reference(d_voxel_indices, {valid_num, 4}, spconv::DataType::Int32)
      .save((prefix + ".indices.tensor").c_str(), stream);
  std::vector<int64_t> shape;
  for (auto d : result->features_shape()) shape.push_back(d);
  printf("bev:");
  for (auto d : shape) printf(" %ld", (long)d);
  printf("\n");
  spconv::Tensor::from_data_reference(result->features_data(), shape, spconv::DataType::Float16)
      .save((prefix + ".bev.tensor").c_str(), stream);
  (void)hipFree(points);
  (void)hipStreamDestroy(stream);
  return 0;
}
