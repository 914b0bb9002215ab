// CenterPoint-style caller of the older single-call engine interface (include/legacy/spconv/engine.hpp):
// what CUDA-CenterPoint/src/centerpoint.cpp:136-150 does with the backbone -- one forward(...) call that
// takes shapes, types and device pointers and returns the dense BEV tensor -- plus the precision overrides
// of that interface.
//
//   infer_legacy <model.scn.onnx> <features.tensor> <indices.tensor> <g0> <g1> <g2> [fp16|int8] [output prefix] [all-fp16|calibrate]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include <spconv/engine.hpp>  // the legacy header: this file is compiled with -Iinclude/legacy first
#include <spconv/tensor.hpp>

int main(int argc, char** argv) {
  if (argc < 7) {
    printf("usage: %s model.onnx features.tensor indices.tensor g0 g1 g2 [fp16|int8] [output prefix] [all-fp16|calibrate]\n", argv[0]);
    return 1;
  }
  const auto precision = (argc > 7 && !strcmp(argv[7], "int8")) ? spconv::Precision::Int8 : spconv::Precision::Float16;
  const std::string out_prefix = argc > 8 ? argv[8] : "output";
  const bool all_fp16 = argc > 9 && !strcmp(argv[9], "all-fp16");
  const bool calibrate = argc > 9 && !strcmp(argv[9], "calibrate");
  const std::vector<int> grid = {atoi(argv[4]), atoi(argv[5]), atoi(argv[6])};
  hipStream_t stream;
  if (hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) != hipSuccess) return 2;

  auto engine = spconv::load_engine_from_onnx(argv[1], precision);
  if (engine == nullptr) {
    printf("Failed to load the model %s\n", argv[1]);
    return 3;
  }
  if (all_fp16) {
    // every node back to fp16, then re-plan: the int8 model must now give the fp16 engine's result
    engine->set_node_precision_byoptype("SparseConvolution", spconv::Precision::Float16, spconv::Precision::Float16);
    engine->set_node_precision_byoptype("Add", spconv::Precision::Float16, spconv::Precision::Float16);
    engine->reconfigure();
  }
  auto features = spconv::Tensor::load(argv[2], true, stream);
  auto indices = spconv::Tensor::load(argv[3], true, stream);
  if (features.empty() || indices.empty()) {
    printf("Failed to load the input tensors\n");
    return 4;
  }
  if (calibrate) {
    // implicit calibration: one forward records every tensor's largest magnitude, then every convolution and
    // Add is switched to int8 and the engine is planned again with those ranges
    engine->set_int8_calibration(true);
    if (engine->forward({features.size(0), features.size(1)}, spconv::DType::Float16, features.ptr(),
                        {indices.size(0), indices.size(1)}, spconv::DType::Int32, indices.ptr(), 1, grid, stream) == nullptr)
      return 5;
    engine->set_int8_calibration(false);
    engine->set_node_precision_byoptype("SparseConvolution", spconv::Precision::Int8, spconv::Precision::Int8);
    engine->set_node_precision_byoptype("Add", spconv::Precision::Int8, spconv::Precision::Int8);
    engine->reconfigure();
  }
  spconv::DTensor* result = nullptr;
  for (int rep = 0; rep < 2; ++rep)   // the second call re-uses everything the first one allocated
    result = engine->forward({features.size(0), features.size(1)}, spconv::DType::Float16, features.ptr(),
                             {indices.size(0), indices.size(1)}, spconv::DType::Int32, indices.ptr(), 1, grid, stream);
  if (result == nullptr) {
    printf("forward failed\n");
    return 5;
  }
  if (hipStreamSynchronize(stream) != hipSuccess) return 6;
  const auto shape = result->features_shape();
  printf("output shape:");
  for (auto v : shape) printf(" %lld", (long long)v);
  printf("  (%s)\n", spconv::get_precision_string(precision));
  spconv::Tensor out = spconv::Tensor::from_data_reference(result->features_data(), shape, spconv::DataType::Float16, true);
  if (!out.save((out_prefix + ".0.tensor").c_str(), stream)) return 7;
  return 0;
}
