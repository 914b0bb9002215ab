// Command-line driver of the SCN engine written against include/spconv/*.hpp only.
//
// Plays the role of the reference's demo driver (libraries/3DSparseConvolution/src/main.cpp:121-205):
// load a model, alias caller-owned device buffers as the engine input, optionally capture forward()
// into a HIP graph (SCN_USE_HIPGRAPH=1; a device-side row count is then used, like SPCONV_USE_DDS),
// run once and save the outputs, or time 100 + 1000 iterations with PROFILE=1.
//
//   infer <model.scn.onnx> <features.tensor> <indices.tensor> <g0> <g1> <g2> [fp16|int8] [output prefix]
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include <spconv/check.hpp>
#include <spconv/engine.hpp>
#include <spconv/onnx-parser.hpp>
#include <spconv/timer.hpp>
#include <spconv/version.hpp>

static bool env_is_1(const char* name) {
  const char* v = getenv(name);
  return v && !strcmp(v, "1");
}

int main(int argc, char** argv) {
  if (argc < 7) {
    printf("usage: %s model.onnx features.tensor indices.tensor g0 g1 g2 [fp16|int8] [output prefix]\n", argv[0]);
    printf("spconv-compatible API %s on %s\n", NVSPCONV_VERSION, SCN_BACKEND);
    return 1;
  }
  const auto precision = (argc > 7 && !strcmp(argv[7], "int8")) ? spconv::Precision::Int8 : spconv::Precision::Float16;
  const std::string out_prefix = argc > 8 ? argv[8] : "output";
  const std::vector<int> grid = {atoi(argv[4]), atoi(argv[5]), atoi(argv[6])};

  hipStream_t stream;
  if (!check_hip_api(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking))) return 2;
  spconv::set_logger_level(spconv::LoggerLevel::Warn);

  auto engine = spconv::load_engine_from_onnx(argv[1], precision);
  if (engine == nullptr) {
    printf("Failed to load the model %s\n", argv[1]);
    return 3;
  }
  auto src_features = spconv::Tensor::load(argv[2], true, stream);
  auto src_indices = spconv::Tensor::load(argv[3], true, stream);
  if (src_features.empty() || src_indices.empty()) {
    printf("Failed to load the input tensors\n");
    return 4;
  }
  // the engine aliases these buffers; their contents are filled in after the (optional) capture
  auto features = src_features.clone(stream);
  auto indices = src_indices.clone(stream);
  features.memset(0, stream);
  indices.memset(0, stream);
  engine->input(0)->features().reference(features.ptr(), features.shape, features.dtype(), true);
  engine->input(0)->indices().reference(indices.ptr(), indices.shape, indices.dtype(), true);
  engine->input(0)->set_grid_size(grid);

  const bool use_graph = env_is_1("SCN_USE_HIPGRAPH");
  uint32_t* num_rows_dev = nullptr;
  if (use_graph || env_is_1("SCN_USE_DDS")) {
    const uint32_t n = (uint32_t)src_features.size(0);
    check_hip_api(hipMalloc(&num_rows_dev, sizeof(uint32_t)));
    check_hip_api(hipMemcpy(num_rows_dev, &n, sizeof(uint32_t), hipMemcpyHostToDevice));
    engine->input(0)->set_dds_num_of_points_pointer(num_rows_dev);
    printf("device-side number of rows: %u\n", n);
  }
  hipGraph_t graph = nullptr;
  hipGraphExec_t graph_exec = nullptr;
  if (use_graph) {
    check_hip_api(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
    engine->forward(stream);
    check_hip_api(hipStreamEndCapture(stream, &graph));
    check_hip_api(hipGraphInstantiate(&graph_exec, graph, nullptr, nullptr, 0));
  }
  check_hip_api(hipMemcpyAsync(features.ptr(), src_features.ptr(), features.bytes(), hipMemcpyDeviceToDevice, stream));
  check_hip_api(hipMemcpyAsync(indices.ptr(), src_indices.ptr(), indices.bytes(), hipMemcpyDeviceToDevice, stream));

  auto run = [&]() {
    if (use_graph)
      check_hip_api(hipGraphLaunch(graph_exec, stream));
    else
      engine->forward(stream);
  };
  if (env_is_1("PROFILE")) {
    spconv::set_logger_level(spconv::LoggerLevel::Error);
    for (int i = 0; i < 100; ++i) run();
    spconv::EventTimer timer;
    timer.start(stream);
    for (int i = 0; i < 1000; ++i) run();
    printf("forward: %.4f ms per frame (%s, %s)\n", timer.stop(nullptr, false) / 1000.f,
           spconv::get_precision_string(precision), use_graph ? "hip graph" : "direct launches");
  } else {
    run();
    check_hip_api(hipStreamSynchronize(stream));
    for (size_t i = 0; i < engine->num_output(); ++i) {
      auto& t = engine->output((unsigned)i)->features();
      const std::string file = out_prefix + "." + std::to_string(i) + ".tensor";
      printf("output[%zu] %s %s -> %s (absmax %.5f)\n", i, spconv::dtype_string(t.dtype()), spconv::format_shape(t.shape),
             file.c_str(), t.absmax(stream));
      t.save(file.c_str(), stream);
    }
  }
  engine.reset();
  if (graph_exec) check_hip_api(hipGraphExecDestroy(graph_exec));
  if (graph) check_hip_api(hipGraphDestroy(graph));
  if (num_rows_dev) check_hip_api(hipFree(num_rows_dev));
  check_hip_api(hipStreamDestroy(stream));
  return 0;
}
