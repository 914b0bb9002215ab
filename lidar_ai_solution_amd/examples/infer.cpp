// Command-line driver of the SCN engine written against include/spconv/*.hpp only.
//
// Plays the role of the reference's demo drivers (libraries/3DSparseConvolution/src/main.cpp:121-205 and
// src/infer.cpp:253-466, libspconv/example/infer.cpp:344-367,499-553): load a model, alias caller-owned device
// buffers as the engine input, optionally capture forward() into a HIP graph with a device-side row count, then
//   - run once and save the outputs (default),
//   - time 100 + 1000 iterations (PROFILE=1),
//   - stress: many forwards on an input that shrinks by a seeded random amount each time, through the
//     device-side count (graph / DDS) or by re-referencing the input tensors, every result compared with a
//     plain second engine's on the same rows; stops at the first mismatch (STRESS=<iterations>),
//   - search the fastest of {graph, fixed_launch_points, sortmask, auxiliary stream} (SEARCH_BEST_PERF=1).
// Switches come from the environment so that the positional command line stays what it was:
//   SCN_USE_HIPGRAPH=1  SCN_USE_DDS=1  SCN_SORTMASK=1  SCN_AUX_STREAM=1  SCN_FIXED_LAUNCH_POINTS=<n>  SCN_SEED=<n>
//
//   infer <model.scn.onnx> <features.tensor> <indices.tensor> <g0> <g1> <g2> [fp16|int8] [output prefix]
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <tuple>
#include <vector>

#include <spconv/check.hpp>
#include <spconv/engine.hpp>
#include <spconv/memory.hpp>
#include <spconv/onnx-parser.hpp>
#include <spconv/timer.hpp>
#include <spconv/version.hpp>

static bool env_is_1(const char* name) {
  const char* v = getenv(name);
  return v && !strcmp(v, "1");
}
static long env_int(const char* name, long dflt) {
  const char* v = getenv(name);
  return v && *v ? atol(v) : dflt;
}

struct Task {
  std::string onnx;
  spconv::Precision precision = spconv::Precision::Float16;
  std::vector<int> grid;
  spconv::Tensor src_features, src_indices;  // on the device
  bool use_graph = false, use_dds = false, sortmask = false, aux_stream = false;
  unsigned fixed_launch_points = 10000;
  bool profiling = false;
  int stress_iterations = 0;
  unsigned seed = 1;
  std::string out_prefix = "output";
  float latency_ms = 0.f;  // result of a profiling run
};

// One engine with its staging buffers: the engine aliases `features` / `indices`, which are typed views of
// buffers handed out by a GPUDataManager (the way the reference's Python module holds its inputs,
// libraries/3DSparseConvolution/src/pyscn.cpp:47-125).
struct Runner {
  std::shared_ptr<spconv::Engine> engine;
  spconv::GPUDataManager buffers;
  spconv::GPUMemory<unsigned short> features;
  spconv::GPUMemory<unsigned int> indices;
  uint32_t* num_rows_dev = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t graph_exec = nullptr;
  int64_t channels = 0;

  bool init(const Task& t, bool graph_mode, bool dds, bool sortmask, bool aux, unsigned flp, hipStream_t stream) {
    engine = spconv::load_engine_from_onnx(t.onnx, t.precision, sortmask, false, aux, flp, stream);
    if (!engine) return false;
    channels = t.src_features.size(1);
    features.set_gpudata(buffers.query_or_alloc("features", true, stream));
    indices.set_gpudata(buffers.query_or_alloc("indices", true, stream));
    features.alloc((size_t)t.src_features.numel, stream);
    indices.alloc((size_t)t.src_indices.numel, stream);
    if (features.empty() || indices.empty()) return false;
    // zero contents while (possibly) capturing: the real rows are copied in afterwards
    scn_memset_async(features.ptr(), 0, features.bytes(), stream);
    scn_memset_async(indices.ptr(), 0, indices.bytes(), stream);
    bind(t, (int64_t)t.src_features.size(0));
    engine->input(0)->set_grid_size(t.grid);
    if (graph_mode || dds) {
      const uint32_t n = (uint32_t)t.src_features.size(0);
      if (!check_hip_api(hipMalloc(&num_rows_dev, sizeof(uint32_t)))) return false;
      check_hip_api(hipMemcpyAsync(num_rows_dev, &n, sizeof(uint32_t), hipMemcpyHostToDevice, stream));
      engine->input(0)->set_dds_num_of_points_pointer(num_rows_dev);
    }
    if (graph_mode) {
      check_hip_api(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
      engine->forward(stream);
      if (!check_hip_api(hipStreamEndCapture(stream, &graph))) return false;
      if (!check_hip_api(hipGraphInstantiate(&graph_exec, graph, nullptr, nullptr, 0))) return false;
    }
    check_hip_api(hipMemcpyAsync(features.ptr(), t.src_features.ptr(), features.bytes(), hipMemcpyDeviceToDevice, stream));
    check_hip_api(hipMemcpyAsync(indices.ptr(), t.src_indices.ptr(), indices.bytes(), hipMemcpyDeviceToDevice, stream));
    return true;
  }
  // the engine's input = the first n rows of the staging buffers
  void bind(const Task& t, int64_t n) {
    engine->input(0)->features().reference(features.ptr(), {n, channels}, t.src_features.dtype(), true);
    engine->input(0)->indices().reference(indices.ptr(), {n, t.src_indices.size(1)}, t.src_indices.dtype(), true);
  }
  void set_device_rows(uint32_t n, hipStream_t stream) {
    check_hip_api(hipMemcpyAsync(num_rows_dev, &n, sizeof(uint32_t), hipMemcpyHostToDevice, stream));
    check_hip_api(hipStreamSynchronize(stream));  // n is a stack variable
  }
  void forward(hipStream_t stream) {
    if (graph_exec)
      check_hip_api(hipGraphLaunch(graph_exec, stream));
    else
      engine->forward(stream);
  }
  ~Runner() {
    engine.reset();
    if (graph_exec) check_hip_api(hipGraphExecDestroy(graph_exec));
    if (graph) check_hip_api(hipGraphDestroy(graph));
    if (num_rows_dev) check_hip_api(hipFree(num_rows_dev));
  }
};

static std::vector<unsigned char> download(spconv::Engine& e, hipStream_t stream) {
  auto& t = e.output(0)->features();
  std::vector<unsigned char> host(t.bytes());
  check_hip_api(hipMemcpyAsync(host.data(), t.ptr(), t.bytes(), hipMemcpyDeviceToHost, stream));
  check_hip_api(hipStreamSynchronize(stream));
  return host;
}

// returns 0, or the exit code of the failure
static int run_task(Task& t, hipStream_t stream) {
  Runner r;
  if (!r.init(t, t.use_graph, t.use_dds, t.sortmask, t.aux_stream, t.fixed_launch_points, stream)) {
    printf("Failed to load the model %s\n", t.onnx.c_str());
    return 3;
  }
  if (t.profiling) {
    const auto level = spconv::get_logger_level();
    spconv::set_logger_level(spconv::LoggerLevel::Error);
    for (int i = 0; i < 100; ++i) r.forward(stream);
    spconv::EventTimer timer;
    timer.start(stream);
    for (int i = 0; i < 1000; ++i) r.forward(stream);
    t.latency_ms = timer.stop(nullptr, false) / 1000.f;
    spconv::set_logger_level(level);
    return 0;
  }
  if (t.stress_iterations > 0) {
    // the checker: a plain engine (direct launches, one stream, no sorting) given exactly the rows under test
    Runner ref;
    if (!ref.init(t, false, false, false, false, 10000, stream)) return 3;
    srand(t.seed);
    int64_t rows = t.src_features.size(0);
    const bool by_count = t.use_graph || t.use_dds;
    for (int i = 0; i < t.stress_iterations && rows >= 0; ++i) {
      if ((i + 1) % 100 == 0) printf("Stress test: %d / %d, num_inputs: %ld\n", i + 1, t.stress_iterations, (long)rows);
      if (by_count) {
        if (rows == 0) break;  // (the reference stops this branch at zero rows too)
        r.set_device_rows((uint32_t)rows, stream);
      } else {
        r.bind(t, rows);
      }
      ref.bind(t, rows);
      r.forward(stream);
      ref.forward(stream);
      const auto got = download(*r.engine, stream), want = download(*ref.engine, stream);
      if (got.size() != want.size() || memcmp(got.data(), want.data(), got.size()) != 0) {
        printf("Stress test: MISMATCH at forward %d with %ld rows (seed %u)\n", i, (long)rows, t.seed);
        return 5;
      }
      rows -= rand() % 200;
    }
    printf("Stress test passed: every forward equal to the plain engine's (graph %d, dds %d, sortmask %d, aux stream %d)\n",
           (int)t.use_graph, (int)t.use_dds, (int)t.sortmask, (int)t.aux_stream);
    return 0;
  }
  r.forward(stream);
  check_hip_api(hipStreamSynchronize(stream));
  for (size_t i = 0; i < r.engine->num_output(); ++i) {
    auto& out = r.engine->output((unsigned)i)->features();
    const std::string file = t.out_prefix + "." + std::to_string(i) + ".tensor";
    printf("output[%zu] %s %s -> %s (absmax %.5f)\n", i, spconv::dtype_string(out.dtype()), spconv::format_shape(out.shape),
           file.c_str(), out.absmax(stream));
    out.save(file.c_str(), stream);
  }
  return 0;
}

// The reference's search over its performance switches (src/infer.cpp:371-466); there is no Blackwell switch here.
static int search_best_perf(Task& t, hipStream_t stream) {
  printf("Search the best performance configuration for the model: %s\n", t.onnx.c_str());
  const unsigned n = (unsigned)t.src_features.size(0);
  const unsigned p2 = (unsigned)(n * 0.2f) / 256 * 256, p3 = (unsigned)(n * 0.6f) / 256 * 256;
  printf("Proposed fixed launch points: %u, %u, %u\n", p2, p3, t.fixed_launch_points);
  typedef std::tuple<bool, unsigned, bool, bool, float> Config;  // graph, fixed launch points, sortmask, aux, latency
  std::vector<Config> done;
  float best = 1e30f;
  for (bool graph : {true, false}) {
    // the launch bound only matters where launch sizes cannot follow the input: under a captured graph
    const std::vector<unsigned> flps = graph ? std::vector<unsigned>{p2, p3, t.fixed_launch_points}
                                             : std::vector<unsigned>{t.fixed_launch_points};
    for (unsigned flp : flps)
      for (bool sortmask : {true, false})
        for (bool aux : {true, false}) {
          Task c = t;
          c.use_graph = graph, c.fixed_launch_points = flp, c.sortmask = sortmask, c.aux_stream = aux, c.profiling = true;
          const int rc = run_task(c, stream);
          if (rc) return rc;
          best = std::min(best, c.latency_ms);
          done.emplace_back(graph, flp, sortmask, aux, c.latency_ms);
          printf("  Iteration %zu / 16: Hipgraph: %s, Fixed Launch Points: %u, Sortmask: %s, Auxiliary Stream: %s, "
                 "Latency: %.3f ms. Best latency: %.3f ms\n", done.size(), graph ? "yes" : "no", flp, sortmask ? "yes" : "no",
                 aux ? "yes" : "no", c.latency_ms, best);
        }
  }
  std::sort(done.begin(), done.end(), [](const Config& a, const Config& b) { return std::get<4>(a) < std::get<4>(b); });
  const Config& b = done.front();
  printf("\nBest configuration found: \n   Hipgraph: %s, Fixed Launch Points: %u, Sortmask: %s, Auxiliary Stream: %s, "
         "Latency: %.3f ms\n\n", std::get<0>(b) ? "yes" : "no", std::get<1>(b), std::get<2>(b) ? "yes" : "no",
         std::get<3>(b) ? "yes" : "no", std::get<4>(b));
  printf("Sorted configuration list (%zu configurations): \n", done.size());
  for (size_t i = 0; i < done.size(); ++i)
    printf("  %02zu. Hipgraph: %s, Fixed Launch Points: %u, Sortmask: %s, Auxiliary Stream: %s, Latency: %.3f ms\n", i + 1,
           std::get<0>(done[i]) ? "yes" : "no", std::get<1>(done[i]), std::get<2>(done[i]) ? "yes" : "no",
           std::get<3>(done[i]) ? "yes" : "no", std::get<4>(done[i]));
  return 0;
}

int main(int argc, char** argv) {
  if (argc < 7) {
    printf("usage: %s model.onnx features.tensor indices.tensor g0 g1 g2 [fp16|int8] [output prefix]\n", argv[0]);
    printf("spconv-compatible API %s on %s\n", NVSPCONV_VERSION, SCN_BACKEND);
    return 1;
  }
  Task t;
  t.onnx = argv[1];
  t.precision = (argc > 7 && !strcmp(argv[7], "int8")) ? spconv::Precision::Int8 : spconv::Precision::Float16;
  if (argc > 8) t.out_prefix = argv[8];
  t.grid = {atoi(argv[4]), atoi(argv[5]), atoi(argv[6])};
  t.use_graph = env_is_1("SCN_USE_HIPGRAPH");
  t.use_dds = env_is_1("SCN_USE_DDS");
  t.sortmask = env_is_1("SCN_SORTMASK");
  t.aux_stream = env_is_1("SCN_AUX_STREAM");
  t.fixed_launch_points = (unsigned)env_int("SCN_FIXED_LAUNCH_POINTS", 10000);
  t.profiling = env_is_1("PROFILE");
  t.stress_iterations = (int)env_int("STRESS", 0);
  t.seed = (unsigned)env_int("SCN_SEED", 1);

  hipStream_t stream;
  if (!check_hip_api(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking))) return 2;
  spconv::set_logger_level(spconv::LoggerLevel::Warn);
  t.src_features = spconv::Tensor::load(argv[2], true, stream);
  t.src_indices = spconv::Tensor::load(argv[3], true, stream);
  if (t.src_features.empty() || t.src_indices.empty()) {
    printf("Failed to load the input tensors\n");
    return 4;
  }
  int rc;
  if (env_is_1("SEARCH_BEST_PERF")) {
    rc = search_best_perf(t, stream);
  } else {
    if (t.use_graph || t.use_dds) printf("device-side number of rows: %u\n", (unsigned)t.src_features.size(0));
    rc = run_task(t, stream);
    if (rc == 0 && t.profiling)
      printf("forward: %.4f ms per frame (%s, %s)\n", t.latency_ms, spconv::get_precision_string(t.precision),
             t.use_graph ? "hip graph" : "direct launches");
  }
  t.src_features = spconv::Tensor();
  t.src_indices = spconv::Tensor();
  check_hip_api(hipStreamDestroy(stream));
  return rc;
}
