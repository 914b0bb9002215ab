// points -> BEV with bevfusion::lidar::SCN (include/bevfusion/lidar-scn.hpp), the way the reference's
// CUDA-BEVFusion pipeline drives its lidar branch (CUDA-BEVFusion/src/bevfusion/lidar-scn.cpp:34-50), plus
// what the reference cannot do there: voxelization and backbone captured together into ONE HIP graph (no host
// round trip between them) and replayed on frames of different sizes.
//
//   lidar_scn <model.scn.onnx> <points.tensor fp16 [N, F]> <xyz|zyx> <fp16|int8> <output prefix> [aux]
//
// Runs the full frame eagerly and saves it to <prefix>.eager.tensor, then captures one forward and replays the
// graph on frames of N, N/2, N/3 and N points, comparing every replay with an eager forward of the same points.
// (The point count of a captured voxelizer launch is fixed, so a shorter frame is the same buffer with the
// remaining points moved outside the range, which the voxelizer drops; the eager forward is given the shorter
// count.)  Exit code 0 only when every comparison is bit-exact.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include <bevfusion/lidar-scn.hpp>
#include <spconv/check.hpp>
#include <spconv/tensor.hpp>

using namespace bevfusion::lidar;

static std::vector<unsigned char> download(const void* dev, size_t bytes, hipStream_t stream) {
  std::vector<unsigned char> host(bytes);
  check_hip_api(hipMemcpyAsync(host.data(), dev, bytes, hipMemcpyDeviceToHost, stream));
  check_hip_api(hipStreamSynchronize(stream));
  return host;
}

int main(int argc, char** argv) {
  if (argc < 6) {
    printf("usage: %s model.onnx points.tensor xyz|zyx fp16|int8 output-prefix [aux]\n", argv[0]);
    return 1;
  }
  hipStream_t stream;
  if (!check_hip_api(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking))) return 2;
  spconv::set_logger_level(spconv::LoggerLevel::Warn);
  auto points = spconv::Tensor::load(argv[2], true, stream);
  if (points.empty() || points.shape.size() != 2 || points.dtype() != spconv::DataType::Float16) {
    printf("points must be a Float16 [N, F] .tensor file\n");
    return 4;
  }
  const unsigned n_points = (unsigned)points.size(0);
  const int nf = (int)points.size(1);

  SCNParameter param;
  param.voxelization.min_range = nvtype::Float3(-54.0f, -54.0f, -5.0f);
  param.voxelization.max_range = nvtype::Float3(+54.0f, +54.0f, +3.0f);
  param.voxelization.voxel_size = nvtype::Float3(0.075f, 0.075f, 0.2f);
  param.voxelization.grid_size = VoxelizationParameter::compute_grid_size(
      param.voxelization.max_range, param.voxelization.min_range, param.voxelization.voxel_size);
  param.voxelization.num_feature = nf;
  param.voxelization.max_voxels = 160000;
  param.voxelization.max_points_per_voxel = 10;
  param.voxelization.max_points = (int)std::max(300000u, n_points);
  param.model = argv[1];
  param.order = !strcmp(argv[3], "zyx") ? CoordinateOrder::ZYX : CoordinateOrder::XYZ;
  param.precision = !strcmp(argv[4], "int8") ? Precision::Int8 : Precision::Float16;
  param.with_auxiliary_stream = argc > 6 && !strcmp(argv[6], "aux");
  const std::string prefix = argv[5];

  auto scn = create_scn(param);
  if (!scn) {
    printf("Failed to create the lidar SCN from %s\n", argv[1]);
    return 3;
  }
  // the frame the graph reads: same address every replay, contents replaced between replays
  spconv::Tensor frame = points.clone(stream);
  const nvtype::half* frame_ptr = frame.ptr<nvtype::half>();

  // eager forward of the whole frame (the first call also allocates everything)
  const nvtype::half* bev = scn->forward(frame_ptr, n_points, stream);
  const auto shape = scn->shape();
  size_t out_bytes = 2;
  for (auto d : shape) out_bytes *= (size_t)d;
  printf("output %s\n", spconv::format_shape(shape));
  const auto eager_full = download(bev, out_bytes, stream);
  spconv::Tensor::from_data_reference((void*)bev, shape, spconv::DataType::Float16, true)
      .save((prefix + ".eager.tensor").c_str(), stream);

  // one graph: voxelization + backbone
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
  check_hip_api(hipStreamBeginCapture(stream, hipStreamCaptureModeGlobal));
  scn->forward(frame_ptr, n_points, stream);
  if (!check_hip_api(hipStreamEndCapture(stream, &graph))) return 5;
  if (!check_hip_api(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0))) return 5;

  // frames of different sizes: the first k points, the rest moved far outside the range
  std::vector<unsigned short> host_pts((size_t)n_points * nf);
  check_hip_api(hipMemcpy(host_pts.data(), points.ptr(), host_pts.size() * 2, hipMemcpyDeviceToHost));
  const unsigned short far_away = 0x7bff;  // 65504 in fp16: outside every axis range
  int failures = 0;
  for (unsigned k : {n_points, n_points / 2, n_points / 3, n_points}) {
    std::vector<unsigned short> cut = host_pts;
    for (size_t p = k; p < n_points; ++p)
      for (int a = 0; a < 3; ++a) cut[p * nf + a] = far_away;
    check_hip_api(hipMemcpyAsync(frame.ptr(), cut.data(), cut.size() * 2, hipMemcpyHostToDevice, stream));
    check_hip_api(hipStreamSynchronize(stream));
    check_hip_api(hipGraphLaunch(exec, stream));
    const auto replay = download(bev, out_bytes, stream);
    // the same k points, eagerly and as a shorter frame
    scn->forward(frame_ptr, k, stream);
    const auto eager = download(bev, out_bytes, stream);
    const bool same = replay == eager && (k != n_points || replay == eager_full);
    size_t nonzero = 0;
    for (size_t i = 0; i < replay.size(); i += 2) nonzero += (replay[i] | replay[i + 1]) != 0;
    printf("graph replay with %u of %u points: %s (%zu non-zero outputs)\n", k, n_points, same ? "bit-exact" : "MISMATCH", nonzero);
    failures += same ? 0 : 1;
  }
  check_hip_api(hipGraphExecDestroy(exec));
  check_hip_api(hipGraphDestroy(graph));
  scn.reset();
  check_hip_api(hipStreamDestroy(stream));
  return failures ? 6 : 0;
}
