// spconv::load_engine_from_onnx for the MI355X SCN engine.
// Same signature as libraries/3DSparseConvolution/src/onnx-parser.hpp:32-40; the model file is read by
// libscn_hip.so itself (a protobuf wire-format reader, no libprotobuf).  Returns nullptr on failure.
#ifndef SCN_SPCONV_ONNX_PARSER_HPP
#define SCN_SPCONV_ONNX_PARSER_HPP

#include <memory>
#include <string>

#include "engine.hpp"

namespace spconv {

/**
 * onnx_file: the custom "scn" ONNX dialect written by the reference's exporters.
 * precision: Float16 forces every layer to fp16; Int8 honours the per-layer precision attributes
 *            (layers without dynamic ranges stay fp16).
 * sortmask: a hint, passed on (the engine re-orders rows only where that is faster; results never change).
 * with_auxiliary_stream: passed on (rulebooks are built on a second stream ahead of the convolutions).
 * enable_blackwell: accepted for source compatibility, ignored.
 * stream: the stream used for one-time uploads; avoid the default stream for forward().
 */
inline std::shared_ptr<Engine> load_engine_from_onnx(const std::string& onnx_file, Precision precision = Precision::Float16,
                                                     bool sortmask = false, bool enable_blackwell = false,
                                                     bool with_auxiliary_stream = false,
                                                     unsigned int fixed_launch_points = 10000, void* stream = nullptr) {
  (void)enable_blackwell;
  const unsigned flags = (sortmask ? SCN_BUILD_SORTMASK : 0u) | (with_auxiliary_stream ? SCN_BUILD_AUX_STREAM : 0u);
  scn_engine* e = scn_engine_create_from_onnx(onnx_file.c_str(), static_cast<int>(precision), flags, fixed_launch_points, stream);
  if (!e) return nullptr;
  return std::shared_ptr<Engine>(new detail::EngineImpl(e));
}

}  // namespace spconv

#endif  // SCN_SPCONV_ONNX_PARSER_HPP
