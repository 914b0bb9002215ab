// spconv::Engine / EngineBuilder / SparseDTensor for the MI355X SCN engine.
//
// Header-only C++ surface with the class, method and enum names of the reference's public header
// (libraries/3DSparseConvolution/libspconv/include/spconv/engine.hpp:25-176), implemented over the C
// ABI of libscn_hip.so (include/scn_c_api.h).  Code written against the reference's engine API keeps
// compiling after its CUDA runtime calls are turned into HIP ones; `void* stream` is a hipStream_t.
//
// Differences that a caller can observe:
//   * build()'s enable_blackwell is accepted and ignored; sortmask and with_auxiliary_stream are passed on
//     (performance-only switches: results are bit-identical with and without them).
//   * device buffers are allocated when the grid size is set (set_grid_size) so that forward() is
//     legal inside hipStreamBeginCapture from the very first call.
#ifndef SCN_SPCONV_ENGINE_HPP
#define SCN_SPCONV_ENGINE_HPP

#include <cstdarg>
#include <cstdio>
#include <memory>
#include <string>
#include <vector>

#include "../scn_c_api.h"
#include "tensor.hpp"

namespace spconv {

#define Exported __attribute__((visibility("default")))

enum class Precision : int { None = 0, Float16 = 1, Int8 = 2 };
enum class TensorLayout : int { None = 0, NCHW = 1, NCHW32 = 2, NHWzC = 3 };
enum class LoggerLevel : int { Verb = 0, Warn = 1, Error = 2, Quiet = 99 };

class ILogger {
 public:
  virtual ~ILogger() = default;
  virtual void log(const char* message, LoggerLevel level, const char* file, int line) const = 0;
};

namespace detail {
inline ILogger*& logger_slot() {
  static ILogger* logger = nullptr;
  return logger;
}
inline void log_trampoline(const char* message, int level, const char* file, int line, void*) {
  if (ILogger* l = logger_slot()) l->log(message, static_cast<LoggerLevel>(level), file, line);
}
}  // namespace detail

inline const char* get_precision_string(Precision precision) {
  switch (precision) {
    case Precision::Float16: return "Float16";
    case Precision::Int8: return "Int8";
    default: return "None";
  }
}
inline const char* get_tensor_layout_string(TensorLayout layout) {
  switch (layout) {
    case TensorLayout::NCHW: return "NCHW";
    case TensorLayout::NCHW32: return "NCHW32";
    case TensorLayout::NHWzC: return "NHWzC";
    default: return "None";
  }
}
inline const char* logger_level_string(LoggerLevel level) {
  switch (level) {
    case LoggerLevel::Verb: return "verb";
    case LoggerLevel::Warn: return "warn";
    case LoggerLevel::Error: return "error";
    default: return "quiet";
  }
}
inline void set_logger_level(LoggerLevel level) { scn_set_log_level(static_cast<int>(level)); }
inline LoggerLevel get_logger_level() { return static_cast<LoggerLevel>(scn_get_log_level()); }
inline void set_logger(ILogger* logger) {
  detail::logger_slot() = logger;
  scn_set_log_callback(logger ? detail::log_trampoline : nullptr, nullptr);
}
inline ILogger* get_logger() { return detail::logger_slot(); }
inline void logger_output(const char* file, int line, LoggerLevel level, const char* fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  std::vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  scn_log(file, line, static_cast<int>(level), buf);
}

/** Sparse tensor handle of an engine: features [N, C], indices [N, 4] int32 (batch, i0, i1, i2) in the
    axis order of the grid, grid size, and the optional device-side row count. */
class SparseDTensor {
 public:
  virtual ~SparseDTensor() {}
  virtual Tensor& features() = 0;
  virtual Tensor& indices() = 0;
  virtual void set_grid_size(const std::vector<int>& grid_size) = 0;
  virtual std::vector<int> grid_size() const = 0;
  virtual int device() const = 0;
  virtual const char* name() const = 0;
  virtual void set_dds_num_of_points_pointer(uint32_t* pointer) = 0;
  virtual uint32_t* get_dds_num_of_points_pointer() = 0;
};

/** Inference engine.  input(0): features Float16 [N, C] and indices Int32 [N, 4] referenced from caller
    device memory, batch 1.  forward() only enqueues work on the stream. */
class Engine {
 public:
  virtual ~Engine() {}
  virtual void forward(void* stream = nullptr) = 0;
  virtual size_t num_input() const = 0;
  virtual SparseDTensor* input(unsigned int index) = 0;
  virtual size_t num_output() const = 0;
  virtual SparseDTensor* output(unsigned int index) = 0;
};

class ITensor {
 public:
  virtual ~ITensor() {}
  virtual const char* name() = 0;
};

class INode {
 public:
  virtual ~INode() {}
  virtual const char* name() = 0;
  virtual const char* optype() = 0;
  virtual ITensor* input(unsigned int index) = 0;
  virtual ITensor* output(unsigned int index) = 0;
  virtual unsigned int num_output() = 0;
  virtual unsigned int num_input() = 0;
};

class EngineBuilder {
 public:
  virtual ~EngineBuilder() {}
  virtual ITensor* push_input(const char* name) = 0;
  virtual INode* push_add(const char* name, ITensor* a, ITensor* b, float a_dynamic_range, float b_dynamic_range,
                          const char* output_name, Precision precision, Precision output_precision,
                          uint32_t fixed_launch_points) = 0;
  virtual INode* push_relu(const char* name, ITensor* x, const char* output_name) = 0;
  virtual INode* push_dense(const char* name, ITensor* x, const char* format, const char* output_name,
                            const std::vector<int>& input_spatial_shape, const std::vector<int>& output_shape,
                            TensorLayout output_layout = TensorLayout::NCHW, float input_dynamic_range = 0.0f,
                            uint32_t input_bound = 0) = 0;
  virtual INode* push_reshape(const char* name, ITensor* x, const std::vector<int64_t>& shape, const char* output_name) = 0;
  virtual INode* push_transpose(const char* name, ITensor* x, const std::vector<int64_t>& dims, const char* output_name) = 0;
  virtual INode* push_sparse_conv(const char* name, ITensor* x, const std::vector<unsigned short>& weight,
                                  const std::vector<int>& weight_shape, const std::vector<float>& weight_dynamic_ranges,
                                  const std::vector<unsigned short>& bias, const std::vector<int>& bias_shape,
                                  const char* activation, const std::vector<int>& kernel_size,
                                  const std::vector<int>& stride, const std::vector<int>& padding,
                                  const std::vector<int>& dilation, float input_dynamic_range, bool submanifold,
                                  uint32_t max_output_points, uint32_t fixed_launch_points, const char* rulebook,
                                  Precision precision, Precision output_precision, const char* output_name,
                                  bool inverse) = 0;
  virtual void push_output(ITensor* value) = 0;
  virtual std::shared_ptr<Engine> build(Precision precision, bool sortmask = false, bool enable_blackwell = false,
                                        bool with_auxiliary_stream = false, void* stream = nullptr) = 0;
};

// ------------------------------------------------------------------------------------------------
// implementation over the C ABI
// ------------------------------------------------------------------------------------------------
namespace detail {

class SparseHandle : public SparseDTensor {
 public:
  SparseHandle(scn_engine* e, int index, bool is_input) : e_(e), index_(index), is_input_(is_input) {}
  Tensor& features() override { return features_; }
  Tensor& indices() override { return indices_; }
  void set_grid_size(const std::vector<int>& g) override {
    grid_ = g;
    if (is_input_ && g.size() == 3) {
      const int g3[3] = {g[0], g[1], g[2]};
      (void)scn_engine_prepare(e_, g3);  // allocate now: forward() must be capturable from its first call
    }
  }
  std::vector<int> grid_size() const override { return grid_; }
  int device() const override {
    int d = 0;
    (void)hipGetDevice(&d);
    return d;
  }
  const char* name() const override { return name_.c_str(); }
  void set_dds_num_of_points_pointer(uint32_t* p) override { dds_ = p; }
  uint32_t* get_dds_num_of_points_pointer() override { return dds_; }

  // pushes the caller's current references into the engine (inputs) ...
  bool bind_input() {
    if (grid_.size() != 3) return false;
    const int g3[3] = {grid_[0], grid_[1], grid_[2]};
    const uint32_t n = features_.shape.empty() ? 0u : (uint32_t)features_.size(0);
    const uint32_t c = features_.shape.size() > 1 ? (uint32_t)features_.size(1) : 0u;
    if (scn_engine_set_input(e_, index_, features_.ptr(), n, c, indices_.ptr<int32_t>(), g3) != SCN_OK) return false;
    return scn_engine_set_num_points_device_ptr(e_, index_, dds_) == SCN_OK;
  }
  // ... and refreshes the views of an output
  void refresh_output() {
    scn_tensor_view v;
    if (scn_engine_output(e_, index_, &v) != SCN_OK) return;
    name_ = v.name ? v.name : "";
    std::vector<int64_t> shape(v.shape, v.shape + v.ndim);
    features_.reference(v.features_dev, shape, static_cast<DataType>(v.dtype), true);
    if (v.indices_dev) {
      indices_.reference(const_cast<int32_t*>(v.indices_dev), {v.shape[0], 4}, DataType::Int32, true);
      grid_ = {v.grid_size[0], v.grid_size[1], v.grid_size[2]};
      dds_ = const_cast<uint32_t*>(v.num_dev);
    }
  }
  void set_name(const std::string& n) { name_ = n; }

 private:
  scn_engine* e_;
  int index_;
  bool is_input_;
  Tensor features_, indices_;
  std::vector<int> grid_;
  uint32_t* dds_ = nullptr;
  std::string name_;
};

class EngineImpl : public Engine {
 public:
  explicit EngineImpl(scn_engine* e) : e_(e) {
    for (int i = 0; i < scn_engine_num_input(e_); ++i) inputs_.emplace_back(new SparseHandle(e_, i, true));
    for (int i = 0; i < scn_engine_num_output(e_); ++i) {
      outputs_.emplace_back(new SparseHandle(e_, i, false));
      outputs_.back()->refresh_output();
    }
  }
  ~EngineImpl() override { scn_engine_destroy(e_); }
  void forward(void* stream = nullptr) override {
    for (auto& in : inputs_)
      if (!in->bind_input()) {
        logger_output(__FILE__, __LINE__, LoggerLevel::Error, "forward: input is not fully specified (%s)", scn_last_error());
        return;
      }
    if (scn_engine_forward(e_, stream) != SCN_OK) {
      logger_output(__FILE__, __LINE__, LoggerLevel::Error, "forward failed: %s", scn_last_error());
      return;
    }
    for (auto& out : outputs_) out->refresh_output();
  }
  size_t num_input() const override { return inputs_.size(); }
  SparseDTensor* input(unsigned int index) override { return index < inputs_.size() ? inputs_[index].get() : nullptr; }
  size_t num_output() const override { return outputs_.size(); }
  SparseDTensor* output(unsigned int index) override { return index < outputs_.size() ? outputs_[index].get() : nullptr; }
  scn_engine* handle() const { return e_; }

 private:
  scn_engine* e_;
  std::vector<std::unique_ptr<SparseHandle>> inputs_, outputs_;
};

class TensorImpl : public ITensor {
 public:
  TensorImpl(int handle, std::string name) : handle_(handle), name_(std::move(name)) {}
  const char* name() override { return name_.c_str(); }
  int handle() const { return handle_; }

 private:
  int handle_;
  std::string name_;
};

class NodeImpl : public INode {
 public:
  NodeImpl(std::string name, std::string op, std::vector<ITensor*> in, ITensor* out)
      : name_(std::move(name)), op_(std::move(op)), in_(std::move(in)), out_(out) {}
  const char* name() override { return name_.c_str(); }
  const char* optype() override { return op_.c_str(); }
  ITensor* input(unsigned int i) override { return i < in_.size() ? in_[i] : nullptr; }
  ITensor* output(unsigned int i) override { return i == 0 ? out_ : nullptr; }
  unsigned int num_output() override { return 1; }
  unsigned int num_input() override { return (unsigned int)in_.size(); }

 private:
  std::string name_, op_;
  std::vector<ITensor*> in_;
  ITensor* out_;
};

class BuilderImpl : public EngineBuilder {
 public:
  BuilderImpl() : b_(scn_builder_create()) {}
  ~BuilderImpl() override { scn_builder_destroy(b_); }

  ITensor* push_input(const char* name) override { return wrap(scn_builder_push_input(b_, name), name); }
  INode* push_add(const char* name, ITensor* a, ITensor* b, float a_dynamic_range, float b_dynamic_range,
                  const char* output_name, Precision precision, Precision output_precision,
                  uint32_t fixed_launch_points) override {
    if (!a || !b) return nullptr;
    const int out = scn_builder_push_add(b_, name, h(a), h(b), a_dynamic_range, b_dynamic_range, output_name,
                                         (int)precision, (int)output_precision, fixed_launch_points);
    return node(name, "Add", {a, b}, out, output_name);
  }
  INode* push_relu(const char* name, ITensor* x, const char* output_name) override {
    if (!x) return nullptr;
    return node(name, "Relu", {x}, scn_builder_push_relu(b_, name, h(x), output_name), output_name);
  }
  INode* push_dense(const char* name, ITensor* x, const char* format, const char* output_name,
                    const std::vector<int>& input_spatial_shape, const std::vector<int>& output_shape,
                    TensorLayout output_layout, float input_dynamic_range, uint32_t input_bound) override {
    if (!x || input_spatial_shape.size() != 3) return nullptr;
    const int out = scn_builder_push_dense(b_, name, h(x), format, output_name, input_spatial_shape.data(),
                                           output_shape.data(), (int)output_shape.size(), (int)output_layout,
                                           input_dynamic_range, input_bound);
    return node(name, "ScatterDense", {x}, out, output_name);
  }
  INode* push_reshape(const char* name, ITensor* x, const std::vector<int64_t>& shape, const char* output_name) override {
    if (!x) return nullptr;
    return node(name, "Reshape", {x}, scn_builder_push_reshape(b_, name, h(x), shape.data(), (int)shape.size(), output_name),
                output_name);
  }
  INode* push_transpose(const char* name, ITensor* x, const std::vector<int64_t>& dims, const char* output_name) override {
    if (!x) return nullptr;
    return node(name, "Transpose", {x}, scn_builder_push_transpose(b_, name, h(x), dims.data(), (int)dims.size(), output_name),
                output_name);
  }
  INode* push_sparse_conv(const char* name, ITensor* x, const std::vector<unsigned short>& weight,
                          const std::vector<int>& weight_shape, const std::vector<float>& weight_dynamic_ranges,
                          const std::vector<unsigned short>& bias, const std::vector<int>& bias_shape,
                          const char* activation, const std::vector<int>& kernel_size, const std::vector<int>& stride,
                          const std::vector<int>& padding, const std::vector<int>& dilation, float input_dynamic_range,
                          bool submanifold, uint32_t max_output_points, uint32_t fixed_launch_points,
                          const char* rulebook, Precision precision, Precision output_precision,
                          const char* output_name, bool inverse) override {
    (void)bias_shape;
    if (!x || weight_shape.size() != 5 || kernel_size.size() != 3) return nullptr;
    const int out = scn_builder_push_sparse_conv(
        b_, name, h(x), weight.data(), weight_shape.data(), weight_dynamic_ranges.empty() ? nullptr : weight_dynamic_ranges.data(),
        (int)weight_dynamic_ranges.size(), bias.empty() ? nullptr : bias.data(), (int)bias.size(), activation,
        kernel_size.data(), stride.size() == 3 ? stride.data() : nullptr, padding.size() == 3 ? padding.data() : nullptr,
        dilation.size() == 3 ? dilation.data() : nullptr, input_dynamic_range, submanifold ? 1 : 0, max_output_points,
        fixed_launch_points, rulebook, (int)precision, (int)output_precision, output_name, inverse ? 1 : 0);
    return node(name, "SparseConvolution", {x}, out, output_name);
  }
  void push_output(ITensor* value) override {
    if (value) (void)scn_builder_push_output(b_, h(value));
  }
  std::shared_ptr<Engine> build(Precision precision, bool sortmask, bool enable_blackwell, bool with_auxiliary_stream,
                                void* stream) override {
    (void)enable_blackwell;
    const unsigned flags = (sortmask ? SCN_BUILD_SORTMASK : 0u) | (with_auxiliary_stream ? SCN_BUILD_AUX_STREAM : 0u);
    scn_engine* e = scn_builder_build(b_, (int)precision, flags, stream);
    if (!e) return nullptr;
    return std::shared_ptr<Engine>(new EngineImpl(e));
  }

 private:
  static int h(ITensor* t) { return static_cast<TensorImpl*>(t)->handle(); }
  ITensor* wrap(int handle, const char* name) {
    if (handle < 0) return nullptr;
    tensors_.emplace_back(new TensorImpl(handle, name ? name : ""));
    return tensors_.back().get();
  }
  INode* node(const char* name, const char* op, std::vector<ITensor*> in, int out_handle, const char* out_name) {
    ITensor* out = wrap(out_handle, out_name);
    if (!out) return nullptr;
    nodes_.emplace_back(new NodeImpl(name ? name : "", op, std::move(in), out));
    return nodes_.back().get();
  }
  scn_builder* b_;
  std::vector<std::unique_ptr<TensorImpl>> tensors_;
  std::vector<std::unique_ptr<NodeImpl>> nodes_;
};

}  // namespace detail

/** To build an engine node by node. */
inline std::shared_ptr<EngineBuilder> create_engine_builder() { return std::make_shared<detail::BuilderImpl>(); }

}  // namespace spconv

#endif  // SCN_SPCONV_ENGINE_HPP
