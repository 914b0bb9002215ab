// The older single-call engine interface (the one CUDA-CenterPoint is written against:
// CUDA-CenterPoint/3rdparty/libspconv/include/spconv/engine.hpp:36-128, used by
// CUDA-CenterPoint/src/centerpoint.cpp:136-150) over the C ABI of libscn_hip.so.  Same namespace, class and
// method names and argument meaning, so a caller of that interface only changes its include path
// (-I<this repository>/include/legacy) and links libscn_hip.so + the HIP runtime.
//
// reconfigure() re-reads the model file with the precision overrides and the calibrated ranges collected so
// far (the engine is planned once per build).  set_int8_calibration(true) switches to an fp16 engine that keeps
// every tensor; each forward then records the largest magnitude of every tensor; set_int8_calibration(false)
// + reconfigure() return to the requested precision with those ranges in place of the model's.
#ifndef SCN_LEGACY_SPCONV_ENGINE_HPP
#define SCN_LEGACY_SPCONV_ENGINE_HPP

#include <cstdio>
#include <memory>
#include <string>
#include <vector>

#include "scn_c_api.h"

namespace spconv {

enum class DType : int { None = 0, Int32 = 1, Float16 = 2 };
enum class Precision : int { None = 0, Float16 = 1, Int8 = 2 };

class DTensor {
 public:
  virtual ~DTensor() {}
  virtual std::vector<int64_t> features_shape() const = 0;
  virtual DType features_dtype() const = 0;
  virtual void* features_data() = 0;
  virtual std::vector<int64_t> indices_shape() const = 0;
  virtual DType indices_dtype() const = 0;
  virtual void* indices_data() = 0;
  virtual std::vector<int> grid_size() const = 0;
  virtual int device() const = 0;
};

class Engine {
 public:
  virtual ~Engine() {}
  // features: [n, channels] fp16 on the device, indices: [n, 4] int32 on the device, batch 1.  The returned
  // tensor is owned by the engine and describes output 0 after this forward (enqueued on `stream`).
  virtual DTensor* forward(const std::vector<int64_t>& features_shape, DType features_dtype, void* features_data,
                           const std::vector<int64_t>& indices_shape, DType indices_dtype, void* indices_data,
                           int batch, std::vector<int> grid_size, void* stream = nullptr) = 0;
  virtual void reconfigure() = 0;
  virtual void set_int8_calibration(bool enable) = 0;
  virtual void set_node_precision_byname(const char* name, Precision compute_precision, Precision output_precision) = 0;
  virtual void set_node_precision_byoptype(const char* optype, Precision compute_precision,
                                           Precision output_precision) = 0;
};

namespace detail {

class OutputView : public DTensor {
 public:
  void assign(const scn_tensor_view& v) { v_ = v; }
  std::vector<int64_t> features_shape() const override {
    return std::vector<int64_t>(v_.shape, v_.shape + v_.ndim);
  }
  DType features_dtype() const override { return v_.dtype == SCN_DTYPE_FP16 ? DType::Float16 : DType::None; }
  void* features_data() override { return v_.features_dev; }
  std::vector<int64_t> indices_shape() const override {
    if (!v_.indices_dev) return {};
    return {v_.shape[0], 4};
  }
  DType indices_dtype() const override { return v_.indices_dev ? DType::Int32 : DType::None; }
  void* indices_data() override { return const_cast<int32_t*>(v_.indices_dev); }
  std::vector<int> grid_size() const override {
    return {v_.grid_size[0], v_.grid_size[1], v_.grid_size[2]};
  }
  int device() const override { return 0; }

 private:
  scn_tensor_view v_{};
};

class LegacyEngine : public Engine {
 public:
  LegacyEngine(const std::string& file, Precision precision) : file_(file), precision_(precision) { rebuild(); }
  ~LegacyEngine() override {
    if (e_) scn_engine_destroy(e_);
  }
  bool valid() const { return e_ != nullptr; }

  DTensor* forward(const std::vector<int64_t>& features_shape, DType features_dtype, void* features_data,
                   const std::vector<int64_t>& indices_shape, DType indices_dtype, void* indices_data, int batch,
                   std::vector<int> grid_size, void* stream = nullptr) override {
    if (!e_) return nullptr;
    if (features_shape.size() != 2 || indices_shape.size() != 2 || indices_shape[1] != 4 ||
        features_shape[0] != indices_shape[0] || features_dtype != DType::Float16 || indices_dtype != DType::Int32 ||
        batch != 1 || grid_size.size() != 3) {
      fprintf(stderr, "[scn] forward: expects fp16 features [n, c], int32 indices [n, 4], batch 1 and a 3-element grid\n");
      return nullptr;
    }
    if (scn_engine_set_input(e_, 0, features_data, (uint32_t)features_shape[0], (uint32_t)features_shape[1],
                             static_cast<const int32_t*>(indices_data), grid_size.data()) != SCN_OK ||
        scn_engine_forward(e_, stream) != SCN_OK) {
      fprintf(stderr, "[scn] forward failed: %s\n", scn_last_error());
      return nullptr;
    }
    if (calibrating_) record_ranges(stream);
    scn_tensor_view v;
    if (scn_engine_output(e_, 0, &v) != SCN_OK) return nullptr;
    out_.assign(v);
    return &out_;
  }

  void reconfigure() override { rebuild(); }

  void set_int8_calibration(bool enable) override {
    if (enable == calibrating_) return;
    calibrating_ = enable;
    if (enable) rebuild();   // fp16, every tensor kept; leaving the mode takes effect at reconfigure()
  }

  void set_node_precision_byname(const char* name, Precision compute_precision, Precision output_precision) override {
    add_override(name, 0, compute_precision, output_precision);
  }
  void set_node_precision_byoptype(const char* optype, Precision compute_precision,
                                   Precision output_precision) override {
    add_override(optype, 1, compute_precision, output_precision);
  }

 private:
  void add_override(const char* selector, int by_optype, Precision c, Precision o) {
    if (!selector) return;
    selectors_.emplace_back(selector);
    pending_.push_back({by_optype, (int)c, (int)o});
  }
  void record_ranges(void* stream) {
    std::vector<scn_tensor_amax> got(4096);
    const int n = scn_engine_collect_amax(e_, stream, got.data(), (int)got.size());
    for (int i = 0; i < n; ++i) {
      size_t j = 0;
      while (j < range_names_.size() && range_names_[j] != got[i].tensor) ++j;
      if (j == range_names_.size()) {
        range_names_.emplace_back(got[i].tensor);
        range_values_.push_back(0.f);
      }
      if (got[i].amax > range_values_[j]) range_values_[j] = got[i].amax;
    }
  }
  void rebuild() {
    std::vector<scn_precision_override> ov(pending_.size());
    for (size_t i = 0; i < pending_.size(); ++i)
      ov[i] = {selectors_[i].c_str(), pending_[i].by_optype, pending_[i].precision, pending_[i].output_precision};
    std::vector<scn_tensor_amax> rg(calibrating_ ? 0 : range_names_.size());
    for (size_t i = 0; i < rg.size(); ++i) rg[i] = {range_names_[i].c_str(), range_values_[i]};
    scn_load_options opt = {ov.empty() ? nullptr : ov.data(), (int)ov.size(), rg.empty() ? nullptr : rg.data(),
                            (int)rg.size()};
    scn_engine* fresh = scn_engine_create_from_onnx_ex(file_.c_str(), calibrating_ ? (int)Precision::Float16 : (int)precision_,
                                                       calibrating_ ? SCN_BUILD_KEEP_ALL : 0u, 10000u, &opt, nullptr);
    if (!fresh) {
      fprintf(stderr, "[scn] load_engine_from_onnx(%s) failed: %s\n", file_.c_str(), scn_last_error());
      return;  // keeps the previous engine, if any
    }
    if (e_) scn_engine_destroy(e_);
    e_ = fresh;
  }
  struct Pending {
    int by_optype, precision, output_precision;
  };
  std::string file_;
  Precision precision_;
  std::vector<std::string> selectors_;
  std::vector<Pending> pending_;
  std::vector<std::string> range_names_;
  std::vector<float> range_values_;
  bool calibrating_ = false;
  scn_engine* e_ = nullptr;
  OutputView out_;
};

}  // namespace detail

// With precision Float16 the per-node "precision" attributes of the model are ignored, as in the reference.
inline std::shared_ptr<Engine> load_engine_from_onnx(const std::string& onnx_file,
                                                     Precision precision = Precision::Float16) {
  auto e = std::make_shared<detail::LegacyEngine>(onnx_file, precision);
  if (!e->valid()) return nullptr;
  return e;
}

inline void set_verbose(bool enable) { scn_set_log_level(enable ? 0 : 1); }  // Verb or Warn
inline const char* get_precision_string(Precision precision) {
  switch (precision) {
    case Precision::Float16: return "Float16";
    case Precision::Int8: return "Int8";
    default: return "None";
  }
}

}  // namespace spconv

#endif  // SCN_LEGACY_SPCONV_ENGINE_HPP
