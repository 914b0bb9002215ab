// spconv::Tensor / TensorData / DataType for the MI355X SCN engine (header-only, HIP runtime).
//
// Same names and semantics as the reference's public tensor header
// (libraries/3DSparseConvolution/libspconv/include/spconv/tensor.hpp:28-124): a shape plus a shared
// buffer that either owns its memory or aliases caller memory (`reference`).  File I/O uses the
// `.tensor` format of libraries/3DSparseConvolution/tool/tensor.py:24-69.
// `void* stream` arguments are hipStream_t.
#ifndef SCN_SPCONV_TENSOR_HPP
#define SCN_SPCONV_TENSOR_HPP

#include <hip/hip_runtime.h>

#include "../scn_c_api.h"

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace spconv {

enum class DataType : int { None = 0, Int32 = 1, Float16 = 2, Float32 = 3, Int64 = 4, UInt64 = 5, UInt32 = 6, Int8 = 7, UInt8 = 8 };

inline size_t dtype_bytes(DataType dtype) {
  switch (dtype) {
    case DataType::Int32: case DataType::Float32: case DataType::UInt32: return 4;
    case DataType::Float16: return 2;
    case DataType::Int64: case DataType::UInt64: return 8;
    case DataType::Int8: case DataType::UInt8: return 1;
    default: return 0;
  }
}

inline const char* dtype_string(DataType dtype) {
  static const char* names[] = {"None", "Int32", "Float16", "Float32", "Int64", "UInt64", "UInt32", "Int8", "UInt8"};
  const int i = static_cast<int>(dtype);
  return (i >= 0 && i <= 8) ? names[i] : "Unknown";
}

inline float native_half2float(const unsigned short h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  const uint32_t exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu, bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = 0;
      while (!(man & 0x400u)) { man <<= 1; ++e; }
      bits = sign | ((uint32_t)(113 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

inline std::vector<int64_t> toshape(const std::vector<int>& ishape) { return std::vector<int64_t>(ishape.begin(), ishape.end()); }
inline std::vector<int> toshape(const std::vector<int64_t>& ishape) { return std::vector<int>(ishape.begin(), ishape.end()); }

// Note: this is a thread unsafe function (one static buffer), like the reference's.
template <typename T>
inline const char* format_shape(const std::vector<T>& shape, bool space = true) {
  static char buf[256];
  size_t pos = 0;
  buf[0] = 0;
  for (size_t i = 0; i < shape.size() && pos + 32 < sizeof(buf); ++i)
    pos += (size_t)std::snprintf(buf + pos, sizeof(buf) - pos, i + 1 < shape.size() ? (space ? "%lld x " : "%lldx") : "%lld",
                                 (long long)shape[i]);
  return buf;
}

struct TensorData {
  void* data = nullptr;
  DataType dtype = DataType::None;
  size_t bytes = 0;
  size_t capacity = 0;
  bool device = true;
  bool owner = false;

  bool empty() const { return data == nullptr; }
  void free() {
    if (owner && data) {
      if (device) (void)hipFree(data); else (void)hipHostFree(data);
    }
    data = nullptr;
    bytes = capacity = 0;
    owner = false;
  }
  void reference(void* ptr, size_t nbytes, DataType dt, bool on_device) {
    free();
    data = ptr; bytes = capacity = nbytes; dtype = dt; device = on_device; owner = false;
  }
  void rearrange_and_realloc(size_t nbytes, DataType dt, bool on_device) {
    if (!owner || capacity < nbytes || device != on_device) {
      free();
      if (nbytes) {
        if (on_device) (void)hipMalloc(&data, nbytes); else (void)hipHostMalloc(&data, nbytes, hipHostMallocDefault);
      }
      capacity = nbytes;
      owner = true;
    }
    bytes = nbytes; dtype = dt; device = on_device;
  }
  virtual ~TensorData() { free(); }
  static TensorData* reference_new(void* ptr, size_t nbytes, DataType dt, bool on_device) {
    auto* t = new TensorData();
    t->reference(ptr, nbytes, dt, on_device);
    return t;
  }
  static TensorData* create(size_t nbytes, DataType dt, bool on_device) {
    auto* t = new TensorData();
    t->rearrange_and_realloc(nbytes, dt, on_device);
    return t;
  }
};

struct Tensor {
  std::vector<int64_t> shape;
  std::shared_ptr<TensorData> data;
  size_t numel = 0;
  size_t ndim = 0;

  template <typename T> T* ptr() const { return data ? (T*)data->data : nullptr; }
  void* ptr() const { return data ? data->data : nullptr; }
  template <typename T> T* begin() const { return ptr<T>(); }
  template <typename T> T* end() const { return data ? (T*)data->data + numel : nullptr; }

  int64_t size(int index) const { return shape[index]; }
  size_t bytes() const { return data ? data->bytes : 0; }
  bool empty() const { return data == nullptr || data->empty(); }
  DataType dtype() const { return data ? data->dtype : DataType::None; }
  bool device() const { return data ? data->device : false; }

  Tensor() = default;
  Tensor(std::vector<int64_t> shp, DataType dt, bool on_device = true) { create_(shp, dt, on_device); }

  void set_shape_(const std::vector<int64_t>& shp) {
    shape = shp;
    ndim = shp.size();
    numel = shp.empty() ? 0 : 1;
    for (auto v : shp) numel *= (size_t)v;
  }
  void reference(void* ptr_, std::vector<int64_t> shp, DataType dt, bool on_device = true) {
    set_shape_(shp);
    if (!data) data.reset(new TensorData());
    data->reference(ptr_, numel * dtype_bytes(dt), dt, on_device);
  }
  void create_(const std::vector<int64_t>& shp, DataType dt, bool on_device = true) {
    set_shape_(shp);
    if (!data) data.reset(new TensorData());
    data->rearrange_and_realloc(numel * dtype_bytes(dt), dt, on_device);
  }
  static Tensor create(std::vector<int64_t> shp, DataType dt, bool on_device = true) { return Tensor(shp, dt, on_device); }
  static Tensor create(std::vector<int32_t> shp, DataType dt, bool on_device = true) {
    return Tensor(std::vector<int64_t>(shp.begin(), shp.end()), dt, on_device);
  }
  static Tensor from_data_reference(void* ptr_, std::vector<int64_t> shp, DataType dt, bool on_device = true) {
    Tensor t;
    t.reference(ptr_, shp, dt, on_device);
    return t;
  }
  // copies host data into a new tensor (on the device when on_device is set)
  static Tensor from_data(void* ptr_, std::vector<int64_t> shp, DataType dt, bool on_device = true, void* stream = nullptr) {
    Tensor t(shp, dt, on_device);
    if (t.bytes()) {
      (void)hipMemcpyAsync(t.ptr(), ptr_, t.bytes(), on_device ? hipMemcpyHostToDevice : hipMemcpyHostToHost, (hipStream_t)stream);
      (void)hipStreamSynchronize((hipStream_t)stream);
    }
    return t;
  }
  static Tensor from_data(void* ptr_, std::vector<int32_t> shp, DataType dt, bool on_device = true, void* stream = nullptr) {
    return from_data(ptr_, std::vector<int64_t>(shp.begin(), shp.end()), dt, on_device, stream);
  }

  Tensor clone(void* stream = nullptr) const {
    Tensor t(shape, dtype(), device());
    if (bytes()) {
      (void)hipMemcpyAsync(t.ptr(), ptr(), bytes(), device() ? hipMemcpyDeviceToDevice : hipMemcpyHostToHost, (hipStream_t)stream);
      (void)hipStreamSynchronize((hipStream_t)stream);
    }
    return t;
  }
  Tensor to_device(void* stream = nullptr) const {
    if (device()) return *this;
    Tensor t(shape, dtype(), true);
    if (bytes()) {
      (void)hipMemcpyAsync(t.ptr(), ptr(), bytes(), hipMemcpyHostToDevice, (hipStream_t)stream);
      (void)hipStreamSynchronize((hipStream_t)stream);
    }
    return t;
  }
  Tensor to_host(void* stream = nullptr) const {
    if (!device()) return *this;
    Tensor t(shape, dtype(), false);
    if (bytes()) {
      (void)hipMemcpyAsync(t.ptr(), ptr(), bytes(), hipMemcpyDeviceToHost, (hipStream_t)stream);
      (void)hipStreamSynchronize((hipStream_t)stream);
    }
    return t;
  }
  void to_device_(void* stream = nullptr) { *this = to_device(stream); }
  void to_host_(void* stream = nullptr) { *this = to_host(stream); }
  void memset(unsigned char value = 0, void* stream = nullptr) {
    if (!bytes()) return;
    // device memory is filled by a kernel of the library: a memset node must not end up in a captured graph
    if (device()) (void)scn_memset_async(ptr(), value, bytes(), stream); else std::memset(ptr(), value, bytes());
  }
  // fills an Int32 tensor with 0..num-1
  void arange(size_t num, void* stream = nullptr) {
    std::vector<int32_t> v(num);
    for (size_t i = 0; i < num; ++i) v[i] = (int32_t)i;
    create_({(int64_t)num}, DataType::Int32, device());
    if (device()) {
      (void)hipMemcpyAsync(ptr(), v.data(), num * 4, hipMemcpyHostToDevice, (hipStream_t)stream);
      (void)hipStreamSynchronize((hipStream_t)stream);
    } else {
      std::memcpy(ptr(), v.data(), num * 4);
    }
  }
  float absmax(void* stream = nullptr) const {
    Tensor h = to_host(stream);
    float m = 0.f;
    for (size_t i = 0; i < numel; ++i) {
      float v = 0.f;
      switch (dtype()) {
        case DataType::Float16: v = native_half2float(h.ptr<unsigned short>()[i]); break;
        case DataType::Float32: v = h.ptr<float>()[i]; break;
        case DataType::Int32: v = (float)h.ptr<int32_t>()[i]; break;
        case DataType::Int8: v = (float)h.ptr<int8_t>()[i]; break;
        default: break;
      }
      m = std::fmax(m, std::fabs(v));
    }
    return m;
  }
  Tensor to_half(void* stream = nullptr) const;  // Float32 -> Float16 (defined below)

  void print(const char* prefix = "Tensor", size_t offset = 0, size_t num_per_line = 10, size_t lines = 1, void* stream = nullptr) const {
    Tensor h = to_host(stream);
    std::printf("%s[%s] %s: ", prefix, dtype_string(dtype()), format_shape(shape));
    for (size_t l = 0; l < lines; ++l) {
      for (size_t j = 0; j < num_per_line; ++j) {
        const size_t i = offset + l * num_per_line + j;
        if (i >= numel) break;
        switch (dtype()) {
          case DataType::Float16: std::printf("%.5f ", native_half2float(h.ptr<unsigned short>()[i])); break;
          case DataType::Float32: std::printf("%.5f ", h.ptr<float>()[i]); break;
          case DataType::Int32: std::printf("%d ", h.ptr<int32_t>()[i]); break;
          case DataType::Int8: std::printf("%d ", (int)h.ptr<int8_t>()[i]); break;
          default: break;
        }
      }
      std::printf("\n");
    }
  }

  bool save(const char* file, void* stream = nullptr) const {
    Tensor h = to_host(stream);
    FILE* f = std::fopen(file, "wb");
    if (!f) return false;
    int32_t head[3] = {0x33ff1101, (int32_t)ndim, (int32_t)dtype()};
    bool ok = std::fwrite(head, 4, 3, f) == 3;
    for (auto d : shape) {
      int32_t v = (int32_t)d;
      ok = ok && std::fwrite(&v, 4, 1, f) == 1;
    }
    if (h.bytes()) ok = ok && std::fwrite(h.ptr(), 1, h.bytes(), f) == h.bytes();
    std::fclose(f);
    return ok;
  }
  static bool save(const Tensor& tensor, const char* file, void* stream = nullptr) { return tensor.save(file, stream); }
  static Tensor load(const char* file, bool on_device = true, void* stream = nullptr) {
    FILE* f = std::fopen(file, "rb");
    if (!f) return Tensor();
    int32_t head[3] = {0, 0, 0};
    if (std::fread(head, 4, 3, f) != 3 || head[0] != 0x33ff1101 || head[1] < 0 || head[1] > 16 || head[2] < 1 || head[2] > 8) {
      std::fclose(f);
      return Tensor();
    }
    std::vector<int64_t> shp(head[1]);
    for (auto& d : shp) {
      int32_t v = 0;
      if (std::fread(&v, 4, 1, f) != 1) { std::fclose(f); return Tensor(); }
      d = v;
    }
    Tensor h(shp, (DataType)head[2], false);
    const bool ok = h.bytes() == 0 || std::fread(h.ptr(), 1, h.bytes(), f) == h.bytes();
    std::fclose(f);
    if (!ok) return Tensor();
    return on_device ? h.to_device(stream) : h;
  }
  static Tensor load_from_raw(const char* file, std::vector<int64_t> shp, DataType dt, bool on_device = true, void* stream = nullptr) {
    FILE* f = std::fopen(file, "rb");
    if (!f) return Tensor();
    Tensor h(shp, dt, false);
    const bool ok = h.bytes() == 0 || std::fread(h.ptr(), 1, h.bytes(), f) == h.bytes();
    std::fclose(f);
    if (!ok) return Tensor();
    return on_device ? h.to_device(stream) : h;
  }
};

inline Tensor Tensor::to_half(void* stream) const {
  if (dtype() != DataType::Float32) return *this;
  Tensor h = to_host(stream);
  Tensor o(shape, DataType::Float16, false);
  for (size_t i = 0; i < numel; ++i) {
    // round to nearest even via the float bit pattern
    uint32_t x;
    const float v = h.ptr<float>()[i];
    std::memcpy(&x, &v, 4);
    const uint32_t sign = (x >> 16) & 0x8000u, ax = x & 0x7fffffffu;
    uint16_t r;
    if (ax >= 0x7f800000u) r = (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0));
    else if (ax >= 0x477ff000u) r = (uint16_t)(sign | 0x7c00u);
    else if (ax < 0x33000001u) r = (uint16_t)sign;
    else {
      const int e = (int)(ax >> 23) - 127;
      const uint32_t m = (ax & 0x7fffffu) | 0x800000u;
      if (e < -14) {
        const int shift = -1 - e;
        uint32_t q = m >> shift;
        const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1))) ++q;
        r = (uint16_t)(sign | q);
      } else {
        uint32_t out = ((uint32_t)(e + 15) << 10) + ((m >> 13) & 0x3ffu);
        const uint32_t rem = m & 0x1fffu;
        if (rem > 0x1000u || (rem == 0x1000u && ((m >> 13) & 1))) ++out;
        r = (uint16_t)(sign | out);
      }
    }
    o.ptr<unsigned short>()[i] = r;
  }
  return device() ? o.to_device(stream) : o;
}

}  // namespace spconv

#endif  // SCN_SPCONV_TENSOR_HPP
