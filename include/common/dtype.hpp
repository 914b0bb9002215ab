// Plain value types of the lidar pipeline's public headers (nvtype::Int3, Float3, half), as the reference
// declares them in CUDA-BEVFusion/src/common/dtype.hpp:27-68: callers pass these by value.
#ifndef SCN_COMMON_DTYPE_HPP
#define SCN_COMMON_DTYPE_HPP

namespace nvtype {

struct Int2 {
  int x = 0, y = 0;
  Int2() = default;
  Int2(int x_, int y_ = 0) : x(x_), y(y_) {}
};
struct Int3 {
  int x = 0, y = 0, z = 0;
  Int3() = default;
  Int3(int x_, int y_ = 0, int z_ = 0) : x(x_), y(y_), z(z_) {}
};
struct Float2 {
  float x = 0, y = 0;
  Float2() = default;
  Float2(float x_, float y_ = 0) : x(x_), y(y_) {}
};
struct Float3 {
  float x = 0, y = 0, z = 0;
  Float3() = default;
  Float3(float x_, float y_ = 0, float z_ = 0) : x(x_), y(y_), z(z_) {}
};
struct Float4 {
  float x = 0, y = 0, z = 0, w = 0;
  Float4() = default;
  Float4(float x_, float y_ = 0, float z_ = 0, float w_ = 0) : x(x_), y(y_), z(z_), w(w_) {}
};

// names the 16-bit float type in signatures without pulling in a device header
struct half {
  unsigned short __x;
};

}  // namespace nvtype

#endif  // SCN_COMMON_DTYPE_HPP
