// spconv::PinnedMemoryData / GPUData / GPUMemory<T> / GPUDataManager for the MI355X SCN engine (header-only).
//
// Same class and method names as the reference's public header
// (libraries/3DSparseConvolution/libspconv/include/spconv/memory.hpp:25-183), over the HIP runtime: growable
// buffers that remember their capacity, a typed view on a shared buffer, and a by-name registry of shared
// buffers whose input/output entries can be sized up front.  `stream` arguments are hipStream_t; nothing here
// aborts: failures go to the logger (check.hpp) and leave the object empty.
#ifndef SCN_SPCONV_MEMORY_HPP
#define SCN_SPCONV_MEMORY_HPP

#include <hip/hip_runtime.h>

#include <memory>
#include <string>
#include <unordered_map>

#include "check.hpp"

namespace spconv {

namespace detail {

struct DeviceAllocator {
  static bool allocate(void** p, size_t n) { return check_hip_api(hipMalloc(p, n)); }
  static void release(void* p) { check_hip_api(hipFree(p)); }
};
// pinned host memory is always allocated, never registered after the fact
struct PinnedAllocator {
  static bool allocate(void** p, size_t n) { return check_hip_api(hipHostMalloc(p, n, hipHostMallocDefault)); }
  static void release(void* p) { check_hip_api(hipHostFree(p)); }
};

// A buffer with a size in use (bytes) and an allocated size (capacity): growing re-allocates and loses the
// contents, shrinking only lowers the size in use.
template <typename Allocator>
class Block {
 public:
  Block() = default;
  explicit Block(const std::string& name) : name_(name) {}
  Block(const Block&) = delete;
  Block& operator=(const Block&) = delete;
  virtual ~Block() { free_memory(nullptr); }

  void* ptr() const { return ptr_; }
  size_t bytes() const { return bytes_; }
  bool empty() const { return ptr_ == nullptr; }

  void alloc_or_resize_to(size_t nbytes, hipStream_t stream) {
    if (nbytes > capacity_) {
      free_memory(stream);
      void* p = nullptr;
      if (!Allocator::allocate(&p, nbytes)) return;
      ptr_ = p;
      capacity_ = nbytes;
    }
    bytes_ = nbytes;
  }
  void alloc(size_t nbytes, hipStream_t stream) { alloc_or_resize_to(nbytes, stream); }
  // a new size in use inside the allocation; a larger one is an error that is logged and ignored
  void resize(size_t nbytes) {
    spconv_assertf(nbytes <= capacity_, "%s Failed to resize memory to %zu bytes. capacity = %zu", name_.c_str(), nbytes,
                   capacity_);
    if (nbytes <= capacity_) bytes_ = nbytes;
  }
  void free_memory(hipStream_t /*stream*/) {
    if (!ptr_) return;
    Allocator::release(ptr_);
    ptr_ = nullptr;
    bytes_ = capacity_ = 0;
  }

 private:
  void* ptr_ = nullptr;
  size_t bytes_ = 0, capacity_ = 0;
  std::string name_;
};

}  // namespace detail

class PinnedMemoryData : public detail::Block<detail::PinnedAllocator> {
 public:
  using Block::Block;
};

class GPUData : public detail::Block<detail::DeviceAllocator> {
 public:
  using Block::Block;
};

// Typed view of a (possibly shared) GPUData: sizes are in elements.
template <typename T>
class GPUMemory {
 public:
  virtual ~GPUMemory() = default;
  T* ptr() const { return data_ ? static_cast<T*>(data_->ptr()) : nullptr; }
  size_t size() const { return size_; }
  size_t bytes() const { return data_ ? data_->bytes() : 0; }
  bool empty() const { return !data_ || data_->empty(); }
  bool unset() const { return !data_; }
  void set_gpudata(std::shared_ptr<GPUData> data) { data_ = std::move(data); }

  void alloc_or_resize_to(size_t size, hipStream_t stream) {
    spconv_asserts(data_ != nullptr, "Failed to alloc or resize memory that because data is nullptr.");
    if (!data_) return;
    size_ = size;
    data_->alloc_or_resize_to(size * sizeof(T), stream);
  }
  void alloc(size_t size, hipStream_t stream) { alloc_or_resize_to(size, stream); }
  void resize(size_t size) {
    spconv_asserts(data_ != nullptr, "Failed to resize memory that because data is nullptr.");
    if (!data_) return;
    size_ = size;
    data_->resize(size * sizeof(T));
  }

 private:
  std::shared_ptr<GPUData> data_;
  size_t size_ = 0;
};

// Buffers by tensor id: the same id gives the same buffer, so tensors whose lifetimes do not overlap can be
// given one id and share storage.  Input/output tensors are allocated at max_bytes_for_io_tensor when it is
// non-zero, so that they never re-allocate later (a forward() under graph capture must not).
class GPUDataManager {
 public:
  explicit GPUDataManager(size_t max_bytes_for_io_tensor = 0) : io_bytes_(max_bytes_for_io_tensor) {}

  std::shared_ptr<GPUData> query_or_alloc(const std::string& tensor_id, bool is_iotensor = false, hipStream_t stream = nullptr) {
    if (tensor_id == "__no_reuse_policy_here__") return std::make_shared<GPUData>(tensor_id);  // private, unregistered
    auto it = table_.find(tensor_id);
    if (it != table_.end()) return it->second;
    auto made = std::make_shared<GPUData>(tensor_id);
    if (is_iotensor && io_bytes_ > 0) made->alloc(io_bytes_, stream);
    table_.emplace(tensor_id, made);
    return made;
  }

 private:
  size_t io_bytes_ = 0;
  std::unordered_map<std::string, std::shared_ptr<GPUData>> table_;
};

}  // namespace spconv

#endif  // SCN_SPCONV_MEMORY_HPP
