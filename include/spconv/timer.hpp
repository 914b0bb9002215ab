// spconv::EventTimer on HIP events (reference: libspconv/include/spconv/timer.hpp:22-51).
#ifndef SCN_SPCONV_TIMER_HPP
#define SCN_SPCONV_TIMER_HPP

#include <hip/hip_runtime.h>

#include <cstdio>

#include "check.hpp"

namespace spconv {

class EventTimer {
 public:
  EventTimer() {
    check_hip_api(hipEventCreate(&begin_));
    check_hip_api(hipEventCreate(&end_));
  }
  virtual ~EventTimer() {
    check_hip_api(hipEventDestroy(begin_));
    check_hip_api(hipEventDestroy(end_));
  }
  void start(void* stream) {
    stream_ = (hipStream_t)stream;
    check_hip_api(hipEventRecord(begin_, stream_));
  }
  // elapsed milliseconds since start(); synchronises on the end event
  float stop(const char* prefix, bool print = true) {
    float ms = 0;
    check_hip_api(hipEventRecord(end_, stream_));
    check_hip_api(hipEventSynchronize(end_));
    check_hip_api(hipEventElapsedTime(&ms, begin_, end_));
    if (print) std::printf("[Times %s]: %.3f ms\n", prefix ? prefix : "", ms);
    return ms;
  }

 private:
  hipStream_t stream_ = nullptr;
  hipEvent_t begin_ = nullptr, end_ = nullptr;
};

}  // namespace spconv

#endif  // SCN_SPCONV_TIMER_HPP
