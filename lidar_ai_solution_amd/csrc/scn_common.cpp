// Logging, error state and fp16 host conversions of libscn_hip.
#include "scn_common.hpp"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace scn {

static int g_level = kWarn;
static scn_log_callback g_cb = nullptr;
static void* g_cb_user = nullptr;
static thread_local std::string g_last_error;
static int g_debug_sync = -1;   // -1: not decided yet (SCN_DEBUG_SYNC in the environment decides on first use)

bool debug_sync_enabled() {
  if (g_debug_sync < 0) {
    const char* e = getenv("SCN_DEBUG_SYNC");
    g_debug_sync = (e && *e && strcmp(e, "0") != 0) ? 1 : 0;
  }
  return g_debug_sync != 0;
}

int debug_sync_check(hipStream_t stream, const char* what) {
  hipError_t err = hipStreamSynchronize(stream);
  if (err == hipSuccess) err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("debug sync: %s failed: %s", what, hipGetErrorString(err));
    return SCN_ERR_HIP;
  }
  return SCN_OK;
}

static const char* level_name(int level) {
  switch (level) {
    case kVerb: return "verb";
    case kWarn: return "warn";
    case kError: return "error";
    default: return "quiet";
  }
}

static void emit(const char* file, int line, int level, const char* msg) {
  if (level < g_level) return;
  if (g_cb) {
    g_cb(msg, level, file, line, g_cb_user);
    return;
  }
  const char* base = strrchr(file, '/');
  fprintf(level >= kError ? stderr : stdout, "[%s][%s:%d]: %s\n", level_name(level), base ? base + 1 : file, line, msg);
}

void log_message(const char* file, int line, int level, const char* fmt, ...) {
  if (level < g_level) return;
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  emit(file, line, level, buf);
}

std::atomic<size_t>& device_bytes_counter() {
  static std::atomic<size_t> bytes{0};
  return bytes;
}

void set_error(const char* fmt, ...) {
  char buf[2048];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  emit("libscn_hip", 0, kError, buf);
}

float half_bits_to_float(uint16_t h) {
  const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  int exp = (h >> 10) & 0x1f;
  uint32_t man = h & 0x3ffu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int e = 0;
      while (!(man & 0x400u)) {
        man <<= 1;
        e++;
      }
      man &= 0x3ffu;
      bits = sign | ((uint32_t)(127 - 14 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7f800000u | (man << 13);
  } else {
    bits = sign | ((uint32_t)(exp + 112) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

uint16_t float_to_half_bits(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0));
  if (ax >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);
  if (ax < 0x33000001u) return (uint16_t)sign;
  const int e = (int)(ax >> 23) - 127;
  const uint32_t m = (ax & 0x7fffffu) | 0x800000u;
  if (e < -14) {
    const int shift = (-14 - e) + 13;
    uint32_t q = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    return (uint16_t)(sign | q);
  }
  uint32_t q = m >> 13;
  const uint32_t rem = m & 0x1fffu;
  uint32_t out = ((uint32_t)(e + 15) << 10) + (q & 0x3ffu);
  if (rem > 0x1000u || (rem == 0x1000u && (q & 1))) out++;
  return (uint16_t)(sign | out);
}

}  // namespace scn

extern "C" {
int scn_version(void) { return 10000; }
size_t scn_device_bytes_in_use(void) { return scn::device_bytes_counter().load(); }
const char* scn_last_error(void) { return scn::g_last_error.c_str(); }
void scn_set_log_level(int level) { scn::g_level = level; }
int scn_get_log_level(void) { return scn::g_level; }
void scn_set_debug_sync(int enabled) { scn::g_debug_sync = enabled ? 1 : 0; }
int scn_get_debug_sync(void) { return scn::debug_sync_enabled() ? 1 : 0; }
void scn_set_log_callback(scn_log_callback cb, void* user) {
  scn::g_cb = cb;
  scn::g_cb_user = user;
}
void scn_log(const char* file, int line, int level, const char* message) {
  scn::log_message(file ? file : "", line, level, "%s", message ? message : "");
}
}
