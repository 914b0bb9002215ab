// Feeds the model loader (ONNX wire reader -> builder calls -> graph planning) truncated and damaged copies of a
// valid model.  Built with -fsanitize=address,undefined -fno-sanitize-recover=all against the engine's host code and
// the host-only stand-ins of the kernel side: any out-of-bounds read, overflow or leak ends the process.
//   loader_fuzz <model.onnx> <int8|fp16> <mutations> <seed> <graph_end>
// graph_end: offset of the first byte behind the model's graph field; shorter prefixes cut the graph (whose length is
// declared up front) and must be refused by the reader, longer ones only drop trailing model fields.
// Prints one summary line; exit code 0 = every case ended in a null engine with an error text or in an engine that
// could be destroyed, and every strict prefix of the model was refused before any allocation on a device.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>
#include <random>
#include <string>

#include "scn_c_api.h"

static bool g_alloc_seen = false;
static void on_log(const char* msg, int, const char*, int, void*) {
  if (strstr(msg, "hipMalloc") || strstr(msg, "hipMemset")) g_alloc_seen = true;
}

// 0: refused while reading / checking, 1: refused at a device allocation (the model got through every host check),
// 2: an engine was built
static int load(const std::string& bytes, int precision, unsigned flags) {
  g_alloc_seen = false;
  scn_engine* e = scn_engine_create_from_onnx_memory(bytes.data(), bytes.size(), precision, flags, 10000, nullptr, nullptr);
  if (e) {
    (void)scn_engine_num_output(e);
    scn_engine_destroy(e);
    return 2;
  }
  if (!*scn_last_error()) {
    fprintf(stderr, "null engine without an error text\n");
    exit(3);
  }
  return g_alloc_seen ? 1 : 0;
}

int main(int argc, char** argv) {
  if (argc < 6) return 2;
  std::ifstream fin(argv[1], std::ios::binary);
  const std::string model((std::istreambuf_iterator<char>(fin)), std::istreambuf_iterator<char>());
  const int precision = !strcmp(argv[2], "int8") ? SCN_PRECISION_INT8 : SCN_PRECISION_FP16;
  const int mutations = atoi(argv[3]);
  std::mt19937_64 rng((uint64_t)atoll(argv[4]));
  scn_set_log_callback(on_log, nullptr);
  scn_set_log_level(2);
  const int whole = load(model, precision, 0);
  if (whole == 0) {
    fprintf(stderr, "the undamaged model was refused: %s\n", scn_last_error());
    return 4;
  }
  // prefixes that cut the graph: every length near both ends (where the field headers and the small fields are),
  // every 13th in the bulk of the weights
  const size_t graph_end = (size_t)atoll(argv[5]);
  long prefixes = 0;
  for (size_t n = 0; n < graph_end && n < model.size(); n += (n < 8192 || n + 8192 > graph_end) ? 1 : 13) {
    if (load(model.substr(0, n), precision, 0) != 0) {
      fprintf(stderr, "a prefix of %zu of %zu bytes (graph ends at %zu) was accepted\n", n, model.size(), graph_end);
      return 5;
    }
    ++prefixes;
  }
  for (size_t n = graph_end; n < model.size(); ++n) (void)load(model.substr(0, n), precision, 0);
  // damaged copies: flipped bits, replaced bytes, varints blown up, a stretch removed or repeated; any outcome is
  // fine as long as it is reached without a sanitizer report
  long by_outcome[3] = {0, 0, 0};
  for (int m = 0; m < mutations; ++m) {
    std::string b = model;
    const int kind = (int)(rng() % 5);
    // half of the damage goes to the first and last 16 KB, where the nodes, their attributes and the graph's
    // inputs / outputs are; the rest anywhere (mostly weight bytes and the headers of the initializers)
    size_t at = (size_t)(rng() % b.size());
    if ((rng() & 1) && b.size() > 32768) at = (rng() & 1) ? at % 16384 : b.size() - 1 - at % 16384;
    if (kind == 0) b[at] = (char)(b[at] ^ (1u << (rng() % 8)));
    else if (kind == 1) b[at] = (char)(rng() & 0xFF);
    else if (kind == 2) for (size_t k = at; k < b.size() && k < at + 9; ++k) b[k] = (char)0xFF;   // an endless varint
    else if (kind == 3) b.erase(at, (size_t)(rng() % 64) + 1);
    else b.insert(at, b.substr(at, (size_t)(rng() % 64) + 1));
    const unsigned flags = (rng() & 1 ? SCN_BUILD_SORTMASK : 0u) | (rng() & 2 ? SCN_BUILD_KEEP_ALL : 0u);
    by_outcome[load(b, precision, flags)]++;
  }
  printf("loader fuzz: whole model -> %s; %ld prefixes refused; %d damaged copies: %ld refused by the reader or the "
         "checks, %ld got to the device allocation, %ld built\n",
         whole == 2 ? "engine" : "device allocation", prefixes, mutations, by_outcome[0], by_outcome[1], by_outcome[2]);
  return 0;
}
