// Single translation unit of libp2hip.so: every kernel file is included here so
// the shared device tables exist once and one hipcc call builds the library.
#include "common.h"
#include "ranker.hip"
#include "unblocked.hip"
#include "showdown.hip"
#include "cfr_ops.hip"
#include "cfr_iter.hip"
#include "chance.hip"
#include "best_response.hip"
#include "tree.hip"
#include "datagen.hip"
#include "stream_probe.hip"
#include "placement.hip"

extern "C" {
// Library / ABI version, bumped whenever an exported signature changes.
int p2hip_abi_version(void) { return 5; }
// Number of visible HIP devices (0 when there is none); never throws.
int p2hip_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}
const char* p2hip_error_string(int code) { return hipGetErrorString((hipError_t)code); }
}
