// Device memory that is only held while other allocations are made.
//
// Where the state tensors of a search lie in the card's memory changes how fast the iteration
// kernel streams them: 4096 three-raise river roots, same binary, same bytes: 11.1 ms per
// iteration with the tensors allocated one after another by a fresh process, 10.5 ms when each
// of them was allocated while a block of 8 GiB or more, allocated just before it, was still held
// (the block can be given back right after).  The effect follows the physical placement, not the
// virtual addresses (reserving address space alone, or aligning the tensors' addresses to 1 GiB,
// changes nothing), and a flat stream does not show it.  These two calls are the block: plain
// hipMalloc / hipFree, kept apart from any caching allocator the caller uses for its tensors.
#pragma once
#include "common.h"

extern "C" {

int p2hip_device_reserve(int64_t bytes, void** out) {
  if (!out) return P2_EINVAL;
  *out = nullptr;
  if (bytes <= 0) return P2_EINVAL;
  const hipError_t e = hipMalloc(out, (size_t)bytes);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // an allocation that does not fit is an answer, not a sticky error
    *out = nullptr;
    return (int)e;
  }
  return 0;
}

int p2hip_device_release(void* ptr) {
  if (!ptr) return 0;
  return (int)hipFree(ptr);
}

}  // extern "C"
