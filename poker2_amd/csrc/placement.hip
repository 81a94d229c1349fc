// Where the state tensors of a search lie in the card's memory.
//
// The iteration kernel writes about ten tensors at once, and the card's memory takes such a set of write
// streams about a quarter faster when the written arrays lie in two different thirds of its physical
// address space than when they all lie in one (a row-streaming probe, 12 rows read and 8 written per
// node from 20 arrays: 4.2 TB/s with all arrays in one third, 5.2-5.3 TB/s with the written ones split
// between two; moving only read arrays changes nothing; a third region adds 2 %.  4096 three-raise river
// roots: 11.0 ms per iteration against 9.9-10.0 ms).  The thirds are ~96 GiB each; virtual addresses,
// alignment and address translation play no part, and where an allocation lands physically is not visible
// to a process - but it can be MEASURED: p2hip_placement_probe times that probe with its arrays dealt
// alternately to two buffers, and two buffers in different thirds show by a time a fifth shorter than two
// halves of one buffer.  p2hip_device_reserve / _release hold memory (plain hipMalloc / hipFree, apart
// from any caching allocator) so that the next allocation lands elsewhere.
#pragma once
#include "common.h"

namespace p2 {

constexpr int PL_READ = 12, PL_WRITTEN = 8, PL_ARRAYS = PL_READ + PL_WRITTEN, PL_SLOTS = PL_ARRAYS / 2;
constexpr int PL_NODES_PER_WG = 12;
constexpr int64_t PL_MAX_ROWS = 12288;          // 65 MB per array, 1.3 GB per launch: well past the caches

struct PlacementArrays { float* p[PL_ARRAYS]; };

// A workgroup walks PL_NODES_PER_WG consecutive nodes; per node it reads row n of the first PL_READ arrays
// and writes row n of the others (a lane three float2 of the 663 of a row).  The LDS array only sets the
// occupancy to that of the iteration kernel, three workgroups per compute unit.
__global__ __launch_bounds__(256, 3) void placement_probe_kernel(PlacementArrays a, int64_t rows) {
  __shared__ float occupancy[13000];
  if (threadIdx.x == 9999) occupancy[0] = 1.f;
  const int64_t n0 = (int64_t)blockIdx.x * PL_NODES_PER_WG;
  for (int i = 0; i < PL_NODES_PER_WG; ++i) {
    const int64_t n = n0 + i;
    if (n >= rows) break;
    float2 v[PL_READ][3];
#pragma unroll
    for (int k = 0; k < PL_READ; ++k) {
      const float2* src = reinterpret_cast<const float2*>(a.p[k] + n * P2_H);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int idx = threadIdx.x + j * 256;
        v[k][j] = src[idx < P2_HPAIRS ? idx : 0];
      }
    }
    float2 acc[3] = {{0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}};
#pragma unroll
    for (int k = 0; k < PL_READ; ++k)
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        acc[j].x += v[k][j].x;
        acc[j].y += v[k][j].y;
      }
#pragma unroll
    for (int k = 0; k < PL_WRITTEN; ++k) {
      float2* dst = reinterpret_cast<float2*>(a.p[PL_READ + k] + n * P2_H);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int idx = threadIdx.x + j * 256;
        if (idx < P2_HPAIRS) dst[idx] = make_float2(acc[j].x + (float)k, acc[j].y);
      }
    }
  }
}

}  // namespace p2

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

int p2hip_placement_probe(void* a, void* b, int64_t bytes_each, int reps, float* ms_out, void* stream) {
  if (!a || !b || !ms_out || reps < 1 || reps > 64) return P2_EINVAL;
  if (!p2_aligned8(a) || !p2_aligned8(b)) return P2_EINVAL;
  const int64_t slot = bytes_each / p2::PL_SLOTS / 256 * 256;        // ten arrays spread over each buffer
  int64_t rows = slot / (int64_t)(P2_H * sizeof(float));
  if (rows > p2::PL_MAX_ROWS) rows = p2::PL_MAX_ROWS;
  if (rows < 256) return P2_EINVAL;                                    // too small to say anything
  p2::PlacementArrays arr;
  for (int k = 0; k < p2::PL_ARRAYS; ++k)
    arr.p[k] = reinterpret_cast<float*>(static_cast<char*>(k & 1 ? b : a) + (int64_t)(k >> 1) * slot);
  hipStream_t st = (hipStream_t)stream;
  hipEvent_t e0, e1;
  hipError_t e = hipEventCreate(&e0);
  if (e != hipSuccess) return (int)e;
  e = hipEventCreate(&e1);
  if (e != hipSuccess) {
    (void)hipEventDestroy(e0);
    return (int)e;
  }
  const dim3 grid((unsigned)((rows + p2::PL_NODES_PER_WG - 1) / p2::PL_NODES_PER_WG)), block(256);
  hipLaunchKernelGGL(p2::placement_probe_kernel, grid, block, 0, st, arr, rows);      // warm-up
  (void)hipEventRecord(e0, st);
  for (int r = 0; r < reps; ++r) hipLaunchKernelGGL(p2::placement_probe_kernel, grid, block, 0, st, arr, rows);
  (void)hipEventRecord(e1, st);
  e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (e != hipSuccess) return (int)e;
  e = hipGetLastError();
  if (e != hipSuccess) return (int)e;
  *ms_out = ms / (float)reps;
  return 0;
}

}  // extern "C"
