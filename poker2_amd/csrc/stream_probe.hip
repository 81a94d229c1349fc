// Measurement aid, not part of the search path: a structure-free element-wise stream over n_read input
// and n_write output arrays of `pairs` float2 each (array k starts k * pairs float2 after the base
// pointer).  One 8-byte access per lane and array, workgroups in address order: what HBM gives a kernel
// of that read / write mix when nothing else limits it.  bench.py reports it beside the iteration
// kernel's rate (12 vectors read and 17 written per node: 5 + 7 arrays are the same 41 % / 59 % mix).
#pragma once
#include "common.h"

namespace p2 {

constexpr int PROBE_BLOCK = 256;

template <int NR, int NW>
__global__ __launch_bounds__(PROBE_BLOCK) void stream_probe_kernel(const float2* __restrict__ in,
                                                                    float2* __restrict__ out, int64_t pairs) {
  const int64_t i = (int64_t)blockIdx.x * PROBE_BLOCK + threadIdx.x;
  if (i >= pairs) return;
  float2 s = make_float2(1.f, 2.f);
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const float2 v = in[k * pairs + i];
    s.x += v.x;
    s.y += v.y;
  }
  if (NW == 0) {
    if (s.x == 12345.678f) out[i] = s;     // keeps the loads alive; never true for the inputs bench.py uses
    return;
  }
#pragma unroll
  for (int k = 0; k < NW; ++k) out[k * pairs + i] = make_float2(s.x + (float)k, s.y);
}

}  // namespace p2

extern "C" {

int p2hip_stream_probe(const float* in, float* out, int64_t pairs, int n_read, int n_write, void* stream) {
  if (pairs <= 0 || pairs > ((int64_t)0x7FFFFFFF) * p2::PROBE_BLOCK || !out || (n_read > 0 && !in)) return P2_EINVAL;
  if (!p2_aligned8(in) || !p2_aligned8(out)) return P2_EINVAL;
  const dim3 grid((unsigned)((pairs + p2::PROBE_BLOCK - 1) / p2::PROBE_BLOCK)), block(p2::PROBE_BLOCK);
  const float2* i2 = reinterpret_cast<const float2*>(in);
  float2* o2 = reinterpret_cast<float2*>(out);
  hipStream_t st = (hipStream_t)stream;
  if (n_read == 5 && n_write == 7) hipLaunchKernelGGL((p2::stream_probe_kernel<5, 7>), grid, block, 0, st, i2, o2, pairs);
  else if (n_read == 1 && n_write == 1) hipLaunchKernelGGL((p2::stream_probe_kernel<1, 1>), grid, block, 0, st, i2, o2, pairs);
  else if (n_read == 2 && n_write == 0) hipLaunchKernelGGL((p2::stream_probe_kernel<2, 0>), grid, block, 0, st, i2, o2, pairs);
  else if (n_read == 0 && n_write == 2) hipLaunchKernelGGL((p2::stream_probe_kernel<0, 2>), grid, block, 0, st, i2, o2, pairs);
  else return P2_EINVAL;
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
