// Measurement aid, not part of the search path: a structure-free element-wise stream over n_read input
// and n_write output arrays of `pairs` float2 each (array k starts k * pairs float2 after the base
// pointer).  One 8-byte access per lane and array, workgroups in address order: what HBM gives a kernel
// of that read / write mix when nothing else limits it.  bench.py reports it beside the iteration
// kernel's rate (12 vectors read and 17 written per node: 5 + 7 arrays are the same 41 % / 59 % mix).
#pragma once
#include "common.h"

namespace p2 {

constexpr int PROBE_BLOCK = 256;

typedef float probe_f2 __attribute__((ext_vector_type(2)));

// NT: loads and stores marked non-temporal (every byte is touched once).
template <int NR, int NW, bool NT>
__global__ __launch_bounds__(PROBE_BLOCK) void stream_probe_kernel(const probe_f2* __restrict__ in,
                                                                    probe_f2* __restrict__ out, int64_t pairs) {
  const int64_t i = (int64_t)blockIdx.x * PROBE_BLOCK + threadIdx.x;
  if (i >= pairs) return;
  probe_f2 s = {1.f, 2.f};
#pragma unroll
  for (int k = 0; k < NR; ++k) s += NT ? __builtin_nontemporal_load(in + k * pairs + i) : in[k * pairs + i];
  if (NW == 0) {
    if (s.x == 12345.678f) out[i] = s;     // keeps the loads alive; never true for the inputs bench.py uses
    return;
  }
#pragma unroll
  for (int k = 0; k < NW; ++k) {
    const probe_f2 o = {s.x + (float)k, s.y};
    if (NT) __builtin_nontemporal_store(o, out + k * pairs + i);
    else out[k * pairs + i] = o;
  }
}

}  // namespace p2

extern "C" {

int p2hip_stream_probe(const float* in, float* out, int64_t pairs, int n_read, int n_write, int non_temporal,
                       void* stream) {
  if (pairs <= 0 || pairs > ((int64_t)0x7FFFFFFF) * p2::PROBE_BLOCK || !out || (n_read > 0 && !in)) return P2_EINVAL;
  if (!p2_aligned8(in) || !p2_aligned8(out)) return P2_EINVAL;
  const dim3 grid((unsigned)((pairs + p2::PROBE_BLOCK - 1) / p2::PROBE_BLOCK)), block(p2::PROBE_BLOCK);
  const p2::probe_f2* i2 = reinterpret_cast<const p2::probe_f2*>(in);
  p2::probe_f2* o2 = reinterpret_cast<p2::probe_f2*>(out);
  hipStream_t st = (hipStream_t)stream;
#define P2_PROBE(NR, NW)                                                                                      \
  if (n_read == NR && n_write == NW) {                                                                        \
    if (non_temporal) hipLaunchKernelGGL((p2::stream_probe_kernel<NR, NW, true>), grid, block, 0, st, i2, o2, pairs);  \
    else hipLaunchKernelGGL((p2::stream_probe_kernel<NR, NW, false>), grid, block, 0, st, i2, o2, pairs);      \
  } else
  P2_PROBE(5, 7) P2_PROBE(1, 1) P2_PROBE(2, 0) P2_PROBE(0, 2) return P2_EINVAL;
#undef P2_PROBE
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
