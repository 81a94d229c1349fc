// Unblocked (card-compatible) mass of a 1326-vector and the ratio of two.
//
//   out[(a,b)] = max(S - cs[a] - cs[b] + t[(a,b)], 0),  S = sum t,
//   cs[c] = sum of t over the 51 combos containing card c
//
// Replaces the float64 1326x1326 product of src/p2/env/card_utils.py:196-222
// and the "matmul + finalize" pair of src/p2/search/fused_cfr_triton.py:928-959,
// :1008-1026, :1408-1496.  One workgroup per row: the row is staged in LDS,
// each wave reduces 13 cards (lane j = j-th partner card), sums run in float64
// so the result rounds like the float64 product does.
#pragma once
#include "common.h"

namespace p2 {

constexpr int UB_BLOCK = 256;
constexpr int UB_WAVES = UB_BLOCK / 64;

// Card sums of `nvec` vectors held in LDS (vector v starts at t + v*stride):
// cs[v*52 + c] = sum of the 51 combos of vector v that hold card c, in float64.
// Four lanes share one (vector, card) task: each adds 13 partner cards, two shuffles
// combine them.  Every thread must call it after an LDS barrier that covers the staged
// vectors; it ends with an LDS barrier.
__device__ __forceinline__ void card_sums_multi(const float* t, int stride, int nvec, double* cs) {
  const int sub = threadIdx.x & 3;
  const int ntask = nvec * P2_CARDS;
  for (int base = 0; base < ntask; base += UB_BLOCK / 4) {
    const int task = base + (threadIdx.x >> 2);
    const bool valid = task < ntask;
    double v = 0.0;
    if (valid) {
      const int vec = task / P2_CARDS, c = task - vec * P2_CARDS;
      const float* tv = t + vec * stride;
#pragma unroll
      for (int i = 0; i < 13; ++i) {
        const int j = sub + 4 * i;
        if (j < 51) {
          const int x = j < c ? j : j + 1;  // partner card
          const int lo = x < c ? x : c, hi = x < c ? c : x;
          v += (double)tv[p2_combo_index(lo, hi)];
        }
      }
    }
    v += __shfl_xor(v, 1, P2_WAVE);
    v += __shfl_xor(v, 2, P2_WAVE);
    if (valid && sub == 0) cs[task] = v;
  }
  p2_sync_lds();
}

// Total mass of a vector from its 52 card sums (every combo is counted under both of its
// cards).  Wave-level: every lane of every wave gets the value; no barrier.
__device__ __forceinline__ double card_total(const double* cs52) {
  const int lane = threadIdx.x & 63;
  const double x = lane < P2_CARDS ? cs52[lane] : 0.0;
  return 0.5 * p2_wave_sum(x);
}

__device__ __forceinline__ float unblocked_at(const float* t, const double* cs, double S, int h) {
  const double v = S - cs[p2_combo.a[h]] - cs[p2_combo.b[h]] + (double)t[h];
  return fmaxf((float)v, 0.f);
}

__device__ __forceinline__ void load_row(const float* __restrict__ src, float* lds) {
  const float2* s2 = reinterpret_cast<const float2*>(src);
  float2* l2 = reinterpret_cast<float2*>(lds);
  for (int i = threadIdx.x; i < P2_HPAIRS; i += UB_BLOCK) l2[i] = s2[i];
}

// rows: out[r] = unblocked(target[src_row(r)])
//   gather == nullptr : src_row(r) = r over a [rows, H] tensor
//   gather != nullptr : target is [total, 2, H]; src_row(r) = 2*r + (to_act[r] ^ flip)
__global__ __launch_bounds__(UB_BLOCK) void unblocked_mass_kernel(const float* __restrict__ target,
                                                                   const int64_t* __restrict__ to_act, int flip,
                                                                   float* __restrict__ out) {
  __shared__ __align__(8) float t[P2_H + 2];
  __shared__ double cs[P2_CARDS];
  const int64_t r = blockIdx.x;
  int64_t src = r;
  if (to_act) src = 2 * r + ((int)to_act[r] ^ flip);
  load_row(target + src * P2_H, t);
  p2_sync_lds();
  card_sums_multi(t, 0, 1, cs);
  const double s = card_total(cs);
  float2* o2 = p2_row2(out, r);
  for (int i = threadIdx.x; i < P2_HPAIRS; i += UB_BLOCK) {
    float2 v;
    v.x = unblocked_at(t, cs, s, 2 * i);
    v.y = unblocked_at(t, cs, s, 2 * i + 1);
    o2[i] = v;
  }
}

// out[c] = d > eps ? unblocked(numer[c]) / d : 0 with d = unblocked(denom[parent(c)])
__global__ __launch_bounds__(UB_BLOCK) void unblocked_ratio_kernel(const float* __restrict__ numer,
                                                                    const float* __restrict__ denom,
                                                                    const int64_t* __restrict__ parent_index,
                                                                    float eps, float* __restrict__ out) {
  __shared__ __align__(8) float tt[2][P2_H + 2];  // numerator row, denominator row
  __shared__ double cs2[2 * P2_CARDS];
  float* tn = tt[0];
  float* td = tt[1];
  const double* csn = cs2;
  const double* csd = cs2 + P2_CARDS;
  const int64_t c = blockIdx.x;
  const int64_t p = parent_index ? parent_index[c] : c;
  load_row(numer + c * P2_H, tn);
  load_row(denom + p * P2_H, td);
  p2_sync_lds();
  card_sums_multi(tt[0], P2_H + 2, 2, cs2);
  const double sn = card_total(csn), sd = card_total(csd);
  float2* o2 = p2_row2(out, c);
  for (int i = threadIdx.x; i < P2_HPAIRS; i += UB_BLOCK) {
    float r[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int h = 2 * i + k;
      const float n = unblocked_at(tn, csn, sn, h);
      const float d = unblocked_at(td, csd, sd, h);
      r[k] = d > eps ? n / d : 0.f;
    }
    o2[i] = make_float2(r[0], r[1]);
  }
}

}  // namespace p2

extern "C" {

int p2hip_unblocked_mass(const float* target, int64_t rows, float* out, void* stream) {
  if (rows < 0 || (rows > 0 && (!target || !out))) return P2_EINVAL;
  if (rows == 0) return 0;
  if (!p2_aligned8(target) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_mass_kernel, dim3((unsigned)rows), dim3(p2::UB_BLOCK), 0, (hipStream_t)stream,
                     target, (const int64_t*)nullptr, 0, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_unblocked_mass_by_player(const float* beliefs, const int64_t* to_act, int64_t top, int opponent,
                                   float* out, void* stream) {
  if (top < 0 || (top > 0 && (!beliefs || !to_act || !out))) return P2_EINVAL;
  if (top == 0) return 0;
  if (!p2_aligned8(beliefs) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_mass_kernel, dim3((unsigned)top), dim3(p2::UB_BLOCK), 0, (hipStream_t)stream,
                     beliefs, to_act, opponent ? 1 : 0, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_unblocked_mass_ratio(const float* numer, const float* denom, const int64_t* parent_index,
                               int64_t rows, float eps, float* out, void* stream) {
  if (rows < 0 || (rows > 0 && (!numer || !denom || !out))) return P2_EINVAL;
  if (rows == 0) return 0;
  if (!p2_aligned8(numer) || !p2_aligned8(denom) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_ratio_kernel, dim3((unsigned)rows), dim3(p2::UB_BLOCK), 0, (hipStream_t)stream,
                     numer, denom, parent_index, eps, out);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
