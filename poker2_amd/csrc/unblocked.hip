// Unblocked (card-compatible) mass of a 1326-vector and the ratio of two.
//
//   out[(a,b)] = max(S - cs[a] - cs[b] + t[(a,b)], 0),  S = sum t,
//   cs[c] = sum of t over the 51 combos containing card c
//
// Replaces the float64 1326x1326 product of src/p2/env/card_utils.py:196-222
// and the "matmul + finalize" pair of src/p2/search/fused_cfr_triton.py:928-959,
// :1008-1026, :1408-1496.  Rows are staged in LDS, four lanes share one card sum,
// sums run in float64 so the result rounds like the float64 product does.
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

// ---- standalone kernels -------------------------------------------------------------
// A workgroup takes a group of UB_ROWS vectors: rows through registers into LDS, one card-sum pass
// for the group, outputs.  The launch gives every group its own workgroup (see ub_grid); the
// group loop with its register prefetch of the next group only repeats on grids that were capped.
constexpr int UB_ROWS = 4;
constexpr int UB_PPT = 3;                  // float2 pairs per thread and row: 3 * 256 >= 663
constexpr int UB_STRIDE = P2_H + 2;

struct UnblockedLds {
  __align__(8) float t[UB_ROWS][UB_STRIDE];
  double cs[UB_ROWS * P2_CARDS];
};

// Card sums for the standalone kernels: lanes 4c..4c+3 own card c for the whole kernel, so
// the LDS offsets of a lane's 13 partner combos are computed once and kept in registers.
// Same partner split and shuffle order as card_sums_multi: the sums are bit-identical.
struct CardLane {
  int idx[13];   // offset of the combo (c, partner sub + 4i) inside a 1326-vector; -1 = none
  int card;      // 0..51, or -1 for the 48 idle lanes of the workgroup
};

__device__ __forceinline__ void card_lane_init(CardLane& cl) {
  const int c = threadIdx.x >> 2, sub = threadIdx.x & 3;
  cl.card = c < P2_CARDS ? c : -1;
#pragma unroll
  for (int i = 0; i < 13; ++i) {
    const int j = sub + 4 * i;
    int off = -1;
    if (c < P2_CARDS && j < 51) {
      const int x = j < c ? j : j + 1;
      off = p2_combo_index(x < c ? x : c, x < c ? c : x);
    }
    cl.idx[i] = off;
  }
}

// cs[v*52 + c] for the `nvec` vectors staged at t + v*stride.  Ends with an LDS barrier.
__device__ __forceinline__ void card_sums_fixed(const CardLane& cl, const float* t, int stride, int nvec,
                                                double* cs) {
  for (int v = 0; v < nvec; ++v) {
    const float* tv = t + v * stride;
    double acc = 0.0;
#pragma unroll
    for (int i = 0; i < 13; ++i)
      if (cl.idx[i] >= 0) acc += (double)tv[cl.idx[i]];
    acc += __shfl_xor(acc, 1, P2_WAVE);
    acc += __shfl_xor(acc, 2, P2_WAVE);
    if (cl.card >= 0 && (threadIdx.x & 3) == 0) cs[v * P2_CARDS + cl.card] = acc;
  }
  p2_sync_lds();
}

// The two cards of the six hands a lane writes (hands 2i, 2i+1 of pairs i = tid + k*256).
struct HandCards { uint32_t ab[UB_PPT][2]; };   // a | b << 8

__device__ __forceinline__ void hand_cards_init(HandCards& hc) {
#pragma unroll
  for (int k = 0; k < UB_PPT; ++k) {
    const int i = threadIdx.x + k * UB_BLOCK;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int h = i < P2_HPAIRS ? 2 * i + q : 0;
      hc.ab[k][q] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8);
    }
  }
}

__device__ __forceinline__ float unblocked_of(float t, const double* cs, double S, uint32_t ab) {
  const double v = S - cs[ab & 0xFFu] - cs[ab >> 8] + (double)t;
  return fmaxf((float)v, 0.f);
}

__device__ __forceinline__ void fetch_row(const float* __restrict__ src, float2 (&pre)[UB_PPT]) {
  const float2* s2 = reinterpret_cast<const float2*>(src);
#pragma unroll
  for (int k = 0; k < UB_PPT; ++k) {
    const int i = threadIdx.x + k * UB_BLOCK;
    pre[k] = i < P2_HPAIRS ? s2[i] : make_float2(0.f, 0.f);
  }
}

__device__ __forceinline__ void stage_row(const float2 (&pre)[UB_PPT], float* lds) {
  float2* l2 = reinterpret_cast<float2*>(lds);
#pragma unroll
  for (int k = 0; k < UB_PPT; ++k) {
    const int i = threadIdx.x + k * UB_BLOCK;
    if (i < P2_HPAIRS) l2[i] = pre[k];
  }
}

// rows: out[r] = unblocked(target[src_row(r)])
//   to_act == nullptr : src_row(r) = r over a [rows, H] tensor
//   to_act != nullptr : target is [total, 2, H]; src_row(r) = 2*r + (to_act[r] ^ flip)
__global__ __launch_bounds__(UB_BLOCK) void unblocked_mass_kernel(const float* __restrict__ target,
                                                                   const int64_t* __restrict__ to_act, int flip,
                                                                   int64_t rows, float* __restrict__ out) {
  __shared__ UnblockedLds s;
  const int64_t ngroups = (rows + UB_ROWS - 1) / UB_ROWS;
  CardLane cl;
  HandCards hc;
  card_lane_init(cl);
  hand_cards_init(hc);
  float2 pre[UB_ROWS][UB_PPT];
  auto fetch = [&](int64_t g) {
#pragma unroll
    for (int v = 0; v < UB_ROWS; ++v) {
      const int64_t r = g * UB_ROWS + v;
      if (r < rows) {
        const int64_t src = to_act ? 2 * r + ((int)to_act[r] ^ flip) : r;
        fetch_row(target + src * P2_H, pre[v]);
      }
    }
  };
  int64_t g = blockIdx.x;
  if (g < ngroups) fetch(g);
  for (; g < ngroups; g += gridDim.x) {
    const int nv = (int)(rows - g * UB_ROWS < UB_ROWS ? rows - g * UB_ROWS : UB_ROWS);
#pragma unroll
    for (int v = 0; v < UB_ROWS; ++v)
      if (v < nv) stage_row(pre[v], s.t[v]);
    p2_sync_lds();
    if (g + gridDim.x < ngroups) fetch(g + gridDim.x);
    card_sums_fixed(cl, s.t[0], UB_STRIDE, nv, s.cs);
    for (int v = 0; v < nv; ++v) {
      const double* cs = s.cs + v * P2_CARDS;
      const double total = card_total(cs);
      float2* o2 = p2_row2(out, g * UB_ROWS + v);
      const float2* t2 = reinterpret_cast<const float2*>(s.t[v]);
#pragma unroll
      for (int k = 0; k < UB_PPT; ++k) {
        const int i = threadIdx.x + k * UB_BLOCK;
        if (i < P2_HPAIRS) {
          const float2 tv = t2[i];
          o2[i] = make_float2(unblocked_of(tv.x, cs, total, hc.ab[k][0]), unblocked_of(tv.y, cs, total, hc.ab[k][1]));
        }
      }
    }
    p2_sync_lds();  // the next group overwrites the staged rows and the card sums
  }
}

// out[c] = d > eps ? unblocked(numer[c]) / d : 0 with d = unblocked(denom[parent(c)]);
// two (numerator, denominator) pairs per group.
__global__ __launch_bounds__(UB_BLOCK) void unblocked_ratio_kernel(const float* __restrict__ numer,
                                                                    const float* __restrict__ denom,
                                                                    const int64_t* __restrict__ parent_index,
                                                                    float eps, int64_t rows, float* __restrict__ out) {
  __shared__ UnblockedLds s;
  constexpr int ITEMS = UB_ROWS / 2;
  const int64_t ngroups = (rows + ITEMS - 1) / ITEMS;
  CardLane cl;
  HandCards hc;
  card_lane_init(cl);
  hand_cards_init(hc);
  float2 pre[UB_ROWS][UB_PPT];
  auto fetch = [&](int64_t g) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int64_t c = g * ITEMS + it;
      if (c < rows) {
        const int64_t p = parent_index ? parent_index[c] : c;
        fetch_row(numer + c * P2_H, pre[2 * it]);
        fetch_row(denom + p * P2_H, pre[2 * it + 1]);
      }
    }
  };
  int64_t g = blockIdx.x;
  if (g < ngroups) fetch(g);
  for (; g < ngroups; g += gridDim.x) {
    const int ni = (int)(rows - g * ITEMS < ITEMS ? rows - g * ITEMS : ITEMS);
#pragma unroll
    for (int v = 0; v < UB_ROWS; ++v)
      if (v < 2 * ni) stage_row(pre[v], s.t[v]);
    p2_sync_lds();
    if (g + gridDim.x < ngroups) fetch(g + gridDim.x);
    card_sums_fixed(cl, s.t[0], UB_STRIDE, 2 * ni, s.cs);
    for (int it = 0; it < ni; ++it) {
      const float2* tn = reinterpret_cast<const float2*>(s.t[2 * it]);
      const float2* td = reinterpret_cast<const float2*>(s.t[2 * it + 1]);
      const double* csn = s.cs + (2 * it) * P2_CARDS;
      const double* csd = csn + P2_CARDS;
      const double sn = card_total(csn), sd = card_total(csd);
      float2* o2 = p2_row2(out, g * ITEMS + it);
#pragma unroll
      for (int k = 0; k < UB_PPT; ++k) {
        const int i = threadIdx.x + k * UB_BLOCK;
        if (i < P2_HPAIRS) {
          const float2 vn = tn[i], vd = td[i];
          const float n0 = unblocked_of(vn.x, csn, sn, hc.ab[k][0]), d0 = unblocked_of(vd.x, csd, sd, hc.ab[k][0]);
          const float n1 = unblocked_of(vn.y, csn, sn, hc.ab[k][1]), d1 = unblocked_of(vd.y, csd, sd, hc.ab[k][1]);
          o2[i] = make_float2(d0 > eps ? n0 / d0 : 0.f, d1 > eps ? n1 / d1 : 0.f);
        }
      }
    }
    p2_sync_lds();
  }
}

// out[c] = d > eps ? unblocked(numer[c]) / d : 0 with d = denom_unblocked[parent(c)] already computed
// (one row per parent): siblings share their parent's row, so the denominator's card sums are taken once
// per parent instead of once per child.  Four numerators per group.
__global__ __launch_bounds__(UB_BLOCK) void unblocked_ratio_of_kernel(const float* __restrict__ numer,
                                                                       const float* __restrict__ denom_unblocked,
                                                                       const int64_t* __restrict__ parent_index,
                                                                       float eps, int64_t rows, float* __restrict__ out) {
  __shared__ UnblockedLds s;
  const int64_t g = blockIdx.x;
  const int nv = (int)(rows - g * UB_ROWS < UB_ROWS ? rows - g * UB_ROWS : UB_ROWS);
  CardLane cl;
  HandCards hc;
  card_lane_init(cl);
  hand_cards_init(hc);
  float2 pre[UB_ROWS][UB_PPT], den[UB_ROWS][UB_PPT];
#pragma unroll
  for (int v = 0; v < UB_ROWS; ++v) {
    const int64_t c = g * UB_ROWS + (v < nv ? v : nv - 1);       // past the end: the last one again, not stored
    fetch_row(numer + c * P2_H, pre[v]);
    fetch_row(denom_unblocked + parent_index[c] * P2_H, den[v]);
  }
#pragma unroll
  for (int v = 0; v < UB_ROWS; ++v) stage_row(pre[v], s.t[v]);
  p2_sync_lds();
  card_sums_fixed(cl, s.t[0], UB_STRIDE, nv, s.cs);
#pragma unroll
  for (int v = 0; v < UB_ROWS; ++v) {
    if (v >= nv) break;
    const double* cs = s.cs + v * P2_CARDS;
    const double total = card_total(cs);
    float2* o2 = p2_row2(out, g * UB_ROWS + v);
#pragma unroll
    for (int k = 0; k < UB_PPT; ++k) {
      const int i = threadIdx.x + k * UB_BLOCK;
      if (i < P2_HPAIRS) {
        const float n0 = unblocked_of(pre[v][k].x, cs, total, hc.ab[k][0]);
        const float n1 = unblocked_of(pre[v][k].y, cs, total, hc.ab[k][1]);
        const float d0 = den[v][k].x, d1 = den[v][k].y;
        o2[i] = make_float2(d0 > eps ? n0 / d0 : 0.f, d1 > eps ? n1 / d1 : 0.f);
      }
    }
  }
}

// One workgroup per group of rows, dispatched in address order (measured 3 % faster than a
// resident grid walking the groups with a stride, although each workgroup then recomputes its
// lanes' combo offsets); the kernels' loops only run more than once beyond 2^30 groups.
static inline unsigned ub_grid(int64_t groups, int /*per_cu*/) {
  const int64_t cap = (int64_t)1 << 30;
  return (unsigned)(groups < cap ? groups : cap);
}

}  // namespace p2

extern "C" {

int p2hip_unblocked_mass(const float* target, int64_t rows, float* out, void* stream) {
  if (rows < 0 || (rows > 0 && (!target || !out))) return P2_EINVAL;
  if (rows == 0) return 0;
  if (!p2_aligned8(target) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_mass_kernel, dim3(p2::ub_grid((rows + p2::UB_ROWS - 1) / p2::UB_ROWS, 4)),
                     dim3(p2::UB_BLOCK), 0, (hipStream_t)stream, target, (const int64_t*)nullptr, 0, rows, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_unblocked_mass_by_player(const float* beliefs, const int64_t* to_act, int64_t top, int opponent,
                                   float* out, void* stream) {
  if (top < 0 || (top > 0 && (!beliefs || !to_act || !out))) return P2_EINVAL;
  if (top == 0) return 0;
  if (!p2_aligned8(beliefs) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_mass_kernel, dim3(p2::ub_grid((top + p2::UB_ROWS - 1) / p2::UB_ROWS, 4)),
                     dim3(p2::UB_BLOCK), 0, (hipStream_t)stream, beliefs, to_act, opponent ? 1 : 0, top, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_unblocked_mass_ratio(const float* numer, const float* denom, const int64_t* parent_index,
                               int64_t rows, float eps, float* out, void* stream) {
  if (rows < 0 || (rows > 0 && (!numer || !denom || !out))) return P2_EINVAL;
  if (rows == 0) return 0;
  if (!p2_aligned8(numer) || !p2_aligned8(denom) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_ratio_kernel, dim3(p2::ub_grid((rows + 1) / 2, 4)), dim3(p2::UB_BLOCK), 0,
                     (hipStream_t)stream, numer, denom, parent_index, eps, rows, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_unblocked_mass_ratio_of(const float* numer, const float* denom_unblocked, const int64_t* parent_index,
                                  int64_t rows, float eps, float* out, void* stream) {
  if (rows < 0 || rows > ((int64_t)0x7FFFFFFF) * p2::UB_ROWS) return P2_EINVAL;
  if (rows > 0 && (!numer || !denom_unblocked || !parent_index || !out)) return P2_EINVAL;
  if (rows == 0) return 0;
  if (!p2_aligned8(numer) || !p2_aligned8(denom_unblocked) || !p2_aligned8(out)) return P2_EINVAL;
  hipLaunchKernelGGL(p2::unblocked_ratio_of_kernel, dim3((unsigned)((rows + p2::UB_ROWS - 1) / p2::UB_ROWS)),
                     dim3(p2::UB_BLOCK), 0, (hipStream_t)stream, numer, denom_unblocked, parent_index, eps, rows, out);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
