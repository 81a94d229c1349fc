// Local best response, one tree level per launch (bottom-up from the host).
//
// Replaces the per-depth body of _best_response_values
// (src/p2/search/cfr_evaluator.py:636-714) on the sparse tree.  For a parent p with actor a,
// deviating player d and children c (contiguous rows, action ascending):
//   a == d : V[p][a][h] = max_c V[c][a][h] (first maximum wins, like argmax);
//            w_c[h] = 1 if c is h's maximising child else 0
//   a != d : V[p][a][h] = sum_c policy[c][h] V[c][a][h];  w_c[h] = policy[c][h]
//   other player o:  V[p][o][h] = sum_c U(b_a w_c)[h] / U(b_a)[h] * V[c][o][h]   (0 where
//            U(b_a)[h] <= 1e-5), U = unblocked mass, b_a = beliefs[p][a]
// which covers the reference's four cases (:690-703) because the opponent-conditioned policy
// of the ordinary backup is the same ratio with w_c = policy[c].  Rows without children keep
// the leaf values the caller put there.  One workgroup per parent; the weighted beliefs of all
// children and b_a are card-summed in one pass.  The kernel is compiled for at most five and at most
// eight children per parent: 34 KB of LDS (four workgroups per CU) against 51 KB (three).
#pragma once
#include "common.h"
#include "unblocked.hip"

namespace p2 {

constexpr int BR_BLOCK = 256;
constexpr int BR_PPT = 3;
constexpr int BR_MAXC = 8;
constexpr int BR_GRP = 4;   // children whose rows are in flight together
constexpr int BR_STRIDE = P2_H + 2;
static_assert(BR_BLOCK == UB_BLOCK, "card_sums_multi assumes the block size");

template <int MAXC>
__global__ __launch_bounds__(BR_BLOCK) void best_response_level_kernel(
    float* __restrict__ values, const float* __restrict__ policy, const float* __restrict__ beliefs,
    const int64_t* __restrict__ to_act, const int64_t* __restrict__ deviating_player,
    const int64_t* __restrict__ child_offsets, const int64_t* __restrict__ child_count, int64_t parent_base) {
  __shared__ __align__(8) float t[MAXC + 1][BR_STRIDE];
  __shared__ double cs[(MAXC + 1) * P2_CARDS];
  const int64_t p = parent_base + blockIdx.x;
  const int nc = (int)child_count[p];
  if (nc <= 0 || nc > MAXC) return;
  const int64_t c0 = child_offsets[p];
  const int actor = (int)to_act[p];
  const bool is_dev = (int)deviating_player[p] == actor;

  float b[BR_PPT][2], av[BR_PPT][2];
  int best[BR_PPT][2];
  uint32_t ab[BR_PPT][2];
#pragma unroll
  for (int k = 0; k < BR_PPT; ++k) {
    const int idx = threadIdx.x + k * BR_BLOCK;
    const bool in = idx < P2_HPAIRS;
    float2 x = make_float2(0.f, 0.f);
    if (in) x = p2_row2(beliefs, p * 2 + actor)[idx];
    b[k][0] = x.x; b[k][1] = x.y;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int h = in ? 2 * idx + q : 0;
      ab[k][q] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8);
      av[k][q] = is_dev ? -3.402823466e+38f : 0.f;
      best[k][q] = 0;
    }
    if (in) reinterpret_cast<float2*>(t[nc])[idx] = x;
  }
  // Children are taken in groups of BR_GRP whose rows are all requested before the first is used
  // (indices beyond the last child repeat it: a cache hit instead of a branch around every load), so a
  // parent with up to four children costs one round trip to memory per pass instead of one per child.
  auto load_group = [&](const float* __restrict__ base, int64_t row0, int64_t row_step, int plane, int g0,
                        float2 (&dst)[BR_GRP][BR_PPT]) {
#pragma unroll
    for (int j = 0; j < BR_GRP; ++j) {
      const int c = g0 + j < nc ? g0 + j : nc - 1;
      const float2* src = p2_row2(base, (row0 + c) * row_step + plane);
#pragma unroll
      for (int k = 0; k < BR_PPT; ++k) {
        const int idx = threadIdx.x + k * BR_BLOCK;
        dst[j][k] = src[idx < P2_HPAIRS ? idx : 0];
      }
    }
  };
  // pass 1: the actor's value and (for a deviating actor) each hand's maximising child
  for (int g0 = 0; g0 < nc; g0 += BR_GRP) {
    float2 v[BR_GRP][BR_PPT], pi[BR_GRP][BR_PPT];
    load_group(values, c0, 2, actor, g0, v);
    if (!is_dev) load_group(policy, c0, 1, 0, g0, pi);
#pragma unroll
    for (int j = 0; j < BR_GRP; ++j) {
      const int c = g0 + j;
      if (c >= nc) break;
#pragma unroll
      for (int k = 0; k < BR_PPT; ++k) {
        const int idx = threadIdx.x + k * BR_BLOCK;
        if (idx >= P2_HPAIRS) continue;
        const float vv[2] = {v[j][k].x, v[j][k].y};
        if (is_dev) {
#pragma unroll
          for (int q = 0; q < 2; ++q)
            if (vv[q] > av[k][q]) { av[k][q] = vv[q]; best[k][q] = c; }
        } else {
          av[k][0] += vv[0] * pi[j][k].x;
          av[k][1] += vv[1] * pi[j][k].y;
          reinterpret_cast<float2*>(t[c])[idx] = make_float2(b[k][0] * pi[j][k].x, b[k][1] * pi[j][k].y);
        }
      }
    }
  }
  if (is_dev) {
    for (int c = 0; c < nc; ++c) {
#pragma unroll
      for (int k = 0; k < BR_PPT; ++k) {
        const int idx = threadIdx.x + k * BR_BLOCK;
        if (idx < P2_HPAIRS)
          reinterpret_cast<float2*>(t[c])[idx] =
              make_float2(best[k][0] == c ? b[k][0] : 0.f, best[k][1] == c ? b[k][1] : 0.f);
      }
    }
  }
  // the other player's values of the first group are requested before the card sums and arrive behind them
  float2 vo[BR_GRP][BR_PPT];
  load_group(values, c0, 2, 1 - actor, 0, vo);
  p2_sync_lds();
  card_sums_multi(t[0], BR_STRIDE, nc + 1, cs);
  // pass 2: the other player's value under the projected action probabilities
  const double total_b = card_total(cs + nc * P2_CARDS);
  float ub[BR_PPT][2], ov[BR_PPT][2];
#pragma unroll
  for (int k = 0; k < BR_PPT; ++k)
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const double v = total_b - cs[nc * P2_CARDS + (ab[k][q] & 0xFFu)] - cs[nc * P2_CARDS + (ab[k][q] >> 8)] + (double)b[k][q];
      // one reciprocal per hand instead of a division per hand and child (0 where the opponent has no
      // compatible mass: the projected probability is then 0, cfr_evaluator.py:700-703)
      const float u0 = fmaxf((float)v, 0.f);
      ub[k][q] = u0 > 1e-5f ? 1.0f / u0 : 0.f;
      ov[k][q] = 0.f;
    }
  for (int g0 = 0; g0 < nc; g0 += BR_GRP) {
    if (g0 > 0) load_group(values, c0, 2, 1 - actor, g0, vo);
#pragma unroll
    for (int j = 0; j < BR_GRP; ++j) {
      const int c = g0 + j;
      if (c >= nc) break;
      const double* csc = cs + c * P2_CARDS;
      const double total_c = card_total(csc);
#pragma unroll
      for (int k = 0; k < BR_PPT; ++k) {
        const int idx = threadIdx.x + k * BR_BLOCK;
        if (idx >= P2_HPAIRS) continue;
        const float2 m = reinterpret_cast<const float2*>(t[c])[idx];
        const float mm[2] = {m.x, m.y}, vv[2] = {vo[j][k].x, vo[j][k].y};
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const double u = total_c - csc[ab[k][q] & 0xFFu] - csc[ab[k][q] >> 8] + (double)mm[q];
          const float uc = fmaxf((float)u, 0.f);
          ov[k][q] += (uc * ub[k][q]) * vv[q];
        }
      }
    }
  }
  float2* oa = p2_row2(values, p * 2 + actor);
  float2* oo = p2_row2(values, p * 2 + (1 - actor));
#pragma unroll
  for (int k = 0; k < BR_PPT; ++k) {
    const int idx = threadIdx.x + k * BR_BLOCK;
    if (idx < P2_HPAIRS) {
      oa[idx] = make_float2(av[k][0], av[k][1]);
      oo[idx] = make_float2(ov[k][0], ov[k][1]);
    }
  }
}

}  // namespace p2

extern "C" {

int p2hip_best_response_level(float* values, const float* policy, const float* beliefs, const int64_t* to_act,
                              const int64_t* deviating_player, const int64_t* child_offsets,
                              const int64_t* child_count, int64_t parent_base, int64_t num_parents,
                              int max_children, void* stream) {
  if (num_parents < 0 || parent_base < 0 || max_children < 1 || max_children > p2::BR_MAXC) return P2_EINVAL;
  if (num_parents == 0) return 0;
  if (!values || !policy || !beliefs || !to_act || !deviating_player || !child_offsets || !child_count) return P2_EINVAL;
  if (!p2_aligned8(values) || !p2_aligned8(policy) || !p2_aligned8(beliefs)) return P2_EINVAL;
  if (max_children <= 5)
    hipLaunchKernelGGL((p2::best_response_level_kernel<5>), dim3((unsigned)num_parents), dim3(p2::BR_BLOCK), 0,
                       (hipStream_t)stream, values, policy, beliefs, to_act, deviating_player, child_offsets,
                       child_count, parent_base);
  else
    hipLaunchKernelGGL((p2::best_response_level_kernel<p2::BR_MAXC>), dim3((unsigned)num_parents),
                       dim3(p2::BR_BLOCK), 0, (hipStream_t)stream, values, policy, beliefs, to_act,
                       deviating_player, child_offsets, child_count, parent_base);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
