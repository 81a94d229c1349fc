// Kernels either side of the search in data generation: feature encoding of public states,
// bet amounts of the action bins, and policy targets gathered from the children.
//
// RebelFeatureEncoder.encode (src/p2/models/mlp/rebel_feature_encoder.py:55-127),
// HUNLTensorEnv.legal_bins_amounts_and_mask (src/p2/env/hunl_tensor_env.py:348-423, amounts only)
// and the policy targets of CFREvaluator.training_data (src/p2/search/cfr_evaluator.py:1392-1393:
// _pull_back of the average policy, then [node, hand, action]).
#pragma once
#include "common.h"

namespace p2 {

constexpr int DG_BLOCK = 256;
constexpr int DG_MAX_ACTIONS = 8;

// context [m,4] = (to_act, (to_act - button) mod 2, clamp(pot / max(start0 + start1, 1), 0, 10),
//                  committed differ and at least one action this round);
// board_out [m,5] = last_board where pre_chance (a byte per state, or the same flag for all), else board.
__global__ __launch_bounds__(DG_BLOCK) void encode_context_kernel(
    const int64_t* __restrict__ to_act, const int64_t* __restrict__ button, const int64_t* __restrict__ starting_stacks,
    const int64_t* __restrict__ pot, const int64_t* __restrict__ committed, const int64_t* __restrict__ actions,
    const uint8_t* __restrict__ pre_chance, int pre_chance_all, const int64_t* __restrict__ last_board,
    const int64_t* __restrict__ board, int64_t m, float* __restrict__ context, int64_t* __restrict__ board_out) {
  const int64_t i = (int64_t)blockIdx.x * DG_BLOCK + threadIdx.x;
  if (i >= m) return;
  const int64_t ta = to_act[i];
  const float total = fmaxf((float)starting_stacks[2 * i] + (float)starting_stacks[2 * i + 1], 1.0f);
  const float frac = fminf(fmaxf((float)pot[i] / total, 0.0f), 10.0f);
  const bool bet = committed[2 * i] != committed[2 * i + 1] && actions[i] > 0;
  float4 c;
  c.x = (float)ta;
  c.y = (float)(((ta - button[i]) % 2 + 2) % 2);
  c.z = frac;
  c.w = bet ? 1.0f : 0.0f;
  reinterpret_cast<float4*>(context)[i] = c;
  const bool pre = pre_chance ? pre_chance[i] != 0 : pre_chance_all != 0;
  const int64_t* src = (pre ? last_board : board) + 5 * i;
#pragma unroll
  for (int j = 0; j < 5; ++j) board_out[5 * i + j] = src[j];
}

struct DgBins {
  float bins[DG_MAX_ACTIONS - 3];
  int n_bins;
};

// amounts [m, n_bins + 3]: -1 for fold and call, to_call + trunc(bin * pot) for the bet bins
// (whether legal or not), the actor's stack for all-in.
__global__ __launch_bounds__(DG_BLOCK) void bet_amounts_kernel(const int64_t* __restrict__ to_act,
                                                                const int64_t* __restrict__ stacks,
                                                                const int64_t* __restrict__ committed,
                                                                const int64_t* __restrict__ pot, int64_t m, DgBins B,
                                                                int64_t* __restrict__ amounts) {
  const int64_t i = (int64_t)blockIdx.x * DG_BLOCK + threadIdx.x;
  if (i >= m) return;
  const int nb = B.n_bins + 3;
  const int me = (int)to_act[i], opp = 1 - me;
  const int64_t to_call = committed[2 * i + opp] - committed[2 * i + me];
  const float pot_f = (float)pot[i];
  int64_t* out = amounts + i * nb;
  out[0] = -1;
  out[1] = -1;
  for (int b = 0; b < B.n_bins; ++b) out[2 + b] = to_call + (int64_t)(B.bins[b] * pot_f);
  out[nb - 1] = stacks[2 * i + me];
}

// out[k, h, a] = policy_avg[c, h] for the child c of node rows[k] reached by action a, 0 where the
// action has no child.  One workgroup per node: the children's rows are read whole (coalesced
// float2) and scattered into LDS in the output's own [hand][action] order, so the node's output is
// a plain copy of that LDS image as one contiguous run.  A is a template parameter.
template <int A, bool WIDE>
__global__ __launch_bounds__(DG_BLOCK) void policy_targets_kernel(const float* __restrict__ policy_avg,
                                                                   const int64_t* __restrict__ rows,
                                                                   const int64_t* __restrict__ child_offsets,
                                                                   const int64_t* __restrict__ child_count,
                                                                   const int64_t* __restrict__ action_from_parent,
                                                                   float* __restrict__ out) {
  constexpr int HA = P2_H * A;                     // even: 1326 is
  __shared__ __align__(16) float tile[HA + 4];     // tile[h * A + a]
  const int64_t k = blockIdx.x;
  const int64_t r = rows[k];
  const int64_t first = child_offsets[r];
  const int n_children = (int)child_count[r];
  // All of the node's rows are requested before the first is scattered: one round trip to memory per
  // node instead of one per child and piece (children beyond A cannot exist; the loop after the
  // unrolled part only keeps such input from being dropped silently).
  constexpr int PIECES = (P2_HPAIRS + DG_BLOCK - 1) / DG_BLOCK;
  float2 x[A][PIECES];
  int act[A];
#pragma unroll
  for (int j = 0; j < A; ++j) {
    const bool have = j < n_children;
    // a slot without a child repeats the first child's row (a cache hit) and drops what it read; a node
    // without any child requests its own row instead: its child_offsets entry may equal the row count
    const int64_t row = have ? first + j : (n_children > 0 ? first : r);
    const int a = have ? (int)action_from_parent[row] : -1;
    act[j] = (a >= 0 && a < A) ? a : -1;
    const float2* src = p2_row2(policy_avg, row);
#pragma unroll
    for (int q = 0; q < PIECES; ++q) {
      const int idx = threadIdx.x + q * DG_BLOCK;
      x[j][q] = idx < P2_HPAIRS ? src[idx] : make_float2(0.f, 0.f);
    }
  }
  uint32_t present = 0;
#pragma unroll
  for (int j = 0; j < A; ++j) {
    if (act[j] < 0) continue;
    present |= 1u << act[j];
#pragma unroll
    for (int q = 0; q < PIECES; ++q) {
      const int idx = threadIdx.x + q * DG_BLOCK;
      if (idx >= P2_HPAIRS) continue;
      tile[2 * idx * A + act[j]] = x[j][q].x;
      tile[(2 * idx + 1) * A + act[j]] = x[j][q].y;
    }
  }
  for (int j = A; j < n_children; ++j) {
    const int a = (int)action_from_parent[first + j];
    if (a < 0 || a >= A) continue;
    present |= 1u << a;
    const float2* src = p2_row2(policy_avg, first + j);
    for (int idx = threadIdx.x; idx < P2_HPAIRS; idx += DG_BLOCK) {
      const float2 v = src[idx];
      tile[2 * idx * A + a] = v.x;
      tile[(2 * idx + 1) * A + a] = v.y;
    }
  }
#pragma unroll
  for (int a = 0; a < A; ++a)
    if (!((present >> a) & 1u))
      for (int h = threadIdx.x; h < P2_H; h += DG_BLOCK) tile[h * A + a] = 0.f;
  p2_sync_lds();
  const float2* tile2 = reinterpret_cast<const float2*>(tile);
  if (!WIDE) {
    float2* dst = reinterpret_cast<float2*>(out + k * (int64_t)HA);   // 8-byte aligned: HA * 4 is a multiple of 8
    for (int e2 = threadIdx.x; e2 < HA / 2; e2 += DG_BLOCK) dst[e2] = tile2[e2];
    return;
  }
  // `out` is 16-byte aligned: float4 at absolute positions, lanes placed on absolute 128-byte lines,
  // so every wave-wide store covers whole lines although a node's run starts on none (HA * 4 bytes
  // is a multiple of 8 only).  A float4 that straddles the run's start or end (at most one each) is
  // written as the float2 that belongs to this node.
  const int64_t span0 = k * (int64_t)HA;           // first float of the node, even
  const int64_t g_first = span0 >> 2, g_end = (span0 + HA + 3) >> 2;
  for (int64_t g = (g_first & ~7ll) + threadIdx.x; g < g_end; g += DG_BLOCK) {
    const int e = (int)((g << 2) - span0);         // the float4's first float inside the node: even, may be < 0
    const bool lo_ok = e >= 0 && e + 2 <= HA, hi_ok = e + 2 >= 0 && e + 4 <= HA;
    const int i2 = e >= 0 ? e >> 1 : 0;
    const float2 lo = tile2[i2], hi = tile2[e + 2 >= 0 ? (e + 2) >> 1 : 0];   // inside the padded tile either way
    if (lo_ok && hi_ok) reinterpret_cast<float4*>(out)[g] = make_float4(lo.x, lo.y, hi.x, hi.y);
    else if (lo_ok) reinterpret_cast<float2*>(out)[2 * g] = lo;
    else if (hi_ok) reinterpret_cast<float2*>(out)[2 * g + 1] = hi;
  }
}


// ---- leaf rows to and from the value network -------------------------------------------------
// A leaf's two ranges are one 2 x 1326 row of the [total, 2, 1326] float32 node table.  The network
// wants the rows of ITS leaves as one dense matrix, possibly in bf16 / fp16 and with further feature
// columns behind the ranges; its answers go back into the node table.  One workgroup per leaf, four
// floats per lane and step (rows are 8-byte aligned: two 8-byte loads, one 8- or 16-byte store).
constexpr int LEAF_ROW = 2 * P2_H;            // 2652 floats
constexpr int LEAF_CHUNKS = LEAF_ROW / 4;     // 663

// dst[i, 0:2652] = src[rows[i]] converted to DT (0 float32, 1 bfloat16, 2 float16); dst rows are
// dst_stride elements apart (columns behind 2652 are left alone).
template <int DT>
__global__ __launch_bounds__(DG_BLOCK) void gather_leaf_rows_kernel(const float* __restrict__ src,
                                                                    const int64_t* __restrict__ rows, int64_t total_rows,
                                                                    void* __restrict__ dst, int64_t dst_stride) {
  const int64_t i = blockIdx.x;
  const int64_t r = rows[i];
  if (r < 0 || r >= total_rows) return;
  const float2* s = reinterpret_cast<const float2*>(src + r * LEAF_ROW);
  for (int c = threadIdx.x; c < LEAF_CHUNKS; c += DG_BLOCK) {
    const float2 a = s[2 * c], b = s[2 * c + 1];
    if (DT == 0) {
      float2* d = reinterpret_cast<float2*>(reinterpret_cast<float*>(dst) + i * dst_stride);
      d[2 * c] = a;
      d[2 * c + 1] = b;
    } else {
      uint2* d = reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(dst) + i * dst_stride);
      d[c] = DT == 1 ? make_uint2(pack_bf16(a.x, a.y), pack_bf16(b.x, b.y)) : make_uint2(pack_f16(a.x, a.y), pack_f16(b.x, b.y));
    }
  }
}

// dst[rows[i]] = src[i, 0:2652] converted to float32; src rows are src_stride elements apart.
template <int DT>
__global__ __launch_bounds__(DG_BLOCK) void scatter_leaf_rows_kernel(const void* __restrict__ src, int64_t src_stride,
                                                                     const int64_t* __restrict__ rows, int64_t total_rows,
                                                                     float* __restrict__ dst) {
  const int64_t i = blockIdx.x;
  const int64_t r = rows[i];
  if (r < 0 || r >= total_rows) return;
  float2* d = reinterpret_cast<float2*>(dst + r * LEAF_ROW);
  for (int c = threadIdx.x; c < LEAF_CHUNKS; c += DG_BLOCK) {
    float2 a, b;
    if (DT == 0) {
      const float2* s = reinterpret_cast<const float2*>(reinterpret_cast<const float*>(src) + i * src_stride);
      a = s[2 * c];
      b = s[2 * c + 1];
    } else {
      const uint2 u = reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(src) + i * src_stride)[c];
      if (DT == 1) {
        a = make_float2(__builtin_bit_cast(float, u.x << 16), __builtin_bit_cast(float, u.x & 0xFFFF0000u));
        b = make_float2(__builtin_bit_cast(float, u.y << 16), __builtin_bit_cast(float, u.y & 0xFFFF0000u));
      } else {
        auto h = [](uint32_t v) -> float { return (float)__builtin_bit_cast(_Float16, (uint16_t)v); };
        a = make_float2(h(u.x & 0xFFFFu), h(u.x >> 16));
        b = make_float2(h(u.y & 0xFFFFu), h(u.y >> 16));
      }
    }
    d[2 * c] = a;
    d[2 * c + 1] = b;
  }
}

}  // namespace p2

extern "C" {

int p2hip_encode_context(const int64_t* to_act, const int64_t* button, const int64_t* starting_stacks,
                         const int64_t* pot, const int64_t* committed, const int64_t* actions_this_round,
                         const uint8_t* pre_chance, int pre_chance_all, const int64_t* last_board,
                         const int64_t* board, int64_t m, float* context, int64_t* board_out, void* stream) {
  if (m < 0) return P2_EINVAL;
  if (m == 0) return 0;
  if (!to_act || !button || !starting_stacks || !pot || !committed || !actions_this_round || !last_board || !board ||
      !context || !board_out)
    return P2_EINVAL;
  if (((uintptr_t)context & 15) != 0) return P2_EINVAL;
  const int64_t grid = (m + p2::DG_BLOCK - 1) / p2::DG_BLOCK;
  if (grid > 0x7FFFFFFF) return P2_EINVAL;
  hipLaunchKernelGGL(p2::encode_context_kernel, dim3((unsigned)grid), dim3(p2::DG_BLOCK), 0, (hipStream_t)stream,
                     to_act, button, starting_stacks, pot, committed, actions_this_round, pre_chance, pre_chance_all,
                     last_board, board, m, context, board_out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_bet_amounts(const int64_t* to_act, const int64_t* stacks, const int64_t* committed, const int64_t* pot,
                      int64_t m, const float* host_bins, int n_bins, int64_t* amounts, void* stream) {
  if (m < 0 || n_bins < 0 || n_bins > p2::DG_MAX_ACTIONS - 3 || (n_bins > 0 && !host_bins)) return P2_EINVAL;
  if (m == 0) return 0;
  if (!to_act || !stacks || !committed || !pot || !amounts) return P2_EINVAL;
  p2::DgBins B;
  for (int b = 0; b < p2::DG_MAX_ACTIONS - 3; ++b) B.bins[b] = b < n_bins ? host_bins[b] : 0.f;
  B.n_bins = n_bins;
  const int64_t grid = (m + p2::DG_BLOCK - 1) / p2::DG_BLOCK;
  if (grid > 0x7FFFFFFF) return P2_EINVAL;
  hipLaunchKernelGGL(p2::bet_amounts_kernel, dim3((unsigned)grid), dim3(p2::DG_BLOCK), 0, (hipStream_t)stream, to_act,
                     stacks, committed, pot, m, B, amounts);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_policy_targets(const float* policy_avg, const int64_t* rows, int64_t n_rows, const int64_t* child_offsets,
                         const int64_t* child_count, const int64_t* action_from_parent, int num_actions, float* out,
                         void* stream) {
  if (n_rows < 0 || num_actions < 1 || num_actions > p2::DG_MAX_ACTIONS) return P2_EINVAL;
  if (n_rows == 0) return 0;
  if (!policy_avg || !rows || !child_offsets || !child_count || !action_from_parent || !out) return P2_EINVAL;
  if (n_rows > 0x7FFFFFFF) return P2_EINVAL;
  if ((reinterpret_cast<uintptr_t>(policy_avg) & 7u) || (reinterpret_cast<uintptr_t>(out) & 7u)) return P2_EINVAL;
  const bool wide = (reinterpret_cast<uintptr_t>(out) & 15u) == 0;
#define P2_PT_CASE(A)                                                                                          \
  case A:                                                                                                      \
    if (wide)                                                                                                  \
      hipLaunchKernelGGL((p2::policy_targets_kernel<A, true>), dim3((unsigned)n_rows), dim3(p2::DG_BLOCK), 0,  \
                         (hipStream_t)stream, policy_avg, rows, child_offsets, child_count,                    \
                         action_from_parent, out);                                                             \
    else                                                                                                       \
      hipLaunchKernelGGL((p2::policy_targets_kernel<A, false>), dim3((unsigned)n_rows), dim3(p2::DG_BLOCK), 0, \
                         (hipStream_t)stream, policy_avg, rows, child_offsets, child_count,                    \
                         action_from_parent, out);                                                             \
    break;
  switch (num_actions) {
    P2_PT_CASE(1) P2_PT_CASE(2) P2_PT_CASE(3) P2_PT_CASE(4) P2_PT_CASE(5) P2_PT_CASE(6) P2_PT_CASE(7) P2_PT_CASE(8)
    default: return P2_EINVAL;
  }
#undef P2_PT_CASE
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_gather_leaf_rows(const float* src, const int64_t* rows, int64_t k, int64_t total_rows, void* dst, int dst_dtype,
                           int64_t dst_stride, void* stream) {
  if (k < 0 || total_rows < 0 || dst_dtype < 0 || dst_dtype > 2 || dst_stride < p2::LEAF_ROW) return P2_EINVAL;
  if (k == 0) return 0;
  if (!src || !rows || !dst || k > 0x7FFFFFFF) return P2_EINVAL;
  // 8-byte accesses on both sides: float32 rows need an even stride, 16-bit rows a multiple of four
  if (!p2_aligned8(src) || !p2_aligned8(dst) || (dst_stride % (dst_dtype == 0 ? 2 : 4)) != 0) return P2_EINVAL;
  const dim3 grid((unsigned)k), block(p2::DG_BLOCK);
  if (dst_dtype == 0)
    hipLaunchKernelGGL(p2::gather_leaf_rows_kernel<0>, grid, block, 0, (hipStream_t)stream, src, rows, total_rows, dst, dst_stride);
  else if (dst_dtype == 1)
    hipLaunchKernelGGL(p2::gather_leaf_rows_kernel<1>, grid, block, 0, (hipStream_t)stream, src, rows, total_rows, dst, dst_stride);
  else
    hipLaunchKernelGGL(p2::gather_leaf_rows_kernel<2>, grid, block, 0, (hipStream_t)stream, src, rows, total_rows, dst, dst_stride);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_scatter_leaf_rows(const void* src, int src_dtype, int64_t src_stride, const int64_t* rows, int64_t k, float* dst,
                            int64_t total_rows, void* stream) {
  if (k < 0 || total_rows < 0 || src_dtype < 0 || src_dtype > 2 || src_stride < p2::LEAF_ROW) return P2_EINVAL;
  if (k == 0) return 0;
  if (!src || !rows || !dst || k > 0x7FFFFFFF) return P2_EINVAL;
  if (!p2_aligned8(src) || !p2_aligned8(dst) || (src_stride % (src_dtype == 0 ? 2 : 4)) != 0) return P2_EINVAL;
  const dim3 grid((unsigned)k), block(p2::DG_BLOCK);
  if (src_dtype == 0)
    hipLaunchKernelGGL(p2::scatter_leaf_rows_kernel<0>, grid, block, 0, (hipStream_t)stream, src, src_stride, rows, total_rows, dst);
  else if (src_dtype == 1)
    hipLaunchKernelGGL(p2::scatter_leaf_rows_kernel<1>, grid, block, 0, (hipStream_t)stream, src, src_stride, rows, total_rows, dst);
  else
    hipLaunchKernelGGL(p2::scatter_leaf_rows_kernel<2>, grid, block, 0, (hipStream_t)stream, src, src_stride, rows, total_rows, dst);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
