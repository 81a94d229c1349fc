// Per-operation CFR kernels: one entry point per fused op of
// src/p2/search/fused_cfr_triton.py, same arithmetic order, float32.
//
// Rows are 1326 floats (5304 B, 8-byte aligned) and are moved as float2; flat
// element-wise ops run over float2 too (every tensor here has an even element
// count).  Scalars that change with the iteration number are read through
// device pointers so a captured launch sequence can be replayed for any t.
// Built with -ffp-contract=off: a*b+c stays two roundings, like the eager torch
// ops these replace.
#pragma once
#include "common.h"

namespace p2 {

constexpr int OPS_BLOCK = 256;
constexpr int OPS_WAVES = OPS_BLOCK / 64;
constexpr int OPS_PAIRS_PER_THREAD = 3;  // 3 * 256 = 768 >= 663
constexpr int FLAT_BLOCK = 256;

static inline unsigned flat_grid(int64_t npairs) {
  int64_t g = (npairs + FLAT_BLOCK - 1) / FLAT_BLOCK;
  // One pair per lane up to 2^30 workgroups: workgroups start in address order, which keeps the
  // DRAM accesses of the whole chip sequential in time; a capped grid with a long stride between a
  // lane's iterations measured 20 % slower (4.97 vs 5.92 TB/s on the DCFR update).
  const int64_t cap = (int64_t)1 << 30;
  return (unsigned)(g < cap ? g : cap);
}

#define P2_FLAT_LOOP(i, npairs) \
  for (int64_t i = (int64_t)blockIdx.x * FLAT_BLOCK + threadIdx.x; i < (npairs); i += (int64_t)gridDim.x * FLAT_BLOCK)

#define P2_ROW_LOOP(i) for (int i = threadIdx.x; i < P2_HPAIRS; i += OPS_BLOCK)

// K1 -- fused_cfr_triton.py:71-120
__global__ __launch_bounds__(FLAT_BLOCK) void dcfr_update_kernel(
    const float2* __restrict__ regrets, float2* __restrict__ cumul, float2* __restrict__ weight,
    float2* __restrict__ pos_out, const float* __restrict__ ta_num, const float* __restrict__ tb_num,
    const float* __restrict__ ta_den, const float* __restrict__ tb_den, int64_t npairs, int apply_dcfr,
    int cfr_plus) {
  float an = 1.f, bn = 1.f, ad = 1.f, bd = 1.f;
  if (apply_dcfr) { an = *ta_num; bn = *tb_num; ad = *ta_den; bd = *tb_den; }
  P2_FLAT_LOOP(i, npairs) {
    const float2 r = regrets[i];
    float2 c = cumul[i], w = weight[i];
    float cc[2] = {c.x, c.y}, ww[2] = {w.x, w.y};
    const float rr[2] = {r.x, r.y};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      if (apply_dcfr) {
        const bool positive = cc[k] > 0.f;
        const float num = positive ? an : bn, den = positive ? ad : bd;
        cc[k] = cc[k] * num;
        cc[k] = cc[k] / den;
        ww[k] = ww[k] * num;
        ww[k] = ww[k] / den;
      }
      ww[k] = ww[k] + 1.0f;
      cc[k] = cc[k] + rr[k];
      if (cfr_plus) cc[k] = fmaxf(cc[k], 0.f);
    }
    cumul[i] = make_float2(cc[0], cc[1]);
    weight[i] = make_float2(ww[0], ww[1]);
    if (pos_out) pos_out[i] = make_float2(fmaxf(cc[0], 0.f), fmaxf(cc[1], 0.f));
  }
}

// K2 -- fused_cfr_triton.py:245-283.  target row r uses mask / fallback row r / stride.  A workgroup takes
// two rows: both are requested before either is used and their sums share one block reduction (a row's
// own sum is formed exactly as when it had the workgroup to itself).
constexpr int K2_ROWS = 2;
__global__ __launch_bounds__(OPS_BLOCK) void block_normalize_kernel(float* __restrict__ target,
                                                                     const uint8_t* __restrict__ allowed,
                                                                     const float* __restrict__ allowed_prob,
                                                                     int64_t rows, int stride, float eps) {
  __shared__ float red[K2_ROWS][OPS_WAVES];
  const int64_t row0 = (int64_t)blockIdx.x * K2_ROWS;
  float2 x[K2_ROWS][OPS_PAIRS_PER_THREAD];
  uchar2 m[K2_ROWS][OPS_PAIRS_PER_THREAD];
#pragma unroll
  for (int r = 0; r < K2_ROWS; ++r) {
    const int64_t row = row0 + r < rows ? row0 + r : rows - 1;   // past the end: the last row again, not stored
    const float2* t2 = p2_row2(target, row);
    const uchar2* m2 = reinterpret_cast<const uchar2*>(allowed + (row / stride) * P2_H);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      const int ic = i < P2_HPAIRS ? i : 0;
      x[r][j] = t2[ic];
      m[r][j] = m2[ic];
    }
  }
  float local[K2_ROWS];
#pragma unroll
  for (int r = 0; r < K2_ROWS; ++r) {
    local[r] = 0.f;
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      const bool in = i < P2_HPAIRS;
      x[r][j].x = (in && m[r][j].x) ? x[r][j].x : 0.f;
      x[r][j].y = (in && m[r][j].y) ? x[r][j].y : 0.f;
      if (in) local[r] += x[r][j].x + x[r][j].y;
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int r = 0; r < K2_ROWS; ++r) {
    const float w = p2_wave_sum(local[r]);
    if (lane == 0) red[r][wave] = w;
  }
  p2_sync_lds();
#pragma unroll
  for (int r = 0; r < K2_ROWS; ++r) {
    if (row0 + r >= rows) break;
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < OPS_WAVES; ++w) total += red[r][w];
    float2* t2 = p2_row2(target, row0 + r);
    const float2* f2 = p2_row2(allowed_prob, (row0 + r) / stride);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      if (i < P2_HPAIRS) t2[i] = total > eps ? make_float2(x[r][j].x / total, x[r][j].y / total) : f2[i];
    }
  }
}

// K3 -- fused_cfr_triton.py:345-366
__global__ __launch_bounds__(FLAT_BLOCK) void regret_matching_divide_kernel(
    const float2* __restrict__ pos, const float2* __restrict__ den, const float2* __restrict__ fallback,
    float2* __restrict__ out, int64_t npairs, float eps) {
  P2_FLAT_LOOP(i, npairs) {
    const float2 p = pos[i], d = den[i], f = fallback[i];
    float2 o;
    o.x = d.x > eps ? p.x / fmaxf(d.x, eps) : f.x;
    o.y = d.y > eps ? p.y / fmaxf(d.y, eps) : f.y;
    out[i] = o;
  }
}

// K4 -- fused_cfr_triton.py:409-435; two workgroups per row, neighbours in the grid: together they read and write the
// row's two players as one contiguous run
__global__ __launch_bounds__(OPS_BLOCK) void weight_child_values_kernel(
    const float* __restrict__ values, const int64_t* __restrict__ prev_actor, const float* __restrict__ pol_hero,
    const float* __restrict__ pol_opp, float* __restrict__ out) {
  const int64_t m = blockIdx.x >> 1;
  const int p = blockIdx.x & 1;
  const bool hero = (int64_t)p == prev_actor[m];
  const float2* v2 = p2_row2(values, m * 2 + p);
  const float2* w2 = p2_row2(hero ? pol_hero : pol_opp, m);
  float2* o2 = p2_row2(out, m * 2 + p);
  P2_ROW_LOOP(i) {
    const float2 v = v2[i], w = w2[i];
    o2[i] = make_float2(v.x * w.x, v.y * w.y);
  }
}

// K5 -- fused_cfr_triton.py:487-506
__global__ __launch_bounds__(FLAT_BLOCK) void update_average_values_kernel(
    float2* __restrict__ avg, const float2* __restrict__ latest, const float* __restrict__ old_p,
    const float* __restrict__ new_p, const float* __restrict__ inv_p, int64_t npairs) {
  const float o = *old_p, n = *new_p, inv = *inv_p;
  P2_FLAT_LOOP(i, npairs) {
    const float2 a = avg[i], v = latest[i];
    avg[i] = make_float2((a.x * o + v.x * n) * inv, (a.y * o + v.y * n) * inv);
  }
}

// K6 -- fused_cfr_triton.py:571-620; one workgroup per node
__global__ __launch_bounds__(OPS_BLOCK) void avg_values_zero_sum_kernel(
    float* __restrict__ avg, const float* __restrict__ latest, const float* __restrict__ beliefs,
    const uint8_t* __restrict__ ignore_mask, const float* __restrict__ old_p, const float* __restrict__ new_p,
    const float* __restrict__ inv_p, int enforce_zs) {
  __shared__ float red[OPS_WAVES];
  const int64_t n = blockIdx.x;
  const float o = *old_p, nw = *new_p, inv = *inv_p;
  float2 v[2][OPS_PAIRS_PER_THREAD];
  float local = 0.f;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const float2* a2 = p2_row2(avg, n * 2 + p);
    const float2* l2 = p2_row2(latest, n * 2 + p);
    const float2* b2 = p2_row2(beliefs, n * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      v[p][j] = make_float2(0.f, 0.f);
      if (i < P2_HPAIRS) {
        const float2 a = a2[i], l = l2[i];
        v[p][j] = make_float2((a.x * o + l.x * nw) * inv, (a.y * o + l.y * nw) * inv);
        if (enforce_zs) {
          const float2 b = b2[i];
          local += v[p][j].x * b.x + v[p][j].y * b.y;
        }
      }
    }
  }
  float s = 0.f;
  if (enforce_zs) {
    s = 0.5f * p2_block_sum<OPS_WAVES>(local, red);
    if (ignore_mask && ignore_mask[n]) s = 0.f;
  }
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    float2* a2 = p2_row2(avg, n * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      if (i < P2_HPAIRS) a2[i] = make_float2(v[p][j].x - s, v[p][j].y - s);
    }
  }
}

// K7 -- fused_cfr_triton.py:678-709; one workgroup per child row c = blockIdx.x + bottom
__global__ __launch_bounds__(OPS_BLOCK) void regret_tail_kernel(
    const float* __restrict__ achieved, const float* __restrict__ actor_values, const float* __restrict__ src_w,
    const int64_t* __restrict__ parent_index, const int64_t* __restrict__ prev_actor, float* __restrict__ regrets,
    int64_t bottom) {
  const int64_t c = blockIdx.x + bottom;
  const int64_t parent = parent_index[c], pa = prev_actor[c];
  const float2* e2 = p2_row2(actor_values, parent);
  const float2* w2 = p2_row2(src_w, parent);
  const float2* a2 = p2_row2(achieved, c * 2 + pa);
  float2* o2 = p2_row2(regrets, c);
  P2_ROW_LOOP(i) {
    const float2 e = e2[i], w = w2[i], a = a2[i];
    o2[i] = make_float2(w.x * (a.x - e.x), w.y * (a.y - e.y));
  }
}

// K8 -- fused_cfr_triton.py:776-820
__global__ __launch_bounds__(OPS_BLOCK) void average_policy_mix_kernel(
    const float* __restrict__ reach, const float* __restrict__ reach_avg, const float* __restrict__ policy,
    float* __restrict__ policy_avg, const int64_t* __restrict__ to_act, const int64_t* __restrict__ parent_index,
    const float* __restrict__ old_p, const float* __restrict__ new_p, const float* __restrict__ tot_p,
    int64_t bottom, float eps) {
  const int64_t c = blockIdx.x + bottom;
  const int64_t parent = parent_index[c], actor = to_act[parent];
  const float o = *old_p, n = *new_p, tot = *tot_p;
  const float2* r2 = p2_row2(reach, parent * 2 + actor);
  const float2* ra2 = p2_row2(reach_avg, parent * 2 + actor);
  const float2* p2v = p2_row2(policy, c);
  float2* av2 = p2_row2(policy_avg, c);
  P2_ROW_LOOP(i) {
    const float2 r = r2[i], ra = ra2[i], cur = p2v[i], avg = av2[i];
    float out[2];
    const float rr[2] = {r.x, r.y}, rra[2] = {ra.x, ra.y}, cc[2] = {cur.x, cur.y}, aa[2] = {avg.x, avg.y};
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const float reach_a = rra[k] * o, reach_n = rr[k] * n;
      const float num = reach_a * aa[k] + reach_n * cc[k];
      const float den = reach_a + reach_n;
      const float unweighted = (o * aa[k] + n * cc[k]) / tot;
      out[k] = den > eps ? num / den : unweighted;
    }
    av2[i] = make_float2(out[0], out[1]);
  }
}

// K10a / K11 -- fused_cfr_triton.py:1167-1238; one workgroup per parent.
// broadcast == 0: out[p] = sum over children; broadcast != 0: every child row gets the sum.
__global__ __launch_bounds__(OPS_BLOCK) void parent_sum_kernel(const float* __restrict__ values,
                                                                const int64_t* __restrict__ child_offsets,
                                                                const int64_t* __restrict__ child_count,
                                                                float* __restrict__ out, int broadcast,
                                                                int64_t out_offset) {
  const int64_t p = blockIdx.x;
  const int64_t first = child_offsets[p];
  const int count = (int)child_count[p];
  // a lane's three pairs of every child row; the rows of two children are requested before either is added
  // (children are still added in ascending order)
  float2 acc[OPS_PAIRS_PER_THREAD];
#pragma unroll
  for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) acc[j] = make_float2(0.f, 0.f);
  auto fetch = [&](int k, float2 (&v)[OPS_PAIRS_PER_THREAD]) {
    const float2* row = p2_row2(values, first + k);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      v[j] = row[i < P2_HPAIRS ? i : 0];
    }
  };
  int k = 0;
  for (; k + 2 <= count; k += 2) {
    float2 a[OPS_PAIRS_PER_THREAD], b[OPS_PAIRS_PER_THREAD];
    fetch(k, a);
    fetch(k + 1, b);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      acc[j].x += a[j].x; acc[j].y += a[j].y;
      acc[j].x += b[j].x; acc[j].y += b[j].y;
    }
  }
  if (k < count) {
    float2 a[OPS_PAIRS_PER_THREAD];
    fetch(k, a);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) { acc[j].x += a[j].x; acc[j].y += a[j].y; }
  }
#pragma unroll
  for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
    const int i = threadIdx.x + j * OPS_BLOCK;
    if (i >= P2_HPAIRS) continue;
    if (broadcast) {
      for (int c = 0; c < count; ++c) p2_row2(out, first + c - out_offset)[i] = acc[j];
    } else {
      p2_row2(out, p)[i] = acc[j];
    }
  }
}

// K10b -- fused_cfr_triton.py:1240-1276; one workgroup per child row
// (`out` may be the same buffer as `pos` or `fallback`: element-wise in place)
__global__ __launch_bounds__(OPS_BLOCK) void divide_by_parent_sum_kernel(
    const float* pos, const float* fallback, const float* __restrict__ parent_sum,
    const int64_t* __restrict__ parent_index, float* out, float eps) {
  const int64_t c = blockIdx.x;
  const int64_t parent = parent_index[c];
  const float2* p2v = p2_row2(pos, c);
  const float2* f2 = p2_row2(fallback, c);
  const float2* d2 = p2_row2(parent_sum, parent);
  float2* o2 = p2_row2(out, c);
  P2_ROW_LOOP(i) {
    const float2 p = p2v[i], f = f2[i], d = d2[i];
    float2 o;
    o.x = d.x > eps ? p.x / fmaxf(d.x, eps) : f.x;
    o.y = d.y > eps ? p.y / fmaxf(d.y, eps) : f.y;
    o2[i] = o;
  }
}

// K13 -- fused_cfr_triton.py:1612-1630
__global__ __launch_bounds__(FLAT_BLOCK) void model_values_mix_kernel(
    const float2* __restrict__ h, const float2* __restrict__ l, float2* __restrict__ out,
    const float* __restrict__ onon_p, const float* __restrict__ oon_p, int64_t npairs) {
  const float onon = *onon_p, oon = *oon_p;
  P2_FLAT_LOOP(i, npairs) {
    const float2 a = h[i], b = l[i];
    out[i] = make_float2(onon * a.x - oon * b.x, onon * a.y - oon * b.y);
  }
}

// K13 zero-sum variant -- fused_cfr_triton.py:1691-1736
__global__ __launch_bounds__(OPS_BLOCK) void model_values_mix_zs_kernel(
    const float* __restrict__ h, const float* __restrict__ l, const float* __restrict__ beliefs,
    float* __restrict__ out, const float* __restrict__ onon_p, const float* __restrict__ oon_p, int enforce_zs) {
  __shared__ float red[OPS_WAVES];
  const int64_t m = blockIdx.x;
  const float onon = *onon_p, oon = *oon_p;
  float2 u[2][OPS_PAIRS_PER_THREAD];
  float local = 0.f;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const float2* h2 = p2_row2(h, m * 2 + p);
    const float2* l2 = p2_row2(l, m * 2 + p);
    const float2* b2 = p2_row2(beliefs, m * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      u[p][j] = make_float2(0.f, 0.f);
      if (i < P2_HPAIRS) {
        const float2 a = h2[i], b = l2[i];
        u[p][j] = make_float2(a.x * onon - b.x * oon, a.y * onon - b.y * oon);
        if (enforce_zs) {
          const float2 w = b2[i];
          local += u[p][j].x * w.x + u[p][j].y * w.y;
        }
      }
    }
  }
  float s = 0.f;
  if (enforce_zs) s = 0.5f * p2_block_sum<OPS_WAVES>(local, red);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    float2* o2 = p2_row2(out, m * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      if (i < P2_HPAIRS) o2[i] = make_float2(u[p][j].x - s, u[p][j].y - s);
    }
  }
}

// K14 -- fused_cfr_triton.py:1787-1835; two workgroups per parent (one per player), neighbours in the grid
__global__ __launch_bounds__(OPS_BLOCK) void weighted_parent_sum_kernel(
    float* __restrict__ values, const int64_t* __restrict__ prev_actor, const float* __restrict__ pol_hero,
    const float* __restrict__ pol_opp, const int64_t* __restrict__ child_offsets,
    const int64_t* __restrict__ child_count, int64_t parent_base) {
  const int64_t p = blockIdx.x >> 1;
  const int player = blockIdx.x & 1;
  const int64_t first = child_offsets[p];
  const int count = (int)child_count[p];
  if (count == 0) return;  // leaf at an intermediate depth keeps its value
  float2* o2 = p2_row2(values, (parent_base + p) * 2 + player);
  // a lane's three pairs of every child; value and policy rows of two children are requested before
  // either is used (children are still added in ascending order)
  float2 acc[OPS_PAIRS_PER_THREAD];
#pragma unroll
  for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) acc[j] = make_float2(0.f, 0.f);
  auto fetch = [&](int k, float2 (&v)[OPS_PAIRS_PER_THREAD], float2 (&w)[OPS_PAIRS_PER_THREAD]) {
    const int64_t child = first + k;
    const float* pol = (prev_actor[child] == (int64_t)player) ? pol_hero : pol_opp;
    const float2* wr = p2_row2(pol, child);
    const float2* vr = p2_row2(values, child * 2 + player);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      w[j] = wr[i < P2_HPAIRS ? i : 0];
      v[j] = vr[i < P2_HPAIRS ? i : 0];
    }
  };
  int k = 0;
  for (; k + 2 <= count; k += 2) {
    float2 va[OPS_PAIRS_PER_THREAD], wa[OPS_PAIRS_PER_THREAD], vb[OPS_PAIRS_PER_THREAD], wb[OPS_PAIRS_PER_THREAD];
    fetch(k, va, wa);
    fetch(k + 1, vb, wb);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      acc[j].x += va[j].x * wa[j].x; acc[j].y += va[j].y * wa[j].y;
      acc[j].x += vb[j].x * wb[j].x; acc[j].y += vb[j].y * wb[j].y;
    }
  }
  if (k < count) {
    float2 va[OPS_PAIRS_PER_THREAD], wa[OPS_PAIRS_PER_THREAD];
    fetch(k, va, wa);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) { acc[j].x += va[j].x * wa[j].x; acc[j].y += va[j].y * wa[j].y; }
  }
#pragma unroll
  for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
    const int i = threadIdx.x + j * OPS_BLOCK;
    if (i < P2_HPAIRS) o2[i] = acc[j];
  }
}

// K15 -- fused_cfr_triton.py:1900-1941; one workgroup per child row c = blockIdx.x + start
__global__ __launch_bounds__(OPS_BLOCK) void reach_weights_kernel(float* __restrict__ reach,
                                                                   const float* __restrict__ policy,
                                                                   const uint8_t* __restrict__ allowed,
                                                                   const int64_t* __restrict__ parent_index,
                                                                   const int64_t* __restrict__ prev_actor,
                                                                   int64_t start) {
  const int64_t c = blockIdx.x + start;
  const int64_t parent = parent_index[c], pa = prev_actor[c];
  const float2* pol2 = p2_row2(policy, c);
  const uchar2* m2 = reinterpret_cast<const uchar2*>(allowed + c * P2_H);
  const float2* s0 = p2_row2(reach, parent * 2);
  const float2* s1 = p2_row2(reach, parent * 2 + 1);
  float2* d0 = p2_row2(reach, c * 2);
  float2* d1 = p2_row2(reach, c * 2 + 1);
  P2_ROW_LOOP(i) {
    const float2 pol = pol2[i];
    const uchar2 al = m2[i];
    float2 v0 = s0[i], v1 = s1[i];
    if (pa == 0) { v0.x *= pol.x; v0.y *= pol.y; } else { v1.x *= pol.x; v1.y *= pol.y; }
    d0[i] = make_float2(al.x ? v0.x : 0.f, al.y ? v0.y : 0.f);
    d1[i] = make_float2(al.x ? v1.x : 0.f, al.y ? v1.y : 0.f);
  }
}

// K16 -- fused_cfr_triton.py:1996-2036; one workgroup per row below the roots, both players: the four input
// rows are requested together and the two sums share one block reduction.
__global__ __launch_bounds__(OPS_BLOCK) void deep_beliefs_kernel(const float* __restrict__ root_beliefs,
                                                                  const float* __restrict__ reach,
                                                                  const float* __restrict__ allowed_prob,
                                                                  const int64_t* __restrict__ root_index,
                                                                  float* __restrict__ out, int64_t n_roots,
                                                                  float eps) {
  __shared__ float red[2][OPS_WAVES];
  const int64_t i_row = blockIdx.x + n_roots;
  const int64_t root = root_index[i_row];
  float2 v[2][OPS_PAIRS_PER_THREAD];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    const float2* rb2 = p2_row2(root_beliefs, root * 2 + p);
    const float2* rw2 = p2_row2(reach, i_row * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      const int ic = i < P2_HPAIRS ? i : 0;
      const float2 a = rb2[ic], b = rw2[ic];
      v[p][j] = i < P2_HPAIRS ? make_float2(a.x * b.x, a.y * b.y) : make_float2(0.f, 0.f);
    }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    float local = 0.f;
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j)
      if (threadIdx.x + j * OPS_BLOCK < P2_HPAIRS) local += v[p][j].x + v[p][j].y;
    const float w = p2_wave_sum(local);
    if (lane == 0) red[p][wave] = w;
  }
  p2_sync_lds();
  const float2* f2 = p2_row2(allowed_prob, i_row);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < OPS_WAVES; ++w) total += red[p][w];
    float2* o2 = p2_row2(out, i_row * 2 + p);
#pragma unroll
    for (int j = 0; j < OPS_PAIRS_PER_THREAD; ++j) {
      const int i = threadIdx.x + j * OPS_BLOCK;
      if (i < P2_HPAIRS) o2[i] = total > eps ? make_float2(v[p][j].x / total, v[p][j].y / total) : f2[i];
    }
  }
}

// policy_probs_sample <- where(t_sample == t, policy_probs, policy_probs_sample); one workgroup per row
__global__ __launch_bounds__(OPS_BLOCK) void sample_snapshot_kernel(const float* __restrict__ policy,
                                                                     float* __restrict__ sample,
                                                                     const int64_t* __restrict__ t_sample,
                                                                     const int64_t* __restrict__ t_now) {
  const int64_t r = blockIdx.x;
  if (t_sample[r] != *t_now) return;
  const float2* s2 = p2_row2(policy, r);
  float2* d2 = p2_row2(sample, r);
  P2_ROW_LOOP(i) d2[i] = s2[i];
}

}  // namespace p2

#define P2_ST ((hipStream_t)stream)
#define P2_REQ(cond) do { if (!(cond)) return P2_EINVAL; } while (0)

extern "C" {

int p2hip_dcfr_update(float* cumulative_regrets, float* regret_weight_sums, const float* regrets,
                      const float* t_alpha_num, const float* t_beta_num, const float* t_alpha_den,
                      const float* t_beta_den, int64_t n, int apply_dcfr, int cfr_plus, float* positive_out,
                      void* stream) {
  P2_REQ(n >= 0 && (n & 1) == 0);
  if (n == 0) return 0;
  P2_REQ(cumulative_regrets && regret_weight_sums && regrets);
  P2_REQ(!apply_dcfr || (t_alpha_num && t_beta_num && t_alpha_den && t_beta_den));
  P2_REQ(p2_aligned8(cumulative_regrets) && p2_aligned8(regret_weight_sums) && p2_aligned8(regrets) &&
         p2_aligned8(positive_out));
  const int64_t np = n / 2;
  hipLaunchKernelGGL(p2::dcfr_update_kernel, dim3(p2::flat_grid(np)), dim3(p2::FLAT_BLOCK), 0, P2_ST,
                     (const float2*)regrets, (float2*)cumulative_regrets, (float2*)regret_weight_sums,
                     (float2*)positive_out, t_alpha_num, t_beta_num, t_alpha_den, t_beta_den, np, apply_dcfr,
                     cfr_plus);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_block_and_normalize(float* target, const uint8_t* allowed, const float* allowed_prob, int64_t rows,
                              int players_per_row, float eps, void* stream) {
  P2_REQ(rows >= 0 && players_per_row >= 1);
  if (rows == 0) return 0;
  P2_REQ(target && allowed && allowed_prob && p2_aligned8(target) && p2_aligned8(allowed_prob) &&
         (reinterpret_cast<uintptr_t>(allowed) & 1u) == 0);
  hipLaunchKernelGGL(p2::block_normalize_kernel, dim3((unsigned)((rows + p2::K2_ROWS - 1) / p2::K2_ROWS)),
                     dim3(p2::OPS_BLOCK), 0, P2_ST, target, allowed, allowed_prob, rows, players_per_row, eps);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_regret_matching_divide(const float* positive, const float* denom, const float* fallback, float* out,
                                 int64_t n, float eps, void* stream) {
  P2_REQ(n >= 0 && (n & 1) == 0);
  if (n == 0) return 0;
  P2_REQ(positive && denom && fallback && out);
  P2_REQ(p2_aligned8(positive) && p2_aligned8(denom) && p2_aligned8(fallback) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::regret_matching_divide_kernel, dim3(p2::flat_grid(n / 2)), dim3(p2::FLAT_BLOCK), 0, P2_ST,
                     (const float2*)positive, (const float2*)denom, (const float2*)fallback, (float2*)out, n / 2,
                     eps);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_weight_child_values(const float* values, const int64_t* prev_actor, const float* policy_hero,
                              const float* policy_opp, float* out, int64_t m, void* stream) {
  P2_REQ(m >= 0);
  if (m == 0) return 0;
  P2_REQ(values && prev_actor && policy_hero && policy_opp && out);
  P2_REQ(p2_aligned8(values) && p2_aligned8(policy_hero) && p2_aligned8(policy_opp) && p2_aligned8(out));
  P2_REQ(m <= 0x3FFFFFFF);
  hipLaunchKernelGGL(p2::weight_child_values_kernel, dim3((unsigned)(2 * m)), dim3(p2::OPS_BLOCK), 0, P2_ST, values,
                     prev_actor, policy_hero, policy_opp, out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_update_average_values(float* values_avg, const float* latest, const float* old_w, const float* new_w,
                                const float* inv_total, int64_t n, void* stream) {
  P2_REQ(n >= 0 && (n & 1) == 0);
  if (n == 0) return 0;
  P2_REQ(values_avg && latest && old_w && new_w && inv_total && p2_aligned8(values_avg) && p2_aligned8(latest));
  hipLaunchKernelGGL(p2::update_average_values_kernel, dim3(p2::flat_grid(n / 2)), dim3(p2::FLAT_BLOCK), 0, P2_ST,
                     (float2*)values_avg, (const float2*)latest, old_w, new_w, inv_total, n / 2);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_avg_values_zero_sum(float* values_avg, const float* latest, const float* beliefs,
                              const uint8_t* ignore_mask, const float* old_w, const float* new_w,
                              const float* inv_total, int64_t nodes, int enforce_zero_sum, void* stream) {
  P2_REQ(nodes >= 0);
  if (nodes == 0) return 0;
  P2_REQ(values_avg && latest && beliefs && old_w && new_w && inv_total);
  P2_REQ(p2_aligned8(values_avg) && p2_aligned8(latest) && p2_aligned8(beliefs));
  hipLaunchKernelGGL(p2::avg_values_zero_sum_kernel, dim3((unsigned)nodes), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     values_avg, latest, beliefs, ignore_mask, old_w, new_w, inv_total, enforce_zero_sum);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_regret_tail(float* regrets, const float* values_achieved, const float* actor_values,
                      const float* src_weights, const int64_t* parent_index, const int64_t* prev_actor,
                      int64_t bottom, int64_t total, void* stream) {
  P2_REQ(bottom >= 0 && total >= bottom);
  if (total == bottom) return 0;
  P2_REQ(regrets && values_achieved && actor_values && src_weights && parent_index && prev_actor);
  P2_REQ(p2_aligned8(regrets) && p2_aligned8(values_achieved) && p2_aligned8(actor_values) &&
         p2_aligned8(src_weights));
  hipLaunchKernelGGL(p2::regret_tail_kernel, dim3((unsigned)(total - bottom)), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     values_achieved, actor_values, src_weights, parent_index, prev_actor, regrets, bottom);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_average_policy_mix(float* policy_probs_avg, const float* policy_probs, const float* self_reach,
                             const float* self_reach_avg, const int64_t* to_act, const int64_t* parent_index,
                             const float* old_w, const float* new_w, const float* total_w, int64_t bottom,
                             int64_t total, float eps, void* stream) {
  P2_REQ(bottom >= 0 && total >= bottom);
  if (total == bottom) return 0;
  P2_REQ(policy_probs_avg && policy_probs && self_reach && self_reach_avg && to_act && parent_index && old_w &&
         new_w && total_w);
  P2_REQ(p2_aligned8(policy_probs_avg) && p2_aligned8(policy_probs) && p2_aligned8(self_reach) &&
         p2_aligned8(self_reach_avg));
  hipLaunchKernelGGL(p2::average_policy_mix_kernel, dim3((unsigned)(total - bottom)), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     self_reach, self_reach_avg, policy_probs, policy_probs_avg, to_act, parent_index, old_w,
                     new_w, total_w, bottom, eps);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_parent_sum(const float* values, const int64_t* child_offsets, const int64_t* child_count,
                     int64_t num_parents, float* out, void* stream) {
  P2_REQ(num_parents >= 0);
  if (num_parents == 0) return 0;
  P2_REQ(values && child_offsets && child_count && out && p2_aligned8(values) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::parent_sum_kernel, dim3((unsigned)num_parents), dim3(p2::OPS_BLOCK), 0, P2_ST, values,
                     child_offsets, child_count, out, 0, (int64_t)0);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_sibling_sum(const float* values, const int64_t* child_offsets, const int64_t* child_count,
                      int64_t num_parents, int64_t bottom, float* out, void* stream) {
  P2_REQ(num_parents >= 0);
  if (num_parents == 0) return 0;
  P2_REQ(values && child_offsets && child_count && out && p2_aligned8(values) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::parent_sum_kernel, dim3((unsigned)num_parents), dim3(p2::OPS_BLOCK), 0, P2_ST, values,
                     child_offsets, child_count, out, 1, bottom);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_divide_by_parent_sum(const float* pos, const float* fallback, const float* parent_sum,
                               const int64_t* parent_index, float* out, int64_t num_children, float eps,
                               void* stream) {
  P2_REQ(num_children >= 0);
  if (num_children == 0) return 0;
  P2_REQ(pos && fallback && parent_sum && parent_index && out);
  P2_REQ(p2_aligned8(pos) && p2_aligned8(fallback) && p2_aligned8(parent_sum) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::divide_by_parent_sum_kernel, dim3((unsigned)num_children), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     pos, fallback, parent_sum, parent_index, out, eps);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_model_values_mix(const float* hand_values, const float* last_values, const float* onon,
                           const float* oon, float* out, int64_t n, void* stream) {
  P2_REQ(n >= 0 && (n & 1) == 0);
  if (n == 0) return 0;
  P2_REQ(hand_values && last_values && onon && oon && out);
  P2_REQ(p2_aligned8(hand_values) && p2_aligned8(last_values) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::model_values_mix_kernel, dim3(p2::flat_grid(n / 2)), dim3(p2::FLAT_BLOCK), 0, P2_ST,
                     (const float2*)hand_values, (const float2*)last_values, (float2*)out, onon, oon, n / 2);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_model_values_mix_zero_sum(const float* hand_values, const float* last_values, const float* beliefs,
                                    const float* onon, const float* oon, float* out, int64_t rows,
                                    int enforce_zero_sum, void* stream) {
  P2_REQ(rows >= 0);
  if (rows == 0) return 0;
  P2_REQ(hand_values && last_values && beliefs && onon && oon && out);
  P2_REQ(p2_aligned8(hand_values) && p2_aligned8(last_values) && p2_aligned8(beliefs) && p2_aligned8(out));
  hipLaunchKernelGGL(p2::model_values_mix_zs_kernel, dim3((unsigned)rows), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     hand_values, last_values, beliefs, out, onon, oon, enforce_zero_sum);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_weighted_parent_sum(float* values, const int64_t* prev_actor, const float* policy_hero,
                              const float* policy_opp, const int64_t* child_offsets, const int64_t* child_count,
                              int64_t num_parents, int64_t parent_base, void* stream) {
  P2_REQ(num_parents >= 0 && parent_base >= 0);
  if (num_parents == 0) return 0;
  P2_REQ(values && prev_actor && policy_hero && policy_opp && child_offsets && child_count);
  P2_REQ(p2_aligned8(values) && p2_aligned8(policy_hero) && p2_aligned8(policy_opp));
  P2_REQ(num_parents <= 0x3FFFFFFF);
  hipLaunchKernelGGL(p2::weighted_parent_sum_kernel, dim3((unsigned)(2 * num_parents)), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     values, prev_actor, policy_hero, policy_opp, child_offsets, child_count, parent_base);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_reach_weights_depth(float* reach, const float* policy, const uint8_t* allowed_mask,
                              const int64_t* parent_index, const int64_t* prev_actor, int64_t start, int64_t end,
                              void* stream) {
  P2_REQ(start >= 0);
  if (end <= start) return 0;
  P2_REQ(reach && policy && allowed_mask && parent_index && prev_actor);
  P2_REQ(p2_aligned8(reach) && p2_aligned8(policy) && (reinterpret_cast<uintptr_t>(allowed_mask) & 1u) == 0);
  hipLaunchKernelGGL(p2::reach_weights_kernel, dim3((unsigned)(end - start)), dim3(p2::OPS_BLOCK), 0, P2_ST, reach,
                     policy, allowed_mask, parent_index, prev_actor, start);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_deep_beliefs(float* out, const float* root_beliefs, const float* reach, const float* allowed_prob,
                       const int64_t* root_index, int64_t n_roots, int64_t total, float eps, void* stream) {
  P2_REQ(n_roots >= 0 && total >= 0);
  if (total <= n_roots) return 0;
  P2_REQ(out && root_beliefs && reach && allowed_prob && root_index);
  P2_REQ(p2_aligned8(out) && p2_aligned8(root_beliefs) && p2_aligned8(reach) && p2_aligned8(allowed_prob));
  hipLaunchKernelGGL(p2::deep_beliefs_kernel, dim3((unsigned)(total - n_roots)), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     root_beliefs, reach, allowed_prob, root_index, out, n_roots, eps);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_sample_snapshot(const float* policy_probs, float* policy_probs_sample, const int64_t* t_sample,
                          const int64_t* t_now, int64_t total, void* stream) {
  P2_REQ(total >= 0);
  if (total == 0) return 0;
  P2_REQ(policy_probs && policy_probs_sample && t_sample && t_now);
  P2_REQ(p2_aligned8(policy_probs) && p2_aligned8(policy_probs_sample));
  hipLaunchKernelGGL(p2::sample_snapshot_kernel, dim3((unsigned)total), dim3(p2::OPS_BLOCK), 0, P2_ST,
                     policy_probs, policy_probs_sample, t_sample, t_now);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
