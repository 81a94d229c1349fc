// One kernel = one whole CFR iteration.  One workgroup owns one root's subtree and
// walks it three times:
//   sweep 1 (families independent): opponent unblocked mass at the parent, instantaneous
//            regrets, DCFR discount + accumulate, regret matching -> policy_probs
//   sweep 2 (top-down): reach, beliefs, average-policy mix + renormalise, reach_avg,
//            beliefs_avg
//   sweep 3: showdown leaves first (their values depend only on the new beliefs), then
//            bottom-up: opponent-conditioned policy, value backup, average values
// which is the order of FusedSparseCFREvaluator.cfr_iteration
// (src/p2/search/fused_sparse_cfr_evaluator.py:478-533) with every per-op launch of
// src/p2/search/fused_cfr_triton.py folded in.  `phases` lets the host split the
// iteration where the leaf network has to run (after sweep 2).
//
// A "family" is a parent and its contiguous child rows.  Every thread owns the same
// three float2 pairs (six hands) of every 1326-vector for the whole kernel, so all
// per-hand work is register-to-register; only sums over hands go through LDS.
#include "common.h"
#include "unblocked.hip"
#include "showdown.hip"
#include "../../include/p2hip.h"

namespace p2 {

constexpr int IT_BLOCK = 256;
constexpr int IT_WAVES = IT_BLOCK / 64;
constexpr int IT_PPT = 3;  // pairs per thread: 3 * 256 = 768 >= 663
// Tuning of the iteration kernel per instantiation (MAXC = most children of a parent):
//   waves per SIMD the register budget is capped for, and how many rows are requested together —
//   SB parents staged for the card sums, G1 children of a family in the regret sweep, G3 children of a
//   family in the value sweep.  Up to five children everything fits 168 registers without spilling
//   (a single spill reload costs more than it saves: it waits for every outstanding store); with up to
//   eight the kernel takes 256 registers and two workgroups per CU instead.
template <int MAXC>
struct ItTune {
  static constexpr int min_waves = MAXC <= 5 ? 3 : 2;
  static constexpr int SB = 4;
  static constexpr int G1 = MAXC <= 5 ? 2 : 4;
  static constexpr int G3 = MAXC <= 5 ? 1 : 2;
};
static_assert(IT_BLOCK == UB_BLOCK && IT_BLOCK == SD_BLOCK, "shared helpers assume one block size");

constexpr uint8_t NODE_SHOWDOWN = 1;  // river showdown leaf: value from the showdown evaluator
constexpr uint8_t NODE_DONE = 2;      // terminal node: excluded from the zero-sum shift
constexpr uint8_t NODE_PARENT = 4;    // the row has children
constexpr uint8_t NODE_LEAF_EVAL = 8; // childless row whose ranges feed a leaf evaluation (showdown, leaf network)
// vectors card-summed per batch: what the LDS union holds next to the showdown buffers, and
// never less than one family (parent + children)
template <int MAXC>
struct ItChunk { static constexpr int value = (MAXC + 1) > 9 ? (MAXC + 1) : 9; };

struct IterArgs {
  // tree (row-major arrays over all nodes of all roots, as the evaluator keeps them)
  const int64_t* child_offsets;
  const int64_t* child_count;
  const int64_t* to_act;
  const uint8_t* node_flags;
  const int64_t* root_parent_offsets;    // [roots+1] into root_parents
  const int64_t* root_parents;           // rows with children of each root's subtree, ascending (= top-down)
  const int64_t* root_showdown_offsets;  // [roots+1] into root_showdown_nodes
  const int64_t* root_showdown_nodes;    // river showdown rows of each root's subtree
  const int64_t* t_sample;           // [total]
  const uint8_t* allowed;            // [total,H] bytes
  const float* allowed_prob;         // [total,H]
  const uint8_t* tables;             // [roots, SD_TABLE_BYTES] board strength tables (may be null)
  const float* potential;            // [total,2] chips won by player p at a showdown row
  const float* scale;                // [total]
  // state
  float* policy;
  float* policy_avg;
  float* policy_sample;
  float* cum;
  float* wsum;
  float* beliefs;
  float* beliefs_avg;
  float* reach;
  float* reach_avg;
  float* latest;
  float* values_avg;
  float* scratch;                    // [total,H] workspace
  const float* reach_avg_prev;       // [total,2,H] or null: reach_avg as the previous iteration left it (see PHASE_LEAN)
  // iteration-dependent scalars in device memory
  const float* fscal;    // t_alpha_num, t_beta_num, t_alpha_den, t_beta_den, mix_old, mix_new, mix_total, mix_inv_total
  const int64_t* iscal;  // t, apply_dcfr, cfr_plus, avg_policy_copy, enforce_zero_sum, update_avg_values, cfr_avg, linear
  // Work items (optional; null = one item per root, item w is root w).  An item is a run of the
  // root_parents / root_showdown_nodes lists that one workgroup walks: a whole root, or — to fill
  // the chip when there are few roots — the top of a root's tree above a cut level (item_top = 1)
  // or the subtree under one node of the cut level (item_top = 0).  Every family and every
  // showdown row belongs to exactly one item; item_root[w] is the root the item belongs to.
  const int64_t* item_root;
  const uint8_t* item_top;
  int phases;            // PHASE_* bits
};

// Which sweeps a launch runs.  Sweep 1 of a family reads its parent's beliefs, values and reach_avg
// as the PREVIOUS iteration left them; sweep 2 needs sweep 1 of its family and sweep 2 of its
// ancestors (it rewrites the rows sweep 1 of the families below reads); sweep 3 needs sweep 2 of its
// subtree and sweep 3 of its descendants.  Inside one workgroup that walks a whole root the three
// simply follow each other (PHASE_12 | PHASE_3).  With a root split into work items it takes four
// launches: every item sweep 1, tree tops sweep 2, subtrees sweeps 2 + 3, tree tops sweep 3.
constexpr int PHASE_12 = 1, PHASE_3 = 2, PHASE_1 = 4, PHASE_2 = 8;
// PHASE_LEAN: an iteration whose result nobody looks at before the next one runs.  Sweep 2 then stores
// only the rows a later sweep or the next iteration reads: reach and reach_avg of rows that have
// children (a family reads its parent's), beliefs of rows that have children or feed a leaf evaluation
// (from beliefs_avg instead under cfr_avg), beliefs_avg only where cfr_avg or the zero-sum shift read
// it.  Every skipped row is a pure function of rows that are kept, so one ordinary iteration afterwards
// leaves all eleven tensors exactly as a run of ordinary iterations would.
//
// reach_avg_prev (independent of PHASE_LEAN): the average-policy mix of a family needs its parent's
// reach_avg[actor] from BEFORE this iteration, which the family above has overwritten by then.  With
// reach_avg_prev null, sweep 1 stashes that row in `scratch`; with two reach_avg buffers that the host
// swaps from iteration to iteration, sweep 2 reads it from the buffer of the previous iteration
// instead: one row read per parent in place of a read, a write and a re-read.
constexpr int PHASE_LEAN = 16;

constexpr int IT_VSTRIDE = P2_H + 2;  // floats between vectors staged in LDS
constexpr int IT_RED = 20;            // block-reduction slots: 2 + 2 * 8 children, rounded up

template <int CH>
struct IterLds {
  union {
    float vecs[CH][IT_VSTRIDE];  // vectors whose card sums are being taken
    ShowdownLds sd;              // showdown scans (never live at the same time)
  } u;
  double cs[CH * P2_CARDS];
  float red[2][IT_WAVES][IT_RED];   // two buffers, used alternately by consecutive block reductions
};

#define IT_FOR(j) _Pragma("unroll") for (int j = 0; j < IT_PPT; ++j)

// Section timing for tuning builds only (-DP2_ITER_PROFILE); compiled out of the library.
#ifdef P2_ITER_PROFILE
__device__ long long g_iter_prof[8192][8];
#define PROF_BEGIN(var) const long long var = wall_clock64()
#define PROF_END(slot, var) \
  do { if (threadIdx.x == 0) atomicAdd((unsigned long long*)&g_iter_prof[blockIdx.x & 8191][slot], \
                                       (unsigned long long)(wall_clock64() - (var))); } while (0)
#else
#define PROF_BEGIN(var)
#define PROF_END(slot, var)
#endif

// Which pairs of a 1326-vector a lane owns.  A wave owns IT_WAVE_PAIRS consecutive pairs (1328 B of
// every row), a lane three of them, 64 pairs apart: every load and store instruction of a wave covers
// one contiguous 512-byte run, and the three of a row follow each other in memory.  Slots 0 and 1 are
// pairs of the row for every lane; slot 2 only for the first 38 (37 in the last wave) lanes, the
// others keep a clamped index there so that loads need no branch, and read zero.
constexpr int IT_WAVE_PAIRS = 166;  // 4 * 166 = 664 >= 663
static_assert(IT_WAVES * IT_WAVE_PAIRS >= P2_HPAIRS && IT_WAVE_PAIRS <= IT_PPT * 64, "lane ownership");

struct Lane {
  int idx[IT_PPT];      // pair index (slot 2: clamped into the row where the lane has no third pair)
  bool ok2;             // slot 2 is a pair of its own
  uint32_t ab[IT_PPT];  // cards of the two hands of each pair: a0 | b0 << 8 | a1 << 16 | b1 << 24
};

__device__ __forceinline__ void lane_init(Lane& ln) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  IT_FOR(j) {
    const int q = j * 64 + lane;
    const int i = wave * IT_WAVE_PAIRS + q;
    const bool ok = j < 2 || (q < IT_WAVE_PAIRS && i < P2_HPAIRS);
    if (j == 2) ln.ok2 = ok;
    ln.idx[j] = ok ? i : P2_HPAIRS - 1;
    const int h = 2 * ln.idx[j];
    ln.ab[j] = (uint32_t)p2_combo.a[h] | ((uint32_t)p2_combo.b[h] << 8) | ((uint32_t)p2_combo.a[h + 1] << 16) |
               ((uint32_t)p2_combo.b[h + 1] << 24);
  }
}

__device__ __forceinline__ void ld(float2 (&dst)[IT_PPT], const float* base, int64_t row, const Lane& ln) {
  const float2* s = p2_row2(base, row);
  IT_FOR(j) dst[j] = s[ln.idx[j]];
  dst[2] = ln.ok2 ? dst[2] : make_float2(0.f, 0.f);
}
__device__ __forceinline__ void st(float* base, int64_t row, const float2 (&src)[IT_PPT], const Lane& ln) {
  float2* d = p2_row2(base, row);
  d[ln.idx[0]] = src[0];
  d[ln.idx[1]] = src[1];
  if (ln.ok2) d[ln.idx[2]] = src[2];
}
__device__ __forceinline__ void to_lds(float* vec, const float2 (&src)[IT_PPT], const Lane& ln) {
  float2* d = reinterpret_cast<float2*>(vec);
  d[ln.idx[0]] = src[0];
  d[ln.idx[1]] = src[1];
  if (ln.ok2) d[ln.idx[2]] = src[2];
}
__device__ __forceinline__ void from_lds(float2 (&dst)[IT_PPT], const float* vec, const Lane& ln) {
  const float2* v2 = reinterpret_cast<const float2*>(vec);
  IT_FOR(j) dst[j] = v2[ln.idx[j]];
  dst[2] = ln.ok2 ? dst[2] : make_float2(0.f, 0.f);
}

// unblocked mass of the vector whose card sums are in (cs, S) for this lane's hands
__device__ __forceinline__ void unblocked_regs(float2 (&out)[IT_PPT], const float2 (&t)[IT_PPT], const double* cs,
                                               double S, const Lane& ln) {
  IT_FOR(j) {
    const uint32_t ab = ln.ab[j];
    const double x = S - cs[ab & 0xFFu] - cs[(ab >> 8) & 0xFFu] + (double)t[j].x;
    const double y = S - cs[(ab >> 16) & 0xFFu] - cs[ab >> 24] + (double)t[j].y;
    out[j] = make_float2(fmaxf((float)x, 0.f), fmaxf((float)y, 0.f));
  }
}

// Sums of up to four per-thread partials over the block; results to all threads.
__device__ __forceinline__ void block_sum4(float (&v)[4], float (*red)[IT_RED]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int q = 0; q < 4; ++q) v[q] = p2_wave_sum(v[q]);
  p2_sync_lds();
  if (lane == 0) {
#pragma unroll
    for (int q = 0; q < 4; ++q) red[wave][q] = v[q];
  }
  p2_sync_lds();
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < IT_WAVES; ++w) s += red[w][q];
    v[q] = s;
  }
}

// Sums of the first `n` (<= N) per-thread partials over the block; results to all threads.  One
// barrier: the caller alternates between two `red` buffers from call to call, so a buffer is
// rewritten only after a later barrier has seen every thread finish reading it.
template <int N>
__device__ __forceinline__ void block_sums(float (&v)[N], int n, float (*red)[IT_RED]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int q = 0; q < N; ++q)
    if (q < n) v[q] = p2_wave_sum(v[q]);
  if (lane == 0) {
#pragma unroll
    for (int q = 0; q < N; ++q)
      if (q < n) red[wave][q] = v[q];
  }
  p2_sync_lds();
#pragma unroll
  for (int q = 0; q < N; ++q) {
    if (q < n) {
      float s = 0.f;
#pragma unroll
      for (int w = 0; w < IT_WAVES; ++w) s += red[w][q];
      v[q] = s;
    }
  }
}

// A copy of a wave-uniform count that the optimiser cannot relate to the original: guards written
// with different copies stay separate branches instead of being threaded into one path per count
// (which ties the register allocator's hands where rows are requested in batches).
__device__ __forceinline__ int opaque(int x) {
  asm volatile("" : "+s"(x));
  return x;
}

__device__ __forceinline__ float2 mul2(float2 a, float2 b) { return make_float2(a.x * b.x, a.y * b.y); }

// A window of 64 consecutive entries of a work item's family list, one per lane: the parent row, the
// row of its first child, the child count and who acts.  The kernel broadcasts an entry with a lane
// read, so walking the tree costs no dependent global loads per family; every wave keeps its own copy.
struct FamWin {
  int p, first, ca;   // ca = child count | actor << 8 | kinds << 16
  int base;           // list position (relative to the item's first family) held by lane 0
};
// KINDS: also collect, per child k, bit 2k = the child has children, bit 2k + 1 = its ranges feed a
// leaf evaluation (what a lean iteration decides its stores by).
template <int MAXC, bool KINDS>
__device__ __forceinline__ void fam_load(FamWin& F, const IterArgs& A, int64_t pp0, int nfam, int base) {
  const int l = base + (int)(threadIdx.x & 63);
  F.base = base;
  F.p = 0;
  F.first = 0;
  F.ca = 0;
  if (l < nfam) {
    const int64_t p = A.root_parents[pp0 + l];
    const int64_t first = A.child_offsets[p];
    const int cnt = (int)A.child_count[p];
    F.p = (int)p;
    F.first = (int)first;
    int kinds = 0;
    if (KINDS) {
#pragma unroll
      for (int k = 0; k < MAXC; ++k)
        if (k < cnt) kinds |= (((int)A.node_flags[first + k] >> 2) & 3) << (2 * k);
    }
    F.ca = cnt | ((int)A.to_act[p] << 8) | (kinds << 16);
  }
}
struct Fam { int64_t p, first; int cnt, actor, kinds; };
__device__ __forceinline__ Fam fam_get(const FamWin& F, int i) {
  const int s = i - F.base;
  Fam f;
  f.p = __builtin_amdgcn_readlane(F.p, s);
  f.first = __builtin_amdgcn_readlane(F.first, s);
  const int ca = __builtin_amdgcn_readlane(F.ca, s);
  f.cnt = ca & 0xFF;
  f.actor = (ca >> 8) & 0xFF;
  f.kinds = (int)((unsigned)ca >> 16);
  return f;
}

// The same for the item's showdown rows: row, chips at stake for either player, scale.
struct SdWin {
  int c;
  float pot0, pot1, scale;
  int base;
};
__device__ __forceinline__ void sd_load(SdWin& S, const IterArgs& A, int64_t sd0, int nsd, int base) {
  const int l = base + (int)(threadIdx.x & 63);
  S.base = base;
  S.c = 0;
  S.pot0 = S.pot1 = 0.f;
  S.scale = 1.f;
  if (l < nsd) {
    const int64_t c = A.root_showdown_nodes[sd0 + l];
    S.c = (int)c;
    S.pot0 = A.potential[2 * c];
    S.pot1 = A.potential[2 * c + 1];
    S.scale = A.scale[c];
  }
}
__device__ __forceinline__ float readlane_f(float v, int s) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), s));
}

template <int MAXC, bool LEAN, bool ALT>
__global__ __launch_bounds__(IT_BLOCK, ItTune<MAXC>::min_waves) void cfr_iteration_kernel(IterArgs A) {
  constexpr int IT_CHUNK = ItChunk<MAXC>::value;
  // how many rows are requested together: parents staged for the card sums, children of a family in
  // the regret sweep, children of a family in the value sweep
  constexpr int SB = ItTune<MAXC>::SB, GRP = ItTune<MAXC>::G1, GRP3 = ItTune<MAXC>::G3;
  __shared__ IterLds<IT_CHUNK> L;
  const int64_t w = blockIdx.x;                               // work item: indexes the per-item lists
  const int64_t r = A.item_root ? A.item_root[w] : w;         // its root: root-level inputs (ranges, board, table)
  const bool top = A.item_top ? A.item_top[w] != 0 : true;    // the item's first family is the root's own
  const int64_t pp0 = A.root_parent_offsets[w];
  const int nfam = (int)(A.root_parent_offsets[w + 1] - pp0);

  Lane ln;
  lane_init(ln);
  FamWin F;
  fam_load<MAXC, LEAN>(F, A, pp0, nfam, 0);
  constexpr bool stash = !ALT;   // the pre-update reach_avg of a parent goes through `scratch`

  const float f_an = A.fscal[0], f_bn = A.fscal[1], f_ad = A.fscal[2], f_bd = A.fscal[3];
  const float mix_old = A.fscal[4], mix_new = A.fscal[5], mix_total = A.fscal[6], mix_inv = A.fscal[7];
  const int64_t t_now = A.iscal[0];
  const bool apply_dcfr = A.iscal[1] != 0, cfr_plus = A.iscal[2] != 0, avg_copy = A.iscal[3] != 0;
  const bool enforce_zs = A.iscal[4] != 0, update_avg = A.iscal[5] != 0;
  // cfr_avg: regret weights and showdown values come from the average-policy beliefs
  // (fused_sparse_cfr_evaluator.py:322,455); linear: the regrets of the player whose turn it is
  // not (t mod 2) are dropped and nothing is discounted (:503-507)
  const bool cfr_avg = A.iscal[6] != 0, linear = A.iscal[7] != 0;
  const float* leaf_beliefs = cfr_avg ? A.beliefs_avg : A.beliefs;

  if (A.phases & (PHASE_12 | PHASE_1)) {
    // ---------------- sweep 1: regrets -> DCFR -> regret matching ----------------
    PROF_BEGIN(t_s1);
    const bool take_sample = A.t_sample[r] == t_now;
    if (top) {
      // The root row takes part in the flat DCFR update like every other row: its regret is
      // zero (never positive), so only its weight sum moves.
      float2 ws[IT_PPT];
      ld(ws, A.wsum, r, ln);
      IT_FOR(j) {
        float ww[2] = {ws[j].x, ws[j].y};
#pragma unroll
        for (int e = 0; e < 2; ++e) {
          if (apply_dcfr) {
            ww[e] = ww[e] * f_bn;
            ww[e] = ww[e] / f_bd;
          }
          ww[e] = ww[e] + 1.0f;
        }
        ws[j] = make_float2(ww[0], ww[1]);
      }
      st(A.wsum, r, ws, ln);
    }
    for (int i0 = 0; i0 < nfam; i0 += IT_CHUNK) {
      const int nch = (nfam - i0) < IT_CHUNK ? (nfam - i0) : IT_CHUNK;
      if (i0 < F.base || i0 + nch > F.base + 64) fam_load<MAXC, LEAN>(F, A, pp0, nfam, i0);
      // opponent beliefs of every parent of the chunk: requested together, staged together,
      // card-summed in one pass
      PROF_BEGIN(t_c1);
#pragma unroll
      for (int u0 = 0; u0 < IT_CHUNK; u0 += SB) {
        if (u0 < nch) {
          // straight-line requests: slots past the chunk's end repeat its last parent and store nothing
          float2 bo[SB][IT_PPT], ra[SB][IT_PPT];
#pragma unroll
          for (int uu = 0; uu < SB; ++uu) {
            const int u = u0 + uu < nch ? u0 + uu : nch - 1;
            const Fam f = fam_get(F, i0 + u);
            ld(bo[uu], leaf_beliefs, f.p * 2 + (1 - f.actor), ln);
            if (stash) ld(ra[uu], A.reach_avg, f.p * 2 + f.actor, ln);  // the mix in sweep 2 needs the pre-update value
          }
#pragma unroll
          for (int uu = 0; uu < SB; ++uu) {
            const int u = u0 + uu;
            if (u < IT_CHUNK && u < nch) {
              const Fam f = fam_get(F, i0 + u);
              to_lds(L.u.vecs[u], bo[uu], ln);
              if (stash) st(A.scratch, f.p, ra[uu], ln);
            }
          }
        }
      }
      p2_sync_lds();
      card_sums_multi(L.u.vecs[0], IT_VSTRIDE, nch, L.cs);
      PROF_END(4, t_c1);
      for (int u = 0; u < nch; ++u) {
        const Fam f = fam_get(F, i0 + u);
        const int cnt = f.cnt, actor = f.actor;
        const int64_t first = f.first;
        if (take_sample) {
          for (int k = 0; k < cnt; ++k) {
            float2 tmp[IT_PPT];
            ld(tmp, A.policy, first + k, ln);
            st(A.policy_sample, first + k, tmp, ln);
          }
        }
        float2 ex[IT_PPT], pos[MAXC][IT_PPT], sum[IT_PPT], wgt[IT_PPT];
        ld(ex, A.latest, f.p * 2 + actor, ln);
        IT_FOR(j) sum[j] = make_float2(0.f, 0.f);
#pragma unroll
        for (int g0 = 0; g0 < MAXC; g0 += GRP) {
          if (g0 < cnt) {
            float2 ach[GRP][IT_PPT], cu[GRP][IT_PPT], ws[GRP][IT_PPT];
#pragma unroll
            for (int kk = 0; kk < GRP; ++kk) {
              const int k = g0 + kk;
              if (k < MAXC && k < cnt) {
                const int64_t c = first + k;
                ld(ach[kk], A.latest, c * 2 + actor, ln);
                ld(cu[kk], A.cum, c, ln);
                ld(ws[kk], A.wsum, c, ln);
              }
            }
            if (g0 == 0) {
              float2 bo[IT_PPT];
              from_lds(bo, L.u.vecs[u], ln);
              unblocked_regs(wgt, bo, L.cs + u * P2_CARDS, card_total(L.cs + u * P2_CARDS), ln);
              if (linear && actor == (int)(t_now & 1)) {
                IT_FOR(j) wgt[j] = make_float2(0.f, 0.f);   // this player's regrets are skipped at this t
              }
            }
#pragma unroll
            for (int kk = 0; kk < GRP; ++kk) {
              const int k = g0 + kk;
              if (k < MAXC && k < cnt) {
                const int64_t c = first + k;
                IT_FOR(j) {
                  float cc[2] = {cu[kk][j].x, cu[kk][j].y}, ww[2] = {ws[kk][j].x, ws[kk][j].y};
                  const float rg[2] = {wgt[j].x * (ach[kk][j].x - ex[j].x), wgt[j].y * (ach[kk][j].y - ex[j].y)};
#pragma unroll
                  for (int e = 0; e < 2; ++e) {
                    if (apply_dcfr) {
                      const bool positive = cc[e] > 0.f;
                      const float num = positive ? f_an : f_bn, den = positive ? f_ad : f_bd;
                      cc[e] = cc[e] * num;
                      cc[e] = cc[e] / den;
                      ww[e] = ww[e] * num;
                      ww[e] = ww[e] / den;
                    }
                    ww[e] = ww[e] + 1.0f;
                    cc[e] = cc[e] + rg[e];
                    if (cfr_plus) cc[e] = fmaxf(cc[e], 0.f);
                  }
                  cu[kk][j] = make_float2(cc[0], cc[1]);
                  ws[kk][j] = make_float2(ww[0], ww[1]);
                  pos[k][j] = make_float2(fmaxf(cc[0], 0.f), fmaxf(cc[1], 0.f));
                  sum[j].x += pos[k][j].x;
                  sum[j].y += pos[k][j].y;
                }
                st(A.cum, c, cu[kk], ln);
                st(A.wsum, c, ws[kk], ln);
              }
            }
          }
        }
        const float uniform = 1.0f / (float)cnt;
#pragma unroll
        for (int k = 0; k < MAXC; ++k) {
          if (k < cnt) {
            float2 pol[IT_PPT];
            IT_FOR(j) {
              pol[j].x = sum[j].x > 1e-8f ? pos[k][j].x / fmaxf(sum[j].x, 1e-8f) : uniform;
              pol[j].y = sum[j].y > 1e-8f ? pos[k][j].y / fmaxf(sum[j].y, 1e-8f) : uniform;
            }
            st(A.policy, first + k, pol, ln);
          }
        }
      }
      p2_sync_lds();  // the staged vectors and L.cs are rewritten by the next chunk
    }
    PROF_END(0, t_s1);
  }

  if (A.phases & (PHASE_12 | PHASE_2)) {
    PROF_BEGIN(t_s2);
    // ---------------- sweep 2: reach, beliefs, average policy ----------------
    // (re-reads policy / reach rows that the same lane wrote: no cross-lane hand-off)
    // The root's ranges scale every belief below it.  Where the LDS vectors have four slots to spare
    // next to a family's children they wait there (in this lane's own slots: no barrier) instead of
    // occupying 24 registers through the whole sweep.
    constexpr bool ROOT_LDS = IT_CHUNK - MAXC >= 4;
    // Which rows a lean iteration keeps (see PHASE_LEAN): beliefs_avg everywhere for the zero-sum shift
    // of sweep 3, under cfr_avg where they take the place of beliefs, else nowhere.
    const bool bavg_all = !LEAN || enforce_zs, bavg_any = bavg_all || cfr_avg;
    float2 rbk[2][IT_PPT], rbak[2][IT_PPT], ap[IT_PPT];
    uchar2 am[IT_PPT];
    ld(rbk[0], A.beliefs, r * 2, ln);
    ld(rbk[1], A.beliefs, r * 2 + 1, ln);
    if (bavg_any) {
      ld(rbak[0], A.beliefs_avg, r * 2, ln);
      ld(rbak[1], A.beliefs_avg, r * 2 + 1, ln);
    } else {
      IT_FOR(j) rbak[0][j] = rbak[1][j] = make_float2(0.f, 0.f);
    }
    ld(ap, A.allowed_prob, r, ln);
    {
      const uchar2* m2 = reinterpret_cast<const uchar2*>(A.allowed + r * P2_H);
      IT_FOR(j) am[j] = m2[ln.idx[j]];
      am[2] = ln.ok2 ? am[2] : make_uchar2(0, 0);
    }
    if (ROOT_LDS) {
      to_lds(L.u.vecs[MAXC + 0], rbk[0], ln);
      to_lds(L.u.vecs[MAXC + 1], rbk[1], ln);
      to_lds(L.u.vecs[MAXC + 2], rbak[0], ln);
      to_lds(L.u.vecs[MAXC + 3], rbak[1], ln);
    }
    for (int i = 0; i < nfam; ++i) {
      if (i < F.base || i >= F.base + 64) fam_load<MAXC, LEAN>(F, A, pp0, nfam, i);
      const Fam f = fam_get(F, i);
      const int64_t p = f.p, first = f.first;
      const int cnt = f.cnt, actor = f.actor;
      // per child: does it have children (its reach rows are read by its own family), do its ranges feed
      // a leaf evaluation; an ordinary iteration keeps every row
      const int has_children = LEAN ? f.kinds & 0x5555 : 0x5555, leaf_eval = LEAN ? (f.kinds >> 1) & 0x5555 : 0x5555;
      const int keep_b = cfr_avg ? has_children : (has_children | leaf_eval);
      const int keep_ba = bavg_all ? 0x5555 : (cfr_avg ? (has_children | leaf_eval) : 0);
      float2 rn[2][IT_PPT], ran[2][IT_PPT], ra_old[IT_PPT];
      float2 cur[MAXC][IT_PPT], pav[MAXC][IT_PPT];
      ld(rn[0], A.reach, p * 2, ln);
      ld(rn[1], A.reach, p * 2 + 1, ln);
      ld(ran[0], A.reach_avg, p * 2, ln);
      ld(ran[1], A.reach_avg, p * 2 + 1, ln);
      if (stash) ld(ra_old, A.scratch, p, ln);
      else ld(ra_old, A.reach_avg_prev, p * 2 + actor, ln);
#pragma unroll
      for (int k = 0; k < MAXC; ++k)
        if (k < cnt) ld(cur[k], A.policy, first + k, ln);
      if (!avg_copy) {
#pragma unroll
        for (int k = 0; k < MAXC; ++k)
          if (k < cnt) ld(pav[k], A.policy_avg, first + k, ln);   // the old average; mixed in place below
      }

      float2 rn_act[IT_PPT];  // new reach of the acting player at the parent
      IT_FOR(j) rn_act[j] = actor == 0 ? rn[0][j] : rn[1][j];
      float2 psum[IT_PPT];
      IT_FOR(j) psum[j] = make_float2(0.f, 0.f);
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt) {
          if (avg_copy) {
            IT_FOR(j) pav[k][j] = cur[k][j];
          } else {
            IT_FOR(j) {
              const float rr[2] = {rn_act[j].x, rn_act[j].y}, rao[2] = {ra_old[j].x, ra_old[j].y};
              const float cc[2] = {cur[k][j].x, cur[k][j].y}, aa[2] = {pav[k][j].x, pav[k][j].y};
              float o[2];
#pragma unroll
              for (int e = 0; e < 2; ++e) {
                const float reach_a = rao[e] * mix_old, reach_n = rr[e] * mix_new;
                const float num = reach_a * aa[e] + reach_n * cc[e];
                const float den = reach_a + reach_n;
                const float unweighted = (mix_old * aa[e] + mix_new * cc[e]) / mix_total;
                o[e] = den > 1e-5f ? num / den : unweighted;
              }
              pav[k][j] = make_float2(o[0], o[1]);
              psum[j].x += o[0];
              psum[j].y += o[1];
            }
          }
        }
      }
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt) {
          if (!avg_copy) {
            IT_FOR(j) {
              if (psum[j].x > 1e-5f) pav[k][j].x = pav[k][j].x / fmaxf(psum[j].x, 1e-5f);
              if (psum[j].y > 1e-5f) pav[k][j].y = pav[k][j].y / fmaxf(psum[j].y, 1e-5f);
            }
          }
          st(A.policy_avg, first + k, pav[k], ln);
        }
      }
      // From here on a child's policy is only needed as its new reach x = reach(actor) * policy
      // (allowed hands only), and its average policy as y likewise: x goes to this lane's own slots
      // of the LDS vectors (idle in this sweep; no other lane touches them, so no barrier), y takes
      // the place of the average policy in registers.
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt) {
          float2 xa[IT_PPT];
          IT_FOR(j) {
            const float2 x = mul2(rn_act[j], cur[k][j]);
            xa[j] = make_float2(am[j].x ? x.x : 0.f, am[j].y ? x.y : 0.f);
            const float2 y = mul2(actor == 0 ? ran[0][j] : ran[1][j], pav[k][j]);
            pav[k][j] = make_float2(am[j].x ? y.x : 0.f, am[j].y ? y.y : 0.f);
          }
          to_lds(L.u.vecs[k], xa, ln);
        }
      }
      // Belief normalisers of the whole family in one block reduction: the player who does not
      // act has the same reach at every child (two sums), the actor's differ per child.  The rows
      // are then written array by array, so that each array receives the family's children as one
      // contiguous run.
      float2 rn_opp[IT_PPT], ran_opp[IT_PPT], rb_act[IT_PPT], rb_opp[IT_PPT], rba_act[IT_PPT], rba_opp[IT_PPT];
      if (ROOT_LDS) {
        from_lds(rb_act, L.u.vecs[MAXC + actor], ln);
        from_lds(rb_opp, L.u.vecs[MAXC + 1 - actor], ln);
        from_lds(rba_act, L.u.vecs[MAXC + 2 + actor], ln);
        from_lds(rba_opp, L.u.vecs[MAXC + 3 - actor], ln);
      } else {
        IT_FOR(j) {
          const bool a0 = actor == 0;
          rb_act[j] = a0 ? rbk[0][j] : rbk[1][j];
          rb_opp[j] = a0 ? rbk[1][j] : rbk[0][j];
          rba_act[j] = a0 ? rbak[0][j] : rbak[1][j];
          rba_opp[j] = a0 ? rbak[1][j] : rbak[0][j];
        }
      }
      IT_FOR(j) {
        const bool a0 = actor == 0;
        rn_opp[j] = a0 ? rn[1][j] : rn[0][j];
        ran_opp[j] = a0 ? ran[1][j] : ran[0][j];
        rn_opp[j] = make_float2(am[j].x ? rn_opp[j].x : 0.f, am[j].y ? rn_opp[j].y : 0.f);
        ran_opp[j] = make_float2(am[j].x ? ran_opp[j].x : 0.f, am[j].y ? ran_opp[j].y : 0.f);
      }
      float sums[2 + 2 * MAXC];
#pragma unroll
      for (int q = 0; q < 2 + 2 * MAXC; ++q) sums[q] = 0.f;
      IT_FOR(j) {
        const float2 vb = mul2(rb_opp[j], rn_opp[j]), vba = mul2(rba_opp[j], ran_opp[j]);
        sums[0] += vb.x + vb.y;
        sums[1] += vba.x + vba.y;
      }
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt) {
          float2 xa[IT_PPT];
          from_lds(xa, L.u.vecs[k], ln);
          IT_FOR(j) {
            const float2 vb = mul2(rb_act[j], xa[j]);
            sums[2 + 2 * k] += vb.x + vb.y;
          }
          if (keep_ba) {
            IT_FOR(j) {
              const float2 vba = mul2(rba_act[j], pav[k][j]);
              sums[3 + 2 * k] += vba.x + vba.y;
            }
          }
        }
      }
      PROF_BEGIN(t_b2);
      block_sums<2 + 2 * MAXC>(sums, 2 + 2 * cnt, L.red[i & 1]);
      PROF_END(6, t_b2);
      const float so = sums[0], soa = sums[1];
      // reach
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt && ((has_children >> (2 * k)) & 1)) {
          const int64_t c = first + k;
          float2 xa[IT_PPT];
          from_lds(xa, L.u.vecs[k], ln);
          if (actor == 0) { st(A.reach, c * 2, xa, ln); st(A.reach, c * 2 + 1, rn_opp, ln); }
          else { st(A.reach, c * 2, rn_opp, ln); st(A.reach, c * 2 + 1, xa, ln); }
        }
      }
      // reach_avg
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt && ((has_children >> (2 * k)) & 1)) {
          const int64_t c = first + k;
          if (actor == 0) { st(A.reach_avg, c * 2, pav[k], ln); st(A.reach_avg, c * 2 + 1, ran_opp, ln); }
          else { st(A.reach_avg, c * 2, ran_opp, ln); st(A.reach_avg, c * 2 + 1, pav[k], ln); }
        }
      }
      // beliefs
      float2 bo[IT_PPT], boa[IT_PPT];
      IT_FOR(j) {
        const float2 vb = mul2(rb_opp[j], rn_opp[j]), vba = mul2(rba_opp[j], ran_opp[j]);
        bo[j] = so > 1e-5f ? make_float2(vb.x / so, vb.y / so) : ap[j];
        boa[j] = soa > 1e-5f ? make_float2(vba.x / soa, vba.y / soa) : ap[j];
      }
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt && ((keep_b >> (2 * k)) & 1)) {
          const int64_t c = first + k;
          const float sa = sums[2 + 2 * k];
          float2 o[IT_PPT], xa[IT_PPT];
          from_lds(xa, L.u.vecs[k], ln);
          IT_FOR(j) {
            const float2 vb = mul2(rb_act[j], xa[j]);
            o[j] = sa > 1e-5f ? make_float2(vb.x / sa, vb.y / sa) : ap[j];
          }
          if (actor == 0) { st(A.beliefs, c * 2, o, ln); st(A.beliefs, c * 2 + 1, bo, ln); }
          else { st(A.beliefs, c * 2, bo, ln); st(A.beliefs, c * 2 + 1, o, ln); }
        }
      }
      // beliefs_avg
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt && ((keep_ba >> (2 * k)) & 1)) {
          const int64_t c = first + k;
          const float saa = sums[3 + 2 * k];
          float2 oa[IT_PPT];
          IT_FOR(j) {
            const float2 vba = mul2(rba_act[j], pav[k][j]);
            oa[j] = saa > 1e-5f ? make_float2(vba.x / saa, vba.y / saa) : ap[j];
          }
          if (actor == 0) { st(A.beliefs_avg, c * 2, oa, ln); st(A.beliefs_avg, c * 2 + 1, boa, ln); }
          else { st(A.beliefs_avg, c * 2, boa, ln); st(A.beliefs_avg, c * 2 + 1, oa, ln); }
        }
      }
    }
    PROF_END(1, t_s2);
  }

  if (A.phases & PHASE_3) {
    // ---------------- sweep 3a: showdown leaves ----------------
    PROF_BEGIN(t_s3);
    const int64_t sd0 = A.root_showdown_offsets[w];
    const int nsd = (int)(A.root_showdown_offsets[w + 1] - sd0);
    if (nsd > 0 && A.tables) {
      PROF_BEGIN(t_sd);
      ShowdownRegs sdr;
      SdWin S;
      showdown_load_regs(A.tables + r * SD_TABLE_BYTES, sdr);
      sd_load(S, A, sd0, nsd, 0);
      // beliefs written in sweep 2 are gathered by other lanes here: the one hand-off through
      // global memory, hence a full barrier
      __syncthreads();
      float vk[2][SD_PPT];
      showdown_gather(leaf_beliefs + (int64_t)__builtin_amdgcn_readlane(S.c, 0) * 2 * P2_H, sdr, vk);
      for (int i = 0; i < nsd; ++i) {
        if (i >= S.base + 64) sd_load(S, A, sd0, nsd, i);
        const int sl = i - S.base;
        const int64_t c = __builtin_amdgcn_readlane(S.c, sl);
        const float pot0 = readlane_f(S.pot0, sl), pot1 = readlane_f(S.pot1, sl), scl = readlane_f(S.scale, sl);
        float vnext[2][SD_PPT];
        if (i + 1 < nsd) {
          const int64_t cn = sl + 1 < 64 ? (int64_t)__builtin_amdgcn_readlane(S.c, (sl + 1) & 63)
                                         : A.root_showdown_nodes[sd0 + i + 1];
          showdown_gather(leaf_beliefs + cn * 2 * P2_H, sdr, vnext);
        }
        // the EVs land in the sorted-range buffers, which the evaluation no longer needs by then
        showdown_eval(vk, sdr, L.u.sd, L.u.sd.v, pot0, pot1, scl);
        p2_sync_lds();
        float2 v[2][IT_PPT];
        IT_FOR(j) {
          // hands 2*idx and 2*idx+1, each holding (hero 0, hero 1)
          const float2 x = L.u.sd.v[2 * ln.idx[j]];
          const float2 y = L.u.sd.v[2 * ln.idx[j] + 1];
          v[0][j] = make_float2(x.x, y.x);
          v[1][j] = make_float2(x.y, y.y);
        }
        st(A.latest, c * 2, v[0], ln);
        st(A.latest, c * 2 + 1, v[1], ln);
        p2_sync_lds();  // the next evaluation overwrites the buffers just read
        if (i + 1 < nsd) {
#pragma unroll
          for (int q = 0; q < SD_PPT; ++q) { vk[0][q] = vnext[0][q]; vk[1][q] = vnext[1][q]; }
        }
      }
      PROF_END(3, t_sd);
    }

    // ---------------- sweep 3b: backup, bottom-up ----------------
    for (int i = nfam - 1; i >= 0; --i) {
      if (i < F.base || i >= F.base + 64) fam_load<MAXC, LEAN>(F, A, pp0, nfam, i > 63 ? i - 63 : 0);
      const Fam f = fam_get(F, i);
      const int64_t p = f.p, first = f.first;
      const int cnt = f.cnt, actor = f.actor;

      // actor beliefs at the parent and the marginal of every action, card-summed in one pass
      PROF_BEGIN(t_c3);
      float2 ab[IT_PPT], dn[IT_PPT], polk[MAXC][IT_PPT];
      ld(ab, A.beliefs, p * 2 + actor, ln);
#pragma unroll
      for (int k = 0; k < MAXC; ++k)
        if (k < cnt) ld(polk[k], A.policy, first + k, ln);
      to_lds(L.u.vecs[0], ab, ln);
#pragma unroll
      for (int k = 0; k < MAXC; ++k) {
        if (k < cnt) {
          float2 mg[IT_PPT];
          IT_FOR(j) mg[j] = mul2(ab[j], polk[k][j]);
          to_lds(L.u.vecs[1 + k], mg, ln);
        }
      }
      p2_sync_lds();

      float2 vp[2][IT_PPT];
      IT_FOR(j) vp[0][j] = vp[1][j] = make_float2(0.f, 0.f);
      // The children's values and running averages are requested GRP3 children at a time, as
      // straight-line code (slots past the last child repeat it and are not used); the first
      // group's requests are in flight while the card sums are taken.
#pragma unroll
      for (int g0 = 0; g0 < MAXC; g0 += GRP3) {
        if (g0 == 0 || g0 < cnt) {
          float2 v[GRP3][2][IT_PPT], av[GRP3][2][IT_PPT];
#pragma unroll
          for (int kk = 0; kk < GRP3; ++kk) {
            const int64_t c = first + (g0 + kk < cnt ? g0 + kk : cnt - 1);
            ld(v[kk][0], A.latest, c * 2, ln);
            ld(v[kk][1], A.latest, c * 2 + 1, ln);
            if (update_avg) {
              ld(av[kk][0], A.values_avg, c * 2, ln);
              ld(av[kk][1], A.values_avg, c * 2 + 1, ln);
            }
          }
          if (g0 == 0) {
            card_sums_multi(L.u.vecs[0], IT_VSTRIDE, cnt + 1, L.cs);
            unblocked_regs(dn, ab, L.cs, card_total(L.cs), ln);
            PROF_END(5, t_c3);
          }
#pragma unroll
          for (int kk = 0; kk < GRP3; ++kk) {
            const int k = g0 + kk;
            if (k < MAXC && k < cnt) {
              const int64_t c = first + k;
              if (update_avg) {
                // values_avg[c] <- (avg*old + latest*new) * inv_total, then the optional zero-sum shift
                float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int pl = 0; pl < 2; ++pl) {
                  IT_FOR(j) av[kk][pl][j] = make_float2((av[kk][pl][j].x * mix_old + v[kk][pl][j].x * mix_new) * mix_inv,
                                                        (av[kk][pl][j].y * mix_old + v[kk][pl][j].y * mix_new) * mix_inv);
                  if (enforce_zs) {
                    float2 ba[IT_PPT];
                    ld(ba, A.beliefs_avg, c * 2 + pl, ln);
                    IT_FOR(j) s4[0] += av[kk][pl][j].x * ba[j].x + av[kk][pl][j].y * ba[j].y;
                  }
                }
                float shift = 0.f;
                if (enforce_zs) {
                  block_sum4(s4, L.red[0]);
                  shift = (A.node_flags[c] & NODE_DONE) ? 0.f : 0.5f * s4[0];
                }
#pragma unroll
                for (int pl = 0; pl < 2; ++pl) {
                  IT_FOR(j) av[kk][pl][j] = make_float2(av[kk][pl][j].x - shift, av[kk][pl][j].y - shift);
                  st(A.values_avg, c * 2 + pl, av[kk][pl], ln);
                }
              }
              float2 nm[IT_PPT], occ[IT_PPT];
              {
                float2 mg[IT_PPT];
                IT_FOR(j) mg[j] = mul2(ab[j], polk[k][j]);
                unblocked_regs(nm, mg, L.cs + (1 + k) * P2_CARDS, card_total(L.cs + (1 + k) * P2_CARDS), ln);
              }
              IT_FOR(j) {
                occ[j].x = dn[j].x > 1e-5f ? nm[j].x / dn[j].x : 0.f;
                occ[j].y = dn[j].y > 1e-5f ? nm[j].y / dn[j].y : 0.f;
              }
              IT_FOR(j) {
                const float2 wa = polk[k][j], wo = occ[j];
                if (actor == 0) {
                  vp[0][j].x += v[kk][0][j].x * wa.x; vp[0][j].y += v[kk][0][j].y * wa.y;
                  vp[1][j].x += v[kk][1][j].x * wo.x; vp[1][j].y += v[kk][1][j].y * wo.y;
                } else {
                  vp[1][j].x += v[kk][1][j].x * wa.x; vp[1][j].y += v[kk][1][j].y * wa.y;
                  vp[0][j].x += v[kk][0][j].x * wo.x; vp[0][j].y += v[kk][0][j].y * wo.y;
                }
              }
            }
          }
        }
      }
      st(A.latest, p * 2, vp[0], ln);
      st(A.latest, p * 2 + 1, vp[1], ln);
      if (i == 0 && update_avg && top) {
        // the root is nobody's child: update its average values here
        float2 nv[2][IT_PPT];
        float s4[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int pl = 0; pl < 2; ++pl) {
          float2 av[IT_PPT];
          ld(av, A.values_avg, p * 2 + pl, ln);
          IT_FOR(j) nv[pl][j] = make_float2((av[j].x * mix_old + vp[pl][j].x * mix_new) * mix_inv,
                                            (av[j].y * mix_old + vp[pl][j].y * mix_new) * mix_inv);
          if (enforce_zs) {
            float2 ba[IT_PPT];
            ld(ba, A.beliefs_avg, p * 2 + pl, ln);
            IT_FOR(j) s4[0] += nv[pl][j].x * ba[j].x + nv[pl][j].y * ba[j].y;
          }
        }
        float shift = 0.f;
        if (enforce_zs) {
          block_sum4(s4, L.red[0]);
          shift = (A.node_flags[p] & NODE_DONE) ? 0.f : 0.5f * s4[0];
        }
#pragma unroll
        for (int pl = 0; pl < 2; ++pl) {
          IT_FOR(j) nv[pl][j] = make_float2(nv[pl][j].x - shift, nv[pl][j].y - shift);
          st(A.values_avg, p * 2 + pl, nv[pl], ln);
        }
      }
      p2_sync_lds();  // the staged vectors and L.cs are rewritten by the next family
    }
    PROF_END(2, t_s3);
  }
}

struct ScalarPack {
  float f[8];
  int64_t i[8];
};

// The values travel as kernel arguments, so the host may reuse its buffers at once.
__global__ void write_scalars_kernel(float* __restrict__ fscal, int64_t* __restrict__ iscal, ScalarPack v) {
  const int k = threadIdx.x;
  if (k < 8) {
    fscal[k] = v.f[k];
    iscal[k] = v.i[k];
  }
}

struct FloatPack { float f[8]; };

__global__ void upload_floats_kernel(float* __restrict__ dst, FloatPack v, int n) {
  const int k = threadIdx.x;
  if (k < n) dst[k] = v.f[k];
}

}  // namespace p2

extern "C" {

#ifdef P2_ITER_PROFILE
int p2hip_iter_prof_read(long long* host, int reset) {
  hipError_t e = hipMemcpyFromSymbol(host, HIP_SYMBOL(p2::g_iter_prof), sizeof(long long) * 8192 * 8);
  if (e != hipSuccess) return (int)e;
  if (reset) {
    static long long zeros[8192 * 8];
    e = hipMemcpyToSymbol(HIP_SYMBOL(p2::g_iter_prof), zeros, sizeof(zeros));
  }
  return (int)e;
}
#endif

int p2hip_write_scalars(float* fscal, int64_t* iscal, const float* host_f, const int64_t* host_i, void* stream) {
  if (!fscal || !iscal || !host_f || !host_i) return P2_EINVAL;
  p2::ScalarPack v;
  for (int k = 0; k < 8; ++k) {
    v.f[k] = host_f[k];
    v.i[k] = host_i[k];
  }
  hipLaunchKernelGGL(p2::write_scalars_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, fscal, iscal, v);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_upload_floats(float* dst, const float* host_values, int n, void* stream) {
  if (!dst || !host_values || n < 0 || n > 8) return P2_EINVAL;
  if (n == 0) return 0;
  p2::FloatPack v;
  for (int k = 0; k < 8; ++k) v.f[k] = k < n ? host_values[k] : 0.f;
  hipLaunchKernelGGL(p2::upload_floats_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream, dst, v, n);
  P2_LAUNCH_CHECK();
  return 0;
}

// P2HipIterArgs (include/p2hip.h) mirrors p2::IterArgs field by field.

int p2hip_cfr_iteration(const P2HipIterArgs* host_args, int64_t n_items, int max_children, int phases,
                        void* stream) {
  if (!host_args || n_items < 0 || n_items > 0x7FFFFFFF || max_children < 1 || max_children > 8 || (phases & ~31) ||
      (phases & 15) == 0)
    return P2_EINVAL;
  if (n_items == 0) return 0;
  const P2HipIterArgs& h = *host_args;
  if ((h.item_root == nullptr) != (h.item_top == nullptr)) return P2_EINVAL;
  const void* required[] = {h.child_offsets, h.child_count, h.to_act, h.node_flags, h.root_parent_offsets, h.root_parents,
                            h.root_showdown_offsets,  // root_showdown_nodes is empty (null) without showdown rows
                            h.t_sample, h.allowed, h.allowed_prob, h.potential, h.scale, h.policy, h.policy_avg,
                            h.policy_sample, h.cum, h.wsum, h.beliefs, h.beliefs_avg, h.reach, h.reach_avg, h.latest,
                            h.values_avg, h.fscal, h.iscal};
  for (const void* p : required)
    if (!p) return P2_EINVAL;
  // the pre-update reach_avg of a parent travels through `scratch` unless the previous iteration's buffer is given
  if (!h.scratch && !h.reach_avg_prev) return P2_EINVAL;
  if (h.reach_avg_prev == h.reach_avg) return P2_EINVAL;
  const void* rows[] = {h.allowed_prob, h.policy, h.policy_avg, h.policy_sample, h.cum, h.wsum, h.beliefs,
                        h.beliefs_avg, h.reach, h.reach_avg, h.latest, h.values_avg, h.scratch, h.tables,
                        h.reach_avg_prev};
  for (const void* p : rows)
    if (!p2_aligned8(p)) return P2_EINVAL;
  p2::IterArgs a;
  a.child_offsets = h.child_offsets; a.child_count = h.child_count; a.to_act = h.to_act;
  a.node_flags = h.node_flags; a.root_parent_offsets = h.root_parent_offsets; a.root_parents = h.root_parents;
  a.root_showdown_offsets = h.root_showdown_offsets; a.root_showdown_nodes = h.root_showdown_nodes;
  a.t_sample = h.t_sample; a.allowed = h.allowed; a.allowed_prob = h.allowed_prob; a.tables = h.tables;
  a.potential = h.potential; a.scale = h.scale; a.policy = h.policy; a.policy_avg = h.policy_avg;
  a.policy_sample = h.policy_sample; a.cum = h.cum; a.wsum = h.wsum; a.beliefs = h.beliefs;
  a.beliefs_avg = h.beliefs_avg; a.reach = h.reach; a.reach_avg = h.reach_avg; a.latest = h.latest;
  a.values_avg = h.values_avg; a.scratch = h.scratch; a.fscal = h.fscal; a.iscal = h.iscal;
  a.item_root = h.item_root; a.item_top = h.item_top;
  a.reach_avg_prev = h.reach_avg_prev;
  a.phases = phases & 15;
  const bool lean = (phases & p2::PHASE_LEAN) != 0;
  const dim3 grid((unsigned)n_items), block(p2::IT_BLOCK);
  const bool alt = h.reach_avg_prev != nullptr;
#define P2_ITER_LAUNCH(MAXC, LEAN, ALT) \
  hipLaunchKernelGGL((p2::cfr_iteration_kernel<MAXC, LEAN, ALT>), grid, block, 0, (hipStream_t)stream, a)
#define P2_ITER_MODES(MAXC)                                  \
  do {                                                       \
    if (lean && alt) P2_ITER_LAUNCH(MAXC, true, true);       \
    else if (lean) P2_ITER_LAUNCH(MAXC, true, false);        \
    else if (alt) P2_ITER_LAUNCH(MAXC, false, true);         \
    else P2_ITER_LAUNCH(MAXC, false, false);                 \
  } while (0)
  if (max_children <= 5) P2_ITER_MODES(5);
  else P2_ITER_MODES(8);
#undef P2_ITER_MODES
#undef P2_ITER_LAUNCH
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
