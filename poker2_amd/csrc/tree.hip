// Betting-tree construction on the device, one level per launch pair.
//
// Replaces the host depth loop of SparseCFREvaluator over HUNLTensorEnv
// (src/p2/search/sparse_cfr_evaluator.py:142-306) with two per-node kernels that restate the
// environment's rules: legal action bins (src/p2/env/hunl_tensor_env.py:348-423), chips and
// fold reward of an action (:684-724) and the step / betting-round closure (:766-992).
// A node is a row of TREE_COLS int64 (floats by bit pattern); a level is a [n, TREE_COLS]
// matrix.  The host prefix-sums the per-parent child counts between the two launches.
#pragma once
#include "common.h"

namespace p2 {

constexpr int TREE_COLS = 21;
enum TreeCol {
  TC_STREET = 0, TC_TO_ACT, TC_BUTTON, TC_POT, TC_STACK0, TC_STACK1, TC_COMM0, TC_COMM1, TC_MIN_RAISE,
  TC_ACTIONS, TC_ALLIN0, TC_ALLIN1, TC_START0, TC_START1, TC_DONE, TC_RAISES,
  TC_SCALE,    // float32 bits
  TC_ROOT,     // row of the root this node descends from
  TC_PARENT,   // global row of the parent, -1 for roots
  TC_ACTION,   // action bin taken at the parent, -1 for roots
  TC_REWARD,   // float32 bits: player 0's payoff / scale when the action was a fold, else 0
};
constexpr int TREE_MAX_BINS = 5;   // bet fractions; + fold, call, all-in = at most 8 actions
constexpr int TREE_BLOCK = 256;

struct TreeRules {
  float bins[TREE_MAX_BINS];
  int n_bins;
  int max_raises;   // < 0: no cap
  int64_t bb;
};

// Legal bins of a node as a bit mask (bit b = bin b) and the chips of each bet bin.
__device__ __forceinline__ uint32_t tree_legal_bits(const int64_t* s, const TreeRules& R, int64_t (&amounts)[TREE_MAX_BINS]) {
  const int nb = R.n_bins + 3;
  const int me = (int)s[TC_TO_ACT], opp = 1 - me;
  const int64_t me_stack = s[TC_STACK0 + me], opp_stack = s[TC_STACK0 + opp];
  const int64_t to_call = s[TC_COMM0 + opp] - s[TC_COMM0 + me];
  uint32_t mask = 0;
  if (to_call > 0) mask |= 1u;
  mask |= 2u;
  const bool can = me_stack > 0 && opp_stack > 0;
  const float pot_f = (float)s[TC_POT];
  for (int b = 0; b < R.n_bins; ++b) {
    const int64_t additional = (int64_t)(R.bins[b] * pot_f);   // truncates, like the int64 cast of the product
    const int64_t amt = to_call + additional;
    amounts[b] = amt;
    if (can && amt <= me_stack && additional >= s[TC_MIN_RAISE]) mask |= 1u << (2 + b);
  }
  if (me_stack > 0) mask |= 1u << (nb - 1);
  if (R.max_raises >= 0 && s[TC_RAISES] >= R.max_raises) mask &= 3u;
  if (s[TC_ALLIN0 + opp]) mask = 3u;
  if (s[TC_ALLIN0 + me]) mask = 2u;
  if (s[TC_DONE]) mask = 0;
  return mask;
}

// legal_out [n, nb] bytes = the raw legal mask of every node of the level;
// count_out [n] = number of children the node gets: its legal actions if `expand`, none for
// nodes below the root level whose betting round has just closed (actions_this_round == 0).
__global__ __launch_bounds__(TREE_BLOCK) void tree_legal_kernel(const int64_t* __restrict__ nodes, int64_t n,
                                                                 TreeRules R, int is_root_level, int expand,
                                                                 uint8_t* __restrict__ legal_out,
                                                                 int64_t* __restrict__ count_out) {
  const int64_t i = (int64_t)blockIdx.x * TREE_BLOCK + threadIdx.x;
  if (i >= n) return;
  const int64_t* s = nodes + i * TREE_COLS;
  int64_t amounts[TREE_MAX_BINS];
  const uint32_t mask = tree_legal_bits(s, R, amounts);
  const int nb = R.n_bins + 3;
  for (int b = 0; b < nb; ++b) legal_out[i * nb + b] = (mask >> b) & 1u;
  const bool grows = expand && (is_root_level || s[TC_ACTIONS] != 0);
  count_out[i] = grows ? __popc(mask) : 0;
}

// One thread per parent writes its children (action ascending) at children[child_start[i] ...].
__global__ __launch_bounds__(TREE_BLOCK) void tree_step_kernel(const int64_t* __restrict__ parents, int64_t n,
                                                                int64_t parent_row_base, TreeRules R, int is_root_level,
                                                                const int64_t* __restrict__ child_start,
                                                                int64_t* __restrict__ children) {
  const int64_t i = (int64_t)blockIdx.x * TREE_BLOCK + threadIdx.x;
  if (i >= n) return;
  const int64_t* s = parents + i * TREE_COLS;
  if (!is_root_level && s[TC_ACTIONS] == 0) return;
  int64_t amounts[TREE_MAX_BINS];
  const uint32_t mask = tree_legal_bits(s, R, amounts);
  const int nb = R.n_bins + 3;
  const int me = (int)s[TC_TO_ACT], opp = 1 - me;
  const int64_t to_call = s[TC_COMM0 + opp] - s[TC_COMM0 + me];
  const int64_t me_stack = s[TC_STACK0 + me];
  int64_t k = child_start[i];
  for (int a = 0; a < nb; ++a) {
    if (!((mask >> a) & 1u)) continue;
    int64_t c[TREE_COLS];
#pragma unroll
    for (int j = 0; j < TREE_COLS; ++j) c[j] = s[j];
    const bool fold = a == 0, call = a == 1, allin = a == nb - 1, bet = !(fold || call || allin);
    int64_t chips = 0;
    if (call) chips = to_call < me_stack ? to_call : me_stack;
    if (allin) chips = me_stack;
    if (bet) chips = amounts[a - 2];
    c[TC_STACK0 + me] -= chips;
    c[TC_COMM0 + me] += chips;
    c[TC_POT] += chips;
    if (allin) c[TC_ALLIN0 + me] = 1;
    if (bet) c[TC_MIN_RAISE] = c[TC_MIN_RAISE] > chips - to_call ? c[TC_MIN_RAISE] : chips - to_call;
    c[TC_RAISES] += (bet || allin) ? 1 : 0;
    // fold: the other player takes the pot; payoff of player 0 in units of `scale`
    const float share = opp == 0 ? (float)c[TC_POT] : 0.0f;
    const float scale = __builtin_bit_cast(float, (uint32_t)c[TC_SCALE]);
    const float r = ((float)c[TC_STACK0] + share - (float)c[TC_START0]) / scale;
    c[TC_REWARD] = (int64_t)__builtin_bit_cast(uint32_t, fold ? r : 0.0f);
    if (fold) c[TC_DONE] = 1;
    c[TC_TO_ACT] = 1 - me;
    c[TC_ACTIONS] += 1;
    const bool a0 = c[TC_ALLIN0] != 0, a1 = c[TC_ALLIN1] != 0;
    const bool equal = c[TC_COMM0] == c[TC_COMM1];
    const bool covered = (a0 && a1) || (a0 && c[TC_COMM0] <= c[TC_COMM1]) || (a1 && c[TC_COMM1] <= c[TC_COMM0]);
    const bool closed = !c[TC_DONE] && (equal || covered) && c[TC_ACTIONS] >= 2;
    if (closed) {
      c[TC_COMM0] = 0;
      c[TC_COMM1] = 0;
      c[TC_ACTIONS] = 0;
      c[TC_RAISES] = 0;
      c[TC_TO_ACT] = 1 - c[TC_BUTTON];
      c[TC_MIN_RAISE] = R.bb;
      if (c[TC_STREET] == 3) c[TC_DONE] = 1;   // the river closes into a showdown
      c[TC_STREET] += 1;
    }
    c[TC_PARENT] = parent_row_base + i;
    c[TC_ACTION] = a;
    int64_t* dst = children + k * TREE_COLS;
#pragma unroll
    for (int j = 0; j < TREE_COLS; ++j) dst[j] = c[j];
    ++k;
  }
}

static inline int tree_rules(const float* bins, int n_bins, int max_raises, int64_t bb, TreeRules& R) {
  if (n_bins < 0 || n_bins > TREE_MAX_BINS || (n_bins > 0 && !bins)) return P2_EINVAL;
  for (int b = 0; b < TREE_MAX_BINS; ++b) R.bins[b] = b < n_bins ? bins[b] : 0.f;
  R.n_bins = n_bins;
  R.max_raises = max_raises;
  R.bb = bb;
  return 0;
}

}  // namespace p2

extern "C" {

int64_t p2hip_tree_node_columns(void) { return p2::TREE_COLS; }

int p2hip_tree_legal(const int64_t* nodes, int64_t n, const float* host_bins, int n_bins, int max_raises,
                     int is_root_level, int expand, uint8_t* legal_out, int64_t* count_out, void* stream) {
  p2::TreeRules R;
  if (p2::tree_rules(host_bins, n_bins, max_raises, 0, R)) return P2_EINVAL;
  if (n < 0) return P2_EINVAL;
  if (n == 0) return 0;
  if (!nodes || !legal_out || !count_out) return P2_EINVAL;
  const unsigned grid = (unsigned)((n + p2::TREE_BLOCK - 1) / p2::TREE_BLOCK);
  hipLaunchKernelGGL(p2::tree_legal_kernel, dim3(grid), dim3(p2::TREE_BLOCK), 0, (hipStream_t)stream, nodes, n, R,
                     is_root_level, expand, legal_out, count_out);
  P2_LAUNCH_CHECK();
  return 0;
}

int p2hip_tree_step(const int64_t* parents, int64_t n, int64_t parent_row_base, const float* host_bins, int n_bins,
                    int max_raises, int64_t bb, int is_root_level, const int64_t* child_start, int64_t* children,
                    void* stream) {
  p2::TreeRules R;
  if (p2::tree_rules(host_bins, n_bins, max_raises, bb, R)) return P2_EINVAL;
  if (n < 0 || parent_row_base < 0) return P2_EINVAL;
  if (n == 0) return 0;
  if (!parents || !child_start || !children) return P2_EINVAL;
  const unsigned grid = (unsigned)((n + p2::TREE_BLOCK - 1) / p2::TREE_BLOCK);
  hipLaunchKernelGGL(p2::tree_step_kernel, dim3(grid), dim3(p2::TREE_BLOCK), 0, (hipStream_t)stream, parents, n,
                     parent_row_base, R, is_root_level, child_start, children);
  P2_LAUNCH_CHECK();
  return 0;
}

}  // extern "C"
