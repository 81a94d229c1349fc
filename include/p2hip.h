/* libp2hip.so -- C ABI of the MI355X (gfx950) kernels for the ReBeL search hot path.
 *
 * Conventions shared by every entry point
 *   - plain pointers and sizes only; all pointers are DEVICE pointers unless named host_*;
 *   - H = 1326 hole-card combos, combo (a<b) at index a*(103-a)/2 + (b-a-1); float32
 *     data rows are H floats, row-major, contiguous; index arrays are int64; masks are
 *     one byte per element (0 / non-zero); float rows must be 8-byte aligned;
 *   - work is enqueued on `stream` (a hipStream_t, NULL = default stream); nothing
 *     synchronises, allocates or keeps a pointer after returning;
 *   - return value: 0 on success, otherwise a hipError_t (1 = invalid argument).
 *
 * The reference (phulin/poker2) has no FFI: the interface each function replaces is the
 * Python/Triton wrapper cited next to it (paths relative to the reference's src/p2/).
 */
#ifndef P2HIP_H
#define P2HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int p2hip_abi_version(void);
int p2hip_device_count(void);
const char* p2hip_error_string(int code);

/* ---- 7-card hand ranker -------------------------------------------------------- */

/* cards [n,7] ids 0..51 of elem_size bytes (1, 2 or 8) -> out[n] packed int32 score
 * (type nibble << 20 | five kicker nibbles).  Replaces rank_7_cards_single_batch_triton,
 * env/rules_triton.py:96-117 (kernel :617-632). */
int p2hip_rank7_cards(const void* cards, int elem_size, int64_t n, int32_t* out, void* stream);

/* cards [n,2,7] -> out[n] in {-1,0,1}, 1 = first hand stronger.  Replaces
 * compare_7_cards_single_batch_triton, env/rules_triton.py:78-93 (kernel :600-614). */
int p2hip_compare7_cards(const void* cards, int elem_size, int64_t n, int32_t* out, void* stream);

/* planes [n,4,13] bytes -> packed score.  flush_first = 1: flush suit is the first suit
 * with >= 5 ranks (env/rules_triton.py:229-242); 0: the fullest suit (env/rules.py:215-219).
 * Replaces create_comparison_vector + packing, env/rules.py:136-299, :406-407. */
int p2hip_rank7_planes(const uint8_t* planes, int64_t n, int32_t* out, int flush_first, void* stream);

/* planes [n,2,4,13] bytes -> out[n] in {-1,0,1}.  Replaces compare_7_single_batch
 * (env/rules.py:390-409) and compare_7_single_batch_triton (env/rules_triton.py:36-51). */
int p2hip_compare7_planes(const uint8_t* planes, int64_t n, int32_t* out, int flush_first, void* stream);

/* ---- river showdown --------------------------------------------------------------- */

/* Bytes of one per-board strength table (fixed). */
int64_t p2hip_showdown_table_bytes(void);

/* boards [m,5] ids of elem_size bytes (1,2,4,8).  Any of the three outputs may be NULL.
 *   mode 0: combos touching the board are ranked as 6-card hands; ranks_out [m,H] int32 =
 *           dense 1-based strength group ids            (rank_hands, env/rules.py:66-133)
 *   mode 1: 7 card ids, hole cards first, repeated ids count twice; ranks_out = packed scores
 *                                                 (rank_hands_triton, env/rules_triton.py:120-148)
 *   order_out [m,H] int64: stable ascending argsort of the scores;
 *   table_out [m, p2hip_showdown_table_bytes()]: what p2hip_showdown_both reads; replaces the
 *           HandRankData built by _init_hand_rank_data, search/cfr_evaluator.py:406-482. */
int p2hip_showdown_setup(const void* boards, int elem_size, int64_t m, int mode, int32_t* ranks_out,
                         int64_t* order_out, uint8_t* table_out, void* stream);

/* The same table from hands that are already in strength order, without a board: per row and
 * sorted position the hand's two cards c1_sorted, c2_sorted [m,H] int32 and its tie group
 * [L_idx, R_idx) [m,H] int32 -- the inputs of showdown_ev_triton, search/fused_cfr_triton.py:2271-2314.
 * bad [m] int32 receives 1 for a row that does not list each of the 1326 hands once with
 * 0 <= L <= k < R <= H (its table is filled with in-range values but means nothing), else 0. */
int p2hip_showdown_setup_sorted(const int32_t* c1_sorted, const int32_t* c2_sorted, const int32_t* L_idx,
                                const int32_t* R_idx, int64_t m, uint8_t* table_out, int32_t* bad, void* stream);

/* beliefs [m,2,H] -> out [m,2,H]: blocker-corrected showdown EV of both players per hand,
 * times potential[m,p] / scale[m].  table_row [m] (or NULL = identity) selects the board
 * table of each node.  Replaces _showdown_value_both / _showdown_value,
 * search/cfr_evaluator.py:484-601. */
int p2hip_showdown_both(const float* beliefs, const uint8_t* tables, const int64_t* table_row,
                        const float* potential, const float* scale, int64_t m, float* out, void* stream);

/* ---- single-card chance node around the leaf network --------------------------------- */

/* For each of n public states (state i reads row root_indices[i] of pre_beliefs [*,2,H] and of
 * board [*,5] int64, -1 = empty slot; root_indices NULL = identity) and every card c not on its
 * board, in (i, c) ascending order: post_beliefs[s] = the ranges with the hands that hold c or
 * a board card removed, renormalised per player (uniform over the allowed hands when the sum
 * is <= 1e-12); board_samples[s] = the board with c in its first empty slot; root_lookup[s] = i.
 * sample_offsets [n+1] int64 (device) = prefix sums of 52 - cards on board.  source_rows = rows of
 * pre_beliefs / board, total_samples = rows the three outputs hold: a state whose row index lies
 * outside 0..source_rows-1 is skipped and no sample at or beyond total_samples is written, so
 * offsets that disagree with the boards cannot make the kernel leave its buffers; where a state
 * yields fewer samples than its share [sample_offsets[i], sample_offsets[i+1]) of the outputs (more
 * cards on its board than the offsets assume, no empty slot, a skipped row) the rest of the share is
 * filled with zeros and root_lookup with i, so no output row is left uninitialised.  Replaces the
 * expansion half of ChanceNodeHelper.single_card_chance_values,
 * search/chance_node_helper.py:394-443. */
int p2hip_chance_expand(const float* pre_beliefs, const int64_t* root_indices, const int64_t* board, int64_t n,
                        const int64_t* sample_offsets, int64_t source_rows, int64_t total_samples,
                        float* post_beliefs, int64_t* board_samples, int64_t* root_lookup, void* stream);

/* The same expansion written as rows of a value network's INPUT MATRIX: input_rows [total_samples, 2704]
 * in element type dtype (0 float32, 1 bfloat16, 2 float16), row s = the sample's 2 x 1326 ranges followed
 * by the 52-entry one-hot of its board (the state's cards and the dealt one) — what the reference builds
 * with a concatenation and a cast in front of its network (models/mlp/rebel_ffn.py forward; the ranges
 * are the `beliefs` of the MLPFeatures that search/chance_node_helper.py:445-456 assembles).
 * input_rows and pre_beliefs must be 16-byte aligned; board_samples may be NULL. */
int p2hip_chance_expand_input(const float* pre_beliefs, const int64_t* root_indices, const int64_t* board, int64_t n,
                              const int64_t* sample_offsets, int64_t source_rows, int64_t total_samples,
                              void* input_rows, int dtype, int64_t* board_samples, int64_t* root_lookup, void* stream);

/* expected[i] = mean of hand_values [S,2,H] over samples sample_offsets[i] .. sample_offsets[i+1]
 * (index_add_ + divide of search/chance_node_helper.py:467-477). */
int p2hip_chance_mean(const float* hand_values, const int64_t* sample_offsets, int64_t n, float* expected,
                      void* stream);

/* Three-card (flop) chance node, flop_chance_values of search/chance_node_helper.py:219-357.
 * out [n, n_flops, 2, H]: the ranges of state i (row root_indices[i] of pre_beliefs [*,2,H], NULL =
 * identity) with the hands holding a card of flops[f] (int64 [n_flops,3]) removed, renormalised per
 * player (uniform over the 1176 surviving hands when the sum is <= 1e-12). */
int p2hip_flop_expand(const float* pre_beliefs, const int64_t* root_indices, int64_t n, const int64_t* flops,
                      int64_t n_flops, float* out, void* stream);

/* out [n,2,H] (+= if accumulate) sum_f weight[f] * mean_q hand_values[i][f][p][perms[q][h]]:
 * hand_values [n, n_flops, 2, H], perms int16 [n_perms <= 24, H] hand permutations, 4-byte aligned
 * (the suit-orbit mean of _avg_over_perms, :18-28, and the weighted flop sum, :352-357).  Evaluated as
 * mean_q Y[perms[q][h]] with Y = sum_f weight[f] * hand_values[i][f][p] summed in float64 - the same
 * number, since the permutations do not depend on the flop: a read stream and one permutation pass.
 * shares >= 1 splits the flops over that many workgroups per (state, player) - use it when
 * 2 * n alone leaves most of the GPU idle (a few hundred workgroups are enough); shares > 1 needs workspace [shares, n, 2, H] float32, whose
 * partial sums are added in ascending order (results do not depend on scheduling). */
int p2hip_perm_mean(const float* hand_values, int64_t n, int64_t n_flops, const int16_t* perms, int n_perms,
                    const float* weight, int accumulate, float* out, float* workspace, int shares, void* stream);

/* p2hip_perm_mean for the case of ALL 24 suit permutations (the rows of combo_suit_permutation_tensor,
 * env/card_utils.py:161-181): the mean over the orbit of a hand is the mean over its class of
 * starting hands (13 pairs, 78 suited, 78 offsuit), so
 * out[i][p][h] (+)= sum_f weight[f] * mean over the class of h of hand_values[i][f][p][.].
 * Same arguments otherwise; the class tables are built into the library. */
int p2hip_orbit_mean(const float* hand_values, int64_t n, int64_t n_flops, const float* weight, int accumulate,
                     float* out, float* workspace, int shares, void* stream);

/* p2hip_orbit_mean without the workspace argument.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  The partial sums of shares > 1 go to an array inside the
 * library (P2HIP_ORBIT_SCRATCH_FLOATS float32 = 16 MiB per GPU, held until the process ends); the
 * call allocates and frees nothing.  shares * n * 2 * 1326 floats must fit it: a larger request
 * returns 2 (hipErrorOutOfMemory) before anything is launched.  Same results, bit for bit, as
 * p2hip_orbit_mean with the same `shares`.  Every call on one GPU uses that GPU's array: calls
 * that overlap on one GPU (different streams, threads) race; calls on one stream do not.
 * The array's address on a device is resolved by the first call made with that device current
 * (hipGetSymbolAddress, which may load the code object): make that call OUTSIDE graph capture — a call
 * with n = 0 does the resolution and nothing else (null pointers allowed).  Later calls on the device
 * neither allocate nor resolve anything. */
#define P2HIP_ORBIT_SCRATCH_FLOATS (4 * 1024 * 1024)
int p2hip_orbit_mean_static(const float* hand_values, int64_t n, int64_t n_flops, const float* weight,
                            int accumulate, float* out, int shares, void* stream);

/* ---- either side of the search in data generation ------------------------------------------ */

/* Context features and board of RebelFeatureEncoder.encode (models/mlp/rebel_feature_encoder.py:55-127)
 * for m public states: context [m,4] float32 (16-byte aligned) = (to_act, (to_act - button) mod 2,
 * clamp(pot / max(starting_stack0 + starting_stack1, 1), 0, 10), committed chips differ and
 * actions_this_round > 0); board_out [m,5] = last_board where the state is encoded before its
 * chance event (pre_chance [m] bytes; NULL = pre_chance_all for every state), else board.
 * All inputs int64: [m] or [m,2] / [m,5]. */
int p2hip_encode_context(const int64_t* to_act, const int64_t* button, const int64_t* starting_stacks,
                         const int64_t* pot, const int64_t* committed, const int64_t* actions_this_round,
                         const uint8_t* pre_chance, int pre_chance_all, const int64_t* last_board,
                         const int64_t* board, int64_t m, float* context, int64_t* board_out, void* stream);

/* Chip amounts of the action bins, the first result of HUNLTensorEnv.legal_bins_amounts_and_mask
 * (env/hunl_tensor_env.py:348-405): amounts [m, n_bins + 3] = -1 for fold and call,
 * to_call + trunc(bin * pot) for each bet bin (legal or not), the actor's stack for all-in.
 * host_bins: at most 5 pot fractions in HOST memory. */
int p2hip_bet_amounts(const int64_t* to_act, const int64_t* stacks, const int64_t* committed, const int64_t* pot,
                      int64_t m, const float* host_bins, int n_bins, int64_t* amounts, void* stream);

/* The rows of the node table that go to the leaf network, and its answers coming back: the evaluator's
 * `beliefs[model_indices]` gather and `latest_values.index_copy_(0, model_indices, values)`
 * (search/cfr_evaluator.py:1030-1043, search/fused_sparse_cfr_evaluator.py:431-445), with the
 * conversion to and from the network's dtype folded in (under autocast the reference casts in separate
 * passes).  src / dst [total_rows, 2, 1326] float32; rows [k] int64 (entries outside [0, total_rows)
 * are skipped); dtype 0 = float32, 1 = bfloat16 (round to nearest even), 2 = float16.
 * gather : dst[i, 0:2652] = src[rows[i]] in dst_dtype; dst rows are dst_stride ELEMENTS apart, so the
 *          target may be the network's input matrix with further feature columns behind the ranges.
 * scatter: dst[rows[i]] = src[i, 0:2652] as float32; src rows are src_stride elements apart.
 * Both sides 8-byte aligned; strides even (float32) or a multiple of four (16-bit types). */
int p2hip_gather_leaf_rows(const float* src, const int64_t* rows, int64_t k, int64_t total_rows, void* dst, int dst_dtype,
                           int64_t dst_stride, void* stream);
int p2hip_scatter_leaf_rows(const void* src, int src_dtype, int64_t src_stride, const int64_t* rows, int64_t k, float* dst,
                            int64_t total_rows, void* stream);

/* Policy targets of CFREvaluator.training_data (search/cfr_evaluator.py:1392-1393; _pull_back,
 * search/sparse_cfr_evaluator.py:465-489): out [n_rows, H, num_actions] with
 * out[k,h,a] = policy_avg[c,h] for the child c of node rows[k] that action a leads to, 0 for
 * actions without a child.  policy_avg [total,H]; the three index arrays are [total] int64. */
int p2hip_policy_targets(const float* policy_avg, const int64_t* rows, int64_t n_rows, const int64_t* child_offsets,
                         const int64_t* child_count, const int64_t* action_from_parent, int num_actions, float* out,
                         void* stream);

/* ---- local best response -------------------------------------------------------------- */

/* One tree level of _best_response_values (search/cfr_evaluator.py:636-714), in place on
 * values [total,2,H]: for the parents parent_base .. parent_base+num_parents-1 that have
 * children (rows child_offsets[p] .. +child_count[p], at most max_children <= 8: a parent with more
 * is skipped), the player to act takes the
 * per-hand maximum over children where deviating_player[p] == to_act[p] and the policy-weighted
 * mean elsewhere; the other player gets the expectation of its child values under the
 * blocker-projected action probabilities.  Rows without children are left as they are (leaf
 * values).  Call once per level, deepest parents first.  All index arrays are [total] int64. */
int p2hip_best_response_level(float* values, const float* policy, const float* beliefs, const int64_t* to_act,
                              const int64_t* deviating_player, const int64_t* child_offsets,
                              const int64_t* child_count, int64_t parent_base, int64_t num_parents,
                              int max_children, void* stream);

/* ---- betting tree on the device ----------------------------------------------------------- */

/* A node is a row of p2hip_tree_node_columns() int64 (21): street, to_act, button, pot, stack0,
 * stack1, committed0, committed1, min_raise, actions_this_round, is_allin0, is_allin1,
 * starting_stack0, starting_stack1, done, raises, scale (float32 bits), root row, parent row (-1),
 * action from parent (-1), fold reward (float32 bits).  Two launches per level replace the host
 * depth loop over HUNLTensorEnv (search/sparse_cfr_evaluator.py:142-306; rules of
 * env/hunl_tensor_env.py:348-423, 684-724, 766-992); the caller prefix-sums count_out in
 * between.  host_bins: bet fractions of the pot, at most 5, in HOST memory. */
int64_t p2hip_tree_node_columns(void);

/* legal_out [n, n_bins+3] bytes: legal action bins (fold, call, bets..., all-in) of every node;
 * count_out [n]: children the node gets (0 unless `expand`; 0 below the root level when the
 * node's betting round has just closed).  max_raises < 0: no cap on bets and raises per round. */
int p2hip_tree_legal(const int64_t* nodes, int64_t n, const float* host_bins, int n_bins, int max_raises,
                     int is_root_level, int expand, uint8_t* legal_out, int64_t* count_out, void* stream);

/* Children of the n parents (global rows parent_row_base ..), action ascending, written from row
 * child_start[i] of `children` on (exclusive prefix sums of count_out). */
int p2hip_tree_step(const int64_t* parents, int64_t n, int64_t parent_row_base, const float* host_bins, int n_bins,
                    int max_raises, int64_t bb, int is_root_level, const int64_t* child_start, int64_t* children,
                    void* stream);

/* ---- unblocked (card-compatible) mass --------------------------------------------- */

/* target [rows,H] -> out [rows,H] = max(S - cs[a] - cs[b] + t, 0).  Replaces
 * calculate_unblocked_mass (env/card_utils.py:196-222) and unblocked_mass_triton
 * (search/fused_cfr_triton.py:1110-1157). */
int p2hip_unblocked_mass(const float* target, int64_t rows, float* out, void* stream);

/* beliefs [total,2,H], to_act [total]; out[r] = unblocked(beliefs[r, to_act[r] ^ opponent])
 * for r < top.  Replaces unblocked_mass_opp_at_parents_triton,
 * search/fused_cfr_triton.py:1067-1107. */
int p2hip_unblocked_mass_by_player(const float* beliefs, const int64_t* to_act, int64_t top, int opponent,
                                   float* out, void* stream);

/* out[c] = d > eps ? unblocked(numer[c]) / d : 0, d = unblocked(denom[parent_index[c]])
 * (parent_index NULL = identity).  Replaces unblocked_mass_ratio_indirect_triton /
 * unblocked_mass_ratio_triton, search/fused_cfr_triton.py:1499-1602. */
int p2hip_unblocked_mass_ratio(const float* numer, const float* denom, const int64_t* parent_index,
                               int64_t rows, float eps, float* out, void* stream);

/* The same quotient from denominators that are already unblocked masses: d = denom_unblocked[parent_index[c]]
 * ([parents,H], e.g. from p2hip_unblocked_mass).  Siblings share their parent's row, so its card sums are
 * taken once per parent; the reference passes precomputed denominator statistics for the same purpose
 * (denom_stats of unblocked_mass_ratio_indirect_triton, search/fused_cfr_triton.py:1499-1556). */
int p2hip_unblocked_mass_ratio_of(const float* numer, const float* denom_unblocked, const int64_t* parent_index,
                                  int64_t rows, float eps, float* out, void* stream);

/* ---- per-operation CFR kernels (search/fused_cfr_triton.py) ------------------------- */
/* Scalars that depend on the iteration number are 0-D device tensors (const float*). */

/* fused_dcfr_update_with_tensors_ :200-235 (kernel :71-120).  n = element count (even).
 * positive_out may be NULL. */
int p2hip_dcfr_update(float* cumulative_regrets, float* regret_weight_sums, const float* regrets,
                      const float* t_alpha_num, const float* t_beta_num, const float* t_alpha_den,
                      const float* t_beta_den, int64_t n, int apply_dcfr, int cfr_plus, float* positive_out,
                      void* stream);

/* fused_block_and_normalize_beliefs_ :286-335.  target has rows*1 rows of H; row r uses
 * mask / fallback row r / players_per_row. */
int p2hip_block_and_normalize(float* target, const uint8_t* allowed, const float* allowed_prob, int64_t rows,
                              int players_per_row, float eps, void* stream);

/* fused_regret_matching_divide_ :369-399 */
int p2hip_regret_matching_divide(const float* positive, const float* denom, const float* fallback, float* out,
                                 int64_t n, float eps, void* stream);

/* fused_weight_child_values :438-477; values/out [m,2,H] */
int p2hip_weight_child_values(const float* values, const int64_t* prev_actor, const float* policy_hero,
                              const float* policy_opp, float* out, int64_t m, void* stream);

/* fused_update_average_values_with_tensors_ :538-560 */
int p2hip_update_average_values(float* values_avg, const float* latest, const float* old_w, const float* new_w,
                                const float* inv_total, int64_t n, void* stream);

/* fused_avg_values_zero_sum_ :623-668; ignore_mask [nodes] bytes or NULL */
int p2hip_avg_values_zero_sum(float* values_avg, const float* latest, const float* beliefs,
                              const uint8_t* ignore_mask, const float* old_w, const float* new_w,
                              const float* inv_total, int64_t nodes, int enforce_zero_sum, void* stream);

/* fused_regret_tail_ :712-766; writes rows [bottom,total) of regrets */
int p2hip_regret_tail(float* regrets, const float* values_achieved, const float* actor_values,
                      const float* src_weights, const int64_t* parent_index, const int64_t* prev_actor,
                      int64_t bottom, int64_t total, void* stream);

/* fused_average_policy_mix_with_tensors_ :879-914 */
int p2hip_average_policy_mix(float* policy_probs_avg, const float* policy_probs, const float* self_reach,
                             const float* self_reach_avg, const int64_t* to_act, const int64_t* parent_index,
                             const float* old_w, const float* new_w, const float* total_w, int64_t bottom,
                             int64_t total, float eps, void* stream);

/* fused_parent_sum :1279-1313 -> out [num_parents,H] */
int p2hip_parent_sum(const float* values, const int64_t* child_offsets, const int64_t* child_count,
                     int64_t num_parents, float* out, void* stream);

/* fused_sibling_sum :1355-1398 -> out [num_children,H], row = child - bottom */
int p2hip_sibling_sum(const float* values, const int64_t* child_offsets, const int64_t* child_count,
                      int64_t num_parents, int64_t bottom, float* out, void* stream);

/* fused_divide_by_parent_sum_ :1316-1352; out may alias pos or fallback */
int p2hip_divide_by_parent_sum(const float* pos, const float* fallback, const float* parent_sum,
                               const int64_t* parent_index, float* out, int64_t num_children, float eps,
                               void* stream);

/* fused_model_values_mix_with_tensors :1658-1680 */
int p2hip_model_values_mix(const float* hand_values, const float* last_values, const float* onon,
                           const float* oon, float* out, int64_t n, void* stream);

/* fused_model_values_mix_zero_sum :1739-1775; tensors [rows,2,H] */
int p2hip_model_values_mix_zero_sum(const float* hand_values, const float* last_values, const float* beliefs,
                                    const float* onon, const float* oon, float* out, int64_t rows,
                                    int enforce_zero_sum, void* stream);

/* fused_weighted_parent_sum :1838-1889; child_offsets/count already sliced to the depth */
int p2hip_weighted_parent_sum(float* values, const int64_t* prev_actor, const float* policy_hero,
                              const float* policy_opp, const int64_t* child_offsets, const int64_t* child_count,
                              int64_t num_parents, int64_t parent_base, void* stream);

/* fused_reach_weights_depth_ :1944-1986; rows [start,end) */
int p2hip_reach_weights_depth(float* reach, const float* policy, const uint8_t* allowed_mask,
                              const int64_t* parent_index, const int64_t* prev_actor, int64_t start, int64_t end,
                              void* stream);

/* fused_deep_beliefs_ :2039-2092; rows [n_roots,total) are written */
int p2hip_deep_beliefs(float* out, const float* root_beliefs, const float* reach, const float* allowed_prob,
                       const int64_t* root_index, int64_t n_roots, int64_t total, float eps, void* stream);

/* policy_probs_sample <- where(t_sample == *t_now, policy_probs, policy_probs_sample),
 * search/fused_sparse_cfr_evaluator.py:494-499 */
int p2hip_sample_snapshot(const float* policy_probs, float* policy_probs_sample, const int64_t* t_sample,
                          const int64_t* t_now, int64_t total, void* stream);

/* ---- one kernel = one CFR iteration ------------------------------------------------- */

/* Device pointers of one subgame batch.  Tree arrays and state tensors are the evaluator's
 * own (row-major over all nodes of all roots); the rest is derived once per subgame:
 *   node_flags [total] bytes: bit0 = river showdown row, bit1 = terminal row, bit2 = the row has children,
 *             bit3 = childless row whose ranges feed a leaf evaluation (a showdown row, or a row the caller's
 *             leaf network is asked about); bits 2 and 3 are read by lean launches only
 *   root_parent_offsets [roots+1], root_parents: rows that have children, per root, ascending
 *   root_showdown_offsets [roots+1], root_showdown_nodes: river showdown rows per root
 *   tables [roots, p2hip_showdown_table_bytes()] (NULL when no row is a showdown)
 *   potential [total,2] float, scale [total] float: showdown pay-off factors per row
 *   scratch [total,H] float workspace (may be NULL when reach_avg_prev is given)
 *   fscal[8]: t^alpha, t^beta, t^alpha+1, t^beta+1, mix_old, mix_new, mix_old+mix_new, 1/(mix_old+mix_new)
 *   iscal[8]: t, apply_dcfr, cfr_plus, average_policy_is_copied, enforce_zero_sum, update_average_values,
 *             cfr_avg (regret weights and showdown values from beliefs_avg), linear (regrets of player t mod 2
 *             dropped, no discount) */
typedef struct P2HipIterArgs {
  const int64_t* child_offsets;
  const int64_t* child_count;
  const int64_t* to_act;
  const uint8_t* node_flags;
  const int64_t* root_parent_offsets;
  const int64_t* root_parents;
  const int64_t* root_showdown_offsets;
  const int64_t* root_showdown_nodes;
  const int64_t* t_sample;
  const uint8_t* allowed;
  const float* allowed_prob;
  const uint8_t* tables;
  const float* potential;
  const float* scale;
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
  float* scratch;
  const float* fscal;
  const int64_t* iscal;
  /* Optional work items (both NULL: one item per root, item w = root w, n_items = roots).
   * root_parent_offsets / root_showdown_offsets then have n_items + 1 entries and delimit, per item,
   * the families and showdown rows one workgroup walks; item_root [n_items] names the root an item
   * belongs to.  With few roots a root's tree may be cut at a level into a top item (item_top = 1: the
   * families and showdown rows above the cut) and one subtree item per node of the cut level that has
   * children (item_top = 0); every family and showdown row belongs to exactly one item.  An iteration
   * is then four launches: all items with phases 4, top items with 8, subtree items with 8|2, top items
   * with 2 (the regret part of a family reads rows that the reach / belief part of the family above
   * rewrites, so it runs everywhere first).  The tops may be cut again the same way (tiers of items:
   * reach / belief parts tier by tier downwards, value parts upwards; two launches more per cut). */
  const int64_t* item_root;
  const uint8_t* item_top;
  /* Optional, [total,2,H]: reach_avg as the PREVIOUS iteration left it, in a buffer of its own.  The
   * average-policy mix (search/fused_sparse_cfr_evaluator.py:355-398) weighs the old average policy by the
   * parent's reach_avg from before this iteration; with NULL the kernel saves that row in `scratch`
   * before it overwrites reach_avg in place.  A caller that keeps two reach_avg buffers and swaps them
   * from iteration to iteration passes the other one here and saves a row write and a row read per
   * parent.  Root rows of both buffers hold the roots' reach (1); must differ from reach_avg. */
  const float* reach_avg_prev;
} P2HipIterArgs;

/* One workgroup per root runs the whole iteration of FusedSparseCFREvaluator.cfr_iteration
 * (search/fused_sparse_cfr_evaluator.py:478-533; base search/cfr_evaluator.py:1330-1381) with
 * cfr_avg = False: sample snapshot, instantaneous regrets, DCFR update, regret matching, reach,
 * beliefs, average policy, reach_avg, beliefs_avg (phases bit 0; bit 2 = the regret part alone, bit 3 = the
 * reach / belief / average-policy part alone); showdown leaf values, value backup, average values
 * (phases bit 1).  phases bit 4 (16) marks a LEAN iteration, for callers that run many iterations and
 * look at the state only after the last (evaluate_cfr, search/cfr_evaluator.py:1497-1528): the reach /
 * belief part then stores only rows that a later part of this iteration or the next iteration reads —
 * reach and reach_avg of rows with children, beliefs of rows with children or a leaf evaluation
 * (node_flags bits 2, 3), beliefs_avg only under cfr_avg or enforce_zero_sum.  The rows left out are
 * functions of rows that are kept: one iteration without the bit afterwards leaves all eleven tensors
 * bit-identical to a run that never set it.  host_args is a HOST pointer to a struct of device
 * pointers; n_items = workgroups to launch (= roots unless the work-item lists are given);
 * max_children = largest child count in the tree (<= 8). */
int p2hip_cfr_iteration(const P2HipIterArgs* host_args, int64_t n_items, int max_children, int phases,
                        void* stream);

/* Copy 8 floats and 8 int64 from HOST arrays into the device arrays fscal[8] / iscal[8] read by
 * p2hip_cfr_iteration.  The values travel as kernel arguments: the host arrays may be reused as
 * soon as the call returns.  Plays the role of TScalars.update, search/fused_cfr_triton.py:2131-2158. */
int p2hip_write_scalars(float* fscal, int64_t* iscal, const float* host_f, const int64_t* host_i, void* stream);

/* dst[0..n) (device, n <= 8) = host_values[0..n): the values travel as kernel arguments, in
 * stream order, so the scalar-taking wrappers (fused_dcfr_update_ etc., fused_cfr_triton.py:123-197)
 * need no host-to-device copies.  No counterpart in the reference, which passes Python floats to
 * Triton. */
int p2hip_upload_floats(float* dst, const float* host_values, int n, void* stream);

/* ---- measurement aid ------------------------------------------------------------------------ */

/* No counterpart in the reference and not on the search path: a structure-free element-wise stream over
 * n_read input and n_write output arrays of `pairs` float2 each (array k starts k * pairs float2 after the
 * base pointer), for (n_read, n_write) in {(5,7), (1,1), (2,0), (0,2)}; non_temporal != 0 marks every access
 * non-temporal.  bench.py times it to report what HBM gives a kernel of the iteration kernel's read / write
 * mix on the same machine. */
int p2hip_stream_probe(const float* in, float* out, int64_t pairs, int n_read, int n_write, int non_temporal,
                       void* stream);

/* ---- placement aid --------------------------------------------------------------------------- */

/* No counterpart in the reference (PyTorch's allocator places its tensors).  The iteration kernel writes
 * about ten tensors at once, and the card's memory takes that 10 % faster when the written tensors lie in
 * two different thirds (~96 GiB each) of its physical address space instead of one.  Where an allocation
 * lies physically is not visible, but it can be measured and steered:
 *
 * p2hip_placement_probe: time of one launch (ms, mean of `reps`, 1..64) of a row-streaming kernel - 12 rows
 *   of 1326 floats read and 8 written per node - whose 20 arrays are dealt alternately to the buffers `a`
 *   and `b` (ten arrays spread over the first `bytes_each` bytes of each; at least 14 MB each; contents
 *   are OVERWRITTEN).  Two buffers in different thirds take about a fifth less than two halves of one
 *   buffer, which is the comparison to make.  Synchronises the stream.
 * p2hip_device_reserve / _release: `bytes` of device memory from hipMalloc, untouched, to be HELD while
 *   something else is allocated so that it lands elsewhere; out of memory: the HIP error code, *out =
 *   NULL, nothing left pending.  Release synchronises the device. */
int p2hip_placement_probe(void* a, void* b, int64_t bytes_each, int reps, float* ms_out, void* stream);
int p2hip_device_reserve(int64_t bytes, void** out);
int p2hip_device_release(void* block);

#ifdef __cplusplus
}
#endif
#endif /* P2HIP_H */
