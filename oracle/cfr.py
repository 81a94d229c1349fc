"""CFR iteration on the sparse tree, numpy float32 restatement of the
reference's un-fused (CPU-runnable) torch path.  TEST INFRASTRUCTURE ONLY.

Follows ``src/p2/search/cfr_evaluator.py`` (base class, plain torch ops) with
the sparse tree helpers of ``src/p2/search/sparse_cfr_evaluator.py``:

  fan_out / pull_back_sum / fan_out_deep   <- sparse_cfr_evaluator.py:428-538
  normalize_beliefs                        <- cfr_evaluator.py:254-273
  mixing_weights                           <- :285-303
  calculate_reach_weights                  <- :332-361
  propagate_all_beliefs                    <- :363-380
  initialize_subgame (state part)          <- :770-828, sparse :262-301
  initialize_policy_and_beliefs            <- :830-886 (+ :305-330, sparse :312-323)
  set_leaf_values                          <- :1025-1047, :982-1018
  compute_expected_values                  <- :1049-1115
  compute_instantaneous_regrets            <- :1117-1165
  update_policy                            <- :1167-1193
  update_average_policy                    <- :1195-1258
  update_average_values / zero-sum         <- :1260-1274, :957-980
  apply_schedules                          <- :1294-1328
  cfr_iteration                            <- :1330-1381
  evaluate_cfr (loop part)                 <- :1497-1528
  warm_start                               <- :888-955

Every state tensor keeps the reference's name, shape and meaning; a child's row
holds the quantity "for the action that leads to it".  Arithmetic is float32
with Python-scalar operands rounded to float32 first, as torch does.

PINNED by vectors written from the reference itself: tests/golden/cfr_golden.npz holds the
11 state tensors of the reference's own SparseCFREvaluator (run on the CPU of the build
container by tests/golden/gen_cfr_golden.py) after the preparation step and after iterations
of eight searches — discounted, discounted_plus with delay, linear + cfr_avg with and without
CFR+, standard, warm start ``model_br`` and ``model`` (twice); depths 2 and 3 — and its local exploitability;
tests/test_oracle_cfr_golden.py holds this restatement to them (1e-5 relative on the first
iterations).  Further pinned by (tests/test_oracle_cfr.py) an explicit hand-pair game that
reproduces reach, conditional values and regrets at depths 2-4, the closed form of the average
policy, a textbook CFR / best response, and structural identities.

The ``fused_variant`` switches (what FusedSparseCFREvaluator does differently: root rows of
self_reach keep 1.0 on board-blocked hands, root beliefs are not re-normalised, average values
use (a*old + v*new) * (1/(old+new)), linear CFR accumulates without the CFR+ clamp) are PINNED by
tests/golden/fused_cfr_golden.npz: the same eight searches run through the reference's own
FusedSparseCFREvaluator, its Triton kernels executing under Triton's CPU interpreter
(``gen_cfr_golden.py --fused``); with ``fused_variant=True`` this restatement is held to those
vectors on every entry, board-blocked hands included (tests/test_oracle_cfr_golden.py).  One of the
eight (model warm start with a discount delay shorter than the warm start) leaves NaN in the
reference's average policy — its device scalars are still zero at that point — so the four
tensors derived from it are compared with the base class's vectors only.
"""
from __future__ import annotations

from typing import Callable

import numpy as np

from .cards import NUM_HANDS, allowed_hands_for_boards
from .showdown import init_hand_rank_data, showdown_value_both
from .unblocked import calculate_unblocked_mass

F32 = np.float32
CFR_TYPES = ("standard", "linear", "discounted", "discounted_plus")


def padded_indices(mask: np.ndarray, alignment: int) -> np.ndarray:
    """cfr_evaluator.py:90-101 -- indices of True entries, padded to a multiple
    of ``alignment`` by repeating the last one."""
    idx = np.nonzero(mask)[0]
    if idx.size > 0 and idx.size % alignment != 0:
        pad = alignment - idx.size % alignment
        idx = np.concatenate([idx, np.repeat(idx[-1:], pad)])
    return idx


class OracleCFR:
    def __init__(
        self,
        tree: dict,
        boards: np.ndarray,
        initial_beliefs: np.ndarray | None = None,
        *,
        cfr_type: str = "discounted",
        dcfr_alpha: float = 1.5,
        dcfr_beta: float = 0.0,
        dcfr_gamma: float = 2.0,
        dcfr_delay: int = 0,
        cfr_plus: bool = False,
        cfr_avg: bool = False,
        cfr_iterations: int = 200,
        warm_start_iterations: int = 0,
        warm_start_type: str = "model_br",
        warm_start_multiplier: float = 1.0,
        use_final_policy_values: bool = False,
        enforce_zero_sum: bool = False,
        dcfr_alpha_final: float | None = None,
        dcfr_beta_final: float | None = None,
        dcfr_gamma_final: float | None = None,
        leaf_value_fn: Callable | None = None,
        policy_logits_fn: Callable | None = None,
        t_sample_roots: np.ndarray | None = None,
        ranker=None,
        fused_variant: bool = False,
    ) -> None:
        assert cfr_type in CFR_TYPES
        # fused_variant=True follows FusedSparseCFREvaluator where it departs from the base
        # class on rows / hands that carry no probability mass:
        #   * root rows of self_reach(_avg) stay 1.0 on board-blocked hands (the fused reach
        #     kernel only writes child rows, fused_sparse_cfr_evaluator.py:153-172);
        #   * root rows of beliefs(_avg) are not re-normalised every iteration (the fused
        #     belief kernel skips them, fused_cfr_triton.py:2008-2011);
        #   * average values use (a*old + v*new) * (1/(old+new)) (fused_cfr_triton.py:604-605).
        self.fused_variant = fused_variant
        self.tree = tree
        self.depth_offsets = list(tree["depth_offsets"])
        self.tree_depth = max(0, len(self.depth_offsets) - 2)
        self.total_nodes = self.depth_offsets[-1]
        self.root_nodes = self.depth_offsets[1]
        self.num_actions = tree["legal_mask"].shape[1]
        self.parent_index = tree["parent_index"]
        self.action_from_parent = tree["action_from_parent"]
        self.child_count = tree["child_count"]
        self.child_offsets = tree["child_offsets"]
        self.prev_actor = tree["prev_actor"]
        self.to_act = tree["to_act"]
        self.done = tree["done"]
        self.leaf_mask = tree["leaf_mask"]
        self.new_street_mask = tree["new_street_mask"]
        self.legal_mask = tree["legal_mask"]
        self.cfr_type = cfr_type
        self.dcfr_alpha = self.dcfr_alpha_initial = dcfr_alpha
        self.dcfr_beta = self.dcfr_beta_initial = dcfr_beta
        self.dcfr_gamma = self.dcfr_gamma_initial = dcfr_gamma
        self.dcfr_alpha_final = dcfr_alpha_final
        self.dcfr_beta_final = dcfr_beta_final
        self.dcfr_gamma_final = dcfr_gamma_final
        self.dcfr_delay = dcfr_delay
        self.cfr_plus = cfr_plus
        self.cfr_avg = cfr_avg
        self.cfr_iterations = cfr_iterations
        self.warm_start_iterations = warm_start_iterations
        assert warm_start_type in ("model", "model_br")
        self.warm_start_type = warm_start_type
        self.warm_start_multiplier = warm_start_multiplier
        self.use_final_policy_values = use_final_policy_values
        self.enforce_zero_sum = enforce_zero_sum
        self.leaf_value_fn = leaf_value_fn
        self.policy_logits_fn = policy_logits_fn
        self.last_model_values = None

        N, T = self.root_nodes, self.total_nodes
        z1 = lambda: np.zeros((T, NUM_HANDS), F32)  # noqa: E731
        z2 = lambda: np.zeros((T, 2, NUM_HANDS), F32)  # noqa: E731
        self.policy_probs, self.policy_probs_avg, self.policy_probs_sample = z1(), z1(), z1()
        self.cumulative_regrets, self.regret_weight_sums = z1(), z1()
        self.uniform_policy = z1()
        cc_dest = self.fan_out(self.child_count)
        self.uniform_policy[N:] = (F32(1.0) / cc_dest.astype(F32))[:, None]
        self.beliefs, self.beliefs_avg = z2(), z2()
        self.self_reach, self.self_reach_avg = z2(), z2()
        self.self_reach[:N] = 1.0
        self.self_reach_avg[:N] = 1.0
        self.latest_values = z2()
        fold = tree["fold_mask"]
        self.latest_values[fold, 0] = tree["reward"][fold][:, None]
        self.latest_values[fold, 1] = -tree["reward"][fold][:, None]
        self.values_avg = self.latest_values.copy()

        if initial_beliefs is None:
            initial_beliefs = np.full((N, 2, NUM_HANDS), 1.0 / NUM_HANDS, F32)
        initial_beliefs = np.asarray(initial_beliefs, dtype=F32)
        self.beliefs[:N] = initial_beliefs
        self.beliefs_avg[:N] = initial_beliefs
        self.root_pre_chance_beliefs = initial_beliefs.copy()

        model_mask = self.leaf_mask & ~self.done
        self.model_indices = padded_indices(model_mask, N)
        root_allowed, root_prob = allowed_hands_for_boards(np.asarray(boards)[:N])
        self.allowed_hands = self.fan_out_deep(root_allowed)
        self.allowed_hands_prob = self.fan_out_deep(root_prob)

        sd_mask = tree["showdown_mask"]
        self.showdown_indices = padded_indices(sd_mask, max(1, N // 2))
        self.showdown_potential = tree["showdown_potential"][self.showdown_indices]
        self.showdown_scale = tree["scale"][self.showdown_indices]
        self.root_index = self.fan_out_deep(np.arange(N))
        kw = {} if ranker is None else {"ranker": ranker}
        if self.showdown_indices.size:
            sd_boards = np.asarray(boards)[self.root_index[self.showdown_indices]]
            self.hand_rank_data = init_hand_rank_data(
                sd_boards, self.allowed_hands[self.showdown_indices], **kw)
        else:
            self.hand_rank_data = None
        if t_sample_roots is None:
            t_sample_roots = np.full(N, -1, dtype=np.int64)
        self.t_sample = self.fan_out_deep(np.asarray(t_sample_roots, dtype=np.int64))

    # ---- tree helpers (sparse_cfr_evaluator.py:428-538) ---------------------
    def _level(self, level):
        if level is None:
            return 0, self.depth_offsets[-2], self.depth_offsets[1], self.total_nodes
        return (self.depth_offsets[level], self.depth_offsets[level + 1],
                self.depth_offsets[level + 1], self.depth_offsets[level + 2])

    def fan_out(self, x: np.ndarray, level: int | None = None) -> np.ndarray:
        ps, pe, _, _ = self._level(level)
        return np.repeat(x[ps:pe], self.child_count[ps:pe], axis=0)

    def pull_back_sum(self, src: np.ndarray, out: np.ndarray, level: int | None = None) -> None:
        _, _, cs, ce = self._level(level)
        if src.shape[0] == self.total_nodes:
            src = src[cs:ce]
        assert src.shape[0] == ce - cs
        np.add.at(out, self.parent_index[cs:ce], src)

    def fan_out_deep(self, x: np.ndarray) -> np.ndarray:
        out = np.zeros((self.total_nodes,) + x.shape[1:], dtype=x.dtype)
        out[: self.root_nodes] = x
        for d in range(self.tree_depth):
            s, e = self.depth_offsets[d + 1], self.depth_offsets[d + 2]
            out[s:e] = self.fan_out(out, d)
        return out

    # ---- beliefs / reach ------------------------------------------------------
    def block_beliefs(self, target: np.ndarray) -> None:
        target[np.broadcast_to(~self.allowed_hands[:, None, :], target.shape)] = 0.0

    def normalize_beliefs(self, target: np.ndarray) -> None:
        denom = target.sum(axis=-1, keepdims=True, dtype=F32)
        safe = np.where(denom > F32(1e-5), denom, F32(1.0))
        target[:] = np.where(denom > F32(1e-5), target / safe, self.allowed_hands_prob[:, None, :])

    def calculate_reach_weights(self, target: np.ndarray, policy: np.ndarray) -> None:
        for d in range(self.tree_depth):
            s, e = self.depth_offsets[d + 1], self.depth_offsets[d + 2]
            dest = self.fan_out(target, d)
            rows = np.arange(e - s)
            dest[rows, self.prev_actor[s:e]] *= policy[s:e]
            target[s:e] = dest
        if self.fused_variant:
            n = self.root_nodes
            target[n:][np.broadcast_to(~self.allowed_hands[n:, None, :], target[n:].shape)] = 0.0
        else:
            self.block_beliefs(target)

    def propagate_all_beliefs(self, target: np.ndarray, reach: np.ndarray) -> None:
        roots = target[: self.root_nodes].copy()
        target[:] = self.fan_out_deep(roots) * reach
        self.normalize_beliefs(target)
        if self.fused_variant:
            target[: self.root_nodes] = roots

    # ---- schedules / weights --------------------------------------------------
    def mixing_weights(self, t: int):
        if self.cfr_type == "standard":
            return t, 1
        if self.cfr_type == "linear":
            return t, 2
        if self.cfr_type == "discounted":
            return t ** self.dcfr_gamma, (t + 1) ** self.dcfr_gamma
        if t > self.dcfr_delay:
            return t - self.dcfr_delay, 2
        return 0, 1

    def apply_schedules(self, t: int) -> None:
        total = max(1, self.cfr_iterations - self.warm_start_iterations)
        prog = max(0, t - self.warm_start_iterations)
        x = min(1.0, max(0.0, prog / float(total)))

        def lerp(a0, a1):
            return a0 if a1 is None else a0 + (a1 - a0) * x

        self.dcfr_alpha = lerp(self.dcfr_alpha_initial, self.dcfr_alpha_final)
        self.dcfr_beta = lerp(self.dcfr_beta_initial, self.dcfr_beta_final)
        self.dcfr_gamma = lerp(self.dcfr_gamma_initial, self.dcfr_gamma_final)

    # ---- initial policy (cfr_evaluator.py:830-886) ----------------------------
    def initialize_policy_and_beliefs(self) -> None:
        self.policy_probs[:] = 0.0
        if self.tree_depth == 0:
            self.block_beliefs(self.beliefs)
            self.normalize_beliefs(self.beliefs)
        for d in range(self.tree_depth):
            o, on, onn = self.depth_offsets[d], self.depth_offsets[d + 1], self.depth_offsets[d + 2]
            k = on - o
            if self.policy_logits_fn is None:
                logits = np.zeros((k, NUM_HANDS, self.num_actions), F32)
            else:
                logits = np.asarray(self.policy_logits_fn(self.beliefs, np.arange(o, on)), F32)
            legal = self.legal_mask[o:on][:, None, :]
            masked = np.where(legal, logits, F32(-np.inf))
            mx = masked.max(axis=-1, keepdims=True)
            mx = np.where(np.isfinite(mx), mx, F32(0.0))
            ex = np.where(legal, np.exp(masked - mx, dtype=F32), F32(0.0))
            den = ex.sum(axis=-1, keepdims=True, dtype=F32)
            probs = np.where(den > 0, ex / np.where(den > 0, den, F32(1.0)), F32(0.0))
            probs[self.child_count[o:on] == 0] = 0.0
            src = np.transpose(probs, (0, 2, 1))  # [k, B, H]
            self.policy_probs[on:onn] = src[self.parent_index[on:onn] - o, self.action_from_parent[on:onn]]
            # beliefs one level down: copy parent, multiply the actor's slice by the policy
            child = self.fan_out(self.beliefs, d)
            rows = np.arange(onn - on)
            child[rows, self.prev_actor[on:onn]] *= self.policy_probs[on:onn]
            self.beliefs[on:onn] = child
            self.block_beliefs(self.beliefs)
            self.normalize_beliefs(self.beliefs)
        self.calculate_reach_weights(self.self_reach, self.policy_probs)
        self.policy_probs_avg[:] = self.policy_probs
        self.self_reach_avg[:] = self.self_reach
        self.beliefs_avg[:] = self.beliefs

    # ---- leaf values ------------------------------------------------------------
    def maybe_enforce_zero_sum(self, values, beliefs, ignore_mask=None):
        if not self.enforce_zero_sum:
            return values
        s = (values * beliefs).sum(axis=2, keepdims=True, dtype=F32).mean(axis=1, keepdims=True, dtype=F32)
        if ignore_mask is not None:
            s = np.where(ignore_mask[:, None, None], F32(0.0), s)
        return (values - s).astype(F32)

    def set_leaf_values(self, t: int, beliefs: np.ndarray | None = None) -> None:
        if beliefs is None:
            beliefs = self.beliefs_avg if self.cfr_avg else self.beliefs
        if self.model_indices.size:
            mb = beliefs[self.model_indices]
            if self.leaf_value_fn is None:
                hv = np.zeros_like(mb)
            else:
                hv = np.asarray(self.leaf_value_fn(beliefs, self.model_indices), F32)
            if (not self.cfr_avg) or t <= 1 or self.last_model_values is None:
                self.latest_values[self.model_indices] = hv
            else:
                old, new = self.mixing_weights(t)
                unmixed = (F32(old + new) * hv - F32(old) * self.last_model_values) / F32(new)
                unmixed = self.maybe_enforce_zero_sum(unmixed.astype(F32), mb)
                self.latest_values[self.model_indices] = unmixed
            self.last_model_values = hv.copy()
        if self.showdown_indices.size:
            sd = showdown_value_both(beliefs[self.showdown_indices], self.hand_rank_data,
                                     self.showdown_potential, self.showdown_scale)
            self.latest_values[self.showdown_indices] = sd

    # ---- value backup (cfr_evaluator.py:1049-1115) ------------------------------
    def compute_expected_values(self, policy=None, beliefs=None, leaf_values=None, values=None) -> None:
        policy = self.policy_probs if policy is None else policy
        beliefs = self.beliefs if beliefs is None else beliefs
        leaf_values = self.latest_values if leaf_values is None else leaf_values
        values = leaf_values if values is None else values
        if leaf_values is values:
            values[~self.leaf_mask] = 0.0
        else:
            values[:] = np.where(self.leaf_mask[:, None, None], leaf_values, F32(0.0))
        bottom, top = self.depth_offsets[1], self.depth_offsets[-2]
        actor_beliefs = beliefs[np.arange(top), self.to_act[:top]]
        beliefs_dest = self.fan_out(actor_beliefs)
        marginal = beliefs_dest * policy[bottom:]
        policy_blocked = calculate_unblocked_mass(marginal)
        matchup = calculate_unblocked_mass(beliefs_dest)
        occ = np.zeros_like(policy)
        safe = np.where(matchup > F32(1e-5), matchup, F32(1.0))
        occ[bottom:] = np.where(matchup > F32(1e-5), policy_blocked / safe, F32(0.0))
        self.opponent_conditioned_policy = occ
        for d in range(self.tree_depth - 1, -1, -1):
            on, onn = self.depth_offsets[d + 1], self.depth_offsets[d + 2]
            rows = np.arange(onn - on)
            pa = self.prev_actor[on:onn]
            w = values[on:onn].copy()
            w[rows, pa] *= policy[on:onn]
            w[rows, 1 - pa] *= occ[on:onn]
            self.pull_back_sum(w, values, level=d)

    # ---- regrets (cfr_evaluator.py:1117-1165) -----------------------------------
    def compute_instantaneous_regrets(self, values_achieved, values_expected=None) -> np.ndarray:
        if values_expected is None:
            values_expected = values_achieved
        bottom, top = self.depth_offsets[1], self.depth_offsets[-2]
        beliefs = self.beliefs_avg if self.cfr_avg else self.beliefs
        regrets = np.zeros_like(self.policy_probs)
        rows = np.arange(top)
        src_weights = calculate_unblocked_mass(beliefs[rows, 1 - self.to_act[:top]])
        weights = self.fan_out(src_weights)
        actor_values = values_expected[rows, self.to_act[:top]]
        expected = self.fan_out(actor_values)
        achieved = values_achieved[np.arange(bottom, self.total_nodes), self.prev_actor[bottom:]]
        regrets[bottom:] = weights * (achieved - expected)
        return regrets

    # ---- policy update (cfr_evaluator.py:1167-1258) -----------------------------
    def update_policy(self, t: int) -> None:
        bottom = self.depth_offsets[1]
        pos = np.maximum(self.cumulative_regrets, F32(0.0))
        rsum = np.zeros((self.depth_offsets[-2], NUM_HANDS), F32)
        self.pull_back_sum(pos, rsum)
        denom = self.fan_out(rsum)
        self.policy_probs[bottom:] = np.where(
            denom > F32(1e-8), pos[bottom:] / np.maximum(denom, F32(1e-8)), self.uniform_policy[bottom:])
        self.calculate_reach_weights(self.self_reach, self.policy_probs)
        self.propagate_all_beliefs(self.beliefs, self.self_reach)
        self.update_average_policy(t)
        self.calculate_reach_weights(self.self_reach_avg, self.policy_probs_avg)
        self.propagate_all_beliefs(self.beliefs_avg, self.self_reach_avg)

    def update_average_policy(self, t: int) -> None:
        if self.cfr_type in ("discounted", "discounted_plus") and t <= self.dcfr_delay:
            self.policy_probs_avg[:] = self.policy_probs
            return
        if t == 0:
            self.policy_probs_avg[:] = self.policy_probs
            return
        N, top = self.root_nodes, self.depth_offsets[-2]
        old, new = self.mixing_weights(t)
        rows = np.arange(top)
        reach_actor = self.self_reach[rows, self.to_act[:top]] * F32(new)
        reach_avg_actor = self.self_reach_avg[rows, self.to_act[:top]] * F32(old)
        ra = self.fan_out(reach_actor)
        raa = self.fan_out(reach_avg_actor)
        num = raa * self.policy_probs_avg[N:] + ra * self.policy_probs[N:]
        den = raa + ra
        unweighted = (F32(old) * self.policy_probs_avg[N:] + F32(new) * self.policy_probs[N:]) / F32(old + new)
        safe = np.where(den > F32(1e-5), den, F32(1.0))
        self.policy_probs_avg[N:] = np.where(den > F32(1e-5), num / safe, unweighted)
        psum = np.zeros((top, NUM_HANDS), F32)
        self.pull_back_sum(self.policy_probs_avg, psum)
        pden = self.fan_out(psum)
        safe = np.where(pden > F32(1e-5), pden, F32(1.0))
        self.policy_probs_avg[N:] = np.where(pden > F32(1e-5), self.policy_probs_avg[N:] / safe,
                                             self.policy_probs_avg[N:])
        self.policy_probs_avg[:N] = 0.0

    def update_average_values(self, t: int) -> None:
        old, new = self.mixing_weights(t)
        if self.fused_variant:
            inv = F32(1.0 / (float(old) + float(new)))
            self.values_avg[:] = (self.values_avg * F32(old) + self.latest_values * F32(new)) * inv
        else:
            self.values_avg *= F32(old)
            self.values_avg += F32(new) * self.latest_values
            self.values_avg /= F32(old + new)
        self.values_avg[:] = self.maybe_enforce_zero_sum(self.values_avg, self.beliefs_avg, ignore_mask=self.done)

    # ---- one iteration (cfr_evaluator.py:1330-1381) -----------------------------
    def cfr_iteration(self, t: int) -> None:
        self.apply_schedules(t)
        hit = (self.t_sample == t)[:, None]
        self.policy_probs_sample[:] = np.where(hit, self.policy_probs, self.policy_probs_sample)
        regrets = self.compute_instantaneous_regrets(self.latest_values)
        if self.cfr_type == "linear":
            regrets[self.prev_actor == t % 2] = 0.0
        elif self.cfr_type in ("discounted", "discounted_plus"):
            pos = self.cumulative_regrets > 0
            a, b = t ** self.dcfr_alpha, t ** self.dcfr_beta
            num = np.where(pos, F32(a), F32(b))
            den = np.where(pos, F32(a + 1), F32(b + 1))
            self.cumulative_regrets *= num
            self.cumulative_regrets /= den
            self.regret_weight_sums *= num
            self.regret_weight_sums /= den
        self.regret_weight_sums += F32(1.0)
        self.cumulative_regrets += regrets
        # the fused evaluator accumulates linear-CFR regrets without the CFR+ clamp
        # (fused_sparse_cfr_evaluator.py:503-507); the base class clamps for every type (:1366-1368)
        if self.cfr_plus and not (self.fused_variant and self.cfr_type == "linear"):
            np.maximum(self.cumulative_regrets, F32(0.0), out=self.cumulative_regrets)
        self.update_policy(t)
        self.set_leaf_values(t)
        self.compute_expected_values()
        if not self.use_final_policy_values:
            self.update_average_values(t)

    # ---- warm start (cfr_evaluator.py:888-955) -----------------------------------
    def warm_start(self) -> None:
        from .best_response import best_response_values
        self.set_leaf_values(0)
        self.compute_expected_values(policy=self.policy_probs, beliefs=self.beliefs,
                                     leaf_values=self.latest_values, values=self.latest_values)
        t_ws = self.warm_start_iterations
        scale = F32(float(t_ws) * float(self.warm_start_multiplier))
        self.apply_schedules(t_ws)
        bottom = self.depth_offsets[1]
        if self.warm_start_type == "model":
            regrets = self.compute_instantaneous_regrets(self.latest_values)
            weights = scale * np.maximum(regrets[bottom:], F32(0.0)).mean(axis=-1, dtype=F32)
            self.cumulative_regrets[bottom:] = self.policy_probs[bottom:] * weights[:, None]
            self.regret_weight_sums[bottom:] = weights[:, None]
            self.update_policy(t_ws)
            return
        br0 = best_response_values(self, self.policy_probs, self.beliefs, self.latest_values,
                                   np.zeros_like(self.to_act))
        br1 = best_response_values(self, self.policy_probs, self.beliefs, self.latest_values,
                                   np.ones_like(self.to_act))
        values_br = np.where((self.prev_actor == 0)[:, None, None], br0, br1)
        regrets = self.compute_instantaneous_regrets(values_br, self.latest_values)
        self.cumulative_regrets += scale * regrets
        self.regret_weight_sums += scale
        self.update_policy(t_ws)

    def prepare(self) -> None:
        """The part of evaluate_cfr that precedes the loop (:1505-1515)."""
        self.initialize_policy_and_beliefs()
        if self.warm_start_iterations > 0:
            self.warm_start()
        self.set_leaf_values(0)
        self.compute_expected_values()
        self.values_avg[:] = self.latest_values

    def evaluate_cfr(self) -> None:
        self.prepare()
        for t in range(self.warm_start_iterations, self.cfr_iterations):
            self.cfr_iteration(t)
        if self.use_final_policy_values:
            self.update_average_values_final()

    def update_average_values_final(self) -> None:
        """cfr_evaluator.py:1276-1292: values of the final average strategy, leaves re-evaluated
        on the average ranges."""
        self.set_leaf_values(0, beliefs=self.beliefs_avg)
        self.compute_expected_values(self.policy_probs_avg, self.beliefs_avg,
                                     self.latest_values, self.values_avg)
        self.values_avg[:] = self.maybe_enforce_zero_sum(self.values_avg, self.beliefs_avg,
                                                         ignore_mask=self.done)

    STATE_NAMES = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets",
                   "regret_weight_sums", "self_reach", "self_reach_avg", "beliefs", "beliefs_avg",
                   "latest_values", "values_avg")
