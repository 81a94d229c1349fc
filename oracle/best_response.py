"""Local best response and exploitability of a CFR evaluator state.  TEST INFRASTRUCTURE ONLY.

Follows ``src/p2/search/cfr_evaluator.py``:
  best_response_values   <- _best_response_values   :603-716
  compute_exploitability <- _compute_exploitability :718-764
on the sparse tree (per-parent action slices built like ``_pull_back``,
``sparse_cfr_evaluator.py:465-489``).  Bottom-up per level, with ``actor`` the player to act at
a parent and ``dev`` the deviating player there:
  actor == dev : actor's value per hand = max over legal children (first maximum wins);
                 the actor's belief mass is split by chosen child, projected onto the
                 opponent's hands by unblocked mass and divided by the unblocked mass of the
                 whole belief (0 where that is <= 1e-5); the opponent's value is the
                 expectation of its child values under those probabilities;
  actor != dev : the ordinary backup (own policy for the actor, opponent-conditioned policy for
                 the other player).
Leaf rows keep ``base_values``.

Pinned by the reference's own numbers (local exploitability and best-response values of six
searches in tests/golden/cfr_golden.npz, and the ``model_br`` warm start, which is built on
these values) and by (tests/test_oracle_best_response.py) an exact best response on the explicit
hand-pair game (every compatible pair enumerated) — per-hand root values of the deviating
player agree for random full-support strategies at depths 2-4 — and by
best response >= on-policy value, with equality when the strategy already is a best response.
"""
from __future__ import annotations

import numpy as np

from .cards import NUM_HANDS
from .unblocked import calculate_unblocked_mass

F32 = np.float32


def pull_back(o, x: np.ndarray, level: int | None = None) -> np.ndarray:
    """Child-aligned [total, ...] -> [parents, num_actions, ...] (zeros where no child)."""
    ps, pe, cs, ce = o._level(level)
    out = np.zeros((pe - ps, o.num_actions) + x.shape[1:], dtype=x.dtype)
    out[o.parent_index[cs:ce] - ps, o.action_from_parent[cs:ce]] = x[cs:ce]
    return out


def best_response_values(o, policy, beliefs, base_values, deviating_player=None) -> np.ndarray:
    n, top = o.root_nodes, o.depth_offsets[-2]
    if deviating_player is None:
        deviating_player = o.fan_out_deep(o.to_act[:n])
    values_br = np.where(o.leaf_mask[:, None, None], base_values, F32(0.0)).astype(F32)
    min_value = np.finfo(np.float32).min
    child_mask = o.legal_mask & ~o.leaf_mask[:, None]
    policy_src_all = pull_back(o, policy)                                   # [top, B, H]
    actor_beliefs = beliefs[np.arange(o.total_nodes), o.to_act][:top]      # [top, H]
    marginal = policy_src_all * actor_beliefs[:, None, :]
    policy_blocked = calculate_unblocked_mass(marginal)
    matchup = calculate_unblocked_mass(actor_beliefs)
    safe = np.where(matchup > F32(1e-5), matchup, F32(1.0))[:, None, :]
    occ = np.where(matchup[:, None, :] > F32(1e-5), policy_blocked / safe, F32(0.0)).astype(F32)
    for depth in range(o.tree_depth - 1, -1, -1):
        s, e = o.depth_offsets[depth], o.depth_offsets[depth + 1]
        k = e - s
        rows = np.arange(k)
        actor = o.to_act[s:e]
        deviator = deviating_player[s:e]
        invalid = ~child_mask[s:e]
        values_src = pull_back(o, values_br, level=depth)                   # [k, B, 2, H]
        actor_v = values_src[rows, :, actor]                                # [k, B, H]
        opp_v = values_src[rows, :, 1 - actor]
        for_best = np.where(invalid[:, :, None], min_value, actor_v)
        best = for_best.argmax(axis=1)                                      # [k, H]
        best_v = np.take_along_axis(actor_v, best[:, None, :], axis=1)[:, 0]
        dev_beliefs = actor_beliefs[s:e]
        mass = np.zeros((k, o.num_actions, NUM_HANDS), F32)
        np.put_along_axis(mass, best[:, None, :], dev_beliefs[:, None, :], axis=1)
        mass_blocked = calculate_unblocked_mass(mass)
        dm = matchup[s:e][:, None, :]
        p_dev = np.where(dm > F32(1e-5), mass_blocked / np.where(dm > F32(1e-5), dm, F32(1.0)), F32(0.0))
        v_opp_exp = (p_dev * opp_v).sum(axis=1, dtype=F32)
        is_dev = (deviator == actor)[:, None]
        a_vals = np.where(is_dev, best_v, (actor_v * policy_src_all[s:e]).sum(axis=1, dtype=F32))
        o_vals = np.where(is_dev, v_opp_exp, (opp_v * occ[s:e]).sum(axis=1, dtype=F32))
        values_br[s + rows, actor] = a_vals
        values_br[s + rows, 1 - actor] = o_vals
        values_br[s:e] = np.where(o.leaf_mask[s:e, None, None], base_values[s:e], values_br[s:e])
    return values_br


def compute_exploitability(o):
    """(local_exploitability [N], local_best_response_values [N,2]) of the average strategy."""
    n = o.root_nodes
    policy, beliefs = o.policy_probs_avg, o.beliefs_avg
    leaf_values = np.clip(o.values_avg, F32(-1.0), F32(1.0))
    base = np.zeros_like(leaf_values)
    o.compute_expected_values(policy=policy, beliefs=beliefs, leaf_values=leaf_values, values=base)
    improvements, br_agg = [], []
    for player in range(2):
        dev = o.fan_out_deep(np.full(n, player, dtype=o.to_act.dtype))
        br = best_response_values(o, policy, beliefs, leaf_values, dev)
        rb = beliefs[:n, player]
        improvements.append(((br[:n, player] - base[:n, player]) * rb).sum(axis=-1, dtype=F32))
        br_agg.append((br[:n, player] * rb).sum(axis=-1, dtype=F32))
    return improvements[0] + improvements[1], np.stack(br_agg, axis=-1)
