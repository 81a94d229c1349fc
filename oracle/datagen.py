"""Feature encoding and training targets either side of the search.  TEST INFRASTRUCTURE ONLY.

Follows
  encode          RebelFeatureEncoder.encode (src/p2/models/mlp/rebel_feature_encoder.py:55-127)
  bet_amounts     HUNLTensorEnv.legal_bins_amounts_and_mask, amounts (src/p2/env/hunl_tensor_env.py:348-405)
  previous_board  the env's last_board_indices (:862: every action saves the board before the deal)
  policy_targets  _pull_back of the average policy, [node, hand, action] (src/p2/search/cfr_evaluator.py:1392-1393)
  training_data   CFREvaluator.training_data (:1383-1495)
on the oracle's search state (``oracle.cfr.OracleCFR``) and tree arrays (``oracle.tree.build_tree``).

Pinned by tests/golden/training_data_golden.npz (tests/golden/gen_training_data_golden.py runs the
reference's evaluator, encoder and chance helper: roots of every street at the start and in the
middle of a betting round, reset-state roots; the encoder alone on every node with the leaf rule
for the board; all three batches with their statistics) through tests/test_oracle_datagen.py.
"""
from __future__ import annotations

import numpy as np

from . import best_response as BR
from . import chance as CH
from .cards import NUM_HANDS

F32 = np.float32
CARDS_ON_STREET = np.array([0, 3, 4, 5, 5])


def encode(env: dict, beliefs: np.ndarray, pre_chance_node=None, indices=None) -> dict:
    """env: arrays to_act, button, starting_stacks [M,2], pot, committed [M,2], actions_this_round,
    board_indices [M,5], last_board_indices [M,5].  Returns context [B,4], street [B] zeros, to_act,
    board [B,5], beliefs [B, 2*1326]."""
    def get(name):
        v = np.asarray(env[name])
        return v[indices] if indices is not None else v
    if indices is not None:
        beliefs = beliefs[indices]
        if isinstance(pre_chance_node, np.ndarray):
            pre_chance_node = pre_chance_node[indices]
    m = beliefs.shape[0]
    if pre_chance_node is None:
        pre = np.zeros(m, dtype=bool)
    elif isinstance(pre_chance_node, (bool, np.bool_)):
        pre = np.full(m, bool(pre_chance_node))
    else:
        pre = np.asarray(pre_chance_node, dtype=bool)
    to_act = get("to_act")
    context = np.zeros((m, 4), F32)
    context[:, 0] = to_act.astype(F32)
    context[:, 1] = np.mod(to_act - get("button"), 2).astype(F32)
    starting = get("starting_stacks").astype(F32)
    total = np.maximum(starting[:, 0] + starting[:, 1], F32(1.0))
    context[:, 2] = np.clip(get("pot").astype(F32) / total, F32(0.0), F32(10.0))
    committed = get("committed")
    context[:, 3] = ((committed[:, 0] != committed[:, 1]) & (get("actions_this_round") > 0)).astype(F32)
    board = np.where(pre[:, None], get("last_board_indices"), get("board_indices"))
    return {"context": context, "street": np.zeros(m, F32), "to_act": to_act, "board": board,
            "beliefs": beliefs.reshape(m, 2 * NUM_HANDS)}


def bet_amounts(env: dict, bins: list[float]) -> np.ndarray:
    m = env["to_act"].shape[0]
    nb = len(bins) + 3
    rows = np.arange(m)
    me, opp = env["to_act"], 1 - env["to_act"]
    to_call = env["committed"][rows, opp] - env["committed"][rows, me]
    amounts = np.full((m, nb), -1, dtype=np.int64)
    for i, frac in enumerate(bins):
        amounts[:, 2 + i] = to_call + (F32(frac) * env["pot"].astype(F32)).astype(np.int64)
    amounts[:, nb - 1] = env["stacks"][rows, me]
    return amounts


def previous_board(street, actions_this_round, board) -> np.ndarray:
    street = np.clip(np.asarray(street), 0, 4)
    at_start = (np.asarray(actions_this_round) == 0) & (street >= 1)
    keep = np.where(at_start, CARDS_ON_STREET[np.maximum(street - 1, 0)], 5)
    return np.where(np.arange(5)[None, :] < keep[:, None], board, -1)


def tree_env(tree: dict, root_boards: np.ndarray, root_last_boards: np.ndarray | None = None) -> dict:
    """Per-node env arrays for ``encode``: every node shows its root's board; below the roots the
    previous board is that board too."""
    n = tree["depth_offsets"][1]
    total = tree["depth_offsets"][-1]
    root_index = np.arange(total)
    for i in range(n, total):
        root_index[i] = root_index[tree["parent_index"][i]]
    env = {k: tree[k] for k in ("to_act", "button", "starting_stacks", "pot", "committed", "actions_this_round",
                                "stacks", "street")}
    env["board_indices"] = np.asarray(root_boards)[root_index]
    last = env["board_indices"].copy()
    last[:n] = (previous_board(tree["street"][:n], tree["actions_this_round"][:n], root_boards)
                if root_last_boards is None else root_last_boards)
    env["last_board_indices"] = last
    return env


def policy_targets(o) -> np.ndarray:
    """[top, 1326, num_actions]."""
    top = o.depth_offsets[-2]
    return np.transpose(BR.pull_back(o, o.policy_probs_avg)[:top], (0, 2, 1))


def _take(batch: dict, sel) -> dict:
    out = {}
    for k, v in batch.items():
        out[k] = _take(v, sel) if isinstance(v, dict) else v[sel]
    return out


def training_data(o, env: dict, bins: list[float], model_fn, exclude_start: bool = True,
                  flop_tables=None):
    """(value, pre_value, policy) batches as dicts {features, legal_masks, value_targets /
    policy_targets, statistics}.  ``model_fn(context, street, to_act, board, beliefs) -> [S,2,H]``
    is the value network (used by the chance nodes); ``flop_tables`` = (canonical, count,
    combo_perm) of oracle.chance, needed when a flop root stands at the start of its round."""
    n = o.root_nodes
    top = o.depth_offsets[-2] if len(o.depth_offsets) > 1 else n
    value_targets = np.clip(o.values_avg[:n], F32(-1.0), F32(1.0))
    feats = _take(encode(env, o.beliefs_avg, pre_chance_node=False), slice(0, top))
    amounts = bet_amounts(env, bins)
    legal = o.legal_mask
    stats = {"to_act": env["to_act"], "street": env["street"], "stage": 2 * env["street"],
             "board": env["board_indices"], "pot": env["pot"], "bet_amounts": amounts}
    expl, br_values = BR.compute_exploitability(o)
    value_stats = {k: v[:n] for k, v in stats.items()}
    value_stats["local_exploitability"] = expl
    value_stats["local_best_response_values"] = br_values
    valid_top = ~o.leaf_mask[:top]
    value = {"features": _take(feats, slice(0, n)), "value_targets": value_targets, "legal_masks": legal[:n],
             "statistics": value_stats}
    street_root, actions_root = env["street"][:n], env["actions_this_round"][:n]
    if exclude_start:
        value = _take(value, ~((street_root == 0) & (actions_root == 0)))
    policy = {"features": _take(feats, valid_top), "policy_targets": policy_targets(o)[valid_top],
              "legal_masks": legal[:top][valid_top], "statistics": {k: v[:top][valid_top] for k, v in stats.items()}}

    pre_feats = _take(encode(env, o.beliefs, pre_chance_node=True), slice(0, n))
    pre_feats["beliefs"] = o.root_pre_chance_beliefs[:n].reshape(n, -1).copy()
    targets_pre = value_targets.copy()
    pre_stats = {k: v.copy() for k, v in value_stats.items()}
    pre_stats["board"] = env["last_board_indices"][:n].copy()
    prev_street = np.where((street_root > 0) & (street_root < 4) & (actions_root == 0), street_root - 1, street_root)
    pre_stats["street"] = prev_street
    pre_stats["stage"] = 2 * prev_street + 1
    start = actions_root == 0
    root_feats = _take(feats, slice(0, n))
    turn_river = start & ((street_root == 2) | (street_root == 3))
    if turn_river.any():
        targets_pre[turn_river] = CH.single_card_chance_values(
            np.nonzero(turn_river)[0], root_feats["context"], root_feats["street"], root_feats["to_act"],
            o.root_pre_chance_beliefs, env["last_board_indices"][:n], model_fn)
    flop = start & (street_root == 1)
    if flop.any():
        canonical, count, combo_perm = flop_tables
        targets_pre[flop] = CH.flop_chance_values(
            np.nonzero(flop)[0], root_feats["context"], root_feats["street"], root_feats["to_act"],
            o.root_pre_chance_beliefs, model_fn, canonical, count, combo_perm)
    pre_value = _take({"features": pre_feats, "value_targets": targets_pre, "legal_masks": legal[:n],
                       "statistics": pre_stats}, turn_river | flop)
    return value, pre_value, policy
