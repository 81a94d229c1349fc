"""Per-operation restatements (numpy float32) of the fused CFR kernels of
``src/p2/search/fused_cfr_triton.py``.  TEST INFRASTRUCTURE ONLY.

Each function states what one reference kernel computes, element by element,
in the arithmetic order of that kernel:

  dcfr_update                <- _fused_dcfr_update_kernel             :71-120
  block_and_normalize        <- _fused_block_normalize_kernel         :245-283
  regret_matching_divide     <- _fused_regret_matching_divide_kernel  :345-366
  weight_child_values        <- _fused_weight_child_values_kernel     :409-435
  update_average_values      <- _fused_update_average_values_kernel   :487-506
  avg_values_zero_sum        <- _fused_avg_values_zs_kernel           :571-620
  regret_tail                <- _fused_regret_tail_kernel             :678-709
  average_policy_mix         <- _fused_average_policy_mix_kernel      :776-820
  parent_sum / sibling_sum   <- _parent_sum_kernel / _sibling_sum_kernel :1167-1238
  divide_by_parent_sum       <- _fused_divide_by_parent_sum_kernel    :1240-1276
  model_values_mix(_zs)      <- :1612-1630, :1691-1736
  weighted_parent_sum        <- _fused_weighted_parent_sum_kernel     :1787-1835
  reach_weights_depth        <- _fused_reach_weights_kernel           :1900-1941
  deep_beliefs               <- _fused_deep_beliefs_kernel            :1996-2036

Pinned by tests/golden/fused_ops_golden.npz: outputs of the reference's own Triton kernels,
run on seeded inputs under Triton's CPU interpreter by tests/golden/gen_fused_ops_golden.py
(every function above, through the reference's public wrappers; tests/test_oracle_fused_ops.py
holds these restatements to them at 1e-5 relative).  Also by: the same identities the reference's own tests assert in
``tests/test_fused_cfr_triton.py`` (each of those tests spells the op out with
plain torch ops; the spellings agree with these), and by ``oracle/cfr.py``,
whose whole-iteration results are built from the un-fused forms of the same
steps and are compared against compositions of these functions.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32


def dcfr_update(cumul, weight, regrets, t, alpha, beta, apply_dcfr=True, cfr_plus=False):
    c = np.array(cumul, dtype=F32)
    w = np.array(weight, dtype=F32)
    if apply_dcfr:
        a, b = F32(float(t ** alpha)), F32(float(t ** beta))
        ad, bd = F32(float(t ** alpha) + 1.0), F32(float(t ** beta) + 1.0)
        pos = c > 0
        num = np.where(pos, a, b)
        den = np.where(pos, ad, bd)
        c = (c * num) / den
        w = (w * num) / den
    w = w + F32(1.0)
    c = c + np.asarray(regrets, dtype=F32)
    if cfr_plus:
        c = np.maximum(c, F32(0.0))
    return c, w, np.maximum(c, F32(0.0))


def block_and_normalize(target, allowed, allowed_prob, eps=1e-5):
    t = np.array(target, dtype=F32)
    if t.ndim == 3:
        mask = allowed[:, None, :]
        fb = np.broadcast_to(allowed_prob[:, None, :], t.shape)
    else:
        mask = allowed
        fb = allowed_prob
    t = np.where(mask, t, F32(0.0))
    s = t.sum(axis=-1, keepdims=True, dtype=F32)
    safe = np.where(s > F32(eps), s, F32(1.0))
    return np.where(s > F32(eps), t / safe, fb).astype(F32)


def regret_matching_divide(pos, den, fallback, eps=1e-8):
    return np.where(den > F32(eps), pos / np.maximum(den, F32(eps)), fallback).astype(F32)


def weight_child_values(values, prev_actor, pol_hero, pol_opp):
    out = np.array(values, dtype=F32)
    for p in (0, 1):
        hero = (prev_actor == p)[:, None]
        out[:, p] = values[:, p] * np.where(hero, pol_hero, pol_opp)
    return out


def update_average_values(avg, latest, old, new):
    inv = F32(1.0 / (float(old) + float(new)))
    return ((avg * F32(old) + latest * F32(new)) * inv).astype(F32)


def avg_values_zero_sum(avg, latest, beliefs, old, new, enforce, ignore=None):
    v = update_average_values(avg, latest, old, new)
    if enforce:
        s = F32(0.5) * ((v * beliefs).sum(axis=2, dtype=F32).sum(axis=1, dtype=F32))
        if ignore is not None:
            s = np.where(ignore, F32(0.0), s)
        v = v - s[:, None, None]
    return v.astype(F32)


def regret_tail(achieved, actor_values, src_w, parent_index, prev_actor, bottom):
    total = achieved.shape[0]
    out = np.zeros((total, achieved.shape[2]), dtype=F32)
    c = np.arange(bottom, total)
    par = parent_index[c]
    out[c] = src_w[par] * (achieved[c, prev_actor[c]] - actor_values[par])
    return out


def average_policy_mix(policy_avg, policy, reach, reach_avg, to_act, parent_index, old, new, bottom, eps=1e-5):
    out = np.array(policy_avg, dtype=F32)
    total = policy.shape[0]
    c = np.arange(bottom, total)
    par = parent_index[c]
    actor = to_act[par]
    ra = reach_avg[par, actor] * F32(old)
    rn = reach[par, actor] * F32(new)
    num = ra * policy_avg[c] + rn * policy[c]
    den = ra + rn
    unw = (F32(old) * policy_avg[c] + F32(new) * policy[c]) / F32(float(old) + float(new))
    safe = np.where(den > F32(eps), den, F32(1.0))
    out[c] = np.where(den > F32(eps), num / safe, unw)
    return out


def parent_sum(values, child_offsets, child_count):
    out = np.zeros((child_offsets.shape[0], values.shape[1]), dtype=F32)
    for p in range(child_offsets.shape[0]):
        for k in range(int(child_count[p])):
            out[p] += values[child_offsets[p] + k]
    return out


def sibling_sum(values, child_offsets, child_count, bottom, num_children):
    ps = parent_sum(values, child_offsets, child_count)
    out = np.zeros((num_children, values.shape[1]), dtype=F32)
    for p in range(child_offsets.shape[0]):
        for k in range(int(child_count[p])):
            out[child_offsets[p] + k - bottom] = ps[p]
    return out


def divide_by_parent_sum(pos, fallback, psum, parent_index, eps=1e-8):
    d = psum[parent_index]
    return np.where(d > F32(eps), pos / np.maximum(d, F32(eps)), fallback).astype(F32)


def model_values_mix(h, last, old, new):
    onon, oon = F32((old + new) / new), F32(old / new)
    return (onon * h - oon * last).astype(F32)


def model_values_mix_zero_sum(h, last, beliefs, old, new, enforce):
    onon, oon = F32((old + new) / new), F32(old / new)
    u = (h * onon - last * oon).astype(F32)
    if enforce:
        s = F32(0.5) * (u * beliefs).sum(axis=2, dtype=F32).sum(axis=1, dtype=F32)
        u = u - s[:, None, None]
    return u.astype(F32)


def weighted_parent_sum(values, prev_actor, pol_hero, pol_opp, child_offsets, child_count, parent_base):
    out = np.array(values, dtype=F32)
    for p in range(child_offsets.shape[0]):
        cnt = int(child_count[p])
        if cnt == 0:
            continue
        for pl in (0, 1):
            acc = np.zeros(values.shape[2], dtype=F32)
            for k in range(cnt):
                c = child_offsets[p] + k
                pol = pol_hero[c] if prev_actor[c] == pl else pol_opp[c]
                acc = acc + values[c, pl] * pol
            out[parent_base + p, pl] = acc
    return out


def reach_weights_depth(reach, policy, allowed, parent_index, prev_actor, start, end):
    out = np.array(reach, dtype=F32)
    for c in range(start, end):
        par = parent_index[c]
        v = out[par].copy()
        v[prev_actor[c]] = v[prev_actor[c]] * policy[c]
        out[c] = np.where(allowed[c][None, :], v, F32(0.0))
    return out


def deep_beliefs(out_in, root_beliefs, reach, allowed_prob, root_index, n_roots, eps=1e-5):
    out = np.array(out_in, dtype=F32)
    total = out.shape[0]
    rows = np.arange(n_roots, total)
    v = root_beliefs[root_index[rows]] * reach[rows]
    s = v.sum(axis=-1, keepdims=True, dtype=F32)
    safe = np.where(s > F32(eps), s, F32(1.0))
    out[rows] = np.where(s > F32(eps), v / safe, allowed_prob[rows][:, None, :])
    return out
