"""HIP kernels for a single CFR iteration with the reference's function names.

Drop-in for the free functions of ``src/p2/search/fused_cfr_triton.py`` (names,
argument order, keyword names, in-place semantics and exceptions are kept;
``block_*`` tuning keywords are accepted and ignored).  Functions ending in ``_``
mutate their first argument(s) and return ``None``.  Everything launches on the
current stream, never synchronises, and the ``_with_tensors_`` variants read
iteration-dependent scalars through 0-D device tensors so a captured graph can
be replayed for any ``t``.

``CFRType`` mirrors the enum of ``src/p2/core/structured_config.py:46-50``.
"""
from __future__ import annotations

from enum import Enum

import torch

from . import _lib
from ._lib import hip_is_available

_H = 1326


class CFRType(Enum):
    standard = "standard"
    linear = "linear"
    discounted = "discounted"
    discounted_plus = "discounted_plus"


def triton_is_available() -> bool:
    """Kept under the reference's name (fused_cfr_triton.py:65)."""
    return hip_is_available()


def _need() -> None:
    if not hip_is_available():
        raise RuntimeError("libp2hip.so or a GPU is not available; there is no other backend.")


def _scalars(values, like: torch.Tensor):
    """Python floats -> 0-dim float32 device tensors, written by ONE tiny kernel whose arguments
    carry the values (stream ordered; no host-to-device copies)."""
    import ctypes
    n = len(values)
    buf = torch.empty(n, dtype=torch.float32, device=like.device)
    host = (ctypes.c_float * n)(*[float(v) for v in values])
    _lib.call("p2hip_upload_floats", _lib.ptr(buf), ctypes.cast(host, ctypes.c_void_p), n, _lib.stream_ptr())
    return [buf[k] for k in range(n)]


def _scalar(value: float, like: torch.Tensor) -> torch.Tensor:
    return _scalars([value], like)[0]


_S = _lib.stream_ptr
_p = _lib.ptr


# --------------------------------------------------------------------------- K1
def fused_dcfr_update_(cumulative_regrets, regret_weight_sums, regrets, t: int, cfr_type, dcfr_alpha: float,
                       dcfr_beta: float, cfr_plus: bool, positive_regrets_out=None, block_size: int = 1024) -> None:
    """DCFR rescale + weight bump + accumulate + optional clamp (fused_cfr_triton.py:123-197)."""
    _need()
    if cumulative_regrets.device.type != "cuda":
        raise ValueError("fused_dcfr_update_ requires GPU tensors.")
    if getattr(cfr_type, "name", cfr_type) == "linear":
        raise NotImplementedError("Linear CFR path not supported; default config uses discounted_plus.")
    assert cumulative_regrets.is_contiguous()
    assert regret_weight_sums.is_contiguous()
    assert regrets.is_contiguous()
    assert cumulative_regrets.shape == regret_weight_sums.shape == regrets.shape
    apply_dcfr = getattr(cfr_type, "name", cfr_type) in ("discounted", "discounted_plus")
    if apply_dcfr:
        a = float(t ** dcfr_alpha)
        b = float(t ** dcfr_beta)
        vals = (a, b, a + 1.0, b + 1.0)
    else:
        vals = (1.0, 1.0, 1.0, 1.0)
    an, bn, ad, bd = _scalars(vals, cumulative_regrets)
    fused_dcfr_update_with_tensors_(cumulative_regrets, regret_weight_sums, regrets, an, bn, ad, bd, apply_dcfr,
                                    cfr_plus, positive_regrets_out=positive_regrets_out, block_size=block_size)


def fused_dcfr_update_with_tensors_(cumulative_regrets, regret_weight_sums, regrets, t_alpha_num, t_beta_num,
                                    t_alpha_den, t_beta_den, apply_dcfr: bool, cfr_plus: bool,
                                    positive_regrets_out=None, block_size: int = 1024) -> None:
    """fused_cfr_triton.py:200-235."""
    _need()
    _lib.call("p2hip_dcfr_update", _p(cumulative_regrets), _p(regret_weight_sums), _p(regrets), _p(t_alpha_num),
              _p(t_beta_num), _p(t_alpha_den), _p(t_beta_den), cumulative_regrets.numel(), int(bool(apply_dcfr)),
              int(bool(cfr_plus)), _p(positive_regrets_out), _S())


# --------------------------------------------------------------------------- K2
def fused_block_and_normalize_beliefs_(target, allowed_hands, allowed_hands_prob, eps: float = 1e-5) -> None:
    """Mask by ``allowed_hands``, normalise rows, fall back to ``allowed_hands_prob`` where the
    row sum is <= eps (fused_cfr_triton.py:286-335)."""
    _need()
    assert target.is_contiguous()
    assert allowed_hands.is_contiguous()
    assert allowed_hands_prob.is_contiguous()
    assert target.device.type == "cuda"
    if target.dim() == 3:
        n, p, h = target.shape
        rows, stride = n * p, p
    elif target.dim() == 2:
        n, h = target.shape
        rows, stride = n, 1
    else:
        raise ValueError(f"target must be 2D or 3D, got {target.shape}")
    assert h == _H
    assert allowed_hands.shape == (n, h) and allowed_hands.dtype == torch.bool
    assert allowed_hands_prob.shape == (n, h)
    _lib.call("p2hip_block_and_normalize", _p(target), _p(allowed_hands), _p(allowed_hands_prob), rows, stride,
              float(eps), _S())


# --------------------------------------------------------------------------- K3
def fused_regret_matching_divide_(positive_regrets, denom, uniform_fallback, out, eps: float = 1e-8,
                                  block_size: int = 1024) -> None:
    """out = where(denom > eps, pos / max(denom, eps), uniform) (fused_cfr_triton.py:369-399)."""
    _need()
    assert positive_regrets.is_contiguous()
    assert denom.is_contiguous()
    assert uniform_fallback.is_contiguous()
    assert out.is_contiguous()
    assert positive_regrets.shape == denom.shape == uniform_fallback.shape == out.shape
    _lib.call("p2hip_regret_matching_divide", _p(positive_regrets), _p(denom), _p(uniform_fallback), _p(out),
              positive_regrets.numel(), float(eps), _S())


# --------------------------------------------------------------------------- K4
def fused_weight_child_values(values_src, prev_actor, policy_hero, policy_opp, out, block_h: int = 512) -> None:
    """out[m,p] = values_src[m,p] * (policy_hero[m] if p == prev_actor[m] else policy_opp[m])
    (fused_cfr_triton.py:438-477)."""
    _need()
    assert values_src.is_contiguous() and values_src.dim() == 3
    assert out.is_contiguous() and out.shape == values_src.shape
    assert prev_actor.is_contiguous() and prev_actor.dim() == 1
    assert policy_hero.is_contiguous() and policy_opp.is_contiguous()
    m, p, h = values_src.shape
    assert p == 2, "Only supports 2 players."
    assert prev_actor.shape[0] == m
    assert policy_hero.shape == (m, h) and policy_opp.shape == (m, h)
    _lib.call("p2hip_weight_child_values", _p(values_src), _p(prev_actor), _p(policy_hero), _p(policy_opp), _p(out),
              m, _S())


# --------------------------------------------------------------------------- K5 / K6
def fused_update_average_values_(values_avg, latest_values, old: float, new: float, block_size: int = 1024) -> None:
    """values_avg = (values_avg*old + latest*new) * (1/(old+new)) (fused_cfr_triton.py:509-535)."""
    _need()
    assert values_avg.is_contiguous()
    assert latest_values.is_contiguous()
    assert values_avg.shape == latest_values.shape
    total = float(old) + float(new)
    assert total != 0.0
    o_t, n_t, inv_t = _scalars([old, new, 1.0 / total], values_avg)
    fused_update_average_values_with_tensors_(values_avg, latest_values, o_t, n_t, inv_t, block_size=block_size)


def fused_update_average_values_with_tensors_(values_avg, latest_values, old, new, inv_total,
                                              block_size: int = 1024) -> None:
    """fused_cfr_triton.py:538-560."""
    _need()
    _lib.call("p2hip_update_average_values", _p(values_avg), _p(latest_values), _p(old), _p(new), _p(inv_total),
              values_avg.numel(), _S())


def fused_avg_values_zero_sum_(values_avg, latest_values, beliefs, old, new, inv_total, enforce_zero_sum: bool,
                               ignore_mask=None, block_h: int = 2048) -> None:
    """Mix, then optionally subtract 0.5 * sum_p sum_h v_p*b_p per node (0 where ``ignore_mask``)
    (fused_cfr_triton.py:623-668)."""
    _need()
    assert values_avg.is_contiguous() and latest_values.is_contiguous()
    assert beliefs.is_contiguous()
    assert values_avg.shape == latest_values.shape == beliefs.shape
    assert values_avg.dim() == 3 and values_avg.shape[1] == 2
    n_rows, _, h = values_avg.shape
    assert h == _H
    if ignore_mask is not None:
        assert ignore_mask.is_contiguous() and ignore_mask.shape == (n_rows,) and ignore_mask.dtype == torch.bool
    _lib.call("p2hip_avg_values_zero_sum", _p(values_avg), _p(latest_values), _p(beliefs), _p(ignore_mask), _p(old),
              _p(new), _p(inv_total), n_rows, int(bool(enforce_zero_sum)), _S())


# --------------------------------------------------------------------------- K7
def fused_regret_tail_(regrets, values_achieved, actor_values, src_weights, parent_index, prev_actor, bottom: int,
                       block_h: int = 512) -> None:
    """regrets[c] = src_weights[parent(c)] * (values_achieved[c, prev_actor[c]] - actor_values[parent(c)])
    for c >= bottom (fused_cfr_triton.py:712-766)."""
    _need()
    assert regrets.is_contiguous() and regrets.dim() == 2
    assert values_achieved.is_contiguous() and values_achieved.dim() == 3
    assert values_achieved.shape[1] == 2
    assert actor_values.is_contiguous() and actor_values.dim() == 2
    assert src_weights.is_contiguous() and src_weights.dim() == 2
    assert actor_values.shape == src_weights.shape
    assert parent_index.is_contiguous() and parent_index.dim() == 1
    assert prev_actor.is_contiguous() and prev_actor.dim() == 1
    total, h = regrets.shape
    assert values_achieved.shape == (total, 2, h)
    assert parent_index.shape == (total,)
    assert prev_actor.shape == (total,)
    _lib.call("p2hip_regret_tail", _p(regrets), _p(values_achieved), _p(actor_values), _p(src_weights),
              _p(parent_index), _p(prev_actor), int(bottom), total, _S())


# --------------------------------------------------------------------------- K8
def fused_average_policy_mix_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act, parent_index,
                              old: float, new: float, bottom: int, eps: float = 1e-5, block_h: int = 512) -> None:
    """Reach-weighted average-policy mix before renormalisation (fused_cfr_triton.py:823-876)."""
    _need()
    assert policy_probs_avg.is_contiguous() and policy_probs_avg.dim() == 2
    assert policy_probs.is_contiguous() and policy_probs.dim() == 2
    assert self_reach.is_contiguous() and self_reach.dim() == 3
    assert self_reach_avg.is_contiguous() and self_reach_avg.dim() == 3
    assert self_reach.shape[1] == 2 and self_reach_avg.shape[1] == 2
    total, h = policy_probs_avg.shape
    assert policy_probs.shape == (total, h)
    assert self_reach.shape == (total, 2, h)
    assert self_reach_avg.shape == (total, 2, h)
    assert to_act.shape == (total,)
    assert parent_index.shape == (total,)
    total_weight = float(old) + float(new)
    assert total_weight != 0.0
    o_t, n_t, tot_t = _scalars([old, new, total_weight], policy_probs_avg)
    fused_average_policy_mix_with_tensors_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act,
                                           parent_index, o_t, n_t, tot_t, bottom=bottom, eps=eps, block_h=block_h)


def fused_average_policy_mix_with_tensors_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act,
                                           parent_index, old, new, total_weight, bottom: int, eps: float = 1e-5,
                                           block_h: int = 512) -> None:
    """fused_cfr_triton.py:879-914."""
    _need()
    total, _ = policy_probs_avg.shape
    _lib.call("p2hip_average_policy_mix", _p(policy_probs_avg), _p(policy_probs), _p(self_reach), _p(self_reach_avg),
              _p(to_act), _p(parent_index), _p(old), _p(new), _p(total_weight), int(bottom), total, float(eps), _S())


# --------------------------------------------------------------------------- K9 / K12
def unblocked_mass_triton(target: torch.Tensor) -> torch.Tensor:
    """[..., 1326] -> unblocked mass of each combo (fused_cfr_triton.py:1110-1157)."""
    _need()
    if target.device.type != "cuda":
        raise ValueError("unblocked_mass requires GPU tensors.")
    orig_shape = target.shape
    assert orig_shape[-1] == _H, f"last dim must be {_H}, got {orig_shape}"
    flat = target.reshape(-1, _H).contiguous()
    out = torch.empty_like(flat)
    _lib.call("p2hip_unblocked_mass", _p(flat), flat.shape[0], _p(out), _S())
    return out.view(orig_shape)


unblocked_mass_hip = unblocked_mass_triton


def unblocked_mass_opp_at_parents_triton(beliefs, to_act, top: int, cached_stats=None) -> torch.Tensor:
    """unblocked(beliefs[i, 1 - to_act[i]]) for parents i < top -> [top, 1326]
    (fused_cfr_triton.py:1067-1107).  ``cached_stats`` is accepted and ignored."""
    _need()
    total, p, h = beliefs.shape
    assert p == 2 and h == _H
    assert beliefs.is_contiguous() and to_act.is_contiguous() and to_act.dtype == torch.int64
    out = torch.empty((top, h), device=beliefs.device, dtype=beliefs.dtype)
    _lib.call("p2hip_unblocked_mass_by_player", _p(beliefs), _p(to_act), int(top), 1, _p(out), _S())
    return out


def unblocked_mass_ratio_indirect_triton(numer_target, denom_target, parent_index, eps: float = 1e-5,
                                         denom_stats=None) -> torch.Tensor:
    """where(unblk(denom[parent]) > eps, unblk(numer) / unblk(denom[parent]), 0)
    (fused_cfr_triton.py:1499-1556).  ``denom_stats`` is accepted and ignored."""
    _need()
    assert numer_target.is_contiguous() and numer_target.dim() == 2
    assert denom_target.is_contiguous() and denom_target.dim() == 2
    assert parent_index.is_contiguous() and parent_index.dim() == 1
    num_children, h = numer_target.shape
    top = denom_target.shape[0]
    assert denom_target.shape == (top, h)
    assert parent_index.shape == (num_children,)
    assert h == _H
    out = torch.empty_like(numer_target)
    _lib.call("p2hip_unblocked_mass_ratio", _p(numer_target), _p(denom_target), _p(parent_index), num_children,
              float(eps), _p(out), _S())
    return out


def unblocked_mass_ratio_triton(numer_target, denom_target, eps: float = 1e-5) -> torch.Tensor:
    """fused_cfr_triton.py:1559-1602."""
    _need()
    assert numer_target.shape == denom_target.shape
    orig = numer_target.shape
    n = numer_target.reshape(-1, _H).contiguous()
    d = denom_target.reshape(-1, _H).contiguous()
    out = torch.empty_like(n)
    _lib.call("p2hip_unblocked_mass_ratio", _p(n), _p(d), None, n.shape[0], float(eps), _p(out), _S())
    return out.view(orig)


# --------------------------------------------------------------------------- K10 / K11
def fused_parent_sum(values, child_offsets, child_count, max_children: int = 8, block_h: int = 512) -> torch.Tensor:
    """Per-parent sum over its contiguous child rows -> [num_parents, H] (fused_cfr_triton.py:1279-1313)."""
    _need()
    assert values.is_contiguous() and values.dim() == 2
    assert child_offsets.is_contiguous() and child_offsets.dim() == 1
    assert child_count.is_contiguous() and child_count.shape == child_offsets.shape
    num_parents = child_offsets.shape[0]
    out = torch.empty(num_parents, values.shape[1], device=values.device, dtype=values.dtype)
    _lib.call("p2hip_parent_sum", _p(values), _p(child_offsets), _p(child_count), num_parents, _p(out), _S())
    return out


def fused_divide_by_parent_sum_(pos, fallback, parent_sum, parent_index, out, eps: float = 1e-8, block_c: int = 32,
                                block_h: int = 128) -> None:
    """out[c] = where(parent_sum[parent(c)] > eps, pos[c] / max(parent_sum, eps), fallback[c])
    (fused_cfr_triton.py:1316-1352); ``out`` may alias ``pos`` or ``fallback``."""
    _need()
    assert pos.is_contiguous() and fallback.is_contiguous() and out.is_contiguous()
    assert parent_sum.is_contiguous() and parent_index.is_contiguous()
    assert pos.dim() == 2 and fallback.shape == pos.shape == out.shape
    assert parent_sum.dim() == 2 and parent_sum.shape[1] == pos.shape[1]
    num_children, _ = pos.shape
    assert parent_index.shape == (num_children,)
    _lib.call("p2hip_divide_by_parent_sum", _p(pos), _p(fallback), _p(parent_sum), _p(parent_index), _p(out),
              num_children, float(eps), _S())


def fused_sibling_sum(values, child_offsets, child_count, bottom: int, num_children: int, max_children: int = 8,
                      block_h: int = 512) -> torch.Tensor:
    """Sum over each child's siblings, child-aligned -> [num_children, H] (fused_cfr_triton.py:1355-1398)."""
    _need()
    assert values.is_contiguous() and values.dim() == 2
    assert child_offsets.is_contiguous() and child_offsets.dim() == 1
    assert child_count.is_contiguous() and child_count.dim() == 1
    assert child_offsets.shape == child_count.shape
    out = torch.empty(num_children, values.shape[1], device=values.device, dtype=values.dtype)
    _lib.call("p2hip_sibling_sum", _p(values), _p(child_offsets), _p(child_count), child_offsets.shape[0],
              int(bottom), _p(out), _S())
    return out


# --------------------------------------------------------------------------- K13
def fused_model_values_mix(hand_values, last_model_values, old: float, new: float,
                           block_size: int = 1024) -> torch.Tensor:
    """((old+new)*hand - old*last)/new with pre-divided scalars (fused_cfr_triton.py:1633-1655)."""
    _need()
    assert hand_values.is_contiguous() and last_model_values.is_contiguous()
    assert hand_values.shape == last_model_values.shape
    assert new != 0.0
    out = torch.empty_like(hand_values)
    onon_t, oon_t = _scalars([(old + new) / new, old / new], hand_values)
    fused_model_values_mix_with_tensors(hand_values, last_model_values, onon_t, oon_t, out, block_size=block_size)
    return out


def fused_model_values_mix_with_tensors(hand_values, last_model_values, old_plus_new_over_new, old_over_new, out,
                                        block_size: int = 1024) -> None:
    """fused_cfr_triton.py:1658-1680."""
    _need()
    _lib.call("p2hip_model_values_mix", _p(hand_values), _p(last_model_values), _p(old_plus_new_over_new),
              _p(old_over_new), _p(out), hand_values.numel(), _S())


def fused_model_values_mix_zero_sum(hand_values, last_model_values, beliefs, old_plus_new_over_new, old_over_new,
                                    out, enforce_zero_sum: bool, block_h: int = 2048) -> None:
    """fused_cfr_triton.py:1739-1775."""
    _need()
    assert hand_values.is_contiguous() and last_model_values.is_contiguous()
    assert beliefs.is_contiguous() and out.is_contiguous()
    assert hand_values.shape == last_model_values.shape == beliefs.shape == out.shape
    assert hand_values.dim() == 3 and hand_values.shape[1] == 2
    m, _, h = hand_values.shape
    assert h == _H
    _lib.call("p2hip_model_values_mix_zero_sum", _p(hand_values), _p(last_model_values), _p(beliefs),
              _p(old_plus_new_over_new), _p(old_over_new), _p(out), m, int(bool(enforce_zero_sum)), _S())


# --------------------------------------------------------------------------- K14 / K15 / K16
def fused_weighted_parent_sum(values, prev_actor, policy_hero, policy_opp, child_offsets, child_count,
                              parent_base: int, max_children: int = 8, block_h: int = 2048) -> None:
    """values[parent_base+p, pl] = sum_children values[c, pl] * (policy_hero[c] if pl == prev_actor[c]
    else policy_opp[c]); parents without children keep their value (fused_cfr_triton.py:1838-1889)."""
    _need()
    assert values.is_contiguous() and values.dim() == 3 and values.shape[1] == 2
    assert policy_hero.is_contiguous() and policy_opp.is_contiguous()
    assert child_offsets.is_contiguous() and child_count.is_contiguous()
    total, _, h = values.shape
    assert policy_hero.shape == (total, h) and policy_opp.shape == (total, h)
    assert prev_actor.shape == (total,)
    _lib.call("p2hip_weighted_parent_sum", _p(values), _p(prev_actor), _p(policy_hero), _p(policy_opp),
              _p(child_offsets), _p(child_count), child_offsets.shape[0], int(parent_base), _S())


def fused_reach_weights_depth_(reach, policy, allowed_mask, parent_index, prev_actor, start: int, end: int,
                               block_h: int = 2048) -> None:
    """reach[c,p] = reach[parent(c),p] * (policy[c] if p == prev_actor[c] else 1), zero where
    ``allowed_mask[c]`` is False, for c in [start, end) (fused_cfr_triton.py:1944-1986)."""
    _need()
    assert reach.is_contiguous() and reach.dim() == 3 and reach.shape[1] == 2
    assert policy.is_contiguous() and policy.dim() == 2
    total, _, h = reach.shape
    assert policy.shape == (total, h)
    assert allowed_mask.shape == (total, h) and allowed_mask.is_contiguous() and allowed_mask.dtype == torch.bool
    assert parent_index.shape == (total,) and prev_actor.shape == (total,)
    if end - start <= 0:
        return
    _lib.call("p2hip_reach_weights_depth", _p(reach), _p(policy), _p(allowed_mask), _p(parent_index),
              _p(prev_actor), int(start), int(end), _S())


def fused_deep_beliefs_(out, root_beliefs, reach_weights, allowed_prob, root_index, num_roots: int | None = None,
                        eps: float = 1e-5, block_h: int = 2048) -> None:
    """out[i,p] = normalise(root_beliefs[root_index[i],p] * reach_weights[i,p]) with fallback
    ``allowed_prob[i]``; root rows are left untouched (fused_cfr_triton.py:2039-2092)."""
    _need()
    assert out.is_contiguous() and out.dim() == 3 and out.shape[1] == 2
    assert root_beliefs.is_contiguous() and root_beliefs.dim() == 3
    assert reach_weights.is_contiguous() and reach_weights.shape == out.shape
    total, _, h = out.shape
    n = num_roots if num_roots is not None else root_beliefs.shape[0]
    assert root_beliefs.shape[0] >= n and tuple(root_beliefs.shape[1:]) == (2, h)
    assert allowed_prob.shape == (total, h) and allowed_prob.is_contiguous()
    assert root_index.shape == (total,) and root_index.is_contiguous()
    if total <= n:
        return
    _lib.call("p2hip_deep_beliefs", _p(out), _p(root_beliefs), _p(reach_weights), _p(allowed_prob), _p(root_index),
              int(n), total, float(eps), _S())


def fused_sample_snapshot_(policy_probs_sample, policy_probs, t_sample, t_tensor) -> None:
    """policy_probs_sample <- where(t_sample == t, policy_probs, policy_probs_sample)
    (fused_sparse_cfr_evaluator.py:494-499); ``t_tensor`` is a 0-D int64 device tensor."""
    _need()
    assert policy_probs_sample.is_contiguous() and policy_probs.is_contiguous()
    assert policy_probs_sample.shape == policy_probs.shape
    assert t_sample.is_contiguous() and t_sample.dtype == torch.int64 and t_tensor.dtype == torch.int64
    _lib.call("p2hip_sample_snapshot", _p(policy_probs), _p(policy_probs_sample), _p(t_sample), _p(t_tensor),
              policy_probs.shape[0], _S())


# --------------------------------------------------------------------------- TScalars
class TScalars:
    """0-D device tensors holding the iteration-dependent scalars (fused_cfr_triton.py:2100-2158).
    ``update`` copies host values in and must run outside any captured region."""

    def __init__(self, device: torch.device, dtype: torch.dtype = torch.float32) -> None:
        def _z():
            return torch.zeros((), dtype=dtype, device=device)

        self.device = device
        self.dtype = dtype
        self.t_alpha_num = _z()
        self.t_beta_num = _z()
        self.t_alpha_den = _z()
        self.t_beta_den = _z()
        self.mix_old = _z()
        self.mix_new = _z()
        self.mix_total = _z()
        self.mix_inv_total = _z()
        self.mix_onon = _z()
        self.mix_oon = _z()
        self.t_tensor = torch.zeros((), dtype=torch.long, device=device)

    def update(self, t: int, dcfr_alpha: float, dcfr_beta: float, mix_old: float, mix_new: float) -> None:
        t_alpha_num = float(t ** dcfr_alpha)
        t_beta_num = float(t ** dcfr_beta)
        self.t_alpha_num.fill_(t_alpha_num)
        self.t_beta_num.fill_(t_beta_num)
        self.t_alpha_den.fill_(t_alpha_num + 1.0)
        self.t_beta_den.fill_(t_beta_num + 1.0)
        total = float(mix_old) + float(mix_new)
        self.mix_old.fill_(float(mix_old))
        self.mix_new.fill_(float(mix_new))
        self.mix_total.fill_(total)
        self.mix_inv_total.fill_(1.0 / total if total != 0.0 else 1.0)
        if float(mix_new) != 0.0:
            self.mix_onon.fill_(total / float(mix_new))
            self.mix_oon.fill_(float(mix_old) / float(mix_new))
        self.t_tensor.fill_(int(t))


class ParentBeliefUnblockedStats:
    """Total and per-card sums of both players' beliefs at the parent rows
    (fused_cfr_triton.py:1029-1064).  The HIP kernels take their card sums inside the kernel, so
    passing this object as ``cached_stats`` changes nothing; it exists for callers that build it."""

    def __init__(self, beliefs_parents: torch.Tensor) -> None:
        assert beliefs_parents.dim() == 3 and beliefs_parents.shape[1] == 2
        self.top = beliefs_parents.shape[0]
        self.beliefs_parents = beliefs_parents

    def slice_for_player(self, player_per_node: torch.Tensor):
        from .card_utils import combo_to_onehot_tensor
        rows = torch.arange(self.top, device=self.beliefs_parents.device)
        target = self.beliefs_parents[rows, player_per_node, :].contiguous()
        onehot = combo_to_onehot_tensor(device=target.device).to(target.dtype)
        return target, target.sum(dim=-1), target @ onehot


def __getattr__(name):
    # GraphedCFRIteration lives with the evaluator (which imports this module); the reference
    # exports it from fused_cfr_triton.py:2359-2451
    if name == "GraphedCFRIteration":
        from .evaluator import GraphedCFRIteration
        return GraphedCFRIteration
    raise AttributeError(name)
