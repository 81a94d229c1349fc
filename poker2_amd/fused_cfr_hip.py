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

import ctypes
from enum import Enum

import torch

from . import _lib
from ._lib import hip_is_available
from ._guards import require as _req

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


def discount_pair(t: int, exponent: float) -> tuple[float, float]:
    """(t**e, t**e + 1): numerator and denominator of the DCFR discount t**e / (t**e + 1)
    (cfr_evaluator.py:1346-1362).  At t = 0 with a negative exponent — beta = -1 in the reference's
    own settings — t**e does not exist; the factor's limit is 1, returned as (1, 1).  (The reference
    evaluates ``0 ** e`` there and raises; its runs start after a warm start, so t >= 1.)"""
    if t == 0 and exponent < 0:
        return 1.0, 1.0
    num = float(t ** exponent)
    return num, num + 1.0


def _scalar(value: float, like: torch.Tensor) -> torch.Tensor:
    return _scalars([value], like)[0]


_S = _lib.stream_ptr
_p = _lib.ptr


def _f32(**tensors) -> None:
    """Every named tensor is contiguous float32 on the GPU (the kernels read raw fp32 rows)."""
    for name, t in tensors.items():
        _req(t.dtype == torch.float32 and t.is_contiguous() and t.device.type == "cuda",
             f"{name} must be a contiguous float32 GPU tensor, got {t.dtype} on {t.device}")


def _i64(rows: int, **tensors) -> None:
    """Every named tensor is a contiguous int64 GPU vector with at least ``rows`` entries (the
    kernels read index arrays as 8-byte integers)."""
    for name, t in tensors.items():
        _req(t.dtype == torch.int64 and t.is_contiguous() and t.dim() == 1 and t.shape[0] >= rows
             and t.device.type == "cuda", f"{name} must be a contiguous int64 GPU vector of >= {rows} entries, "
             f"got {t.dtype} {tuple(t.shape)} on {t.device}")


def _scalar_ptrs(**tensors) -> None:
    for name, t in tensors.items():
        _req(t.dtype == torch.float32 and t.numel() >= 1 and t.device.type == "cuda",
             f"{name} must be a float32 GPU scalar tensor")


# --------------------------------------------------------------------------- K1
def fused_dcfr_update_(cumulative_regrets, regret_weight_sums, regrets, t: int, cfr_type, dcfr_alpha: float,
                       dcfr_beta: float, cfr_plus: bool, positive_regrets_out=None, block_size: int = 1024) -> None:
    """DCFR rescale + weight bump + accumulate + optional clamp (fused_cfr_triton.py:123-197)."""
    _need()
    if cumulative_regrets.device.type != "cuda":
        raise ValueError("fused_dcfr_update_ requires GPU tensors.")
    if getattr(cfr_type, "name", cfr_type) == "linear":
        raise NotImplementedError("Linear CFR path not supported; default config uses discounted_plus.")
    _req(cumulative_regrets.is_contiguous(), "cumulative_regrets.is_contiguous()")
    _req(regret_weight_sums.is_contiguous(), "regret_weight_sums.is_contiguous()")
    _req(regrets.is_contiguous(), "regrets.is_contiguous()")
    _req(cumulative_regrets.shape == regret_weight_sums.shape == regrets.shape,
         "cumulative_regrets.shape == regret_weight_sums.shape == regrets.shape")
    apply_dcfr = getattr(cfr_type, "name", cfr_type) in ("discounted", "discounted_plus")
    if apply_dcfr:
        (a, a_den), (b, b_den) = discount_pair(t, dcfr_alpha), discount_pair(t, dcfr_beta)
        vals = (a, b, a_den, b_den)
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
    _f32(cumulative_regrets=cumulative_regrets, regret_weight_sums=regret_weight_sums, regrets=regrets)
    _req(cumulative_regrets.shape == regret_weight_sums.shape == regrets.shape, "regret tensors differ in shape")
    _scalar_ptrs(t_alpha_num=t_alpha_num, t_beta_num=t_beta_num, t_alpha_den=t_alpha_den, t_beta_den=t_beta_den)
    if positive_regrets_out is not None:
        _f32(positive_regrets_out=positive_regrets_out)
        _req(positive_regrets_out.shape == cumulative_regrets.shape, "positive_regrets_out differs in shape")
    _lib.call("p2hip_dcfr_update", _p(cumulative_regrets), _p(regret_weight_sums), _p(regrets), _p(t_alpha_num),
              _p(t_beta_num), _p(t_alpha_den), _p(t_beta_den), cumulative_regrets.numel(), int(bool(apply_dcfr)),
              int(bool(cfr_plus)), _p(positive_regrets_out), _S())


# --------------------------------------------------------------------------- K2
def fused_block_and_normalize_beliefs_(target, allowed_hands, allowed_hands_prob, eps: float = 1e-5) -> None:
    """Mask by ``allowed_hands``, normalise rows, fall back to ``allowed_hands_prob`` where the
    row sum is <= eps (fused_cfr_triton.py:286-335)."""
    _need()
    _req(target.is_contiguous(), "target.is_contiguous()")
    _req(allowed_hands.is_contiguous(), "allowed_hands.is_contiguous()")
    _req(allowed_hands_prob.is_contiguous(), "allowed_hands_prob.is_contiguous()")
    _req(target.device.type == "cuda", "target.device.type == \"cuda\"")
    if target.dim() == 3:
        n, p, h = target.shape
        rows, stride = n * p, p
    elif target.dim() == 2:
        n, h = target.shape
        rows, stride = n, 1
    else:
        raise ValueError(f"target must be 2D or 3D, got {target.shape}")
    _req(h == _H, "h == _H")
    _req(allowed_hands.shape == (n, h) and allowed_hands.dtype == torch.bool,
         "allowed_hands.shape == (n, h) and allowed_hands.dtype == torch.bool")
    _req(allowed_hands_prob.shape == (n, h), "allowed_hands_prob.shape == (n, h)")
    _f32(target=target, allowed_hands_prob=allowed_hands_prob)
    _lib.call("p2hip_block_and_normalize", _p(target), _p(allowed_hands), _p(allowed_hands_prob), rows, stride,
              float(eps), _S())


# --------------------------------------------------------------------------- K3
def fused_regret_matching_divide_(positive_regrets, denom, uniform_fallback, out, eps: float = 1e-8,
                                  block_size: int = 1024) -> None:
    """out = where(denom > eps, pos / max(denom, eps), uniform) (fused_cfr_triton.py:369-399)."""
    _need()
    _req(positive_regrets.is_contiguous(), "positive_regrets.is_contiguous()")
    _req(denom.is_contiguous(), "denom.is_contiguous()")
    _req(uniform_fallback.is_contiguous(), "uniform_fallback.is_contiguous()")
    _req(out.is_contiguous(), "out.is_contiguous()")
    _req(positive_regrets.shape == denom.shape == uniform_fallback.shape == out.shape,
         "positive_regrets.shape == denom.shape == uniform_fallback.shape == out.shape")
    _f32(positive_regrets=positive_regrets, denom=denom, uniform_fallback=uniform_fallback, out=out)
    _lib.call("p2hip_regret_matching_divide", _p(positive_regrets), _p(denom), _p(uniform_fallback), _p(out),
              positive_regrets.numel(), float(eps), _S())


# --------------------------------------------------------------------------- K4
def fused_weight_child_values(values_src, prev_actor, policy_hero, policy_opp, out, block_h: int = 512) -> None:
    """out[m,p] = values_src[m,p] * (policy_hero[m] if p == prev_actor[m] else policy_opp[m])
    (fused_cfr_triton.py:438-477)."""
    _need()
    _req(values_src.is_contiguous() and values_src.dim() == 3, "values_src.is_contiguous() and values_src.dim() == 3")
    _req(out.is_contiguous() and out.shape == values_src.shape,
         "out.is_contiguous() and out.shape == values_src.shape")
    _req(prev_actor.is_contiguous() and prev_actor.dim() == 1, "prev_actor.is_contiguous() and prev_actor.dim() == 1")
    _req(policy_hero.is_contiguous() and policy_opp.is_contiguous(),
         "policy_hero.is_contiguous() and policy_opp.is_contiguous()")
    m, p, h = values_src.shape
    _req(p == 2, "Only supports 2 players.")
    _req(prev_actor.shape[0] == m, "prev_actor.shape[0] == m")
    _req(policy_hero.shape == (m, h) and policy_opp.shape == (m, h),
         "policy_hero.shape == (m, h) and policy_opp.shape == (m, h)")
    _f32(values_src=values_src, policy_hero=policy_hero, policy_opp=policy_opp, out=out)
    _i64(m, prev_actor=prev_actor)
    _lib.call("p2hip_weight_child_values", _p(values_src), _p(prev_actor), _p(policy_hero), _p(policy_opp), _p(out),
              m, _S())


# --------------------------------------------------------------------------- K5 / K6
def fused_update_average_values_(values_avg, latest_values, old: float, new: float, block_size: int = 1024) -> None:
    """values_avg = (values_avg*old + latest*new) * (1/(old+new)) (fused_cfr_triton.py:509-535)."""
    _need()
    _req(values_avg.is_contiguous(), "values_avg.is_contiguous()")
    _req(latest_values.is_contiguous(), "latest_values.is_contiguous()")
    _req(values_avg.shape == latest_values.shape, "values_avg.shape == latest_values.shape")
    total = float(old) + float(new)
    _req(total != 0.0, "total != 0.0")
    o_t, n_t, inv_t = _scalars([old, new, 1.0 / total], values_avg)
    fused_update_average_values_with_tensors_(values_avg, latest_values, o_t, n_t, inv_t, block_size=block_size)


def fused_update_average_values_with_tensors_(values_avg, latest_values, old, new, inv_total,
                                              block_size: int = 1024) -> None:
    """fused_cfr_triton.py:538-560."""
    _need()
    _f32(values_avg=values_avg, latest_values=latest_values)
    _req(values_avg.shape == latest_values.shape, "values_avg.shape == latest_values.shape")
    _scalar_ptrs(old=old, new=new, inv_total=inv_total)
    _lib.call("p2hip_update_average_values", _p(values_avg), _p(latest_values), _p(old), _p(new), _p(inv_total),
              values_avg.numel(), _S())


def fused_avg_values_zero_sum_(values_avg, latest_values, beliefs, old, new, inv_total, enforce_zero_sum: bool,
                               ignore_mask=None, block_h: int = 2048) -> None:
    """Mix, then optionally subtract 0.5 * sum_p sum_h v_p*b_p per node (0 where ``ignore_mask``)
    (fused_cfr_triton.py:623-668)."""
    _need()
    _req(values_avg.is_contiguous() and latest_values.is_contiguous(),
         "values_avg.is_contiguous() and latest_values.is_contiguous()")
    _req(beliefs.is_contiguous(), "beliefs.is_contiguous()")
    _req(values_avg.shape == latest_values.shape == beliefs.shape,
         "values_avg.shape == latest_values.shape == beliefs.shape")
    _req(values_avg.dim() == 3 and values_avg.shape[1] == 2, "values_avg.dim() == 3 and values_avg.shape[1] == 2")
    n_rows, _, h = values_avg.shape
    _req(h == _H, "h == _H")
    if ignore_mask is not None:
        _req(ignore_mask.is_contiguous() and ignore_mask.shape == (n_rows,) and ignore_mask.dtype == torch.bool,
             "ignore_mask.is_contiguous() and ignore_mask.shape == (n_rows,) and ignore_mask.dtype == torch.bool")
    _f32(values_avg=values_avg, latest_values=latest_values, beliefs=beliefs)
    _scalar_ptrs(old=old, new=new, inv_total=inv_total)
    _lib.call("p2hip_avg_values_zero_sum", _p(values_avg), _p(latest_values), _p(beliefs), _p(ignore_mask), _p(old),
              _p(new), _p(inv_total), n_rows, int(bool(enforce_zero_sum)), _S())


# --------------------------------------------------------------------------- K7
def fused_regret_tail_(regrets, values_achieved, actor_values, src_weights, parent_index, prev_actor, bottom: int,
                       block_h: int = 512) -> None:
    """regrets[c] = src_weights[parent(c)] * (values_achieved[c, prev_actor[c]] - actor_values[parent(c)])
    for c >= bottom (fused_cfr_triton.py:712-766)."""
    _need()
    _req(regrets.is_contiguous() and regrets.dim() == 2, "regrets.is_contiguous() and regrets.dim() == 2")
    _req(values_achieved.is_contiguous() and values_achieved.dim() == 3,
         "values_achieved.is_contiguous() and values_achieved.dim() == 3")
    _req(values_achieved.shape[1] == 2, "values_achieved.shape[1] == 2")
    _req(actor_values.is_contiguous() and actor_values.dim() == 2,
         "actor_values.is_contiguous() and actor_values.dim() == 2")
    _req(src_weights.is_contiguous() and src_weights.dim() == 2,
         "src_weights.is_contiguous() and src_weights.dim() == 2")
    _req(actor_values.shape == src_weights.shape, "actor_values.shape == src_weights.shape")
    _req(parent_index.is_contiguous() and parent_index.dim() == 1,
         "parent_index.is_contiguous() and parent_index.dim() == 1")
    _req(prev_actor.is_contiguous() and prev_actor.dim() == 1, "prev_actor.is_contiguous() and prev_actor.dim() == 1")
    total, h = regrets.shape
    _req(values_achieved.shape == (total, 2, h), "values_achieved.shape == (total, 2, h)")
    _req(parent_index.shape == (total,), "parent_index.shape == (total,)")
    _req(prev_actor.shape == (total,), "prev_actor.shape == (total,)")
    _f32(regrets=regrets, values_achieved=values_achieved, actor_values=actor_values, src_weights=src_weights)
    _i64(total, parent_index=parent_index, prev_actor=prev_actor)
    _req(0 <= int(bottom) <= total, f"bottom={bottom} outside the {total} rows")
    _req(actor_values.shape[1] == h, "actor_values.shape[1] == h")
    _lib.call("p2hip_regret_tail", _p(regrets), _p(values_achieved), _p(actor_values), _p(src_weights),
              _p(parent_index), _p(prev_actor), int(bottom), total, _S())


# --------------------------------------------------------------------------- K8
def fused_average_policy_mix_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act, parent_index,
                              old: float, new: float, bottom: int, eps: float = 1e-5, block_h: int = 512) -> None:
    """Reach-weighted average-policy mix before renormalisation (fused_cfr_triton.py:823-876)."""
    _need()
    _req(policy_probs_avg.is_contiguous() and policy_probs_avg.dim() == 2,
         "policy_probs_avg.is_contiguous() and policy_probs_avg.dim() == 2")
    _req(policy_probs.is_contiguous() and policy_probs.dim() == 2,
         "policy_probs.is_contiguous() and policy_probs.dim() == 2")
    _req(self_reach.is_contiguous() and self_reach.dim() == 3, "self_reach.is_contiguous() and self_reach.dim() == 3")
    _req(self_reach_avg.is_contiguous() and self_reach_avg.dim() == 3,
         "self_reach_avg.is_contiguous() and self_reach_avg.dim() == 3")
    _req(self_reach.shape[1] == 2 and self_reach_avg.shape[1] == 2,
         "self_reach.shape[1] == 2 and self_reach_avg.shape[1] == 2")
    total, h = policy_probs_avg.shape
    _req(policy_probs.shape == (total, h), "policy_probs.shape == (total, h)")
    _req(self_reach.shape == (total, 2, h), "self_reach.shape == (total, 2, h)")
    _req(self_reach_avg.shape == (total, 2, h), "self_reach_avg.shape == (total, 2, h)")
    _req(to_act.shape == (total,), "to_act.shape == (total,)")
    _req(parent_index.shape == (total,), "parent_index.shape == (total,)")
    total_weight = float(old) + float(new)
    _req(total_weight != 0.0, "total_weight != 0.0")
    o_t, n_t, tot_t = _scalars([old, new, total_weight], policy_probs_avg)
    fused_average_policy_mix_with_tensors_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act,
                                           parent_index, o_t, n_t, tot_t, bottom=bottom, eps=eps, block_h=block_h)


def fused_average_policy_mix_with_tensors_(policy_probs_avg, policy_probs, self_reach, self_reach_avg, to_act,
                                           parent_index, old, new, total_weight, bottom: int, eps: float = 1e-5,
                                           block_h: int = 512) -> None:
    """fused_cfr_triton.py:879-914."""
    _need()
    _req(policy_probs_avg.dim() == 2, "policy_probs_avg.dim() == 2")
    total, h = policy_probs_avg.shape
    _f32(policy_probs_avg=policy_probs_avg, policy_probs=policy_probs, self_reach=self_reach,
         self_reach_avg=self_reach_avg)
    _req(policy_probs.shape == (total, h) and self_reach.shape == (total, 2, h)
         and self_reach_avg.shape == (total, 2, h), "policy / reach tensors differ in shape")
    _i64(total, to_act=to_act, parent_index=parent_index)
    _scalar_ptrs(old=old, new=new, total_weight=total_weight)
    _req(0 <= int(bottom) <= total, f"bottom={bottom} outside the {total} rows")
    _lib.call("p2hip_average_policy_mix", _p(policy_probs_avg), _p(policy_probs), _p(self_reach), _p(self_reach_avg),
              _p(to_act), _p(parent_index), _p(old), _p(new), _p(total_weight), int(bottom), total, float(eps), _S())


# --------------------------------------------------------------------------- K9 / K12
def unblocked_mass_triton(target: torch.Tensor) -> torch.Tensor:
    """[..., 1326] -> unblocked mass of each combo (fused_cfr_triton.py:1110-1157)."""
    _need()
    if target.device.type != "cuda":
        raise ValueError("unblocked_mass requires GPU tensors.")
    orig_shape = target.shape
    _req(orig_shape[-1] == _H, f"last dim must be {_H}, got {orig_shape}")
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
    _req(p == 2 and h == _H, "p == 2 and h == _H")
    _req(beliefs.is_contiguous() and to_act.is_contiguous() and to_act.dtype == torch.int64,
         "beliefs.is_contiguous() and to_act.is_contiguous() and to_act.dtype == torch.int64")
    _req(0 <= int(top) <= total, f"top={top} outside the {total} rows of beliefs")
    _i64(int(top), to_act=to_act)
    _f32(beliefs=beliefs)
    out = torch.empty((top, h), device=beliefs.device, dtype=beliefs.dtype)
    _lib.call("p2hip_unblocked_mass_by_player", _p(beliefs), _p(to_act), int(top), 1, _p(out), _S())
    return out


def unblocked_mass_ratio_indirect_triton(numer_target, denom_target, parent_index, eps: float = 1e-5,
                                         denom_stats=None) -> torch.Tensor:
    """where(unblk(denom[parent]) > eps, unblk(numer) / unblk(denom[parent]), 0)
    (fused_cfr_triton.py:1499-1556).  ``denom_stats`` is accepted and ignored."""
    _need()
    _req(numer_target.is_contiguous() and numer_target.dim() == 2,
         "numer_target.is_contiguous() and numer_target.dim() == 2")
    _req(denom_target.is_contiguous() and denom_target.dim() == 2,
         "denom_target.is_contiguous() and denom_target.dim() == 2")
    _req(parent_index.is_contiguous() and parent_index.dim() == 1,
         "parent_index.is_contiguous() and parent_index.dim() == 1")
    num_children, h = numer_target.shape
    top = denom_target.shape[0]
    _req(denom_target.shape == (top, h), "denom_target.shape == (top, h)")
    _req(parent_index.shape == (num_children,), "parent_index.shape == (num_children,)")
    _req(h == _H, "h == _H")
    _f32(numer_target=numer_target, denom_target=denom_target)
    _i64(num_children, parent_index=parent_index)
    out = torch.empty_like(numer_target)
    if num_children > top:
        # siblings share a denominator: its unblocked mass once per parent, then the quotients
        denom_unblocked = torch.empty_like(denom_target)
        _lib.call("p2hip_unblocked_mass", _p(denom_target), top, _p(denom_unblocked), _S())
        _lib.call("p2hip_unblocked_mass_ratio_of", _p(numer_target), _p(denom_unblocked), _p(parent_index),
                  num_children, float(eps), _p(out), _S())
    else:
        _lib.call("p2hip_unblocked_mass_ratio", _p(numer_target), _p(denom_target), _p(parent_index), num_children,
                  float(eps), _p(out), _S())
    return out


def unblocked_mass_ratio_triton(numer_target, denom_target, eps: float = 1e-5) -> torch.Tensor:
    """fused_cfr_triton.py:1559-1602."""
    _need()
    _req(numer_target.shape == denom_target.shape, "numer_target.shape == denom_target.shape")
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
    _req(values.is_contiguous() and values.dim() == 2, "values.is_contiguous() and values.dim() == 2")
    _req(child_offsets.is_contiguous() and child_offsets.dim() == 1,
         "child_offsets.is_contiguous() and child_offsets.dim() == 1")
    _req(child_count.is_contiguous() and child_count.shape == child_offsets.shape,
         "child_count.is_contiguous() and child_count.shape == child_offsets.shape")
    num_parents = child_offsets.shape[0]
    _f32(values=values)
    _req(values.shape[1] == _H, "values.shape[1] == 1326")
    _i64(num_parents, child_offsets=child_offsets, child_count=child_count)
    out = torch.empty(num_parents, values.shape[1], device=values.device, dtype=values.dtype)
    _lib.call("p2hip_parent_sum", _p(values), _p(child_offsets), _p(child_count), num_parents, _p(out), _S())
    return out


def fused_divide_by_parent_sum_(pos, fallback, parent_sum, parent_index, out, eps: float = 1e-8, block_c: int = 32,
                                block_h: int = 128) -> None:
    """out[c] = where(parent_sum[parent(c)] > eps, pos[c] / max(parent_sum, eps), fallback[c])
    (fused_cfr_triton.py:1316-1352); ``out`` may alias ``pos`` or ``fallback``."""
    _need()
    _req(pos.is_contiguous() and fallback.is_contiguous() and out.is_contiguous(),
         "pos.is_contiguous() and fallback.is_contiguous() and out.is_contiguous()")
    _req(parent_sum.is_contiguous() and parent_index.is_contiguous(),
         "parent_sum.is_contiguous() and parent_index.is_contiguous()")
    _req(pos.dim() == 2 and fallback.shape == pos.shape == out.shape,
         "pos.dim() == 2 and fallback.shape == pos.shape == out.shape")
    _req(parent_sum.dim() == 2 and parent_sum.shape[1] == pos.shape[1],
         "parent_sum.dim() == 2 and parent_sum.shape[1] == pos.shape[1]")
    num_children, _ = pos.shape
    _req(parent_index.shape == (num_children,), "parent_index.shape == (num_children,)")
    _f32(pos=pos, fallback=fallback, parent_sum=parent_sum, out=out)
    _i64(num_children, parent_index=parent_index)
    _lib.call("p2hip_divide_by_parent_sum", _p(pos), _p(fallback), _p(parent_sum), _p(parent_index), _p(out),
              num_children, float(eps), _S())


def fused_sibling_sum(values, child_offsets, child_count, bottom: int, num_children: int, max_children: int = 8,
                      block_h: int = 512) -> torch.Tensor:
    """Sum over each child's siblings, child-aligned -> [num_children, H] (fused_cfr_triton.py:1355-1398)."""
    _need()
    _req(values.is_contiguous() and values.dim() == 2, "values.is_contiguous() and values.dim() == 2")
    _req(child_offsets.is_contiguous() and child_offsets.dim() == 1,
         "child_offsets.is_contiguous() and child_offsets.dim() == 1")
    _req(child_count.is_contiguous() and child_count.dim() == 1,
         "child_count.is_contiguous() and child_count.dim() == 1")
    _req(child_offsets.shape == child_count.shape, "child_offsets.shape == child_count.shape")
    _f32(values=values)
    _req(values.shape[1] == _H, "values.shape[1] == 1326")
    _i64(child_offsets.shape[0], child_offsets=child_offsets, child_count=child_count)
    _req(0 <= int(bottom) and 0 <= int(num_children) and int(bottom) + int(num_children) <= values.shape[0],
         f"children [{bottom}, {bottom}+{num_children}) outside the {values.shape[0]} rows of values")
    out = torch.empty(num_children, values.shape[1], device=values.device, dtype=values.dtype)
    _lib.call("p2hip_sibling_sum", _p(values), _p(child_offsets), _p(child_count), child_offsets.shape[0],
              int(bottom), _p(out), _S())
    return out


# --------------------------------------------------------------------------- K13
def fused_model_values_mix(hand_values, last_model_values, old: float, new: float,
                           block_size: int = 1024) -> torch.Tensor:
    """((old+new)*hand - old*last)/new with pre-divided scalars (fused_cfr_triton.py:1633-1655)."""
    _need()
    _req(hand_values.is_contiguous() and last_model_values.is_contiguous(),
         "hand_values.is_contiguous() and last_model_values.is_contiguous()")
    _req(hand_values.shape == last_model_values.shape, "hand_values.shape == last_model_values.shape")
    _req(new != 0.0, "new != 0.0")
    out = torch.empty_like(hand_values)
    onon_t, oon_t = _scalars([(old + new) / new, old / new], hand_values)
    fused_model_values_mix_with_tensors(hand_values, last_model_values, onon_t, oon_t, out, block_size=block_size)
    return out


def fused_model_values_mix_with_tensors(hand_values, last_model_values, old_plus_new_over_new, old_over_new, out,
                                        block_size: int = 1024) -> None:
    """fused_cfr_triton.py:1658-1680."""
    _need()
    _f32(hand_values=hand_values, last_model_values=last_model_values, out=out)
    _req(hand_values.shape == last_model_values.shape == out.shape, "hand_values / last_model_values / out differ")
    _scalar_ptrs(old_plus_new_over_new=old_plus_new_over_new, old_over_new=old_over_new)
    _lib.call("p2hip_model_values_mix", _p(hand_values), _p(last_model_values), _p(old_plus_new_over_new),
              _p(old_over_new), _p(out), hand_values.numel(), _S())


def fused_model_values_mix_zero_sum(hand_values, last_model_values, beliefs, old_plus_new_over_new, old_over_new,
                                    out, enforce_zero_sum: bool, block_h: int = 2048) -> None:
    """fused_cfr_triton.py:1739-1775."""
    _need()
    _req(hand_values.is_contiguous() and last_model_values.is_contiguous(),
         "hand_values.is_contiguous() and last_model_values.is_contiguous()")
    _req(beliefs.is_contiguous() and out.is_contiguous(), "beliefs.is_contiguous() and out.is_contiguous()")
    _req(hand_values.shape == last_model_values.shape == beliefs.shape == out.shape,
         "hand_values.shape == last_model_values.shape == beliefs.shape == out.shape")
    _req(hand_values.dim() == 3 and hand_values.shape[1] == 2, "hand_values.dim() == 3 and hand_values.shape[1] == 2")
    m, _, h = hand_values.shape
    _req(h == _H, "h == _H")
    _f32(hand_values=hand_values, last_model_values=last_model_values, beliefs=beliefs, out=out)
    _scalar_ptrs(old_plus_new_over_new=old_plus_new_over_new, old_over_new=old_over_new)
    _lib.call("p2hip_model_values_mix_zero_sum", _p(hand_values), _p(last_model_values), _p(beliefs),
              _p(old_plus_new_over_new), _p(old_over_new), _p(out), m, int(bool(enforce_zero_sum)), _S())


# --------------------------------------------------------------------------- K14 / K15 / K16
def fused_weighted_parent_sum(values, prev_actor, policy_hero, policy_opp, child_offsets, child_count,
                              parent_base: int, max_children: int = 8, block_h: int = 2048) -> None:
    """values[parent_base+p, pl] = sum_children values[c, pl] * (policy_hero[c] if pl == prev_actor[c]
    else policy_opp[c]); parents without children keep their value (fused_cfr_triton.py:1838-1889)."""
    _need()
    _req(values.is_contiguous() and values.dim() == 3 and values.shape[1] == 2,
         "values.is_contiguous() and values.dim() == 3 and values.shape[1] == 2")
    _req(policy_hero.is_contiguous() and policy_opp.is_contiguous(),
         "policy_hero.is_contiguous() and policy_opp.is_contiguous()")
    _req(child_offsets.is_contiguous() and child_count.is_contiguous(),
         "child_offsets.is_contiguous() and child_count.is_contiguous()")
    total, _, h = values.shape
    _req(policy_hero.shape == (total, h) and policy_opp.shape == (total, h),
         "policy_hero.shape == (total, h) and policy_opp.shape == (total, h)")
    _req(prev_actor.shape == (total,), "prev_actor.shape == (total,)")
    _f32(values=values, policy_hero=policy_hero, policy_opp=policy_opp)
    _req(h == _H, "values.shape[2] == 1326")
    num_parents = child_offsets.shape[0]
    _i64(total, prev_actor=prev_actor)
    _i64(num_parents, child_offsets=child_offsets, child_count=child_count)
    _req(0 <= int(parent_base) and int(parent_base) + num_parents <= total,
         f"parents [{parent_base}, {parent_base}+{num_parents}) outside the {total} rows")
    _lib.call("p2hip_weighted_parent_sum", _p(values), _p(prev_actor), _p(policy_hero), _p(policy_opp),
              _p(child_offsets), _p(child_count), child_offsets.shape[0], int(parent_base), _S())


def fused_reach_weights_depth_(reach, policy, allowed_mask, parent_index, prev_actor, start: int, end: int,
                               block_h: int = 2048) -> None:
    """reach[c,p] = reach[parent(c),p] * (policy[c] if p == prev_actor[c] else 1), zero where
    ``allowed_mask[c]`` is False, for c in [start, end) (fused_cfr_triton.py:1944-1986)."""
    _need()
    _req(reach.is_contiguous() and reach.dim() == 3 and reach.shape[1] == 2,
         "reach.is_contiguous() and reach.dim() == 3 and reach.shape[1] == 2")
    _req(policy.is_contiguous() and policy.dim() == 2, "policy.is_contiguous() and policy.dim() == 2")
    total, _, h = reach.shape
    _req(policy.shape == (total, h), "policy.shape == (total, h)")
    _req(allowed_mask.shape == (total, h) and allowed_mask.is_contiguous() and allowed_mask.dtype == torch.bool,
         "allowed_mask.shape == (total, h) and allowed_mask.is_contiguous() and allowed_mask.dtype == torch.bool")
    _req(parent_index.shape == (total,) and prev_actor.shape == (total,),
         "parent_index.shape == (total,) and prev_actor.shape == (total,)")
    _f32(reach=reach, policy=policy)
    _req(h == _H, "reach.shape[2] == 1326")
    _i64(total, parent_index=parent_index, prev_actor=prev_actor)
    if end - start <= 0:
        return
    _req(0 <= int(start) and int(end) <= total, f"rows [{start}, {end}) outside the {total} rows")
    _lib.call("p2hip_reach_weights_depth", _p(reach), _p(policy), _p(allowed_mask), _p(parent_index),
              _p(prev_actor), int(start), int(end), _S())


def fused_deep_beliefs_(out, root_beliefs, reach_weights, allowed_prob, root_index, num_roots: int | None = None,
                        eps: float = 1e-5, block_h: int = 2048) -> None:
    """out[i,p] = normalise(root_beliefs[root_index[i],p] * reach_weights[i,p]) with fallback
    ``allowed_prob[i]``; root rows are left untouched (fused_cfr_triton.py:2039-2092)."""
    _need()
    _req(out.is_contiguous() and out.dim() == 3 and out.shape[1] == 2,
         "out.is_contiguous() and out.dim() == 3 and out.shape[1] == 2")
    _req(root_beliefs.is_contiguous() and root_beliefs.dim() == 3,
         "root_beliefs.is_contiguous() and root_beliefs.dim() == 3")
    _req(reach_weights.is_contiguous() and reach_weights.shape == out.shape,
         "reach_weights.is_contiguous() and reach_weights.shape == out.shape")
    total, _, h = out.shape
    n = num_roots if num_roots is not None else root_beliefs.shape[0]
    _req(root_beliefs.shape[0] >= n and tuple(root_beliefs.shape[1:]) == (2, h),
         "root_beliefs.shape[0] >= n and tuple(root_beliefs.shape[1:]) == (2, h)")
    _req(allowed_prob.shape == (total, h) and allowed_prob.is_contiguous(),
         "allowed_prob.shape == (total, h) and allowed_prob.is_contiguous()")
    _req(root_index.shape == (total,) and root_index.is_contiguous(),
         "root_index.shape == (total,) and root_index.is_contiguous()")
    _f32(out=out, root_beliefs=root_beliefs, reach_weights=reach_weights, allowed_prob=allowed_prob)
    _req(h == _H, "out.shape[2] == 1326")
    _i64(total, root_index=root_index)
    if total <= n:
        return
    _lib.call("p2hip_deep_beliefs", _p(out), _p(root_beliefs), _p(reach_weights), _p(allowed_prob), _p(root_index),
              int(n), total, float(eps), _S())


def showdown_ev_triton(b_opp_sorted, c1_sorted, c2_sorted, L_idx, R_idx, eps: float = 1e-8, block_k: int = 32,
                       block_j: int = 128) -> torch.Tensor:
    """Showdown EV per hand, in strength order, from strength-sorted inputs: the villain range
    ``b_opp_sorted`` [M, 1326], the two cards of each sorted hand and its tie group [L, R)
    (fused_cfr_triton.py:2271-2314; un-sorting, the board mask and potential / scale stay with the
    caller, as there).  Each row must list every one of the 1326 hands once.  Runs the same kernels
    as the evaluator's showdown: a table is built from the sorted hands, then both prefix passes."""
    _need()
    from . import rules_hip
    _req(b_opp_sorted.is_contiguous() and b_opp_sorted.dim() == 2, "b_opp_sorted must be contiguous [M, H]")
    m, h = b_opp_sorted.shape
    _req(h == _H, "b_opp_sorted.shape[1] == 1326")
    _req(c1_sorted.shape == (m, h) and c2_sorted.shape == (m, h), "c1_sorted / c2_sorted must be [M, H]")
    _req(L_idx.shape == (m, h) and R_idx.shape == (m, h), "L_idx / R_idx must be [M, H]")
    _f32(b_opp_sorted=b_opp_sorted)
    if float(eps) != 1e-8:
        raise NotImplementedError("the showdown kernels are built for eps = 1e-8, the evaluator's value")
    dev = b_opp_sorted.device
    if m == 0:
        return torch.empty(0, h, device=dev, dtype=torch.float32)
    c1 = c1_sorted.to(device=dev, dtype=torch.int32).contiguous()
    c2 = c2_sorted.to(device=dev, dtype=torch.int32).contiguous()
    lo_idx = L_idx.to(device=dev, dtype=torch.int32).contiguous()
    hi_idx = R_idx.to(device=dev, dtype=torch.int32).contiguous()
    tables = torch.empty(m, rules_hip.showdown_table_bytes(), dtype=torch.uint8, device=dev)
    bad = torch.empty(m, dtype=torch.int32, device=dev)
    _lib.call("p2hip_showdown_setup_sorted", _p(c1), _p(c2), _p(lo_idx), _p(hi_idx), m, _p(tables), _p(bad), _S())
    if bool(bad.any()):
        rows = torch.nonzero(bad).flatten().tolist()[:8]
        raise ValueError(f"rows {rows} do not list each of the 1326 hands once with a tie group 0 <= L <= k < R <= 1326")
    lo, hi = torch.minimum(c1, c2).long(), torch.maximum(c1, c2).long()
    combo = lo * (103 - lo) // 2 + (hi - lo - 1)                       # index of (lo, hi) among the 1326 hands
    beliefs = torch.zeros(m, 2, h, device=dev, dtype=torch.float32)
    beliefs[:, 1].scatter_(1, combo, b_opp_sorted)                      # hero 0 faces this range
    ones = torch.ones(m, 2, device=dev, dtype=torch.float32)
    ev = rules_hip.showdown_value_both(beliefs, tables, ones, ones[:, 0].contiguous())
    return ev[:, 0].gather(1, combo)


def fused_sample_snapshot_(policy_probs_sample, policy_probs, t_sample, t_tensor) -> None:
    """policy_probs_sample <- where(t_sample == t, policy_probs, policy_probs_sample)
    (fused_sparse_cfr_evaluator.py:494-499); ``t_tensor`` is a 0-D int64 device tensor."""
    _need()
    _req(policy_probs_sample.is_contiguous() and policy_probs.is_contiguous(),
         "policy_probs_sample.is_contiguous() and policy_probs.is_contiguous()")
    _req(policy_probs_sample.shape == policy_probs.shape, "policy_probs_sample.shape == policy_probs.shape")
    _req(t_sample.is_contiguous() and t_sample.dtype == torch.int64 and t_tensor.dtype == torch.int64,
         "t_sample.is_contiguous() and t_sample.dtype == torch.int64 and t_tensor.dtype == torch.int64")
    _f32(policy_probs_sample=policy_probs_sample, policy_probs=policy_probs)
    _req(policy_probs.dim() == 2 and policy_probs.shape[1] == _H, "policy_probs must be [rows, 1326]")
    _i64(policy_probs.shape[0], t_sample=t_sample)
    _req(t_tensor.numel() >= 1 and t_tensor.device.type == "cuda", "t_tensor must be a GPU scalar tensor")
    _lib.call("p2hip_sample_snapshot", _p(policy_probs), _p(policy_probs_sample), _p(t_sample), _p(t_tensor),
              policy_probs.shape[0], _S())


# --------------------------------------------------------------------------- TScalars
class TScalars:
    """0-D device tensors holding the iteration-dependent scalars (fused_cfr_triton.py:2100-2158).
    ``update`` copies host values in and must run outside any captured region.

    On the GPU the float scalars are views into one array (``floats``: alpha and beta numerators,
    their denominators, mix_old, mix_new, their sum, its reciprocal, then mix_onon and mix_oon) and
    ``t_tensor`` is element 0 of ``ints``, so that one small launch that carries the values as kernel
    arguments refreshes all of them (a ``fill_`` per scalar is eleven launches, 50-60 us of an
    iteration however small the batch).  The first eight floats and the eight ints are the arrays the
    one-kernel iteration reads."""

    _NAMES = ("t_alpha_num", "t_beta_num", "t_alpha_den", "t_beta_den", "mix_old", "mix_new", "mix_total",
              "mix_inv_total", "mix_onon", "mix_oon")

    def __init__(self, device: torch.device, dtype: torch.dtype = torch.float32) -> None:
        self.device = torch.device(device)
        self.dtype = dtype
        self._packed = self.device.type == "cuda" and dtype == torch.float32
        if self._packed:
            self.floats = torch.zeros(16, dtype=torch.float32, device=device)
            self.ints = torch.zeros(8, dtype=torch.int64, device=device)
            for k, name in enumerate(self._NAMES):
                setattr(self, name, self.floats[k])
            self.t_tensor = self.ints[0]
            self._host_f = (ctypes.c_float * 8)()
            self._host_i = (ctypes.c_int64 * 8)()
            self._host_x = (ctypes.c_float * 8)()
        else:
            for name in self._NAMES:
                setattr(self, name, torch.zeros((), dtype=dtype, device=device))
            self.t_tensor = torch.zeros((), dtype=torch.long, device=device)

    def write(self, host_f, host_i, onon_oon: tuple[float, float] | None = None) -> None:
        """``floats[:8]`` and ``ints[:8]`` from two host arrays of eight (ctypes float / int64), and the
        two CFR-AVG de-averaging factors if given: one launch, or two."""
        _req(self._packed, "TScalars.write: float32 scalars on the GPU")
        _lib.call("p2hip_write_scalars", _lib.ptr(self.floats), _lib.ptr(self.ints),
                  ctypes.cast(host_f, ctypes.c_void_p), ctypes.cast(host_i, ctypes.c_void_p), _lib.stream_ptr())
        if onon_oon is not None:
            x = self._host_x
            x[0], x[1] = onon_oon
            _lib.call("p2hip_upload_floats", _lib.ptr(self.floats) + 8 * 4, ctypes.cast(x, ctypes.c_void_p), 2,
                      _lib.stream_ptr())

    @staticmethod
    def deaveraging_factors(mix_old: float, mix_new: float) -> tuple[float, float] | None:
        """(total / new, old / new) of the CFR-AVG de-averaging; None while ``mix_new`` is zero (the
        scalars then keep their last values, fused_cfr_triton.py:2150-2156)."""
        if float(mix_new) == 0.0:
            return None
        return (float(mix_old) + float(mix_new)) / float(mix_new), float(mix_old) / float(mix_new)

    def update(self, t: int, dcfr_alpha: float, dcfr_beta: float, mix_old: float, mix_new: float) -> None:
        (t_alpha_num, t_alpha_den), (t_beta_num, t_beta_den) = discount_pair(t, dcfr_alpha), discount_pair(t, dcfr_beta)
        total = float(mix_old) + float(mix_new)
        inv_total = 1.0 / total if total != 0.0 else 1.0
        extra = self.deaveraging_factors(mix_old, mix_new)
        if self._packed:
            f, i = self._host_f, self._host_i
            f[0], f[1], f[2], f[3] = t_alpha_num, t_beta_num, t_alpha_den, t_beta_den
            f[4], f[5], f[6], f[7] = float(mix_old), float(mix_new), total, inv_total
            i[0] = int(t)                      # ints[1:] belong to whoever reads them: zero here
            self.write(f, i, extra)
            return
        for name, value in zip(self._NAMES[:8], (t_alpha_num, t_beta_num, t_alpha_den, t_beta_den, float(mix_old),
                                                 float(mix_new), total, inv_total)):
            getattr(self, name).fill_(value)
        if extra is not None:
            self.mix_onon.fill_(extra[0])
            self.mix_oon.fill_(extra[1])
        self.t_tensor.fill_(int(t))


class ParentBeliefUnblockedStats:
    """Total and per-card sums of both players' beliefs at the parent rows
    (fused_cfr_triton.py:1029-1064).  The HIP kernels take their card sums inside the kernel, so
    passing this object as ``cached_stats`` changes nothing; it exists for callers that build it."""

    def __init__(self, beliefs_parents: torch.Tensor) -> None:
        _req(beliefs_parents.dim() == 3 and beliefs_parents.shape[1] == 2,
             "beliefs_parents.dim() == 3 and beliefs_parents.shape[1] == 2")
        self.top = beliefs_parents.shape[0]
        self.beliefs_parents = beliefs_parents

    def slice_for_player(self, player_per_node: torch.Tensor):
        from .card_utils import combo_to_onehot_tensor
        rows = torch.arange(self.top, device=self.beliefs_parents.device)
        target = self.beliefs_parents[rows, player_per_node, :].contiguous()
        onehot = combo_to_onehot_tensor(device=target.device).to(target.dtype)
        return target, target.sum(dim=-1), target @ onehot


def __getattr__(name):
    # The graph runner and the state snapshot live with the evaluator (which imports this module);
    # the reference exports both from fused_cfr_triton.py:2322-2451
    if name in ("GraphedCFRIteration", "_EvaluatorStateSnapshot"):
        from . import evaluator
        return getattr(evaluator, name)
    raise AttributeError(name)
