"""Seeded inputs of the per-operation CFR kernels and three ways to run them.

One table serves the fixture writer (tests/golden/gen_fused_ops_golden.py: the reference's own
Triton kernels under Triton's CPU interpreter), the CPU test of the oracle and the GPU test of
the product.  ``torch_ops(F, t)`` works for any module that exports the reference's function names
(the reference's ``fused_cfr_triton`` and ``poker2_amd.fused_cfr_hip`` alike); ``oracle_ops(x)``
runs the numpy restatement.  Every case returns a dict of named outputs.
"""
from __future__ import annotations

import numpy as np

from tests.helpers import H, random_tree

F32 = np.float32


def _tree(seed, n_roots, depth):
    return random_tree(np.random.default_rng(seed), n_roots, depth)


def _norm(x):
    return (x / x.sum(-1, keepdims=True)).astype(F32)


# ---- inputs ---------------------------------------------------------------------------------
def inputs(name: str) -> dict:
    rng = np.random.default_rng(abs(hash_name(name)))
    r = lambda *s: rng.random(s).astype(F32)             # noqa: E731
    g = lambda *s: rng.standard_normal(s).astype(F32)    # noqa: E731
    if name.startswith("dcfr_update"):
        t, apply_dcfr, cfr_plus = {"dcfr_update_t7": (7, True, False), "dcfr_update_t50_plus": (50, True, True),
                                   "dcfr_update_standard": (3, False, False), "dcfr_update_t0": (0, True, False)}[name]
        return dict(cum=g(19, H), wsum=r(19, H) * 5, regrets=g(19, H) * F32(0.1), t=t, apply_dcfr=apply_dcfr,
                    cfr_plus=cfr_plus, alpha=1.5, beta=0.5)
    if name in ("block_normalize_3d", "block_normalize_2d"):
        n = 13
        target = r(n, 2, H) if name.endswith("3d") else r(n, H)
        allowed = rng.random((n, H)) > 0.3
        allowed[3] = False
        if name.endswith("3d"):
            target[5, 1] = 0.0
        return dict(target=target, allowed=allowed, prob=r(n, H))
    if name == "regret_matching_divide":
        den = r(17, H)
        den[::3] = 0.0
        return dict(pos=r(17, H), den=den, uni=r(17, H))
    if name == "weight_child_values":
        return dict(values=g(15, 2, H), prev_actor=rng.integers(0, 2, 15).astype(np.int64), hero=r(15, H), opp=r(15, H))
    if name == "update_average_values":
        return dict(avg=g(12, 2, H), latest=g(12, 2, H), old=9.0, new=16.0)
    if name.startswith("avg_values_zero_sum"):
        n = 11
        enforce, with_ignore = {"avg_values_zero_sum": (True, False), "avg_values_zero_sum_ignore": (True, True),
                                "avg_values_zero_sum_off": (False, False)}[name]
        return dict(avg=g(n, 2, H), latest=g(n, 2, H), beliefs=_norm(r(n, 2, H)), old=4.0, new=9.0, enforce=enforce,
                    ignore=(rng.random(n) > 0.5) if with_ignore else None)
    if name == "regret_tail":
        tr = _tree(1, 4, 3)
        return dict(tree=tr, achieved=g(tr["total"], 2, H), actor_values=g(tr["top"], H), src_w=g(tr["top"], H))
    if name == "average_policy_mix":
        tr = _tree(2, 4, 3)
        reach, reach_avg = r(tr["total"], 2, H), r(tr["total"], 2, H)
        reach[:, :, ::5] = 0.0
        reach_avg[:, :, ::5] = 0.0
        return dict(tree=tr, reach=reach, reach_avg=reach_avg, policy=r(tr["total"], H), policy_avg=r(tr["total"], H),
                    old=3.0, new=2.0)
    if name == "parent_sibling_divide":
        tr = _tree(3, 5, 3)
        nchild = tr["total"] - tr["bottom"]
        return dict(tree=tr, values=g(tr["total"], H), pos=r(nchild, H), fallback=r(nchild, H))
    if name == "model_values_mix":
        return dict(h=g(14, 2, H), last=g(14, 2, H), beliefs=_norm(r(14, 2, H)), old=5.0, new=3.0)
    if name == "weighted_parent_sum":
        tr = _tree(4, 4, 3)
        return dict(tree=tr, values=g(tr["total"], 2, H), hero=r(tr["total"], H), opp=r(tr["total"], H))
    if name == "reach_and_deep_beliefs":
        tr = _tree(5, 3, 3)
        total = tr["total"]
        reach = r(total, 2, H)
        reach[: tr["bottom"]] = 1.0          # root rows as the evaluator keeps them: 1 on every hand, blocked ones included
        return dict(tree=tr, reach=reach, policy=r(total, H), allowed=rng.random((total, H)) > 0.2,
                    beliefs=r(total, 2, H), prob=r(total, H))
    if name == "unblocked_mass":
        return dict(target=r(9, 2, H))
    if name == "unblocked_opp_and_ratio":
        total, top, nchild = 21, 8, 26
        actor = _norm(r(top, H))
        actor[2] = 0.0
        pidx = rng.integers(0, top, nchild).astype(np.int64)
        return dict(beliefs=r(total, 2, H), to_act=rng.integers(0, 2, total).astype(np.int64), top=top, actor=actor,
                    pidx=pidx, numer=(actor[pidx] * r(nchild, H)).astype(F32))
    if name == "showdown_sorted":
        # the boards of the reference's showdown scenarios (tests/test_rebel_cfr_evaluator.py:1220-1537:
        # "Ac Qh 9d 7s 4h", the royal board where every hand ties, a paired board) and two drawn ones
        from oracle import cards as OC
        from oracle import showdown as OS
        card = lambda txt: "23456789TJQKA".index(txt[0]) + 13 * "cdhs".index(txt[1])    # noqa: E731
        boards = [[card(c) for c in b.split()] for b in ("Ac Qh 9d 7s 4h", "Ah Kh Qh Jh Th", "Tc Th Ts 7d 7h")]
        boards += [rng.permutation(52)[:5].tolist() for _ in range(2)]
        boards = np.asarray(boards, dtype=np.int64)
        allowed = OC.allowed_hands_for_boards(boards)[0]
        hrd = OS.init_hand_rank_data(boards, allowed)
        bel = rng.gamma(0.5, size=(len(boards), 2, H)).astype(F32) * allowed[:, None, :]
        bel[4, 1, :] = 0.0
        bel[4, 1, np.nonzero(allowed[4])[0][:3]] = 1.0          # a villain range of three hands
        bel = _norm(bel)
        return dict(boards=boards, allowed=allowed, beliefs=bel, hrd=hrd)
    raise KeyError(name)


NAMES = ("dcfr_update_t0", "dcfr_update_t7", "dcfr_update_t50_plus", "dcfr_update_standard", "block_normalize_3d",
         "block_normalize_2d", "regret_matching_divide", "weight_child_values", "update_average_values",
         "avg_values_zero_sum", "avg_values_zero_sum_ignore", "avg_values_zero_sum_off", "regret_tail",
         "average_policy_mix", "parent_sibling_divide", "model_values_mix", "weighted_parent_sum",
         "reach_and_deep_beliefs", "unblocked_mass", "unblocked_opp_and_ratio", "showdown_sorted")


def hash_name(name: str) -> int:
    """A stable seed per case (Python's hash() is salted per process)."""
    h = 2166136261
    for ch in name.encode():
        h = ((h ^ ch) * 16777619) & 0xFFFFFFFF
    return h


# ---- the numpy oracle ---------------------------------------------------------------------------
def oracle_ops(name: str, x: dict) -> dict:
    from oracle import cfr_ops as O
    from oracle import unblocked as OU
    if name.startswith("dcfr_update"):
        c, w, p = O.dcfr_update(x["cum"], x["wsum"], x["regrets"], x["t"], x["alpha"], x["beta"], x["apply_dcfr"],
                                x["cfr_plus"])
        return dict(cum=c, wsum=w, positive=p)
    if name.startswith("block_normalize"):
        return dict(target=O.block_and_normalize(x["target"], x["allowed"], x["prob"]))
    if name == "regret_matching_divide":
        return dict(out=O.regret_matching_divide(x["pos"], x["den"], x["uni"]))
    if name == "weight_child_values":
        return dict(out=O.weight_child_values(x["values"], x["prev_actor"], x["hero"], x["opp"]))
    if name == "update_average_values":
        a = O.update_average_values(x["avg"], x["latest"], x["old"], x["new"])
        return dict(avg=a, avg_floats=a)
    if name.startswith("avg_values_zero_sum"):
        return dict(avg=O.avg_values_zero_sum(x["avg"], x["latest"], x["beliefs"], x["old"], x["new"], x["enforce"],
                                              x["ignore"]))
    tr = x.get("tree")
    if name == "regret_tail":
        return dict(regrets=O.regret_tail(x["achieved"], x["actor_values"], x["src_w"], tr["parent_index"],
                                          tr["prev_actor"], tr["bottom"]))
    if name == "average_policy_mix":
        a = O.average_policy_mix(x["policy_avg"], x["policy"], x["reach"], x["reach_avg"], tr["to_act"],
                                 tr["parent_index"], x["old"], x["new"], tr["bottom"])
        return dict(policy_avg=a, policy_avg_tensors=a)
    if name == "parent_sibling_divide":
        top, bottom = tr["top"], tr["bottom"]
        co, cc = tr["child_offsets"][:top], tr["child_count"][:top]
        ps = O.parent_sum(x["values"], co, cc)
        ss = O.sibling_sum(x["values"], co, cc, bottom, tr["total"] - bottom)
        psum = np.abs(ps)
        psum[:, ::4] = 0.0
        return dict(parent_sum=ps, sibling_sum=ss,
                    divided=O.divide_by_parent_sum(x["pos"], x["fallback"], psum, tr["parent_index"][bottom:]))
    if name == "model_values_mix":
        m = O.model_values_mix(x["h"], x["last"], x["old"], x["new"])
        return dict(mix=m, mix_tensors=m,
                    mix_zs=O.model_values_mix_zero_sum(x["h"], x["last"], x["beliefs"], x["old"], x["new"], True),
                    mix_nozs=O.model_values_mix_zero_sum(x["h"], x["last"], x["beliefs"], x["old"], x["new"], False))
    if name == "weighted_parent_sum":
        v, offs = x["values"].copy(), tr["depth_offsets"]
        for d in range(len(offs) - 3, -1, -1):
            base, end = offs[d], offs[d + 1]
            v = O.weighted_parent_sum(v, tr["prev_actor"], x["hero"], x["opp"], tr["child_offsets"][base:end],
                                      tr["child_count"][base:end], base)
        return dict(values=v)
    if name == "reach_and_deep_beliefs":
        reach, offs, n = x["reach"].copy(), tr["depth_offsets"], tr["bottom"]
        for d in range(len(offs) - 2):
            reach = O.reach_weights_depth(reach, x["policy"], x["allowed"], tr["parent_index"], tr["prev_actor"],
                                          offs[d + 1], offs[d + 2])
        dead = reach.copy()
        dead[n + 1] = 0.0
        return dict(reach=reach, beliefs=O.deep_beliefs(x["beliefs"], x["beliefs"], dead, x["prob"], tr["root_index"], n))
    if name == "unblocked_mass":
        return dict(out=OU.calculate_unblocked_mass(x["target"]))
    if name == "unblocked_opp_and_ratio":
        top = x["top"]
        opp = OU.calculate_unblocked_mass(x["beliefs"][np.arange(top), 1 - x["to_act"][:top]])
        ratio = OU.unblocked_mass_ratio(x["numer"], x["actor"], 1e-5, x["pidx"])
        return dict(opp_at_parents=opp, ratio_indirect=ratio, ratio=ratio)
    if name == "showdown_sorted":
        from oracle import showdown as OS
        m = len(x["boards"])
        ones = np.ones((m, 2), F32)
        return {f"ev_hero{p}": OS.showdown_value(x["beliefs"], p, x["hrd"], ones, ones[:, 0]) for p in (0, 1)}
    raise KeyError(name)


# ---- the reference's function names (its Triton module, or the product's drop-in) ----------------
def torch_ops(name: str, x: dict, F, device, raw=None) -> dict:
    """``raw``: optional dict name -> callable for the two reference wrappers that refuse CPU
    tensors before launching (block-and-normalise, unblocked mass); the writer of the fixture passes
    functions that repeat those wrappers' own launch lines."""
    import torch

    def T(a):
        return torch.from_numpy(np.array(a, order="C", copy=True)).to(device)     # never aliases the numpy input

    def S(v):
        return torch.tensor(v, dtype=torch.float32, device=device)
    raw = raw or {}
    if name.startswith("dcfr_update"):
        c, w, r = T(x["cum"]), T(x["wsum"]), T(x["regrets"])
        pos = torch.empty_like(c)
        t = x["t"]
        an, bn = float(t ** x["alpha"]), float(t ** x["beta"])
        if not x["apply_dcfr"]:
            an = bn = 1.0
        ad, bd = (an + 1.0, bn + 1.0) if x["apply_dcfr"] else (1.0, 1.0)
        F.fused_dcfr_update_with_tensors_(c, w, r, S(an), S(bn), S(ad), S(bd), x["apply_dcfr"], x["cfr_plus"],
                                          positive_regrets_out=pos)
        return dict(cum=c, wsum=w, positive=pos)
    if name.startswith("block_normalize"):
        t = T(x["target"])
        raw.get("block_normalize", F.fused_block_and_normalize_beliefs_)(t, T(x["allowed"]), T(x["prob"]))
        return dict(target=t)
    if name == "regret_matching_divide":
        out = torch.empty(x["pos"].shape, dtype=torch.float32, device=device)
        F.fused_regret_matching_divide_(T(x["pos"]), T(x["den"]), T(x["uni"]), out)
        return dict(out=out)
    if name == "weight_child_values":
        out = torch.empty(x["values"].shape, dtype=torch.float32, device=device)
        F.fused_weight_child_values(T(x["values"]), T(x["prev_actor"]), T(x["hero"]), T(x["opp"]), out)
        return dict(out=out)
    if name == "update_average_values":
        a = T(x["avg"])
        F.fused_update_average_values_with_tensors_(a, T(x["latest"]), S(x["old"]), S(x["new"]),
                                                    S(1.0 / (x["old"] + x["new"])))
        b = T(x["avg"])
        F.fused_update_average_values_(b, T(x["latest"]), x["old"], x["new"])
        return dict(avg=a, avg_floats=b)
    if name.startswith("avg_values_zero_sum"):
        a = T(x["avg"])
        F.fused_avg_values_zero_sum_(a, T(x["latest"]), T(x["beliefs"]), S(x["old"]), S(x["new"]),
                                     S(1.0 / (x["old"] + x["new"])), x["enforce"],
                                     ignore_mask=T(x["ignore"]) if x["ignore"] is not None else None)
        return dict(avg=a)
    tr = x.get("tree")
    if name == "regret_tail":
        reg = torch.zeros(tr["total"], H, dtype=torch.float32, device=device)
        F.fused_regret_tail_(reg, T(x["achieved"]), T(x["actor_values"]), T(x["src_w"]), T(tr["parent_index"]),
                             T(tr["prev_actor"]), tr["bottom"])
        return dict(regrets=reg)
    if name == "average_policy_mix":
        a = T(x["policy_avg"])
        F.fused_average_policy_mix_(a, T(x["policy"]), T(x["reach"]), T(x["reach_avg"]), T(tr["to_act"]),
                                    T(tr["parent_index"]), x["old"], x["new"], tr["bottom"])
        b = T(x["policy_avg"])
        F.fused_average_policy_mix_with_tensors_(b, T(x["policy"]), T(x["reach"]), T(x["reach_avg"]), T(tr["to_act"]),
                                                 T(tr["parent_index"]), S(x["old"]), S(x["new"]),
                                                 S(x["old"] + x["new"]), tr["bottom"])
        return dict(policy_avg=a, policy_avg_tensors=b)
    if name == "parent_sibling_divide":
        top, bottom = tr["top"], tr["bottom"]
        nchild = tr["total"] - bottom
        co, cc = T(tr["child_offsets"][:top].copy()), T(tr["child_count"][:top].copy())
        v = T(x["values"])
        ps = F.fused_parent_sum(v, co, cc)
        ss = F.fused_sibling_sum(v, co, cc, bottom, nchild)
        psum = ps.abs().clone()
        psum[:, ::4] = 0.0
        out = torch.empty(nchild, H, dtype=torch.float32, device=device)
        F.fused_divide_by_parent_sum_(T(x["pos"]), T(x["fallback"]), psum.contiguous(),
                                      T(tr["parent_index"][bottom:].copy()), out)
        return dict(parent_sum=ps, sibling_sum=ss, divided=out)
    if name == "model_values_mix":
        h, last, bel = T(x["h"]), T(x["last"]), T(x["beliefs"])
        old, new = x["old"], x["new"]
        outs = {"mix": F.fused_model_values_mix(h, last, old, new), "mix_tensors": torch.empty_like(h)}
        F.fused_model_values_mix_with_tensors(h, last, S((old + new) / new), S(old / new), outs["mix_tensors"])
        for key, enforce in (("mix_zs", True), ("mix_nozs", False)):
            o = torch.empty_like(h)
            F.fused_model_values_mix_zero_sum(h, last, bel, S((old + new) / new), S(old / new), o, enforce)
            outs[key] = o
        return outs
    if name == "weighted_parent_sum":
        v, offs = T(x["values"]), tr["depth_offsets"]
        pa, hero, opp = T(tr["prev_actor"]), T(x["hero"]), T(x["opp"])
        for d in range(len(offs) - 3, -1, -1):
            base, end = offs[d], offs[d + 1]
            F.fused_weighted_parent_sum(v, pa, hero, opp, T(tr["child_offsets"][base:end].copy()),
                                        T(tr["child_count"][base:end].copy()), base)
        return dict(values=v)
    if name == "reach_and_deep_beliefs":
        reach, offs, n = T(x["reach"]), tr["depth_offsets"], tr["bottom"]
        pol, allowed, pidx, pa = T(x["policy"]), T(x["allowed"]), T(tr["parent_index"]), T(tr["prev_actor"])
        for d in range(len(offs) - 2):
            F.fused_reach_weights_depth_(reach, pol, allowed, pidx, pa, offs[d + 1], offs[d + 2])
        dead = reach.clone()
        dead[n + 1] = 0.0
        b = T(x["beliefs"])
        F.fused_deep_beliefs_(b, b, dead, T(x["prob"]), T(tr["root_index"]), num_roots=n)
        return dict(reach=reach, beliefs=b)
    if name == "unblocked_mass":
        return dict(out=raw.get("unblocked_mass", F.unblocked_mass_triton)(T(x["target"])))
    if name == "unblocked_opp_and_ratio":
        opp = F.unblocked_mass_opp_at_parents_triton(T(x["beliefs"]), T(x["to_act"]), x["top"])
        numer, actor, pidx = T(x["numer"]), T(x["actor"]), T(x["pidx"])
        return dict(opp_at_parents=opp, ratio_indirect=F.unblocked_mass_ratio_indirect_triton(numer, actor, pidx),
                    ratio=F.unblocked_mass_ratio_triton(numer, actor[pidx].contiguous()))
    if name == "showdown_sorted":
        # EV per hand in combo order with potential = scale = 1: the reference's kernel works on the
        # strength-sorted villain range and leaves un-sorting and the board mask to its caller
        hrd, out = x["hrd"], {}
        order, inv = T(hrd.sorted_indices), T(hrd.inv_sorted)
        c1, c2 = T(hrd.hands_c1c2_sorted[..., 0].copy()), T(hrd.hands_c1c2_sorted[..., 1].copy())
        ok = T(x["allowed"]).float()
        for p in (0, 1):
            b_sorted = torch.gather(T(x["beliefs"][:, 1 - p]), 1, order).contiguous()
            ev_sorted = F.showdown_ev_triton(b_sorted, c1, c2, T(hrd.L_idx), T(hrd.R_idx))
            out[f"ev_hero{p}"] = torch.gather(ev_sorted, 1, inv) * ok
        return out
    raise KeyError(name)
