"""Per-operator timings on the workloads of the reference's three micro-benchmarks
(benchmarks/bench_fused_cfr_triton.py:53-351, bench_rules_triton.py:25-126,
bench_calculate_unblocked_mass.py:24-60), through this package's drop-in functions.

    python -m poker2_amd.bench_ops [--repeats 100] [--json]

Each line: mean time per call (HIP events around `repeats` calls after 10 warm-ups), the
algorithmic bytes of the call (every input read once, every output written once) and the
resulting GB/s.  Inputs are seeded and resident in HBM before timing.
"""
from __future__ import annotations

import argparse
import json

import numpy as np
import torch

from . import fused_cfr_hip as F
from . import rules_hip as R
from .card_utils import hand_combos_tensor

H = 1326


def timed(fn, repeats: int, warmup: int = 10) -> float:
    for _ in range(warmup):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(repeats):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / repeats * 1e-3


def random_hands(n: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return np.argsort(rng.random((n, 52)), axis=1)[:, :7]


def cases(repeats: int):
    dev = torch.device("cuda")
    g = torch.Generator(device="cpu").manual_seed(42)

    # --- DCFR discount + accumulate, [10 000, 1326] (bench_fused_cfr_triton.py:53-121)
    for rows in (10_000, 86_016):
        cum = torch.randn(rows, H, generator=g).to(dev)
        wsum = (torch.rand(rows, H, generator=g) * 5).to(dev)
        reg = (torch.randn(rows, H, generator=g) * 0.1).to(dev)
        yield (f"dcfr_update rows={rows}", 5 * rows * H * 4,
               lambda cum=cum, wsum=wsum, reg=reg: F.fused_dcfr_update_(cum, wsum, reg, 7, F.CFRType.discounted, 1.5, 0.0, False))

    # --- sibling sum / parent sum + divide, 30 000 parents x ~5 children (:193-326)
    parents = 30_000
    rng = np.random.default_rng(42)
    child_count = torch.from_numpy(np.clip(5 + rng.integers(-1, 2, parents), 1, None)).to(dev)
    n_children = int(child_count.sum())
    child_offsets = (torch.cumsum(child_count, 0) - child_count + parents).contiguous()
    parent_index = torch.arange(parents, device=dev).repeat_interleave(child_count)
    values = torch.zeros(parents + n_children, H, device=dev)
    values[parents:] = torch.rand(n_children, H, device=dev)
    yield ("sibling_sum parents=30000", 2 * n_children * H * 4,
           lambda: F.fused_sibling_sum(values, child_offsets, child_count, parents, n_children))
    pos = torch.rand(n_children, H, device=dev)
    fallback = torch.rand(n_children, H, device=dev)
    out = torch.empty_like(pos)
    full_pos = torch.zeros(parents + n_children, H, device=dev)
    full_pos[parents:] = pos

    def parent_sum_then_divide():
        ps = F.fused_parent_sum(full_pos, child_offsets, child_count)
        F.fused_divide_by_parent_sum_(pos, fallback, ps, parent_index, out)
    yield ("parent_sum + divide parents=30000", (4 * n_children + 2 * parents) * H * 4, parent_sum_then_divide)

    # --- unblocked mass (bench_calculate_unblocked_mass.py:24-42, bench_fused_cfr_triton.py:329-351)
    for rows in (10_000, 400_000):
        t = torch.rand(rows, H, generator=g)
        t = (t / t.sum(-1, keepdim=True)).to(dev)
        yield (f"unblocked_mass rows={rows}", 2 * rows * H * 4, lambda t=t: F.unblocked_mass_triton(t))
        del t

    # --- 7-card ranker (bench_rules_triton.py:25-126)
    for n in (1024, 8192, 65536, 1 << 20):
        a, b = random_hands(n, 7 + n), random_hands(n, 8 + n)
        cards = torch.from_numpy(np.stack([a, b], 1).astype(np.int16)).to(dev)
        planes = torch.zeros(n, 2, 4, 13, dtype=torch.bool, device=dev)
        idx = torch.arange(n, device=dev)[:, None]
        for p in range(2):
            c = cards[:, p].long()
            planes[idx, p, c // 13, c % 13] = True
        yield (f"compare_7 planes n={n}", n * (104 + 4), lambda planes=planes: R.compare_7_single_batch_triton(planes))
        yield (f"compare_7 cards(int16) n={n}", n * (28 + 4),
               lambda cards=cards: R.compare_7_cards_single_batch_triton(cards))
        one = cards[:, 0].to(torch.int8).contiguous()
        yield (f"rank_7 cards(int8) n={n}", n * (7 + 4), lambda one=one: R.rank_7_cards_single_batch_triton(one))

    # --- river showdown, 4096 public states
    m = 4096
    boards = torch.from_numpy(np.argsort(rng.random((m, 52)), axis=1)[:, :5].astype(np.int64)).to(dev)
    combos = hand_combos_tensor(dev)
    on_board = torch.zeros(m, 52, dtype=torch.bool, device=dev)
    on_board.scatter_(1, boards, True)
    allowed = ~(on_board[:, combos[:, 0]] | on_board[:, combos[:, 1]])
    bel = torch.from_numpy(rng.gamma(0.5, size=(m, 2, H)).astype(np.float32)).to(dev) * allowed[:, None, :]
    bel = bel / bel.sum(-1, keepdim=True)
    yield ("rank_hands (tables) boards=4096", m * (5 * 8 + R.showdown_table_bytes()),
           lambda: R.build_showdown_tables(boards))
    tables = R.build_showdown_tables(boards)
    pot = torch.ones(m, 2, device=dev)
    sc = torch.ones(m, device=dev)
    res = torch.empty_like(bel)
    yield ("showdown_value_both states=4096", 4 * m * H * 4,
           lambda: R.showdown_value_both(bel, tables, pot, sc, out=res))
    del tables, res

    # --- single-card chance node: 3584 turn leaves (512 roots x 7) x 48 river cards
    from . import chance_node_helper as CH
    k = 3584
    tb = torch.full((k, 5), -1, dtype=torch.int64, device=dev)
    tb[:, :4] = boards[:k, :4]
    roots = torch.arange(k, device=dev)
    pre = bel[:k].contiguous()
    post, _, _, offsets = CH.chance_expand(pre, roots, tb, cards_on_board=4)
    yield ("chance_expand states=3584 x48", k * (2 + 2 * 48) * H * 4,
           lambda: CH.chance_expand(pre, roots, tb, cards_on_board=4, check_rows=False))
    # the same expansion written as rows of a value network's input matrix: [ranges | board one-hot], 2704 elements
    for name, dt, size in (("float32", torch.float32, 4), ("bfloat16", torch.bfloat16, 2)):
        yield (f"chance_expand -> input rows {name}", k * (2 * H * 4 + 48 * 2704 * size),
               lambda dt=dt: CH.chance_expand(pre, roots, tb, cards_on_board=4, check_rows=False, input_dtype=dt))
    yield ("chance_mean states=3584 x48", k * (2 * 48 + 2) * H * 4, lambda: CH.chance_mean(post, offsets))
    del post

    # --- flop chance node: 64 preflop states x 256 drawn canonical flops, 6 of 24 suit permutations
    from .card_utils import combo_suit_permutation_tensor
    ks, kf = 64, 256
    canonical = CH.canonical_flops()[0]
    flops = torch.from_numpy(canonical[rng.integers(0, canonical.shape[0], kf)]).to(dev)
    pre_f = bel[:ks].contiguous()
    roots_f = torch.arange(ks, device=dev)
    yield (f"flop_expand states={ks} x{kf}", ks * (2 + 2 * kf) * H * 4, lambda: CH.flop_expand(pre_f, roots_f, flops, check_rows=False))
    hv = CH.flop_expand(pre_f, roots_f, flops)
    perms = combo_suit_permutation_tensor(dev)[:6].to(torch.int16).contiguous()
    w = torch.full((kf,), 1.0 / kf, device=dev)
    yield (f"perm_mean states={ks} x{kf} perms=6", ks * (2 * kf + 2) * H * 4, lambda: CH.perm_mean(hv, perms, w, check_perms=False))
    yield (f"orbit_mean states={ks} x{kf} (all 24)", ks * (2 * kf + 2) * H * 4, lambda: CH.orbit_mean(hv, w))
    del hv
    # the same at 1024 states (2.9 GB of network answers)
    ks = 1024
    pre_f = (torch.rand(ks, 2, H, device=dev) + 1e-3)
    pre_f = pre_f / pre_f.sum(-1, keepdim=True)
    roots_f = torch.arange(ks, device=dev)
    yield (f"flop_expand states={ks} x{kf}", ks * (2 + 2 * kf) * H * 4, lambda: CH.flop_expand(pre_f, roots_f, flops, check_rows=False))
    hv = CH.flop_expand(pre_f, roots_f, flops)
    yield (f"perm_mean states={ks} x{kf} perms=6", ks * (2 * kf + 2) * H * 4, lambda: CH.perm_mean(hv, perms, w, check_perms=False))
    yield (f"orbit_mean states={ks} x{kf} (all 24)", ks * (2 * kf + 2) * H * 4, lambda: CH.orbit_mean(hv, w))
    del hv, pre_f

    # --- data generation: policy targets and features of a 4096-root river search (21 nodes per root)
    from .config import river_dcfr_config
    from .evaluator import HipSparseCFREvaluator
    from .tree import RootStates
    n = 4096
    roots_r = RootStates.at_round_start(3, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards.cpu().numpy())
    ev = HipSparseCFREvaluator(None, dev, river_dcfr_config(n, iterations=1, depth=2))
    ev.initialize_subgame(roots_r, np.arange(n), bel)
    ev.policy_probs_avg.uniform_()
    top = ev.depth_offsets[-2]
    rows = torch.nonzero(~ev.leaf_mask[:top]).squeeze(1)
    n_children = int(ev.child_count[rows].sum())
    yield (f"policy_targets nodes={rows.numel()}", (n_children + rows.numel() * ev.num_actions) * H * 4,
           lambda: ev._policy_targets(rows, check_rows=False))
    yield (f"encode nodes={ev.total_nodes}", ev.total_nodes * (13 * 8 + 16 + 5 * 8 + 10 * 8),
           lambda: ev.feature_encoder.encode(ev.beliefs, pre_chance_node=ev.new_street_mask))

    # --- the remaining per-operation kernels, on the tensors of the same search: T = 86 016 nodes in three
    # levels (4096 roots, 16 384 children of the roots, 65 536 leaves); rows counted: read once, written once,
    # a parent's rows once per parent
    T, N = ev.total_nodes, n
    top = int(ev.depth_offsets[-2])                          # rows that can have children
    C = T - N
    l1, l2 = int(ev.depth_offsets[1]), int(ev.depth_offsets[2])
    n_l1, n_l2 = l2 - l1, T - l2
    row = H * 4
    bel3 = torch.rand(T, 2, H, device=dev)
    yield (f"block_and_normalize rows={T}x2", 4 * T * row + T * H,
           lambda: F.fused_block_and_normalize_beliefs_(bel3, ev.allowed_hands, ev.allowed_hands_prob))
    posr = torch.rand(C, H, device=dev)
    den = torch.rand(C, H, device=dev)
    uni = torch.full((C, H), 0.25, device=dev)
    outc = torch.empty(C, H, device=dev)
    yield (f"regret_matching_divide children={C}", 4 * C * row,
           lambda: F.fused_regret_matching_divide_(posr, den, uni, outc))
    vals3 = torch.rand(T, 2, H, device=dev)
    vsrc = vals3[N:].contiguous()
    outv = torch.empty_like(vsrc)
    prev_c = ev.prev_actor[N:].contiguous()
    yield (f"weight_child_values children={C}", 6 * C * row,
           lambda: F.fused_weight_child_values(vsrc, prev_c, posr, den, outv))
    del vsrc, outv
    vavg = torch.rand(T, 2, H, device=dev)
    yield (f"update_average_values rows={T}x2", 6 * T * row,
           lambda: F.fused_update_average_values_(vavg, vals3, 3.0, 1.0))
    o_t, n_t, inv_t = (torch.tensor(x, device=dev) for x in (3.0, 1.0, 0.25))
    yield (f"avg_values_zero_sum rows={T}x2", 8 * T * row,
           lambda: F.fused_avg_values_zero_sum_(vavg, vals3, bel3, o_t, n_t, inv_t, True))
    regrets = torch.zeros(T, H, device=dev)
    actor_v = torch.rand(top, H, device=dev)
    src_w = torch.rand(top, H, device=dev)
    yield (f"regret_tail children={C}", (2 * C + 2 * top) * row,
           lambda: F.fused_regret_tail_(regrets, vals3, actor_v, src_w, ev.parent_index, ev.prev_actor, N))
    pavg = torch.rand(T, H, device=dev)
    pol = torch.rand(T, H, device=dev)
    reach_avg3 = torch.rand(T, 2, H, device=dev)
    yield (f"average_policy_mix children={C}", (3 * C + 2 * top) * row,
           lambda: F.fused_average_policy_mix_(pavg, pol, bel3, reach_avg3, ev.env.to_act, ev.parent_index, 3.0, 1.0, N))
    co1, cc1 = ev.child_offsets[l1:l2].contiguous(), ev.child_count[l1:l2].contiguous()
    yield (f"weighted_parent_sum parents={n_l1}", (4 * n_l2 + 2 * n_l1) * row,
           lambda: F.fused_weighted_parent_sum(vals3, ev.prev_actor, pol, pavg, co1, cc1, l1))
    yield (f"reach_weights_depth children={n_l2}", (3 * n_l2 + 2 * n_l1) * row + n_l2 * H,
           lambda: F.fused_reach_weights_depth_(reach_avg3, pol, ev.allowed_hands, ev.parent_index, ev.prev_actor, l2, T))
    root_b = ev.beliefs[:N].contiguous()
    yield (f"deep_beliefs rows={C}x2", (4 * C + 2 * N) * row,
           lambda: F.fused_deep_beliefs_(bel3, root_b, reach_avg3, ev.allowed_hands_prob, ev._root_index, N))
    t_all = torch.zeros(T, dtype=torch.int64, device=dev)
    t0 = torch.zeros((), dtype=torch.int64, device=dev)
    yield (f"sample_snapshot rows={T}", 2 * T * row, lambda: F.fused_sample_snapshot_(pavg, pol, t_all, t0))
    yield (f"unblocked_mass_opp_at_parents parents={top}", 2 * top * row,
           lambda: F.unblocked_mass_opp_at_parents_triton(bel3, ev.env.to_act, top))
    par_c = ev.parent_index[N:].contiguous()
    yield (f"unblocked_mass_ratio_indirect children={C}", (2 * C + top) * row,
           lambda: F.unblocked_mass_ratio_indirect_triton(posr, actor_v, par_c))
    m_leaves = 20_000
    hv, last, outm = (torch.rand(m_leaves, 2, H, device=dev) for _ in range(3))
    bl = bel3[:m_leaves]
    onon, oon = torch.tensor(1.25, device=dev), torch.tensor(0.25, device=dev)
    yield (f"model_values_mix_zero_sum leaves={m_leaves}", 8 * m_leaves * row,
           lambda: F.fused_model_values_mix_zero_sum(hv, last, bl, onon, oon, outm, True))
    del bel3, posr, den, uni, outc, vals3, vavg, regrets, actor_v, src_w, pavg, pol, reach_avg3, hv, last, outm

    # --- local best response, one tree level of the same search: the 16 384 parents of level 1, four
    # children each.  Per parent: the actor's range in, both value rows out; per child both value rows in and,
    # where the parent's actor is not the deviating player, its policy row (a deviating actor takes the maximum
    # over its children and reads no policy).  A search asks for both players' best responses, so every parent
    # is in either case once: here every second parent deviates.
    from . import _lib
    base, end = int(ev.depth_offsets[1]), int(ev.depth_offsets[2])
    n_par, n_ch = end - base, int(ev.child_count[base:end].sum())
    deviator = ev.env.to_act.clone()
    deviator[base + 1:end:2] = 1 - deviator[base + 1:end:2]
    follows = deviator[base:end] != ev.env.to_act[base:end]
    n_policy_rows = int(ev.child_count[base:end][follows].sum())
    vals = torch.rand(ev.total_nodes, 2, H, device=dev)
    yield (f"best_response_level parents={n_par}", (3 * n_par + 2 * n_ch + n_policy_rows) * H * 4,
           lambda: _lib.call("p2hip_best_response_level", _lib.ptr(vals), _lib.ptr(ev.policy_probs_avg),
                             _lib.ptr(ev.beliefs), _lib.ptr(ev.env.to_act), _lib.ptr(deviator),
                             _lib.ptr(ev.child_offsets), _lib.ptr(ev.child_count), base, n_par,
                             int(ev._max_children), _lib.stream_ptr()))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--repeats", type=int, default=100)
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args()
    if not torch.cuda.is_available():
        raise SystemExit("bench_ops needs a GPU (the product path has no CPU fallback)")
    rows = []
    for name, nbytes, fn in cases(args.repeats):
        sec = timed(fn, args.repeats)
        rows.append({"op": name, "us": sec * 1e6, "algorithmic_bytes": nbytes, "GBps": nbytes / sec / 1e9})
        if not args.json:
            print(f"{name:40s} {sec * 1e6:10.1f} us  {nbytes / 1e6:10.1f} MB  {nbytes / sec / 1e9:8.1f} GB/s", flush=True)
    if args.json:
        print(json.dumps(rows))


if __name__ == "__main__":
    main()
