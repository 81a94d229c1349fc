"""Headline benchmark: fused DCFR iteration on river subgames, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--roots B] [--tree raise3|raise1|raise2|depth2] [--mode search|plain]

A step is ONE CFR iteration over a batch of B seeded synthetic river subgames (random
5-card boards, Dirichlet(0.5) ranges with board-blocked combos removed, pot 200, stacks
800/800 = stack/pot 4, bet bins {0.5, 1.0} + all-in, at most three raises: 105 nodes per root, every
leaf a fold or a showdown; discounted CFR alpha 1.5 / beta 0 / gamma 2).  All inputs are
resident in HBM before the timed region.  The steps run the way a search runs them
(``HipSparseCFREvaluator.run_search_iterations``: every iteration but a search's last leaves rows
unwritten that nothing reads before the next iteration rewrites them, and reach_avg alternates
between two buffers; the final state of a search is bit-identical either way); ``--mode plain`` times
the iteration that writes all eleven tensors in full, as ``cfr_iteration(t)`` does.  Both are in the line.
Prints ONE JSON line:
  value        subgame-iterations per second (iterations/s x subgames)
  roofline     canonical algorithmic bytes of an iteration (29 vectors per node) / the mean time of
               the iteration's launches (HIP events on the launch stream) against the 8 TB/s HBM
               peak; `traffic` = HBM bytes the launches really move (rocprofv3 counters), with the
               fraction of peak on those bytes beside it
  cpu_baseline the numpy oracle (a CPU restatement of the reference's torch path) timed on
               this box's host cores on a small sample of the same workload
  extra        showdown evaluations/s (B=4096 boards), 7-card hands ranked/s (2^20 hands), each with
               its CPU leg; the iteration at the reference's own batch of 192 roots; and the same
               iteration kernel on the other river workloads (three-raise tree, 1024 roots), so that
               the headline is not read as the only case
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

H = 1326
BYTES_PER_NODE_ITER = 29 * H * 4          # 17 vectors written + 12 read per node per iteration
HBM_PEAK_GBS = 8000.0
TREES = {"depth2": (2, None), "raise1": (16, 1), "raise2": (16, 2), "raise3": (16, 3), "depth5": (5, None)}
# HBM bytes per launch of the iteration kernel from two rocprofv3 --pmc passes (FETCH_SIZE, then
# WRITE_SIZE, each scaled by what the same counter reads for a plain 1 GiB copy).  NOT measured by this
# program: counters need the profiler, so these are constants taken from the summary file named
# below, one per workload that has a counter run; None elsewhere.  (read bytes, written bytes)
TRAFFIC_SOURCE = "profiles/cfr_iteration_kernel_river.hbm_counters.txt"
MEASURED_TRAFFIC_BYTES = {("raise3", 4096, "plain"): (34.30e9, 35.73e9), ("raise3", 4096, "search"): (32.76e9, 23.10e9),
                          ("depth2", 4096, "plain"): (5.87e9, 6.69e9), ("depth2", 4096, "search"): (5.68e9, 3.82e9),
                          ("raise1", 4096, "plain"): (6.60e9, 7.02e9), ("raise1", 4096, "search"): (6.35e9, 4.61e9),
                          ("raise3", 1024, "plain"): (8.58e9, 8.94e9), ("raise3", 1024, "search"): (8.20e9, 5.78e9)}
# how the iterations of a search run (all but its last) / how cfr_iteration(t) runs one
MODES = {"search": dict(lean=True, alternate_reach_avg=True), "plain": {}}


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def synth_roots(n: int, seed: int):
    from poker2_amd.card_utils import hand_combos_tensor
    rng = np.random.default_rng(seed)
    boards = np.argsort(rng.random((n, 52)), axis=1)[:, :5].astype(np.int64)
    combos = hand_combos_tensor().numpy()
    on_board = np.zeros((n, 52), dtype=bool)
    on_board[np.arange(n)[:, None], boards] = True
    allowed = ~(on_board[:, combos[:, 0]] | on_board[:, combos[:, 1]])
    x = rng.gamma(0.5, size=(n, 2, H)).astype(np.float32) * allowed[:, None, :]
    x /= x.sum(axis=-1, keepdims=True)
    return boards, x.astype(np.float32)


def make_evaluator(n_roots: int, tree: str, seed: int, iterations: int, spread_state: bool = False):
    import torch
    from poker2_amd.config import river_dcfr_config
    from poker2_amd.evaluator import HipSparseCFREvaluator
    from poker2_amd.tree import RootStates
    depth, max_raises = TREES[tree]
    boards, beliefs = synth_roots(n_roots, seed)
    roots = RootStates.at_round_start(3, np.full(n_roots, 200), np.tile([[800, 800]], (n_roots, 1)), boards,
                                      button=np.arange(n_roots) % 2)
    cfg = river_dcfr_config(n_roots, iterations=iterations, depth=depth, dcfr_delay=0)
    ev = HipSparseCFREvaluator(None, torch.device("cuda"), cfg, fused_iteration=True, max_raises=max_raises,
                               spread_state=spread_state)
    ev.initialize_subgame(roots, np.arange(n_roots), torch.from_numpy(beliefs))
    ev.prepare_search()
    return ev, boards, beliefs


def cpu_baseline(tree: str, seed: int, budget_s: float = 20.0) -> dict:
    """Time the oracle's iteration (numpy float32 port of the reference CPU path)."""
    from oracle import cfr as ocfr
    from poker2_amd.tree import RootStates, build_sparse_tree
    depth, max_raises = TREES[tree]
    n = 16
    boards, beliefs = synth_roots(n, seed)
    roots = RootStates.at_round_start(3, np.full(n, 200), np.tile([[800, 800]], (n, 1)), boards,
                                      button=np.arange(n) % 2)
    t = build_sparse_tree(roots, [0.5, 1.0], depth, max_raises=max_raises)
    d = {k: getattr(t, k) for k in ("depth_offsets", "parent_index", "action_from_parent", "child_count",
                                    "child_offsets", "prev_actor", "legal_mask", "leaf_mask", "new_street_mask",
                                    "fold_mask", "showdown_mask", "reward")}
    d.update({k: t.state[k] for k in ("to_act", "done", "scale")})
    d["showdown_potential"] = t.showdown_potential
    orc = ocfr.OracleCFR(d, boards, beliefs, cfr_iterations=200)
    orc.prepare()
    orc.cfr_iteration(0)  # two warm-up iterations
    orc.cfr_iteration(1)
    times = []
    t_it = 2
    start = time.perf_counter()
    while time.perf_counter() - start < budget_s and len(times) < 40:
        t0 = time.perf_counter()
        orc.cfr_iteration(t_it)
        times.append(time.perf_counter() - t0)
        t_it += 1
    med = float(np.median(times))
    try:
        from threadpoolctl import threadpool_info
        cores = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
    except Exception:
        cores = os.cpu_count() or 1
    return {"value": n / med, "unit": "subgame-iterations/s", "cores": int(cores), "cpu_model": cpu_model(),
            "kind": "port",
            "sample": f"{n} river subgames ({t.total // n} nodes each), median of {len(times)} iterations "
                      f"of the numpy oracle, {med * 1e3:.1f} ms per iteration"}


def flat_stream_rate(pairs: int = 1 << 26, reps: int = 5) -> dict:
    """GB/s of a structure-free element-wise stream with the iteration kernel's read / write mix (5 input
    and 7 output arrays of 512 MiB each, one 8-byte access per lane and array), with ordinary and with
    non-temporal accesses: what HBM gives such a kernel on THIS machine when nothing else limits it.
    Measurement aid of the library (p2hip_stream_probe); runs after the timed region, on its own buffers."""
    import torch
    from poker2_amd import _lib
    src = torch.zeros(5 * pairs * 2, dtype=torch.float32, device="cuda")
    dst = torch.empty(7 * pairs * 2, dtype=torch.float32, device="cuda")
    out = {}
    for name, nt in (("plain", 0), ("non_temporal", 1)):
        run = lambda: _lib.call("p2hip_stream_probe", src.data_ptr(), dst.data_ptr(), pairs, 5, 7, nt, _lib.stream_ptr())
        for _ in range(2):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            run()
        e1.record()
        torch.cuda.synchronize()
        out[name] = 12 * pairs * 8 / (e0.elapsed_time(e1) / reps * 1e-3) / 1e9
    del src, dst
    torch.cuda.empty_cache()
    return out


def side_metrics(skip=(), spread_state: bool = False) -> dict:
    """Showdown evaluations/s (B=4096 public states) and hands ranked/s (2^20 hands)."""
    import torch
    from poker2_amd import rules_hip
    out = {}
    boards, beliefs = synth_roots(4096, 42)
    tables = rules_hip.build_showdown_tables(torch.from_numpy(boards).cuda())
    b = torch.from_numpy(beliefs).cuda()
    pot = torch.ones(4096, 2, device="cuda")
    sc = torch.ones(4096, device="cuda")
    res = torch.empty_like(b)
    for _ in range(5):
        rules_hip.showdown_value_both(b, tables, pot, sc, out=res)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = 50
    ev0.record()
    for _ in range(reps):
        rules_hip.showdown_value_both(b, tables, pot, sc, out=res)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / reps
    out["showdown_states_per_s"] = 4096 / (ms * 1e-3)
    out["showdown_ms_per_call_B4096"] = ms
    out["showdown_algorithmic_GBps"] = 4096 * 4 * H * 4 / (ms * 1e-3) / 1e9
    # the per-board strength table is static input that every call re-reads; it is not algorithmic
    # traffic and is stated apart
    table = rules_hip.showdown_table_bytes()
    out["showdown_table_bytes_per_state"] = table
    out["showdown_GBps_with_tables"] = 4096 * (4 * H * 4 + table) / (ms * 1e-3) / 1e9
    rng = np.random.default_rng(7)
    cards = torch.from_numpy(np.argsort(rng.random((1 << 20, 52)), axis=1)[:, :7].astype(np.int8)).cuda()
    for _ in range(5):
        rules_hip.rank_7_cards_single_batch_triton(cards)
    ev0.record()
    for _ in range(reps):
        rules_hip.rank_7_cards_single_batch_triton(cards)
    ev1.record()
    torch.cuda.synchronize()
    ms = ev0.elapsed_time(ev1) / reps
    out["rank7_hands_per_s"] = (1 << 20) / (ms * 1e-3)
    out["rank7_ms_per_call_2e20"] = ms
    # the batch the reference's own settings search at a time (num_envs: 192), on the three-raise tree: few roots
    # are cut into work items that get a workgroup each
    small, _, _ = make_evaluator(192, "raise3", 42, iterations=64, spread_state=spread_state)
    out["state_placed_B192"] = bool(small.state_placement.get("placed"))
    for mode, kw in MODES.items():
        for t in range(1, 6):
            small.cfr_iteration(t, **kw)
        ev0.record()
        for t in range(6, 6 + reps):
            small.cfr_iteration(t, **kw)
        ev1.record()
        torch.cuda.synchronize()
        ms = ev0.elapsed_time(ev1) / reps
        tag = "" if mode == "search" else "_plain"
        out["iteration_ms_B192_three_raise_tree" + tag] = ms
        out["subgame_iterations_per_s_B192" + tag] = 192 / (ms * 1e-3)
        out["algorithmic_GBps_B192" + tag] = BYTES_PER_NODE_ITER * small.total_nodes / (ms * 1e-3) / 1e9
    del small
    # the same iteration kernel on the other river workloads (HIP events around 20 iterations each), as a search
    # runs them and in full
    others = []
    for roots, tree in ((4096, "depth2"), (4096, "raise1"), (1024, "depth2"), (1024, "raise3")):
        if (roots, tree) == tuple(skip):
            continue
        ev, _, _ = make_evaluator(roots, tree, 42, iterations=64, spread_state=spread_state)
        p = ev.state_placement
        row = {"roots": roots, "tree": tree, "nodes_per_root": ev.total_nodes // roots,
               "state_placed": bool(p.get("placed")),
               "probe_ns_per_row": ([p["probe_ns_per_row_inside_first_slab"]] + p["probe_ns_per_row_candidates"])
               if p.get("placed") else None}
        for mode, kw in MODES.items():
            for t in range(6):
                ev.cfr_iteration(t, **kw)
            torch.cuda.synchronize()
            ev0.record()
            for t in range(6, 26):
                ev.cfr_iteration(t, **kw)
            ev1.record()
            torch.cuda.synchronize()
            ms = ev0.elapsed_time(ev1) / 20
            gbs = BYTES_PER_NODE_ITER * ev.total_nodes / (ms * 1e-3) / 1e9
            row[mode] = {"iteration_ms": ms, "algorithmic_GBps": gbs, "frac": gbs / HBM_PEAK_GBS}
        others.append(row)
        del ev
        torch.cuda.empty_cache()
    out["iteration_other_workloads"] = others
    return out


def cpu_side_baselines(budget_s: float = 6.0) -> dict:
    """CPU legs of the two side metrics on this box's host cores: the C restatement of the reference's
    rules evaluator on 2^20 hands (one thread), and the numpy restatement of its showdown
    (cfr_evaluator.py:492-601, the [M,1327,52] prefix-sum formulation) on a sample of the 4096 states."""
    from oracle import ranker_c
    from oracle import showdown as osd
    from oracle import cards as ocards
    out = {"cpu_model": cpu_model()}
    rng = np.random.default_rng(7)
    cards = np.argsort(rng.random((1 << 20, 52)), axis=1)[:, :7].astype(np.int8)
    ranker_c.rank_cards(cards[:1024])
    t0 = time.perf_counter()
    ranker_c.rank_cards(cards)
    dt = time.perf_counter() - t0
    out["rank7_hands_per_s"] = (1 << 20) / dt
    out["rank7_sample"] = f"2^20 hands, oracle/ranker.c, 1 thread, {dt * 1e3:.0f} ms"
    m = 32
    boards, beliefs = synth_roots(m, 42)
    allowed, _ = ocards.allowed_hands_for_boards(boards)
    hrd = osd.init_hand_rank_data(boards, allowed)
    pot, scale = np.ones((m, 2), np.float32), np.ones(m, np.float32)
    osd.showdown_value_both(beliefs, hrd, pot, scale)
    times = []
    start = time.perf_counter()
    while time.perf_counter() - start < budget_s and len(times) < 9:
        t0 = time.perf_counter()
        osd.showdown_value_both(beliefs, hrd, pot, scale)
        times.append(time.perf_counter() - t0)
    med = float(np.median(times))
    out["showdown_states_per_s"] = m / med
    out["showdown_sample"] = f"{m} of the 4096 states (tables prepared beforehand, as on the GPU), numpy oracle, " \
                             f"median of {len(times)} calls, {med * 1e3:.0f} ms per call"
    return out


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=60)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--roots", type=int, default=4096)
    ap.add_argument("--tree", choices=sorted(TREES), default="raise3")
    ap.add_argument("--mode", choices=sorted(MODES), default="search",
                    help="search: the iterations as a search runs all but its last; plain: every tensor written in full")
    ap.add_argument("--seed", type=int, default=42)
    ap.add_argument("--no-spread", action="store_true",
                    help="allocate the state tensors as they come (the evaluator's default) instead of dealing them to two "
                         "slabs in different thirds of the card's memory (its spread_state option, made for long searches)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy three times (reference point for "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: every box of this build has one GPU and the path shards by root "
              "without communication; run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists for the product path).", file=sys.stderr)
        sys.exit(1)
    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    torch.zeros(1, device="cuda")
    torch.cuda.synchronize()
    t_build = time.perf_counter()
    ev, _, _ = make_evaluator(args.roots, args.tree, args.seed, iterations=args.warmup + args.steps + 1,
                              spread_state=not args.no_spread)
    torch.cuda.synchronize()
    t_build = time.perf_counter() - t_build
    placed = dict(ev.state_placement)
    if placed.get("placed"):
        # the probe streams 20 rows of 5304 B per node: its rate with all arrays in one third of the card's
        # memory, and dealt to the two slabs the state lies in
        per_row = 20 * H * 4
        placed["probe_GBps_inside_first_slab"] = per_row / placed["probe_ns_per_row_inside_first_slab"]
        placed["probe_GBps_chosen_slabs"] = per_row / placed["probe_ns_per_row_candidates"][placed["chosen"]]
    nodes_per_root = ev.total_nodes // ev.root_nodes
    launches = 1 if ev._items is None else 2 * len(ev._items.tiers)

    def timed(mode: str, steps: int, warmup: int, t: int):
        """Mean time of an iteration's launches (HIP events on the launch stream) and the wall clock per step."""
        kw = MODES[mode]
        for _ in range(warmup):
            ev.cfr_iteration(t, **kw)
            t += 1
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
        ev._skip_t_scalars_update = True
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for k in range(steps):
            ev.prepare_replay(t)          # tiny scalar-upload kernel, outside the kernel timing
            starts[k].record()
            ev.cfr_iteration(t, **kw)     # the iteration's launches: one per root-sized tree, six over work items in three tiers
            ends[k].record()
            t += 1
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ev._skip_t_scalars_update = False
        return float(np.mean([s.elapsed_time(e) for s, e in zip(starts, ends)])), wall * 1e3 / steps, t

    kernel_ms, ms_per_step, t_next = timed(args.mode, args.steps, args.warmup, 0)
    other_mode = "plain" if args.mode == "search" else "search"
    other_kernel_ms, other_ms_per_step, _ = timed(other_mode, min(args.steps, 20), 3, t_next)
    value = args.roots / (ms_per_step * 1e-3)
    algo_bytes = BYTES_PER_NODE_ITER * ev.total_nodes
    achieved = algo_bytes / (kernel_ms * 1e-3) / 1e9
    assert torch.isfinite(ev.values_avg).all()
    rw = MEASURED_TRAFFIC_BYTES.get((args.tree, args.roots, args.mode))
    rw_other = MEASURED_TRAFFIC_BYTES.get((args.tree, args.roots, other_mode))
    traffic = float(sum(rw)) if rw else None
    total_nodes = ev.total_nodes
    del ev
    torch.cuda.empty_cache()

    flat = flat_stream_rate()
    moved = traffic if traffic else algo_bytes
    mode_text = {"search": "iterations as a search runs all but its last (rows nothing reads before the next iteration "
                           "rewrites them are not stored; reach_avg alternates between two buffers)",
                 "plain": "every iteration writes all eleven tensors in full, as cfr_iteration(t) does"}
    result = {
        "metric": "river CFR iters/sec x subgames",
        "value": value,
        "unit": "subgame-iterations/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"fused DCFR iteration, river subgames, B={args.roots}, tree={args.tree} "
                               f"({nodes_per_root} nodes/root, bins 0.5/1.0 + all-in, pot 200, stacks 800)",
                   "roots": args.roots, "nodes_per_root": nodes_per_root, "total_nodes": total_nodes,
                   "cfr": "discounted alpha=1.5 beta=0 gamma=2, cfr_plus=False, delay=0",
                   "mode": args.mode, "mode_note": mode_text[args.mode],
                   "launches_per_iteration": launches,
                   "state_placement": {"spread_state": not args.no_spread, **placed,
                                       "subgame_construction_s": t_build,
                                       "note": "evaluator option for long searches: the state tensors are dealt to two slabs "
                                               "in different thirds of the card's memory, the second chosen by a measured "
                                               "probe; outside the timed region"}},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS,
                     "traffic": traffic,
                     "traffic_note": "offline constant from " + TRAFFIC_SOURCE + " (rocprofv3 --pmc FETCH_SIZE / "
                                     "WRITE_SIZE runs of this command), not measured by this run" if traffic else
                                     "no counter run exists for this workload",
                     "traffic_read_write": list(rw) if rw else None,
                     "frac_of_peak_on_measured_traffic": (traffic / (kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if traffic else None,
                     "kernel": "cfr_iteration_kernel", "kernel_ms": kernel_ms,
                     "algorithmic_bytes_per_launch": algo_bytes,
                     "algorithmic_bytes_note": "29 vectors of 1326 floats per node and iteration (17 written, 12 read), "
                                               "the canonical count of one iteration whatever the mode",
                     "other_mode": {"mode": other_mode, "mode_note": mode_text[other_mode], "kernel_ms": other_kernel_ms,
                                    "ms_per_step": other_ms_per_step,
                                    "value": args.roots / (other_ms_per_step * 1e-3),
                                    "frac": algo_bytes / (other_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                    "traffic": float(sum(rw_other)) if rw_other else None,
                                    "frac_of_peak_on_measured_traffic":
                                        (sum(rw_other) / (other_kernel_ms * 1e-3) / 1e9 / HBM_PEAK_GBS) if rw_other else None},
                     "flat_stream_same_mix_GBps": flat,
                     "flat_stream_note": "p2hip_stream_probe: 5 arrays read + 7 written, 512 MiB each, ordinary and "
                                         "non-temporal accesses, measured by this run after the timed region; the "
                                         "kernel's bytes (counted traffic where a counter run exists, else "
                                         "algorithmic) over its time, as a share of the faster of the two; the probe's "
                                         "arrays lie back to back, i.e. in one third of the card's memory, so this is "
                                         "no ceiling for a state placed across two thirds (config.state_placement)",
                     "frac_of_flat_stream": moved / (kernel_ms * 1e-3) / 1e9 / max(flat.values())},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(args.tree, args.seed)
    if not args.no_extra:
        result["extra"] = side_metrics(skip=(args.roots, args.tree), spread_state=not args.no_spread)
        if not args.no_cpu_baseline:
            result["extra"]["cpu"] = cpu_side_baselines()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
