"""``HipSparseCFREvaluator`` -- the search evaluator of the reference with every
per-iteration step on hand-written HIP kernels.

Mirrors the method set that ``FusedSparseCFREvaluator`` overrides
(src/p2/search/fused_sparse_cfr_evaluator.py:144-550) on top of the state layout of
``SparseCFREvaluator`` (src/p2/search/sparse_cfr_evaluator.py:142-306) and the iteration
logic of ``CFREvaluator`` (src/p2/search/cfr_evaluator.py:285-303, :770-886, :1294-1381,
:1497-1528).  State tensors keep the reference's names, shapes and dtypes.

Two execution modes share the same state:
  * ``fused_iteration=True`` (default): ``cfr_iteration`` is ONE kernel launch
    (``p2hip_cfr_iteration``), or two around the leaf network when the tree has
    non-terminal leaves and a leaf model is attached;
  * ``fused_iteration=False``: one launch per operation through the functions of
    ``fused_cfr_hip`` -- the call sequence of the reference's fused evaluator.

Leaf model protocol (the value network itself stays ordinary PyTorch): ``model`` is
``None`` (zero leaf values and a uniform initial policy, i.e. the reference tests' zero
``MockModel``) or an object with
    enforce_zero_sum: bool
    leaf_values(beliefs[K,2,1326], node_rows[K], evaluator) -> [K,2,1326]
    policy_logits(beliefs[T,2,1326], node_rows[K], evaluator) -> [K,1326,A]   (optional)

Also here, either side of the iterations: warm start (``warm_start``), leaf sampling
(``sample_leaves``), training-data assembly (``training_data``) and the local best response /
exploitability statistics (``_compute_exploitability``).
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from types import SimpleNamespace

import numpy as np
import torch

from . import _lib
from . import fused_cfr_hip as F
from . import rules_hip
from .card_utils import NUM_HANDS, combo_to_onehot_tensor
from .fused_cfr_hip import CFRType
from .chance_node_helper import ChanceNodeHelper
from .rebel_batch import RebelBatch
from .rebel_feature_encoder import RebelFeatureEncoder
from .tree import (CARDS_ON_STREET, RootStates, SparseTree, build_sparse_tree, build_sparse_tree_device,
                   launch_order, split_work_items)
from ._guards import require as _req

STATE_NAMES = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets",
               "regret_weight_sums", "self_reach", "self_reach_avg", "beliefs", "beliefs_avg",
               "latest_values", "values_avg")

_NODE_SHOWDOWN, _NODE_DONE, _NODE_PARENT, _NODE_LEAF_EVAL = 1, 2, 4, 8


class _IterArgs(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in (
        "child_offsets", "child_count", "to_act", "node_flags", "root_parent_offsets", "root_parents",
        "root_showdown_offsets", "root_showdown_nodes", "t_sample",
        "allowed", "allowed_prob", "tables", "potential", "scale", "policy", "policy_avg", "policy_sample", "cum",
        "wsum", "beliefs", "beliefs_avg", "reach", "reach_avg", "latest", "values_avg", "scratch", "fscal", "iscal",
        "item_root", "item_top", "reach_avg_prev")]


# Sweeps a launch of the iteration kernel runs (include/p2hip.h): 1 = regrets + reach/beliefs, 2 = values,
# 4 = regrets alone, 8 = reach/beliefs alone.
_PHASE_12, _PHASE_3, _PHASE_1, _PHASE_2 = 1, 2, 4, 8
# Lean launch (include/p2hip.h): the reach / belief part stores only the rows that the rest of the
# iteration or the next iteration reads.  ``evaluate_cfr`` runs every iteration but its last that way.
_PHASE_LEAN = 16
# One workgroup per root fills the chip (256 CUs x 3 resident workgroups) from 768 roots on.  Below
# SPLIT_ROOTS_BELOW roots each root's tree is cut at level SPLIT_CUT_LEVEL into work items (the top of
# the tree, and one subtree per node of that level) that get a workgroup each.  Measured on the
# three-raise river tree (105 nodes per root), ms per iteration unsplit -> split: 96 roots 1.28 -> 0.71,
# 192 roots 1.40 -> 1.01, 384 roots 1.82 -> 1.66, 767 roots 2.90 -> 2.63 (and slower than unsplit on
# another tree); depth-2 tree (21 nodes per root): 96 roots 0.21 -> 0.13, 384 roots 0.36 -> 0.34, 500 roots
# 0.38 -> 0.42; a cut right under the root leaves subtrees whose chain of families is as long as
# half the tree, deeper cuts put more of the tree into the few top items.
SPLIT_ROOTS_BELOW = 400
# Placement of the state tensors (``HipSparseCFREvaluator._place_state``): slabs below the minimum are allocated
# as they come; a second slab that the probe finds in the same third of the card's memory as the first is held,
# together with blocks that add up to the step size, while the next candidate is allocated, at most so many
# times (the thirds are ~96 GiB: three steps cross one); a candidate counts as lying elsewhere when the probe
# runs in under 0.9 of the time it takes with all of its arrays packed into the start of the first slab
# (measured: 0.80-0.85 against 1.0).
STATE_SPREAD_MIN_SLAB_BYTES = 256 << 20
STATE_SPREAD_STEP_BYTES = 31 << 30         # held as blocks of 16, 8, 4, 2 and 1 GiB: the driver hands out the highest free
                                           # block of a request's size class, so every class has to be taken out of the way
STATE_SPREAD_TRIES = 6
STATE_SPREAD_ACCEPT = 0.9
_PROBE_PACKED_BYTES = 10 * 12288 * 1326 * 4     # ten of the probe's arrays at their largest, back to back
_PROBE_MIN_BYTES = 10 * (256 * 1326 * 4 + 256)  # per buffer: the probe refuses arrays of fewer than 256 rows
SPLIT_CUT_LEVEL = 2
# The tree tops (one workgroup per root, five families in a row) are few and long: a second cut right under
# the root makes the root's family one item and each of its children's families another (six launches per
# iteration instead of four).  First made for few roots (192 roots: 0.80 -> 0.77 ms), it pays at every batch
# size: 4096 three-raise roots 10.84 -> 10.41 ms per search iteration, 13.79 -> 12.75 ms per plain one; 2048
# roots 5.52 -> 5.28 ms; 1024 roots unchanged (2.86 ms); 512 roots 1.46 -> 1.40 ms.
SPLIT_MID_LEVEL = 1
# Trees with raises (57 and 105 nodes per root against 21) gain from the cut at every batch size: their
# subtrees differ in size, so whole roots leave long tails (three raises: 1024 roots 3.96 -> 3.73 ms,
# 4096 roots 14.75 -> 14.41 ms with all items started largest first, -> 12.8 ms with the items in row order
# and only the last rounds' items by size; two raises: 1024 roots 2.15 -> 2.07 ms, 4096 roots 7.93 -> 7.76 ms;
# the 21-node trees lose 3-7 % above 400 roots).
SPLIT_NODES_PER_ROOT = 50


def _cfr_type_name(x) -> str:
    return getattr(x, "name", str(x))


@dataclass
class ExploitabilityStats:
    """src/p2/search/cfr_evaluator.py:35-38."""
    local_exploitability: torch.Tensor          # [N]
    local_best_response_values: torch.Tensor    # [N, 2]


@dataclass
class SampledLeaves:
    """What ``sample_leaves`` hands to the next search: the sampled non-root leaf rows, their
    public beliefs and their game states as roots (the reference wraps the same three things in a
    PublicBeliefState, sparse_cfr_evaluator.py:413-426)."""
    nodes: torch.Tensor      # [K] rows of this evaluator's tree
    beliefs: torch.Tensor    # [K, 2, 1326]
    roots: RootStates        # K root states for ``initialize_subgame``

    @property
    def env(self) -> RootStates:
        """The public states under the reference's attribute name (PublicBeliefState.env)."""
        return self.roots


class _TreeEnv(SimpleNamespace):
    """Per-node public states of the tree under the reference env's attribute names."""

    def legal_bins_amounts_and_mask(self, bet_bins: list[float] | None = None):
        """(amounts [N,B] int64, mask [N,B] bool) of src/p2/env/hunl_tensor_env.py:348-423."""
        bins = list(self.default_bet_bins if bet_bins is None else bet_bins)
        if bins != list(self.default_bet_bins):
            raise ValueError("the tree was built for bet bins %r" % (self.default_bet_bins,))
        amounts = torch.empty(self.N, len(bins) + 3, dtype=torch.int64, device=self.to_act.device)
        bins_c = (ctypes.c_float * max(1, len(bins)))(*bins)
        _lib.call("p2hip_bet_amounts", _lib.ptr(self.to_act), _lib.ptr(self.stacks), _lib.ptr(self.committed),
                  _lib.ptr(self.pot), self.N, bins_c, len(bins), _lib.ptr(amounts), _lib.stream_ptr())
        return amounts, self.legal_mask


class HipSparseCFREvaluator:
    def __init__(self, model, device, cfg, generator: torch.Generator | None = None, *,
                 compile_model: bool = True, fused_iteration: bool = True,
                 max_raises: int | None = None, tree_builder: str = "device",
                 split_small_batches: bool | None = None, lean_search: bool = True,
                 spread_state: bool = False, reuse_state: bool = False) -> None:
        self.device = torch.device(device)
        if model is not None and not hasattr(model, "leaf_values"):
            # the reference hands its network over as is (cfr_evaluator.py:306-322, 1025-1047): its
            # leaf rule and initial policy are NetworkLeafModel's
            from .leaf_models import NetworkLeafModel
            model = NetworkLeafModel(model, self.device)
        self.model = model
        self.cfg = cfg
        if self.device.type != "cuda":
            raise ValueError("HipSparseCFREvaluator requires a GPU device.")
        if not F.triton_is_available():
            raise RuntimeError("libp2hip.so or a GPU is not available; HipSparseCFREvaluator has no other backend.")
        # work items of the last three rounds of a launch start largest first (tree.launch_order): the
        # iteration kernel keeps three workgroups per compute unit resident
        self._sorted_tail = 3 * 3 * int(torch.cuda.get_device_properties(self.device).multi_processor_count)
        if getattr(cfg.env, "flop_showdown", False):
            raise NotImplementedError("the env's flop_showdown game variant (showdown right after the preflop round, "
                                      "hunl_tensor_env.py:900) is not built; the tree builders follow the full game")
        s = cfg.search
        self.float_dtype = torch.float32
        self.num_players = 2
        self.bet_bins = list(cfg.env.bet_bins)
        self.num_actions = len(self.bet_bins) + 3
        if self.num_actions > 8:
            raise ValueError("at most 8 action bins are supported")
        self.max_depth = s.depth
        self.cfr_iterations = s.iterations
        self.warm_start_iterations = max(0, min(s.warm_start_iterations, max(1, self.cfr_iterations - 1)))
        self.warm_start_type = str(getattr(s.warm_start_type, "name", s.warm_start_type))
        if self.warm_start_type not in ("model", "model_br"):
            raise ValueError(f"unknown warm_start_type {self.warm_start_type!r} (model | model_br)")
        self.warm_start_multiplier = float(s.warm_start_multiplier)
        self.cfr_type = CFRType[_cfr_type_name(s.cfr_type)]
        self.cfr_avg = bool(s.cfr_avg)
        self.cfr_plus = bool(s.cfr_plus)
        self.dcfr_alpha = self.dcfr_alpha_initial = s.dcfr_alpha
        self.dcfr_beta = self.dcfr_beta_initial = s.dcfr_beta
        self.dcfr_gamma = self.dcfr_gamma_initial = s.dcfr_gamma
        self.dcfr_alpha_final = s.dcfr_alpha_final
        self.dcfr_beta_final = s.dcfr_beta_final
        self.dcfr_gamma_final = s.dcfr_gamma_final
        self.dcfr_delay = s.dcfr_plus_delay
        self.use_final_policy_values = bool(s.value_targets_from_final_policy)
        self.sample_epsilon = float(getattr(s, "sample_epsilon", 0.25))
        self.generator = generator
        self.fused_iteration = bool(fused_iteration)
        self.max_raises = max_raises
        if tree_builder not in ("device", "host"):
            raise ValueError("tree_builder must be 'device' or 'host'")
        self.tree_builder = tree_builder     # both give identical trees; 'host' is the numpy builder
        # None: split each root into several workgroups when there are too few roots to fill the chip
        self.split_small_batches = split_small_batches
        # evaluate_cfr runs every iteration but the last one lean (rows nobody reads before the next
        # iteration are not stored) and lets reach_avg alternate between two buffers; the final state is
        # bit-identical either way.  False: every iteration as ``cfr_iteration`` runs it.
        self.lean_search = bool(lean_search)
        # True: the state tensors are dealt to two slabs that lie in different thirds of the card's physical
        # memory, found by measurement (``_place_state``): iterations 6-11 % faster from 1024 roots on; costs
        # a few probe launches in a process that is the first to use the memory and seconds per subgame once
        # memory has been used and given back, so it is for long searches.  ``state_placement``: what was done
        # for the current subgame
        self.spread_state = bool(spread_state)
        self.state_placement: dict = {"placed": False}
        # True: the state tensors of successive subgames are views into the same two slabs (a quarter larger
        # than the first subgame needs, replaced when one needs more), so a placement is paid for once.  The
        # reference allocates a fresh state per subgame: with this option every state tensor of an EARLIER
        # subgame, and any view of one, is overwritten by the next ``initialize_subgame``
        self.reuse_state = bool(reuse_state)
        self._arena: tuple[torch.Tensor, torch.Tensor] | None = None
        self.stats: dict = {}
        self.root_nodes = cfg.num_envs
        self.total_nodes = 0
        self.tree_depth = 0
        self.depth_offsets = [0]
        self.last_model_values = None
        self._last_model_values_buf = None
        self._t_scalars = F.TScalars(self.device, dtype=self.float_dtype)
        self._skip_t_scalars_update = False
        self._skip_record_stats = True
        self._fused_positive_regrets_buf = None
        self._fscal = self._t_scalars.floats      # the one-kernel iteration reads the first eight
        self._iscal = self._t_scalars.ints
        self._fscal_host = (ctypes.c_float * 8)()
        self._iscal_host = (ctypes.c_int64 * 8)()
        self._iter_bundles: dict = {}
        self._reach_avg_alt = None
        self._chance_helper = None
        self.subgame_serial = 0

    @property
    def enforce_zero_sum(self) -> bool:
        return bool(getattr(self.model, "enforce_zero_sum", False)) if self.model is not None else False

    # ------------------------------------------------------------------ subgame setup
    def _t(self, x: np.ndarray, dtype=None) -> torch.Tensor:
        t = torch.from_numpy(np.ascontiguousarray(x))
        if dtype is not None:
            t = t.to(dtype)
        return t.to(self.device)

    def _probe_ns_per_row(self, a: int, b: int, nbytes: int) -> float:
        """Time of the placement probe over the first ``nbytes`` of two buffers, per row it streams (the
        probe takes as many rows as fit, at most 12 288, so launches over buffers of different size compare)."""
        ms = ctypes.c_float()
        _lib.call("p2hip_placement_probe", a, b, nbytes, 3, ctypes.byref(ms), _lib.stream_ptr())
        rows = min(nbytes // 10 // 256 * 256 // (4 * NUM_HANDS), 12288)
        return float(ms.value) * 1e6 / rows

    def _place_state(self, shapes: list[tuple[int, ...]]) -> list[torch.Tensor]:
        """Zero-filled float tensors of the given shapes: the state of a search.

        The iteration kernel writes about ten of them at once, and the card's memory takes that faster when
        the written tensors lie in two different thirds (~96 GiB each) of its physical address space than when
        all lie in one: 4096 three-raise river roots 11.0 -> 9.9-10.0 ms per iteration, 2048 roots 5.56 ->
        5.0 ms, the depth-2 tree 1.86 -> 1.65 ms (tensors carved out of one large allocation at chosen offsets;
        a state allocated back to back by a fresh process lies inside one third).  Virtual addresses play no
        part and physical ones are not visible, but two buffers in different thirds show in the time of a
        small row-streaming kernel (``p2hip_placement_probe``: a fifth less than on two halves of one buffer).
        With ``spread_state`` the tensors are therefore dealt alternately to two slabs, and the second slab is
        chosen by that measurement: a candidate in the same third as the first slab is held, together with
        blocks of 16, 8, 4, 2 and 1 GiB, while the next one is allocated; the fastest candidate stays, the
        rest goes back.  The arithmetic does not change.  Cost: a handful of probe launches (0.3 ms each) and
        allocations - nothing measurable in a process that is the first to use the memory, up to seconds once
        memory has been used and given back (the driver clears what it hands out again).  Off by default."""
        dev = self.device
        sizes = [(4 * int(np.prod(sh)) + 255) // 256 * 256 for sh in shapes]
        side = [k % 2 for k in range(len(shapes))]
        slab_bytes = [sum(n for n, c in zip(sizes, side) if c == q) for q in (0, 1)]

        def carve(slabs):
            out, cursor = [], [0, 0]
            for sh, n, c in zip(shapes, sizes, side):
                nbytes = 4 * int(np.prod(sh))
                out.append(slabs[c][cursor[c]:cursor[c] + nbytes].view(self.float_dtype).view(*sh))
                cursor[c] += n
            for c in (0, 1):
                slabs[c][:cursor[c]].zero_()
            return out

        if self.reuse_state and self._arena is not None:
            if all(self._arena[q].numel() >= slab_bytes[q] for q in (0, 1)):
                self.state_placement = dict(self.state_placement, reused=True)
                return carve(self._arena)
            self._drop_state()                               # the slabs are too small: give them back first
        self.state_placement = {"placed": False}
        place = self.spread_state and min(slab_bytes) >= max(STATE_SPREAD_MIN_SLAB_BYTES, 2 * _PROBE_MIN_BYTES)
        if not place and not self.reuse_state:
            return [torch.zeros(*sh, dtype=self.float_dtype, device=dev) for sh in shapes]
        if self.reuse_state:
            slab_bytes = [(b + b // 4 + 255) // 256 * 256 for b in slab_bytes]
        first = torch.empty(slab_bytes[0], dtype=torch.uint8, device=dev)
        if place:
            second = self._second_slab_elsewhere(first, slab_bytes)
        else:
            second = torch.empty(slab_bytes[1], dtype=torch.uint8, device=dev)
        if self.reuse_state:
            self._arena = (first, second)
        return carve((first, second))

    def _second_slab_elsewhere(self, first: torch.Tensor, slab_bytes: list[int]) -> torch.Tensor:
        """The second slab of ``_place_state``: of the candidates probed against ``first`` the one with the
        shortest probe time; candidates that were not taken go back to the card."""
        dev = self.device
        # what the probe takes when all of its arrays lie in one third: the arrays packed into the first
        # 1.2 GiB of the first slab (a stretch that short hardly ever reaches across a boundary)
        half = min(slab_bytes[0] // 2 // 256 * 256, _PROBE_PACKED_BYTES)
        same_ns = self._probe_ns_per_row(first.data_ptr(), first.data_ptr() + half, half)
        probe_bytes = min(slab_bytes)
        tried: list[tuple[float, torch.Tensor]] = []
        blocks: list[ctypes.c_void_p] = []
        try:
            for attempt in range(STATE_SPREAD_TRIES):
                free, total = torch.cuda.mem_get_info(dev)
                if tried and free - slab_bytes[1] < total // 8:
                    break                                    # no room for another candidate without pressure
                try:
                    cand = torch.empty(slab_bytes[1], dtype=torch.uint8, device=dev)
                except torch.cuda.OutOfMemoryError:
                    if not tried:
                        raise
                    break                                    # what was found so far has to do
                tried.append((self._probe_ns_per_row(first.data_ptr(), cand.data_ptr(), probe_bytes), cand))
                cand = None
                if tried[-1][0] < STATE_SPREAD_ACCEPT * same_ns or attempt == STATE_SPREAD_TRIES - 1:
                    break
                free, total = torch.cuda.mem_get_info(dev)
                if free - STATE_SPREAD_STEP_BYTES - slab_bytes[1] >= total // 8:
                    piece = STATE_SPREAD_STEP_BYTES + (1 << 30)
                    while piece > 1 << 30:
                        piece >>= 1
                        block = ctypes.c_void_p()
                        if _lib.load().p2hip_device_reserve(piece, ctypes.byref(block)) == 0 and block.value:
                            blocks.append(block)
        finally:
            for block in blocks:
                _lib.call("p2hip_device_release", block)
        best = min(range(len(tried)), key=lambda k: tried[k][0])
        second = tried[best][1]
        self.state_placement = {"placed": True, "probe_ns_per_row_inside_first_slab": same_ns,
                                "probe_ns_per_row_candidates": [t for t, _ in tried], "chosen": best,
                                "slab_GiB": [b / 2 ** 30 for b in slab_bytes]}
        rejected = len(tried) > 1
        tried.clear()
        if rejected:
            torch.cuda.empty_cache()                         # the candidates that were not taken go back to the card
        return second

    _STATE_TENSORS = ("policy_probs", "policy_probs_avg", "policy_probs_sample", "cumulative_regrets",
                      "regret_weight_sums", "beliefs", "beliefs_avg", "self_reach", "self_reach_avg", "latest_values",
                      "values_avg", "_scratch", "_reach_avg_alt")

    def _drop_state(self) -> None:
        """Let go of the state tensors and their slabs (``reuse_state``), so that larger slabs can take
        their place on the card."""
        for name in self._STATE_TENSORS:
            setattr(self, name, None)
        self._arena = None
        self._iter_bundles = {}
        self.last_model_values = None
        torch.cuda.empty_cache()

    def _construct_subgame(self, src_env, src_indices) -> None:
        """Build the sparse tree and allocate the state (sparse_cfr_evaluator.py:142-306)."""
        if isinstance(src_env, RootStates):
            idx = src_indices.cpu().numpy() if hasattr(src_indices, "cpu") else np.asarray(src_indices)
            roots = src_env.select(idx)
        else:
            roots = RootStates.from_env(src_env, src_indices)
        if self.tree_builder == "device":
            tree = build_sparse_tree_device(roots, self.bet_bins, self.max_depth, max_raises=self.max_raises,
                                            device=self.device)
        else:
            tree = build_sparse_tree(roots, self.bet_bins, self.max_depth, max_raises=self.max_raises)
        self.tree: SparseTree = tree
        self.subgame_serial += 1           # lets leaf models drop what they cached for the previous subgame
        resident = getattr(tree, "device_arrays", None) or {}

        def tt(name, host_array):
            """The tree array as a device tensor: the builder's own tensor when it left one."""
            t = resident.get(name)
            return t if t is not None else self._t(host_array)
        dev = self.device
        self.depth_offsets = list(tree.depth_offsets)
        self.tree_depth = tree.tree_depth
        self.total_nodes = tree.total
        self.root_nodes = tree.n_roots
        self.top_nodes = tree.top
        T, N = tree.total, tree.n_roots
        self.valid_mask = torch.ones(T, dtype=torch.bool, device=dev)
        self.parent_index = tt("parent_index", tree.parent_index)
        self.action_from_parent = tt("action_from_parent", tree.action_from_parent)
        self.child_count = tt("child_count", tree.child_count)
        self.child_offsets = tt("child_offsets", tree.child_offsets)
        self.prev_actor = tt("prev_actor", tree.prev_actor)
        self.legal_mask = tt("legal_mask", tree.legal_mask)
        self.leaf_mask = tt("leaf_mask", tree.leaf_mask)
        self.new_street_mask = tt("new_street_mask", tree.new_street_mask)
        self.child_mask = self.legal_mask & (~self.leaf_mask)[:, None]
        st = tree.state
        # Boards per node.  Every action saves the board before cards are dealt
        # (hunl_tensor_env.py:862): below the roots the previous board is the root's board.  The
        # current board of a node that closed a betting round shows the next cards only when the
        # roots carry their runout.
        d_root_index = tt("root_index", tree.root_index)
        d_last_board = self._t(tree.board)[d_root_index]
        d_last_board[:N] = self._t(roots.previous_board())
        if roots.runout is not None:
            cards = self._t(CARDS_ON_STREET)[tt("street", st["street"]).clamp(0, 4)]
            shown = torch.arange(5, device=dev)[None, :] < cards[:, None]
            d_node_board = torch.where(shown, self._t(roots.runout)[d_root_index], torch.full_like(d_last_board, -1))
        else:
            d_node_board = self._t(tree.board)[d_root_index]
        self._roots = roots
        self.env = _TreeEnv(
            N=T, to_act=tt("to_act", st["to_act"]), done=tt("done", st["done"]), street=tt("street", st["street"]),
            pot=tt("pot", st["pot"]), stacks=tt("stacks", st["stacks"]), committed=tt("committed", st["committed"]),
            starting_stacks=tt("starting_stacks", st["starting_stacks"]), scale=tt("scale", st["scale"]),
            actions_this_round=tt("actions_this_round", st["actions_this_round"]), button=tt("button", st["button"]),
            min_raise=tt("min_raise", st["min_raise"]), is_allin=tt("is_allin", st["is_allin"]),
            board_indices=d_node_board, last_board_indices=d_last_board, bb=roots.bb,
            default_bet_bins=list(self.bet_bins), legal_mask=self.legal_mask)
        self.feature_encoder = (self.model.create_feature_encoder(self.env, device=dev, dtype=self.float_dtype)
                                if hasattr(self.model, "create_feature_encoder")
                                else RebelFeatureEncoder(self.env, device=dev, dtype=self.float_dtype))
        self._root_index = tt("root_index", tree.root_index)
        model_mask = tree.leaf_mask & ~st["done"]
        self.model_indices = self._t(np.nonzero(model_mask)[0].astype(np.int64))
        self.showdown_indices = self._t(np.nonzero(tree.showdown_mask)[0].astype(np.int64))
        self.showdown_actors = self.env.to_act[self.showdown_indices]
        d_potential = resident.get("showdown_potential")
        if d_potential is None:
            d_potential = self._t(tree.showdown_potential)
        self.showdown_potential = d_potential[self.showdown_indices]
        self._potential_all = d_potential.to(torch.float32)

        # the state of the search, in the order it is dealt to the two slabs of ``_place_state``: five [T, H]
        # tensors, six [T, 2, H], the scratch rows, and the second reach_avg buffer of a lean search
        one, two = (T, NUM_HANDS), (T, 2, NUM_HANDS)
        with_alt = self.fused_iteration and self.lean_search
        pool = self._place_state([one] * 5 + [two] * 6 + [one] + ([two] if with_alt else []))
        self._reach_avg_alt = pool.pop() if with_alt else None
        if with_alt:
            self._reach_avg_alt[:N] = 1.0
        pool.reverse()

        def z1():
            t = pool.pop()
            _req(tuple(t.shape) == one, "state pool: a [T, H] tensor is next")
            return t

        def z2():
            t = pool.pop()
            _req(tuple(t.shape) == two, "state pool: a [T, 2, H] tensor is next")
            return t

        self.policy_probs, self.policy_probs_avg, self.policy_probs_sample = z1(), z1(), z1()
        self.cumulative_regrets, self.regret_weight_sums = z1(), z1()
        self.uniform_policy = torch.zeros(T, NUM_HANDS, dtype=self.float_dtype, device=dev)
        cc_dest = self.child_count[:tree.top].repeat_interleave(self.child_count[:tree.top])
        self.uniform_policy[N:] = (1.0 / cc_dest)[:, None].expand(-1, NUM_HANDS)
        self.beliefs, self.beliefs_avg = z2(), z2()
        self.root_pre_chance_beliefs = torch.zeros(N, 2, NUM_HANDS, dtype=self.float_dtype, device=dev)
        self.self_reach = z2()
        self.self_reach[:N] = 1.0
        self.self_reach_avg = z2().copy_(self.self_reach)
        self.latest_values = z2()
        folded = tt("fold_mask", tree.fold_mask)
        rew = tt("reward", tree.reward)
        self.latest_values[folded, 0] = rew[folded][:, None]
        self.latest_values[folded, 1] = -rew[folded][:, None]
        self.values_avg = z2().copy_(self.latest_values)
        self.last_model_values = None
        self._scratch = z1()
        flags = np.zeros(T, dtype=np.uint8)
        flags[tree.showdown_mask] |= _NODE_SHOWDOWN
        flags[st["done"]] |= _NODE_DONE
        # what a lean iteration decides its stores by: rows with children, and childless rows whose ranges
        # are read by a leaf evaluation (the showdown kernel, or the leaf network when there is one)
        flags[tree.child_count > 0] |= _NODE_PARENT
        flags[tree.showdown_mask & (tree.child_count == 0)] |= _NODE_LEAF_EVAL
        if self.model is not None:
            flags[model_mask & (tree.child_count == 0)] |= _NODE_LEAF_EVAL
        self._node_flags = self._t(flags)
        def per_root(mask):
            """Rows selected by ``mask`` grouped by root (ascending inside a root) + offsets [N+1]."""
            rows = np.nonzero(mask)[0]
            roots_of = tree.root_index[rows]
            order = np.argsort(roots_of, kind="stable")
            counts = np.bincount(roots_of, minlength=N)
            return (self._t(rows[order].astype(np.int64)),
                    self._t(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)))

        self._root_parents, self._root_parent_offsets = per_root(tree.child_count > 0)
        self._root_showdown_nodes, self._root_showdown_offsets = per_root(tree.showdown_mask)
        self._max_children = int(tree.child_count.max()) if T else 1
        self._has_model_leaves = bool(model_mask.any())
        self._iter_bundles = {}
        split = self.split_small_batches
        if split is None:
            split = N < SPLIT_ROOTS_BELOW or T >= SPLIT_NODES_PER_ROOT * N
        self._items = self._split_items(tree, SPLIT_MID_LEVEL) if split else None
        # The regret part has no order among families: it runs over the coarser of the two partitions
        # (whole tree tops), which makes fewer and longer workgroups of the same work.
        self._items_regret = (self._split_items(tree) if self._items is not None and len(self._items.tiers) > 2
                              else self._items)
        self._root_items = None
        if self._items is None and T:
            # Roots of unequal size (mixed streets, stacks, pots): one work item per root, largest tree first, so
            # that the launch does not end on a long root that started last.  (Row order with only the last
            # rounds by size, which wins for the work items of equal trees, loses here: 16 384 mixed roots 23.2 ms
            # per iteration against 22.3 ms.)
            size = np.bincount(tree.root_index, minlength=N)
            if size.min() != size.max():
                order = launch_order(size, N)

                def per_item(mask):
                    rows = np.nonzero(mask)[0]
                    slot = np.argsort(order)[tree.root_index[rows]]                 # position of the row's root in the order
                    by_slot = np.argsort(slot, kind="stable")
                    counts = np.bincount(slot, minlength=N)
                    return (self._t(rows[by_slot].astype(np.int64)),
                            self._t(np.concatenate([[0], np.cumsum(counts)]).astype(np.int64)))
                parents, parent_offsets = per_item(tree.child_count > 0)
                showdown, showdown_offsets = per_item(tree.showdown_mask)
                self._root_items = SimpleNamespace(parents=parents, parent_offsets=parent_offsets, showdown=showdown,
                                                   showdown_offsets=showdown_offsets, item_root=self._t(order),
                                                   item_top=self._t(np.ones(N, np.uint8)))

    def _split_items(self, tree: SparseTree, mid_level: int | None = None):
        """``tree.split_work_items`` with the arrays on the device (None if the tree is too shallow to cut)."""
        # equal trees: items in row order, the last rounds' items by size; roots of unequal size: all by size
        sizes = np.bincount(tree.root_index, minlength=self.root_nodes)
        tail = self._sorted_tail if sizes.min() == sizes.max() else tree.total
        it = split_work_items(tree, self.root_nodes, SPLIT_CUT_LEVEL, mid_level, sorted_tail=tail)
        if it is None:
            return None
        for name in ("parents", "parent_offsets", "showdown", "showdown_offsets", "item_root", "item_top"):
            setattr(it, name, self._t(getattr(it, name)))
        return it

    def initialize_subgame(self, src_env, src_indices, initial_beliefs: torch.Tensor | None = None) -> None:
        """cfr_evaluator.py:770-828."""
        self._construct_subgame(src_env, src_indices)
        N = self.root_nodes
        if initial_beliefs is None:
            initial_beliefs = torch.full((N, 2, NUM_HANDS), 1.0 / NUM_HANDS, dtype=self.float_dtype, device=self.device)
        else:
            initial_beliefs = initial_beliefs.to(device=self.device, dtype=self.float_dtype)
        self.beliefs[:N] = initial_beliefs
        self.beliefs_avg[:N] = initial_beliefs
        self.root_pre_chance_beliefs[:] = initial_beliefs
        self.self_reach[:N] = 1.0
        self.self_reach_avg[:N] = 1.0
        board = self._t(self.tree.board)
        onehot = combo_to_onehot_tensor(device=self.device).float()
        board_mask = torch.zeros(N, 52, dtype=self.float_dtype, device=self.device)
        valid = board >= 0
        rows = torch.arange(N, device=self.device)[:, None].expand_as(board)
        board_mask[rows[valid], board[valid]] = 1.0
        root_allowed = (onehot @ board_mask.T).T < 0.5
        root_prob = root_allowed.float()
        root_prob /= root_prob.sum(dim=-1, keepdim=True).clamp(min=1.0)
        self.allowed_hands = root_allowed[self._root_index].contiguous()
        self.allowed_hands_prob = root_prob[self._root_index].contiguous()
        self._init_hand_rank_data()
        self.t_sample = torch.full((self.total_nodes,), -1, dtype=torch.long, device=self.device)
        self.stats["evaluator_total_nodes"] = float(self.total_nodes)
        self.stats["evaluator_root_nodes"] = float(self.root_nodes)
        self.stats["evaluator_tree_depth"] = float(self.tree_depth)

    def _init_hand_rank_data(self) -> None:
        """Per-root strength tables for the showdown kernel (replaces the HandRankData of
        cfr_evaluator.py:406-482; the card-id ranker is the one the reference's fused
        evaluator installs, fused_sparse_cfr_evaluator.py:70-78)."""
        if self.showdown_indices.numel() == 0:
            self.hand_rank_data = None
            return
        board = self._t(self.tree.board)
        self.hand_rank_data = rules_hip.build_showdown_tables(board, triton_order=True)
        self._showdown_rows = self._root_index[self.showdown_indices].contiguous()
        self._showdown_scale = self.env.scale[self.showdown_indices].contiguous()
        self._showdown_potential_f = self.showdown_potential.to(self.float_dtype).contiguous()

    def _showdown_value_both(self, beliefs: torch.Tensor) -> torch.Tensor:
        """beliefs [M,2,H] of the showdown rows -> [M,2,H] (cfr_evaluator.py:484-601)."""
        if self.showdown_indices.numel() == 0:
            return torch.zeros(0, 2, NUM_HANDS, device=self.device, dtype=self.float_dtype)
        return rules_hip.showdown_value_both(beliefs, self.hand_rank_data, self._showdown_potential_f,
                                             self._showdown_scale, table_row=self._showdown_rows)

    def _showdown_value(self, beliefs: torch.Tensor, hero: int) -> torch.Tensor:
        """[M,H] showdown values of player ``hero`` at the showdown rows (cfr_evaluator.py:492-601); one
        launch computes both players, so callers that want both use ``_showdown_value_both``."""
        _req(hero in (0, 1), "hero in (0, 1)")
        return self._showdown_value_both(beliefs)[:, hero]

    # ------------------------------------------------------------------ host-side scalars
    def _get_mixing_weights(self, t: int):
        """cfr_evaluator.py:285-303."""
        if self.cfr_type == CFRType.standard:
            return t, 1
        if self.cfr_type == CFRType.linear:
            return t, 2
        if self.cfr_type == CFRType.discounted:
            return t ** self.dcfr_gamma, (t + 1) ** self.dcfr_gamma
        if t > self.dcfr_delay:
            return t - self.dcfr_delay, 2
        return 0, 1

    def apply_schedules(self, t: int) -> None:
        """cfr_evaluator.py:1294-1328."""
        total = max(1, self.cfr_iterations - self.warm_start_iterations)
        progress = max(0, t - self.warm_start_iterations)
        x = min(1.0, max(0.0, progress / float(total)))

        def lerp(a0, a1):
            return a0 if a1 is None else a0 + (a1 - a0) * x

        self.dcfr_alpha = lerp(self.dcfr_alpha_initial, self.dcfr_alpha_final)
        self.dcfr_beta = lerp(self.dcfr_beta_initial, self.dcfr_beta_final)
        self.dcfr_gamma = lerp(self.dcfr_gamma_initial, self.dcfr_gamma_final)

    def _avg_policy_copies(self, t: int) -> bool:
        return (self.cfr_type in (CFRType.discounted, CFRType.discounted_plus) and t <= self.dcfr_delay) or t == 0

    def prepare_replay(self, t: int) -> None:
        """Refresh every iteration-dependent device scalar for iteration ``t``; call outside
        any captured region (fused_sparse_cfr_evaluator.py:535-550)."""
        self.apply_schedules(t)
        mix_old, mix_new = self._get_mixing_weights(t)
        apply_dcfr = self.cfr_type in (CFRType.discounted, CFRType.discounted_plus)
        (a, a_den), (b, b_den) = F.discount_pair(t, self.dcfr_alpha), F.discount_pair(t, self.dcfr_beta)
        total = float(mix_old) + float(mix_new)
        f = self._fscal_host
        f[0], f[1], f[2], f[3] = a, b, a_den, b_den
        f[4], f[5], f[6] = float(mix_old), float(mix_new), total
        f[7] = 1.0 / total if total != 0.0 else 1.0
        i = self._iscal_host
        linear = self.cfr_type == CFRType.linear
        # the reference's fused evaluator accumulates linear-CFR regrets without the CFR+ clamp
        # (fused_sparse_cfr_evaluator.py:503-507)
        i[0], i[1], i[2] = int(t), int(apply_dcfr), int(self.cfr_plus and not linear)
        i[6], i[7] = int(self.cfr_avg), int(linear)
        i[3], i[4], i[5] = int(self._avg_policy_copies(t)), int(self.enforce_zero_sum), int(not self.use_final_policy_values)
        # one launch for every scalar of the iteration (the per-operation kernels read the same array
        # through the 0-D views of ``_t_scalars``); the de-averaging pair only where something reads it
        needs_pair = self.cfr_avg or not self.fused_iteration
        self._t_scalars.write(f, i, F.TScalars.deaveraging_factors(mix_old, mix_new) if needs_pair else None)

    def _get_sampling_schedule(self) -> torch.Tensor:
        """cfr_evaluator.py:382-404: per-root iteration at which the policy is snapshotted."""
        N = self.root_nodes
        if self.cfr_type == CFRType.discounted_plus:
            low = max(self.warm_start_iterations, self.dcfr_delay) + 1
        else:
            low = self.warm_start_iterations + 1
        low = min(low, self.cfr_iterations)
        high = max(self.cfr_iterations, low + 1)
        if self.cfr_type != CFRType.standard:
            dist = torch.arange(low, high, dtype=torch.float32) + 1
        else:
            dist = torch.ones(high - low)
        dist /= dist.sum()
        gen = self.generator if (self.generator is not None and self.generator.device.type == "cpu") else None
        ts = torch.multinomial(dist, N, replacement=True, generator=gen) + low
        return ts.to(self.device)[self._root_index].contiguous()

    # ------------------------------------------------------------------ per-op building blocks
    def _mask_invalid(self, tensor: torch.Tensor) -> None:
        pass  # every row of the sparse tree is a real node

    def _normalize_beliefs(self, target: torch.Tensor | None = None) -> None:
        F.fused_block_and_normalize_beliefs_(self.beliefs if target is None else target,
                                             self.allowed_hands, self.allowed_hands_prob)

    def _calculate_reach_weights(self, target: torch.Tensor, policy: torch.Tensor) -> None:
        for depth in range(self.tree_depth):
            F.fused_reach_weights_depth_(reach=target, policy=policy, allowed_mask=self.allowed_hands,
                                         parent_index=self.parent_index, prev_actor=self.prev_actor,
                                         start=self.depth_offsets[depth + 1], end=self.depth_offsets[depth + 2])

    def _get_root_index(self) -> torch.Tensor:
        return self._root_index

    def _propagate_all_beliefs(self, target: torch.Tensor | None = None,
                               reach_weights: torch.Tensor | None = None) -> None:
        target = self.beliefs if target is None else target
        reach_weights = self.self_reach if reach_weights is None else reach_weights
        F.fused_deep_beliefs_(out=target, root_beliefs=target, reach_weights=reach_weights,
                              allowed_prob=self.allowed_hands_prob, root_index=self._root_index,
                              num_roots=self.root_nodes)

    def update_policy(self, t: int) -> None:
        """fused_sparse_cfr_evaluator.py:201-236."""
        bottom, top = self.depth_offsets[1], self.depth_offsets[-2]
        if self._fused_positive_regrets_buf is None or \
                self._fused_positive_regrets_buf.shape != self.cumulative_regrets.shape:
            self._fused_positive_regrets_buf = torch.empty_like(self.cumulative_regrets)
        pos = self._fused_positive_regrets_buf
        torch.clamp(self.cumulative_regrets, min=0.0, out=pos)
        parent_sum = F.fused_parent_sum(pos, self.child_offsets[:top].contiguous(),
                                        self.child_count[:top].contiguous(), max_children=self.num_actions)
        F.fused_divide_by_parent_sum_(pos=pos[bottom:], fallback=self.uniform_policy[bottom:], parent_sum=parent_sum,
                                      parent_index=self.parent_index[bottom:].contiguous(),
                                      out=self.policy_probs[bottom:])
        self._calculate_reach_weights(self.self_reach, self.policy_probs)
        self._propagate_all_beliefs(self.beliefs, self.self_reach)
        self.update_average_policy(t)
        self._calculate_reach_weights(self.self_reach_avg, self.policy_probs_avg)
        self._propagate_all_beliefs(self.beliefs_avg, self.self_reach_avg)

    def update_average_policy(self, t: int) -> None:
        """fused_sparse_cfr_evaluator.py:355-398."""
        if self._avg_policy_copies(t):
            self.policy_probs_avg[:] = self.policy_probs
            return
        N, top = self.root_nodes, self.depth_offsets[-2]
        F.fused_average_policy_mix_with_tensors_(
            policy_probs_avg=self.policy_probs_avg, policy_probs=self.policy_probs, self_reach=self.self_reach,
            self_reach_avg=self.self_reach_avg, to_act=self.env.to_act, parent_index=self.parent_index,
            old=self._t_scalars.mix_old, new=self._t_scalars.mix_new, total_weight=self._t_scalars.mix_total,
            bottom=N)
        parent_sum = F.fused_parent_sum(self.policy_probs_avg, self.child_offsets[:top].contiguous(),
                                        self.child_count[:top].contiguous(), max_children=self.num_actions)
        child = self.policy_probs_avg[N:]
        F.fused_divide_by_parent_sum_(pos=child, fallback=child, parent_sum=parent_sum,
                                      parent_index=self.parent_index[N:].contiguous(), out=child, eps=1e-5)
        self.policy_probs_avg[:N] = 0.0

    def compute_instantaneous_regrets(self, values_achieved: torch.Tensor,
                                      values_expected: torch.Tensor | None = None) -> torch.Tensor:
        """fused_sparse_cfr_evaluator.py:312-349."""
        if values_expected is None:
            values_expected = values_achieved
        bottom, top = self.depth_offsets[1], self.depth_offsets[-2]
        beliefs = self.beliefs_avg if self.cfr_avg else self.beliefs
        regrets = torch.zeros_like(self.policy_probs)
        src_weights = F.unblocked_mass_opp_at_parents_triton(beliefs, self.env.to_act, top)
        rows = torch.arange(top, device=self.device)
        actor_values = values_expected[:top][rows, self.env.to_act[:top], :].contiguous()
        F.fused_regret_tail_(regrets=regrets, values_achieved=values_achieved.contiguous(), actor_values=actor_values,
                             src_weights=src_weights, parent_index=self.parent_index, prev_actor=self.prev_actor,
                             bottom=bottom)
        return regrets

    def compute_expected_values(self, policy=None, beliefs=None, leaf_values=None, values=None) -> None:
        """fused_sparse_cfr_evaluator.py:242-306."""
        policy = self.policy_probs if policy is None else policy
        beliefs = self.beliefs if beliefs is None else beliefs
        leaf_values = self.latest_values if leaf_values is None else leaf_values
        values = leaf_values if values is None else values
        if leaf_values is not values:
            torch.where(self.leaf_mask[:, None, None], leaf_values, torch.zeros_like(values), out=values)
        bottom, top = self.depth_offsets[1], self.depth_offsets[-2]
        rows = torch.arange(top, device=self.device)
        actor_beliefs = beliefs[:top][rows, self.env.to_act[:top], :].contiguous()
        marginal = actor_beliefs.index_select(0, self.parent_index[bottom:]) * policy[bottom:]
        occ = torch.zeros_like(policy)
        occ[bottom:] = F.unblocked_mass_ratio_indirect_triton(
            numer_target=marginal.contiguous(), denom_target=actor_beliefs,
            parent_index=self.parent_index[bottom:].contiguous())
        for depth in range(self.tree_depth - 1, -1, -1):
            base, end = self.depth_offsets[depth], self.depth_offsets[depth + 1]
            F.fused_weighted_parent_sum(values=values, prev_actor=self.prev_actor, policy_hero=policy, policy_opp=occ,
                                        child_offsets=self.child_offsets[base:end].contiguous(),
                                        child_count=self.child_count[base:end].contiguous(), parent_base=base,
                                        max_children=self.num_actions)

    def update_average_values(self, t: int) -> None:
        """fused_sparse_cfr_evaluator.py:404-414."""
        F.fused_avg_values_zero_sum_(values_avg=self.values_avg, latest_values=self.latest_values,
                                     beliefs=self.beliefs_avg, old=self._t_scalars.mix_old,
                                     new=self._t_scalars.mix_new, inv_total=self._t_scalars.mix_inv_total,
                                     enforce_zero_sum=self.enforce_zero_sum, ignore_mask=self.env.done)

    # ------------------------------------------------------------------ leaf values
    _LEAF_DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

    def gather_leaf_rows(self, table: torch.Tensor, rows: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """``out[i, :2652] = table[rows[i]]`` in ``out``'s dtype (float32 / bfloat16 / float16), one
        launch: the gather of the leaves' ranges with the cast to the network's dtype folded in.
        ``out`` may be wider than 2652 columns (the network's input matrix); the rest is left alone."""
        _req(table.dtype == torch.float32 and table.is_contiguous() and table.dim() == 3 and
             tuple(table.shape[1:]) == (2, NUM_HANDS), "table: contiguous float32 [rows, 2, 1326]")
        _req(out.dtype in self._LEAF_DTYPES and out.dim() == 2 and out.stride(1) == 1 and
             out.shape == (rows.numel(), out.shape[1]) and out.shape[1] >= 2 * NUM_HANDS, "out: [len(rows), >= 2652]")
        _req(rows.dtype == torch.int64 and rows.is_contiguous(), "rows: contiguous int64")
        _lib.require_gpu(table, "gather_leaf_rows")
        _lib.call("p2hip_gather_leaf_rows", _lib.ptr(table), _lib.ptr(rows), rows.numel(), table.shape[0], _lib.ptr(out),
                  self._LEAF_DTYPES[out.dtype], out.stride(0), _lib.stream_ptr())
        return out

    def _scatter_leaf_values(self, values: torch.Tensor) -> None:
        """``latest_values[model_indices] = values`` with the conversion to float32 folded in."""
        k = self.model_indices.numel()
        values = values.reshape(k, 2 * NUM_HANDS)
        if values.dtype not in self._LEAF_DTYPES or values.stride(1) != 1 or values.stride(0) % 4:
            values = values.to(self.float_dtype).contiguous()
        _lib.call("p2hip_scatter_leaf_rows", _lib.ptr(values), self._LEAF_DTYPES[values.dtype], values.stride(0),
                  _lib.ptr(self.model_indices), k, _lib.ptr(self.latest_values), self.total_nodes, _lib.stream_ptr())

    def _model_leaf_values(self, beliefs: torch.Tensor) -> torch.Tensor | None:
        """The network's answer for the model leaves, [K, 2, 1326], in whatever dtype it answers in.
        A model with ``leaf_values_from_nodes`` is handed the whole node table and gathers its rows
        itself (``gather_leaf_rows``: straight into its input matrix, in its dtype)."""
        if self.model_indices.numel() == 0:
            return None
        if self.model is None:
            return torch.zeros(self.model_indices.numel(), 2, NUM_HANDS, dtype=self.float_dtype, device=self.device)
        if hasattr(self.model, "leaf_values_from_nodes") and beliefs.is_contiguous() and beliefs.dtype == torch.float32:
            return self.model.leaf_values_from_nodes(beliefs, self.model_indices, self)
        return self.model.leaf_values(beliefs[self.model_indices], self.model_indices, self)

    def _set_model_values_impl(self, t: int, beliefs: torch.Tensor) -> None:
        """fused_sparse_cfr_evaluator.py:420-445 (CFR-AVG de-averaging included)."""
        hv = self._model_leaf_values(beliefs)
        if hv is None:
            return
        if not self.cfr_avg:
            # nothing reads the previous answer without CFR-AVG: no copy of it is kept
            self._scatter_leaf_values(hv)
            self.last_model_values = hv
            return
        hv = hv.to(self.float_dtype)
        if t <= 1 or self.last_model_values is None:
            self._scatter_leaf_values(hv)
        else:
            unmixed = torch.empty_like(hv)
            F.fused_model_values_mix_zero_sum(hv.contiguous(), self.last_model_values.contiguous(),
                                              beliefs[self.model_indices].contiguous(), self._t_scalars.mix_onon,
                                              self._t_scalars.mix_oon, unmixed, self.enforce_zero_sum)
            self._scatter_leaf_values(unmixed)
        # The previous network output lives in a buffer of its own (the reference pins it the same
        # way, fused_sparse_cfr_evaluator.py:464-469): a captured graph keeps reading this address on
        # every replay, and a network that reuses its output tensor cannot alias "last" and "current".
        buf = self._last_model_values_buf
        if buf is None or buf.shape != hv.shape or buf.dtype != hv.dtype:
            buf = self._last_model_values_buf = torch.empty_like(hv)
        buf.copy_(hv)
        self.last_model_values = buf

    @torch.no_grad()
    def set_leaf_values(self, t: int, beliefs: torch.Tensor | None = None, *, showdown: bool = True) -> None:
        """fused_sparse_cfr_evaluator.py:447-472: model rows through PyTorch, showdown rows
        through the showdown kernel; fold rows are constants set at construction."""
        if beliefs is None:
            beliefs = self.beliefs_avg if self.cfr_avg else self.beliefs
        self._set_model_values_impl(t, beliefs)
        if showdown and self.showdown_indices.numel():
            self.latest_values[self.showdown_indices] = self._showdown_value_both(beliefs[self.showdown_indices])

    # ------------------------------------------------------------------ iteration
    def _build_iter_args(self, items=None, reach_avg=None, reach_avg_prev=None) -> _IterArgs:
        a = _IterArgs()
        p = _lib.ptr
        a.child_offsets, a.child_count, a.to_act = p(self.child_offsets), p(self.child_count), p(self.env.to_act)
        a.node_flags = p(self._node_flags)
        a.root_parent_offsets, a.root_parents = p(self._root_parent_offsets), p(self._root_parents)
        a.root_showdown_offsets, a.root_showdown_nodes = p(self._root_showdown_offsets), p(self._root_showdown_nodes)
        a.t_sample, a.allowed, a.allowed_prob = p(self.t_sample), p(self.allowed_hands), p(self.allowed_hands_prob)
        a.tables = p(self.hand_rank_data) if self.hand_rank_data is not None else None
        a.potential, a.scale = p(self._potential_all), p(self.env.scale)
        a.policy, a.policy_avg, a.policy_sample = p(self.policy_probs), p(self.policy_probs_avg), p(self.policy_probs_sample)
        a.cum, a.wsum = p(self.cumulative_regrets), p(self.regret_weight_sums)
        a.beliefs, a.beliefs_avg = p(self.beliefs), p(self.beliefs_avg)
        a.reach = p(self.self_reach)
        a.reach_avg = p(self.self_reach_avg if reach_avg is None else reach_avg)
        a.reach_avg_prev = p(reach_avg_prev)
        a.latest, a.values_avg, a.scratch = p(self.latest_values), p(self.values_avg), p(self._scratch)
        a.fscal, a.iscal = p(self._fscal), p(self._iscal)
        it = items if items is not None else (self._items if self._items is not None else self._root_items)
        if it is not None:
            a.root_parent_offsets, a.root_parents = p(it.parent_offsets), p(it.parents)
            a.root_showdown_offsets, a.root_showdown_nodes = p(it.showdown_offsets), p(it.showdown)
            a.item_root, a.item_top = p(it.item_root), p(it.item_top)
        return a

    def _launch_items(self, args: _IterArgs, n_items: int, phases: int) -> None:
        if n_items == 0:
            return
        code = _lib.load().p2hip_cfr_iteration(ctypes.byref(args), n_items, self._max_children, phases,
                                               _lib.stream_ptr())
        _lib.check(code, "p2hip_cfr_iteration")

    def _other_reach_avg(self) -> torch.Tensor:
        """The second reach_avg buffer of the alternating scheme (allocated on first use; root rows 1)."""
        if self._reach_avg_alt is None or self._reach_avg_alt.shape != self.self_reach_avg.shape:
            self._reach_avg_alt = torch.empty_like(self.self_reach_avg)
            self._reach_avg_alt[:self.root_nodes] = 1.0
        return self._reach_avg_alt

    def _iter_bundle(self, alternate: bool) -> SimpleNamespace:
        """Argument blocks of the iteration kernel for the tensor ``self_reach_avg`` names right now:
        updated in place (the old row saved in the scratch tensor), or — ``alternate`` — read as the
        previous iteration's and the new one written to the other buffer."""
        key = (self.self_reach_avg.data_ptr(), bool(alternate))
        b = self._iter_bundles.get(key)
        if b is not None:
            return b
        if alternate:
            kw = dict(reach_avg=self._other_reach_avg(), reach_avg_prev=self.self_reach_avg)
        else:
            kw = {}
        b = SimpleNamespace(main=self._build_iter_args(**kw), regret=None, tiers=None)
        if self._items is not None:
            b.regret = (self._build_iter_args(self._items_regret, **kw), sum(self._items_regret.tiers))
            # one argument block per tier: the same lists entered behind the items of the tiers before
            b.tiers, first = [], 0
            for count in self._items.tiers:
                tier = self._build_iter_args(**kw)
                tier.root_parent_offsets += 8 * first
                tier.root_showdown_offsets += 8 * first
                tier.item_root += 8 * first
                tier.item_top += first
                b.tiers.append((tier, count))
                first += count
        self._iter_bundles[key] = b
        return b

    def _launch_iteration(self, phases: int, lean: bool = False, alternate: bool = False) -> None:
        """``phases``: 1 = regrets, policy, reach, beliefs; 2 = leaf values and backup; 3 = both.
        ``lean``: store only what is read again (include/p2hip.h).  ``alternate``: write reach_avg into
        the other of two buffers; ``self_reach_avg`` names the new one when this returns."""
        alternate = alternate and bool(phases & _PHASE_12)
        b = self._iter_bundle(alternate)
        mode = _PHASE_LEAN if lean else 0
        if self._items is None:
            self._launch_items(b.main, self.root_nodes, phases | mode)
        else:
            tiers = b.tiers
            if phases & _PHASE_12:
                self._launch_items(*b.regret, _PHASE_1 | mode)                      # regrets of every family, all items at once
                for args, count in tiers[:-1]:
                    self._launch_items(args, count, _PHASE_2 | mode)                # upper tiers, top-down
            args, count = tiers[-1]
            self._launch_items(args, count, (_PHASE_2 if phases & _PHASE_12 else 0) | (phases & _PHASE_3) | mode)
            if phases & _PHASE_3:
                for args, count in reversed(tiers[:-1]):
                    self._launch_items(args, count, _PHASE_3 | mode)                # the upper tiers' backup comes last
        if alternate:
            self.self_reach_avg, self._reach_avg_alt = self._reach_avg_alt, self.self_reach_avg

    def cfr_iteration(self, t: int, *, lean: bool = False, alternate_reach_avg: bool = False) -> None:
        """One CFR iteration (fused_sparse_cfr_evaluator.py:478-533).  The two keywords are for
        ``evaluate_cfr`` (one-kernel path only): ``lean`` leaves rows unwritten that nothing reads before
        the next iteration rewrites them — the state is complete again after one ordinary iteration —
        and ``alternate_reach_avg`` rebinds ``self_reach_avg`` to the other of two buffers."""
        if not self._skip_t_scalars_update:
            self.prepare_replay(t)
        if self.fused_iteration:
            if self._has_model_leaves and self.model is not None:
                self._launch_iteration(1, lean, alternate_reach_avg)
                self.set_leaf_values(t, showdown=False)
                self._launch_iteration(2, lean)
            else:
                self._launch_iteration(3, lean, alternate_reach_avg)
            return
        F.fused_sample_snapshot_(self.policy_probs_sample, self.policy_probs, self.t_sample, self._t_scalars.t_tensor)
        regrets = self.compute_instantaneous_regrets(self.latest_values)
        if self.cfr_type == CFRType.linear:
            regrets.masked_fill_(self.prev_actor[:, None] == t % self.num_players, 0.0)
            self.regret_weight_sums += 1
            self.cumulative_regrets += regrets
        else:
            F.fused_dcfr_update_with_tensors_(
                cumulative_regrets=self.cumulative_regrets, regret_weight_sums=self.regret_weight_sums,
                regrets=regrets, t_alpha_num=self._t_scalars.t_alpha_num, t_beta_num=self._t_scalars.t_beta_num,
                t_alpha_den=self._t_scalars.t_alpha_den, t_beta_den=self._t_scalars.t_beta_den,
                apply_dcfr=self.cfr_type in (CFRType.discounted, CFRType.discounted_plus), cfr_plus=self.cfr_plus)
        self.update_policy(t)
        self.set_leaf_values(t)
        self.compute_expected_values()
        if not self.use_final_policy_values:
            self.update_average_values(t)

    # ------------------------------------------------------------------ whole search
    @torch.no_grad()
    def initialize_policy_and_beliefs(self) -> None:
        """cfr_evaluator.py:830-886: initial policy from the model's logits (uniform over the
        legal actions without a model), beliefs pushed down level by level."""
        self.policy_probs.zero_()
        if self.tree_depth == 0:
            self._normalize_beliefs()
        for depth in range(self.tree_depth):
            o, on, onn = self.depth_offsets[depth], self.depth_offsets[depth + 1], self.depth_offsets[depth + 2]
            rows = torch.arange(o, on, device=self.device)
            if self.model is not None and hasattr(self.model, "policy_logits"):
                logits = self.model.policy_logits(self.beliefs, rows, self).to(self.float_dtype)
            else:
                logits = torch.zeros(on - o, NUM_HANDS, self.num_actions, dtype=self.float_dtype, device=self.device)
            legal = self.legal_mask[o:on][:, None, :]
            probs = torch.softmax(logits.masked_fill(~legal, float("-inf")), dim=-1)
            probs = torch.nan_to_num(probs, nan=0.0)
            probs.masked_fill_((self.child_count[o:on] == 0)[:, None, None], 0.0)
            src = probs.permute(0, 2, 1)  # [K, A, H]
            self.policy_probs[on:onn] = src[self.parent_index[on:onn] - o, self.action_from_parent[on:onn]]
            child = self.beliefs[self.parent_index[on:onn]].clone()
            idx = torch.arange(onn - on, device=self.device)
            child[idx, self.prev_actor[on:onn]] *= self.policy_probs[on:onn]
            self.beliefs[on:onn] = child
            self._normalize_beliefs()
        self._calculate_reach_weights(self.self_reach, self.policy_probs)
        self.policy_probs_avg[:] = self.policy_probs
        self.self_reach_avg[:] = self.self_reach
        self.beliefs_avg[:] = self.beliefs

    def warm_start(self) -> None:
        """Seed the regrets before the first iteration (cfr_evaluator.py:888-955).
        ``model``: regrets that make regret matching replay the initial (model) policy, weighted
        by the mean positive regret of each action.  ``model_br``: one best-response pass — the
        regret of every action against each player's best-response values, scaled by
        warm_start_iterations x warm_start_multiplier."""
        self.set_leaf_values(0)
        if not torch.isfinite(self.latest_values).all():
            raise ValueError("Non-finite values in latest_values after set_leaf_values")
        self.compute_expected_values(policy=self.policy_probs, beliefs=self.beliefs, leaf_values=self.latest_values,
                                     values=self.latest_values)
        if not torch.isfinite(self.latest_values).all():
            raise ValueError("Non-finite values in latest_values after compute_expected_values")
        self._record_initial_exploitability()
        t_ws = self.warm_start_iterations
        scale = float(t_ws) * self.warm_start_multiplier
        self.prepare_replay(t_ws)
        if self.warm_start_type == "model":
            bottom = self.depth_offsets[1]
            regrets = self.compute_instantaneous_regrets(self.latest_values)
            weights = scale * regrets[bottom:].clamp(min=0.0).mean(dim=-1)
            self.cumulative_regrets[bottom:] = self.policy_probs[bottom:] * weights[:, None]
            self.regret_weight_sums[bottom:] = weights[:, None]
            self.update_policy(t_ws)
            return
        br0 = self._best_response_values(self.policy_probs, self.beliefs, self.latest_values,
                                         torch.zeros_like(self.env.to_act))
        br1 = self._best_response_values(self.policy_probs, self.beliefs, self.latest_values,
                                         torch.ones_like(self.env.to_act))
        # (not meaningful on root rows, which take no part in the regrets)
        values_br = torch.where(self.prev_actor[:, None, None] == 0, br0, br1)
        regrets = self.compute_instantaneous_regrets(values_achieved=values_br, values_expected=self.latest_values)
        self.cumulative_regrets += scale * regrets
        self.regret_weight_sums += scale
        self.update_policy(t_ws)

    def _record_initial_exploitability(self) -> None:
        """cfr_evaluator.py:1618-1633 (mean over roots; no per-street split)."""
        if self._skip_record_stats:
            return
        self.stats["local_exploitability_init"] = self._compute_exploitability().local_exploitability.mean().item()

    def prepare_search(self, t_sample: torch.Tensor | None = None) -> None:
        """Everything ``evaluate_cfr`` does before its loop (cfr_evaluator.py:1505-1515)."""
        self.initialize_policy_and_beliefs()
        if self.warm_start_iterations > 0:
            self.warm_start()
        self.prepare_replay(0)
        self.set_leaf_values(0)
        self.compute_expected_values()
        self.values_avg[:] = self.latest_values
        if t_sample is None:
            t_sample = self._get_sampling_schedule()
        self.t_sample.copy_(t_sample.to(self.device))

    def evaluate_cfr(self, training_mode: bool = True) -> SampledLeaves:
        """cfr_evaluator.py:1497-1528 (statistics recording left out): the search, then the
        leaves from which the next searches continue."""
        self.prepare_search()
        self.run_search_iterations()
        if self.use_final_policy_values:
            self.update_average_values_final()
        return self.sample_leaves(training_mode)

    def run_search_iterations(self) -> None:
        """The loop of ``evaluate_cfr`` (cfr_evaluator.py:1516-1519).  Nobody looks at the state between
        its iterations, so with ``lean_search`` all but the last run lean, and reach_avg alternates
        between two buffers over an even number of iterations — it ends in the tensor it started in (an
        odd first iteration updates it in place).  The state afterwards is bit-identical to a loop of
        plain ``cfr_iteration`` calls."""
        ts = range(self.warm_start_iterations, self.cfr_iterations)
        lean = self.lean_search and self.fused_iteration
        for k, t in enumerate(ts):
            self.cfr_iteration(t, lean=lean and k + 1 < len(ts),
                               alternate_reach_avg=lean and not (len(ts) % 2 == 1 and k == 0))

    def update_average_values_final(self) -> None:
        """cfr_evaluator.py:1276-1292."""
        self.set_leaf_values(0, beliefs=self.beliefs_avg)
        self.compute_expected_values(self.policy_probs_avg, self.beliefs_avg, self.latest_values, self.values_avg)
        if self.enforce_zero_sum:
            s = (self.values_avg * self.beliefs_avg).sum(dim=2, keepdim=True).mean(dim=1, keepdim=True)
            s.masked_fill_(self.env.done[:, None, None], 0.0)
            self.values_avg -= s

    # ------------------------------------------------------------------ leaf sampling
    def _pull_back(self, tensor: torch.Tensor) -> torch.Tensor:
        """Child-aligned [total, ...] -> [top, num_actions, ...] action slices, zero where an
        action has no child (sparse_cfr_evaluator.py:465-489)."""
        top, bottom = self.depth_offsets[-2], self.depth_offsets[1]
        out = torch.zeros((top, self.num_actions, *tensor.shape[1:]), dtype=tensor.dtype, device=self.device)
        out[self.parent_index[bottom:], self.action_from_parent[bottom:]] = tensor[bottom:]
        return out

    def sample_leaves(self, training_mode: bool) -> SampledLeaves:
        """One leaf per root, sampled by walking down with ``policy_probs_sample`` for a hand
        drawn from the root actor's beliefs; with probability ``sample_epsilon`` the randomly
        chosen exploring player acts uniformly; terminal children are never entered
        (sparse_cfr_evaluator.py:325-426).  Host-side control flow on a handful of small tensors."""
        n, top = self.root_nodes, self.depth_offsets[-2]
        gen, dev = self.generator, self.device
        gdev = gen.device if gen is not None else dev      # draws happen where the generator lives

        def multinomial(p):
            return torch.multinomial(p.to(gdev), 1, generator=gen).squeeze(1).to(dev)
        players = torch.randint(0, 2, (n,), generator=gen, device=gdev).to(dev)
        sample_epsilon = self.sample_epsilon if training_mode else 0.0
        done_src = self._pull_back(self.env.done)
        sampling_masks = self.child_mask.clone()
        sampling_masks[:top] &= ~done_src
        sampling_counts = sampling_masks.float().sum(dim=-1, keepdim=True)
        uniform = torch.where(sampling_masks, 1 / sampling_counts, torch.zeros_like(sampling_counts))
        child_action_index = self.child_mask.int().cumsum(dim=1) - self.child_mask.int()
        effective_leaf = self.leaf_mask | (sampling_counts.squeeze(1) == 0)
        actor_beliefs = self.beliefs[:n].gather(
            1, self.env.to_act[:n, None, None].expand(-1, -1, NUM_HANDS)).squeeze(1)
        selected_hands = multinomial(actor_beliefs)
        # Only the column of each root's drawn hand is ever looked at: take it before pulling the
        # sampling policy back to [node, action] (the reference pulls back all 1326 columns).
        hand_of_node = selected_hands[self._root_index]
        probs_node = self.policy_probs_sample.gather(1, hand_of_node[:, None]).squeeze(1)
        probs_by_src = self._pull_back(probs_node)
        probs_by_src.masked_fill_(done_src, 0.0)
        denom = probs_by_src.sum(dim=1, keepdim=True)
        probs_by_src = torch.where(denom >= 1e-12, probs_by_src / denom, uniform[:top])
        sampled = torch.arange(n, device=dev)
        depth = 0
        active = ~effective_leaf[sampled]
        while bool(active.any()):
            _req(depth <= self.tree_depth, "depth <= self.tree_depth")
            nodes = sampled[active]
            to_act = self.env.to_act[nodes]
            explore = torch.rand(nodes.numel(), generator=gen, device=gdev).to(dev) < sample_epsilon
            explore &= to_act == players[active]
            actions = multinomial(torch.where(explore[:, None], uniform[nodes], probs_by_src[nodes]))
            sampled[active] = self.child_offsets[nodes] + child_action_index[nodes, actions]
            active = ~effective_leaf[sampled]
            depth += 1
        _req(bool(effective_leaf[sampled].all()) and not bool(self.env.done[sampled].any()),
             "bool(effective_leaf[sampled].all()) and not bool(self.env.done[sampled].any())")
        keep = sampled[sampled >= n]            # roots that are leaves themselves are not continued
        rows = keep.cpu().numpy()
        tree = self.tree
        root_of = tree.root_index[rows]
        # The cards a sampled leaf sees: a leaf that closed a betting round stands on the next
        # street, whose cards come from its root's runout (the reference env deals them from the
        # deck it was reset with, hunl_tensor_env.py:900-975); roots without one get theirs drawn here.
        if self._roots.runout is not None:
            runout = self._roots.runout[root_of]
        else:
            runout = self._draw_runout(tree.board[root_of])
        street = np.asarray(tree.state["street"])[rows]
        shown = np.arange(5)[None, :] < CARDS_ON_STREET[np.clip(street, 0, 4)][:, None]
        fields = {"board": np.where(shown, runout, -1), "last_board": tree.board[root_of].copy(), "runout": runout,
                  "bb": int(self.env.bb)}
        for name in RootStates.__dataclass_fields__:
            if name not in fields:
                fields[name] = np.asarray(tree.state[name])[rows]
        return SampledLeaves(nodes=keep, beliefs=self.beliefs[keep].clone(), roots=RootStates(**fields))

    def _draw_runout(self, boards: np.ndarray) -> np.ndarray:
        """Complete each board [K,5] to five cards with uniformly drawn cards that are not on it."""
        gen, dev = self.generator, self.device
        gdev = gen.device if gen is not None else dev
        b = torch.from_numpy(np.ascontiguousarray(boards)).to(gdev)
        k = b.shape[0]
        scores = torch.rand(k, 52, generator=gen, device=gdev)
        dealt = b >= 0
        scores[torch.arange(k, device=gdev)[:, None].expand(-1, 5)[dealt], b[dealt]] = -1.0
        fresh = torch.topk(scores, 5, dim=1).indices               # five distinct cards off the board, random order
        slot = (~dealt).long().cumsum(dim=1) - 1                    # which fresh card an empty slot takes
        out = torch.where(dealt, b, fresh.gather(1, slot.clamp(min=0)))
        return out.cpu().numpy()

    # ------------------------------------------------------------------ training data
    @property
    def chance_helper(self) -> ChanceNodeHelper:
        """Chance-node enumeration around the value network (sparse_cfr_evaluator.py:65-71).  The
        network is the leaf model's ``net`` (or the model itself when it maps features to an
        object with ``hand_values``)."""
        if self._chance_helper is None:
            helper = getattr(self.model, "helper", None)
            if not isinstance(helper, ChanceNodeHelper):
                net = getattr(self.model, "net", None)
                if net is None and callable(self.model):
                    net = self.model
                if net is None:
                    raise RuntimeError("pre-chance value targets need a value network (model.net)")
                helper = ChanceNodeHelper(self.device, self.float_dtype, self.num_players, net,
                                          generator=self.generator,
                                          autocast_dtype=getattr(self.model, "autocast_dtype", None))
            self._chance_helper = helper
        return self._chance_helper

    def _policy_targets(self, rows: torch.Tensor, check_rows: bool = True) -> torch.Tensor:
        """[K, 1326, num_actions]: the average policy of the children of ``rows`` by action, zero
        for actions without a child (cfr_evaluator.py:1392-1393 on the selected rows)."""
        rows = rows.to(device=self.device, dtype=torch.int64).contiguous()
        if check_rows and rows.numel() and bool(((rows < 0) | (rows >= self.total_nodes)).any()):
            raise IndexError("policy target rows out of range")
        out = torch.empty(rows.numel(), NUM_HANDS, self.num_actions, dtype=self.float_dtype, device=self.device)
        _lib.call("p2hip_policy_targets", _lib.ptr(self.policy_probs_avg), _lib.ptr(rows), rows.numel(),
                  _lib.ptr(self.child_offsets), _lib.ptr(self.child_count), _lib.ptr(self.action_from_parent),
                  self.num_actions, _lib.ptr(out), _lib.stream_ptr())
        return out

    @torch.no_grad()
    def training_data(self, exclude_start: bool = True) -> tuple[RebelBatch, RebelBatch, RebelBatch]:
        """(value batch, pre-chance value batch, policy batch) of a finished search
        (cfr_evaluator.py:1383-1495).  Value targets: the roots' average values clamped to
        [-1, 1].  Policy targets: the average policy of every expanded node, [node, hand, action].
        Roots standing at the start of a betting round after a deal also give a sample for the
        state BEFORE that deal: its value is the network's answer averaged over the cards that
        could have come (single card on turn and river, canonical flops on the flop)."""
        N = self.root_nodes
        top = self.depth_offsets[-2] if len(self.depth_offsets) > 1 else N
        dev = self.device
        value_targets = self.values_avg[:N].clamp(-1.0, 1.0)
        features = self.feature_encoder.encode(self.beliefs_avg, pre_chance_node=False,
                                               indices=torch.arange(top, device=dev))
        bin_amounts, legal_masks = self.env.legal_bins_amounts_and_mask()
        statistics = {"to_act": self.env.to_act, "street": self.env.street, "stage": 2 * self.env.street,
                      "board": self.env.board_indices, "pot": self.env.pot, "bet_amounts": bin_amounts}
        exploit_stats = self._compute_exploitability()
        value_statistics = {k: v[:N] for k, v in statistics.items()}
        value_statistics["local_exploitability"] = exploit_stats.local_exploitability
        value_statistics["local_best_response_values"] = exploit_stats.local_best_response_values
        valid_top = self.valid_mask[:top] & ~self.leaf_mask[:top]
        policy_rows = torch.nonzero(valid_top).squeeze(1)
        policy_statistics = {k: v[:top][valid_top] for k, v in statistics.items()}
        value_batch = RebelBatch(features=features[:N], value_targets=value_targets, legal_masks=legal_masks[:N],
                                 statistics=value_statistics)
        street_root = self.env.street[:N]
        actions_root = self.env.actions_this_round[:N]
        if exclude_start:
            value_batch = value_batch[~((street_root == 0) & (actions_root == 0))]
        elif self.reuse_state:
            # the features of all roots would be a view of the state, which the next subgame overwrites
            value_batch = value_batch[torch.arange(N, device=dev)]
        policy_batch = RebelBatch(features=features[valid_top], policy_targets=self._policy_targets(policy_rows, check_rows=False),
                                  legal_masks=legal_masks[:top][valid_top], statistics=policy_statistics)

        pre_features_root = self.feature_encoder.encode(self.beliefs, pre_chance_node=True,
                                                        indices=torch.arange(N, device=dev)).clone()
        pre_features_root.beliefs = self.root_pre_chance_beliefs[:N].reshape(N, -1).clone()
        value_targets_pre = value_targets.clone()
        value_statistics_pre = {k: v.clone() for k, v in value_statistics.items()}
        value_statistics_pre["board"] = self.env.last_board_indices[:N].clone()
        prev_street = torch.where((street_root > 0) & (street_root < 4) & (actions_root == 0), street_root - 1,
                                  street_root)
        value_statistics_pre["street"] = prev_street
        value_statistics_pre["stage"] = 2 * prev_street + 1
        start_mask = actions_root == 0
        turn_river_mask = start_mask & ((street_root == 2) | (street_root == 3))
        if bool(turn_river_mask.any()):
            value_targets_pre[turn_river_mask] = self.chance_helper.single_card_chance_values(
                torch.where(turn_river_mask)[0], features[:N], self.root_pre_chance_beliefs,
                self.env.last_board_indices[:N])
        flop_mask = start_mask & (street_root == 1)
        if bool(flop_mask.any()):
            value_targets_pre[flop_mask] = self.chance_helper.flop_chance_values(
                torch.where(flop_mask)[0], features[:N], self.root_pre_chance_beliefs)
        transition_mask = turn_river_mask | flop_mask
        pre_value_batch = RebelBatch(features=pre_features_root, value_targets=value_targets_pre,
                                     legal_masks=legal_masks[:N], statistics=value_statistics_pre)[transition_mask]
        return value_batch, pre_value_batch, policy_batch

    # ------------------------------------------------------------------ best response
    def _fan_out_deep(self, per_root: torch.Tensor) -> torch.Tensor:
        """Per-root values repeated on every node of the root's subtree (sparse_cfr_evaluator.py:504-523)."""
        return per_root.index_select(0, self._root_index)

    def _best_response_values(self, policy: torch.Tensor, beliefs: torch.Tensor, base_values: torch.Tensor,
                              deviating_player: torch.Tensor | None = None) -> torch.Tensor:
        """Values when ``deviating_player`` (per node; default: the root's player to act) plays a
        per-hand best response and the other player follows ``policy``
        (cfr_evaluator.py:603-716).  One kernel launch per tree level, deepest first."""
        n = self.root_nodes
        if deviating_player is None:
            deviating_player = self._fan_out_deep(self.env.to_act[:n])
        deviating_player = deviating_player.to(device=self.device, dtype=torch.int64).contiguous()
        _req(deviating_player.shape == (self.total_nodes,), "deviating_player.shape == (self.total_nodes,)")
        policy = policy.contiguous()
        beliefs = beliefs.contiguous()
        values_br = torch.where(self.leaf_mask[:, None, None], base_values, torch.zeros_like(base_values)).contiguous()
        for depth in range(self.tree_depth - 1, -1, -1):
            base, end = self.depth_offsets[depth], self.depth_offsets[depth + 1]
            _lib.call("p2hip_best_response_level", _lib.ptr(values_br), _lib.ptr(policy), _lib.ptr(beliefs),
                      _lib.ptr(self.env.to_act), _lib.ptr(deviating_player), _lib.ptr(self.child_offsets),
                      _lib.ptr(self.child_count), int(base), int(end - base), int(self._max_children),
                      _lib.stream_ptr())
        return values_br

    def _compute_exploitability(self) -> ExploitabilityStats:
        """Gain of a per-hand best response over the average strategy, per root, summed over the
        two players and weighted by the root beliefs (cfr_evaluator.py:718-764)."""
        n = self.root_nodes
        if n == 0:
            return ExploitabilityStats(torch.empty(0, device=self.device, dtype=self.float_dtype),
                                       torch.empty(0, 2, device=self.device, dtype=self.float_dtype))
        policy, beliefs = self.policy_probs_avg, self.beliefs_avg
        leaf_values = self.values_avg.clamp(-1.0, 1.0)
        base_values = torch.zeros_like(leaf_values)
        self.compute_expected_values(policy=policy, beliefs=beliefs, leaf_values=leaf_values, values=base_values)
        improvements, br_agg = [], []
        for player in range(2):
            deviator = torch.full((n,), player, device=self.device, dtype=torch.int64)
            br = self._best_response_values(policy, beliefs, leaf_values, self._fan_out_deep(deviator))
            root_beliefs = beliefs[:n, player]
            improvements.append(((br[:n, player] - base_values[:n, player]) * root_beliefs).sum(dim=-1))
            br_agg.append((br[:n, player] * root_beliefs).sum(dim=-1))
        return ExploitabilityStats(local_exploitability=improvements[0] + improvements[1],
                                   local_best_response_values=torch.stack(br_agg, dim=-1))

    def state_dict(self) -> dict:
        return {n: getattr(self, n) for n in STATE_NAMES}


class _EvaluatorStateSnapshot:
    """Copies of the 11 tensors an iteration mutates, to rewind an evaluator or to compare two
    runs (the helper the reference keeps beside its graph runner, fused_cfr_triton.py:2322-2356:
    ``from_evaluator``, ``restore_to``, ``max_abs_diff``, fields ``names`` and ``tensors``)."""

    def __init__(self, saved: dict) -> None:
        self._saved = dict(saved)

    @property
    def names(self) -> tuple:
        return tuple(self._saved)

    @property
    def tensors(self) -> tuple:
        return tuple(self._saved.values())

    @classmethod
    def from_evaluator(cls, evaluator) -> "_EvaluatorStateSnapshot":
        return cls({name: getattr(evaluator, name).detach().clone() for name in STATE_NAMES})

    def restore_to(self, evaluator) -> None:
        for name, kept in self._saved.items():
            getattr(evaluator, name).copy_(kept)

    def max_abs_diff(self, other: "_EvaluatorStateSnapshot") -> dict:
        _req(self.names == other.names, "snapshots hold different tensors")
        return {name: (mine - theirs).abs().max().item()
                for (name, mine), theirs in zip(self._saved.items(), other.tensors)}


class GraphedCFRIteration:
    """Captures ``evaluator.cfr_iteration`` into a HIP graph and replays it for any ``t``
    (src/p2/search/fused_cfr_triton.py:2359-2451).  The iteration-dependent scalars live in
    device memory and are refreshed by ``prepare_replay`` outside the graph."""

    def __init__(self, evaluator: HipSparseCFREvaluator) -> None:
        if evaluator.device.type != "cuda":
            raise ValueError("GraphedCFRIteration requires a GPU evaluator.")
        self.evaluator = evaluator
        self._graph = None
        self._captured_t = None

    def capture(self, t_capture: int, num_warmup: int = 2) -> None:
        ev = self.evaluator
        for i in range(num_warmup):
            ev.cfr_iteration(t_capture + i)
        ev.prepare_replay(t_capture)
        prev = ev._skip_t_scalars_update
        ev._skip_t_scalars_update = True
        try:
            s = torch.cuda.Stream()
            s.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(s):
                ev.cfr_iteration(t_capture)
            torch.cuda.current_stream().wait_stream(s)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=s):
                ev.cfr_iteration(t_capture)
        finally:
            ev._skip_t_scalars_update = prev
        self._graph = graph
        self._captured_t = t_capture

    def replay(self, t: int | None = None) -> None:
        if self._graph is None:
            raise RuntimeError("capture() must be called before replay().")
        if t is not None:
            self.evaluator.prepare_replay(t)
        self._graph.replay()

    @property
    def captured_t(self):
        return self._captured_t
