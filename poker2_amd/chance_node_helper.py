"""Chance-node enumeration around the leaf value network, MI355X path.

Mirror of ``ChanceNodeHelper.single_card_chance_values``
(src/p2/search/chance_node_helper.py:360-479) and of the ``MLPFeatures`` container it hands
to the network (src/p2/models/mlp/mlp_features.py:13-62): same names, arguments, sample
order (state-major, next card ascending) and return value.  The masking / renormalising
expansion and the per-state mean run as HIP kernels (``p2hip_chance_expand``,
``p2hip_chance_mean``); the network itself stays an ordinary PyTorch module.
``flop_chance_values`` (three-card chance nodes, :219-357) enumerates or samples the 1755
suit-canonical flops (:76-216), expands through ``p2hip_flop_expand`` and averages each flop's
answers over its suit orbit with ``p2hip_perm_mean``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

import numpy as np

from . import _lib
from .card_utils import NUM_HANDS, combo_suit_permutation_tensor, suit_permutations_tensor
from ._guards import require as _req


@dataclass
class MLPFeatures:
    """Feature bundle of the value network (src/p2/models/mlp/mlp_features.py:13-62)."""

    context: torch.Tensor   # [N, C]
    street: torch.Tensor    # [N]
    to_act: torch.Tensor    # [N]
    board: torch.Tensor     # [N, 5] card ids, -1 = not dealt
    beliefs: torch.Tensor   # [N, 2 * 1326]

    def __post_init__(self) -> None:
        n = self.context.shape[0]
        _req(self.street.shape == (n,), "self.street.shape == (n,)")
        _req(self.to_act.shape == (n,), "self.to_act.shape == (n,)")
        _req(self.board.shape == (n, 5), "self.board.shape == (n, 5)")
        _req(self.beliefs.shape == (n, 2 * NUM_HANDS), "self.beliefs.shape == (n, 2 * NUM_HANDS)")

    def __len__(self) -> int:
        return self.context.shape[0]

    def __getitem__(self, index) -> "MLPFeatures":
        return MLPFeatures(context=self.context[index], street=self.street[index], to_act=self.to_act[index],
                           board=self.board[index], beliefs=self.beliefs[index])

    def to(self, device) -> "MLPFeatures":
        return MLPFeatures(context=self.context.to(device), street=self.street.to(device),
                           to_act=self.to_act.to(device), board=self.board.to(device),
                           beliefs=self.beliefs.to(device))

    def clone(self) -> "MLPFeatures":
        return MLPFeatures(context=self.context.clone(), street=self.street.clone(), to_act=self.to_act.clone(),
                           board=self.board.clone(), beliefs=self.beliefs.clone())

    @classmethod
    def cat(cls, features_list: list["MLPFeatures"]) -> "MLPFeatures":
        if not features_list:
            raise ValueError("Cannot concatenate an empty list of features.")
        return cls(context=torch.cat([f.context for f in features_list], dim=0),
                   street=torch.cat([f.street for f in features_list], dim=0),
                   to_act=torch.cat([f.to_act for f in features_list], dim=0),
                   board=torch.cat([f.board for f in features_list], dim=0),
                   beliefs=torch.cat([f.beliefs for f in features_list], dim=0))


def _rows_out_of_range(rows: torch.Tensor, n: int) -> bool:
    """One device read: does any index lie outside 0..n-1?"""
    return bool(rows.numel()) and bool(((rows < 0) | (rows >= n)).any())


INPUT_ROW_WIDTH = 2 * NUM_HANDS + 52       # [ranges of both players | one-hot of the board]
_INPUT_DTYPES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}


def chance_expand(pre_chance_beliefs: torch.Tensor, root_indices: torch.Tensor, board_pre: torch.Tensor,
                  cards_on_board: int | None = None, check_rows: bool = True, input_dtype: torch.dtype | None = None):
    """Every (state, next card) sample of a single-card chance node.

    ``input_dtype`` (float32 / bfloat16 / float16): the samples are written as rows of a value network's
    input matrix instead — first return value [S, 2704] in that dtype, each row the sample's ranges
    followed by the 52-entry one-hot of its board — for networks whose input is exactly that
    (``RangeBoardMLP``): no concatenation and no cast in front of the network.

    pre_chance_beliefs [R,2,1326] fp32, board_pre [R,5] int64 (-1 = empty), root_indices [B].
    Returns (post_beliefs [S,2,1326], board_samples [S,5], root_lookup [S], sample_offsets [B+1])
    with samples in (state, card) ascending order.  ``cards_on_board`` (same count for every
    selected state) skips the device-to-host read of the sample count; ``check_rows=False`` skips the
    one that checks ``root_indices`` (for callers whose indices are valid by construction; the kernel
    itself leaves rows outside the table alone).
    """
    if not _lib.hip_is_available():
        raise RuntimeError("chance_expand needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(pre_chance_beliefs, "chance_expand")
    dev = pre_chance_beliefs.device
    _req(pre_chance_beliefs.dim() == 3 and tuple(pre_chance_beliefs.shape[1:]) == (2, NUM_HANDS),
         "pre_chance_beliefs.dim() == 3 and tuple(pre_chance_beliefs.shape[1:]) == (2, NUM_HANDS)")
    _req(board_pre.dim() == 2 and board_pre.shape[1] == 5, "board_pre.dim() == 2 and board_pre.shape[1] == 5")
    pre = pre_chance_beliefs.contiguous().float()
    board = board_pre.to(device=dev, dtype=torch.int64).contiguous()
    roots = root_indices.to(device=dev, dtype=torch.int64).contiguous()
    b = roots.numel()
    source_rows = min(pre.shape[0], board.shape[0])
    if check_rows and _rows_out_of_range(roots, source_rows):
        raise IndexError("root_indices out of range")
    if cards_on_board is None:
        on_board = ((board[roots] >= 0) & (board[roots] < 52)).sum(dim=1)
        offsets = torch.zeros(b + 1, dtype=torch.int64, device=dev)
        torch.cumsum(52 - on_board, dim=0, out=offsets[1:])
        if b and int(on_board.max().item()) >= 5:
            raise ValueError("single-card chance expansion needs an empty board slot (at most 4 cards dealt)")
        total = int(offsets[-1].item()) if b else 0
    else:
        if not 0 <= cards_on_board <= 4:
            raise ValueError("cards_on_board must be in 0..4")
        per_state = 52 - cards_on_board
        total = b * per_state
        offsets = torch.arange(0, total + 1, per_state, dtype=torch.int64, device=dev)   # one launch, no board read
    # With ``cards_on_board`` given the sample count is taken on trust; the kernel gets the buffers'
    # size and writes nothing beyond it if a board holds fewer cards than claimed.  Where a state has
    # fewer samples than its share of the buffers (a board with MORE cards than claimed, no empty slot,
    # or a row outside the table with check_rows=False) the kernel fills the rest of the share with zeros
    # (root_lookup = the state): what a wrong claim leaves behind is defined, never uninitialised memory.
    alloc = torch.empty
    board_samples = alloc(total, 5, dtype=torch.int64, device=dev)
    root_lookup = alloc(total, dtype=torch.int64, device=dev)
    if input_dtype is not None:
        _req(input_dtype in _INPUT_DTYPES, "input_dtype: float32, bfloat16 or float16")
        rows = alloc(total, INPUT_ROW_WIDTH, dtype=input_dtype, device=dev)
        _req(pre.data_ptr() % 16 == 0 and rows.data_ptr() % 16 == 0, "16-byte aligned ranges and input matrix")
        _lib.call("p2hip_chance_expand_input", _lib.ptr(pre), _lib.ptr(roots), _lib.ptr(board), b, _lib.ptr(offsets),
                  source_rows, total, _lib.ptr(rows), _INPUT_DTYPES[input_dtype], _lib.ptr(board_samples),
                  _lib.ptr(root_lookup), _lib.stream_ptr())
        return rows, board_samples, root_lookup, offsets
    post = alloc(total, 2, NUM_HANDS, dtype=torch.float32, device=dev)
    _lib.call("p2hip_chance_expand", _lib.ptr(pre), _lib.ptr(roots), _lib.ptr(board), b, _lib.ptr(offsets),
              source_rows, total, _lib.ptr(post), _lib.ptr(board_samples), _lib.ptr(root_lookup),
              _lib.stream_ptr())
    return post, board_samples, root_lookup, offsets


def chance_mean(hand_values: torch.Tensor, sample_offsets: torch.Tensor) -> torch.Tensor:
    """[S,2,1326] network outputs -> [B,2,1326] mean over each state's samples."""
    if not _lib.hip_is_available():
        raise RuntimeError("chance_mean needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(hand_values, "chance_mean")
    _req(hand_values.dim() == 3 and tuple(hand_values.shape[1:]) == (2, NUM_HANDS),
         "hand_values.dim() == 3 and tuple(hand_values.shape[1:]) == (2, NUM_HANDS)")
    hv = hand_values.contiguous().float()
    offsets = sample_offsets.to(device=hv.device, dtype=torch.int64).contiguous()
    b = offsets.numel() - 1
    out = torch.empty(b, 2, NUM_HANDS, dtype=torch.float32, device=hv.device)
    _lib.call("p2hip_chance_mean", _lib.ptr(hv), _lib.ptr(offsets), b, _lib.ptr(out), _lib.stream_ptr())
    return out


def flop_expand(pre_chance_beliefs: torch.Tensor, root_indices: torch.Tensor, flops: torch.Tensor,
                check_rows: bool = True) -> torch.Tensor:
    """pre_chance_beliefs [R,2,1326] fp32, root_indices [B], flops [K,3] card ids ->
    [B,K,2,1326]: the ranges of each selected state without the hands that touch each flop,
    renormalised per player (uniform over the 1176 hands left where the sum is <= 1e-12).
    ``check_rows=False`` skips the device read that checks ``root_indices`` (the kernel does not check them)."""
    if not _lib.hip_is_available():
        raise RuntimeError("flop_expand needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(pre_chance_beliefs, "flop_expand")
    dev = pre_chance_beliefs.device
    _req(pre_chance_beliefs.dim() == 3 and tuple(pre_chance_beliefs.shape[1:]) == (2, NUM_HANDS),
         "pre_chance_beliefs.dim() == 3 and tuple(pre_chance_beliefs.shape[1:]) == (2, NUM_HANDS)")
    _req(flops.dim() == 2 and flops.shape[1] == 3, "flops.dim() == 2 and flops.shape[1] == 3")
    pre = pre_chance_beliefs.contiguous().float()
    roots = root_indices.to(device=dev, dtype=torch.int64).contiguous()
    if check_rows and _rows_out_of_range(roots, pre.shape[0]):
        raise IndexError("root_indices out of range")
    fl = flops.to(device=dev, dtype=torch.int64).contiguous()
    b, k = roots.numel(), fl.shape[0]
    post = torch.empty(b, k, 2, NUM_HANDS, dtype=torch.float32, device=dev)
    _lib.call("p2hip_flop_expand", _lib.ptr(pre), _lib.ptr(roots), b, _lib.ptr(fl), k, _lib.ptr(post),
              _lib.stream_ptr())
    return post


# Workgroups wanted from the (state, player) x share split of the flop means.  perm_mean is a pure read stream
# (the permutations are applied once per workgroup, to the summed rows) and fastest with few, long workgroups:
# 64 states x 256 flops 48.6 us with one share (128 workgroups), 30.5 us with three (384), 32.3 us with eight,
# 44.2 us with 32; 1024 states 475 us with one share, 505 us with two.  orbit_mean goes through LDS per row and
# wants the chip filled once (1024 states x 256 flops: 470 us with one share against 494 us with two; 64
# states: 32.8 us with eight shares).
PERM_MEAN_TARGET_WORKGROUPS = 384
ORBIT_MEAN_TARGET_WORKGROUPS = 2048   # 256 CUs x 8


def perm_mean(hand_values: torch.Tensor, perms: torch.Tensor, weight: torch.Tensor,
              out: torch.Tensor | None = None, check_perms: bool = True) -> torch.Tensor:
    """hand_values [B,K,2,1326] fp32, perms [P,1326] hand-index maps (P <= 24), weight [K] ->
    [B,2,1326]: sum_k weight[k] * mean_q hand_values[b,k,p,perms[q,h]]; added to ``out`` if given."""
    if not _lib.hip_is_available():
        raise RuntimeError("perm_mean needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(hand_values, "perm_mean")
    dev = hand_values.device
    _req(hand_values.dim() == 4 and tuple(hand_values.shape[2:]) == (2, NUM_HANDS),
         "hand_values.dim() == 4 and tuple(hand_values.shape[2:]) == (2, NUM_HANDS)")
    _req(perms.dim() == 2 and perms.shape[1] == NUM_HANDS and 1 <= perms.shape[0] <= 24,
         "perms.dim() == 2 and perms.shape[1] == NUM_HANDS and 1 <= perms.shape[0] <= 24")
    b, k = hand_values.shape[0], hand_values.shape[1]
    _req(weight.shape == (k,), "weight.shape == (k,)")
    hv = hand_values.contiguous().float()
    if check_perms and (int(perms.min()) < 0 or int(perms.max()) >= NUM_HANDS):   # two device reads: skip for known tables
        raise IndexError("perms must map hands to hand indices 0..1325")
    pt = perms.to(device=dev, dtype=torch.int16).contiguous()
    w = weight.to(device=dev, dtype=torch.float32).contiguous()
    accumulate = out is not None
    if out is None:
        out = torch.empty(b, 2, NUM_HANDS, dtype=torch.float32, device=dev)
    else:
        _req(out.shape == (b, 2, NUM_HANDS) and out.dtype == torch.float32 and out.is_contiguous(),
             "out.shape == (b, 2, NUM_HANDS) and out.dtype == torch.float32 and out.is_contiguous()")
    # enough workgroups to fill the chip: 2 per state, times shares of the flops
    shares = max(1, min(k, -(-PERM_MEAN_TARGET_WORKGROUPS // max(1, 2 * b))))
    workspace = torch.empty(shares, b, 2, NUM_HANDS, dtype=torch.float32, device=dev) if shares > 1 else None
    _lib.call("p2hip_perm_mean", _lib.ptr(hv), b, k, _lib.ptr(pt), int(pt.shape[0]), _lib.ptr(w), int(accumulate),
              _lib.ptr(out), _lib.ptr(workspace), shares, _lib.stream_ptr())
    return out


def _avg_over_perms(hand_values: torch.Tensor, perms: torch.Tensor) -> torch.Tensor:
    """Mean over the rows of ``perms`` [P, 1326] of ``hand_values[..., perms[q]]`` for values of
    any leading shape (chance_node_helper.py:17-27).  Runs ``perm_mean`` with a single flop of
    weight 1; the rows are taken in pairs, which is only a launch shape here."""
    _req(hand_values.shape[-1] == NUM_HANDS, "hand_values.shape[-1] == 1326")
    lead = hand_values.shape[:-1]
    rows = hand_values.reshape(-1, NUM_HANDS).float()
    n = rows.shape[0]
    if n == 0:
        return rows.reshape(*lead, NUM_HANDS)
    if n % 2:
        rows = torch.cat([rows, rows.new_zeros(1, NUM_HANDS)])
    one = torch.ones(1, dtype=torch.float32, device=rows.device)
    mean = perm_mean(rows.view(-1, 1, 2, NUM_HANDS), perms, one)
    return mean.view(-1, NUM_HANDS)[:n].reshape(*lead, NUM_HANDS)


ORBIT_SCRATCH_FLOATS = 4 * 1024 * 1024     # P2HIP_ORBIT_SCRATCH_FLOATS of include/p2hip.h


def orbit_mean(hand_values: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None, *,
               static_scratch: bool = False) -> torch.Tensor:
    """``perm_mean`` over ALL 24 suit permutations: the orbit of a hand is its class of starting
    hands (pair / suited / offsuit of the same ranks), so the mean is taken per class.

    ``static_scratch=True`` (needs ``out``) takes the entry point that allocates nothing
    (``p2hip_orbit_mean_static``): partial sums go to a 16 MiB array inside the library, so the
    call can sit under graph capture; it refuses inputs whose partial sums do not fit and must
    not overlap with another such call on the same GPU.  The first such call on a device resolves the
    array's address there and must itself run outside capture: ``orbit_scratch_init()`` is that call."""
    if not _lib.hip_is_available():
        raise RuntimeError("orbit_mean needs libp2hip.so and a GPU (no CPU fallback exists).")
    _lib.require_gpu(hand_values, "orbit_mean")
    dev = hand_values.device
    _req(hand_values.dim() == 4 and tuple(hand_values.shape[2:]) == (2, NUM_HANDS),
         "hand_values.dim() == 4 and tuple(hand_values.shape[2:]) == (2, NUM_HANDS)")
    b, k = hand_values.shape[0], hand_values.shape[1]
    _req(weight.shape == (k,), "weight.shape == (k,)")
    hv = hand_values.contiguous().float()
    w = weight.to(device=dev, dtype=torch.float32).contiguous()
    accumulate = out is not None
    if out is None:
        out = torch.empty(b, 2, NUM_HANDS, dtype=torch.float32, device=dev)
    else:
        _req(out.shape == (b, 2, NUM_HANDS) and out.dtype == torch.float32 and out.is_contiguous(),
             "out.shape == (b, 2, NUM_HANDS) and out.dtype == torch.float32 and out.is_contiguous()")
    shares = max(1, min(k, -(-ORBIT_MEAN_TARGET_WORKGROUPS // max(1, 2 * b))))
    if static_scratch:
        if not accumulate:
            raise ValueError("static_scratch=True allocates nothing: pass the output tensor as `out`")
        if hv is not hand_values or w is not weight:
            raise ValueError("static_scratch=True allocates nothing: hand_values and weight must already be "
                             "contiguous float32 tensors on the GPU")
        if shares > 1 and shares * b * 2 * NUM_HANDS > ORBIT_SCRATCH_FLOATS:
            raise ValueError(f"{shares} shares x {b} states need {shares * b * 2 * NUM_HANDS} floats of partial sums; "
                             f"the library's static array holds {ORBIT_SCRATCH_FLOATS}")
        _lib.call("p2hip_orbit_mean_static", _lib.ptr(hv), b, k, _lib.ptr(w), 1, _lib.ptr(out), shares,
                  _lib.stream_ptr())
        return out
    workspace = torch.empty(shares, b, 2, NUM_HANDS, dtype=torch.float32, device=dev) if shares > 1 else None
    _lib.call("p2hip_orbit_mean", _lib.ptr(hv), b, k, _lib.ptr(w), int(accumulate), _lib.ptr(out),
              _lib.ptr(workspace), shares, _lib.stream_ptr())
    return out


def orbit_scratch_init() -> None:
    """Resolve the static scratch array of ``p2hip_orbit_mean_static`` on the current device (once per device,
    outside graph capture); launches nothing."""
    _lib.call("p2hip_orbit_mean_static", None, 0, 0, None, 0, None, 1, _lib.stream_ptr())


def canonical_flops():
    """The suit-canonical flops (src/p2/search/chance_node_helper.py:76-216), on the host.

    Every flop's cards are ordered by rank, high first; under each of the 24 suit permutations
    the suits of equal ranks are put in ascending order and the three cards are read as a base-52
    number; the smallest number over the permutations is the flop's canonical form.  Returns
    (canonical [1755,3] int64 cards in that order, count [1755] int64 flops per class,
    flop_to_class [22100] int64 in itertools.combinations order, board_to_flop_id [52,52,52] int64
    with -1 off the c0 < c1 < c2 entries)."""
    from itertools import combinations
    flops = np.array(list(combinations(range(52), 3)), dtype=np.int64)            # [22100, 3], ascending ids
    ranks, suits = flops % 13, flops // 13
    order = np.argsort(-ranks, axis=1, kind="stable")
    ranks_s = np.take_along_axis(ranks, order, axis=1)
    perms = suit_permutations_tensor().numpy()                                     # [24, 4]
    suits_p = np.take_along_axis(perms[:, suits], np.broadcast_to(order, (24,) + order.shape), axis=2)  # [24,N,3]
    eq01, eq12 = ranks_s[:, 0] == ranks_s[:, 1], ranks_s[:, 1] == ranks_s[:, 2]
    all_eq, first2, last2 = eq01 & eq12, eq01 & ~eq12, eq12 & ~eq01
    suits_p[:, all_eq, :] = np.sort(suits_p[:, all_eq, :], axis=2)
    suits_p[:, first2, :2] = np.sort(suits_p[:, first2, :2], axis=2)
    suits_p[:, last2, 1:] = np.sort(suits_p[:, last2, 1:], axis=2)
    cards = suits_p * 13 + ranks_s[None]
    code = cards[..., 0] * 2704 + cards[..., 1] * 52 + cards[..., 2]               # [24, N]
    best = code.min(axis=0)
    unique, flop_to_class = np.unique(best, return_inverse=True)
    canonical = np.stack([unique // 2704, (unique // 52) % 52, unique % 52], axis=1).astype(np.int64)
    count = np.bincount(flop_to_class, minlength=unique.shape[0]).astype(np.int64)
    board_to_flop_id = np.full((52, 52, 52), -1, dtype=np.int64)
    board_to_flop_id[flops[:, 0], flops[:, 1], flops[:, 2]] = flop_to_class
    return canonical, count, flop_to_class.astype(np.int64), board_to_flop_id


class ChanceNodeHelper:
    """Utilities for enumerating chance nodes when generating value targets
    (src/p2/search/chance_node_helper.py:31-75)."""

    FLOP_CHUNK_SIZE = 128
    # Canonical flops drawn per call with probability proportional to their class size; 0 = all
    # 1755 classes, weighted by class size, in chunks of FLOP_CHUNK_SIZE (:36-38)
    FLOP_SAMPLE_SIZE = 256
    # Suit permutations averaged per flop; 0 or >= 24 = the whole orbit (:39-42)
    NUM_PERM_SAMPLES = 6

    def __init__(self, device: torch.device, float_dtype: torch.dtype, num_players: int, model: Any,
                 generator: torch.Generator | None = None, autocast_dtype: torch.dtype | None = torch.float16) -> None:
        if num_players != 2:
            raise ValueError("heads-up only: num_players must be 2")
        self.device = torch.device(device)
        self.float_dtype = float_dtype
        self.num_players = num_players
        self.model = model
        self.generator = generator
        self.autocast_dtype = autocast_dtype   # the reference runs the network under fp16 autocast (:460)
        self.suit_permutations = suit_permutations_tensor(device=self.device)
        self.num_permutations = self.suit_permutations.shape[0]
        self.combo_perm = combo_suit_permutation_tensor(device=self.device)
        self._combo_perm_i16 = self.combo_perm.to(torch.int16).contiguous()
        canonical, count, flop_to_class, board_to_flop_id = canonical_flops()
        self.flop_id_to_canonical = torch.from_numpy(canonical).to(self.device)
        self.flop_id_to_count = torch.from_numpy(count).to(self.device)
        self.board_to_flop_id = torch.from_numpy(board_to_flop_id).to(self.device)
        self.flop_to_canon = torch.from_numpy(flop_to_class).to(self.device)
        self.total_flop_count = int(count.sum())

    def _run_model(self, features: MLPFeatures) -> torch.Tensor:
        model = self.model
        if hasattr(model, "eval"):
            model.eval()
        if self.autocast_dtype is not None:
            with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                hand_values = model(features).hand_values
        else:
            hand_values = model(features).hand_values
        return hand_values.to(torch.float32)

    @torch.no_grad()
    def flop_chance_values(self, root_indices: torch.Tensor, root_features: MLPFeatures,
                           pre_chance_beliefs: torch.Tensor) -> torch.Tensor:
        """Expected network values over the three-card flop chance node (:219-357): the canonical
        flops (all of them weighted by class size, or FLOP_SAMPLE_SIZE drawn in proportion to it),
        each answer averaged over NUM_PERM_SAMPLES suit permutations of the hands (all 24 if 0)."""
        if not _lib.hip_is_available():
            raise RuntimeError("flop_chance_values needs libp2hip.so and a GPU (no CPU fallback exists).")
        if root_indices.numel() == 0:
            return torch.zeros(0, self.num_players, NUM_HANDS, device=self.device, dtype=self.float_dtype)
        dev = self.device
        roots = root_indices.to(device=dev, dtype=torch.int64).contiguous()
        b = roots.numel()
        pre = pre_chance_beliefs.to(device=dev).contiguous().float()
        _lib.require_gpu(pre, "flop_chance_values")
        if _rows_out_of_range(roots, pre.shape[0]):          # once, not per chunk of flops
            raise IndexError("root_indices out of range")
        context_root = root_features.context[roots]
        street_root = root_features.street[roots]
        to_act_root = root_features.to_act[roots]
        num_flops = self.flop_id_to_canonical.shape[0]
        gdev = self.generator.device if self.generator is not None else dev
        out = torch.zeros(b, 2, NUM_HANDS, dtype=torch.float32, device=dev)

        def eval_chunk(canonical_chunk: torch.Tensor, weight: torch.Tensor) -> None:
            k = canonical_chunk.shape[0]
            flops = canonical_chunk.contiguous()
            post = flop_expand(pre, roots, flops, check_rows=False)
            board5 = torch.cat([flops, torch.full((k, 2), -1, device=dev, dtype=torch.int64)], dim=1)
            feats = MLPFeatures(
                context=context_root.unsqueeze(1).expand(-1, k, -1).reshape(-1, context_root.shape[1]),
                street=street_root.unsqueeze(1).expand(-1, k).reshape(-1),
                to_act=to_act_root.unsqueeze(1).expand(-1, k).reshape(-1),
                board=board5.unsqueeze(0).expand(b, -1, -1).reshape(-1, 5),
                beliefs=post.reshape(b * k, -1).to(self.float_dtype))
            hv = self._run_model(feats).reshape(b, k, 2, NUM_HANDS).contiguous()
            p = self.NUM_PERM_SAMPLES
            if 0 < p < self.num_permutations:
                perm_idx = torch.randperm(self.num_permutations, device=gdev, generator=self.generator)[:p].to(dev)
                perm_mean(hv, self._combo_perm_i16[perm_idx], weight, out=out, check_perms=False)
            else:
                orbit_mean(hv, weight, out=out)       # all 24 permutations: the mean over each hand's class

        s = self.FLOP_SAMPLE_SIZE
        if 0 < s < num_flops:
            probs = self.flop_id_to_count.to(torch.float32)
            idx = torch.multinomial(probs.to(gdev), s, replacement=True, generator=self.generator).to(dev)
            eval_chunk(self.flop_id_to_canonical[idx], torch.full((s,), 1.0 / s))
            return out.to(self.float_dtype)
        for start in range(0, num_flops, self.FLOP_CHUNK_SIZE):
            end = min(start + self.FLOP_CHUNK_SIZE, num_flops)
            eval_chunk(self.flop_id_to_canonical[start:end], self.flop_id_to_count[start:end].to(torch.float32))
        return (out / float(self.total_flop_count)).to(self.float_dtype)

    @torch.no_grad()
    def single_card_chance_values(self, root_indices: torch.Tensor, root_features: MLPFeatures,
                                  pre_chance_beliefs: torch.Tensor, board_pre: torch.Tensor,
                                  cards_on_board: int | None = None, check_rows: bool = True) -> torch.Tensor:
        """Expected network values over a single-card chance node (turn or river card).
        ``cards_on_board`` / ``check_rows``: see ``chance_expand`` (two device reads a caller can spare)."""
        if root_indices.numel() == 0:
            return torch.zeros(0, self.num_players, NUM_HANDS, device=self.device, dtype=self.float_dtype)
        root_indices = root_indices.to(self.device)
        model = self.model
        if getattr(model, "input_layout", None) == "ranges|board_onehot" and hasattr(model, "forward_input") \
                and pre_chance_beliefs.dtype == torch.float32 and pre_chance_beliefs.is_contiguous() \
                and pre_chance_beliefs.data_ptr() % 16 == 0:
            # the network reads nothing but the ranges and the board: the expansion writes its input matrix
            in_dtype = self.autocast_dtype if self.autocast_dtype in _INPUT_DTYPES else torch.float32
            rows, _, _, offsets = chance_expand(pre_chance_beliefs, root_indices, board_pre, cards_on_board,
                                                check_rows, input_dtype=in_dtype)
            if rows.shape[0] == 0:
                return torch.zeros(root_indices.numel(), self.num_players, NUM_HANDS, device=self.device,
                                   dtype=self.float_dtype)
            if hasattr(model, "eval"):
                model.eval()
            if self.autocast_dtype is not None:
                with torch.autocast(device_type="cuda", dtype=self.autocast_dtype):
                    hv = model.forward_input(rows).hand_values
            else:
                hv = model.forward_input(rows).hand_values
            return chance_mean(hv.to(torch.float32), offsets).to(self.float_dtype)
        post, board_samples, root_lookup, offsets = chance_expand(pre_chance_beliefs, root_indices, board_pre,
                                                                  cards_on_board, check_rows)
        if post.shape[0] == 0:
            return torch.zeros(root_indices.numel(), self.num_players, NUM_HANDS, device=self.device,
                               dtype=self.float_dtype)
        src = root_indices[root_lookup]
        synthetic_features = MLPFeatures(
            context=root_features.context[src],
            street=root_features.street[src],
            to_act=root_features.to_act[src],
            board=board_samples,
            beliefs=post.reshape(post.shape[0], -1).to(self.float_dtype),
        )
        expected = chance_mean(self._run_model(synthetic_features), offsets)
        return expected.to(self.float_dtype)
