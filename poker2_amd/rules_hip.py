"""7-card hand evaluation on the GPU with the reference's function names.

Drop-in for ``src/p2/env/rules_triton.py`` (:36-148) and for the tensor entry
points of ``src/p2/env/rules.py`` (``compare_7_single_batch`` :390,
``compare_7_batches`` :412, ``rank_hands`` :66): same shapes, dtypes and error
behaviour.  Every function launches a hand-written HIP kernel of libp2hip.so on
the current stream; there is no CPU path.
"""
from __future__ import annotations

from enum import Enum

import torch

from . import _lib
from ._lib import hip_is_available
from ._guards import require as _req

NUM_HANDS = 1326


class HandType(Enum):
    """Hand categories = field 0 of the comparison vector (src/p2/env/rules.py:17-28)."""
    NUM_HAND_TYPES = 10
    STRAIGHT_FLUSH = 9
    FOUR_OF_A_KIND = 8
    FULL_HOUSE = 7
    FLUSH = 6
    STRAIGHT = 5
    THREE_OF_A_KIND = 4
    TWO_PAIR = 3
    ONE_PAIR = 2
    HIGH_CARD = 1
    EMPTY = 0


def rank(card: int) -> int:
    """src/p2/env/rules.py: rank 0..12 = 2..A of card = suit * 13 + rank."""
    return card % 13


def suit(card: int) -> int:
    return card // 13


def triton_is_available() -> bool:
    """Kept under the reference's name: True when the HIP library and a GPU are usable."""
    return hip_is_available()


def _require_backend() -> None:
    if not hip_is_available():
        raise RuntimeError("libp2hip.so or a GPU is not available; the hand evaluator has no other backend.")


def _planes_i8(ab_batch: torch.Tensor, tail: tuple[int, ...]) -> torch.Tensor:
    if ab_batch.dim() != len(tail) + 1 or tuple(ab_batch.shape[1:]) != tail:
        raise ValueError(f"Expected [N, {', '.join(map(str, tail))}] input, got {tuple(ab_batch.shape)}")
    if ab_batch.device.type != "cuda":
        raise ValueError("The HIP hand evaluator requires a GPU tensor.")
    x = ab_batch.contiguous()
    if x.dtype in (torch.bool, torch.int8, torch.uint8):
        return x.view(torch.uint8)            # one byte per card already: no copy (non-zero = present)
    return (x != 0).view(torch.uint8)


def _compare_planes(ab_batch: torch.Tensor, flush_first: int) -> torch.Tensor:
    _require_backend()
    planes = _planes_i8(ab_batch, (2, 4, 13))
    out = torch.empty((planes.shape[0],), device=planes.device, dtype=torch.int32)
    _lib.call("p2hip_compare7_planes", _lib.ptr(planes), planes.shape[0], _lib.ptr(out), flush_first,
              _lib.stream_ptr())
    return out


def compare_7_single_batch_triton(ab_batch: torch.Tensor) -> torch.Tensor:
    """[N,2,4,13] planes -> [N] int32 in {-1,0,1} (rules_triton.py:36-51)."""
    return _compare_planes(ab_batch, 1)


def compare_7_batches_triton(a_batch: torch.Tensor, b_batch: torch.Tensor) -> torch.Tensor:
    """Two [N,4,13] plane batches -> [N] (rules_triton.py:54-60)."""
    if a_batch.shape != b_batch.shape:
        raise ValueError("a_batch and b_batch must have the same shape.")
    if a_batch.dim() != 3 or tuple(a_batch.shape[1:]) != (4, 13):
        raise ValueError(f"Expected [N, 4, 13] inputs, got {tuple(a_batch.shape)}")
    return compare_7_single_batch_triton(torch.stack([a_batch, b_batch], dim=1).bool())


def create_comparison_vector(ab_batch: torch.Tensor) -> torch.Tensor:
    """[N, P, 4, 13] planes -> [N, P, 6] int32 (hand type, five rank fields; 0 where unused), the
    vector whose nibble packing is the score (src/p2/env/rules.py:136-299, :406-407)."""
    _require_backend()
    if ab_batch.dim() != 4 or tuple(ab_batch.shape[2:]) != (4, 13):
        raise ValueError(f"Expected [N, P, 4, 13] input, got {tuple(ab_batch.shape)}")
    n, p = ab_batch.shape[:2]
    packed = rank_7_planes(ab_batch.reshape(n * p, 4, 13)).view(n, p)
    shifts = torch.tensor([20, 16, 12, 8, 4, 0], device=packed.device, dtype=torch.int32)
    return (packed[..., None] >> shifts) & 0xF


def compare_7(a_cards, b_cards) -> int:
    """Two lists of 7 card ids -> 1 / -1 / 0 (src/p2/env/rules.py:358-387)."""
    _req(len(a_cards) == 7, f"Expected 7 cards for hand A, got {len(a_cards)}")
    _req(len(b_cards) == 7, f"Expected 7 cards for hand B, got {len(b_cards)}")
    planes = torch.zeros(1, 2, 4, 13, dtype=torch.bool)
    for p, cards in enumerate((a_cards, b_cards)):
        for card in cards:
            planes[0, p, card // 13, card % 13] = True
    return int(compare_7_single_batch(planes.cuda())[0].item())


def compare_7_single_batch(ab_batch: torch.Tensor) -> torch.Tensor:
    """rules.py:390-409 on the GPU: bool planes only; the flush suit is the fullest suit."""
    _req(ab_batch.dim() == 4, "ab_batch.dim() == 4")
    _req(tuple(ab_batch.shape[1:]) == (2, 4, 13), "tuple(ab_batch.shape[1:]) == (2, 4, 13)")
    _req(ab_batch.dtype == torch.bool, "ab_batch.dtype == torch.bool")
    return _compare_planes(ab_batch, 0)


def compare_7_batches(a_batch: torch.Tensor, b_batch: torch.Tensor) -> torch.Tensor:
    """rules.py:412-426 on the GPU."""
    _req(a_batch.shape == b_batch.shape, "a_batch.shape == b_batch.shape")
    _req(a_batch.dim() == 3, "a_batch.dim() == 3")
    _req(tuple(a_batch.shape[1:]) == (4, 13), "tuple(a_batch.shape[1:]) == (4, 13)")
    return compare_7_single_batch(torch.stack([a_batch, b_batch], dim=1).bool())


def rank_7_planes(planes: torch.Tensor, flush_first: bool = False) -> torch.Tensor:
    """[N,4,13] planes -> [N] packed int32 score (the packed comparison vector of
    rules.py:136-299 / :406-407)."""
    _require_backend()
    p = _planes_i8(planes, (4, 13))
    out = torch.empty((p.shape[0],), device=p.device, dtype=torch.int32)
    _lib.call("p2hip_rank7_planes", _lib.ptr(p), p.shape[0], _lib.ptr(out), int(flush_first), _lib.stream_ptr())
    return out


def _cards_arg(cards_batch: torch.Tensor) -> tuple[torch.Tensor, int]:
    """int8 / int16 / int64 ids pass through; any other integer dtype is narrowed to int16
    (what the reference does for every input, rules_triton.py:73-75, :107)."""
    if cards_batch.device.type != "cuda":
        raise ValueError("The HIP hand evaluator requires a GPU tensor.")
    if cards_batch.dtype not in (torch.int8, torch.int16, torch.int64):
        cards_batch = cards_batch.to(torch.int16)
    cards_batch = cards_batch.contiguous()
    return cards_batch, cards_batch.element_size()


def compare_7_cards_single_batch_triton(cards_batch: torch.Tensor) -> torch.Tensor:
    """[N,2,7] card ids 0..51 -> [N] int32 in {-1,0,1} (rules_triton.py:78-93)."""
    _require_backend()
    if cards_batch.dim() != 3 or tuple(cards_batch.shape[1:]) != (2, 7):
        raise ValueError(f"Expected [N, 2, 7] input, got {tuple(cards_batch.shape)}")
    cards, esz = _cards_arg(cards_batch)
    out = torch.empty((cards.shape[0],), device=cards.device, dtype=torch.int32)
    _lib.call("p2hip_compare7_cards", _lib.ptr(cards), esz, cards.shape[0], _lib.ptr(out), _lib.stream_ptr())
    return out


def rank_7_cards_single_batch_triton(cards_batch: torch.Tensor) -> torch.Tensor:
    """[N,7] card ids -> [N] packed int32 score, higher = stronger (rules_triton.py:96-117)."""
    _require_backend()
    if cards_batch.dim() != 2 or cards_batch.shape[1] != 7:
        raise ValueError(f"Expected [N, 7] input, got {tuple(cards_batch.shape)}")
    cards, esz = _cards_arg(cards_batch)
    out = torch.empty((cards.shape[0],), device=cards.device, dtype=torch.int32)
    _lib.call("p2hip_rank7_cards", _lib.ptr(cards), esz, cards.shape[0], _lib.ptr(out), _lib.stream_ptr())
    return out


def _rank_boards(board: torch.Tensor, mode: int, want_table: bool):
    _require_backend()
    if board.dim() != 2 or board.shape[1] != 5:
        raise ValueError(f"board must be [M, 5], got {tuple(board.shape)}")
    if board.device.type != "cuda":
        raise ValueError("The HIP hand evaluator requires a GPU tensor.")
    if board.dtype not in (torch.int8, torch.int16, torch.int32, torch.int64):
        board = board.to(torch.int64)
    board = board.contiguous()
    m = board.shape[0]
    ranks = torch.empty((m, NUM_HANDS), device=board.device, dtype=torch.int32)
    order = torch.empty((m, NUM_HANDS), device=board.device, dtype=torch.int64)
    table = None
    if want_table:
        table = torch.empty((m, showdown_table_bytes()), device=board.device, dtype=torch.uint8)
    _lib.call("p2hip_showdown_setup", _lib.ptr(board), board.element_size(), m, mode, _lib.ptr(ranks),
              _lib.ptr(order), _lib.ptr(table), _lib.stream_ptr())
    return ranks, order, table


def rank_hands_triton(board: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """[M,5] boards -> (packed scores [M,1326] int32, stable ascending argsort [M,1326] int64)
    (rules_triton.py:120-148)."""
    ranks, order, _ = _rank_boards(board, 1, False)
    return ranks, order


def rank_hands(board: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """[M,5] boards -> (dense 1-based strength ids [M,1326] int32, stable ascending argsort)
    (rules.py:66-133); combos touching the board are ranked as 6-card hands."""
    ranks, order, _ = _rank_boards(board, 0, False)
    return ranks, order


def showdown_table_bytes() -> int:
    return int(_lib.load().p2hip_showdown_table_bytes())


def build_showdown_tables(board: torch.Tensor, triton_order: bool = True) -> torch.Tensor:
    """[M,5] boards -> [M, table_bytes] uint8 per-board strength tables for
    ``showdown_value_both`` (replaces ``_init_hand_rank_data``, cfr_evaluator.py:406-482).
    ``triton_order`` picks the card-id ranker the fused evaluator installs
    (fused_sparse_cfr_evaluator.py:70-78); the two rankers order unblocked hands alike."""
    _, _, table = _rank_boards(board, 1 if triton_order else 0, True)
    return table


def showdown_value_both(beliefs: torch.Tensor, tables: torch.Tensor, potential: torch.Tensor,
                        scale: torch.Tensor, table_row: torch.Tensor | None = None,
                        out: torch.Tensor | None = None) -> torch.Tensor:
    """beliefs [M,2,1326] -> [M,2,1326] showdown EV of both players per hand
    (``_showdown_value_both``, cfr_evaluator.py:484-601): conditional on the villain hands
    that do not share a card with the hero's, times potential[:, p] / scale."""
    _require_backend()
    _lib.require_gpu(beliefs, "showdown_value_both")
    if beliefs.dim() != 3 or tuple(beliefs.shape[1:]) != (2, NUM_HANDS):
        raise ValueError(f"beliefs must be [M, 2, {NUM_HANDS}], got {tuple(beliefs.shape)}")
    m = beliefs.shape[0]
    beliefs = beliefs.contiguous().float()
    potential = potential.to(device=beliefs.device, dtype=torch.float32).contiguous()
    scale = scale.to(device=beliefs.device, dtype=torch.float32).contiguous()
    _req(potential.shape == (m, 2) and scale.shape == (m,), "potential.shape == (m, 2) and scale.shape == (m,)")
    _req(tables.is_contiguous() and tables.dtype == torch.uint8 and tables.shape[1] == showdown_table_bytes(),
         "tables.is_contiguous() and tables.dtype == torch.uint8 and tables.shape[1] == showdown_table_bytes()")
    if table_row is not None:
        table_row = table_row.to(torch.int64).contiguous()
        _req(table_row.shape == (m,), "table_row.shape == (m,)")
    else:
        _req(tables.shape[0] == m, "tables.shape[0] == m")
    if out is None:
        out = torch.empty_like(beliefs)
    _req(out.is_contiguous() and out.shape == beliefs.shape, "out.is_contiguous() and out.shape == beliefs.shape")
    _lib.call("p2hip_showdown_both", _lib.ptr(beliefs), _lib.ptr(tables), _lib.ptr(table_row),
              _lib.ptr(potential), _lib.ptr(scale), m, _lib.ptr(out), _lib.stream_ptr())
    return out
