"""Writes tests/golden/ranker_cards_golden.npz by RUNNING the reference's own card-id ranking kernel
(``_rank_7_cards_single_batch_kernel`` -> ``_evaluate_cards_player``, src/p2/env/rules_triton.py:414-632)
under Triton's CPU interpreter (TRITON_INTERPRET=1) in the build container.
Run once, here only:  python tests/golden/gen_ranker_cards_golden.py

What it pins: how a hand that REPEATS a card id is scored.  ``rules.py`` takes card planes and cannot
express such a hand; ``rank_hands_triton`` (:120-148) feeds exactly such hands for every combo that
holds a board card.  The rule has two halves: rank multiplicities count the repeated card again
(:431-440), and the suit masks are SUMS of the cards' rank bits (:421-425), so a repeated card carries
into the next higher bit of its suit's mask instead of being absorbed — which moves flush and
straight-flush detection.

One substitution, stated here because it is the only thing that is not the reference's code: the two
leaf helpers ``_pop_highest_rank`` and ``_popcount`` (:364-385) are PTX inline assembly (``bfind.u32``,
``popc.b32``), which neither the interpreter nor this hardware executes.  Both instructions are fixed
by their ISA definition — position of the most significant set bit (0xFFFFFFFF for zero, which the
helper then clamps to 0) and number of set bits — and are replaced by plain Triton integer code with
exactly that meaning; everything else runs as the reference wrote it.  ``rank_7_cards_single_batch_triton``
refuses CPU tensors before launching (:107-108), so the wrapper's own launch line is repeated (same
kernel, grid, constants); ``rank_hands_triton``'s card assembly and stable argsort (:136-148) likewise.

The fixture holds inputs and outputs only: hands [n,7] int16, packed scores [n] int32; boards [3,5],
``hand_ranks`` [3,1326] int32 and ``sorted_indices`` [3,1326] int64.
"""
from __future__ import annotations

import os
import sys

os.environ["TRITON_INTERPRET"] = "1"          # before triton is imported

import numpy as np  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402

REF_SRC = "/root/reference/src"
HERE = os.path.dirname(os.path.abspath(__file__))


@triton.jit
def pop_highest_rank(rank_mask):
    # bfind.u32 + the helper's own clamp: index of the most significant set bit, 0 for an empty mask
    best_idx = tl.full((), 0, tl.int32)
    for k in range(1, 32):
        best_idx = best_idx + ((rank_mask >> k) != 0).to(tl.int32)
    return best_idx, rank_mask & ~(tl.full((), 1, tl.int32) << best_idx)


@triton.jit
def popcount(mask):
    # popc.b32: number of set bits
    n = tl.full((), 0, tl.int32)
    for k in range(0, 32):
        n = n + ((mask >> k) & 1)
    return n


def C(r: int, s: int) -> int:
    return s * 13 + r


def repeated_card_hands(rng: np.random.Generator) -> np.ndarray:
    hs: list[list[int]] = []
    # a random hand of seven distinct cards with one card written over another (pair-making)
    for _ in range(60):
        h = rng.permutation(52)[:7].tolist()
        i, j = rng.choice(7, 2, replace=False)
        h[j] = h[i]
        hs.append(h)
    # trips-making: the hand holds a pair of the rank already; quads-making: it holds trips
    for r in (0, 5, 9, 12):
        for rest in ((1, 3, 7, 10), (2, 4, 6, 8)):
            rest = [x for x in rest if x != r][:4]
            hs.append([C(r, 0), C(r, 1), C(r, 0)] + [C(x, (k + 1) % 4) for k, x in enumerate(rest)])
            hs.append([C(r, 0), C(r, 1), C(r, 2), C(r, 1)] + [C(x, (k + 2) % 4) for k, x in enumerate(rest[:3])])
            hs.append([C(r, 3), C(r, 3), C(r, 3)] + [C(x, k % 3) for k, x in enumerate(rest)])          # one card three times
            hs.append([C(r, 2)] * 4 + [C(x, k % 2) for k, x in enumerate(rest[:3])])                       # four times
    # flush-suit duplicates: five or six cards of a suit with one of them repeated; four + a repeat
    for suit in range(4):
        for ranks in ((0, 2, 5, 7, 11), (1, 2, 3, 9, 12), (4, 6, 8, 10, 12), (0, 1, 2, 3, 12), (8, 9, 10, 11, 12)):
            base = [C(r, suit) for r in ranks]
            for dup in (0, 2, 4):
                hs.append(base + [base[dup], C((ranks[dup] + 6) % 13, (suit + 1) % 4)])
                hs.append(base[:4] + [base[dup % 4], base[dup % 4], C((ranks[0] + 7) % 13, (suit + 2) % 4)])
                hs.append(base + [base[dup], base[dup]])
            hs.append(base[:4] + [base[3]] + [C((ranks[1] + 5) % 13, (suit + 1) % 4), C((ranks[2] + 5) % 13, (suit + 3) % 4)])
    # off-suit duplicates next to a flush, a straight, a straight flush
    for lo in (0, 3, 8):
        run = [C(lo + i, 1) for i in range(5)]
        hs.append(run + [C(lo, 2), C(lo, 2)])
        hs.append(run + [run[0], C((lo + 7) % 13, 0)])
        hs.append(run + [run[4], run[4]])
        hs.append(run[:4] + [run[3], C(lo + 4, 3), C((lo + 9) % 13, 0)])
        mixed = [C(lo + i, i % 4) for i in range(5)]
        hs.append(mixed + [mixed[2], C((lo + 8) % 13, 2)])
        hs.append(mixed + [mixed[0], mixed[4]])
    # wheel and ace duplicates (an ace's bit carries out of the thirteen rank bits)
    hs.append([C(12, 0), C(12, 0), C(0, 0), C(1, 0), C(2, 0), C(3, 0), C(7, 1)])
    hs.append([C(12, 2), C(12, 2), C(11, 2), C(10, 2), C(9, 2), C(8, 2), C(3, 1)])
    hs.append([C(12, 1), C(12, 1), C(12, 1), C(12, 1), C(4, 1), C(6, 1), C(8, 1)])
    hs.append([C(12, 3)] * 7)
    hs.append([C(0, 0)] * 7)
    hs.append([C(5, 2)] * 5 + [C(5, 1), C(9, 0)])
    # hands without a repeat, as a check of the substitution against what rules.py gives for them
    for _ in range(64):
        hs.append(rng.permutation(52)[:7].tolist())
    return np.asarray(hs, dtype=np.int16)


def main() -> None:
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.env import rules_triton as RT
    from p2.env import rules as R
    from p2.env.card_utils import NUM_HANDS, hand_combos_tensor

    RT._pop_highest_rank = pop_highest_rank
    RT._popcount = popcount

    def rank_cards(cards: torch.Tensor) -> torch.Tensor:       # rules_triton.py:109-117 without the CUDA check
        cards_i16 = cards.contiguous().to(torch.int16)
        out = torch.empty((cards_i16.shape[0],), dtype=torch.int32)
        RT._rank_7_cards_single_batch_kernel[(cards_i16.shape[0],)](cards_i16, out, CARD_LANES=RT.CARD_LANES,
                                                                   RANK_LANES=RT.RANK_LANES, num_warps=1)
        return out

    rng = np.random.default_rng(2024)
    hands = repeated_card_hands(rng)
    scores = rank_cards(torch.from_numpy(hands)).numpy()
    # the substitution reproduces rules.py on the hands it can express (the last 64, no repeats)
    planes = torch.zeros(64, 52, dtype=torch.bool)
    planes[torch.arange(64)[:, None], torch.from_numpy(hands[-64:].astype(np.int64))] = True
    fields = R.create_comparison_vector(planes.view(64, 1, 4, 13))[:, 0].to(torch.int64)
    packed = sum(fields[:, i] << (4 * (5 - i)) for i in range(6)).numpy()
    assert np.array_equal(packed, scores[-64:]), "substituted helpers disagree with rules.py on plain hands"

    boards = np.array([[C(12, 0), C(10, 1), C(7, 2), C(5, 3), C(2, 1)],          # Ac Qh 9d 7s 4h: no flush possible
                       [C(12, 2), C(11, 2), C(10, 2), C(9, 2), C(0, 3)],         # Ad Kd Qd Jd 2s: flush / straight-flush board
                       [C(8, 0), C(8, 1), C(8, 3), C(5, 2), C(5, 1)]],           # Tc Th Ts 7d 7h: full house on board
                      dtype=np.int64)
    combos = hand_combos_tensor()
    m = boards.shape[0]
    holes = combos[None, :, :].expand(m, NUM_HANDS, 2)                            # :136-143
    boards_b = torch.from_numpy(boards)[:, None, :].expand(m, NUM_HANDS, 5)
    cards_flat = torch.cat([holes, boards_b], dim=-1).to(torch.int16).reshape(-1, 7).contiguous()
    hand_ranks = rank_cards(cards_flat).view(m, NUM_HANDS)
    sorted_indices = torch.argsort(hand_ranks, dim=1, stable=True)                # :146-147
    path = os.path.join(HERE, "ranker_cards_golden.npz")
    np.savez_compressed(path, hands=hands, scores=scores.astype(np.int32), boards=boards,
                        hand_ranks=hand_ranks.numpy().astype(np.int32), sorted_indices=sorted_indices.numpy().astype(np.int64))
    n_rep = int(sum(len(set(h)) < 7 for h in hands.tolist()))
    print("wrote", path, os.path.getsize(path), "bytes;", len(hands), "hands,", n_rep, "with a repeated card")


if __name__ == "__main__":
    main()
