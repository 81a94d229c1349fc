"""Writes tests/golden/ranker_golden.npz by running the reference's own
``p2.env.rules`` (pure torch, CPU) in the build container.

Run once, here only:  python tests/golden/gen_ranker_golden.py
The reference is needed because nothing it ships pins the kicker fields of the
non-standard classes (quads + pair, three pairs, multi-window straights, hands
with fewer than five distinct ranks); see the header of oracle/ranker.py.
The fixture holds inputs and outputs only.
"""
from __future__ import annotations

import os
import sys

import numpy as np

REF_SRC = "/root/reference/src"
HERE = os.path.dirname(os.path.abspath(__file__))


def C(r: int, s: int) -> int:
    return s * 13 + r


def targeted_hands() -> list[list[int]]:
    """Hands (lists of 1..7 distinct cards, padded later with -1) aimed at the
    corner classes."""
    hs: list[list[int]] = []
    # quads + pair + singleton above / below the pair; quads + trips
    for q in (0, 5, 12):
        for p in (1, 7, 11):
            for k in (2, 9, 12):
                if len({q, p, k}) < 3:
                    continue
                hs.append([C(q, 0), C(q, 1), C(q, 2), C(q, 3), C(p, 0), C(p, 1), C(k, 2)])
        for t in (3, 10):
            if t != q:
                hs.append([C(q, 0), C(q, 1), C(q, 2), C(q, 3), C(t, 0), C(t, 1), C(t, 2)])
        hs.append([C(q, 0), C(q, 1), C(q, 2), C(q, 3), C((q + 1) % 13, 0), C((q + 3) % 13, 1), C((q + 6) % 13, 2)])
    # three pairs + singleton above / between / below
    for a, b, c in ((12, 8, 3), (10, 9, 0), (6, 5, 4), (12, 11, 10)):
        for k in (1, 7, 11, 12, 2):
            if k in (a, b, c):
                continue
            hs.append([C(a, 0), C(a, 1), C(b, 1), C(b, 2), C(c, 2), C(c, 3), C(k, 0)])
    # two trips + singleton, trips + two pairs
    hs.append([C(9, 0), C(9, 1), C(9, 2), C(4, 0), C(4, 1), C(4, 2), C(12, 3)])
    hs.append([C(2, 0), C(2, 1), C(2, 2), C(11, 0), C(11, 1), C(11, 2), C(0, 3)])
    hs.append([C(9, 0), C(9, 1), C(9, 2), C(4, 0), C(4, 1), C(12, 2), C(12, 3)])
    hs.append([C(3, 0), C(3, 1), C(3, 2), C(10, 0), C(10, 1), C(7, 2), C(7, 3)])
    # runs of 5, 6 and 7 ranks at every start, mixed suits; wheel combinations
    suits = [0, 1, 2, 3, 0, 1, 2]
    for length in (5, 6, 7):
        for lo in range(-1, 13 - length + 1):
            run = [(lo + i) % 13 for i in range(length)]
            hand = [C(r, suits[i]) for i, r in enumerate(run)]
            fill = [r for r in range(13) if r not in run and (r + 1) % 13 not in run and (r - 1) % 13 not in run]
            j = 0
            while len(hand) < 7 and j < len(fill):
                hand.append(C(fill[j], 3 - (j % 2)))
                j += 1
            while len(hand) < 7:
                # no isolated rank left: pair an existing rank instead
                r = run[len(hand) % length]
                cand = [C(r, s) for s in range(4) if C(r, s) not in hand]
                hand.append(cand[0])
            hs.append(hand)
    # wheel + 2..6 (A-2-3-4-5-6) and wheel + T..A style double windows
    hs.append([C(12, 0), C(0, 1), C(1, 2), C(2, 3), C(3, 0), C(4, 1), C(9, 2)])
    hs.append([C(12, 0), C(0, 1), C(1, 2), C(2, 3), C(3, 0), C(4, 1), C(5, 2)])
    hs.append([C(12, 0), C(0, 1), C(1, 2), C(2, 3), C(3, 0), C(11, 1), C(10, 2)])
    # straight flushes with several windows, and SF + higher plain straight
    hs.append([C(3, 2), C(4, 2), C(5, 2), C(6, 2), C(7, 2), C(8, 2), C(9, 2)])
    hs.append([C(12, 1), C(0, 1), C(1, 1), C(2, 1), C(3, 1), C(4, 1), C(8, 0)])
    hs.append([C(3, 2), C(4, 2), C(5, 2), C(6, 2), C(7, 2), C(8, 0), C(9, 1)])
    hs.append([C(12, 3), C(0, 3), C(1, 3), C(2, 3), C(3, 3), C(4, 0), C(5, 1)])
    # flushes of 5, 6, 7 cards, flush + pair, flush + trips
    hs.append([C(12, 0), C(9, 0), C(7, 0), C(4, 0), C(2, 0), C(0, 0), C(5, 0)])
    hs.append([C(12, 0), C(9, 0), C(7, 0), C(4, 0), C(2, 0), C(0, 0), C(0, 1)])
    hs.append([C(12, 0), C(9, 0), C(7, 0), C(4, 0), C(2, 0), C(2, 1), C(2, 2)])
    # short hands (1..6 cards): padding of the kicker list with absent ranks
    hs.append([C(5, 0)])
    hs.append([C(12, 0), C(12, 1)])
    hs.append([C(0, 0), C(0, 1), C(0, 2)])
    hs.append([C(0, 0), C(0, 1), C(0, 2), C(0, 3)])
    hs.append([C(7, 0), C(7, 1), C(3, 2), C(3, 3)])
    hs.append([C(12, 0), C(11, 1), C(10, 2)])
    hs.append([C(8, 0), C(8, 1), C(8, 2), C(5, 3), C(5, 0)])
    hs.append([C(8, 0), C(8, 1), C(8, 2), C(8, 3), C(5, 0), C(5, 1)])
    hs.append([C(1, 0), C(2, 1), C(3, 2), C(4, 3), C(5, 0), C(6, 1)])
    hs.append([C(1, 0), C(3, 1), C(5, 2), C(7, 3), C(9, 0), C(11, 1)])
    hs.append([C(6, 0), C(6, 1), C(4, 2), C(4, 3), C(2, 0), C(2, 1)])
    hs.append([])
    return hs


def main() -> None:
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.env import rules  # noqa: E402  (reference, CPU torch only)

    rng = np.random.default_rng(20240607)
    rand = np.stack([rng.permutation(52)[:7] for _ in range(4096)]).astype(np.int16)
    tgt = targeted_hands()
    tgt_arr = np.full((len(tgt), 7), -1, dtype=np.int16)
    for i, h in enumerate(tgt):
        assert len(set(h)) == len(h) <= 7
        tgt_arr[i, : len(h)] = h
    cards = np.concatenate([rand, tgt_arr], axis=0)

    planes = torch.zeros(cards.shape[0], 1, 4, 13, dtype=torch.bool)
    for i in range(cards.shape[0]):
        for c in cards[i]:
            if c >= 0:
                planes[i, 0, c // 13, c % 13] = True
    cv = rules.create_comparison_vector(planes)  # [N,1,6]
    offsets = 4 * (5 - torch.arange(6, dtype=torch.int))
    packed = (cv.to(torch.int) << offsets[None, None, :]).sum(dim=-1)[:, 0]

    # pairwise results through the public comparison entry point
    ab = torch.stack([planes[:-1, 0], planes[1:, 0]], dim=1)
    cmp = rules.compare_7_single_batch(ab)

    boards = np.array(
        [
            [C(8, 0), C(8, 1), C(8, 2), C(0, 0), C(1, 0)],
            [C(1, 1), C(2, 1), C(3, 1), C(7, 2), C(12, 2)],
            [C(1, 1), C(6, 2), C(9, 1), C(10, 0), C(8, 0)],
            [C(5, 0), C(5, 1), C(8, 2), C(11, 0), C(9, 0)],
            [C(6, 0), C(6, 3), C(7, 3), C(0, 1), C(12, 0)],
            [C(12, 2), C(11, 2), C(10, 2), C(9, 2), C(8, 2)],
            [C(3, 0), C(4, 1), C(5, 2), C(6, 3), C(7, 0)],
        ],
        dtype=np.int64,
    )
    ranks, order = rules.rank_hands(torch.from_numpy(boards))

    np.savez_compressed(
        os.path.join(HERE, "ranker_golden.npz"),
        cards=cards,
        fields=cv[:, 0].numpy().astype(np.int8),
        packed=packed.numpy().astype(np.int32),
        cmp_adjacent=cmp.numpy().astype(np.int8),
        boards=boards.astype(np.int8),
        board_ranks=ranks.numpy().astype(np.int16),
        board_order=order.numpy().astype(np.int16),
    )
    print("wrote ranker_golden.npz:", cards.shape, boards.shape)


if __name__ == "__main__":
    main()
