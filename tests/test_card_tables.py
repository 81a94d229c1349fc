"""The product's own combo / blocker tables (poker2_amd/card_utils.py), bit-exact against the
oracle's tables, the closed forms and the known answers the reference's tests hold
(tests/test_card_utils.py:44-47, :96-104, :118-128, :154-210, :378-408, :506-510 restated as data).
Host tables only: nothing here needs a GPU."""
from itertools import permutations

import numpy as np
import pytest
import torch

from oracle import cards as OC
from poker2_amd import card_utils as CU

H = 1326


def test_hand_combos_order_and_known_rows():
    t = CU.hand_combos_tensor()
    assert t.shape == (H, 2) and t.dtype == torch.long and t.device.type == "cpu"
    assert np.array_equal(t.numpy(), OC.hand_combos())
    assert t[:5].tolist() == [[0, 1], [0, 2], [0, 3], [0, 4], [0, 5]]          # reference :44-47
    assert t[-1].tolist() == [50, 51]
    assert (t[:, 0] < t[:, 1]).all()
    assert len({tuple(r) for r in t.tolist()}) == H
    # lexicographic: rows strictly ascending as (c1, c2) pairs
    key = t[:, 0] * 52 + t[:, 1]
    assert (key[1:] > key[:-1]).all()
    assert CU.hand_combos_tensor() is t                                      # cached like the reference's


def test_lookup_is_symmetric_with_empty_diagonal_and_inverts_the_combos():
    lut = CU.combo_lookup_tensor()
    assert lut.shape == (52, 52) and lut.dtype == torch.long
    assert np.array_equal(lut.numpy(), OC.combo_lookup())
    assert (torch.diag(lut) == -1).all() and torch.equal(lut, lut.T)
    for a, b, idx in [(0, 1, 0), (0, 2, 1), (1, 2, 51)]:                     # reference :96-104
        assert lut[a, b] == idx and lut[b, a] == idx
    combos = CU.hand_combos_tensor()
    assert torch.equal(lut[combos[:, 0], combos[:, 1]], torch.arange(H))
    off_diagonal = lut[~torch.eye(52, dtype=torch.bool)]
    assert sorted(off_diagonal.tolist()) == sorted(list(range(H)) * 2)


def test_combo_index_closed_form_known_answers_and_errors():
    assert CU.combo_index(0, 1) == 0 and CU.combo_index(1, 0) == 0           # reference :118-128
    assert CU.combo_index(0, 2) == 1 and CU.combo_index(2, 0) == 1
    assert CU.combo_index(1, 2) == 51
    assert CU.combo_index(50, 51) == 1325 and CU.combo_index(51, 50) == 1325
    lut = OC.combo_lookup()
    for a in range(52):
        for b in range(52):
            if a == b:
                with pytest.raises(ValueError):
                    CU.combo_index(a, b)
            else:
                lo, hi = min(a, b), max(a, b)
                assert CU.combo_index(a, b) == lut[a, b] == lo * (103 - lo) // 2 + (hi - lo - 1) == OC.combo_index(a, b)
    for bad in [(-1, 3), (3, 52), (60, 61)]:
        with pytest.raises(ValueError):
            CU.combo_index(*bad)


def test_onehot_blocking_and_compatible_tables():
    oh = CU.combo_to_onehot_tensor()
    assert oh.shape == (H, 52) and oh.dtype == torch.bool
    assert np.array_equal(oh.numpy(), OC.combo_onehot())
    assert (oh.sum(dim=1) == 2).all() and (oh.sum(dim=0) == 51).all()         # every card is in 51 combos
    blocking, compatible = CU.combo_blocking_tensor(), CU.combo_compatible_tensor()
    assert blocking.shape == (H, H) and blocking.dtype == torch.bool
    assert np.array_equal(blocking.numpy(), OC.combo_blocking())
    assert np.array_equal(compatible.numpy(), OC.combo_compatible())
    assert torch.equal(compatible, ~blocking) and torch.equal(blocking, blocking.T)        # reference :378-390
    assert blocking.diagonal().all() and not compatible.diagonal().any()      # reference :506-510
    # a combo is blocked by itself and by 50 + 50 others; C(50, 2) = 1225 are compatible
    assert (blocking.sum(dim=1) == 101).all() and (compatible.sum(dim=1) == 1225).all()
    # brute force on a sample of rows
    combos = OC.hand_combos()
    for h in (0, 51, 700, 1325):
        shares = np.array([len({*combos[h]} & {*combos[g]}) > 0 for g in range(H)])
        assert np.array_equal(blocking[h].numpy(), shares)


def test_mask_conflicting_combos_matches_the_oracle_and_counts():
    rng = np.random.default_rng(3)
    assert CU.mask_conflicting_combos(torch.tensor([], dtype=torch.long)).all()                 # reference :154-162
    assert not CU.mask_conflicting_combos(torch.arange(52)).any()                                # :204-210
    a = CU.mask_conflicting_combos(torch.tensor([0, -1, 1, -2]))                                 # :188-197
    assert torch.equal(a, CU.mask_conflicting_combos(torch.tensor([0, 1])))
    for k in range(0, 8):
        cards = rng.choice(52, size=k, replace=False)
        padded = np.concatenate([cards, -np.ones(2, dtype=np.int64)])
        rng.shuffle(padded)
        got = CU.mask_conflicting_combos(torch.from_numpy(padded))
        assert got.dtype == torch.bool and got.shape == (H,)
        assert np.array_equal(got.numpy(), OC.mask_conflicting(padded))
        assert int(got.sum()) == (52 - k) * (51 - k) // 2                   # C(52-k, 2): 1176 flop, 1128 turn, 1081 river
        oh = OC.combo_onehot()
        assert np.array_equal(got.numpy(), ~oh[:, cards].any(axis=1))


def test_suit_permutation_tables_are_bijections_that_permute_suits():
    perms = CU.suit_permutations_tensor()
    assert perms.shape == (24, 4) and perms.tolist() == [list(p) for p in permutations(range(4))]
    table, inverse = CU.combo_suit_permutation_tensor(), CU.combo_suit_permutation_inverse_tensor()
    assert table.shape == (24, H) and table.dtype == torch.long
    assert torch.equal(table[0], torch.arange(H))                            # identity permutation first
    combos = OC.hand_combos()
    for q in range(24):
        assert sorted(table[q].tolist()) == list(range(H))
        assert torch.equal(table[q][inverse[q]], torch.arange(H))
        assert torch.equal(inverse[q][table[q]], torch.arange(H))
        for h in (0, 13, 400, 1000, 1325):
            mapped = sorted(int(perms[q][c // 13]) * 13 + c % 13 for c in combos[h])
            assert combos[int(table[q][h])].tolist() == mapped


def test_device_combo_table_constructor_restated():
    """The kernels index hands through a compile-time table (csrc/common.h: a[h], b[h],
    row_start[c]) and the closed form ``p2_combo_index``; the same loop in Python must give the
    host tables.  The device copy itself is read back through kernels in the GPU twin of this
    test (tests/test_gpu_card_tables.py)."""
    a, b, row_start, k = [], [], [], 0
    for c1 in range(52):
        row_start.append(k)
        for c2 in range(c1 + 1, 52):
            a.append(c1)
            b.append(c2)
            k += 1
    row_start.append(k)
    t = CU.hand_combos_tensor()
    assert a == t[:, 0].tolist() and b == t[:, 1].tolist() and k == H
    assert all(row_start[c] == c * (103 - c) // 2 for c in range(52)) and row_start[52] == H
