"""Pins the oracle's visiting order of a query block's selected KV blocks (paced_visit_order).  The reference
has no such function - its kernel visits the blocks in list order and the result depends on the order only
through rounding - so the pins are the properties the rule is defined by, a hand-worked example and a
sequential restatement written slot by slot."""
import numpy as np
import pytest
import torch

from oracle import bsa_oracle as O


def slot_by_slot(blocks, nbk, width=8):
    """The same rule, told from the slots' side: walk the groups, hand each its own blocks while it has room,
    remember the rest; then walk the slots and hand the remembered blocks to the empty ones; then order every
    group.  Plain Python lists, no numpy indexing."""
    blocks = [int(b) for b in blocks]
    n = len(blocks)
    if n <= width:
        return blocks
    groups = (n + width - 1) // width
    slots = [None] * n
    used = [0] * groups
    rest = []
    for b in blocks:
        g = min(b * n // (nbk * width), groups - 1)
        room = min(width, n - g * width)
        if used[g] < room:
            slots[g * width + used[g]] = b
            used[g] += 1
        else:
            rest.append(b)
    rest.reverse()
    for s in range(n):
        if slots[s] is None:
            slots[s] = rest.pop()
    assert not rest
    out = []
    for g in range(groups):
        out += sorted(slots[g * width:(g + 1) * width])
    return out


@pytest.mark.parametrize("nbk,n", [(1440, 90), (624, 39), (1170, 146), (64, 64), (100, 9), (4096, 1000), (37, 20)])
def test_permutation_and_agreement_with_the_slot_by_slot_restatement(nbk, n):
    rng = np.random.default_rng(nbk * 7 + n)
    for trial in range(20):
        blocks = np.sort(rng.choice(nbk, n, replace=False)).astype(np.int32)
        got = O.paced_visit_order(blocks, nbk)
        assert got.dtype == blocks.dtype and np.array_equal(np.sort(got), blocks)
        assert list(got) == slot_by_slot(blocks, nbk)


def test_evenly_spread_and_short_lists_stay_ascending():
    assert np.array_equal(O.paced_visit_order(np.arange(0, 1440, 16), 1440), np.arange(0, 1440, 16))
    assert np.array_equal(O.paced_visit_order(np.arange(5, 1440, 16), 1440), np.arange(5, 1440, 16))
    assert np.array_equal(O.paced_visit_order(np.arange(64), 64), np.arange(64))          # every block selected
    for n in range(0, 9):
        short = np.array([50, 40, 30, 20, 10, 5, 3, 2][:n][::-1], dtype=np.int64)
        assert np.array_equal(O.paced_visit_order(short, 64), short)


def test_hand_worked_example():
    # 16 blocks of 64, groups of 4 slots: group g owns blocks 16 g .. 16 g + 15
    blocks = np.array([0, 1, 2, 3, 4, 5, 20, 40, 41, 42, 43, 44, 45, 50, 60, 63])
    # group 0 owns 0..5: keeps 0 1 2 3, hands on 4 5.  group 1 owns 20: slots 20 _ _ _.  group 2 owns
    # 40..45: keeps 40 41 42 43, hands on 44 45.  group 3 owns 50 60 63: slots 50 60 63 _.
    # the blocks handed on, ascending 4 5 44 45, fill the empty slots in ascending order:
    # group 1 <- 4 5 44, group 3 <- 45; every group ascending
    want = [0, 1, 2, 3, 4, 5, 20, 44, 40, 41, 42, 43, 45, 50, 60, 63]
    assert list(O.paced_visit_order(blocks, 64, width=4)) == want
    assert slot_by_slot(blocks, 64, width=4) == want


def test_a_crowded_stretch_is_spread_and_the_pace_returns():
    # 90 of 1440 blocks, the first 30 of them crowded into blocks 0..29: the surplus of the first groups
    # moves into the groups that own nothing, and from the place where the list is evenly spread again
    # the blocks sit in the slots of their own groups
    blocks = np.concatenate([np.arange(30), np.arange(480, 1440, 16)]).astype(np.int32)
    got = O.paced_visit_order(blocks, 1440)
    assert np.array_equal(np.sort(got), blocks)
    n = len(blocks)
    groups_of_slots = np.arange(n) // 8
    own_group = np.minimum(got.astype(np.int64) * n // (1440 * 8), 11)
    assert np.all(own_group[32:] == groups_of_slots[32:])


def test_attention_does_not_depend_on_the_visiting_order_beyond_rounding():
    g = torch.Generator().manual_seed(3)
    nbk, n = 40, 20
    q = torch.randn(1, 1, 64, 128, generator=g).bfloat16()
    k = torch.randn(1, 1, nbk * 64, 128, generator=g).bfloat16()
    v = torch.randn(1, 1, nbk * 64, 128, generator=g).bfloat16()
    blocks = np.sort(np.random.default_rng(4).choice(nbk, n, replace=False))
    paced = O.paced_visit_order(blocks, nbk)
    assert not np.array_equal(paced, blocks)
    lens = torch.full((1, 1, 1), n, dtype=torch.int32)
    o_a, lse_a = O.blockwise_attention(q, k, v, torch.from_numpy(blocks).view(1, 1, 1, n), lens, 64, 64, 128 ** -0.5)
    o_b, lse_b = O.blockwise_attention(q, k, v, torch.from_numpy(paced).view(1, 1, 1, n), lens, 64, 64, 128 ** -0.5)
    assert torch.allclose(lse_a, lse_b, atol=1e-5)
    assert float((o_a.float() - o_b.float()).abs().max()) <= 2.0 ** -8
