"""The residency plan of the routed experts (the checker's restatement of moe_route's device-side tiers,
src/kernels/cuda/glm_fast.cu:4262-4375) against worked examples: every expected word below is written out by hand from
the rule the reference documents (include/strata/kernels/glm_fast.hpp:284-292), not computed by the code under test."""
import numpy as np
import pytest


def make_tab(n_layers, ne):
    return np.zeros(n_layers * (2 * ne + 3), dtype=np.uint64)


def test_all_tables_empty_every_entry_misses(oracle):
    # the reference's own expectation of a route with no table entry: miss_mask 255 for k = 8 (tests/hip/glm_handoff.cpp:118)
    ne, k = 16, 8
    tab = make_tab(1, ne)
    ids = np.arange(k, dtype=np.int32)[None, :]
    plan, src, masks = oracle.plan_tiered(ids, 0, ne, tab, np.zeros(0, dtype=np.uint64))
    assert np.all(plan == 0) and np.all(src == 0) and masks.tolist() == [[255, 0, 0, 0]] and np.all(tab == 0)


def test_hits_spares_scratch_and_misses_of_a_window(oracle):
    nl, ne, k, layer = 2, 8, 4, 1
    tab = make_tab(nl, ne)
    n = nl * ne
    tab[8 + 0], tab[8 + 1] = 0x1000, 0x2000                                   # experts 0, 1 of layer 1 in HBM
    for e, a in ((2, 0xA000), (3, 0xB000), (4, 0xC000), (5, 0xD000), (6, 0xE000)):
        tab[n + 8 + e] = a                                                    # experts 2..6 in the second tier
    tab[2 * n + 0:2 * n + 3] = (0x111, 0x222, 0x333)                          # layer 0's spares: not this route's
    tab[2 * n + 3:2 * n + 6] = (0, 0x5000, 0x6000)                            # layer 1's: the first already taken
    scratch = np.array([0x7000, 0x8000], dtype=np.uint64)
    ids = np.array([[0, 2, 7, 3], [2, 4, 5, 6], [-1, -1, -1, -1]], dtype=np.int32)
    plan, src, masks = oracle.plan_tiered(ids, layer, ne, tab, scratch)
    # token 0: a hit; a promotion into the first free spare; in neither tier; a promotion into the last spare
    assert plan[0].tolist() == [0x1000, 0x5000, 0, 0x6000] and src[0].tolist() == [0, 0xA000, 0, 0xB000]
    assert masks[0].tolist() == [0b0100, 0b1010, 0b1010, 0]
    # token 1: expert 2 is resident now; two scratch slots in order; then no slot is left
    assert plan[1].tolist() == [0x5000, 0x7000, 0x8000, 0] and src[1].tolist() == [0, 0xC000, 0xD000, 0]
    assert masks[1].tolist() == [0, 0b0110, 0, 0b1000]
    # a refused row plans nothing
    assert np.all(plan[2] == 0) and np.all(src[2] == 0) and masks[2].tolist() == [0, 0, 0, 0]
    assert tab[8 + 2] == 0x5000 and tab[8 + 3] == 0x6000 and tab[8 + 4] == 0
    assert tab[2 * n:2 * n + 6].tolist() == [0x111, 0x222, 0x333, 0, 0, 0]


def test_promotion_waits_for_the_count_and_counts_age(oracle):
    ne, k = 8, 2
    tab = make_tab(1, ne)
    tab[ne + 3], tab[ne + 4] = 0xA000, 0xB000
    tab[2 * ne:2 * ne + 3] = (0x5000, 0x6000, 0)
    scratch = np.array([0x7000, 0x8000], dtype=np.uint64)
    counts = np.zeros(ne, dtype=np.uint32)
    counts[6] = 7
    seq = np.array([4094], dtype=np.uint32)
    ids = np.array([[3, 4]], dtype=np.int32)
    # first route (seq 4094 -> 4095: no ageing): both counted once, below the bar of 2: scratch, no promotion
    plan, src, masks = oracle.plan_tiered(ids, 0, ne, tab, scratch, counts, seq, promote_min=2)
    assert plan.tolist() == [[0x7000, 0x8000]] and masks.tolist() == [[0, 3, 0, 0]] and tab[3] == 0
    assert counts.tolist() == [0, 0, 0, 1, 1, 0, 7, 0] and seq[0] == 4095
    # second route: (4095 + 1) % 4096 == 0: every count halves first (1 -> 0, 7 -> 3), then the routed keys count 1: still scratch
    plan, src, masks = oracle.plan_tiered(ids, 0, ne, tab, scratch, counts, seq, promote_min=2)
    assert counts.tolist() == [0, 0, 0, 1, 1, 0, 3, 0] and seq[0] == 4096 and masks.tolist() == [[0, 3, 0, 0]]
    # third route: the counts reach 2: promoted into the spares in order
    plan, src, masks = oracle.plan_tiered(ids, 0, ne, tab, scratch, counts, seq, promote_min=2)
    assert plan.tolist() == [[0x5000, 0x6000]] and src.tolist() == [[0xA000, 0xB000]] and masks.tolist() == [[0, 3, 3, 0]]
    assert tab[3] == 0x5000 and tab[4] == 0x6000 and tab[2 * ne:2 * ne + 3].tolist() == [0, 0, 0]
    # fourth: hits, nothing to fetch
    plan, src, masks = oracle.plan_tiered(ids, 0, ne, tab, scratch, counts, seq, promote_min=2)
    assert plan.tolist() == [[0x5000, 0x6000]] and np.all(src == 0) and masks.tolist() == [[0, 0, 0, 0]]
    assert counts[3] == 3 and counts[4] == 3
