"""Pins of the oracle's block-movement functions (CPU only)."""
import numpy as np

from oracle import paged_kv_oracle as orc


def test_swap_blocks_against_element_loops():
    rng = np.random.default_rng(0)
    k = rng.standard_normal((9, 2, 4, 8)).astype(np.float32)
    v = rng.standard_normal((9, 2, 4, 8)).astype(np.float32)
    ks = rng.standard_normal((9, 2, 4)).astype(np.float32)
    src, dst = [1, 3, 3, 7], [0, 2, 5, 8]
    ref = [a.copy() for a in (k, v, ks)]
    for a in ref:  # element loops over a snapshot
        snap = a.copy()
        for s, d in zip(src, dst):
            for idx in np.ndindex(a.shape[1:]):
                a[(d,) + idx] = snap[(s,) + idx]
    orc.swap_blocks([k, v, ks, None], src, dst)
    for got, want in zip((k, v, ks), ref):
        assert np.array_equal(got, want)
    # untouched blocks stay untouched
    assert np.array_equal(k[4], ref[0][4]) and np.array_equal(k[6], ref[0][6])


def test_swap_blocks_gathers_before_it_scatters():
    # chain 0 -> 1, 1 -> 2: block 2 must receive the OLD block 1 (index_select precedes index_copy_)
    a = np.arange(3 * 2, dtype=np.float32).reshape(3, 2)
    old = a.copy()
    orc.swap_blocks([a], [0, 1], [1, 2])
    assert np.array_equal(a[1], old[0]) and np.array_equal(a[2], old[1])
    # an in-place pass in list order would have produced old[0] in block 2
    assert not np.array_equal(a[2], old[0])


def test_block_copy_groups_known_answer_and_round_trip():
    pairs = [(5, 9), (2, 7), (5, 10), (2, 8), (3, 11)]
    src, dst, cum = orc.build_block_copy_groups(pairs)
    assert src == [2, 3, 5]
    assert cum == [2, 3, 5]
    assert dst == [7, 8, 11, 9, 10]
    # expanding the groups gives back the transfer list
    expanded, begin = [], 0
    for g, s in enumerate(src):
        expanded += [(s, d) for d in dst[begin:cum[g]]]
        begin = cum[g]
    assert sorted(expanded) == sorted(pairs)
    assert orc.build_block_copy_groups([]) == ([], [], [])
    assert orc.build_block_copy_groups([(4, 1)]) == ([4], [1], [1])


def test_copy_blocks_equals_swap_over_expanded_pairs():
    rng = np.random.default_rng(1)
    a = rng.integers(-100, 100, size=(12, 3, 2, 4)).astype(np.int8)
    b = a.copy()
    pairs = [(0, 6), (0, 7), (3, 8), (5, 9), (5, 10), (5, 11)]
    src, dst, cum = orc.build_block_copy_groups(pairs)
    orc.copy_blocks([a], src, dst, cum)
    orc.swap_blocks([b], [s for s, _ in pairs], [d for _, d in pairs])
    assert np.array_equal(a, b)
    for s, d in pairs:
        assert np.array_equal(a[d], a[s])
