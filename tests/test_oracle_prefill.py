"""Pins the oracle's pair building, grouping and prefill MoE against the
expected arrays held by the reference's own tests."""
import numpy as np
import pytest

import oracle as O


def _pairs(rows):
    a = np.zeros(len(rows), O.PAIR_DTYPE)
    for i, (t, e, r, w) in enumerate(rows):
        a[i] = (t, e, r, w)
    return a


def test_pair_record_layout_and_token_major_order():
    # PrefillRouterTests.swift:12-31
    assert O.PAIR_DTYPE.itemsize == 16
    assert [O.PAIR_DTYPE.fields[n][1] for n in ("token", "expert", "rank", "weight_bits")] == [0, 4, 8, 12]
    w = O.f16_bits(np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float32)).reshape(2, 3)
    p = O.make_pairs(np.array([[3, 1, 2], [4, 0, 5]], np.uint32), w)
    assert list(p["token"]) == [0, 0, 0, 1, 1, 1]
    assert list(p["rank"]) == [0, 1, 2, 0, 1, 2]
    assert list(p["expert"]) == [3, 1, 2, 4, 0, 5]
    assert np.array_equal(p["weight_bits"], w.reshape(-1))


def test_grouping_sorts_pairs_and_builds_offsets_counts_tiles():
    # PrefillMoEGroupingTests.swift:5-53
    rows = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14),
            (1, 2, 2, 15), (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19),
            (3, 1, 1, 20), (3, 4, 2, 21)]
    g = O.group_pairs(_pairs(rows[::-1]), 4, 3, 6, tile_expert_count=2)
    assert list(g["sorted"]["expert"]) == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[int(p["token"]), int(p["rank"])] for p in g["sorted"]] == [
        [0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1], [2, 1], [0, 2], [2, 0],
        [3, 2], [3, 0]]
    assert list(g["offsets"]) == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert list(g["counts"]) == [0, 4, 1, 3, 3, 1]
    assert [tuple(map(int, x)) for x in g["groups"]] == [(1, 0, 4), (2, 4, 1), (3, 5, 3),
                                                        (4, 8, 3), (5, 11, 1)]
    assert [tuple(map(int, x)) for x in g["tiles"]] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]


def test_grouping_is_input_order_invariant_and_keeps_weight_bits():
    # :55-82
    tm = [(0, 2, 0, 101), (0, 1, 1, 102), (1, 2, 0, 103), (1, 0, 1, 104), (2, 1, 0, 105),
          (2, 2, 1, 106)]
    sh = [tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]]
    a = O.group_pairs(_pairs(tm), 3, 2, 3, 2)
    b = O.group_pairs(_pairs(sh), 3, 2, 3, 2)
    for key in a:
        assert np.array_equal(a[key], b[key])
    assert list(a["sorted"]["weight_bits"]) == [104, 102, 105, 101, 103, 106]


def test_grouping_sort_keys():
    # :84-115
    rows = [(0, 1, 0, 10), (0, 2, 1, 20), (1, 3, 0, 30), (1, 1, 1, 11), (2, 2, 0, 21),
            (2, 3, 1, 31)]
    g = O.group_pairs(_pairs(rows), 3, 2, 4, 2, sort_keys=[0, 30, 10, 20])
    assert list(g["groups"]["expert"]) == [2, 3, 1]
    assert list(g["sorted"]["expert"]) == [2, 2, 3, 3, 1, 1]
    assert list(g["offsets"]) == [0xFFFFFFFF, 4, 0, 2]
    assert [tuple(map(int, x)) for x in g["tiles"]] == [(0, 2, 0, 4), (2, 1, 4, 2)]


def test_grouping_rejects_invalid_metadata():
    # :117-173
    one = _pairs([(0, 0, 0, 1)])
    with pytest.raises(O.GroupingError) as e:
        O.group_pairs(one, 1, 1, 1, 17)
    assert e.value.name == "invalidTileExpertCount"
    with pytest.raises(O.GroupingError) as e:
        O.group_pairs(_pairs([(0, 2, 0, 1)]), 1, 1, 2, 1)
    assert e.value.name == "expertOutOfRange"
    with pytest.raises(O.GroupingError) as e:
        O.group_pairs(_pairs([(0, 0, 0, 1), (0, 1, 0, 2)]), 1, 2, 2, 1)
    assert e.value.name == "duplicateTokenRank"
    with pytest.raises(O.GroupingError) as e:
        O.group_pairs(one, 1, 1, 2, 1, sort_keys=[0])
    assert e.value.name == "expertSortKeyCountMismatch"
    with pytest.raises(O.GroupingError) as e:
        O.group_pairs(one, 2, 1, 1, 1)
    assert e.value.name == "pairCountMismatch"
    for args, name in [((-1, 1, 1, 1), "invalidQueryCount"), ((1, 0, 1, 1), "invalidTopK"),
                       ((1, 1, 0, 1), "invalidNumExperts")]:
        with pytest.raises(O.GroupingError) as e:
            O.group_pairs(one, *args)
        assert e.value.name == name
    # empty input is valid and yields nothing
    g = O.group_pairs(_pairs([]), 0, 8, 4, 16)
    assert g["groups"].size == 0 and g["tiles"].size == 0 and list(g["counts"]) == [0] * 4


def test_grouping_pressure_at_t32():
    # :175-203
    rows = [(t, (t + r * 7) % 74, r, t * 8 + r) for t in range(32) for r in range(8)]
    g = O.group_pairs(_pairs(rows), 32, 8, 128, 16)
    assert g["sorted"].size == 256 and g["groups"].size <= 74
    assert g["tiles"]["group_count"].max() <= 16 and g["tiles"]["pair_count"].min() > 0
    # histogram and permutation invariants
    assert np.array_equal(g["counts"], np.bincount([r[1] for r in rows], minlength=128))
    key = g["sorted"]["expert"].astype(np.int64) * 10**6 + g["sorted"]["token"] * 10 + g["sorted"]["rank"]
    assert np.all(np.diff(key) > 0)


def test_prefill_moe_synthetic_pool():
    # PrefillGroupedRoutedMoETests.swift:271-280 closed-form weights, silu instead
    # of the test's GeGLU; checked against a float64 dense recomputation.
    d, f, E, T, k = 128, 64, 4, 3, 2

    def rows(expert, role, r, c):
        i, j = np.meshgrid(np.arange(r), np.arange(c), indexing="ij")
        return ((expert + 1) * 1e-3 + (role + 1) * 3e-3 + ((i % 7) - 3) * 4e-4
                + ((j % 11) - 5) * 2e-4).astype(np.float32)
    mats = [(rows(e, 0, f, d), rows(e, 1, f, d), rows(e, 2, d, f)) for e in range(E)]
    blobs = np.stack([O.pack_expert(*m, 4) for m in mats])
    hidden = np.array([[(i % 17) - 8 for i in range(d)]] * T, np.float32) * np.float32(0.125)
    hidden += np.arange(T, dtype=np.float32)[:, None] * np.float32(0.25)
    idx = np.array([[0, 2], [1, 2], [3, 0]], np.uint32)
    w = O.f16_bits(np.array([[0.75, 0.25], [0.5, 0.5], [0.625, 0.375]], np.float32))
    h2 = O.prefill_moe(blobs, 4, hidden, d, f, idx, w)
    for t in range(T):
        want = np.zeros(d)
        for r in range(k):
            g_, u_, d_ = [O.dequantize_affine(*O.quantize_affine(m, 4), m.shape[1], 4).astype(np.float64)
                          for m in mats[idx[t, r]]]
            g = g_ @ hidden[t]
            want += float(O.f16_to_float(w[t, r])) * (d_ @ (g / (1 + np.exp(-g)) * (u_ @ hidden[t])))
        assert np.abs(h2[t] - want).max() <= 1e-4
