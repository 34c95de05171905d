"""The oracle's host index math against the known answers the reference's own unit tests hold
(tests/golden/index_math.json) and against published hash vectors."""
import json
import os

import numpy as np

from oracle import paged_kv_oracle as orc

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "index_math.json")))


def test_fnv1a64_published_vectors():
    for s, h in GOLDEN["public_hash_vectors"]["fnv1a64"].items():
        assert orc.fnv1a64(s) == int(h, 16)


def test_splitmix64_published_vectors():
    g = GOLDEN["public_hash_vectors"]
    rng = orc.SplitMix64(g["splitmix64_seed"])
    expected = [int(x) for x in g["splitmix64_first5"]]
    assert [rng.next_u64() for _ in range(5)] == expected
    assert orc.splitmix64_stream(g["splitmix64_seed"], 5).tolist() == expected


def test_seeded_tensor_matches_scalar_generator():
    key = "qwen2_quant_decode.k_cache"
    rng = orc.SplitMix64(orc.fnv1a64(key))
    u = [rng.next_u64() for _ in range(24)]
    f = orc.seeded_tensor(key, (2, 3, 4), np.float32)
    assert f.shape == (2, 3, 4)
    np.testing.assert_array_equal(f.ravel(), np.array([(x >> 11) * 2.0 ** -53 for x in u], np.float64).astype(np.float32))
    assert (f >= 0).all() and (f <= 1).all()
    i8 = orc.seeded_tensor(key, (24,), np.int8)
    np.testing.assert_array_equal(i8, np.array([-128 + x % 256 for x in u], np.int64).astype(np.int8))
    i32 = orc.seeded_tensor(key, (24,), np.int32)
    np.testing.assert_array_equal(i32, np.array([-(1 << 31) + x % (1 << 32) for x in u], np.int64).astype(np.int32))
    b = orc.seeded_tensor(key, (24,), np.bool_)
    np.testing.assert_array_equal(b, np.array([x & 1 for x in u], bool))


def test_seeded_tensor_reference_statistics():
    """The reference's own known answer for a seeded tensor: min / max / sum of a float32 one."""
    g = GOLDEN["seeded_tensor_stats"]
    t = orc.seeded_tensor(g["key"], tuple(g["shape"]), np.float32).astype(np.float64)
    for got, want in ((t.min(), g["expected_min"]), (t.max(), g["expected_max"]), (t.sum(), g["expected_sum"])):
        assert abs(got - want) <= g["atol"] + g["rtol"] * abs(want), (got, want)
    # tighter than the reference asks: the golden values are the true ones rounded to 3-4 digits
    assert abs(t.min() - g["expected_min"]) < 5e-7 and abs(t.sum() - g["expected_sum"]) < 0.1


def test_batch_test_known_answers():
    g = GOLDEN["batch_test_basic"]
    bs = g["block_size"]
    slots, lists, seq_lens, q_lens, positions = [], [], [], [], []
    for s in g["sequences"]:
        start = s["kv_cache_tokens_before"]
        end = start + s["q_len"]
        assert end == s["seq_len"]
        slots += orc.kv_cache_slots(s["blocks"], bs, start, end)
        positions += list(range(start, end))
        lists.append(s["blocks"])
        seq_lens.append(s["seq_len"])
        q_lens.append(s["q_len"])
    assert slots == g["expected_new_cache_slots"]
    assert positions == g["expected_positions"]
    assert orc.pad_block_tables(lists).tolist() == g["expected_block_tables"]
    cu_kv = np.concatenate([[0], np.cumsum(seq_lens)]).tolist()
    cu_q = np.concatenate([[0], np.cumsum(q_lens)]).tolist()
    assert cu_kv == g["expected_kv_seq_lens_cumulative"]
    assert cu_q == g["expected_q_seq_lens_cumulative"]
    assert orc.attention_metadata_kv_seq_lens(cu_kv).tolist() == g["expected_kv_seq_lens_npu_layout"]
    assert max(seq_lens) == g["expected_kv_max_seq_len"] and max(q_lens) == g["expected_q_max_seq_len"]
    # CSR arrays describe the same block lists
    indptr, indices, last = orc.build_paged_kv_csr(lists, seq_lens, bs)
    assert indptr.tolist() == [0, 3, 7, 12, 15]
    assert indices.tolist() == sum(lists, [])
    assert last.tolist() == [1, 4, 4, 4]


def _check_spec_case(g):
    cu = np.concatenate([[0], np.cumsum(g["kv_seq_lens"])]).tolist()
    pos, slots, kv, tables = orc.expand_decode_rows(g["positions"], cu, g["block_tables"], g["block_size"],
                                                    g["position_offsets"])
    assert pos == g["expected_positions"]
    assert slots == g["expected_new_cache_slots"]
    assert kv == g["expected_kv_seq_lens"]
    return tables


def test_spec_draft_rows_known_answers():
    _check_spec_case(GOLDEN["spec_draft_single_row"])


def test_spec_validate_expansion_known_answers():
    g = GOLDEN["spec_validate_expansion"]
    tables = _check_spec_case(g)
    assert len(tables) == g["expected_num_block_table_rows"]
    assert tables[0] == tables[1] == tables[2] == g["block_tables"][0]


def test_calc_slot_id_errors():
    import pytest

    with pytest.raises(IndexError):
        orc.calc_slot_id(12, [0, 1, 2], 4)  # block index 3 is out of range (spec_input_builder_test.cpp:335-341)
    with pytest.raises(ValueError):
        orc.calc_slot_id(-1, [0], 4)
    with pytest.raises(ValueError):
        orc.calc_slot_id(0, [-1], 4)


def test_minimal_decode_metadata():
    g = GOLDEN["minimal_decode_metadata"]
    assert orc.attention_metadata_kv_seq_lens(g["kv_seq_lens_cumulative"]).tolist() == g["expected_kv_seq_lens"]
    indptr, indices, last = orc.build_paged_kv_csr(g["block_tables"], g["expected_kv_seq_lens"], g["block_size"])
    assert indptr.tolist() == g["paged_kv_indptr"]
    assert indices.tolist() == g["paged_kv_indices"]
    assert last.tolist() == g["paged_kv_last_page_len"]
    assert orc.kv_cache_slots(g["block_tables"][0], g["block_size"], 3, 4) == g["new_cache_slots"]
