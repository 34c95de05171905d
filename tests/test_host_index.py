"""The C++ host-side index producers (xllm_wxh_amd/csrc/torch_shim/host_index.h) against the known
answers the reference's own unit tests hold (tests/golden/index_math.json), against the oracle on
random batches, and — on the GPU — feeding a whole write-then-attend step."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import build as xbuild

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "index_math.json")))


@pytest.fixture(scope="module")
def shim():
    if not os.path.exists(xbuild.TORCH_SHIM_PATH):
        xbuild.build_torch_shim(verbose=False)
    from xllm_wxh_amd import _xllm_hip_torch

    return _xllm_hip_torch


def test_batch_test_known_answers(shim):
    g = GOLDEN["batch_test_basic"]
    batch = shim.DecodeBatchInputs(g["block_size"])
    for s in g["sequences"]:
        batch.add_sequence(s["blocks"], s["kv_cache_tokens_before"], s["seq_len"])
    assert batch.positions == g["expected_positions"]
    assert batch.new_cache_slots == g["expected_new_cache_slots"]
    assert batch.q_seq_lens == g["expected_q_seq_lens_cumulative"]
    assert batch.kv_seq_lens == g["expected_kv_seq_lens_cumulative"]
    assert batch.padded_block_tables() == g["expected_block_tables"]
    assert batch.q_max_seq_len == g["expected_q_max_seq_len"]
    assert batch.kv_max_seq_len == g["expected_kv_max_seq_len"]
    assert batch.paged_kv_indptr == [0, 3, 7, 12, 15]
    assert batch.paged_kv_indices == sum((s["blocks"] for s in g["sequences"]), [])
    assert batch.paged_kv_last_page_len == [1, 4, 4, 4]
    # blocks from the first written position on: seq1 all, seq2 block 1 of 4.. , seq3 block 3.., seq4 block 1..
    assert batch.write_block_ids == {1, 2, 3, 5, 6, 7, 11, 12, 14, 15}
    md = shim.build_decode_metadata(batch, "cpu")
    md.plan_info.layer_id = 0
    assert md.kv_seq_lens.tolist() == g["expected_kv_seq_lens_npu_layout"]
    assert md.block_table.tolist() == g["expected_block_tables"]
    assert md.slot_mapping.tolist() == g["expected_new_cache_slots"]
    assert md.paged_kv_indptr.tolist() == [0, 3, 7, 12, 15] and md.total_kv_len == 41


@pytest.mark.parametrize("name", ["spec_draft_single_row", "spec_validate_expansion"])
def test_spec_rows_known_answers(shim, name):
    g = GOLDEN[name]
    cu = np.concatenate([[0], np.cumsum(g["kv_seq_lens"])]).tolist()
    rows = shim.expand_decode_rows(g["positions"], cu, g["block_tables"], g["block_size"], g["position_offsets"])
    assert rows.positions == g["expected_positions"]
    assert rows.new_cache_slots == g["expected_new_cache_slots"]
    assert rows.kv_seq_lens == g["expected_kv_seq_lens"]
    assert rows.kv_max_seq_len == max(g["expected_kv_seq_lens"])
    if "expected_num_block_table_rows" in g:
        assert len(rows.block_tables) == g["expected_num_block_table_rows"]
        assert rows.block_tables[0] == rows.block_tables[2] == g["block_tables"][0]


@pytest.mark.parametrize("name", ["spec_first_decode_rows", "spec_rows_with_offsets", "spec_rows_from_last_step"])
def test_spec_rows_with_their_own_offsets(shim, name):
    g = GOLDEN[name]
    cu = np.concatenate([[0], np.cumsum(g["kv_seq_lens"])]).tolist()
    rows = shim.decode_rows(g["positions"], cu, g["block_tables"], g["block_size"], [tuple(r) for r in g["rows"]])
    assert rows.positions == g["expected_positions"]
    assert rows.new_cache_slots == g["expected_new_cache_slots"]
    assert rows.kv_seq_lens == g["expected_kv_seq_lens"]
    assert len(rows.block_tables) == len(g["rows"])
    # and the oracle's restatement
    for (seq, off), pos, slot, kv in zip(g["rows"], g["expected_positions"], g["expected_new_cache_slots"],
                                         g["expected_kv_seq_lens"]):
        assert g["positions"][seq] + off == pos
        assert orc.calc_slot_id(pos, g["block_tables"][seq], g["block_size"]) == slot
        assert orc.calc_kv_len(cu, seq, off) == kv


def test_minimal_decode_metadata(shim):
    g = GOLDEN["minimal_decode_metadata"]
    batch = shim.DecodeBatchInputs(g["block_size"])
    batch.add_sequence(g["block_tables"][0], 3, 4)
    assert batch.kv_seq_lens == g["kv_seq_lens_cumulative"] and batch.q_seq_lens == g["q_seq_lens_cumulative"]
    assert batch.new_cache_slots == g["new_cache_slots"]
    assert batch.paged_kv_indptr == g["paged_kv_indptr"] and batch.paged_kv_indices == g["paged_kv_indices"]
    assert batch.paged_kv_last_page_len == g["paged_kv_last_page_len"]


def test_errors(shim):
    with pytest.raises(IndexError):
        shim.calc_slot_id(12, [0, 1, 2], 4)  # block index 3 is out of range (spec_input_builder_test.cpp:335-341)
    with pytest.raises(ValueError):
        shim.calc_slot_id(-1, [0], 4)
    with pytest.raises(ValueError):
        shim.calc_slot_id(0, [-1], 4)
    with pytest.raises(ValueError):
        shim.kv_cache_slots([], 4, 0, 1)
    with pytest.raises(IndexError):
        shim.calc_kv_len([0, 5], 1, 0)
    assert shim.calc_kv_len([0, 5, 14], 1, 2) == 11


def test_padding_rows_write_slot_zero(shim):
    """padding_decode_batch_size (batch_input_builder.cpp:496-537): rows added up to a fixed batch size
    write slot 0 and own block 0 with one token."""
    batch = shim.DecodeBatchInputs(16)
    batch.add_sequence([5, 6], 17, 18)
    batch.add_sequence([9], 3, 4)
    batch.pad_decode_batch(1, 4)
    assert batch.num_sequences() == 4
    assert batch.new_cache_slots == [5 * 16 + 16 + 1, 9 * 16 + 3, 0, 0]
    assert batch.kv_seq_lens == [0, 18, 22, 23, 24] and batch.q_seq_lens == [0, 1, 2, 3, 4]
    assert batch.padded_block_tables() == [[5, 6], [9, 0], [0, 0], [0, 0]]
    assert batch.paged_kv_indptr == [0, 2, 3, 4, 5] and batch.paged_kv_last_page_len == [2, 4, 1, 1]
    # a mixed step is not padded
    mixed = shim.DecodeBatchInputs(16)
    mixed.add_sequence([1], 0, 5)
    mixed.pad_decode_batch(1, 4)
    assert mixed.num_sequences() == 1


def test_random_batches_match_the_oracle(shim):
    rng = np.random.default_rng(11)
    for _ in range(20):
        bs = int(rng.choice([1, 4, 16, 128]))
        B = int(rng.integers(1, 9))
        batch = shim.DecodeBatchInputs(bs)
        lists, lens, slots, next_block = [], [], [], 1
        for _b in range(B):
            seq_len = int(rng.integers(1, 300))
            q_len = int(rng.integers(1, min(seq_len, 8) + 1))
            nb = (seq_len + bs - 1) // bs
            blocks = list(range(next_block, next_block + nb))
            rng.shuffle(blocks)
            next_block += nb
            batch.add_sequence(blocks, seq_len - q_len, seq_len)
            lists.append(blocks)
            lens.append(seq_len)
            slots += orc.kv_cache_slots(blocks, bs, seq_len - q_len, seq_len)
        assert batch.new_cache_slots == slots
        assert batch.padded_block_tables() == orc.pad_block_tables(lists).tolist()
        indptr, indices, last = orc.build_paged_kv_csr(lists, lens, bs)
        assert batch.paged_kv_indptr == indptr.tolist() and batch.paged_kv_indices == indices.tolist()
        assert batch.paged_kv_last_page_len == last.tolist()


@pytest.mark.gpu
def test_builder_feeds_a_write_then_attend_step(gpu, shim):
    """Host arrays from DecodeBatchInputs -> AttentionMetadata on the device -> AttentionImpl::forward:
    the new tokens land in the slots the builder computed and the output is the oracle's."""
    print("case host index builder -> AttentionImpl", flush=True)
    Hq, Hkv, D, bs = 32, 8, 128, 16
    lens = [300, 17, 1, 1000, 64]
    rng = np.random.default_rng(4)
    nblocks = sum((l + bs - 1) // bs for l in lens) + 1
    perm = (rng.permutation(nblocks - 1) + 1).tolist()
    batch = shim.DecodeBatchInputs(bs)
    o = 0
    for l in lens:
        nb = (l + bs - 1) // bs
        batch.add_sequence(perm[o:o + nb], l - 1, l)
        o += nb
    md = shim.build_decode_metadata(batch, "cuda:0")
    md.plan_info.layer_id = 0
    # a ragged batch: the step's schedule is made on the host from the builder's own lengths; equal lengths keep
    # the device-side plan
    assert list(md.plan_info.kv_lens_host) == lens
    even = shim.DecodeBatchInputs(bs)
    for i in range(4):
        even.add_sequence(perm[4 * i: 4 * i + 4], 63, 64)
    assert list(shim.build_decode_metadata(even, "cuda:0").plan_info.kv_lens_host) == []
    g = torch.Generator().manual_seed(8)
    kc = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16)
    q = torch.randn(len(lens), Hq * D, generator=g).to(torch.bfloat16)
    nk = torch.randn(len(lens), Hkv * D, generator=g).to(torch.bfloat16)
    nv = torch.randn(len(lens), Hkv * D, generator=g).to(torch.bfloat16)
    k_ref, v_ref = kc.view(torch.int16).numpy().copy(), vc.view(torch.int16).numpy().copy()
    orc.reshape_paged_cache(np.array(batch.new_cache_slots), nk.view(torch.int16).numpy().reshape(-1, Hkv, D),
                            nv.view(torch.int16).numpy().reshape(-1, Hkv, D), k_ref, v_ref, "HND")
    table = np.array(batch.padded_block_tables(), np.int32)
    ref, _ = orc.paged_decode(q.float().numpy().reshape(-1, Hq, D),
                              torch.from_numpy(k_ref).view(torch.bfloat16).float().numpy(),
                              torch.from_numpy(v_ref).view(torch.bfloat16).float().numpy(), table,
                              np.array(lens, np.int32), 1.0 / np.sqrt(D))
    cache = shim.KVCache(kc.to(gpu), vc.to(gpu))
    attn = shim.AttentionImpl(Hq, D, 1.0 / float(np.sqrt(D)), Hkv, -1)
    out, _ = attn.forward(md, q.to(gpu), nk.to(gpu), nv.to(gpu), cache)
    torch.cuda.synchronize()
    assert np.array_equal(cache.get_k_cache().cpu().view(torch.int16).numpy(), k_ref)
    assert np.array_equal(cache.get_v_cache().cpu().view(torch.int16).numpy(), v_ref)
    err = float(np.abs(out.float().cpu().numpy().reshape(ref.shape) - ref).max())
    assert err <= 2e-2, err
