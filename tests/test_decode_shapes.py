"""Which shape of work item a decode step gets, decided on the host (`xllm_hip_paged_decode_describe`: no GPU,
nothing is launched).  The expectations are the rules the kernels' measurements led to: eight-wave items for
small steps over 1-byte caches, a wave per (sequence, kv head) for large batches of short sequences where such
workgroups fill their rounds, the sequences of a partly filled last round cut finer — and, for every step, no
more sequence-chunk slots than the workspace holds."""
import ctypes

import numpy as np
import pytest

from xllm_wxh_amd import _lib

FIELDS = ("workgroups", "waves", "unsplit", "stored", "chunk", "slots_per_cut_seq", "kept_seqs", "kept_slots",
          "kept_chunk", "heads_per_item", "items_per_workgroup", "fused_merge", "slots_held", "slots_used")


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def describe(lib, B, L, kv="bf16", Hq=32, Hkv=8, D=128, n=1, bs=16, layout="HND", hints=True, total=None, longest=None):
    desc = _lib.KvCacheDesc()
    desc.k_cache, desc.v_cache = 0x10000, 0x20000
    desc.num_blocks, desc.block_size, desc.num_kv_heads, desc.head_dim = 1 << 20, bs, Hkv, D
    desc.dtype = {"bf16": _lib.BF16, "fp8": _lib.FP8_E4M3, "int8": _lib.INT8}[kv]
    if layout == "HND":
        desc.stride_block, desc.stride_head, desc.stride_slot = Hkv * bs * D, bs * D, D
        sb, sh, ss = Hkv * bs, bs, 1
    else:
        desc.stride_block, desc.stride_head, desc.stride_slot = Hkv * bs * D, D, Hkv * D
        sb, sh, ss = Hkv * bs, 1, Hkv
    if kv != "bf16":
        desc.k_scale, desc.v_scale = 0x30000, 0x40000
        desc.scale_stride_block, desc.scale_stride_head, desc.scale_stride_slot = sb, sh, ss
    args = _lib.DecodeArgs()
    args.q, args.out = 0x50000, 0x60000
    args.batch, args.q_per_seq, args.num_q_heads, args.q_dtype = B, n, Hq, _lib.BF16
    args.q_token_stride = args.out_token_stride = Hq * D
    args.block_table, args.seq_lens = 0x70000, 0x80000
    args.max_blocks_per_seq = args.block_table_stride = (L + bs - 1) // bs + 1
    args.sm_scale = 0.088
    args.window_left = -1
    if hints:
        args.max_seq_len = L if longest is None else longest
        args.total_kv_len = B * L if total is None else total
    out = (ctypes.c_int64 * len(FIELDS))()
    _lib.check(lib.xllm_hip_paged_decode_describe(ctypes.byref(desc), ctypes.byref(args), 0, out, len(FIELDS)))
    return dict(zip(FIELDS, list(out)))


def test_headline_shape_is_one_launch_of_whole_items(lib):
    d = describe(lib, 64, 4096)
    assert (d["workgroups"], d["waves"], d["unsplit"], d["stored"]) == (512, 4, 1, 0)


def test_without_lengths_a_split_step_stores_its_schedule(lib):
    d = describe(lib, 4, 32768, hints=False)
    assert d["unsplit"] == 0 and d["stored"] == 1 and d["fused_merge"] == 1 and d["waves"] == 4
    d = describe(lib, 4, 32768)
    assert d["stored"] == 0 and d["slots_per_cut_seq"] == 8 and d["workgroups"] == 256  # one workgroup per CU


def test_small_steps_over_one_byte_caches_run_eight_waves(lib):
    for kv in ("fp8", "int8"):
        d = describe(lib, 1, 32768, kv=kv, Hq=64)
        assert (d["workgroups"], d["waves"], d["slots_per_cut_seq"]) == (256, 8, 32)
        d = describe(lib, 32, 8192, kv=kv, Hq=64)
        assert (d["workgroups"], d["waves"], d["unsplit"]) == (256, 8, 1)
        # many CUs would stay empty: every slot gets a four-wave item instead
        d = describe(lib, 20, 8192, kv=kv, Hq=64)
        assert d["waves"] == 4 and d["workgroups"] == 480
    assert describe(lib, 1, 32768)["waves"] == 4  # 16-bit caches keep four


def test_a_wave_per_sequence_and_head_where_such_workgroups_fill_their_rounds(lib):
    d = describe(lib, 1024, 512, kv="fp8", Hq=64)
    assert (d["heads_per_item"], d["workgroups"], d["unsplit"]) == (4, 2048, 1)
    assert describe(lib, 256, 2048, kv="fp8", Hq=64)["heads_per_item"] == 4
    # 1.125 rounds of four-head workgroups: an item per head
    assert describe(lib, 288, 2048, kv="fp8", Hq=64)["heads_per_item"] == 1
    # long sequences, or few items: an item per head
    assert describe(lib, 256, 16384, kv="fp8", Hq=64)["heads_per_item"] == 1
    assert describe(lib, 2048, 128)["heads_per_item"] == 4 and describe(lib, 2048, 512)["heads_per_item"] == 1
    # head counts that are no multiple of four: four neighbouring items per workgroup
    d = describe(lib, 2048, 1024, kv="fp8", Hq=8, Hkv=1)
    assert (d["items_per_workgroup"], d["workgroups"], d["heads_per_item"]) == (4, 512, 1)
    # half as many items: two waves per item
    d = describe(lib, 128, 2048, kv="fp8", Hq=64)
    assert (d["items_per_workgroup"], d["workgroups"]) == (2, 512)
    assert describe(lib, 192, 2048, kv="fp8", Hq=64)["items_per_workgroup"] == 1  # 1.5 rounds
    # ragged lengths: from 2048 four-head items on, over the stored schedule
    d = describe(lib, 1024, 512, kv="fp8", Hq=64, total=1024 * 300, longest=4000)
    assert d["heads_per_item"] == 4 and d["stored"] == 1
    d = describe(lib, 256, 2048, kv="fp8", Hq=64, total=256 * 1200, longest=8000)
    assert d["heads_per_item"] == 1


def test_nhd_one_byte_caches_take_four_heads_per_item_unless_rounds_fill_poorly(lib):
    assert describe(lib, 128, 8192, kv="fp8", Hq=64, layout="NHD")["heads_per_item"] == 4
    assert describe(lib, 160, 4096, kv="fp8", Hq=64, layout="NHD")["heads_per_item"] == 1
    assert describe(lib, 128, 8192, kv="fp8", Hq=64, layout="NHD", hints=False)["heads_per_item"] == 4
    assert describe(lib, 128, 8192, layout="NHD")["heads_per_item"] == 1  # 16-bit rows are long enough


def test_the_last_rounds_sequences_are_cut(lib):
    d = describe(lib, 66, 8192, kv="fp8", Hq=64)
    assert d["kept_seqs"] == 64 and d["kept_slots"] == 1 and d["slots_per_cut_seq"] >= 8 and d["unsplit"] == 0
    assert d["workgroups"] == (64 + 2 * d["slots_per_cut_seq"]) * 8 and d["fused_merge"] == 1
    # 16-bit caches: a round is an item per CU
    d = describe(lib, 33, 8192)
    assert d["kept_seqs"] == 32 and d["slots_per_cut_seq"] == 16 and d["workgroups"] == (32 + 16) * 8
    assert describe(lib, 64, 8192)["unsplit"] == 1 and describe(lib, 60, 8192)["unsplit"] == 1
    # 1-byte caches a little past an item per CU: eight waves, whole items and chunks alike
    d = describe(lib, 36, 8192, kv="fp8", Hq=64)
    assert d["waves"] == 8 and d["kept_seqs"] == 32 and d["kept_slots"] == 1
    # ... further past it: cut in two throughout, the last sequences finer
    d = describe(lib, 41, 8192, kv="fp8", Hq=64)
    assert d["waves"] == 4 and d["kept_slots"] == 2 and d["slots_per_cut_seq"] >= 6
    assert describe(lib, 48, 8192, kv="fp8", Hq=64)["unsplit"] == 1
    # not from 2048 items on
    assert describe(lib, 288, 2048, kv="fp8", Hq=64)["unsplit"] == 1
    # the 32-row kernel (four draft tokens, eight query heads per kv head)
    d = describe(lib, 66, 32768, kv="int8", Hq=64, n=4, bs=128)
    assert d["waves"] == 2 and d["kept_seqs"] == 64 and d["kept_slots"] == 2 and d["slots_per_cut_seq"] == 32
    d = describe(lib, 64, 32768, kv="int8", Hq=64, n=4, bs=128)
    assert d["kept_seqs"] == 0 and d["slots_per_cut_seq"] == 2 and d["workgroups"] == 1024


@pytest.mark.parametrize("seed", range(4))
def test_no_step_addresses_more_chunk_slots_than_the_workspace_holds(lib, seed):
    rng = np.random.default_rng(seed)
    for _ in range(1500):
        Hkv = int(rng.choice([1, 2, 4, 8]))
        n = int(rng.choice([1, 1, 2, 4]))
        g = int(rng.choice([1, 2, 4, 8]))
        D = int(rng.choice([64, 128, 256]))
        kv = str(rng.choice(["bf16", "fp8", "int8"]))
        bs = int(rng.choice([32, 64, 128]))
        B = int(rng.choice([1, 2, 7, 20, 33, 40, 64, 66, 72, 130, 200, 288, 520, 1024, 2050]))
        L = int(rng.choice([100, 512, 2048, 8192, 40000]))
        kind = rng.random()
        total = B * L if kind < 0.6 else int(B * L * rng.uniform(0.3, 1.0))
        d = describe(lib, B, L, kv=kv, Hq=Hkv * g, Hkv=Hkv, D=D, n=n, bs=bs, layout=str(rng.choice(["HND", "NHD"])),
                     hints=kind < 0.9, total=max(1, total))
        assert d["slots_used"] <= d["slots_held"], (B, L, kv, Hkv, g, n, D, d)
        assert d["workgroups"] >= 1 and d["waves"] in (1, 2, 4, 8)
