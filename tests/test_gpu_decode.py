"""Paged-attention decode on the GPU against the fp32 oracle, through the C ABI.

Tolerances (max-abs error of the output): 2e-2 for a bf16 KV cache, 5e-2 for fp8/int8 KV caches
(compared with attention over the dequantised cache).  Tighter regression bounds are checked as well.
The MFMA kernel rounds the probabilities to bf16 before the second MFMA (as tensor-core attention
kernels do) and the output to bf16: each costs up to 2^-9 relative, i.e. about 1e-2 absolute on
N(0,1) values when a sequence has only a handful of tokens (REG_TOL), and it averages out on long
ones.  With a quantised cache the rounded weight is p * v_scale (REG_TOL_QUANT).
"""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.helpers import Case, TOL_BF16_KV, TOL_QUANT_KV, lse_err, max_abs_err, max_rel_err_per_seq
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu

REG_TOL = 1.2e-2
REG_TOL_QUANT = 2.5e-2
LSE_TOL = 1e-4
# ... and relative to the size of the outputs: max-abs error of a sequence's rows within this fraction
# of their RMS (16-bit weights and outputs: a few units of 2^-9 of the largest elements)
REL_TOL = 3e-2


def _check(case, window_left=-1, **kw):
    ref, lse_ref = case.oracle(window_left)
    out, lse = case.run(window_left, **kw)
    assert not torch.isnan(out.float()).any()
    e = max_abs_err(out, ref)
    le = lse_err(lse, lse_ref)
    re = max_rel_err_per_seq(out, ref, case.n)
    print("   variant=%s err=%.3e rel_err=%.3e lse_err=%.3e" % (case.variant(), e, re, le), flush=True)
    assert e <= case.tol, e
    assert e <= (REG_TOL_QUANT if case.kv in ("fp8", "int8") else REG_TOL), e
    assert re <= REL_TOL, re
    assert le <= LSE_TOL, le
    return out, lse


SHAPES = [
    # B, Hq, Hkv, D, bs, lens, n
    (2, 8, 2, 128, 16, [100, 33], 1),
    (4, 32, 8, 128, 16, [1, 31, 32, 33], 1),
    (3, 32, 8, 128, 16, [4096, 777, 128], 1),      # chunk boundaries of the split
    (3, 32, 8, 128, 128, [4096, 129, 127], 1),
    (2, 64, 8, 128, 32, [555, 64], 1),
    (2, 8, 8, 128, 64, [300, 17], 1),              # MHA, g = 1
    (2, 56, 8, 128, 16, [300, 517], 1),            # g = 7
    (2, 64, 8, 128, 128, [3000, 517], 4),          # 32 query rows per kv head: two MFMA tiles
    (2, 64, 4, 128, 16, [700, 90], 4),             # 64 rows: two row groups
    (3, 32, 8, 128, 16, [5, 2, 3], 2),             # draft tokens at the very start of a sequence
]


@pytest.mark.parametrize("kv", ["bf16", "fp8", "int8"])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "B%d_Hq%d_Hkv%d_D%d_bs%d_n%d_L%d" % (s[0], s[1], s[2], s[3], s[4], s[6], max(s[5])))
def test_mfma_decode_matches_oracle(gpu, shape, kv):
    B, Hq, Hkv, D, bs, lens, n = shape
    print("case mfma", shape, kv, flush=True)
    case = Case(B, Hq, Hkv, D, bs, lens, n=n, kv=kv, seed=11)
    assert case.variant() == "mfma_d128"
    _check(case)


@pytest.mark.parametrize("kv", ["fp16", "fp8", "int8"])
@pytest.mark.parametrize("shape", [SHAPES[1], SHAPES[2], SHAPES[7], SHAPES[9]],
                         ids=lambda s: "B%d_Hq%d_n%d_L%d" % (s[0], s[1], s[6], max(s[5])))
def test_mfma_decode_fp16_queries(gpu, shape, kv):
    """fp16 queries and outputs: the MFMA kernels compute in fp16 (an fp16 cache as it is, e4m3 and
    int8 caches converted exactly)."""
    B, Hq, Hkv, D, bs, lens, n = shape
    print("case mfma fp16", shape, kv, flush=True)
    case = Case(B, Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt="fp16", seed=12)
    assert case.variant() == "mfma_d128"
    out, _ = _check(case)
    assert out.dtype == torch.float16


SHAPES_D64 = [
    # B, Hq, Hkv, D, bs, lens, n
    (4, 32, 8, 64, 32, [1, 2, 63, 65], 1),          # odd lengths: the second token of the last row is masked
    (3, 32, 8, 64, 32, [4096, 777, 128], 1),        # chunk boundaries of the split
    (3, 14, 2, 64, 128, [4097, 129, 64], 1),        # g = 7
    (2, 64, 8, 64, 64, [3001, 517], 4),             # 32 query rows per kv head: the two-wave kernel
    (2, 64, 4, 64, 32, [700, 91], 4),               # two row groups
    (3, 32, 8, 64, 32, [5, 2, 3], 2),               # draft tokens at the very start of a sequence
]


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp8", "bf16"), ("int8", "bf16"), ("fp16", "fp16"), ("int8", "fp16")])
@pytest.mark.parametrize("shape", SHAPES_D64, ids=lambda s: "B%d_Hq%d_Hkv%d_bs%d_n%d_L%d" % (s[0], s[1], s[2], s[4], s[6], max(s[5])))
def test_mfma_decode_head_dim_64(gpu, shape, kv, qdt):
    """head_dim 64 runs on the MFMA kernels with two tokens per tile row."""
    B, Hq, Hkv, D, bs, lens, n = shape
    print("case mfma d64", shape, kv, qdt, flush=True)
    case = Case(B, Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=21)
    assert case.variant() == "mfma_d64"
    _check(case)


@pytest.mark.parametrize("kv", ["bf16", "fp8", "int8"])
def test_head_dim_64_nhd_layout(gpu, kv):
    """NHD: the two tokens of a tile row are not adjacent in memory."""
    print("case d64 nhd", kv, flush=True)
    case = Case(3, 16, 4, 64, 32, [700, 33, 64], layout="NHD", kv=kv, seed=22)
    assert case.variant() == "mfma_d64"
    _check(case)


SHAPES_D256 = [
    # B, Hq, Hkv, D, bs, lens, n
    (4, 16, 4, 256, 16, [1, 15, 16, 17], 1),         # sequence ends inside and at the edge of a 16-token tile
    (3, 32, 8, 256, 16, [4096, 777, 128], 1),        # chunk boundaries of the split
    (3, 14, 2, 256, 128, [4097, 129, 64], 1),        # g = 7
    (2, 8, 8, 256, 64, [300, 17], 1),                # MHA, g = 1
    (2, 64, 8, 256, 64, [3001, 517], 4),             # 32 query rows per kv head: the two-wave kernel
    (2, 64, 4, 256, 32, [700, 91], 4),               # two row groups
    (3, 32, 8, 256, 32, [5, 2, 3], 2),               # draft tokens at the very start of a sequence
    (2, 32, 8, 256, 16, [600, 90], 40),              # a prefill chunk: row groups of 32
]


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp8", "bf16"), ("int8", "bf16"), ("fp16", "fp16"), ("int8", "fp16")])
@pytest.mark.parametrize("shape", SHAPES_D256, ids=lambda s: "B%d_Hq%d_Hkv%d_bs%d_n%d_L%d" % (s[0], s[1], s[2], s[4], s[6], max(s[5])))
def test_mfma_decode_head_dim_256(gpu, shape, kv, qdt):
    """head_dim 256 runs on the MFMA kernels with two tile rows per token (16-token tiles)."""
    B, Hq, Hkv, D, bs, lens, n = shape
    print("case mfma d256", shape, kv, qdt, flush=True)
    case = Case(B, Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=31)
    assert case.variant() == "mfma_d256"
    _check(case)


@pytest.mark.parametrize("kv", ["bf16", "fp8", "int8"])
def test_head_dim_256_nhd_layout_and_window(gpu, kv):
    print("case d256 nhd", kv, flush=True)
    case = Case(3, 16, 4, 256, 32, [700, 33, 64], layout="NHD", kv=kv, seed=32)
    assert case.variant() == "mfma_d256"
    _check(case)
    case = Case(2, 32, 8, 256, 32, [3000, 517], n=2, kv=kv, seed=33)
    _check(case, window_left=301)


def test_head_dim_256_equals_generic_kernel(gpu, lib_option):
    print("case d256 vs generic", flush=True)
    case = Case(3, 32, 8, 256, 16, [1500, 40, 333], kv="int8", seed=34)
    out, lse = case.run()
    lib_option("force_generic")
    assert case.variant() == "generic"
    out_g, lse_g = case.run()
    assert max_abs_err(out, out_g.float().cpu().numpy()) <= 2e-2
    assert float((lse - lse_g).abs().max()) <= 1e-4


def test_head_dim_64_small_blocks_take_the_generic_kernel(gpu):
    print("case d64 bs16", flush=True)
    case = Case(2, 8, 2, 64, 16, [100, 33], seed=22)  # half a tile would straddle two blocks
    assert case.variant() == "generic"
    _check(case)


def test_head_dim_64_sliding_window(gpu):
    print("case d64 window", flush=True)
    for kv in ("bf16", "int8"):
        case = Case(2, 32, 8, 64, 32, [3000, 517], n=2, kv=kv, seed=23)
        assert case.variant() == "mfma_d64"
        _check(case, window_left=301)


def test_mixed_16_bit_types_take_the_generic_kernel(gpu):
    print("case mixed 16-bit", flush=True)
    for kv, qdt in (("bf16", "fp16"), ("fp16", "bf16")):
        case = Case(2, 8, 2, 128, 16, [100, 33], kv=kv, qdt=qdt, seed=13)
        assert case.variant() == "generic"
        _check(case)


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp32", "fp32"), ("fp16", "fp16"), ("fp8", "bf16"), ("int8", "bf16")])
@pytest.mark.parametrize("shape", [
    (2, 14, 2, 64, 16, [300, 17], 1),
    (2, 8, 2, 128, 16, [260, 33], 2),
    (2, 6, 3, 80, 8, [70, 9], 1),
    (1, 4, 1, 256, 16, [50], 1),
], ids=lambda s: "Hq%d_Hkv%d_D%d_bs%d_n%d" % (s[1], s[2], s[3], s[4], s[6]))
def test_generic_decode_matches_oracle(gpu, shape, kv, qdt, lib_option):
    B, Hq, Hkv, D, bs, lens, n = shape
    print("case generic", shape, kv, qdt, flush=True)
    lib_option("force_generic")
    case = Case(B, Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=5)
    assert case.variant() == "generic"
    ref, lse_ref = case.oracle()
    out, lse = case.run()
    e = max_abs_err(out, ref)
    print("   err=%.3e" % e, flush=True)
    assert e <= (1e-4 if qdt == "fp32" else 6e-3)  # the generic kernel keeps the probabilities in fp32
    assert lse_err(lse, lse_ref) <= LSE_TOL


@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_nhd_layout_and_csr_form(gpu, kv):
    print("case nhd/csr", kv, flush=True)
    lens = [1000, 77, 16, 4000]
    a = Case(4, 32, 8, 128, 16, lens, kv=kv, layout="HND", seed=3)
    b = Case(4, 32, 8, 128, 16, lens, kv=kv, layout="NHD", seed=3)
    out_a, lse_a = _check(a)
    # Over NHD the 16-row kernel gives a work item four kv heads (one per wave), which changes the order of
    # the sums; with one kv head per item only the strides differ and the values are the same bits.
    out_h, lse_h = _check(b)
    assert torch.allclose(out_h.float(), out_a.float(), rtol=2 ** -7, atol=2e-3)
    assert torch.allclose(lse_h, lse_a, rtol=0, atol=LSE_TOL)
    with ops.option("item_per_head"):
        out_b, lse_b = _check(b)
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)
        # CSR form of the same block lists (xllm/core/framework/batch/batch_input_builder.cpp:438-494)
        lists = [a.table[i, : (L + 15) // 16] for i, L in enumerate(lens)]
        indptr, indices, last = orc.build_paged_kv_csr(lists, lens, 16)
        out_c = torch.empty_like(a.q)
        dev = a.q.device
        ops.batch_decode_csr(a.q, b.k_cache, b.v_cache, torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev),
                             torch.from_numpy(last).to(dev), -1, a.scale, out_c, k_cache_scale=b.k_scale,
                             v_cache_scale=b.v_scale, kv_layout="NHD")
        torch.cuda.synchronize()
        assert torch.equal(out_c, out_a)
    table, seq_lens = ops.csr_to_block_table(torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev),
                                             torch.from_numpy(last).to(dev), 16, a.table.shape[1])
    torch.cuda.synchronize()
    assert seq_lens.cpu().tolist() == lens
    np.testing.assert_array_equal(table.cpu().numpy(), a.table)


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp8", "bf16"), ("int8", "bf16"), ("fp16", "fp16"), ("int8", "fp16")])
@pytest.mark.parametrize("Hq,Hkv,n", [(32, 8, 1), (32, 8, 4), (16, 4, 2), (64, 8, 2), (12, 12, 1), (64, 8, 4), (32, 8, 5)])
def test_work_items_of_four_kv_heads_over_nhd(gpu, kv, qdt, Hq, Hkv, n):
    """Over a 1-byte cache whose kv heads lie side by side within a token (NHD) the 16-row kernel at head_dim
    128 gives a work item four neighbouring kv heads, one per wave, each wave attending all of the chunk's
    tokens, and the 32-row kernel (17 to 32 query rows per kv head: the last two shapes) a pair of waves per head,
    eight waves to the workgroup (16-bit caches, and head counts that are no multiple of four, keep one head per item).  Long and short sequences (split into chunks and merged inside the kernel, or by the merge
    kernel), an empty one, host-side lengths (no stored schedule) and none, a sliding window — against the
    oracle, and against the same step with one kv head per item."""
    print("case four heads per item", kv, qdt, Hq, Hkv, n, flush=True)
    lens = [9000, 300, 0, 33, 4100, 17]
    case = Case(len(lens), Hq, Hkv, 128, 16, lens, n=n, kv=kv, qdt=qdt, layout="NHD", seed=93)
    assert case.variant() == "mfma_d128"
    shape = ops.decode_describe(case.q, case.k_cache, case.v_cache, case.block_table, case.seq_lens, case.k_scale, case.v_scale,
                                q_per_seq=n, kv_layout="NHD")
    assert shape["kv_heads_per_item"] == (4 if kv in ("fp8", "int8") and Hkv % 4 == 0 else 1), shape
    if n * (Hq // Hkv) > 16:
        assert shape["waves_per_workgroup"] == (8 if shape["kv_heads_per_item"] == 4 else 2), shape
    tol = {"bf16": REG_TOL, "fp16": 2e-3}.get(kv, REG_TOL_QUANT)
    lse_tol = LSE_TOL
    for window in (-1, 300):
        ref, lse_ref = case.oracle(window)
        out, lse = case.run(window)
        assert not torch.isnan(out.float()).any()
        assert max_abs_err(out, ref) <= tol
        assert lse_err(lse, lse_ref) <= lse_tol
        with ops.option("item_per_head"):
            out_1, lse_1 = case.run(window)
        assert max_abs_err(out_1, ref) <= tol
        assert torch.allclose(out.float(), out_1.float(), rtol=2 ** -6, atol=4e-3)
        with ops.option("separate_merge"):
            out_s, _ = case.run(window)
        assert max_abs_err(out_s, ref) <= tol
    out_h, lse_h = case.run(hints=True)
    ref, lse_ref = case.oracle()
    assert max_abs_err(out_h, ref) <= tol and lse_err(lse_h, lse_ref) <= lse_tol
    # equal lengths with host-side lengths: no stored schedule
    eq = Case(3, Hq, Hkv, 128, 16, [8192] * 3, n=n, kv=kv, qdt=qdt, layout="NHD", seed=94)
    ref, lse_ref = eq.oracle()
    out, lse = eq.run(hints=True)
    assert max_abs_err(out, ref) <= tol and lse_err(lse, lse_ref) <= lse_tol


def test_kv_len_one_returns_value_row_exactly(gpu):
    # xllm/core/runtime/cuda_graph_executor_test.cpp:150-151
    print("case kv_len 1", flush=True)
    case = Case(5, 32, 8, 128, 16, [1, 1, 1, 1, 1], seed=7)
    out, _ = case.run()
    v = case.v_cache.cpu()
    for b in range(5):
        blk = int(case.table[b, 0])
        for h in range(32):
            assert torch.equal(out[b, h].cpu(), v[blk, h // 4, 0])


def test_fp8_bytes_decode_to_e4m3fn_values(gpu):
    """Known-answer test of the in-register dequant: kv_len 1, scale 1 -> the output is the fp8 value."""
    print("case fp8 KAT", flush=True)
    bytes_ = torch.arange(256, dtype=torch.uint8)
    bytes_ = bytes_[(bytes_ & 0x7F) != 0x7F]  # skip the two NaN encodings
    vals = orc.e4m3fn_to_float(bytes_.numpy())
    n = bytes_.numel()  # 254
    B, Hkv, D, bs = 2, 1, 128, 16
    kc = torch.zeros(B + 1, Hkv, bs, D, dtype=torch.uint8)
    vc = torch.zeros(B + 1, Hkv, bs, D, dtype=torch.uint8)
    vc[1, 0, 0, :] = bytes_[:128]
    vc[2, 0, 0, :n - 128] = bytes_[128:]
    dev = gpu
    q = torch.randn(B, 4, D).to(torch.bfloat16).to(dev)
    out = torch.empty_like(q)
    ones = torch.ones(B + 1, Hkv, bs, device=dev)
    ops.batch_decode(q, kc.view(torch.float8_e4m3fn).to(dev), out, torch.tensor([[1], [2]], dtype=torch.int32, device=dev),
                     torch.tensor([1, 1], dtype=torch.int32, device=dev), vc.view(torch.float8_e4m3fn).to(dev), None, None,
                     ones, ones, scale=1.0, kv_cache_quant_bit_size=8)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    np.testing.assert_array_equal(got[0, 0], vals[:128])
    np.testing.assert_array_equal(got[1, 2, : n - 128], vals[128:])
    assert got[0, 0, 0x7E] == 448.0 and got[0, 0, 0x08] == 2.0 ** -6


def test_block_table_permutation_invariance_is_bitwise(gpu):
    print("case permutation", flush=True)
    case = Case(3, 32, 8, 128, 16, [2000, 333, 48], seed=9)
    out, lse = case.run()
    perm = torch.randperm(case.nblocks, generator=torch.Generator().manual_seed(0))
    k2, v2 = torch.empty_like(case.k_cache), torch.empty_like(case.v_cache)
    k2[perm.to(gpu)] = case.k_cache
    v2[perm.to(gpu)] = case.v_cache
    table2 = perm[torch.from_numpy(case.table).long()].to(torch.int32).to(gpu)
    out2 = torch.empty_like(out)
    ops.batch_decode(case.q, k2, out2, table2, case.seq_lens, v2, scale=case.scale)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("D", [128, 256])
@pytest.mark.parametrize("kv", ["bf16", "fp8"])
def test_garbage_outside_the_sequence_is_ignored(gpu, kv, D):
    """Slots past seq_len, padded block-table entries and unused blocks may hold anything (NaN included)."""
    print("case garbage", kv, D, flush=True)
    lens = [37, 16, 1000, 5]
    case = Case(4, 32, 8, D, 16, lens, kv=kv, seed=13)
    ref_out, _ = case.run()
    used = np.zeros((case.nblocks, 16), bool)
    for b, L in enumerate(lens):
        for t in range(L):
            used[case.table[b, t // 16], t % 16] = True
    mask = torch.from_numpy(~used).to(gpu)  # [blocks, slots]
    nan_bits = 0x7F if kv == "fp8" else None
    for cache in (case.k_cache, case.v_cache):
        c = cache.permute(0, 2, 1, 3)  # [blocks, slots, heads, dim] view
        if kv == "fp8":
            c.view(torch.uint8)[mask] = nan_bits
        else:
            c[mask] = float("nan")
    if case.k_scale is not None:
        case.k_scale.permute(0, 2, 1)[mask] = float("nan")
        case.v_scale.permute(0, 2, 1)[mask] = float("inf")
    # padded entries of the block table point at a block full of NaN (block 0 is never used by make_tables)
    out, _ = case.run()
    assert torch.equal(out, ref_out)


def test_verify_rows_equal_expanded_decode_rows(gpu):
    """n draft tokens with the causal mask == n expanded decode rows with kv lens L-n+1..L
    (xllm/core/runtime/speculative_worker_impl.cpp:230-243)."""
    print("case verify expansion", flush=True)
    n = 4
    lens = [900, 61, 4]
    case = Case(3, 64, 8, 128, 16, lens, n=n, kv="int8", seed=17)
    out, lse = _check(case)
    table_x = case.block_table.repeat_interleave(n, dim=0).contiguous()
    lens_x = torch.tensor([L - (n - 1 - j) for L in lens for j in range(n)], dtype=torch.int32, device=gpu)
    out_x = torch.empty_like(out)
    ops.batch_decode(case.q, case.k_cache, out_x, table_x, lens_x, case.v_cache, None, None, case.k_scale,
                     case.v_scale, scale=case.scale, kv_cache_quant_bit_size=8)
    torch.cuda.synchronize()
    assert float((out.float() - out_x.float()).abs().max()) <= REG_TOL_QUANT


def test_zero_length_and_empty_batch(gpu):
    print("case zero length", flush=True)
    case = Case(3, 32, 8, 128, 16, [0, 50, 0], seed=19)
    out, lse = _check(case)
    assert float(out[0].float().abs().max()) == 0.0 and float(out[2].float().abs().max()) == 0.0
    assert torch.isneginf(lse[0]).all()
    # empty batch: nothing to do, no error
    q = torch.empty(0, 32, 128, dtype=torch.bfloat16, device=gpu)
    ops.batch_decode(q, case.k_cache, torch.empty_like(q), torch.empty(0, 4, dtype=torch.int32, device=gpu),
                     torch.empty(0, dtype=torch.int32, device=gpu), case.v_cache, scale=1.0)
    torch.cuda.synchronize()


@pytest.mark.parametrize("force_generic", [False, True])
def test_block_ids_are_taken_within_the_cache(gpu, force_generic, lib_option):
    """A block id outside 0 .. num_blocks-1 in a used table entry is a caller's mistake; the kernels
    take it within the cache (the nearest valid block) rather than read outside it, so the result is
    that of the table with those ids, bit for bit."""
    print("case block ids within the cache generic=%s" % force_generic, flush=True)
    if force_generic:
        lib_option("force_generic")
    case = Case(2, 32, 8, 128, 16, [64, 40], seed=29)
    last = case.nblocks - 1
    wrong = case.block_table.clone()
    wrong[0, 1] = case.nblocks + 5
    wrong[1, 0] = -3
    right = case.block_table.clone()
    right[0, 1] = last
    right[1, 0] = 0
    out, out2 = torch.empty_like(case.q), torch.empty_like(case.q)
    ops.batch_decode(case.q, case.k_cache, out, right, case.seq_lens, case.v_cache, scale=case.scale)
    ops.batch_decode(case.q, case.k_cache, out2, wrong, case.seq_lens, case.v_cache, scale=case.scale)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("force_generic", [False, True])
def test_lengths_beyond_the_block_list_are_cut_to_it(gpu, force_generic, lib_option):
    """A seq_lens entry above what a block_table row holds is cut to the row's capacity, so that no
    block id is read from the next row (or from past the table): the result is that of the cut
    length, bit for bit.  The rows after the long one hold valid ids, so nothing here reads outside
    the cache either way."""
    print("case length beyond the block list generic=%s" % force_generic, flush=True)
    if force_generic:
        lib_option("force_generic")
    case = Case(3, 32, 8, 128, 16, [64, 40, 64], seed=23)
    assert case.block_table.shape[1] == 4
    out = torch.empty_like(case.q)
    ops.batch_decode(case.q, case.k_cache, out, case.block_table, case.seq_lens, case.v_cache, scale=case.scale)
    longer = torch.tensor([100, 40, 64], dtype=torch.int32, device=gpu)
    out2 = torch.empty_like(case.q)
    ops.batch_decode(case.q, case.k_cache, out2, case.block_table, longer, case.v_cache, scale=case.scale)
    torch.cuda.synchronize()
    assert torch.equal(out, out2)


@pytest.mark.parametrize("force_generic", [False, True])
def test_sliding_window(gpu, force_generic, lib_option):
    print("case window", force_generic, flush=True)
    if force_generic:
        lib_option("force_generic")
    case = Case(3, 32, 8, 128, 16, [3000, 517, 20], n=2, seed=21)
    _check(case, window_left=100)
    _check(case, window_left=0)


@pytest.mark.parametrize("target", ["64", "2048"])
def test_result_does_not_depend_on_the_split(gpu, target, lib_option):
    print("case split target", target, flush=True)
    lib_option("target_items", int(target))
    case = Case(4, 32, 8, 128, 16, [4096, 2500, 128, 129], seed=23)
    _check(case)


def test_plan_once_run_many(gpu):
    """The schedule depends only on the lengths: build it once, reuse it for every layer's cache."""
    print("case plan reuse", flush=True)
    a = Case(3, 32, 8, 128, 16, [1500, 40, 700], seed=25)
    b = Case(3, 32, 8, 128, 16, [1500, 40, 700], seed=25, value_seed=26)  # another layer: same tables, other values
    assert np.array_equal(a.table, b.table)
    ws = torch.empty(ops.decode_workspace_bytes(3, 1, 32, 8, 128), dtype=torch.uint8, device=gpu)
    ref_a, _ = a.run(workspace=ws)
    ref_b, _ = b.run(workspace=ws)
    a.run(workspace=ws, run=False, lse=False)  # plan only
    out_a, _ = a.run(workspace=ws, plan=False)
    out_b, _ = b.run(workspace=ws, plan=False)
    assert torch.equal(out_a, ref_a) and torch.equal(out_b, ref_b)


def test_strided_query_rows(gpu):
    """q is a slice of the fused qkv projection: its token stride is not Hq*D."""
    print("case strided q", flush=True)
    case = Case(2, 32, 8, 128, 16, [300, 40], seed=27)
    ref, _ = case.run()
    T, Hq, D = case.q.shape
    fused = torch.zeros(T, (Hq + 16) * D, dtype=torch.bfloat16, device=gpu)
    fused[:, : Hq * D] = case.q.view(T, -1)
    q_view = fused[:, : Hq * D].view(T, Hq, D)
    assert q_view.stride(0) == (Hq + 16) * D
    out = torch.empty_like(case.q)
    ops.batch_decode(q_view, case.k_cache, out, case.block_table, case.seq_lens, case.v_cache, scale=case.scale)
    torch.cuda.synchronize()
    assert torch.equal(out, ref)


def test_4d_query_shape_of_the_mlu_caller(gpu):
    # query.view({-1, 1, num_heads, head_size}) (xllm/core/layers/mlu/attention.cpp:263-264)
    print("case 4-D query", flush=True)
    case = Case(2, 32, 8, 128, 16, [300, 40], seed=29)
    ref, _ = case.run()
    q4 = case.q.view(2, 1, 32, 128)
    out4 = torch.empty_like(q4)
    ops.batch_decode(q4, case.k_cache, out4, case.block_table, case.seq_lens, case.v_cache, None, None, None, None,
                     None, None, None, "float", 300, -1, -1, case.scale, False, -1)
    torch.cuda.synchronize()
    assert torch.equal(out4.view(2, 32, 128), ref)


def test_errors(gpu):
    case = Case(1, 32, 8, 128, 16, [20], seed=31)
    out = torch.empty_like(case.q)
    with pytest.raises(_lib.XllmHipError) as ei:
        ops.batch_decode(case.q, case.k_cache, out, case.block_table, case.seq_lens, case.v_cache, scale=1.0,
                         workspace=torch.empty(1024, dtype=torch.uint8, device=gpu))
    assert ei.value.status == _lib.WORKSPACE_TOO_SMALL
    with pytest.raises(_lib.XllmHipError):
        ops.batch_decode(case.q, case.k_cache, out, case.block_table, case.seq_lens, case.v_cache, scale=1.0,
                         alibi_slope=torch.zeros(32, device=gpu))
    big = torch.zeros(2, 1, 16, 512, dtype=torch.bfloat16, device=gpu)
    qb = torch.zeros(1, 1, 512, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(_lib.XllmHipError) as ei:
        ops.batch_decode(qb, big, torch.empty_like(qb), case.block_table, case.seq_lens, big, scale=1.0)
    assert ei.value.status == _lib.UNSUPPORTED


@pytest.mark.parametrize("kv,n", [("bf16", 1), ("int8", 4)])
def test_host_length_hints_select_the_unsplit_path(gpu, kv, n):
    """With truthful max_seq_len / total_kv_len the library may skip the split and the merge launch;
    with hints that are wrong the result must still be right."""
    print("case hints", kv, n, flush=True)
    lens = [700, 650, 702, 699, 640, 701, 688, 703] * 8  # 64 near-equal sequences: no split needed
    case = Case(64, 64 if n == 4 else 32, 8, 128, 16, lens, n=n, kv=kv, seed=33)
    ref, lse_ref = case.oracle()
    for kw in ({}, {"hints": True}, {"max_seq_len": 16, "total_kv_len": 100}, {"max_seq_len": 1 << 20, "total_kv_len": 1 << 30}):
        out, lse = case.run(**kw)
        e = max_abs_err(out, ref)
        print("   %s err=%.3e" % (kw, e), flush=True)
        assert e <= (REG_TOL_QUANT if kv == "int8" else REG_TOL)
        assert lse_err(lse, lse_ref) <= LSE_TOL


def test_decode_step_replays_under_hip_graph(gpu):
    """KV write + plan + attention (+ merge) captured once in a HIP graph and replayed while the
    lengths, slots and block tables change in the persistent input buffers (the way the reference's
    graph executor feeds its attention, xllm/core/runtime/cuda_graph_executor_impl.cpp:129-180).
    No host-side length hints are given under capture, so nothing in the graph depends on host
    values.  Every replay is checked against the eager result, with eager work in between."""
    print("case hip graph", flush=True)
    B, Hq, Hkv, D, bs, max_blocks = 6, 32, 8, 128, 16, 300
    nblocks = B * max_blocks + 1
    g = torch.Generator().manual_seed(51)
    k_cache = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16).to(gpu)
    v_cache = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16).to(gpu)
    perm = (torch.randperm(nblocks - 1, generator=g) + 1).to(torch.int32)
    table_full = perm[: B * max_blocks].view(B, max_blocks)
    # persistent buffers the graph reads
    q = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=gpu)
    new_k = torch.zeros(B, Hkv, D, dtype=torch.bfloat16, device=gpu)
    new_v = torch.zeros(B, Hkv, D, dtype=torch.bfloat16, device=gpu)
    slots = torch.zeros(B, dtype=torch.int32, device=gpu)
    block_table = table_full.to(gpu).contiguous()
    seq_lens = torch.ones(B, dtype=torch.int32, device=gpu)
    out = torch.zeros(B, Hq, D, dtype=torch.bfloat16, device=gpu)
    ws = torch.empty(ops.decode_workspace_bytes(B, 1, Hq, Hkv, D), dtype=torch.uint8, device=gpu)
    scale = 1.0 / float(np.sqrt(D))

    def step(o):
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=new_k, value=new_v, k_cache=k_cache, v_cache=v_cache,
                                                            slot_mapping=slots))
        ops.batch_decode(q, k_cache, o, block_table, seq_lens, v_cache, scale=scale, workspace=ws)

    def load_inputs(lens, seed):
        gg = torch.Generator().manual_seed(seed)
        q.copy_(torch.randn(B, Hq, D, generator=gg).to(torch.bfloat16))
        new_k.copy_(torch.randn(B, Hkv, D, generator=gg).to(torch.bfloat16))
        new_v.copy_(torch.randn(B, Hkv, D, generator=gg).to(torch.bfloat16))
        lens_t = torch.tensor(lens, dtype=torch.int32)
        pos = lens_t - 1
        blk = table_full[torch.arange(B), (pos // bs).long()]
        slots.copy_((blk * bs + pos % bs).to(torch.int32))
        seq_lens.copy_(lens_t)

    load_inputs([100, 20, 4000, 1, 777, 64], 0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):  # warm-up on the capture stream
        step(out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(out)
    for it, lens in enumerate(([100, 20, 4000, 1, 777, 64], [4799, 3, 17, 2048, 1, 4800], [5, 5, 5, 5, 5, 5],
                               [1000, 1001, 1002, 4003, 1004, 1005])):
        load_inputs(lens, 10 + it)
        k_before, v_before = k_cache.clone(), v_cache.clone()
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        k_after = k_cache.clone()
        # eager reference on the cache as it was before the replay
        k_cache.copy_(k_before)
        v_cache.copy_(v_before)
        eager = torch.zeros_like(out)
        step(eager)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), "replay %d differs from eager" % it
        assert torch.equal(k_after, k_cache)
        # some unrelated eager work between replays
        _ = (k_cache[:8].float() @ torch.ones(D, 4, device=gpu)).sum().item()


@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_long_context_single_sequence(gpu, kv):
    """131072 cached tokens in one sequence: 64 chunks per kv head, merged."""
    print("case long context", kv, flush=True)
    case = Case(1, 32, 8, 128, 128, [131072], kv=kv, seed=31, std=0.5)
    out, _ = _check(case)
    _check(case, hints=True)
    # with and without the host-side lengths the step is cut the same way; the launch's size differs, and
    # with it the number of waves per work item over a 1-byte cache unless that is held at four
    with ops.option("four_wave_items"):
        out_4, _ = case.run()
        out_h, _ = case.run(hints=True)
    assert torch.equal(out_4, out_h)
    if kv == "bf16":
        assert torch.equal(out, out_h)


@pytest.mark.parametrize("B,top", [(3000, 200), (9000, 60)])
def test_large_batch_of_short_sequences(gpu, B, top):
    """3000 sequences (the plan walks the batch 64 at a time, their lengths held in LDS), lengths 1..200,
    some empty; 9000 sequences (more than the plan holds in LDS)."""
    print("case large batch", B, flush=True)
    rng = np.random.default_rng(3)
    lens = rng.integers(1, top, size=B).astype(np.int32)
    lens[::97] = 0
    lens[5] = 40 * top  # one long sequence: the step is split whatever the mean
    case = Case(B, 32, 8, 128, 16, lens, seed=32)
    ref, _ = case.oracle()
    ws = torch.empty(ops.decode_workspace_bytes(B, 1, 32, 8, 128), dtype=torch.uint8, device=gpu)
    for hints in (False, True):
        out, _ = case.run(hints=hints, workspace=ws)
        assert not torch.isnan(out.float()).any()
        # (sequences of a handful of tokens are where the 16-bit weights and outputs cost most: 1.4e-2 at
        # the worst of 288000 rows)
        assert max_abs_err(out, ref) <= (REG_TOL if B <= 3000 else 1.6e-2)
        assert float(out[::97].float().abs().max()) == 0.0  # empty sequences give zeros


@pytest.mark.parametrize("kv,qdt,n,D,bs", [
    ("bf16", "bf16", 1, 128, 16), ("int8", "bf16", 4, 128, 16), ("bf16", "bf16", 12, 128, 16),
    ("bf16", "bf16", 2, 64, 32), ("int8", "bf16", 1, 64, 32),   # head_dim 64: other column split of the merge
    ("bf16", "bf16", 1, 256, 16), ("fp8", "bf16", 2, 256, 16),  # head_dim 256: four columns per lane
    ("fp16", "fp16", 1, 128, 16), ("int8", "fp16", 2, 128, 16),  # fp16 queries and outputs
])
def test_split_sequences_merge_in_the_attention_kernel_repeatably(gpu, kv, qdt, n, D, bs, lib_option):
    """Split sequences are merged by the workgroup that finishes a row group's last chunk: whichever
    that is, the result is the same bits on every run (the partials are summed in chunk order), the
    finished-chunk counters are left at zero (a second run on the same plan works), and sequences
    of one chunk beside split ones are untouched.  The separate merge kernel
    (XLLM_HIP_OPTION_DECODE_SEPARATE_MERGE) gives the same result from the same partials."""
    print("case fused merge", kv, qdt, n, D, flush=True)
    case = Case(5, 64, 8, D, bs, [9000, 40, 5000, 1, 20000], n=n, kv=kv, qdt=qdt, seed=91)
    assert case.variant() == "mfma_d%d" % D
    ref, lse_ref = case.oracle()
    first, lse_first = case.run()
    assert max_abs_err(first, ref) <= (REG_TOL_QUANT if kv in ("int8", "fp8") else REG_TOL)
    assert max_rel_err_per_seq(first, ref, n) <= REL_TOL
    assert lse_err(lse_first, lse_ref) <= LSE_TOL
    ws = ops.get_workspace(gpu, ops.decode_workspace_bytes(5, n, 64, 8, D))
    for i in range(40):
        out, lse = case.run(workspace=ws, plan=(i == 0))  # one plan, many runs: the counters reset themselves
        assert torch.equal(out, first) and torch.equal(lse, lse_first), i
    # the merge kernel on the same partials: the same sums in the same order, compiled as another
    # instantiation, so equal up to a unit in the last place of the output type
    lib_option("separate_merge")
    out, lse = case.run()
    assert torch.allclose(out.float(), first.float(), rtol=2.0 ** -9, atol=1e-6)
    assert torch.allclose(lse, lse_first, rtol=0.0, atol=1e-5, equal_nan=True)


def test_output_view_that_is_not_16_byte_aligned_takes_the_generic_kernel(gpu):
    """The MFMA kernels write output rows as 16-byte vectors: an output that starts at an odd element
    or has an odd token stride is served by the generic kernel, like such a query would be."""
    print("case misaligned output", flush=True)
    case = Case(3, 32, 8, 128, 16, [700, 33, 129], seed=12)
    ref, _ = case.oracle()
    desc = ops._cache_desc(case.k_cache, case.v_cache, None, None, "HND")
    lib = _lib.load()
    import ctypes
    for offset, pad in ((1, 0), (0, 4)):
        buf = torch.zeros(3 * (32 * 128 + pad) + 8, dtype=torch.bfloat16, device=gpu)
        out = buf[offset:offset + 3 * (32 * 128 + pad)].view(3, 32 * 128 + pad)[:, :32 * 128].view(3, 32, 128)
        args, _keep = ops._decode_args(case.q, out, None, case.block_table, case.seq_lens, None, 1, case.scale, -1, 0, desc)
        assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b"generic"
        ops.batch_decode(case.q, case.k_cache, out, case.block_table, case.seq_lens, case.v_cache, scale=case.scale)
        torch.cuda.synchronize()
        assert max_abs_err(out, ref) <= REG_TOL
        assert float(buf[:offset].float().abs().sum()) == 0.0  # nothing written in front of the view


@pytest.mark.parametrize("kv,n", [("bf16", 5), ("int8", 8), ("bf16", 1)])
def test_csr_form_whose_last_sequence_is_empty_reads_nothing_past_kv_indices(gpu, kv, n):
    """CSR form, trailing empty sequence: kv_indptr[B-1] == kv_indptr[B] == len(kv_indices), so an
    item of that sequence has no block id to read.  kv_indices is the tail of an allocation that is
    followed by a poisoned guard; results equal the block_table form."""
    print("case csr trailing empty", kv, n, flush=True)
    lens = [300, 0, 77, 0]
    case = Case(4, 16, 4, 128, 16, lens, n=n, kv=kv, seed=44)  # 4 heads per kv head x n rows: 20, 32 and 4 rows
    ref_out, ref_lse = case.run()
    lists = [case.table[i, : (L + 15) // 16] for i, L in enumerate(lens)]
    indptr, indices, last = orc.build_paged_kv_csr(lists, lens, 16)
    assert indptr[-1] == indptr[-2] == len(indices)
    dev = case.q.device
    guard = torch.full((len(indices) + 64,), 2 ** 30, dtype=torch.int32, device=dev)  # ids far outside the cache
    guard[: len(indices)] = torch.from_numpy(indices).to(dev)
    out = torch.full_like(case.q, float("nan"))
    ops.batch_decode_csr(case.q, case.k_cache, case.v_cache, torch.from_numpy(indptr).to(dev), guard[: len(indices)],
                         torch.from_numpy(last).to(dev), -1, case.scale, out, k_cache_scale=case.k_scale,
                         v_cache_scale=case.v_scale, q_per_seq=n, kv_layout="HND")
    torch.cuda.synchronize()
    assert torch.equal(out, ref_out)
    assert float(out.view(4, n, 16, 128)[1].float().abs().max()) == 0.0


@pytest.mark.parametrize("kv", ["bf16", "fp8"])
@pytest.mark.parametrize("name,lens", [
    ("equal lengths, a few chunks each", [6000] * 3),
    ("equal lengths, one workgroup per (sequence, head) is enough", [1100] * 24),
    ("one long sequence among short ones", [30000, 700, 900, 650, 100]),
    ("lengths so close that a split would only shed short tails", [2500 + 16 * i for i in range(20)]),
    ("ragged, as many items as the budget takes", [4000, 2500, 900, 3300, 1700, 2900]),
])
def test_small_batch_chunk_choices(gpu, kv, name, lens):
    """Small batches are cut for one workgroup per CU rather than for every slot; each branch of that
    choice (equal lengths, the item budget, the parallelism floor, the short-tail rule) against the
    oracle, with and without the host's length hints."""
    print("case small batch", kv, name, flush=True)
    case = Case(len(lens), 32, 8, 128, 16, lens, kv=kv, seed=57)
    ref, lse_ref = case.oracle()
    out, lse = case.run()
    assert max_abs_err(out, ref) <= (REG_TOL_QUANT if kv == "fp8" else REG_TOL)
    assert lse_err(lse, lse_ref) <= LSE_TOL
    out_h, lse_h = case.run(hints=True)
    assert max_abs_err(out_h, ref) <= (REG_TOL_QUANT if kv == "fp8" else REG_TOL)
    assert lse_err(lse_h, lse_ref) <= LSE_TOL
    # the host's lengths leave the cut as it is, except that over a 1-byte cache a step that fits one work
    # item per CU is then cut for that, its items run by eight waves
    with ops.option("four_wave_items"):
        out_4, _ = case.run()
        out_h4, _ = case.run(hints=True)
    assert torch.equal(out_4, out_h4)
    if kv == "bf16":
        assert torch.equal(out, out_h)


@pytest.mark.parametrize("name,kv,qdt,layout,Hq,Hkv,n,bs,lens", [
    ("equal lengths, fp8", "fp8", "bf16", "HND", 32, 8, 1, 16, [300] * 256),
    ("equal lengths, int8, two draft tokens", "int8", "fp16", "HND", 32, 8, 2, 128, [517] * 256),
    ("equal lengths, four kv heads", "fp8", "bf16", "HND", 16, 4, 1, 32, [130] * 512),
    ("equal lengths, bf16", "bf16", "bf16", "HND", 32, 8, 1, 16, [100] * 512),
    ("equal lengths, bf16 over NHD", "bf16", "bf16", "NHD", 32, 8, 1, 16, [64] * 256),
    ("ragged, int8", "int8", "bf16", "HND", 32, 8, 1, 16, None),
    ("ragged, bf16", "bf16", "bf16", "HND", 32, 8, 1, 16, None),
    # kv heads that are no multiple of four: four neighbouring (sequence, kv head) items to a workgroup
    ("one kv head, fp8, last workgroup with one item", "fp8", "bf16", "HND", 8, 1, 1, 16, [200] * 2045),
    ("two kv heads, int8, two draft tokens", "int8", "fp16", "HND", 8, 2, 2, 32, [300 - (i % 7) for i in range(1023)]),
    ("one kv head, bf16", "bf16", "bf16", "HND", 8, 1, 1, 16, [100] * 2048),
    # half as many items: two waves to an item, two items to a workgroup (the last one with a single item)
    ("eight kv heads, fp8, two waves per item", "fp8", "bf16", "HND", 32, 8, 1, 16, [700] * 128),
    ("one kv head, int8, two waves per item", "int8", "bf16", "HND", 8, 1, 2, 64, [450 - (i % 3) for i in range(1023)]),
    ("six kv heads over NHD, fp8, some sequences empty", "fp8", "bf16", "NHD", 12, 6, 1, 16, [0 if i % 50 == 3 else 333 for i in range(341)]),
])
def test_four_head_items_for_many_short_sequences(gpu, name, kv, qdt, layout, Hq, Hkv, n, bs, lens):
    """A large batch of short sequences, with the host's lengths: a work item is four kv heads of a
    sequence, one per wave (each wave then has a whole sequence to itself), in any layout — from 512 such
    items on when the lengths are nearly equal, from 2048 on when they are ragged (long ones are then cut
    and merged by the merge kernel); with a head count that is no multiple of four, four neighbouring items
    of a step that is not split, and with half as many items two waves to an item.  (Batch sizes whose wider
    workgroups fill whole rounds of the GPU's slots: others keep an item per head.)  Against the oracle
    and against the same step with an item per head."""
    print("case four heads per item, short sequences", name, flush=True)
    if lens is None:
        rng = np.random.default_rng(17)
        top = 700 if kv == "int8" else 190
        lens = rng.integers(1, top, size=1100).astype(np.int32)
        lens[::53] = 0
        lens[7] = 6000 if kv == "int8" else 1500  # one sequence far above the rest: cut into chunks
    case = Case(len(lens), Hq, Hkv, 128, bs, lens, n=n, kv=kv, qdt=qdt, layout=layout, seed=71)
    assert case.variant() == "mfma_d128"
    tol = {"bf16": REG_TOL, "fp16": 2e-3}.get(kv, REG_TOL_QUANT)
    ref, lse_ref = case.oracle()
    out, lse = case.run(hints=True)
    assert not torch.isnan(out.float()).any()
    assert max_abs_err(out, ref) <= tol
    assert lse_err(lse, lse_ref) <= LSE_TOL
    with ops.option("item_per_head"):
        out_1, lse_1 = case.run(hints=True)
    assert max_abs_err(out_1, ref) <= tol
    assert torch.allclose(out.float(), out_1.float(), rtol=2 ** -6, atol=4e-3)
    out2, lse2 = case.run(hints=True)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


@pytest.mark.parametrize("kv,qdt,Hq,Hkv,n", [("fp8", "bf16", 32, 8, 1), ("int8", "bf16", 16, 4, 2), ("int8", "fp16", 32, 8, 1),
                                            ("bf16", "bf16", 32, 8, 1), ("int8", "bf16", 14, 2, 1), ("fp8", "bf16", 14, 2, 1)])
def test_work_items_of_four_kv_heads_over_nhd_at_head_dim_64(gpu, kv, qdt, Hq, Hkv, n):
    """head_dim 64 over a 1-byte NHD cache (rows of 64 bytes, two kv heads to a 128-byte line): work items of four kv
    heads for any step, split sequences included, their waves walking the tokens in step; 16-bit caches and two kv
    heads keep one head per item here (their steps are split)."""
    print("case four heads per item, head_dim 64", kv, qdt, Hq, Hkv, n, flush=True)
    lens = [9000, 300, 0, 33, 4100, 17, 64, 65]
    case = Case(len(lens), Hq, Hkv, 64, 32, lens, n=n, kv=kv, qdt=qdt, layout="NHD", seed=97)
    assert case.variant() == "mfma_d64"
    shape = ops.decode_describe(case.q, case.k_cache, case.v_cache, case.block_table, case.seq_lens, case.k_scale, case.v_scale,
                                q_per_seq=n, kv_layout="NHD")
    assert shape["kv_heads_per_item"] == (4 if kv in ("fp8", "int8") and Hkv % 4 == 0 else 1), shape
    tol = {"bf16": REG_TOL, "fp16": 2e-3}.get(kv, REG_TOL_QUANT)
    for window in (-1, 300):
        ref, lse_ref = case.oracle(window)
        out, lse = case.run(window)
        assert not torch.isnan(out.float()).any()
        assert max_abs_err(out, ref) <= tol
        assert lse_err(lse, lse_ref) <= LSE_TOL
        with ops.option("item_per_head"):
            out_1, _ = case.run(window)
        assert max_abs_err(out_1, ref) <= tol
        assert torch.allclose(out.float(), out_1.float(), rtol=2 ** -6, atol=4e-3)
    out_h, lse_h = case.run(hints=True)
    ref, lse_ref = case.oracle()
    assert max_abs_err(out_h, ref) <= tol and lse_err(lse_h, lse_ref) <= LSE_TOL
    # long equal sequences with host-side lengths: not split, a wave (or two) per (sequence, kv head)
    eq = Case(280, Hq, Hkv, 64, 32, [700 + (i % 3) for i in range(280)], n=n, kv=kv, qdt=qdt, layout="NHD", seed=98)
    ref, lse_ref = eq.oracle()
    out, lse = eq.run(hints=True)
    assert max_abs_err(out, ref) <= tol and lse_err(lse, lse_ref) <= LSE_TOL


@pytest.mark.parametrize("name,kv,qdt,layout,Hq,Hkv,n,bs,lens", [
    ("two kv heads, int8", "int8", "bf16", "HND", 14, 2, 1, 32, [260 - (i % 5) for i in range(1024)]),
    ("two kv heads, bf16, two draft tokens", "bf16", "bf16", "HND", 14, 2, 2, 32, [1500] * 1024),
    ("eight kv heads, fp8 over NHD", "fp8", "fp16", "NHD", 32, 8, 1, 64, [411] * 256),
    ("eight kv heads, fp16, ragged", "fp16", "fp16", "HND", 32, 8, 1, 32, None),
    # rows of 64 bytes, two kv heads to a 128-byte line: the waves of a workgroup walk their tokens in step, each
    # as many tiles as the longest of the four (lengths either side of a tile's end)
    ("two kv heads, int8 over NHD, a wave per item", "int8", "bf16", "NHD", 14, 2, 1, 32, [250 + 5 * (i % 7) for i in range(1024)]),
    ("two kv heads, fp8 over NHD, two waves per item", "fp8", "bf16", "NHD", 14, 2, 1, 32, [1000 + 9 * (i % 5) for i in range(1000)]),
    # ... and over a schedule that is kept (ragged lengths, one sequence split, some empty): two items to a workgroup too
    ("two kv heads, int8 over NHD, ragged", "int8", "bf16", "NHD", 14, 2, 1, 32, None),
    ("two kv heads, fp8 over NHD, ragged, two draft tokens", "fp8", "fp16", "NHD", 14, 2, 2, 64, None),
])
def test_items_per_wave_at_head_dim_64(gpu, name, kv, qdt, layout, Hq, Hkv, n, bs, lens):
    """The same work items (four kv heads, or four neighbouring items, one per wave) at head_dim 64."""
    print("case item per wave, head_dim 64", name, flush=True)
    if lens is None:
        rng = np.random.default_rng(19)
        lens = rng.integers(1, 900, size=1030).astype(np.int32)
        lens[::41] = 0
        lens[3] = 9000
    case = Case(len(lens), Hq, Hkv, 64, bs, lens, n=n, kv=kv, qdt=qdt, layout=layout, seed=73)
    assert case.variant() == "mfma_d64"
    if "per item" in name:
        lens_np = np.asarray(lens)
        shape = ops.decode_describe(case.q, case.k_cache, case.v_cache, case.block_table, case.seq_lens, case.k_scale, case.v_scale,
                                    q_per_seq=n, kv_layout=layout, max_seq_len=int(lens_np.max()), total_kv_len=int(lens_np.sum()))
        assert shape["items_per_workgroup"] == (4 if "a wave per item" in name else 2), shape
    tol = {"bf16": REG_TOL, "fp16": 2e-3}.get(kv, REG_TOL_QUANT)
    ref, lse_ref = case.oracle()
    out, lse = case.run(hints=True)
    assert not torch.isnan(out.float()).any()
    assert max_abs_err(out, ref) <= tol
    assert lse_err(lse, lse_ref) <= LSE_TOL
    with ops.option("item_per_head"):
        out_1, _ = case.run(hints=True)
    assert max_abs_err(out_1, ref) <= tol
    assert torch.allclose(out.float(), out_1.float(), rtol=2 ** -6, atol=4e-3)


@pytest.mark.parametrize("kv,qdt", [("fp8", "bf16"), ("int8", "bf16"), ("int8", "fp16")])
@pytest.mark.parametrize("name,D,bs,n,lens", [
    ("one long sequence", 128, 16, 1, [32768]),
    ("split, every CU an item", 128, 128, 2, [6000] * 4),
    ("not split: a workgroup per (sequence, kv head)", 128, 16, 1, [700 + 16 * i for i in range(30)]),
    ("nearly equal lengths, one empty", 128, 32, 4, [8192, 7000, 0, 8192, 8100, 7777]),
    ("head_dim 64", 64, 32, 2, [9000] * 3),
    ("head_dim 64, not split", 64, 64, 1, [300] * 32),
])
def test_eight_wave_items_over_one_byte_caches(gpu, kv, qdt, name, D, bs, n, lens):
    """With the host's lengths a step over a 1-byte cache that fits one work item per CU runs eight
    waves per item (the waves share the item's tokens and combine at its end as four do): against the
    oracle, and against the same step held at four waves."""
    print("case eight waves", kv, qdt, name, flush=True)
    case = Case(len(lens), 32, 8, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=63)
    ref, lse_ref = case.oracle()
    out, lse = case.run(hints=True)
    assert not torch.isnan(out.float()).any()
    assert max_abs_err(out, ref) <= REG_TOL_QUANT
    assert lse_err(lse, lse_ref) <= LSE_TOL
    with ops.option("four_wave_items"):
        out_4, lse_4 = case.run(hints=True)
    # two roundings of 16-bit outputs (2^-8 relative) and fp32 summation order
    assert max_abs_err(out, out_4.float().cpu().numpy().astype(np.float64)) <= 1.6e-2
    assert lse_err(lse, lse_4.cpu().numpy().astype(np.float64)) <= 1e-5
    out2, lse2 = case.run(hints=True)
    assert torch.equal(out, out2) and torch.equal(lse, lse2)


ALL_KV = ("bf16", "fp8", "int8")


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp8", "bf16"), ("int8", "fp16")])
@pytest.mark.parametrize("name,Hq,Hkv,D,n,bs,lens,cut_for", [
    ("two sequences past one round", 32, 8, 128, 1, 16, [1500] * 66, ALL_KV),
    ("eight past one round, nearly equal lengths, one empty", 32, 8, 128, 2, 32,
     [1400 - 3 * (i % 40) for i in range(71)] + [0], ALL_KV),
    ("a sequence past two rounds", 16, 4, 128, 1, 128, [700] * 257, ALL_KV),
    ("one kv head", 8, 1, 128, 1, 16, [640] * 520, ALL_KV),
    ("head_dim 64", 14, 2, 64, 1, 32, [900] * 260, ALL_KV),
    ("head_dim 256: rounds of 256", 16, 4, 256, 1, 16, [1100] * 66, ALL_KV),
    # up to a quarter more items than CUs: 1-byte caches run eight waves per item, whole items and chunks alike
    ("an item per CU and sixteen more", 32, 8, 128, 1, 16, [3200] * 34, ALL_KV),
    ("an item per CU and eight more, short sequences", 32, 8, 128, 2, 64, [1800] * 33, ALL_KV),
    # fewer items than slots: 1-byte caches are cut in two throughout, the last sequences finer
    ("an item per CU and seventy more", 32, 8, 128, 1, 16, [3300] * 41, ALL_KV),
])
def test_sequences_of_a_partly_filled_round_are_cut(gpu, kv, qdt, name, Hq, Hkv, D, n, bs, lens, cut_for):
    """Equal work items a few more than a whole number of rounds of the GPU (an item per CU over a 16-bit cache,
    every workgroup slot over a 1-byte one): with the host's lengths the sequences of the last round are cut into
    chunks that fill a round once more (merged inside the attention kernel) and the others stay as they are.
    Against the oracle, against the same step left whole (the stored-schedule option keeps it so), on wrong
    host-side lengths, and twice in a row."""
    print("case last round cut", kv, name, flush=True)
    case = Case(len(lens), Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=83)
    tol = {"bf16": REG_TOL, "fp16": 2e-3}.get(kv, REG_TOL_QUANT)
    ref, lse_ref = case.oracle()
    nbytes = ops.decode_workspace_bytes(case.B, n, Hq, Hkv, D)
    ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=gpu)
    out, lse = case.run(workspace=ws, hints=True)
    assert not torch.isnan(out.float()).any()
    assert max_abs_err(out, ref) <= tol
    assert lse_err(lse, lse_ref) <= LSE_TOL
    with ops.option("stored_schedule"):
        out_w, lse_w = case.run(workspace=ws, hints=True)
    assert max_abs_err(out_w, ref) <= tol
    assert torch.allclose(out.float(), out_w.float(), rtol=2 ** -6, atol=4e-3)
    rows = 8 * n
    if kv in cut_for:
        assert not torch.equal(lse[-rows:], lse_w[-rows:]), "the last sequences were not cut"
        if len(lens) >= 64 or kv == "bf16":  # (the first sequences stay whole: the same bits)
            assert torch.equal(out[:rows], out_w[:rows]) and torch.equal(lse[:rows], lse_w[:rows])
    else:
        assert torch.equal(out, out_w) and torch.equal(lse, lse_w)
    # host-side lengths that are too small: a sequence's last chunk takes the rest
    longest, total = int(max(lens)), int(sum(lens))
    out_s, lse_s = case.run(workspace=ws, max_seq_len=max(1, longest * 3 // 4), total_kv_len=max(1, total * 3 // 4))
    assert max_abs_err(out_s, ref) <= tol
    out2, lse2 = case.run(workspace=ws, hints=True, plan=False)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


@pytest.mark.parametrize("name,B,L,kv,qdt", [
    ("cut in four, the 33rd sequence finer", 33, 6200, "int8", "bf16"),
    ("cut in two, the last two sequences finer", 66, 3400, "int8", "bf16"),
    ("whole, the last two sequences cut", 130, 1100, "int8", "fp16"),
    ("16-bit cache: whole, the last two sequences cut", 66, 1300, "bf16", "bf16"),
])
def test_partly_filled_round_of_the_32_row_kernel(gpu, name, B, L, kv, qdt):
    """The same with 32 query rows per kv head (four draft tokens); over a 1-byte cache the step's even cut is
    taken one finer where that overfills a round of the slots by little, and the sequences past the round
    are cut finer still; the merge kernel combines them."""
    print("case last round cut, 32 rows", kv, name, flush=True)
    lens = [L - (i % 3) for i in range(B)]
    case = Case(B, 64, 8, 128, 128, lens, n=4, kv=kv, qdt=qdt, seed=85)
    ref, lse_ref = case.oracle()
    ws = torch.full((ops.decode_workspace_bytes(B, 4, 64, 8, 128),), 0xA5, dtype=torch.uint8, device=gpu)
    out, lse = case.run(workspace=ws, hints=True)
    assert not torch.isnan(out.float()).any()
    assert max_abs_err(out, ref) <= REG_TOL_QUANT
    assert lse_err(lse, lse_ref) <= LSE_TOL
    with ops.option("stored_schedule"):
        out_w, lse_w = case.run(workspace=ws, hints=True)
    assert max_abs_err(out_w, ref) <= REG_TOL_QUANT
    assert torch.allclose(out.float(), out_w.float(), rtol=2 ** -6, atol=4e-3)
    assert not torch.equal(lse[-32:], lse_w[-32:]), "the last sequence was not cut finer"
    out_s, _ = case.run(workspace=ws, max_seq_len=L * 3 // 4, total_kv_len=B * L * 3 // 4)
    assert max_abs_err(out_s, ref) <= REG_TOL_QUANT
    out2, lse2 = case.run(workspace=ws, hints=True, plan=False)
    assert torch.equal(out2, out) and torch.equal(lse2, lse)


@pytest.mark.parametrize("kv,qdt,tol", [("bf16", "bf16", 2e-2), ("fp16", "fp16", 2e-3), ("int8", "bf16", 2e-2)])
def test_two_stage_decode_merged_by_lse_equals_one_stage(gpu, kv, qdt, tol):
    """The returned log-sum-exps are base 2 and merge as the reference merges two partial attentions
    (xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73): attention over a prefix and over the rest
    of each sequence, two calls, combined by that formula, against the one call over the whole — the
    reference's own check of its two-stage decode, with its tolerances
    (xllm/core/layers/cuda/xattention_test.cpp:224-273: fp16 2e-3, bf16 2e-2)."""
    print("case two-stage", kv, qdt, flush=True)
    bs = 16
    lens = [700, 33, 2500, 160, 6000]
    cut = [320, 16, 1024, 96, 4096]  # block-aligned prefix lengths, all inside the sequences
    case = Case(len(lens), 32, 8, 128, bs, lens, kv=kv, qdt=qdt, seed=77)
    whole, lse_whole = case.run()

    def part(table, part_lens):
        saved = case.block_table, case.seq_lens
        case.block_table = torch.from_numpy(np.ascontiguousarray(table)).to(gpu)
        case.seq_lens = torch.tensor(part_lens, dtype=torch.int32, device=gpu)
        try:
            return case.run()
        finally:
            case.block_table, case.seq_lens = saved

    out_a, lse_a = part(case.table, cut)
    width = case.table.shape[1]
    rest = np.zeros_like(case.table)
    for b, c in enumerate(cut):
        rest[b, : width - c // bs] = case.table[b, c // bs:]
    out_b, lse_b = part(rest, [l - c for l, c in zip(lens, cut)])
    merged, lse_m = orc.lse_combine(out_a.float().cpu().numpy(), lse_a.cpu().numpy(),
                                    out_b.float().cpu().numpy(), lse_b.cpu().numpy())
    assert max_abs_err(whole, merged.astype(np.float64)) <= tol
    assert lse_err(lse_whole, lse_m.astype(np.float64)) <= 1e-4


def test_int8_verify_step_replays_under_hip_graph(gpu):
    """The speculative-verify form of the step under a HIP graph: quantising write of 4 draft tokens per
    sequence, plan, the 32-row kernel over an int8 cache and the merge kernel, captured once and
    replayed while lengths and slots change; every replay equals the eager result."""
    print("case hip graph int8 verify", flush=True)
    B, n, Hq, Hkv, D, bs, max_blocks = 3, 4, 64, 8, 128, 32, 200
    nblocks = B * max_blocks + 1
    g = torch.Generator().manual_seed(52)
    k_cache = torch.zeros(nblocks, Hkv, bs, D, dtype=torch.int8, device=gpu)
    v_cache = torch.zeros_like(k_cache)
    k_scale = torch.zeros(nblocks, Hkv, bs, device=gpu)
    v_scale = torch.zeros_like(k_scale)
    # a cache full of quantised random rows, written through the operator itself
    fill = torch.arange(1 * bs, nblocks * bs, dtype=torch.int32, device=gpu)
    for s in range(0, fill.numel(), 4096):
        sl = fill[s:s + 4096]
        kk = torch.randn(sl.numel(), Hkv, D, generator=g).to(torch.bfloat16).to(gpu)
        vv = torch.randn(sl.numel(), Hkv, D, generator=g).to(torch.bfloat16).to(gpu)
        ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(key=kk, value=vv, k_cache=k_cache, v_cache=v_cache,
                                                             slot_mapping=sl, k_cache_scale=k_scale, v_cache_scale=v_scale))
    perm = (torch.randperm(nblocks - 1, generator=g) + 1).to(torch.int32)
    table_full = perm[: B * max_blocks].view(B, max_blocks)
    q = torch.zeros(B * n, Hq, D, dtype=torch.bfloat16, device=gpu)
    new_k = torch.zeros(B * n, Hkv, D, dtype=torch.bfloat16, device=gpu)
    new_v = torch.zeros(B * n, Hkv, D, dtype=torch.bfloat16, device=gpu)
    slots = torch.zeros(B * n, dtype=torch.int32, device=gpu)
    block_table = table_full.to(gpu).contiguous()
    seq_lens = torch.full((B,), n, dtype=torch.int32, device=gpu)
    out = torch.zeros_like(q)
    ws = torch.empty(ops.decode_workspace_bytes(B, n, Hq, Hkv, D), dtype=torch.uint8, device=gpu)
    scale = 1.0 / float(np.sqrt(D))

    def step(o):
        ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(key=new_k, value=new_v, k_cache=k_cache, v_cache=v_cache,
                                                             slot_mapping=slots, k_cache_scale=k_scale,
                                                             v_cache_scale=v_scale))
        ops.batch_decode(q, k_cache, o, block_table, seq_lens, v_cache, None, None, k_scale, v_scale, scale=scale,
                         q_per_seq=n, workspace=ws, kv_cache_quant_bit_size=8)

    def load_inputs(lens, seed):
        gg = torch.Generator().manual_seed(seed)
        q.copy_(torch.randn(B * n, Hq, D, generator=gg).to(torch.bfloat16))
        new_k.copy_(torch.randn(B * n, Hkv, D, generator=gg).to(torch.bfloat16))
        new_v.copy_(torch.randn(B * n, Hkv, D, generator=gg).to(torch.bfloat16))
        sl = []
        for b, L in enumerate(lens):  # the draft tokens are the last n positions of the sequence
            for j in range(n):
                pos = L - n + j
                sl.append(int(table_full[b, pos // bs]) * bs + pos % bs)
        slots.copy_(torch.tensor(sl, dtype=torch.int32))
        seq_lens.copy_(torch.tensor(lens, dtype=torch.int32))

    load_inputs([3000, 40, 6000], 0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(out)
    for it, lens in enumerate(([3000, 40, 6000], [6399, 4, 17], [9, 9, 9], [1000, 5003, 2004])):
        load_inputs(lens, 20 + it)
        saved = [t.clone() for t in (k_cache, v_cache, k_scale, v_scale)]
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        after = [t.clone() for t in (k_cache, v_cache, k_scale, v_scale)]
        for t, s in zip((k_cache, v_cache, k_scale, v_scale), saved):
            t.copy_(s)
        eager = torch.zeros_like(out)
        step(eager)
        torch.cuda.synchronize()
        assert torch.equal(got, eager), "replay %d differs from eager" % it
        for t, a in zip((k_cache, v_cache, k_scale, v_scale), after):
            assert torch.equal(t.view(torch.uint8) if t.dtype == torch.int8 else t, a.view(torch.uint8) if a.dtype == torch.int8 else a)
        _ = (k_scale[:8] * 2).sum().item()  # unrelated eager work between replays


@pytest.mark.parametrize("kv,n,qdt", [("bf16", 1, "bf16"), ("int8", 4, "bf16"), ("fp8", 8, "bf16"), ("fp16", 2, "fp16"),
                                      ("fp32", 1, "fp32")])
@pytest.mark.parametrize("name,lens", [
    ("one long sequence", [32768]),
    ("equal lengths", [8192] * 6),
    ("nearly equal lengths, one of them empty", [8192, 7000, 0, 8192, 8100, 7777, 8192, 8000]),
])
def test_split_step_without_a_stored_schedule(gpu, kv, n, qdt, name, lens):
    """A split step whose host-side lengths (max_seq_len, total_kv_len) are nearly equal stores no
    schedule: every work item derives its chunk from its index and the sequence's length, and no plan
    kernel runs.  Against the oracle, bit for bit against the same step with the stored schedule
    (which cuts the same chunks), and with host-side lengths that are wrong: a max_seq_len below the
    longest sequence (the last chunk then takes the rest) and a total that is too small."""
    print("case no stored schedule", kv, n, qdt, name, flush=True)
    Hq, Hkv = (32, 8) if kv != "fp32" else (14, 2)
    D, bs = (128, 16) if kv != "fp32" else (64, 16)
    case = Case(len(lens), Hq, Hkv, D, bs, lens, n=n, kv=kv, qdt=qdt, seed=91)
    ref, lse_ref = case.oracle()
    nbytes = ops.decode_workspace_bytes(case.B, n, Hq, Hkv, D)
    ws = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=gpu)
    out, lse = case.run(workspace=ws, hints=True)
    # the schedule's header (first 64 bytes of the workspace) was never written
    assert bool((ws[:64] == 0xA5).all()), "a schedule was stored"
    tol = {"bf16": REG_TOL, "fp16": 2e-3, "fp32": 1e-4}.get(kv, REG_TOL_QUANT)
    assert max_abs_err(out, ref) <= tol
    assert lse_err(lse, lse_ref) <= LSE_TOL
    # (the stored schedule's launch is sized for any lengths, and a launch of more work items than CUs
    # runs four waves per item: the comparison holds the other one at four as well)
    with ops.option("four_wave_items"):
        out_4, lse_4 = case.run(workspace=ws, hints=True)
        assert bool((ws[:64] == 0xA5).all())
        with ops.option("stored_schedule"):
            out_s, lse_s = case.run(workspace=ws, hints=True)
    assert not bool((ws[:64] == 0xA5).all())
    assert torch.equal(out_4, out_s) and torch.equal(lse_4, lse_s)
    # wrong host-side lengths
    ws.fill_(0xA5)
    longest, total = int(max(lens)), int(sum(lens))
    out_w, lse_w = case.run(workspace=ws, max_seq_len=max(1, longest * 3 // 4), total_kv_len=max(1, total * 3 // 4))
    assert max_abs_err(out_w, ref) <= tol
    assert lse_err(lse_w, lse_ref) <= LSE_TOL
    # ... and a second step on the same workspace without a plan call in between (the counters of the
    # fused merge reset themselves)
    out2, _ = case.run(workspace=ws, hints=True, plan=False)
    assert torch.equal(out2, out)
