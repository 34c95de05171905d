"""Sequences with different numbers of query tokens (chunked prefill / mixed steps) over the paged
cache, through the C ABI, against the oracle."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.helpers import Case
from xllm_wxh_amd import ops

pytestmark = pytest.mark.gpu


def _run(c, q_counts, max_q, **kw):
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    T = int(q_indptr[-1])
    g = torch.Generator().manual_seed(77)
    q = torch.randn(T, c.Hq, c.D, generator=g).to(torch.bfloat16 if c.qdt == "bf16" else torch.float32)
    qd = q.to(c.q.device)
    out = torch.full_like(qd, 7.0)
    lse = torch.full((T, c.Hq), 3.0, dtype=torch.float32, device=qd.device)
    ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, None, c.k_scale, c.v_scale,
                     scale=c.scale, return_lse=True, kv_cache_quant_bit_size=8 if c.k_scale is not None else -1,
                     q_per_seq=max_q, q_indptr=torch.from_numpy(q_indptr).to(qd.device), **kw)
    torch.cuda.synchronize()
    ref, ref_lse = orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale,
                                           window_left=kw.get("window_size_left", -1))
    return out.float().cpu().numpy(), lse.cpu().numpy(), ref, ref_lse, q_indptr


@pytest.mark.parametrize("kv", ["bf16", "fp8", "int8"])
@pytest.mark.parametrize("Hq,Hkv,D,bs", [(32, 8, 128, 16), (64, 8, 128, 16), (8, 8, 128, 16), (32, 8, 256, 16),
                                         (16, 8, 256, 64), (32, 8, 64, 32)])
def test_mixed_step_matches_oracle(gpu, kv, Hq, Hkv, D, bs):
    """A mixed step: decode sequences (1 token), speculative verify (4) and prefill chunks (up to 70
    tokens, some reaching back to the start of the sequence) in one call."""
    print("case mixed step", kv, Hq, Hkv, D, bs, flush=True)
    lens = [300, 70, 33, 1, 129, 4096, 64, 40]
    q_counts = [1, 70, 4, 1, 17, 64, 0, 40]   # 70 == len and 40 == len: the whole sequence is the chunk
    c = Case(len(lens), Hq, Hkv, D, bs, lens, kv=kv, seed=21)
    assert c.variant() == {64: "mfma_d64", 128: "mfma_d128", 256: "mfma_d256"}[D]
    out, lse, ref, ref_lse, q_indptr = _run(c, q_counts, max(q_counts))
    err = float(np.abs(out - ref).max())
    print("   err %.3e" % err, flush=True)
    assert err <= c.tol
    fin = np.isfinite(ref_lse)
    assert np.allclose(lse[fin], ref_lse[fin], atol=2e-2 if kv == "bf16" else 5e-2)


def test_chunk_equals_expanded_decode_rows(gpu):
    """The reference's equivalence (xllm/core/runtime/speculative_worker_impl.cpp:230-243): a chunk of n
    tokens gives what n separate decode rows with kv lengths L-n+1 .. L over the same blocks give."""
    print("case chunk vs expanded rows", flush=True)
    L, n, Hq, Hkv = 777, 48, 32, 8
    c = Case(1, Hq, Hkv, 128, 16, [L], seed=5)
    out, lse, ref, _, _ = _run(c, [n], n)
    qd = torch.randn(n, Hq, 128, generator=torch.Generator().manual_seed(77)).to(torch.bfloat16).to(c.q.device)
    rows = torch.empty_like(qd)
    table = c.block_table.expand(n, -1).contiguous()
    lens = torch.arange(L - n + 1, L + 1, dtype=torch.int32, device=qd.device)
    ops.batch_decode(qd, c.k_cache, rows, table, lens, c.v_cache, scale=c.scale)
    torch.cuda.synchronize()
    assert float(np.abs(rows.float().cpu().numpy() - out).max()) <= 1.2e-2
    assert float(np.abs(out - ref).max()) <= c.tol


def test_prefill_sized_chunks_and_edge_cases(gpu):
    print("case prefill chunks", flush=True)
    # 512-token chunks at g = 4: 2048 rows per kv head = 64 row groups, never split
    lens = [2048, 512, 700]
    q_counts = [512, 512, 188]
    c = Case(3, 32, 8, 128, 128, lens, seed=9)
    out, lse, ref, ref_lse, q_indptr = _run(c, q_counts, 512)
    assert float(np.abs(out - ref).max()) <= c.tol
    # counts above q_per_seq are cut to it (documented); rows of other sequences are unaffected
    c2 = Case(2, 32, 8, 128, 16, [100, 90], seed=10)
    out2, _, ref2, _, ind2 = _run(c2, [8, 3], 4)
    assert float(np.abs(out2[ind2[1]:] - ref2[ind2[1]:]).max()) <= c2.tol
    assert np.all(out2[4:8] == 7.0)  # tokens 4..7 of sequence 0 were ignored
    # sliding window together with a chunk
    c3 = Case(2, 32, 8, 128, 16, [500, 64], seed=11)
    out3, _, ref3, _, _ = _run(c3, [33, 64], 64, window_size_left=100)
    assert float(np.abs(out3 - ref3).max()) <= c3.tol
    # the generic kernel (fp32, head_dim 64) takes the same arguments
    c4 = Case(3, 14, 2, 64, 16, [50, 333, 20], kv="fp32", qdt="fp32", seed=12)
    out4, _, ref4, _, _ = _run(c4, [5, 40, 20], 40)
    assert float(np.abs(out4 - ref4).max()) <= 1e-4


@pytest.mark.parametrize("D,bs,layout", [(128, 16, "HND"), (128, 128, "NHD"), (64, 32, "HND"), (64, 64, "NHD")])
@pytest.mark.parametrize("qdt", ["bf16", "fp16"])
def test_many_row_kernel_shapes(gpu, D, bs, layout, qdt):
    """16-bit caches with more than 64 query rows per kv head take the 128-row kernel (tiles go from
    global memory straight to LDS): lengths around its tile and buffer counts, chunks that are the
    whole sequence, a chunk shorter than one row group, sequences without query tokens."""
    print("case many rows", D, bs, layout, qdt, flush=True)
    lens = [1, 31, 32, 33, 127, 129, 160, 1000, 97, 2500]
    q_counts = [1, 31, 32, 33, 100, 129, 0, 300, 97, 257]
    kv = "bf16" if qdt == "bf16" else "fp16"
    c = Case(len(lens), 32, 8, D, bs, lens, kv=kv, qdt=qdt, layout=layout, seed=31)
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    T = int(q_indptr[-1])
    dt = torch.bfloat16 if qdt == "bf16" else torch.float16
    q = torch.randn(T, c.Hq, c.D, generator=torch.Generator().manual_seed(78)).to(dt)
    qd = q.to(c.q.device)
    out = torch.full_like(qd, 7.0)
    lse = torch.full((T, c.Hq), 3.0, dtype=torch.float32, device=qd.device)
    ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, scale=c.scale, return_lse=True,
                     q_per_seq=max(q_counts), q_indptr=torch.from_numpy(q_indptr).to(qd.device), kv_layout=layout)
    torch.cuda.synchronize()
    ref, ref_lse = orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale)
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    err = float(np.abs(got - ref).max())
    print("   err %.3e" % err, flush=True)
    assert err <= 1.2e-2
    fin = np.isfinite(ref_lse)
    assert np.allclose(lse.cpu().numpy()[fin], ref_lse[fin], atol=2e-2)


def test_many_row_kernel_split_sequences_and_window(gpu):
    """65 to 128 rows per kv head: one 128-row item per (sequence, kv head), split into chunks like
    any decode step when the batch is small; and a sliding window over a chunked step."""
    print("case many rows split / window", flush=True)
    c = Case(2, 64, 8, 128, 16, [9000, 700], n=12, seed=32)  # 96 rows; 9000 tokens are split
    ref, lse_ref = c.oracle()
    out, lse = c.run()
    assert float(np.abs(out.float().cpu().numpy() - ref).max()) <= 1.2e-2
    c = Case(2, 32, 8, 128, 16, [3000, 517], n=40, seed=33)  # 160 rows, window
    ref, _ = c.oracle(301)
    out, _ = c.run(301)
    assert float(np.abs(out.float().cpu().numpy() - ref).max()) <= 1.2e-2


@pytest.mark.parametrize("D", [128, 256])
def test_garbage_past_the_sequence_end_does_not_reach_the_many_row_kernel(gpu, D):
    print("case many rows garbage", D, flush=True)
    lens = [45, 200]
    c = Case(2, 32, 8, D, 16, lens, n=24, seed=34)
    ref, _ = c.oracle()
    # NaN in every slot past the end of each sequence's last block and in unused blocks
    nan = float("nan")
    used = torch.zeros(c.k_cache.size(0), 16, dtype=torch.bool)
    for b, L in enumerate(lens):
        for t in range(L):
            used[c.table[b, t // 16], t % 16] = True
    mask = (~used).to(c.k_cache.device)
    c.k_cache.permute(0, 2, 1, 3)[mask] = nan
    c.v_cache.permute(0, 2, 1, 3)[mask] = nan
    out, _ = c.run()
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    assert float(np.abs(got - ref).max()) <= 1.2e-2


@pytest.mark.parametrize("g,n,D,bs", [(8, 5, 128, 16), (8, 8, 128, 128), (4, 9, 128, 16), (16, 4, 64, 32), (11, 3, 128, 16)])
@pytest.mark.parametrize("qdt", ["bf16", "fp16"])
def test_thirty_three_to_sixty_four_rows(gpu, g, n, D, bs, qdt):
    """33 to 64 query rows per kv head over a 16-bit cache (speculative verify of five to eight draft
    tokens at eight heads per kv head): the many-row kernel with half of its rows absent.  Sequences
    long enough to be split, shorter than the draft count plus one tile, a sliding window."""
    print("case 33-64 rows", g, n, D, bs, qdt, flush=True)
    assert 32 < g * n <= 64
    kv = "bf16" if qdt == "bf16" else "fp16"
    c = Case(4, 4 * g, 4, D, bs, [9000, n, 517, 40], n=n, kv=kv, qdt=qdt, seed=51)
    ref, lse_ref = c.oracle()
    out, lse = c.run()
    assert not torch.isnan(out.float()).any()
    assert float(np.abs(out.float().cpu().numpy() - ref).max()) <= 1.2e-2
    fin = np.isfinite(lse_ref)
    assert np.allclose(lse.cpu().numpy()[fin], lse_ref[fin], atol=2e-2)
    ref_w, _ = c.oracle(301)
    out_w, _ = c.run(301)
    assert float(np.abs(out_w.float().cpu().numpy() - ref_w).max()) <= 1.2e-2
    # different numbers of query tokens per sequence, at most n
    counts = [n, 1, max(1, n - 2), 0]
    out_r, _, ref_r, _, _ = _run(c, counts, n) if qdt == "bf16" else (None, None, None, None, None)
    if out_r is not None:
        assert float(np.abs(out_r - ref_r).max()) <= 1.2e-2


@pytest.mark.parametrize("kv,bs,qdt", [("fp8", 16, "bf16"), ("int8", 16, "fp16"), ("fp8", 128, "fp16"), ("int8", 128, "bf16")])
def test_many_row_kernel_over_one_byte_caches(gpu, kv, bs, qdt):
    """1-byte caches at head_dim 128 with more than 32 query rows per kv head take the many-row kernels
    that bring raw bytes and scales to LDS and convert each tile once per row group (here, with up to 1200 rows
    per kv head, the 256-row one; the 128-row one in the next test and beside the 256-row one further down): lengths around
    its tile (32 tokens) and its four raw buffers, chunks that are the whole sequence, chunks shorter
    than one row group, sequences without query tokens; then a sliding window."""
    print("case many rows, 1-byte cache", kv, bs, qdt, flush=True)
    lens = [1, 31, 32, 33, 95, 96, 97, 127, 128, 129, 160, 1000, 2500]
    q_counts = [1, 31, 32, 33, 95, 9, 97, 100, 128, 129, 0, 300, 257]
    c = Case(len(lens), 32, 8, 128, bs, lens, kv=kv, qdt=qdt, seed=61)
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    T = int(q_indptr[-1])
    dt = torch.bfloat16 if qdt == "bf16" else torch.float16
    q = torch.randn(T, c.Hq, c.D, generator=torch.Generator().manual_seed(79)).to(dt)
    qd = q.to(c.q.device)
    for window in (-1, 75):
        out = torch.full_like(qd, 7.0)
        lse = torch.full((T, c.Hq), 3.0, dtype=torch.float32, device=qd.device)
        ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, None, c.k_scale, c.v_scale,
                         scale=c.scale, return_lse=True, q_per_seq=max(q_counts), kv_cache_quant_bit_size=8,
                         q_indptr=torch.from_numpy(q_indptr).to(qd.device), window_size_left=window)
        torch.cuda.synchronize()
        ref, ref_lse = orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale,
                                               window_left=window)
        got = out.float().cpu().numpy()
        assert not np.isnan(got).any()
        err = float(np.abs(got - ref).max())
        print("   window %d err %.3e" % (window, err), flush=True)
        assert err <= 1.2e-2
        fin = np.isfinite(ref_lse)
        assert np.allclose(lse.cpu().numpy()[fin], ref_lse[fin], atol=2e-2)


@pytest.mark.parametrize("kv", ["fp8", "int8"])
def test_many_row_kernel_over_one_byte_caches_split_and_garbage(gpu, kv):
    """33 to 128 rows per kv head over a 1-byte cache (one row group, long sequences split into chunks
    and merged), with bytes that decode to NaN / huge values and NaN scales in every slot that no
    sequence owns: none of it may reach the output."""
    print("case many rows, 1-byte cache, split + garbage", kv, flush=True)
    lens = [9000, 45, 700, 12]
    c = Case(4, 64, 8, 128, 16, lens, n=12, kv=kv, seed=62)  # 96 rows per kv head
    ref, lse_ref = c.oracle()
    used = torch.zeros(c.k_cache.size(0), 16, dtype=torch.bool)
    for b, L in enumerate(lens):
        for t in range(L):
            used[c.table[b, t // 16], t % 16] = True
    mask = (~used).to(c.k_cache.device)
    for cache in (c.k_cache, c.v_cache):
        cache.view(torch.uint8).permute(0, 2, 1, 3)[mask] = 0x7F  # NaN in e4m3fn, 127 in int8
    for sc in (c.k_scale, c.v_scale):
        sc.permute(0, 2, 1)[mask] = float("nan")
    out, lse = c.run()
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    assert float(np.abs(got - ref).max()) <= 1.2e-2
    fin = np.isfinite(lse_ref)
    assert np.allclose(lse.cpu().numpy()[fin], lse_ref[fin], atol=2e-2)


@pytest.mark.parametrize("kv,qdt", [("bf16", "bf16"), ("fp32", "fp32")])
def test_long_chunk_on_the_default_workspace(gpu, kv, qdt):
    """One sequence's chunk of 4096 query tokens x 32 heads (never split: no partial rows) runs on the
    shared 128 MiB workspace, on the MFMA and on the generic kernel, which then writes its rows itself.
    Checked against the oracle on sampled query tokens, each as a decode row of its own kv length
    (xllm/core/runtime/speculative_worker_impl.cpp:230-243)."""
    print("case long chunk, default workspace", kv, flush=True)
    L, n, Hq, Hkv, D = 4096, 4096, 32, 8, 128
    c = Case(1, Hq, Hkv, D, 16, [L], kv=kv, qdt=qdt, seed=41)
    assert ops.decode_workspace_bytes(1, n, Hq, Hkv, D) <= 1 << 20
    dt = torch.bfloat16 if qdt == "bf16" else torch.float32
    q = torch.randn(n, Hq, D, generator=torch.Generator().manual_seed(79)).to(dt)
    qd = q.to(c.q.device)
    out = torch.full_like(qd, 7.0)
    lse = torch.full((n, Hq), 3.0, dtype=torch.float32, device=qd.device)
    q_indptr = torch.tensor([0, n], dtype=torch.int32, device=qd.device)
    ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, scale=c.scale, return_lse=True,
                     q_per_seq=n, q_indptr=q_indptr)
    torch.cuda.synchronize()
    got = out.float().cpu().numpy()
    assert not np.isnan(got).any()
    rows = np.array([0, 1, 31, 32, 127, 128, 1000, 2047, 2048, 4094, 4095])
    table = np.repeat(c.table, len(rows), axis=0)
    ref, ref_lse = orc.paged_decode(q.float().numpy()[rows], c.k_ref, c.v_ref, table, (L - n + 1 + rows).astype(np.int32),
                                    c.scale)
    err = float(np.abs(got[rows] - ref).max())
    print("   err %.3e" % err, flush=True)
    assert err <= (1.2e-2 if kv == "bf16" else 1e-4)
    assert np.allclose(lse.cpu().numpy()[rows], ref_lse, atol=2e-2 if kv == "bf16" else 1e-4)


@pytest.mark.parametrize("qdt", ["bf16", "fp16"])
@pytest.mark.parametrize("bs,layout", [(16, "HND"), (128, "NHD")])
def test_256_row_kernel_against_the_128_row_kernel_and_the_oracle(gpu, qdt, bs, layout):
    """More than 128 query rows per kv head over a 16-bit cache at head_dim 128 take the 256-row kernel (eight
    waves in two groups that alternate between matrix and softmax phases).  Its straight-line loop takes the
    tiles every row sees in full, six at a time after the first, and a second form the rest: the prefixes here
    put 0, 1, 6, 7, 8, 13 and 30 tiles in front of the causal edge, the chunks are one item, one item and a
    few rows, and several items, one sequence is its own chunk, and one has no query tokens.  The results match
    the oracle and, to a rounding of a few outputs, the 128-row kernel (XLLM_HIP_OPTION_PREFILL_KERNEL)."""
    print("case 256-row kernel", qdt, bs, layout, flush=True)
    q_counts = [64, 40, 33, 70, 64, 200, 64, 0, 129, 300]
    prefix = [0, 32, 6 * 32, 7 * 32 + 5, 8 * 32, 13 * 32 + 31, 30 * 32 + 1, 100, 0, 1000]
    lens = [p + n for p, n in zip(prefix, q_counts)]
    kv = "bf16" if qdt == "bf16" else "fp16"
    c = Case(len(lens), 32, 8, 128, bs, lens, kv=kv, qdt=qdt, layout=layout, seed=41)
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    T = int(q_indptr[-1])
    dt = torch.bfloat16 if qdt == "bf16" else torch.float16
    q = torch.randn(T, c.Hq, c.D, generator=torch.Generator().manual_seed(79)).to(dt)
    qd = q.to(c.q.device)
    ref, ref_lse = orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale)
    ref_w, _ = orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale, window_left=150)
    got = {}
    for name, value in (("rows256", 0), ("rows128", 1)):
        with ops.option("prefill_kernel", value):
            for window in (-1, 150):
                out = torch.full_like(qd, 7.0)
                lse = torch.full((T, c.Hq), 3.0, dtype=torch.float32, device=qd.device)
                ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, scale=c.scale, return_lse=True,
                                 q_per_seq=max(q_counts), q_indptr=torch.from_numpy(q_indptr).to(qd.device), kv_layout=layout,
                                 window_size_left=window)
                torch.cuda.synchronize()
                got[name, window] = (out.float().cpu().numpy(), lse.cpu().numpy())
    for window, r in ((-1, ref), (150, ref_w)):
        o256, l256 = got["rows256", window]
        o128, l128 = got["rows128", window]
        assert not np.isnan(o256).any()
        err = float(np.abs(o256 - r).max())
        print("   window %d err %.3e" % (window, err), flush=True)
        assert err <= 1.2e-2
        # (the two kernels do the same arithmetic on the same values; where a reference point moves, the compiler
        # fuses one of them's rescaled denominator into a multiply-add, so a few outputs may round the other way)
        assert float(np.abs(o256 - o128).max()) <= 4e-3 and float(np.mean(o256 != o128)) <= 1e-4
        assert np.allclose(l256, l128, atol=1e-5, equal_nan=True)
    fin = np.isfinite(ref_lse)
    assert np.allclose(got["rows256", -1][1][fin], ref_lse[fin], atol=2e-2)
    d = ops.decode_describe(torch.empty(len(lens) * max(q_counts), c.Hq, c.D, dtype=dt, device=qd.device), c.k_cache, c.v_cache, c.block_table, c.seq_lens,
                            q_per_seq=max(q_counts), kv_layout=layout)
    assert d["waves_per_workgroup"] == 8, d


@pytest.mark.parametrize("kv,qdt,bs,layout", [("fp8", "bf16", 16, "HND"), ("int8", "fp16", 16, "HND"),
                                               ("fp8", "fp16", 128, "NHD"), ("int8", "bf16", 128, "NHD")])
def test_256_row_kernel_over_one_byte_caches(gpu, kv, qdt, bs, layout):
    """The same over a 1-byte cache: raw bytes and scales reach LDS by DMA and each wave converts its rows of the
    next tile during its matrix phase, three converted tiles rotating.  Its straight-line loop takes the tiles
    every row sees in full three at a time after the first: the prefixes put 0, 1, 3, 4, 5, 7 and 30 tiles in
    front of the causal edge.  Every slot no sequence owns holds bytes that decode to NaN or 127 and a NaN scale.
    The results match the oracle and the 128-row kernel for 1-byte caches, which converts the same values the
    same way."""
    print("case 256-row kernel, 1-byte cache", kv, qdt, bs, layout, flush=True)
    q_counts = [64, 40, 33, 70, 64, 200, 64, 0, 129, 300]
    prefix = [0, 32, 3 * 32, 4 * 32 + 5, 5 * 32, 7 * 32 + 31, 30 * 32 + 1, 100, 0, 1000]
    lens = [p + n for p, n in zip(prefix, q_counts)]
    c = Case(len(lens), 32, 8, 128, bs, lens, kv=kv, qdt=qdt, layout=layout, seed=43)
    used = torch.zeros(c.k_cache.size(0), bs, dtype=torch.bool)
    for b, L in enumerate(lens):
        for t in range(L):
            used[c.table[b, t // bs], t % bs] = True
    mask = (~used).to(c.k_cache.device)
    for cache in (c.k_cache, c.v_cache):
        view = cache.view(torch.uint8)
        (view if layout == "NHD" else view.permute(0, 2, 1, 3))[mask] = 0x7F  # NaN in e4m3fn, 127 in int8
    for sc in (c.k_scale, c.v_scale):
        (sc if layout == "NHD" else sc.permute(0, 2, 1))[mask] = float("nan")
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    T = int(q_indptr[-1])
    dt = torch.bfloat16 if qdt == "bf16" else torch.float16
    q = torch.randn(T, c.Hq, c.D, generator=torch.Generator().manual_seed(79)).to(dt)
    qd = q.to(c.q.device)
    refs = {w: orc.paged_decode_ragged(q.float().numpy(), c.k_ref, c.v_ref, c.table, c.lens, q_indptr, c.scale, window_left=w)
            for w in (-1, 150)}
    got = {}
    for name, value in (("rows256", 0), ("rows128", 1)):
        with ops.option("prefill_kernel", value):
            for window in (-1, 150):
                out = torch.full_like(qd, 7.0)
                lse = torch.full((T, c.Hq), 3.0, dtype=torch.float32, device=qd.device)
                ops.batch_decode(qd, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, lse, None, c.k_scale, c.v_scale,
                                 scale=c.scale, return_lse=True, q_per_seq=max(q_counts), kv_cache_quant_bit_size=8,
                                 q_indptr=torch.from_numpy(q_indptr).to(qd.device), kv_layout=layout, window_size_left=window)
                torch.cuda.synchronize()
                got[name, window] = (out.float().cpu().numpy(), lse.cpu().numpy())
    for window in (-1, 150):
        ref, ref_lse = refs[window]
        o256, l256 = got["rows256", window]
        o128, l128 = got["rows128", window]
        assert not np.isnan(o256).any()
        err = float(np.abs(o256 - ref).max())
        print("   window %d err %.3e" % (window, err), flush=True)
        assert err <= 1.2e-2
        # (bf16 queries become fp16 operands on one power-of-two factor per work item, which the two kernels take
        # over 256 and over 128 rows: exact either way unless a row lies 2^28 below its item's largest element)
        assert float(np.abs(o256 - o128).max()) <= 4e-3 and float(np.mean(o256 != o128)) <= 1e-4
        assert np.allclose(l256, l128, atol=1e-5, equal_nan=True)
        fin = np.isfinite(ref_lse)
        assert np.allclose(l256[fin], ref_lse[fin], atol=2e-2)
    d = ops.decode_describe(torch.empty(len(lens) * max(q_counts), c.Hq, c.D, dtype=dt, device=qd.device), c.k_cache, c.v_cache,
                            c.block_table, c.seq_lens, q_per_seq=max(q_counts), kv_layout=layout, k_cache_quant_scale=c.k_scale,
                            v_cache_quant_scale=c.v_scale)
    assert d["waves_per_workgroup"] == 8, d
