"""The five benchmark workloads on the GPU: KV write bit-exact, attention within tolerance.

Each workload runs (a) at a reduced size checked in full against the fp32 oracle and (b) at its
full size, where a sample of sequences is gathered back to the host and checked against the oracle
and the whole batch is checked through size-independent properties (block-table permutation
invariance, agreement of the MFMA kernel with the generic kernel on a sample).  Quantised pools are
filled by the path's own quantising KV write and a sample of slots is compared bit-exactly with the
oracle's quantiser.
"""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.helpers import TOL_BF16_KV, TOL_QUANT_KV
from xllm_wxh_amd import ops, workloads

pytestmark = pytest.mark.gpu

REL_TOL = 5e-2  # max-abs error of a sequence's rows over the RMS of its reference rows

TDT = {"bf16": torch.bfloat16, "fp32": torch.float32, "fp8": torch.float8_e4m3fn, "int8": torch.int8}


def build(w, gpu, seed=0):
    """Device tensors of a workload.  KV values come from N(0, value_std); quantised pools are
    written by quant_to_paged_cache from fp32 sources that are kept for the bit-exact check."""
    seq_lens = workloads.make_seq_lens(w, seed)
    table, num_blocks, lists = workloads.make_block_tables(w, seq_lens, seed)
    gen = torch.Generator(device=gpu).manual_seed(100 + seed)
    shape = (num_blocks, w.num_kv_heads, w.block_size, w.head_dim)
    qdt = TDT[w.q_dtype]
    d = dict(w=w, seq_lens=seq_lens, table=table, lists=lists, num_blocks=num_blocks)
    if w.kv_dtype in ("bf16", "fp32"):
        d["k"] = (torch.randn(shape, device=gpu, dtype=torch.float32, generator=gen) * w.value_std).to(TDT[w.kv_dtype])
        d["v"] = (torch.randn(shape, device=gpu, dtype=torch.float32, generator=gen) * w.value_std).to(TDT[w.kv_dtype])
        d["ks"] = d["vs"] = None
    else:
        cdt = TDT[w.kv_dtype]
        d["k"] = torch.zeros(shape, device=gpu, dtype=torch.int8).view(cdt)
        d["v"] = torch.zeros(shape, device=gpu, dtype=torch.int8).view(cdt)
        d["ks"] = torch.zeros(shape[:3], device=gpu)
        d["vs"] = torch.zeros(shape[:3], device=gpu)
        total = num_blocks * w.block_size
        chunk = 1 << 16
        for s0 in range(0, total, chunk):
            t = min(chunk, total - s0)
            g2 = torch.Generator(device=gpu).manual_seed(7919 * (s0 // chunk) + seed)
            # generated in fp32, then quantised per token and head (as the fp8 workload is defined)
            src_k = torch.randn(t, w.num_kv_heads, w.head_dim, device=gpu, dtype=torch.float32, generator=g2)
            src_v = torch.randn(t, w.num_kv_heads, w.head_dim, device=gpu, dtype=torch.float32, generator=g2)
            ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(
                key=src_k, value=src_v, k_cache=d["k"], v_cache=d["v"],
                slot_mapping=torch.arange(s0, s0 + t, device=gpu, dtype=torch.int32),
                k_cache_scale=d["ks"], v_cache_scale=d["vs"]))
            if s0 == 0:  # keep the first chunk's sources for the bit-exact sample check
                d["src_k0"], d["src_v0"] = src_k[:2048].cpu(), src_v[:2048].cpu()
    T = w.batch * w.q_per_seq
    d["q"] = (torch.randn(T, w.num_q_heads, w.head_dim, device=gpu, dtype=torch.float32, generator=gen) * w.q_std).to(qdt)
    d["block_table"] = torch.from_numpy(table).to(gpu)
    d["seq_lens_d"] = torch.from_numpy(seq_lens).to(gpu)
    return d


def decode(d, hints=True, block_table=None, k=None, v=None, ks=None, vs=None):
    w = d["w"]
    out = torch.full_like(d["q"], float("nan"))
    kw = {}
    if hints:
        kw = dict(max_seq_len=int(d["seq_lens"].max()), total_kv_len=int(d["seq_lens"].sum()))
    ops.batch_decode(d["q"], d["k"] if k is None else k, out, d["block_table"] if block_table is None else block_table,
                     d["seq_lens_d"], d["v"] if v is None else v, None, None, d["ks"] if ks is None else ks,
                     d["vs"] if vs is None else vs, scale=w.sm_scale, q_per_seq=w.q_per_seq,
                     kv_cache_quant_bit_size=8 if d["ks"] is not None else -1, **kw)
    torch.cuda.synchronize()
    return out


def oracle_on_sample(d, out, sample):
    """max-abs error of `out` against the fp32 oracle on the sequences in `sample` (their blocks are
    gathered to the host and renumbered)."""
    w = d["w"]
    worst = 0.0
    for b in sample:
        L = int(d["seq_lens"][b])
        nb = (L + w.block_size - 1) // w.block_size
        ids = torch.from_numpy(d["table"][b, :nb].astype(np.int64)).to(d["k"].device)
        kb, vb = d["k"][ids].cpu(), d["v"][ids].cpu()
        if d["ks"] is not None:
            ksb, vsb = d["ks"][ids].cpu().numpy(), d["vs"][ids].cpu().numpy()
            kind = w.kv_dtype
            kq = kb.view(torch.uint8).numpy() if kind == "fp8" else kb.numpy()
            vq = vb.view(torch.uint8).numpy() if kind == "fp8" else vb.numpy()
            kf, vf = orc.dequantize(kq, ksb, kind), orc.dequantize(vq, vsb, kind)
        else:
            kf, vf = kb.float().numpy(), vb.float().numpy()
        n = w.q_per_seq
        qb = d["q"][b * n:(b + 1) * n].float().cpu().numpy()
        ref, _ = orc.paged_decode(qb, kf, vf, np.arange(nb, dtype=np.int32)[None, :], np.array([L], np.int32),
                                  w.sm_scale, q_per_seq=n, acc_dtype=np.float32 if L > 8192 else np.float64)
        got = out[b * n:(b + 1) * n].float().cpu().numpy()
        assert not np.isnan(got).any()
        err = float(np.abs(got - ref).max())
        worst = max(worst, err)
        # Long sequences of zero-mean values have outputs of a few hundredths — the size of the absolute
        # tolerances — so the error is also bounded relative to the sequence's output RMS: a wrong V scale,
        # a dropped chunk or a wrong merge weight fails this where it would pass the absolute bound.
        rms = float(np.sqrt(np.mean(ref.astype(np.float64) ** 2)))
        if rms > 0.0:
            assert err <= REL_TOL * rms, (b, L, err, rms)
    return worst


def check_quant_sample(d):
    """Slots 0..2047 of a quantised pool against the oracle's quantiser, bit for bit."""
    w = d["w"]
    kind = w.kv_dtype
    nblk = 2048 // w.block_size
    for cache, scale, src in ((d["k"], d["ks"], d["src_k0"]), (d["v"], d["vs"], d["src_v0"])):
        q_ref, s_ref = orc.quantize_per_token_head(src.float().numpy(), kind)  # [2048, Hkv, D]
        got = cache[:nblk].cpu().view(torch.uint8).numpy()  # [nblk, Hkv, bs, D]
        got = got.transpose(0, 2, 1, 3).reshape(2048, w.num_kv_heads, w.head_dim)
        ref = q_ref.view(np.uint8)
        if kind == "fp8":
            same = (got == ref) | (((got & 0x7F) == 0) & ((ref & 0x7F) == 0))
            assert same.all()
        else:
            np.testing.assert_array_equal(got, ref)
        got_s = scale[:nblk].cpu().numpy().transpose(0, 2, 1).reshape(2048, w.num_kv_heads)
        np.testing.assert_array_equal(got_s, s_ref)


def kv_write_step(d, gpu):
    """The step's KV write of the new tokens (last q_per_seq positions of every sequence), checked
    bit-exactly: the written slots hold the new rows (quantised by the oracle for quantised caches),
    every other slot of the touched blocks is unchanged."""
    w = d["w"]
    T = w.batch * w.q_per_seq
    gen = torch.Generator(device=gpu).manual_seed(555)
    src_dt = torch.float32 if w.kv_dtype == "fp32" else torch.bfloat16
    new_k = torch.randn(T, w.num_kv_heads, w.head_dim, device=gpu, dtype=torch.float32, generator=gen).to(src_dt)
    new_v = torch.randn(T, w.num_kv_heads, w.head_dim, device=gpu, dtype=torch.float32, generator=gen).to(src_dt)
    slots = workloads.decode_slots(w, d["seq_lens"], d["lists"])
    assert len(np.unique(slots)) == len(slots)
    blocks = torch.from_numpy(np.unique(slots // w.block_size).astype(np.int64)).to(gpu)
    before_k, before_v = d["k"][blocks].clone(), d["v"][blocks].clone()
    p = ops.ReshapePagedCacheParams(key=new_k, value=new_v, k_cache=d["k"], v_cache=d["v"],
                                    slot_mapping=torch.from_numpy(slots).to(gpu), k_cache_scale=d["ks"],
                                    v_cache_scale=d["vs"])
    if d["ks"] is not None:
        ops.quant_to_paged_cache(p)
    else:
        ops.reshape_paged_cache(p)
    torch.cuda.synchronize()
    # expected contents of the touched blocks, built on the host with the oracle
    u8 = lambda t: t.cpu().contiguous().view(torch.uint8).numpy()
    eb = d["k"].element_size()
    for cache, before, new, scale in ((d["k"], before_k, new_k, d["ks"]), (d["v"], before_v, new_v, d["vs"])):
        exp = u8(before).reshape(before.shape + (eb,)) if eb > 1 else u8(before)
        exp = exp.copy()
        if d["ks"] is not None:
            qn, sn = orc.quantize_per_token_head(new.float().cpu().numpy(), w.kv_dtype)
            rows = qn.view(np.uint8)
        else:
            rows = u8(new).reshape(new.shape + (eb,)) if eb > 1 else u8(new)
        blk_index = {int(b): i for i, b in enumerate(blocks.cpu().numpy())}
        for t, s in enumerate(slots):
            exp[blk_index[int(s) // w.block_size], :, int(s) % w.block_size] = rows[t]
        got = u8(cache[blocks]).reshape(exp.shape)
        if w.kv_dtype == "fp8":
            same = (got == exp) | (((got & 0x7F) == 0) & ((exp & 0x7F) == 0))
            assert same.all()
        else:
            np.testing.assert_array_equal(got, exp)
        if scale is not None:
            got_s = scale[blocks].cpu().numpy()
            for t, s in enumerate(slots):
                np.testing.assert_array_equal(got_s[blk_index[int(s) // w.block_size], :, int(s) % w.block_size], sn[t])


SMALL = {
    "cfg1_cpu_fp32": dict(),
    "cfg2_llama3_8b_b64_ctx4k": dict(batch=6, seq_len=4096),
    "cfg3_ragged_b256": dict(batch=24, seq_len_max=6000),
    "cfg4_fp8_qwen3_32b": dict(batch=4, seq_len=2048),
    "cfg5_int8_spec_verify": dict(batch=2, seq_len=4096),
    "aux_d256_bf16_b64_ctx4k": dict(batch=5, seq_len=4096),
    "aux_d256_fp8_b64_ctx8k": dict(batch=3, seq_len=2048),
    "aux_d256_int8_spec_verify": dict(batch=2, seq_len=4096),
    "aux_d64_bf16_b512_ctx4k": dict(batch=6, seq_len=3000),
    "aux_d64_int8_b512_ctx8k": dict(batch=4, seq_len=5000),
    "aux_b1_ctx32k": dict(),
    "aux_b8_ctx8k": dict(batch=3),
}


@pytest.mark.parametrize("name", list(workloads.WORKLOADS))
def test_workload_reduced_size_full_check(gpu, name):
    print("case workload small", name, flush=True)
    w = workloads.scaled(workloads.WORKLOADS[name], **SMALL[name]) if SMALL[name] else workloads.WORKLOADS[name]
    d = build(w, gpu)
    if d["ks"] is not None:
        check_quant_sample(d)
    kv_write_step(d, gpu)  # write first, then attend (flashinfer_attention.cpp:135-153)
    tol = TOL_QUANT_KV if d["ks"] is not None else (1e-5 if w.kv_dtype == "fp32" else TOL_BF16_KV)
    for hints in (False, True):
        out = decode(d, hints=hints)
        err = oracle_on_sample(d, out, range(w.batch))
        print("   %s hints=%s max-abs err %.3e (tol %.0e)" % (w.name, hints, err, tol), flush=True)
        assert err <= tol


FULL = [n for n in workloads.WORKLOADS if n.startswith("cfg") and n != "cfg1_cpu_fp32"]


@pytest.mark.parametrize("name", FULL)
def test_workload_full_size(gpu, name):
    print("case workload full", name, flush=True)
    w = workloads.WORKLOADS[name]
    d = build(w, gpu)
    if d["ks"] is not None:
        check_quant_sample(d)
    kv_write_step(d, gpu)
    out = decode(d)
    assert not torch.isnan(out.float()).any()
    # (1) oracle on a sample of sequences (shortest, longest, first, last)
    order = np.argsort(d["seq_lens"])
    sample = sorted({int(order[0]), int(order[-1]), 0, w.batch - 1})
    if w.seq_len > 16384:
        sample = sample[:2]
    tol = TOL_QUANT_KV if d["ks"] is not None else TOL_BF16_KV
    err = oracle_on_sample(d, out, sample)
    print("   %s sample %s max-abs err %.3e (tol %.0e)" % (w.name, sample, err, tol), flush=True)
    assert err <= tol
    # (2) same result without the host length hints (device-side split decision + merge kernel)
    out_nohint = decode(d, hints=False)
    assert float((out.float() - out_nohint.float()).abs().max()) <= tol / 4
    # (3) block-table permutation invariance, bitwise: move every block, remap the table
    perm = torch.randperm(d["num_blocks"], generator=torch.Generator().manual_seed(1)).to(gpu)
    k2, v2 = torch.empty_like(d["k"]), torch.empty_like(d["v"])
    k2[perm] = d["k"]
    v2[perm] = d["v"]
    ks2 = vs2 = None
    if d["ks"] is not None:
        ks2, vs2 = torch.empty_like(d["ks"]), torch.empty_like(d["vs"])
        ks2[perm] = d["ks"]
        vs2[perm] = d["vs"]
    table2 = perm[d["block_table"].long()].to(torch.int32)
    out2 = decode(d, block_table=table2, k=k2, v=v2, ks=ks2, vs=vs2)
    assert torch.equal(out, out2)
    del k2, v2, ks2, vs2
    # (4) the generic kernel agrees with the MFMA kernel on a slice of the batch
    nb = min(2, w.batch)
    n = w.q_per_seq
    out_g = torch.full_like(d["q"][: nb * n], float("nan"))
    with ops.option("force_generic"):
        assert ops.decode_variant(d["q"][: nb * n], d["k"], d["v"], d["block_table"][:nb], d["seq_lens_d"][:nb],
                                  d["ks"], d["vs"], q_per_seq=n) == "generic"
        ops.batch_decode(d["q"][: nb * n], d["k"], out_g, d["block_table"][:nb], d["seq_lens_d"][:nb], d["v"], None, None,
                         d["ks"], d["vs"], scale=w.sm_scale, q_per_seq=n,
                         kv_cache_quant_bit_size=8 if d["ks"] is not None else -1)
        torch.cuda.synchronize()
    diff = float((out_g.float() - out[: nb * n].float()).abs().max())
    print("   generic vs mfma on %d sequences: %.3e" % (nb, diff), flush=True)
    assert diff <= tol / 2


def test_fp8_workload_full_size_over_nhd(gpu):
    """The fp8 workload at full size over an NHD cache (the reference's CUDA layout), where the 16-row kernel
    gives a work item four kv heads: oracle on sampled sequences, and agreement with the same step in HND."""
    print("case workload full nhd fp8", flush=True)
    w = workloads.WORKLOADS["cfg4_fp8_qwen3_32b"]
    d = build(w, gpu)
    out_hnd = decode(d)
    nhd = lambda t: t.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)  # NHD memory, HND view
    nhd_s = lambda t: t.permute(0, 2, 1).contiguous().permute(0, 2, 1)
    k, v, ks, vs = nhd(d["k"]), nhd(d["v"]), nhd_s(d["ks"]), nhd_s(d["vs"])
    assert k.stride(1) == w.head_dim  # a head's row is followed by the next head's
    out = decode(d, k=k, v=v, ks=ks, vs=vs)
    assert not torch.isnan(out.float()).any()
    err = oracle_on_sample(d, out, [0, w.batch - 1])
    print("   max-abs err %.3e" % err, flush=True)
    assert err <= TOL_QUANT_KV
    assert float((out.float() - out_hnd.float()).abs().max()) <= TOL_QUANT_KV / 4
    with ops.option("item_per_head"):
        out_1 = decode(d, k=k, v=v, ks=ks, vs=vs)
    assert torch.equal(out_1, out_hnd)  # one head per item: only the strides differ
