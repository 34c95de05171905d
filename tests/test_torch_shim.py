"""The libtorch host side (C++ mirrors of xllm::kernel / xllm::layer for the decode path):
host-only behaviour on the CPU, the whole write-then-attend dispatch on the GPU."""
import os

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import build as xbuild


@pytest.fixture(scope="module")
def shim():
    if not os.path.exists(xbuild.TORCH_SHIM_PATH):
        xbuild.build_torch_shim(verbose=False)
    from xllm_wxh_amd import _xllm_hip_torch

    return _xllm_hip_torch


def test_metadata_builder_matches_reference_known_answers(shim):
    # cumulative layout of batch_test.cpp:176-189; kv_seq_lens = diff (attention_metadata_builder.cpp:105)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    md = shim.build_decode_metadata(i32([0, 9, 10, 11, 15]), i32([0, 9, 17, 33, 41]), i32([4, 23, 47, 56]),
                                    i32([[1, 2, 3, 0, 0], [4, 5, 6, 7, 0], [8, 9, 10, 11, 12], [13, 14, 15, 0, 0]]),
                                    9, 16, 41)
    md.plan_info.layer_id = 0
    assert md.kv_seq_lens.tolist() == [9, 8, 16, 8]
    assert md.q_seq_lens.tolist() == [9, 1, 1, 4]
    assert md.max_seq_len == 16 and md.max_query_len == 9 and not md.is_dummy
    dummy = shim.build_decode_metadata(i32([0, 0]), i32([0, 0]), i32([0]), i32([[0]]), 0, 0, 0)
    dummy.plan_info.layer_id = 0
    assert dummy.is_dummy and dummy.slot_mapping.tolist() == [1]


def test_kv_cache_scale_getters(shim):
    k = torch.zeros(2, 1, 4, 8)
    kv = shim.KVCache(k, k)
    assert kv.get_k_cache_scale() is None and not kv.empty()
    kv = shim.KVCache(k.to(torch.int8), k.to(torch.int8), torch.ones(2, 1, 4), torch.ones(2, 1, 4))
    assert kv.get_k_cache_scale() is not None
    kv = shim.KVCache(k.to(torch.int8), k.to(torch.int8), torch.empty(0), torch.empty(0))
    assert kv.get_k_cache_scale() is None  # empty scale tensors mean "not quantised" (kv_cache.cpp:56-67)
    assert shim.KVCache().empty()


def test_contract_violations_throw_before_any_launch(shim):
    p = shim.ReshapePagedCacheParams()
    p.key = torch.zeros(3, 2, 8)
    p.value = torch.zeros(3, 2, 8)
    p.k_cache = torch.zeros(2, 2, 4, 8)
    p.v_cache = torch.zeros(2, 2, 4, 8)
    p.slot_mapping = torch.zeros(3, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="slot_mapping"):
        shim.reshape_paged_cache(p)
    p.slot_mapping = torch.zeros(3, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="k_cache_scale is required"):
        shim.quant_to_paged_cache(p)
    with pytest.raises(RuntimeError, match="GPU"):
        shim.reshape_paged_cache(p)


@pytest.mark.gpu
@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_attention_impl_write_then_attend(gpu, shim, kv):
    """AttentionImpl::forward on a decode step: the new token's K/V land in the cache bit-exactly and
    the output matches the oracle run on the updated cache."""
    print("case shim AttentionImpl", kv, flush=True)
    B, Hq, Hkv, D, bs = 5, 32, 8, 128, 16
    lens = np.array([300, 17, 1, 4096, 64], np.int32)  # kv lengths including the new token
    rng = np.random.default_rng(3)
    need = (lens + bs - 1) // bs
    nblocks = int(need.sum()) + 2
    perm = rng.permutation(nblocks - 1) + 1
    lists, o = [], 0
    for b in range(B):
        lists.append(perm[o:o + need[b]].astype(np.int32))
        o += int(need[b])
    table = orc.pad_block_tables(lists)
    slots = np.array([orc.kv_cache_slots(lists[b], bs, int(lens[b]) - 1, int(lens[b]))[0] for b in range(B)], np.int32)
    g = torch.Generator().manual_seed(5)
    kf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    vf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)  # fused projection output
    q, k, v = qkv[:, : Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:]
    scale = 1.0 / float(np.sqrt(D))

    k_new = k.float().numpy().reshape(B, Hkv, D)
    v_new = v.float().numpy().reshape(B, Hkv, D)
    if kv == "bf16":
        kc, vc = kf.to(torch.bfloat16), vf.to(torch.bfloat16)
        k_ref, v_ref = kc.float().numpy(), vc.float().numpy()
        orc.reshape_paged_cache(slots, k_new, v_new, k_ref, v_ref, "HND")
        cache = shim.KVCache(kc.to(gpu), vc.to(gpu))
        k_deq, v_deq = k_ref, v_ref
    else:
        qk, sk = orc.quantize_per_token_head(kf.numpy(), "int8")
        qv, sv = orc.quantize_per_token_head(vf.numpy(), "int8")
        orc.quant_to_paged_cache(slots, k_new, v_new, qk, qv, sk, sv, "int8", "HND")
        cache = shim.KVCache(torch.from_numpy(orc.quantize_per_token_head(kf.numpy(), "int8")[0]).to(gpu),
                             torch.from_numpy(orc.quantize_per_token_head(vf.numpy(), "int8")[0]).to(gpu),
                             torch.from_numpy(orc.quantize_per_token_head(kf.numpy(), "int8")[1]).to(gpu),
                             torch.from_numpy(orc.quantize_per_token_head(vf.numpy(), "int8")[1]).to(gpu))
        k_deq, v_deq = orc.dequantize(qk, sk, "int8"), orc.dequantize(qv, sv, "int8")
    ref, _ = orc.paged_decode(q.float().numpy().reshape(B, Hq, D), k_deq, v_deq, table, lens, scale)

    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    cu_kv = np.concatenate([[0], np.cumsum(lens)])
    md = shim.build_decode_metadata(i32(np.arange(B + 1)), i32(cu_kv), i32(slots), i32(table), 1, int(lens.max()),
                                    int(lens.sum()))
    md.plan_info.layer_id = 0
    attn = shim.AttentionImpl(Hq, D, scale, Hkv, -1)
    qkv_d = qkv.to(gpu)
    out, lse = attn.forward(md, qkv_d[:, : Hq * D], qkv_d[:, Hq * D:(Hq + Hkv) * D], qkv_d[:, (Hq + Hkv) * D:], cache)
    torch.cuda.synchronize()
    assert lse is None and tuple(out.shape) == (B, Hq * D)
    # the write is bit-exact
    if kv == "bf16":
        assert np.array_equal(cache.get_k_cache().float().cpu().numpy(), k_ref)
        assert np.array_equal(cache.get_v_cache().float().cpu().numpy(), v_ref)
    else:
        assert np.array_equal(cache.get_k_cache().cpu().numpy(), qk)
        assert np.array_equal(cache.get_v_cache_scale().cpu().numpy(), sv)
    err = float(np.abs(out.float().cpu().numpy().reshape(B, Hq, D) - ref).max())
    print("   err %.3e" % err, flush=True)
    assert err <= (5e-2 if kv == "int8" else 2e-2)

    # dummy batch / empty step: untouched buffer of the right shape, nothing launched
    md.is_dummy = True
    out2, _ = attn.forward(md, qkv_d[:, : Hq * D], qkv_d[:, Hq * D:(Hq + Hkv) * D], qkv_d[:, (Hq + Hkv) * D:], cache)
    assert tuple(out2.shape) == (B, Hq * D)
    md.is_dummy = False


@pytest.mark.gpu
def test_cpp_ops_match_python_ops(gpu, shim):
    print("case shim ops", flush=True)
    from tests.helpers import Case

    case = Case(3, 32, 8, 128, 16, [500, 33, 2000], seed=41)
    ref, _ = case.run()
    out = torch.empty_like(case.q).view(3, 1, 32, 128)
    lse = torch.empty(3, 32, dtype=torch.float32, device=gpu)
    shim.batch_decode(case.q.view(3, 1, 32, 128), case.k_cache, out, case.block_table, case.seq_lens, case.v_cache,
                      lse, None, None, 2000, -1, case.scale, True, -1)
    torch.cuda.synchronize()
    assert torch.equal(out.view(3, 32, 128), ref)
    # CSR form with the CUDA backend's NHD cache shape
    lists = [case.table[i, : (int(L) + 15) // 16] for i, L in enumerate(case.lens)]
    indptr, indices, last = orc.build_paged_kv_csr(lists, case.lens, 16)
    out_c = torch.empty_like(case.q)
    shim.batch_decode_csr(case.q, case.k_cache.permute(0, 2, 1, 3).contiguous(),
                          case.v_cache.permute(0, 2, 1, 3).contiguous(), torch.from_numpy(indptr).to(gpu),
                          torch.from_numpy(indices).to(gpu), torch.from_numpy(last).to(gpu), -1, case.scale, out_c)
    torch.cuda.synchronize()
    assert torch.equal(out_c, ref)
    # ... and over a quantised cache (fp8 KV is what the CUDA-shaped caller anticipates,
    # xllm/core/kernels/cuda/utils.cpp:275-293): scales in the same NHD shape
    for kv in ("fp8", "int8"):
        cq = Case(3, 32, 8, 128, 16, [500, 33, 2000], kv=kv, seed=42)
        want, _ = cq.oracle()
        lists = [cq.table[i, : (int(L) + 15) // 16] for i, L in enumerate(cq.lens)]
        indptr, indices, last = orc.build_paged_kv_csr(lists, cq.lens, 16)
        out_q = torch.full_like(cq.q, float("nan"))
        shim.batch_decode_csr(cq.q, cq.k_cache.permute(0, 2, 1, 3).contiguous(), cq.v_cache.permute(0, 2, 1, 3).contiguous(),
                              torch.from_numpy(indptr).to(gpu), torch.from_numpy(indices).to(gpu),
                              torch.from_numpy(last).to(gpu), -1, cq.scale, out_q,
                              k_cache_scale=cq.k_scale.permute(0, 2, 1).contiguous(),
                              v_cache_scale=cq.v_scale.permute(0, 2, 1).contiguous())
        torch.cuda.synchronize()
        assert float(np.abs(out_q.float().cpu().numpy() - want).max()) <= cq.tol


@pytest.mark.gpu
def test_kv_cache_swap_blocks_and_copy_blocks(gpu, shim):
    import numpy as np
    from oracle import paged_kv_oracle as orc

    print("case shim swap_blocks / copy_blocks", flush=True)
    g = torch.Generator().manual_seed(4)
    k = torch.randint(-128, 128, (12, 2, 16, 128), generator=g, dtype=torch.int8)
    v = torch.randint(-128, 128, (12, 2, 16, 128), generator=g, dtype=torch.int8)
    ks, vs = torch.rand(12, 2, 16, generator=g), torch.rand(12, 2, 16, generator=g)
    kv = shim.KVCache(k.to(gpu), v.to(gpu), ks.to(gpu), vs.to(gpu))
    src, dst = [0, 3, 5], [3, 5, 7]  # a chain: each destination must receive the old source
    ref = [t.numpy().copy() for t in (k, v, ks, vs)]
    orc.swap_blocks(ref, src, dst)
    kv.swap_blocks(torch.tensor(src, device=gpu), torch.tensor(dst, device=gpu))
    got = [kv.get_k_cache(), kv.get_v_cache(), kv.get_k_cache_scale(), kv.get_v_cache_scale()]
    for a, b in zip(got, ref):
        assert np.array_equal(a.cpu().numpy(), b)
    s, d, c = orc.build_block_copy_groups([(1, 8), (1, 9), (2, 10)])
    orc.copy_blocks(ref, s, d, c)
    i32 = dict(dtype=torch.int32, device=gpu)
    shim.copy_blocks(got[0], got[1], got[2], got[3], torch.tensor(s, **i32), torch.tensor(d, **i32),
                     torch.tensor(c, **i32))
    for a, b in zip(got, ref):
        assert np.array_equal(a.cpu().numpy(), b)


@pytest.mark.gpu
def test_reshape_from_cache_and_dequant_from_paged_cache_params(gpu, shim):
    """The ReshapeFromCacheParams operators give what the Python mirrors give (those are checked
    bit-exactly against the oracle)."""
    from xllm_wxh_amd import ops

    print("case shim reshape_from_cache / dequant_from_paged_cache", flush=True)
    g = torch.Generator().manual_seed(6)
    k = torch.randint(-128, 128, (12, 2, 16, 128), generator=g, dtype=torch.int8).to(gpu)
    v = torch.randint(-128, 128, (12, 2, 16, 128), generator=g, dtype=torch.int8).to(gpu)
    ks, vs = torch.rand(12, 2, 16, generator=g).to(gpu), torch.rand(12, 2, 16, generator=g).to(gpu)
    lens = torch.tensor([40, 7], dtype=torch.int32, device=gpu)
    bt = torch.tensor([[3, 9, 1], [5, 0, 0]], dtype=torch.int32, device=gpu)

    p = shim.ReshapeFromCacheParams()
    p.key = torch.zeros(47, 2, 128, dtype=torch.bfloat16, device=gpu)
    p.value = torch.zeros_like(p.key)
    p.key_cache, p.value_cache = k, v
    p.key_cache_quant_scale, p.value_cache_quant_scale = ks, vs
    p.context_lengths, p.max_context_len, p.block_tables = lens, 40, bt
    shim.dequant_from_paged_cache(p)
    want_k, want_v = torch.zeros_like(p.key), torch.zeros_like(p.key)
    ops.dequant_from_paged_cache(want_k, want_v, k, v, ks, vs, lens, 40, None, bt)
    assert torch.equal(p.key, want_k) and torch.equal(p.value, want_v)
    assert p.key.abs().sum() > 0

    r = shim.ReshapeFromCacheParams()
    r.key = torch.zeros(47, 2, 128, dtype=torch.int8, device=gpu)
    r.key_cache = k
    r.context_lengths, r.max_context_len, r.block_tables = lens, 40, bt
    shim.reshape_from_cache(r)
    want = torch.zeros_like(r.key)
    ops.reshape_from_cache(want, None, k, None, lens, 40, None, bt)
    assert torch.equal(r.key, want)
    assert torch.equal(r.key[40:47], k[5, :, :7].permute(1, 0, 2))

    r.block_tables = None  # the linear mode is refused, as is a dequant without scales
    with pytest.raises(RuntimeError):
        shim.reshape_from_cache(r)
    p.key_cache_quant_scale = None
    with pytest.raises(RuntimeError):
        shim.dequant_from_paged_cache(p)


@pytest.mark.gpu
@pytest.mark.parametrize("norm", [True, False])
def test_attention_impl_forward_qkv_equals_separate_steps(gpu, shim, norm):
    """forward_qkv (norm + rotation + KV write in one launch, then decode) gives bit for bit what the
    separate operators give: fused_qk_norm_rope / rotary_embedding on the buffer, then forward."""
    from xllm_wxh_amd import ops

    print("case shim forward_qkv", norm, flush=True)
    B, Hq, Hkv, D, bs, nblocks = 6, 32, 8, 128, 16, 64
    lens = np.array([33, 1, 200, 64, 17, 300], np.int32)
    rng = np.random.default_rng(9)
    need = (lens + bs - 1) // bs
    perm = rng.permutation(nblocks - 1) + 1
    lists, o = [], 0
    for b in range(B):
        lists.append(perm[o:o + need[b]].astype(np.int32))
        o += int(need[b])
    table = orc.pad_block_tables(lists)
    slots = np.array([orc.kv_cache_slots(lists[b], bs, int(lens[b]) - 1, int(lens[b]))[0] for b in range(B)], np.int32)
    g = torch.Generator().manual_seed(6)
    kc = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16)
    qkv = torch.randn(B, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    qw = torch.randn(D, generator=g).to(torch.bfloat16).to(gpu) if norm else None
    kw = torch.randn(D, generator=g).to(torch.bfloat16).to(gpu) if norm else None
    theta = torch.rand(512, D // 2, generator=g) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(torch.bfloat16).to(gpu)
    pos = torch.from_numpy(lens.astype(np.int64) - 1).to(gpu)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    cu_kv = np.concatenate([[0], np.cumsum(lens)])
    md = shim.build_decode_metadata(i32(np.arange(B + 1)), i32(cu_kv), i32(slots), i32(table), 1, int(lens.max()),
                                    int(lens.sum()))
    md.plan_info.layer_id = 0
    attn = shim.AttentionImpl(Hq, D, 1.0 / float(np.sqrt(D)), Hkv, -1)

    a = qkv.to(gpu)
    cache_a = shim.KVCache(kc.to(gpu), vc.to(gpu))
    if norm:
        shim.fused_qk_norm_rope(a, Hq, Hkv, Hkv, D, 1e-6, qw, kw, cos_sin, False, pos)
    else:
        shim.rotary_embedding(pos, a[:, : Hq * D], a[:, Hq * D:(Hq + Hkv) * D], cos_sin, True)
    out_a, _ = attn.forward(md, a[:, : Hq * D], a[:, Hq * D:(Hq + Hkv) * D], a[:, (Hq + Hkv) * D:], cache_a)

    b = qkv.to(gpu)
    cache_b = shim.KVCache(kc.to(gpu), vc.to(gpu))
    out_b, _ = attn.forward_qkv(md, pos, b, cos_sin, False, qw, kw, 1e-6, cache_b)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert torch.equal(cache_a.get_k_cache(), cache_b.get_k_cache())
    assert torch.equal(cache_a.get_v_cache(), cache_b.get_v_cache())
    assert torch.equal(out_a, out_b)
    # and the rotation is the oracle's
    want = orc.fused_qk_norm_rope(qkv.float().numpy(), Hq, Hkv, Hkv, D, 1e-6,
                                  qw.float().cpu().numpy() if norm else None,
                                  kw.float().cpu().numpy() if norm else None, cos_sin.float().cpu().numpy(), False,
                                  pos.cpu().numpy(), "bf16", round_each_op=not norm)
    got = b.float().cpu().numpy()
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want) + 1e-30)


@pytest.mark.gpu
@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_attention_impl_chunked_prefill_step(gpu, shim, kv):
    """A mixed step through AttentionImpl::forward: prefill chunks of different sizes and decode tokens,
    the new K/V written through slot_mapping first, then attended from the (quantised) cache."""
    print("case shim chunked prefill", kv, flush=True)
    Hq, Hkv, D, bs = 32, 8, 128, 16
    lens = np.array([200, 48, 1000, 7], np.int32)      # kv lengths including this step's tokens
    q_counts = np.array([40, 48, 1, 7], np.int32)
    B, T = len(lens), int(q_counts.sum())
    rng = np.random.default_rng(13)
    need = (lens + bs - 1) // bs
    nblocks = int(need.sum()) + 2
    perm = rng.permutation(nblocks - 1) + 1
    lists, o = [], 0
    for b in range(B):
        lists.append(perm[o:o + need[b]].astype(np.int32))
        o += int(need[b])
    table = orc.pad_block_tables(lists)
    slots = np.concatenate([orc.kv_cache_slots(lists[b], bs, int(lens[b] - q_counts[b]), int(lens[b]))
                            for b in range(B)]).astype(np.int32)
    g = torch.Generator().manual_seed(8)
    kf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    vf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    q, k, v = qkv[:, : Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:]
    k_new, v_new = k.float().numpy().reshape(T, Hkv, D), v.float().numpy().reshape(T, Hkv, D)
    if kv == "bf16":
        kc, vc = kf.to(torch.bfloat16), vf.to(torch.bfloat16)
        k_ref, v_ref = kc.float().numpy(), vc.float().numpy()
        orc.reshape_paged_cache(slots, k_new, v_new, k_ref, v_ref, "HND")
        cache = shim.KVCache(kc.to(gpu), vc.to(gpu))
    else:
        qk, sk = orc.quantize_per_token_head(kf.numpy(), "int8")
        qv, sv = orc.quantize_per_token_head(vf.numpy(), "int8")
        cache = shim.KVCache(torch.from_numpy(qk.copy()).to(gpu), torch.from_numpy(qv.copy()).to(gpu),
                             torch.from_numpy(sk.copy()).to(gpu), torch.from_numpy(sv.copy()).to(gpu))
        orc.quant_to_paged_cache(slots, k_new, v_new, qk, qv, sk, sv, "int8", "HND")
        k_ref, v_ref = orc.dequantize(qk, sk, "int8"), orc.dequantize(qv, sv, "int8")
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    scale = 1.0 / float(np.sqrt(D))
    ref, _ = orc.paged_decode_ragged(q.float().numpy().reshape(T, Hq, D), k_ref, v_ref, table, lens, q_indptr, scale)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    md = shim.build_decode_metadata(i32(q_indptr), i32(np.concatenate([[0], np.cumsum(lens)])), i32(slots), i32(table),
                                    int(q_counts.max()), int(lens.max()), int(lens.sum()))
    md.plan_info.layer_id = 0
    md.is_chunked_prefill = True
    attn = shim.AttentionImpl(Hq, D, scale, Hkv, -1)
    qkv_d = qkv.to(gpu)
    out, _ = attn.forward(md, qkv_d[:, : Hq * D], qkv_d[:, Hq * D:(Hq + Hkv) * D], qkv_d[:, (Hq + Hkv) * D:], cache)
    torch.cuda.synchronize()
    err = float(np.abs(out.float().cpu().numpy().reshape(T, Hq, D) - ref).max())
    print("   err %.3e" % err, flush=True)
    assert err <= (5e-2 if kv == "int8" else 2e-2)


@pytest.mark.gpu
def test_long_prefill_chunk_runs_on_the_default_workspace(gpu, shim):
    """A chunk of 4096 query tokens x 32 heads through AttentionImpl::forward on the layer's own 128 MiB
    workspace (a never-split step needs no partial rows); same bits as the C ABI called directly."""
    from xllm_wxh_amd import ops

    print("case shim long chunk", flush=True)
    Hq, Hkv, D, bs, L = 32, 8, 128, 16, 4096
    nblocks = L // bs + 2
    lst = (np.random.default_rng(3).permutation(nblocks - 1) + 1)[: L // bs].astype(np.int32)
    slots = np.asarray(orc.kv_cache_slots(lst, bs, 0, L), np.int32)
    g = torch.Generator().manual_seed(19)
    qkv = torch.randn(L, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16).to(gpu)
    cache = shim.KVCache(torch.zeros(nblocks, Hkv, bs, D, dtype=torch.bfloat16, device=gpu),
                         torch.zeros(nblocks, Hkv, bs, D, dtype=torch.bfloat16, device=gpu))
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    md = shim.build_decode_metadata(i32([0, L]), i32([0, L]), i32(slots), i32(lst[None, :]), L, L, L)
    md.plan_info.layer_id = 0
    md.is_chunked_prefill = True
    scale = 1.0 / float(np.sqrt(D))
    attn = shim.AttentionImpl(Hq, D, scale, Hkv, -1)
    out, _ = attn.forward(md, qkv[:, : Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:], cache)
    torch.cuda.synchronize()
    want = torch.empty(L, Hq, D, dtype=torch.bfloat16, device=gpu)
    ops.batch_decode(qkv[:, : Hq * D].reshape(L, Hq, D), cache.get_k_cache(), want, i32(lst[None, :]), i32([L]),
                     cache.get_v_cache(), scale=scale, q_per_seq=L, q_indptr=i32([0, L]))
    torch.cuda.synchronize()
    assert torch.equal(out.reshape(L, Hq, D), want)
    assert float(out.float().abs().max()) > 0.0


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["int8", "fp8"])
def test_prefill_chunks_over_a_quantised_cache_take_the_dense_route(gpu, shim, kind):
    """Large chunks over a 1-byte cache: AttentionImpl dequantises the cached ranges into a dense copy
    and attends that (the reference's MLU order of operations); same result as attending the
    quantised cache in place, and the oracle's."""
    print("case shim dense prefill route", kind, flush=True)
    Hq, Hkv, D, bs = 32, 8, 128, 16
    lens = np.array([700, 300, 1031, 129], np.int32)      # kv lengths including this step's tokens
    q_counts = np.array([300, 300, 131, 129], np.int32)   # rows per kv head: 4 * 215 on average
    B, T = len(lens), int(q_counts.sum())
    rng = np.random.default_rng(17)
    need = (lens + bs - 1) // bs
    nblocks = int(need.sum()) + 2
    perm = rng.permutation(nblocks - 1) + 1
    lists, o = [], 0
    for b in range(B):
        lists.append(perm[o:o + need[b]].astype(np.int32))
        o += int(need[b])
    table = orc.pad_block_tables(lists)
    slots = np.concatenate([orc.kv_cache_slots(lists[b], bs, int(lens[b] - q_counts[b]), int(lens[b]))
                            for b in range(B)]).astype(np.int32)
    g = torch.Generator().manual_seed(18)
    kf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    vf = torch.randn(nblocks, Hkv, bs, D, generator=g)
    qkv = torch.randn(T, (Hq + 2 * Hkv) * D, generator=g).to(torch.bfloat16)
    q = qkv[:, : Hq * D]
    k_new = qkv[:, Hq * D:(Hq + Hkv) * D].float().numpy().reshape(T, Hkv, D)
    v_new = qkv[:, (Hq + Hkv) * D:].float().numpy().reshape(T, Hkv, D)
    qk, sk = orc.quantize_per_token_head(kf.numpy(), kind)
    qv, sv = orc.quantize_per_token_head(vf.numpy(), kind)
    tdt = torch.int8 if kind == "int8" else torch.float8_e4m3fn

    def fresh_cache():
        return shim.KVCache(torch.from_numpy(qk.view(np.uint8).copy()).view(tdt).to(gpu),
                            torch.from_numpy(qv.view(np.uint8).copy()).view(tdt).to(gpu),
                            torch.from_numpy(sk.copy()).to(gpu), torch.from_numpy(sv.copy()).to(gpu))

    qk2, qv2, sk2, sv2 = qk.copy(), qv.copy(), sk.copy(), sv.copy()
    orc.quant_to_paged_cache(slots, k_new, v_new, qk2, qv2, sk2, sv2, kind, "HND")
    k_ref, v_ref = orc.dequantize(qk2, sk2, kind), orc.dequantize(qv2, sv2, kind)
    q_indptr = np.concatenate([[0], np.cumsum(q_counts)]).astype(np.int32)
    scale = 1.0 / float(np.sqrt(D))
    ref, _ = orc.paged_decode_ragged(q.float().numpy().reshape(T, Hq, D), k_ref, v_ref, table, lens, q_indptr, scale)
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    md = shim.build_decode_metadata(i32(q_indptr), i32(np.concatenate([[0], np.cumsum(lens)])), i32(slots), i32(table),
                                    int(q_counts.max()), int(lens.max()), int(lens.sum()))
    md.plan_info.layer_id = 0
    md.is_chunked_prefill = True
    outs = []
    for rows in (128, 0):  # dense route, then in place
        attn = shim.AttentionImpl(Hq, D, scale, Hkv, -1)
        attn.set_prefill_dequant_rows(rows)
        qkv_d = qkv.to(gpu)
        out, _ = attn.forward(md, qkv_d[:, : Hq * D], qkv_d[:, Hq * D:(Hq + Hkv) * D], qkv_d[:, (Hq + Hkv) * D:],
                              fresh_cache())
        torch.cuda.synchronize()
        outs.append(out.float().cpu().numpy().reshape(T, Hq, D))
        err = float(np.abs(outs[-1] - ref).max())
        print("   dequant rows %d: err %.3e" % (rows, err), flush=True)
        assert err <= 5e-2
    # the dense copy is the dequantised cache rounded to bf16: the two routes differ by that rounding only
    assert float(np.abs(outs[0] - outs[1]).max()) <= 2e-2
    # The dense route layer by layer, as the model's loop drives it: layer 0 makes the copy's block table and the
    # step's schedule, later layers reuse both, and every layer's copy goes through the same persistent buffers.
    attn = shim.AttentionImpl(Hq, D, scale, Hkv, -1)
    attn.set_prefill_dequant_rows(128)
    cache = fresh_cache()
    qkv_d = qkv.to(gpu)
    for layer in (0, 1, 2):
        md.plan_info.layer_id = layer
        out, _ = attn.forward(md, qkv_d[:, : Hq * D], qkv_d[:, Hq * D:(Hq + Hkv) * D], qkv_d[:, (Hq + Hkv) * D:], cache)
        torch.cuda.synchronize()
        assert np.array_equal(out.float().cpu().numpy().reshape(T, Hq, D), outs[0]), layer
    md.plan_info.layer_id = 0


@pytest.mark.gpu
@pytest.mark.parametrize("hints", [False, True])
def test_forward_qkv_replays_under_hip_graph(gpu, shim, hints):
    """AttentionImpl::forward_qkv (norm + rotation + KV write, then decode) captured in a HIP graph and
    replayed on changing persistent inputs.  Without hints, total_kv_len = 0 in the metadata keeps host-side
    lengths out of the captured kernel choice.  With hints the graph is captured for its bucket's bounds
    (max_seq_len and total_kv_len = batch x max_seq_len, as an engine captures a batch-size bucket): the
    step then stores no schedule, every work item derives its chunk from the sequence's length on the
    device, and replays with any shorter lengths stay correct.  Every replay is compared with an eager
    call, and the hinted form with the unhinted one."""
    print("case shim graph", hints, flush=True)
    B, Hq, Hkv, D, bs, max_blocks = 4, 32, 8, 128, 16, 260
    nblocks = B * max_blocks + 1
    g = torch.Generator().manual_seed(61)
    perm = (torch.randperm(nblocks - 1, generator=g) + 1).to(torch.int32)
    table_full = perm[: B * max_blocks].view(B, max_blocks)
    k_cache = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16).to(gpu)
    v_cache = torch.randn(nblocks, Hkv, bs, D, generator=g).to(torch.bfloat16).to(gpu)
    theta = torch.rand(8192, D // 2, generator=g) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(torch.bfloat16).to(gpu)
    # persistent inputs
    qkv = torch.zeros(B, (Hq + 2 * Hkv) * D, dtype=torch.bfloat16, device=gpu)
    qkv_src = torch.zeros_like(qkv)
    positions = torch.zeros(B, dtype=torch.int64, device=gpu)
    slots = torch.zeros(B, dtype=torch.int32, device=gpu)
    kv_cu = torch.zeros(B + 1, dtype=torch.int32, device=gpu)
    q_cu = torch.arange(B + 1, dtype=torch.int32, device=gpu)
    block_table = table_full.to(gpu).contiguous()
    md = shim.build_decode_metadata(q_cu, kv_cu, slots, block_table, 1, max_blocks * bs,
                                    B * max_blocks * bs if hints else 0)
    md.plan_info.layer_id = 0
    kv_seq_lens = torch.ones(B, dtype=torch.int32, device=gpu)
    md.kv_seq_lens = kv_seq_lens  # persistent, refreshed in place before every replay
    md_plain = shim.build_decode_metadata(q_cu, kv_cu, slots, block_table, 1, max_blocks * bs, 0)
    md_plain.plan_info.layer_id = 0
    md_plain.kv_seq_lens = kv_seq_lens
    attn = shim.AttentionImpl(Hq, D, 1.0 / float(np.sqrt(D)), Hkv, -1)
    cache = shim.KVCache(k_cache, v_cache)

    def load_inputs(lens, seed):
        gg = torch.Generator().manual_seed(seed)
        qkv_src.copy_(torch.randn(B, (Hq + 2 * Hkv) * D, generator=gg).to(torch.bfloat16))
        lens_t = torch.tensor(lens, dtype=torch.int32)
        pos = lens_t - 1
        blk = table_full[torch.arange(B), (pos // bs).long()]
        slots.copy_((blk * bs + pos % bs).to(torch.int32))
        positions.copy_(pos.to(torch.int64))
        kv_seq_lens.copy_(lens_t)

    def step():
        qkv.copy_(qkv_src)  # forward_qkv rotates in place
        return attn.forward_qkv(md, positions, qkv, cos_sin, False, None, None, 0.0, cache)[0]

    load_inputs([100, 20, 4000, 1], 0)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_graph = step()
    for it, lens in enumerate(([100, 20, 4000, 1], [4100, 3, 17, 2048], [5, 5, 5, 5])):
        load_inputs(lens, 20 + it)
        k_before, v_before = k_cache.clone(), v_cache.clone()
        graph.replay()
        torch.cuda.synchronize()
        got, k_after = out_graph.clone(), k_cache.clone()
        k_cache.copy_(k_before)
        v_cache.copy_(v_before)
        eager = step()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), "replay %d differs from eager" % it
        assert torch.equal(k_after, k_cache)
        if hints:
            k_cache.copy_(k_before)
            v_cache.copy_(v_before)
            qkv.copy_(qkv_src)
            plain = attn.forward_qkv(md_plain, positions, qkv, cos_sin, False, None, None, 0.0, cache)[0]
            torch.cuda.synchronize()
            assert torch.allclose(got.float(), plain.float(), rtol=2 ** -7, atol=2e-3)
        _ = (k_cache[:8].float() @ torch.ones(D, 4, device=gpu)).sum().item()


@pytest.mark.gpu
def test_graphs_of_ascending_batch_sizes_keep_their_workspace(gpu, shim):
    """Two decode graphs captured one after the other, the second for a larger batch (one graph per
    batch-size bucket, xllm/core/runtime/cuda_graph_executor_impl.cpp:548-601): the workspace of a
    stream is allocated once at a fixed capacity and never moved, so the first graph still replays
    correctly after the second was captured and run — split sequences, i.e. plan, partials and counters
    all live in that workspace.  A step that needs more than the capacity is refused, not grown."""
    print("case shim graph buckets", flush=True)
    from tests.helpers import Case

    cap = shim.decode_workspace_capacity()
    assert cap == 128 << 20
    small = Case(2, 32, 8, 128, 16, [9000, 5000], seed=71)
    large = Case(24, 32, 8, 128, 16, [3000 + 100 * i for i in range(24)], seed=72)

    def run(case, out):
        shim.batch_decode(case.q.view(case.B, 1, case.Hq, case.D), case.k_cache, out.view(case.B, 1, case.Hq, case.D),
                          case.block_table, case.seq_lens, case.v_cache, None, None, None, 0, -1, case.scale, False, -1)

    side = torch.cuda.Stream()
    outs, graphs, eager = {}, {}, {}
    for name, case in (("small", small), ("large", large)):
        eager[name] = torch.empty_like(case.q)
        run(case, eager[name])
        torch.cuda.synchronize()
        outs[name] = torch.zeros_like(case.q)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            run(case, outs[name])  # first decode on the capture stream: its workspace is created here, before capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        ptr = shim.decode_workspace_ptr("cuda:0", side.cuda_stream)
        graphs[name] = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graphs[name], stream=side):
            run(case, outs[name])
        assert shim.decode_workspace_ptr("cuda:0", side.cuda_stream) == ptr  # not moved by a capture
        assert ptr != shim.decode_workspace_ptr("cuda:0", torch.cuda.current_stream().cuda_stream)  # one per stream
    for round_ in range(3):
        for name in ("large", "small", "small", "large"):
            outs[name].zero_()
            graphs[name].replay()
            torch.cuda.synchronize()
            assert torch.equal(outs[name], eager[name]), (round_, name)
        # eager work of the program's own between the replays
        _ = (small.k_cache[:8].float() @ torch.ones(128, 4, device=gpu)).sum().item()
    # a step beyond the capacity of its stream's buffer is refused, not grown: a fresh stream gets a
    # 1 MiB buffer here, too small for the partials of any split
    shim.set_decode_workspace_bytes(1 << 20)
    try:
        tiny = torch.cuda.Stream()
        tiny.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(tiny):
            with pytest.raises(RuntimeError, match="set_decode_workspace_bytes"):
                run(small, torch.empty_like(small.q))
    finally:
        shim.set_decode_workspace_bytes(cap)
    torch.cuda.synchronize()


@pytest.mark.gpu
@pytest.mark.parametrize("kv,n", [("bf16", 1), ("int8", 4), ("fp8", 8)])
def test_schedule_built_at_layer_zero_serves_every_layer(gpu, shim, kv, n):
    """The layer loop of a model (xllm/models/llm/llm_model_base.h:115) sets plan_info.layer_id before
    each layer; layer 0 builds the step's split-KV schedule and the later layers run on it
    (xllm/core/layers/cuda/flashinfer_planinfo.cpp:252-253).  Four layers with their own caches, a batch
    small enough to be split: every layer's output equals the one a call that plans for itself gives,
    bit for bit; an unset layer_id and a later layer with other inputs are refused."""
    from tests.helpers import Case

    print("case shim plan once per step", kv, n, flush=True)
    Hq, Hkv, D, bs = 32, 8, 128, 16
    lens = [9000, 700, 4100]
    layers = [Case(3, Hq, Hkv, D, bs, lens, n=n, kv=kv, seed=70, value_seed=70 + i) for i in range(4)]
    c0 = layers[0]
    q_cu = torch.arange(0, 3 * n + 1, n, dtype=torch.int32, device=gpu)
    kv_cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=gpu)
    slots = torch.zeros(3 * n, dtype=torch.int32, device=gpu)
    md = shim.build_decode_metadata(q_cu, kv_cu, slots, c0.block_table, n, max(lens), 0)

    def attend(c, layer_id):
        md.plan_info.layer_id = layer_id
        q4 = c.q.view(3, n, Hq, D)
        out = torch.full_like(q4, float("nan"))
        shim.batch_decode(q4, c.k_cache, out, md.block_table, md.kv_seq_lens, c.v_cache, None, c.k_scale, c.v_scale,
                          0, -1, c.scale, False, 8 if c.k_scale is not None else -1, plan_info=md.plan_info)
        torch.cuda.synchronize()
        return out

    with pytest.raises(RuntimeError, match="layer_id"):
        attend(c0, -1)
    shared = [attend(c, i) for i, c in enumerate(layers)]
    alone = [attend(c, 0) for c in layers]
    for i, (a, b, c) in enumerate(zip(shared, alone, layers)):
        assert not torch.isnan(a.float()).any()
        assert torch.equal(a, b), "layer %d differs from a call that plans for itself" % i
        ref, _ = c.oracle()
        assert float(np.abs(a.float().cpu().numpy().reshape(ref.shape) - ref).max()) <= c.tol
    # a later layer that presents another block table than layer 0's
    attend(c0, 0)
    other = md.block_table
    md.block_table = other.clone()
    with pytest.raises(RuntimeError, match="layer 0"):
        attend(c0, 1)
    md.block_table = other
    # ... or that comes after one of the library's switches was toggled (they shape the work items), or with a cache
    # in another layout
    from xllm_wxh_amd import ops

    attend(c0, 0)
    with ops.option("separate_merge", 1):
        with pytest.raises(RuntimeError, match="layer 0"):
            attend(c0, 1)
    attend(c0, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("kv,n", [("bf16", 1), ("fp8", 2)])
def test_plan_info_host_plan_eager_and_under_a_graph(gpu, shim, kv, n):
    """PlanInfo.kv_lens_host (the engine's kv_seq_lens_vec): layer 0 makes the step's schedule on the host
    (xllm_hip_paged_decode_plan_host) and the later layers run on it; PlanInfo.host_plan alone fixes the kernel and
    its work items by the sizes, so that two layers captured in a graph — layer 0's device-side plan with them —
    serve a replay on other lengths.  Against the oracle."""
    from oracle import paged_kv_oracle as orc
    from tests.helpers import Case

    print("case shim host plan", kv, n, flush=True)
    B, Hq, Hkv, D, bs = 6, 32, 8, 128, 16
    cap = np.full(B, 9000, np.int32)
    layers = [Case(B, Hq, Hkv, D, bs, cap, n=n, kv=kv, seed=80, value_seed=80 + i) for i in range(2)]
    c0 = layers[0]
    seq_lens = c0.seq_lens.clone()
    outs = [torch.zeros_like(c.q.view(B, n, Hq, D)) for c in layers]
    info = shim.PlanInfo()

    def forward():
        for layer_id, (c, out) in enumerate(zip(layers, outs)):
            info.layer_id = layer_id
            shim.batch_decode(c.q.view(B, n, Hq, D), c.k_cache, out, c0.block_table, seq_lens, c.v_cache, None, c.k_scale,
                              c.v_scale, 0, -1, c.scale, False, 8 if c.k_scale is not None else -1, plan_info=info)

    def check(lens):
        torch.cuda.synchronize()
        for c, out in zip(layers, outs):
            ref, _ = orc.paged_decode(c.q_ref, c.k_ref, c.v_ref, c0.table, lens, c.scale, q_per_seq=n)
            assert float(np.abs(out.float().cpu().numpy().reshape(ref.shape) - ref).max()) <= c.tol

    lens = np.array([9000, 17, 4100, 800, 1, 2500], np.int32)
    seq_lens.copy_(torch.from_numpy(lens))
    info.kv_lens_host = lens.tolist()
    forward()
    check(lens)
    # captured: sizes alone decide the kernels, layer 0's plan kernel is part of the graph
    info.kv_lens_host = []
    info.host_plan = True
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        forward()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        forward()
    for lens in (np.array([300, 9000, 9000, 64, 5000, 33], np.int32), np.array([8000, 1, 2, 3, 4, 9000], np.int32)):
        seq_lens.copy_(torch.from_numpy(lens))
        for out in outs:
            out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        check(lens)
