"""Known answer of the reference for the int8 paged decode, on the GPU: the HIP operators, placed in
the reference's Qwen2 attention module with the reference's seeded inputs, must reproduce the output
statistics of Qwen2AttentionTest.QuantizedKVCacheDecodeTest
(xllm/core/layers/common/tests/qwen2_attention_tests.cpp:500-578) and the oracle's attention output.
Two routes: the operators over the C ABI (rotary embedding + quantising write in one launch, then
the decode), and the C++ AttentionImpl twin."""
import os

import numpy as np
import pytest
import torch

import qwen2_int8_decode_case as case
from xllm_wxh_amd import build as xbuild
from xllm_wxh_amd import ops


def check(attn_out, fixed_w, ref_out):
    g = case.golden()
    stats = case.stats(case.output_projection(fixed_w, attn_out.reshape(case.BATCH, -1)))
    ok = [case.within(s, g[name], g["rtol"], g["atol"])
          for s, name in zip(stats, ("expected_min", "expected_max", "expected_sum"))]
    assert ok == [True, True, True], stats
    # against the oracle: value rows are int8-sized (up to 190), so 5e-2 absolute is 3e-4 relative
    err = float(np.abs(attn_out.float().cpu().numpy().reshape(ref_out.shape) - ref_out).max())
    scale = float(np.abs(ref_out).max())
    assert err <= 2.0 ** -8 * scale, (err, scale)  # one bf16 rounding of the output


@pytest.fixture(scope="module")
def fixed():
    w = case.weights()
    cos_sin = case.cos_sin_table()
    qkv = case.qkv_projection(w)
    table, slots, lens = case.metadata()
    ref_out, ref_rot = case.oracle_attend(qkv, cos_sin, table, slots, lens, *case.caches())
    return {"w": w, "cos_sin": cos_sin, "qkv": qkv, "meta": (table, slots, lens), "ref_out": ref_out,
            "ref_rot": ref_rot}


@pytest.mark.gpu
def test_hip_operators_reproduce_the_reference_known_answer(gpu, fixed):
    print("case qwen2 int8 decode known answer: C ABI", flush=True)
    table, slots, lens = fixed["meta"]
    k, v, ks, vs = (torch.from_numpy(a).to(gpu) for a in case.caches())
    qkv = fixed["qkv"].to(gpu).clone()
    pos = torch.full((case.BATCH,), case.SEQ_LEN, dtype=torch.int64, device=gpu)
    dev = lambda a: torch.from_numpy(a).to(gpu)
    ops.rope_kv_write(qkv, case.N_HEADS, case.N_KV_HEADS, case.HEAD_DIM, fixed["cos_sin"].to(gpu), pos, k, v,
                      dev(slots), k_cache_scale=ks, v_cache_scale=vs)
    q = qkv[:, :case.Q_SIZE].view(case.BATCH, case.N_HEADS, case.HEAD_DIM)
    out = torch.empty(case.BATCH, case.N_HEADS, case.HEAD_DIM, dtype=torch.bfloat16, device=gpu)
    ops.batch_decode(q, k, out, dev(table), dev(lens), v, k_cache_quant_scale=ks, v_cache_quant_scale=vs,
                     scale=float(np.sqrt(1.0 / case.HEAD_DIM)), kv_cache_quant_bit_size=8)
    torch.cuda.synchronize()
    assert ops.decode_variant(q, k, v, dev(table), dev(lens), ks, vs) == "mfma_d128"
    # the rotation is the oracle's to the last bit or the one next to it
    got, want = qkv.float().cpu().numpy(), fixed["ref_rot"]
    assert np.all(np.abs(got - want) <= 2.0 ** -7 * np.abs(want))
    check(out, fixed["w"], fixed["ref_out"])
    # the generic kernel, on the same inputs
    with ops.option("force_generic"):
        out2 = torch.empty_like(out)
        ops.batch_decode(q, k, out2, dev(table), dev(lens), v, k_cache_quant_scale=ks, v_cache_quant_scale=vs,
                         scale=float(np.sqrt(1.0 / case.HEAD_DIM)), kv_cache_quant_bit_size=8)
        torch.cuda.synchronize()
    check(out2, fixed["w"], fixed["ref_out"])


@pytest.mark.gpu
def test_attention_impl_reproduces_the_reference_known_answer(gpu, fixed):
    print("case qwen2 int8 decode known answer: AttentionImpl", flush=True)
    if not os.path.exists(xbuild.TORCH_SHIM_PATH):
        pytest.fail("the libtorch host side is not built")
    from xllm_wxh_amd import _xllm_hip_torch as shim

    table, slots, lens = fixed["meta"]
    k, v, ks, vs = (torch.from_numpy(a).to(gpu) for a in case.caches())
    i32 = lambda a: torch.tensor(np.asarray(a), dtype=torch.int32, device=gpu)
    kv_len = case.SEQ_LEN + 1
    md = shim.build_decode_metadata(i32(np.arange(case.BATCH + 1)), i32(np.arange(case.BATCH + 1) * kv_len),
                                    i32(slots), i32(table), 1, kv_len, case.BATCH * kv_len)
    md.plan_info.layer_id = 0
    attn = shim.AttentionImpl(case.N_HEADS, case.HEAD_DIM, float(np.sqrt(1.0 / case.HEAD_DIM)), case.N_KV_HEADS, -1)
    cache = shim.KVCache(k, v, ks, vs)
    qkv = fixed["qkv"].to(gpu).clone()
    pos = torch.full((case.BATCH,), case.SEQ_LEN, dtype=torch.int32, device=gpu)
    out, _ = attn.forward_qkv(md, pos, qkv, fixed["cos_sin"].to(gpu), False, None, None, 1e-6, cache)
    torch.cuda.synchronize()
    check(out, fixed["w"], fixed["ref_out"])
