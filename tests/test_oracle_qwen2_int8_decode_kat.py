"""Known answer of the reference for the int8 paged decode, on the CPU: the numpy oracle, placed in
the reference's Qwen2 attention module with the reference's seeded inputs, must reproduce the output
statistics the reference's own test expects (Qwen2AttentionTest.QuantizedKVCacheDecodeTest,
xllm/core/layers/common/tests/qwen2_attention_tests.cpp:500-578: min -282, max 67, sum -387352.6875,
rtol 0.01, atol 1).  The scores of this case are large (int8 keys times queries near 5.7), so every
softmax is one-hot: the statistics are decided by which cached token each (sequence, head) picks and
by that token's dequantised value row — i.e. by the seeded tensors, the rotary embedding, the block
table walk, the q head -> kv head map and the placement of the per-token-per-head scales.  The
mutants below show which mistakes the known answer catches; it does not see the softmax scale or
the quantising write of the new token (that token never wins), which other tests pin."""
import numpy as np
import pytest
import torch

import qwen2_int8_decode_case as case
from oracle import paged_kv_oracle as orc


@pytest.fixture(scope="module")
def fixed():
    w = case.weights()
    return {"w": w, "cos_sin": case.cos_sin_table(), "qkv": case.qkv_projection(w), "meta": case.metadata()}


def run(fixed, interleaved=False, position=case.SEQ_LEN, table_shift=0, swap_scales=False, head_perm=None,
        unit_k_scale=False, unit_v_scale=False):
    table, slots, lens = fixed["meta"]
    k, v, ks, vs = case.caches()
    if unit_k_scale:
        ks = np.ones_like(ks)
    if unit_v_scale:
        vs = np.ones_like(vs)
    if swap_scales:
        ks, vs = vs, ks
    pos = np.full(case.BATCH, position, np.int64)
    rot = orc.fused_qk_norm_rope(fixed["qkv"].float().numpy(), case.N_HEADS, case.N_KV_HEADS, case.N_KV_HEADS,
                                 case.HEAD_DIM, 0.0, None, None, fixed["cos_sin"].float().numpy(), interleaved, pos,
                                 "bf16")
    q = rot[:, :case.Q_SIZE].reshape(case.BATCH, case.N_HEADS, case.HEAD_DIM)
    if head_perm is not None:
        q = q[:, head_perm]
    new_k = rot[:, case.Q_SIZE:case.Q_SIZE + case.KV_SIZE].reshape(case.BATCH, case.N_KV_HEADS, -1).astype(np.float32)
    new_v = rot[:, case.Q_SIZE + case.KV_SIZE:].reshape(case.BATCH, case.N_KV_HEADS, -1).astype(np.float32)
    orc.quant_to_paged_cache(slots, new_k, new_v, k, v, ks, vs, "int8", "HND")
    out, _ = orc.paged_decode(q, k, v, table + table_shift, lens, float(np.sqrt(1.0 / case.HEAD_DIM)), k_scale=ks,
                              v_scale=vs, kind="int8")
    if head_perm is not None:
        out = out[:, np.argsort(head_perm)]
    o = case.output_projection(fixed["w"], torch.from_numpy(out.reshape(case.BATCH, -1)).to(torch.bfloat16))
    return case.stats(o)


def verdict(stats):
    g = case.golden()
    return [case.within(s, g[name], g["rtol"], g["atol"])
            for s, name in zip(stats, ("expected_min", "expected_max", "expected_sum"))]


def test_oracle_reproduces_the_reference_known_answer(fixed):
    stats = run(fixed)
    assert verdict(stats) == [True, True, True], stats
    # well inside the reference's tolerance: 0.1 % on the sum where 1 % is allowed
    assert abs(stats[2] - case.golden()["expected_sum"]) < 1e-3 * abs(case.golden()["expected_sum"]), stats


def test_softmaxes_of_the_case_are_one_hot(fixed):
    """What makes the statistics a test of indexing: every (sequence, head) puts its whole weight on one
    cached token, and never on the token written in this step."""
    table, slots, lens = fixed["meta"]
    out, rot = case.oracle_attend(fixed["qkv"], fixed["cos_sin"], table, slots, lens, *case.caches())
    k, v, ks, vs = case.caches()
    vals = (v.astype(np.float64) * vs[..., None])  # dequantised values [block, head, slot, d]
    g = case.N_HEADS // case.N_KV_HEADS
    for b in range(case.BATCH):
        rows = vals[table[b]].transpose(1, 0, 2, 3).reshape(case.N_KV_HEADS, -1, case.HEAD_DIM)[:, :case.SEQ_LEN]
        for h in range(case.N_HEADS):
            d = np.abs(rows[h // g] - out[b, h][None, :]).max(axis=1)
            assert d.min() < 0.5 and np.sort(d)[1] > 50.0, (b, h)  # value rows are int8-sized: one row is matched, the rest are far


@pytest.mark.parametrize("mutant", [
    dict(interleaved=True),                    # GPT-J pairing instead of NeoX
    dict(position=case.SEQ_LEN - 1),           # rotary position off by one
    dict(swap_scales=True),                    # K scales applied to V and the other way round
    dict(unit_k_scale=True),                   # K scales ignored
    dict(unit_v_scale=True),                   # V scales ignored
    dict(table_shift=1),                       # block table read one block off
    dict(head_perm=np.array([(h % 8) * 2 + h // 8 for h in range(16)])),  # kv head = h % Hkv instead of h / group
])
def test_known_answer_catches_plausible_mistakes(fixed, mutant):
    assert verdict(run(fixed, **mutant)) != [True, True, True], mutant
