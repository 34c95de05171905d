"""The reference's one numeric known answer that crosses the int8 paged decode: the fixture and inputs of
Qwen2AttentionTest.QuantizedKVCacheDecodeTest (xllm/core/layers/common/tests/qwen2_attention_tests.cpp:31-98,
500-578), rebuilt from their seeds.  Everything in it is deterministic: weights, hidden states, the
int8 caches and their scales come from test::seeded_tensor (FNV-1a of a name -> SplitMix64 stream,
xllm/core/layers/common/tests/tests_utils.cpp:159-272), block tables and slots from closed forms.

The module is Qwen2AttentionImpl::forward (xllm/core/layers/common/qwen2_attention.cpp:132-192):
qkv projection with bias -> NeoX rotary embedding at position 256 -> quantising KV write of the new
token -> int8 paged decode over 257 tokens -> output projection.  The steps around the path (the two
linear layers, the cos/sin table) are plain torch here; `attend` is the part under test and is
supplied by the caller: the numpy oracle on the CPU, the HIP operators on the GPU.
"""
import json
import os

import numpy as np
import torch

from oracle import paged_kv_oracle as orc

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qwen2_int8_decode_stats.json")

# model_args_ of the fixture (qwen2_attention_tests.cpp:36-45)
HIDDEN, N_HEADS, N_KV_HEADS, HEAD_DIM = 1024, 16, 8, 128
MAX_POS, ROPE_THETA = 2048, 1000000.0
# QuantizedKVCacheDecodeTest (:507-515)
BATCH, SEQ_LEN, BLOCK_NUM, BLOCK_SIZE = 4, 256, 100, 16
Q_SIZE, KV_SIZE = N_HEADS * HEAD_DIM, N_KV_HEADS * HEAD_DIM


def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def _seeded_bf16(key, shape):
    return torch.from_numpy(orc.seeded_tensor(key, shape, np.float32)).to(torch.bfloat16)


def weights():
    """InitTestWeights (:70-98): seeded bf16 in [0, 1) divided, in bf16, by sqrt(size(0)) held in bf16."""
    shapes = {
        "q_proj.weight": (Q_SIZE, HIDDEN), "k_proj.weight": (KV_SIZE, HIDDEN), "v_proj.weight": (KV_SIZE, HIDDEN),
        "q_proj.bias": (Q_SIZE,), "k_proj.bias": (KV_SIZE,), "v_proj.bias": (KV_SIZE,),
        "o_proj.weight": (HIDDEN, Q_SIZE),
    }
    w = {}
    for name, shape in shapes.items():
        t = _seeded_bf16("qwen2_attention_test." + name, shape)
        w[name] = t / torch.sqrt(torch.tensor(float(shape[0]), dtype=torch.bfloat16))
    return w


def cos_sin_table():
    """[MAX_POS, HEAD_DIM] bf16, cos of the 64 frequencies then sin: compute_inv_freq and
    create_cos_sin_tensor (xllm/core/layers/common/rotary_embedding_util.cpp:114-145, 303-310) in
    float, cast to the model dtype, reduced to the [cos_half, sin_half] form the kernels index
    (xllm/core/layers/common/rotary_embedding.cpp:44-49)."""
    slice_ = torch.arange(0, HEAD_DIM, 2, dtype=torch.float32)
    inv_freq = 1.0 / torch.pow(torch.tensor(ROPE_THETA, dtype=torch.float32), slice_ / float(HEAD_DIM))
    freqs = torch.einsum("i,j->ij", torch.arange(MAX_POS, dtype=torch.float32), inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], -1).to(torch.bfloat16)


def block_num_per_req(kv_len):
    return (kv_len + BLOCK_SIZE - 1) // BLOCK_SIZE + 1  # GetBlockNum (:100-103)


def metadata():
    """CreateAttentionMetadata(batch, seq_len + 1, false, seq_len + 1) (:144-196): every sequence has
    257 tokens, the new one in the last position; blocks b * per_req + i; slot b * per_req * 16 + 256."""
    kv_len = SEQ_LEN + 1
    per = block_num_per_req(kv_len)
    table = (np.arange(BATCH)[:, None] * per + np.arange(per)[None, :]).astype(np.int32)
    slots = (np.arange(BATCH) * per * BLOCK_SIZE + kv_len - 1).astype(np.int32)
    return table, slots, np.full(BATCH, kv_len, np.int32)


def caches():
    """int8 K/V [100, 8, 16, 128] straight from the seeds, scales 0.5 + seeded fp32 in [0, 1) (:518-543)."""
    shape = (BLOCK_NUM, N_KV_HEADS, BLOCK_SIZE, HEAD_DIM)
    k = orc.seeded_tensor("qwen2_quant_decode.k_cache", shape, np.int8)
    v = orc.seeded_tensor("qwen2_quant_decode.v_cache", shape, np.int8)
    ks = np.float32(0.5) + orc.seeded_tensor("qwen2_quant_decode.k_scale", shape[:3], np.float32)
    vs = np.float32(0.5) + orc.seeded_tensor("qwen2_quant_decode.v_scale", shape[:3], np.float32)
    return k, v, ks.astype(np.float32), vs.astype(np.float32)


def qkv_projection(w, device="cpu"):
    """hidden_states [4, 1024] bf16 -> fused qkv [4, 4096] bf16 (fp32 accumulation, one rounding)."""
    hidden = _seeded_bf16("qwen2_quant_decode.hidden_states", (BATCH, HIDDEN)).to(device)
    wqkv = torch.cat([w["q_proj.weight"], w["k_proj.weight"], w["v_proj.weight"]], 0).to(device)
    bias = torch.cat([w["q_proj.bias"], w["k_proj.bias"], w["v_proj.bias"]], 0).to(device)
    return (hidden.float() @ wqkv.float().t() + bias.float()).to(torch.bfloat16)


def output_projection(w, attn_out):
    """attention output [4, 2048] bf16 -> [4, 1024] bf16."""
    return (attn_out.float() @ w["o_proj.weight"].to(attn_out.device).float().t()).to(torch.bfloat16)


def stats(output):
    flat = output.flatten().float().cpu()
    return float(flat.min()), float(flat.max()), float(flat.sum())


def within(actual, expected, rtol, atol):
    return abs(actual - expected) <= atol + rtol * abs(expected)  # expect_tensor_stats (tests_utils.cpp:105-108)


def oracle_attend(qkv, cos_sin, table, slots, lens, k, v, ks, vs):
    """The path under test through the numpy oracle: rotary embedding, quantising write, decode.
    Returns the attention output [4, 16, 128] in float64 and the rotated qkv."""
    pos = np.full(BATCH, SEQ_LEN, np.int64)
    rot = orc.fused_qk_norm_rope(qkv.float().numpy(), N_HEADS, N_KV_HEADS, N_KV_HEADS, HEAD_DIM, 0.0, None, None,
                                 cos_sin.float().numpy(), False, pos, "bf16")
    q = rot[:, :Q_SIZE].reshape(BATCH, N_HEADS, HEAD_DIM)
    new_k = rot[:, Q_SIZE:Q_SIZE + KV_SIZE].reshape(BATCH, N_KV_HEADS, HEAD_DIM).astype(np.float32)
    new_v = rot[:, Q_SIZE + KV_SIZE:].reshape(BATCH, N_KV_HEADS, HEAD_DIM).astype(np.float32)
    orc.quant_to_paged_cache(slots, new_k, new_v, k, v, ks, vs, "int8", "HND")
    out, _ = orc.paged_decode(q, k, v, table, lens, float(np.sqrt(1.0 / HEAD_DIM)), k_scale=ks, v_scale=vs,
                              kind="int8")
    return out, rot
