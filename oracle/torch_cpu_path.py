"""torch-CPU restatement of the decode path, used as the timed CPU baseline and as a fast checker
for inputs too large for the numpy oracle.  TEST INFRASTRUCTURE ONLY (same rule as
paged_kv_oracle.py: never imported by the product).

The reference has no CPU implementation of paged decode; the arithmetic below is the one its eager
attention uses (xllm/core/layers/cuda/flashinfer_attention.cpp:61-88: GQA head map h -> h / g,
scores = Q K^T * scale by bmm in fp32, softmax in fp32, then attn @ V), applied per sequence after a
gather through the block table (xllm/core/kernels/mlu/mlu_ops_api.h:126-145 contract), and the KV
write is the index math of xllm/core/kernels/cuda/reshape_paged_cache.cu:35-57 by advanced indexing.
Pinned against paged_kv_oracle.paged_decode in tests/test_oracle_attention.py.
"""
import torch


def reshape_paged_cache(slot_ids, keys, values, k_cache_hnd, v_cache_hnd):
    """k_cache_hnd/v_cache_hnd: [blocks, Hkv, bs, D] (any strides)."""
    bs = k_cache_hnd.size(2)
    slot_ids = slot_ids.long()
    blk, off = slot_ids // bs, slot_ids % bs
    k_cache_hnd[blk, :, off, :] = keys
    v_cache_hnd[blk, :, off, :] = values


def dequantize(cache, scale):
    """(float)q * scale; cache [.., D] int8 or float8_e4m3fn, scale [..] fp32."""
    return cache.float() * scale.unsqueeze(-1)


def paged_decode(q, k_cache_hnd, v_cache_hnd, block_table, seq_lens, scale, q_per_seq=1, k_scale=None,
                 v_scale=None):
    """q [B*n, Hq, D]; caches [blocks, Hkv, bs, D]; returns fp32 [B*n, Hq, D]."""
    T, Hq, D = q.shape
    Hkv, bs = k_cache_hnd.size(1), k_cache_hnd.size(2)
    g = Hq // Hkv
    n = q_per_seq
    B = T // n
    out = torch.zeros(T, Hq, D, dtype=torch.float32)
    qf = q.float()
    for b in range(B):
        L = int(seq_lens[b])
        if L <= 0:
            continue
        nb = (L + bs - 1) // bs
        ids = block_table[b, :nb].long()
        K = k_cache_hnd.index_select(0, ids)  # [nb, Hkv, bs, D]
        V = v_cache_hnd.index_select(0, ids)
        if k_scale is not None:
            K = dequantize(K, k_scale.index_select(0, ids))
            V = dequantize(V, v_scale.index_select(0, ids))
        K = K.float().permute(1, 0, 2, 3).reshape(Hkv, nb * bs, D)[:, :L]
        V = V.float().permute(1, 0, 2, 3).reshape(Hkv, nb * bs, D)[:, :L]
        # rows of kv head k: (draft token j, head k*g + r)
        qb = qf[b * n:(b + 1) * n].view(n, Hkv, g, D).permute(1, 0, 2, 3).reshape(Hkv, n * g, D)
        scores = torch.bmm(qb, K.transpose(1, 2)) * scale  # [Hkv, n*g, L]
        if n > 1:
            t = torch.arange(L)
            lim = L - (n - 1 - torch.arange(n))
            vis = (t[None, :] < lim[:, None]).repeat_interleave(g, dim=0)  # [n*g, L]
            scores = scores.masked_fill(~vis[None], float("-inf"))
        attn = torch.softmax(scores, dim=-1)
        o = torch.bmm(attn, V)  # [Hkv, n*g, D]
        out[b * n:(b + 1) * n] = o.view(Hkv, n, g, D).permute(1, 0, 2, 3).reshape(n, Hq, D)
    return out
