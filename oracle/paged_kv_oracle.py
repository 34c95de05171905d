"""CPU oracle of xLLM's paged-KV decode path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module, and only as the checker or the timed CPU baseline; the product
(xllm_wxh_amd) never does.

Every function restates one piece of the reference (paths relative to the xLLM
tree); how each one is pinned is listed beside it:

  fnv1a64 / SplitMix64 / seeded_tensor   xllm/core/layers/common/tests/tests_utils.cpp:159-272
      pinned by the published FNV-1a and SplitMix64 test vectors and by the reference's own statistics of
      a seeded float32 tensor (layers/common/tests/deepseek_v2_decoder_layer_tests.cpp:1594-1599).
  kv_cache_slots                         xllm/core/framework/request/sequence_kv_state.cpp:120-134
  calc_slot_id / calc_kv_len             xllm/core/runtime/spec_input_builder.cpp:76-109
  build_paged_kv_csr / pad_block_tables  xllm/core/framework/batch/batch_input_builder.cpp:438-494,565-582
  attention_metadata_kv_seq_lens         xllm/core/layers/common/attention_metadata_builder.cpp:105
      pinned by the known answers of framework/batch/batch_test.cpp:154-204 and
      runtime/spec_input_builder_test.cpp:55-119 (tests/golden/index_math.json).
  reshape_paged_cache_loops              xllm/core/kernels/cuda/reshape_paged_cache.cu:35-57 (literal)
  reshape_paged_cache                    same, vectorised; pinned against the literal loops.
  paged_decode_loops / paged_decode      softmax(scale q.K^T) V with the GQA head map and fp32-softmax
      arithmetic of xllm/core/layers/cuda/flashinfer_attention.cpp:61-88 over the block_table /
      seq_lens contract of xllm/core/kernels/mlu/mlu_ops_api.h:126-145.  The attention arithmetic
      itself lives in FlashInfer v0.6.2 (docker/Dockerfile.cuda:16) and in the closed `tmo`
      library, neither of which is in the reference tree: pinned by mathematics (kv_len 1 gives the
      value row, identical keys give the mean of values, block-table permutation invariance,
      agreement with scipy/torch softmax, split-merge identity) and by the reference's invariant
      xllm/core/runtime/cuda_graph_executor_test.cpp:150-151.  The int8 decode (with seeded_tensor,
      the rotary embedding and the scale layout [block, head, slot]) is also pinned by the reference's
      one numeric known answer that crosses it: the output statistics of
      Qwen2AttentionTest.QuantizedKVCacheDecodeTest (xllm/core/layers/common/tests/qwen2_attention_tests.cpp:
      500-578), reproduced to 0.1 % of the sum where the reference allows 1 %
      (tests/test_oracle_qwen2_int8_decode_kat.py; its softmaxes are one-hot, so it pins the token
      and head indexing and the dequantisation, not the softmax arithmetic).  Absolute FlashInfer
      outputs and the low-order bits of tmo's: PARITY UNPINNED (tolerance only).
  paged_decode_ragged                    per-sequence query counts (chunked prefill, flashinfer_attention.cpp:224-284):
      one paged_decode call per sequence, so it inherits those pins.
  lse_combine                            xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73
  fused_qk_norm_rope / rope_pairs        xllm/core/kernels/cuda/fused_qknorm_rope.cu:70-262, rope.cu:26-52
      pinned by the torch formula the reference's own test checks its kernel against
      (xllm/core/kernels/cuda/fused_qknorm_rope_test.cpp:28-109, at that test's shapes and tolerances),
      by torch.nn.functional.rms_norm, by complex multiplication (x + iy) e^{i theta}, and by the
      identity at cos = 1, sin = 0.  The last bit of the float arithmetic of the CUDA kernels
      (summation order, fused multiply-adds) is PARITY UNPINNED: outputs are compared within one unit
      in the last place of the element type; the round-each-operation form without norm is exact.
  swap_blocks                            xllm/core/framework/kv_cache/kv_cache.cpp:104-125
  build_block_copy_groups / copy_blocks  xllm/core/framework/batch/batch_input_builder.cpp:691-720,
      xllm/models/llm/npu/llm_model_base.h:69-75; pinned by brute force on tiny caches (element
      loops), by the gather-before-scatter property on a chain a->b, b->c, and by the group arrays
      expanding back to the transfer list they came from.
  reshape_from_cache / dequant_from_paged_cache
      argument contract of xllm/core/kernels/param.h:160-215 and xllm/core/kernels/mlu/mlu_ops_api.h:56-101,
      call site xllm/core/layers/mlu/attention.cpp:179-214; the bodies live in the closed `tmo`
      library: PARITY UNPINNED beyond the documented contract.  Pinned by literal loops on tiny
      caches, by the round trips reshape_paged_cache -> reshape_from_cache = identity and
      quant_to_paged_cache -> dequant_from_paged_cache = dequantize(quantize(x)), and by agreement
      with gather_sequence (the gather the attention oracle itself uses).
  quantize_per_token_head / quant_to_paged_cache
      scale and saturation conventions of xllm/core/kernels/cuda/fp8_quant_utils.cuh:38-53,112-131;
      the int8 rounding of `tmo::quant_to_paged_cache` (xllm/core/kernels/mlu/attention.cpp:50-59) is
      closed source: PARITY UNPINNED, round-half-even chosen.  float_to_e4m3fn is pinned against
      torch's float8_e4m3fn conversion over every finite fp8 value and all midpoints.
"""
import math

import numpy as np

# ---------------------------------------------------------------------------------------
# seeded_tensor (tests_utils.cpp:159-272)
# ---------------------------------------------------------------------------------------

_MASK64 = (1 << 64) - 1


def fnv1a64(s):
    h = 0xCBF29CE484222325
    for c in s.encode("utf-8"):
        h ^= c
        h = (h * 0x100000001B3) & _MASK64
    return h


class SplitMix64:
    def __init__(self, seed):
        self.state = seed & _MASK64

    def next_u64(self):
        self.state = (self.state + 0x9E3779B97F4A7C15) & _MASK64
        z = self.state
        z ^= z >> 30
        z = (z * 0xBF58476D1CE4E5B9) & _MASK64
        z ^= z >> 27
        z = (z * 0x94D049BB133111EB) & _MASK64
        z ^= z >> 31
        return z


def splitmix64_stream(seed, n):
    """n outputs of SplitMix64(seed) as a uint64 array (vectorised; equals repeated next_u64)."""
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z ^= z >> np.uint64(30)
        z *= np.uint64(0xBF58476D1CE4E5B9)
        z ^= z >> np.uint64(27)
        z *= np.uint64(0x94D049BB133111EB)
        z ^= z >> np.uint64(31)
    return z


def seeded_tensor(key, shape, dtype):
    """numpy twin of test::seeded_tensor: floats = (u >> 11) * 2^-53 in [0, 1) cast to dtype,
    bool = u & 1, integers = min + u % span."""
    n = int(np.prod(shape)) if len(shape) else 1
    u = splitmix64_stream(fnv1a64(key), n)
    dt = np.dtype(dtype)
    if dt.kind == "f":
        vals = (u >> np.uint64(11)).astype(np.float64) * (1.0 / float(1 << 53))
        return vals.astype(dt).reshape(shape)
    if dt.kind == "b":
        return (u & np.uint64(1)).astype(np.bool_).reshape(shape)
    if dt.kind in "iu":
        info = np.iinfo(dt)
        span = int(info.max) - int(info.min) + 1
        if span >= (1 << 64):
            rem = u
        else:
            rem = u % np.uint64(span)
        vals = (rem.astype(object) + int(info.min)) if dt.itemsize == 8 else (rem.astype(np.int64) + int(info.min))
        return np.array(vals, dtype=dt).reshape(shape)
    raise ValueError("unsupported dtype for seeded_tensor: %s" % dt)


# ---------------------------------------------------------------------------------------
# host index math
# ---------------------------------------------------------------------------------------


def kv_cache_slots(block_ids, block_size, pos_start, pos_end):
    """KVCacheState::kv_cache_slots: slot = block_id * block_size + pos % block_size."""
    if len(block_ids) == 0:
        raise ValueError("no cache blocks available")
    return [int(block_ids[i // block_size]) * block_size + i % block_size for i in range(pos_start, pos_end)]


def calc_slot_id(position, block_table_row, block_size):
    if block_size <= 0:
        raise ValueError("invalid block_size=%d" % block_size)
    if position < 0:
        raise ValueError("invalid position=%d" % position)
    block_idx = position // block_size
    if block_idx >= len(block_table_row):
        raise IndexError("block table index out of range, block_idx=%d" % block_idx)
    block_id = int(block_table_row[block_idx])
    if block_id < 0:
        raise ValueError("invalid block_id=%d" % block_id)
    return block_id * block_size + position % block_size


def calc_kv_len(kv_seq_lens_cumulative, seq_id, offset):
    """Cumulative layout (every backend except NPU): len = cu[seq+1] - cu[seq] + offset."""
    if seq_id < 0 or seq_id + 1 >= len(kv_seq_lens_cumulative):
        raise IndexError("seq_id out of range for cumulative layout")
    return int(kv_seq_lens_cumulative[seq_id + 1]) - int(kv_seq_lens_cumulative[seq_id]) + offset


def build_paged_kv_csr(block_lists, seq_lens, block_size):
    """BatchInputBuilder::setup_kv_cache_info: (paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len)."""
    indptr, indices, last = [0], [], []
    for blocks, seq_len in zip(block_lists, seq_lens):
        indices.extend(int(b) for b in blocks)
        indptr.append(indptr[-1] + len(blocks))
        last.append(block_size if seq_len % block_size == 0 else seq_len % block_size)
    return (np.array(indptr, np.int32), np.array(indices, np.int32), np.array(last, np.int32))


def pad_block_tables(block_lists, pad_value=0):
    """util::pad_2d_vector(block_tables_vec, 0) + create_2d_tensor."""
    width = max((len(b) for b in block_lists), default=0)
    out = np.full((len(block_lists), width), pad_value, np.int32)
    for i, b in enumerate(block_lists):
        out[i, : len(b)] = b
    return out


def attention_metadata_kv_seq_lens(kv_seq_lens_cumulative):
    """attn_metadata.kv_seq_lens = torch::diff(params.kv_seq_lens)."""
    return np.diff(np.asarray(kv_seq_lens_cumulative, np.int64)).astype(np.int32)


def expand_decode_rows(positions, kv_seq_lens_cumulative, block_tables, block_size, offsets):
    """append_decode_row over every sequence and every position offset in `offsets`:
    returns (positions, slots, per-row kv lens, duplicated block-table rows)."""
    out_pos, out_slots, out_kv, out_tables = [], [], [], []
    for seq_id in range(len(positions)):
        for off in offsets:
            new_pos = int(positions[seq_id]) + off
            out_pos.append(new_pos)
            out_slots.append(calc_slot_id(new_pos, block_tables[seq_id], block_size))
            out_kv.append(calc_kv_len(kv_seq_lens_cumulative, seq_id, off))
            out_tables.append(list(block_tables[seq_id]))
    return out_pos, out_slots, out_kv, out_tables


# ---------------------------------------------------------------------------------------
# KV write
# ---------------------------------------------------------------------------------------


def _hnd_view(cache, layout):
    """Logical [blocks, heads, slots, dim] view of a cache stored as HND or NHD."""
    if layout == "HND":
        return cache
    if layout == "NHD":
        return cache.transpose(0, 2, 1, 3)
    raise ValueError(layout)


def reshape_paged_cache_loops(slot_ids, keys, values, key_cache, value_cache, layout="NHD"):
    """Literal restatement of reshape_paged_cache_kernel: one token at a time, one element at a time."""
    kc, vc = _hnd_view(key_cache, layout), _hnd_view(value_cache, layout)
    n_tokens, n_kv_heads, head_dim = keys.shape
    block_size = kc.shape[2]
    for bid in range(n_tokens):
        slot_id = int(slot_ids[bid])
        block_idx = slot_id // block_size
        block_offset = slot_id % block_size
        for i in range(n_kv_heads * head_dim):
            head_idx = i // head_dim
            head_offset = i % head_dim
            kc[block_idx, head_idx, block_offset, head_offset] = keys[bid, head_idx, head_offset]
            vc[block_idx, head_idx, block_offset, head_offset] = values[bid, head_idx, head_offset]


def reshape_paged_cache(slot_ids, keys, values, key_cache, value_cache, layout="NHD"):
    """Vectorised form; for duplicate slots the last token in order wins (numpy assignment order)."""
    kc = _hnd_view(key_cache, layout)
    block_size = kc.shape[2]
    slot_ids = np.asarray(slot_ids, np.int64)
    blk, off = slot_ids // block_size, slot_ids % block_size
    kc[blk, :, off, :] = keys
    if values is not None:
        _hnd_view(value_cache, layout)[blk, :, off, :] = values


# ---- per-head RMSNorm + rotary embedding -------------------------------------------------


def round_to_dtype(x, kind):
    """float64/float32 array -> the nearest value of kind ('bf16' | 'fp16' | 'fp32'), round half to
    even, returned as float64."""
    x = np.asarray(x, dtype=np.float64)
    if kind == "fp32":
        return x.astype(np.float32).astype(np.float64)
    if kind == "fp16":
        return x.astype(np.float16).astype(np.float64)
    f = x.astype(np.float32)  # double rounding is harmless here: inputs are products of short mantissas
    u = f.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def rope_pairs(rotary_dim, interleaved):
    """Index arrays (x_idx, y_idx) of the rotated pairs, frequency j = position in the arrays:
    NeoX (j, j + rotary_dim/2), GPT-J (2j, 2j + 1) — xllm/core/kernels/cuda/rope.cu:33-46."""
    half = rotary_dim // 2
    j = np.arange(half)
    return (2 * j, 2 * j + 1) if interleaved else (j, j + half)


def fused_qk_norm_rope(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight,
                       cos_sin_cache, interleaved, position_ids, kind, round_each_op=False):
    """Restatement of fused_qknorm_rope_kernel (xllm/core/kernels/cuda/fused_qknorm_rope.cu:70-262): for
    every q and k head x <- x * rsqrt(mean(x^2) + eps) * weight (skipped when the weights are None),
    then x' = x cos - y sin, y' = y cos + x sin on the pairs of rope_pairs with cos = cache[pos, j],
    sin = cache[pos, rotary_dim/2 + j]; elements beyond rotary_dim and the v heads pass through; one
    rounding to `kind` at the end.  round_each_op=True rounds after the norm, after each product and
    after the sum instead: arithmetic on scalar_t operands as in rope.cu:49-52.  Computed in float64;
    qkv is [tokens, (Hq+Hk+Hv)*head_dim] holding values of `kind`.  Returns a new float64 array."""
    out = np.array(qkv, dtype=np.float64, copy=True)
    T = out.shape[0]
    R = cos_sin_cache.shape[1]
    half = R // 2
    xi, yi = rope_pairs(R, interleaved)
    pos = np.asarray(position_ids, dtype=np.int64)
    cos = np.asarray(cos_sin_cache, dtype=np.float64)[pos][:, :half]
    sin = np.asarray(cos_sin_cache, dtype=np.float64)[pos][:, half:R]
    rd = (lambda a: round_to_dtype(a, kind)) if round_each_op else (lambda a: a)
    if round_each_op:
        cos, sin = rd(cos), rd(sin)
    for hh in range(num_heads_q + num_heads_k):
        w = q_weight if hh < num_heads_q else k_weight
        x = out[:, hh * head_dim:(hh + 1) * head_dim]
        if w is not None:
            rms = 1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps)
            x = rd(x * (rms * np.asarray(w, dtype=np.float64)[None, :]))
        a, b = x[:, xi], x[:, yi]
        na = rd(rd(a * cos) - rd(b * sin))
        nb = rd(rd(b * cos) + rd(a * sin))
        x = x.copy()
        x[:, xi], x[:, yi] = na, nb
        out[:, hh * head_dim:(hh + 1) * head_dim] = round_to_dtype(x, kind)
    return out


# ---- whole-block movement ----------------------------------------------------------------


def swap_blocks(arrays, src, dst):
    """KVCache::swap_blocks (xllm/core/framework/kv_cache/kv_cache.cpp:104-125): for every array whose
    first dimension is the block (key cache, value cache, and the scale tensors when defined),
    `selected = index_select(array, 0, src)` and then `array.index_copy_(0, dst, selected)` — all
    sources are read before any destination is written.  In place; `arrays` is an iterable."""
    src = np.asarray(src, dtype=np.int64)
    dst = np.asarray(dst, dtype=np.int64)
    for a in arrays:
        if a is None:
            continue
        selected = a[src].copy()
        a[dst] = selected


def build_block_copy_groups(pairs):
    """The (src_block_indices, dst_block_indices, cum_sum) arrays the batch builder derives from
    its (src, dst) transfer list (xllm/core/framework/batch/batch_input_builder.cpp:691-720): pairs
    sorted by source, one source entry per distinct source, cum_sum[g] = number of destinations up to
    and including group g.  (std::sort there is not stable; this port keeps ties in input order.)"""
    pairs = sorted(pairs, key=lambda sd: sd[0])
    if not pairs:
        return [], [], []
    src_indices, dst_indices, cum_sum = [pairs[0][0]], [pairs[0][1]], []
    current = pairs[0][0]
    for i in range(1, len(pairs)):
        dst_indices.append(pairs[i][1])
        if pairs[i][0] != current:
            src_indices.append(pairs[i][0])
            cum_sum.append(i)
            current = pairs[i][0]
    cum_sum.append(len(pairs))
    return src_indices, dst_indices, cum_sum


def copy_blocks(arrays, src_block_indices, dst_block_indices, cum_sum):
    """What the block-copy step does with those arrays (call site
    xllm/models/llm/npu/llm_model_base.h:69-75): block src_block_indices[g] is copied to every block
    in dst_block_indices[cum_sum[g-1]:cum_sum[g]].  Literal loops."""
    for a in arrays:
        if a is None:
            continue
        begin = 0
        for g, src in enumerate(src_block_indices):
            for i in range(begin, cum_sum[g]):
                a[dst_block_indices[i]] = a[src]
            begin = cum_sum[g]


# ---- sequences read back out of the cache -------------------------------------------------


def reshape_from_cache(key_cache, value_cache, context_lengths, block_tables, context_seq_offset=None,
                       cache_seq_offset=None, total_rows=None, layout="HND", fill=0):
    """Paged mode of xllm::kernel::reshape_from_cache (xllm/core/kernels/param.h:160-201,
    xllm/core/kernels/mlu/mlu_ops_api.h:56-64): token t of sequence b, stored at cache position
    cache_seq_offset[b] + t (block block_tables[b][pos // bs], slot pos % bs), goes to output row
    context_seq_offset[b] + t; without context_seq_offset the sequences are packed in order.
    Returns (key [rows, H, D], value or None); rows no sequence covers hold `fill`.  Literal loops."""
    kc = _hnd_view(key_cache, layout)
    vc = _hnd_view(value_cache, layout) if value_cache is not None else None
    bs = kc.shape[2]
    lens = [int(x) for x in context_lengths]
    if context_seq_offset is None:
        context_seq_offset = np.concatenate([[0], np.cumsum(lens)[:-1]]) if lens else []
    if total_rows is None:
        total_rows = max([int(o) + n for o, n in zip(context_seq_offset, lens)], default=0)
    key = np.full((total_rows, kc.shape[1], kc.shape[3]), fill, dtype=kc.dtype)
    value = np.full((total_rows, vc.shape[1], vc.shape[3]), fill, dtype=vc.dtype) if vc is not None else None
    for b, n in enumerate(lens):
        start = int(cache_seq_offset[b]) if cache_seq_offset is not None else 0
        for t in range(n):
            pos = start + t
            blk = int(block_tables[b][pos // bs])
            key[int(context_seq_offset[b]) + t] = kc[blk, :, pos % bs, :]
            if vc is not None:
                value[int(context_seq_offset[b]) + t] = vc[blk, :, pos % bs, :]
    return key, value


def dequant_from_paged_cache(key_cache, value_cache, key_scale, value_scale, context_lengths, block_tables, kind,
                             out_kind="fp32", quant_mode=1, context_seq_offset=None, total_rows=None):
    """xllm::kernel::dequant_from_paged_cache (xllm/core/kernels/mlu/mlu_ops_api.h:79-101; HND cache,
    call site xllm/core/layers/mlu/attention.cpp:196-214): the gather of reshape_from_cache applied to
    the dequantised cache, (float)q * scale rounded once to the output type.  quant_mode 1: one scale
    per (block, head, slot); quant_mode 0: one per (head, channel), scale arrays [H, D].
    Returns float32 arrays holding values of `out_kind` ("fp32", "bf16", "fp16")."""
    def dense(cache, scale):
        if cache is None:
            return None
        if kind == "int8":
            f = np.asarray(cache, np.int8).astype(np.float32)
        else:
            f = e4m3fn_to_float(np.asarray(cache).view(np.uint8))
        sc = np.asarray(scale, np.float32)
        f = f * (sc[..., None] if quant_mode == 1 else sc[None, :, None, :])
        return round_to_dtype(f.astype(np.float32), out_kind).astype(np.float32)
    return reshape_from_cache(dense(key_cache, key_scale), dense(value_cache, value_scale), context_lengths,
                              block_tables, context_seq_offset=context_seq_offset, total_rows=total_rows)


# ---- quantisers ------------------------------------------------------------------------

FP8_E4M3_MAX = 448.0
INT8_MAX = 127.0
MIN_SCALE_FP8 = np.float32(1.0) / (np.float32(448.0) * np.float32(512.0))
MIN_SCALE_INT8 = np.float32(np.finfo(np.float32).eps)


def e4m3fn_to_float(b):
    """Decode OCP e4m3fn bytes (uint8 array) to float32: 1-4-3, bias 7, no inf, 0x7f/0xff NaN."""
    b = np.asarray(b, np.uint8)
    sign = np.where(b & 0x80, -1.0, 1.0)
    e = ((b >> 3) & 0xF).astype(np.int32)
    m = (b & 7).astype(np.float64)
    val = np.where(e == 0, m / 8.0 * 2.0 ** -6, (1.0 + m / 8.0) * np.exp2(e.astype(np.float64) - 7))
    val = np.where((b & 0x7F) == 0x7F, np.nan, val)
    return (sign * val).astype(np.float32)


def float_to_e4m3fn(x):
    """Round-to-nearest-even float32 -> e4m3fn byte for |x| <= 448 (callers clamp first)."""
    x = np.asarray(x, np.float32)
    sign = (np.signbit(x)).astype(np.uint8) << 7
    a = np.abs(x).astype(np.float64)
    # quantum: subnormal range [0, 2^-6) has spacing 2^-9; normal binade [2^e, 2^(e+1)) has spacing 2^(e-3)
    with np.errstate(divide="ignore"):
        e = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    e = np.clip(e, -6, 8)
    quantum = np.exp2(e - 3)
    q = np.rint(a / quantum)  # numpy rint = round half to even
    val = q * quantum  # exactly representable: may have carried into the next binade
    # re-derive exponent/mantissa from the rounded value
    with np.errstate(divide="ignore"):
        e2 = np.floor(np.log2(np.where(val > 0, val, 1.0)))
    e2 = np.clip(e2, -6, 8)
    is_sub = val < 2.0 ** -6
    mant = np.where(is_sub, val / 2.0 ** -9, (val / np.exp2(e2) - 1.0) * 8.0)
    expo = np.where(is_sub, 0, e2 + 7)
    byte = (expo.astype(np.int64) << 3) | np.rint(mant).astype(np.int64)
    byte = np.where(val == 0, 0, byte)
    return (byte.astype(np.uint8) | sign).astype(np.uint8)


def quantize_per_token_head(x, kind):
    """x: float32 [..., head_dim] -> (q, scale) with one scale per leading index.
    kind 'int8': q int8 = clamp(rint(x/scale), -127, 127), scale = max(absmax/127, FLT_EPSILON)
    kind 'fp8' : q uint8 (e4m3fn bits) = rne(clamp(x/scale, -448, 448)), scale = max(absmax/448, 1/(448*512)).
    Non-finite inputs follow C's fmaxf/fminf, which return the other operand for a NaN: absmax skips NaN
    elements, and clamp(y, -m, m) = fmaxf(-m, fminf(y, m)) — the order of
    xllm/core/kernels/cuda/fp8_quant_utils.cuh:121-122 — turns a NaN quotient (a NaN element, or an
    infinite one: inf / inf) into +m.  (The int8 quantiser of the reference is closed source; the same
    order is used for it.)"""
    x = np.asarray(x, np.float32)
    amax = np.fmax.reduce(np.abs(x), axis=-1, keepdims=True, initial=np.float32(0)).astype(np.float32)
    with np.errstate(invalid="ignore", divide="ignore", over="ignore"):
        if kind == "int8":
            scale = np.maximum(amax / np.float32(INT8_MAX), MIN_SCALE_INT8).astype(np.float32)
            y = (x / scale).astype(np.float32)
            q = np.fmax(np.float32(-127), np.fmin(np.rint(y), np.float32(127))).astype(np.int8)
        elif kind == "fp8":
            scale = np.maximum(amax / np.float32(FP8_E4M3_MAX), MIN_SCALE_FP8).astype(np.float32)
            y = np.fmax(np.float32(-FP8_E4M3_MAX), np.fmin((x / scale).astype(np.float32), np.float32(FP8_E4M3_MAX)))
            q = float_to_e4m3fn(y)
        else:
            raise ValueError(kind)
    return q, scale[..., 0]


def dequantize(q, scale, kind):
    """float32 value of quantised elements: (float)q * scale."""
    if kind == "int8":
        f = np.asarray(q, np.int8).astype(np.float32)
    else:
        f = e4m3fn_to_float(np.asarray(q).view(np.uint8))
    return f * np.asarray(scale, np.float32)[..., None]


def quant_to_paged_cache(slot_ids, keys, values, key_cache, value_cache, key_scale, value_scale, kind,
                         layout="HND"):
    """keys/values float32 [T, Hkv, D] -> quantised caches (int8 / uint8 e4m3 bits) + fp32 scales
    [blocks, Hkv, bs] (HND) or [blocks, bs, Hkv] (NHD), scattered through slot_ids."""
    kc = _hnd_view(key_cache, layout)
    ks = key_scale if layout == "HND" else key_scale.transpose(0, 2, 1)
    block_size = kc.shape[2]
    slot_ids = np.asarray(slot_ids, np.int64)
    blk, off = slot_ids // block_size, slot_ids % block_size
    qk, sk = quantize_per_token_head(keys, kind)
    kc[blk, :, off, :] = qk
    ks[blk, :, off] = sk
    if values is not None:
        vc = _hnd_view(value_cache, layout)
        vs = value_scale if layout == "HND" else value_scale.transpose(0, 2, 1)
        qv, sv = quantize_per_token_head(values, kind)
        vc[blk, :, off, :] = qv
        vs[blk, :, off] = sv


# ---------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------


def gather_sequence(cache_hnd, block_row, seq_len):
    """[Hkv, seq_len, D] rows of one sequence, found through its block-table row."""
    block_size = cache_hnd.shape[2]
    t = np.arange(seq_len)
    blk = np.asarray(block_row, np.int64)[t // block_size]
    return cache_hnd[blk, :, t % block_size, :].transpose(1, 0, 2)


def paged_decode_loops(q, k_cache, v_cache, block_table, seq_lens, scale, q_per_seq=1, window_left=-1,
                       layout="HND"):
    """Scalar-loop attention in float64 (small inputs only): the definition every other path is
    checked against.  q [B*n, Hq, D]; caches already float (dequantised); returns (out, lse2)."""
    kc, vc = _hnd_view(np.asarray(k_cache), layout), _hnd_view(np.asarray(v_cache), layout)
    T, Hq, D = q.shape
    Hkv, bs = kc.shape[1], kc.shape[2]
    g = Hq // Hkv
    n = q_per_seq
    B = T // n
    out = np.zeros((T, Hq, D), np.float64)
    lse2 = np.full((T, Hq), -np.inf, np.float64)
    for b in range(B):
        L = int(seq_lens[b])
        for j in range(n):
            lim = L - (n - 1 - j)
            lo = (lim - 1 - window_left) if window_left >= 0 else 0
            for h in range(Hq):
                kvh = h // g
                scores = []
                toks = []
                for t in range(max(lo, 0), lim):
                    blk = int(block_table[b][t // bs])
                    kvec = kc[blk, kvh, t % bs]
                    s = 0.0
                    for d in range(D):
                        s += float(q[b * n + j, h, d]) * float(kvec[d])
                    scores.append(s * scale)
                    toks.append(t)
                if not scores:
                    continue
                mx = max(scores)
                w = [math.exp(s - mx) for s in scores]
                den = sum(w)
                lse2[b * n + j, h] = (mx + math.log(den)) / math.log(2.0)
                for wt, t in zip(w, toks):
                    blk = int(block_table[b][t // bs])
                    vvec = vc[blk, kvh, t % bs]
                    for d in range(D):
                        out[b * n + j, h, d] += wt / den * float(vvec[d])
    return out, lse2


def paged_decode(q, k_cache, v_cache, block_table, seq_lens, scale, q_per_seq=1, window_left=-1, layout="HND",
                 k_scale=None, v_scale=None, kind=None, acc_dtype=np.float64):
    """Vectorised numpy attention, one sequence at a time.  Quantised caches are dequantised first
    ((float)q * scale per token and head).  Returns (out [T,Hq,D], base-2 lse [T,Hq])."""
    kc, vc = _hnd_view(np.asarray(k_cache), layout), _hnd_view(np.asarray(v_cache), layout)
    if kind is not None:
        ksc = k_scale if layout == "HND" else np.asarray(k_scale).transpose(0, 2, 1)
        vsc = v_scale if layout == "HND" else np.asarray(v_scale).transpose(0, 2, 1)
    q = np.asarray(q)
    T, Hq, D = q.shape
    Hkv = kc.shape[1]
    g = Hq // Hkv
    n = q_per_seq
    B = T // n
    out = np.zeros((T, Hq, D), acc_dtype)
    lse2 = np.full((T, Hq), -np.inf, acc_dtype)
    for b in range(B):
        L = int(seq_lens[b])
        if L <= 0:
            continue
        K = gather_sequence(kc, block_table[b], L)
        V = gather_sequence(vc, block_table[b], L)
        if kind is not None:
            K = dequantize(K, gather_sequence(ksc[..., None], block_table[b], L)[..., 0], kind)
            V = dequantize(V, gather_sequence(vsc[..., None], block_table[b], L)[..., 0], kind)
        K = K.astype(acc_dtype)
        V = V.astype(acc_dtype)
        qb = q[b * n:(b + 1) * n].astype(acc_dtype).reshape(n, Hkv, g, D)
        s = np.einsum("jkgd,ktd->jkgt", qb, K) * scale  # [n, Hkv, g, L]
        t = np.arange(L)
        lim = L - (n - 1 - np.arange(n))
        vis = t[None, :] < lim[:, None]
        if window_left >= 0:
            vis &= t[None, :] >= (lim[:, None] - 1 - window_left)
        s = np.where(vis[:, None, None, :], s, -np.inf)
        mx = np.max(s, axis=-1, keepdims=True)
        mx_safe = np.where(np.isfinite(mx), mx, 0.0)
        w = np.exp(s - mx_safe)
        den = np.sum(w, axis=-1, keepdims=True)
        with np.errstate(divide="ignore", invalid="ignore"):
            p = np.where(den > 0, w / den, 0.0)
            l2 = np.where(den > 0, (mx_safe + np.log(den)) / math.log(2.0), -np.inf)
        o = np.einsum("jkgt,ktd->jkgd", p, V)
        out[b * n:(b + 1) * n] = o.reshape(n, Hq, D)
        lse2[b * n:(b + 1) * n] = l2.reshape(n, Hq)
    return out, lse2


def paged_decode_ragged(q, k_cache, v_cache, block_table, seq_lens, q_indptr, scale, **kw):
    """Sequences with different numbers of query tokens (a chunked-prefill or mixed step,
    xllm/core/layers/cuda/flashinfer_attention.cpp:224-284 with the causal mask): sequence b owns rows
    q_indptr[b]:q_indptr[b+1] of q, the last n_b tokens of its kv range, token j seeing
    seq_lens[b] - (n_b - 1 - j) keys.  One paged_decode call per sequence."""
    q = np.asarray(q)
    out = np.zeros(q.shape, np.float64)
    lse2 = np.full(q.shape[:2], -np.inf, np.float64)
    for b in range(len(q_indptr) - 1):
        q0, q1 = int(q_indptr[b]), int(q_indptr[b + 1])
        if q1 <= q0:
            continue
        o, l = paged_decode(q[q0:q1], k_cache, v_cache, [block_table[b]], [seq_lens[b]], scale, q_per_seq=q1 - q0, **kw)
        out[q0:q1], lse2[q0:q1] = o, l
    return out, lse2


def lse_combine(o_a, lse_a, o_b, lse_b):
    """lse_combine_kernel: merge two partial attentions whose LSEs are base-2."""
    lse_a = np.asarray(lse_a, np.float64)[..., None]
    lse_b = np.asarray(lse_b, np.float64)[..., None]
    lse_max = np.maximum(lse_a, lse_b)
    e_a = np.exp2(lse_a - lse_max)
    e_b = np.exp2(lse_b - lse_max)
    lse_new = lse_max + np.log2(e_a + e_b)
    w_a = np.exp2(lse_a - lse_new)
    w_b = np.exp2(lse_b - lse_new)
    return w_a * o_a + w_b * o_b, lse_new[..., 0]
