// Reading sequences back out of a paged KV cache into dense [total_tokens, num_kv_heads, head_dim]
// tensors for gfx950: xllm::kernel::reshape_from_cache (verbatim copy,
// xllm/core/kernels/ops_api.cpp:182-196, xllm/core/kernels/mlu/mlu_ops_api.h:56-64) and
// xllm::kernel::dequant_from_paged_cache (quantised cache -> 16/32-bit floats,
// xllm/core/kernels/ops_api.cpp:214-232, xllm/core/kernels/mlu/mlu_ops_api.h:79-101), which the
// MLU attention layer runs before a chunked-prefill step over a quantised cache
// (xllm/core/layers/mlu/attention.cpp:179-214).
//
// Token t of sequence b sits at cache position cache_seq_offset[b] + t, i.e. in block
// block_tables[b][pos / block_size], slot pos % block_size, and goes to output row
// context_seq_offset[b] + t (without offsets: the sequences packed one after the other).
// Pure HBM traffic: every cache element is read once and written once.
#include "device_utils.h"
#include "host_utils.h"

namespace xllm_hip {

struct GatherParams {
  const uint8_t* cache[2];  // K, V
  const float* scale[2];
  uint8_t* out[2];
  int64_t out_token_stride[2];  // elements
  int64_t stride_block, stride_head, stride_slot;           // elements
  int64_t sc_stride_block, sc_stride_head, sc_stride_slot;  // floats
  const int32_t* context_lengths;
  const int32_t* context_seq_offset;  // NULL: packed
  const int32_t* cache_seq_offset;    // NULL: 0
  const int32_t* block_tables;
  int64_t bt_stride;
  int64_t num_blocks;
  int32_t max_blocks_per_seq;
  int32_t batch;
  int32_t tiles;  // token tiles per sequence: ceil(max_context_len / kGatherTile)
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t block_size;
  int32_t arrays;       // 1: K only, 2: K and V
  int32_t per_channel;  // scales are [num_kv_heads, head_dim] instead of one per (block, head, slot)
};

constexpr int kGatherTile = 64;  // tokens per workgroup

// N floats -> N elements of ODT at dst (16-byte stores).
template <int ODT, int N>
__device__ inline void store_converted(uint8_t* dst, const float (&x)[N]) {
  if constexpr (ODT == XLLM_HIP_FP32) {
#pragma unroll
    for (int i = 0; i < N; i += 4) *(f32x4*)(dst + i * 4) = f32x4{x[i], x[i + 1], x[i + 2], x[i + 3]};
  } else if constexpr (ODT == XLLM_HIP_BF16) {
#pragma unroll
    for (int i = 0; i < N; i += 8) {
      u32x4 w;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        w[e] = (uint32_t)float_to_bf16_bits(x[i + 2 * e]) | ((uint32_t)float_to_bf16_bits(x[i + 2 * e + 1]) << 16);
      }
      *(u32x4*)(dst + i * 2) = w;
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; i += 8) {
      f16x8 w;
#pragma unroll
      for (int e = 0; e < 8; ++e) w[e] = (_Float16)x[i + e];
      *(f16x8*)(dst + i * 2) = w;
    }
  }
}

// grid.x = (sequence, token tile, head) flattened.  V: elements per thread and step (16 bytes of
// the cache), or 1 when alignment does not allow vectors.  CDT == ODT: verbatim copy.
template <int CDT, int ODT, int V>
__global__ void __launch_bounds__(256) gather_from_cache_kernel(GatherParams p) {
  __shared__ int32_t red[256];
  const int h = blockIdx.x % p.num_kv_heads;
  const int rest = blockIdx.x / p.num_kv_heads;
  const int tile = rest % p.tiles;
  const int b = rest / p.tiles;
  const int len = p.context_lengths[b];
  const int t0 = tile * kGatherTile;
  if (t0 >= len) return;

  // first output row of the sequence
  int64_t row0;
  if (p.context_seq_offset != nullptr) {
    row0 = p.context_seq_offset[b];
  } else {
    int32_t part = 0;
    for (int i = threadIdx.x; i < b; i += 256) part += p.context_lengths[i];
    red[threadIdx.x] = part;
    __syncthreads();
    for (int s = 128; s >= 1; s >>= 1) {
      if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
      __syncthreads();
    }
    row0 = red[0];
  }
  const int pos0 = p.cache_seq_offset != nullptr ? p.cache_seq_offset[b] : 0;
  const int vpr = p.head_dim / V;  // vectors per row
  const int n_tok = min(kGatherTile, len - t0);
  constexpr int kIn = CDT == XLLM_HIP_FP32 ? 4 : (CDT == XLLM_HIP_BF16 || CDT == XLLM_HIP_FP16) ? 2 : 1;
  constexpr int kOut = ODT == XLLM_HIP_FP32 ? 4 : (ODT == XLLM_HIP_BF16 || ODT == XLLM_HIP_FP16) ? 2 : 1;

  for (int idx = threadIdx.x; idx < n_tok * vpr; idx += 256) {
    const int tt = idx / vpr;
    const int d = (idx - tt * vpr) * V;
    const int t = t0 + tt;
    const int pos = pos0 + t;
    const int bi = pos / p.block_size;
    if (bi >= p.max_blocks_per_seq) continue;
    const int64_t blk = p.block_tables[(int64_t)b * p.bt_stride + bi];
    if (blk < 0 || blk >= p.num_blocks) continue;
    const int slot = pos - bi * p.block_size;
    const int64_t src = blk * p.stride_block + (int64_t)h * p.stride_head + (int64_t)slot * p.stride_slot + d;
    const int64_t sc = blk * p.sc_stride_block + (int64_t)h * p.sc_stride_head + (int64_t)slot * p.sc_stride_slot;
    for (int a = 0; a < p.arrays; ++a) {
      uint8_t* dst = p.out[a] + ((row0 + t) * p.out_token_stride[a] + (int64_t)h * p.head_dim + d) * kOut;
      const uint8_t* from = p.cache[a] + src * kIn;
      if constexpr (CDT == ODT) {
        if constexpr (V == 1) {
          if (kIn == 4) *(uint32_t*)dst = *(const uint32_t*)from;
          if (kIn == 2) *(uint16_t*)dst = *(const uint16_t*)from;
          if (kIn == 1) *dst = *from;
        } else {
          *(u32x4*)dst = __builtin_nontemporal_load((const u32x4*)from);
        }
      } else {
        float x[V];
        if constexpr (V == 1) {
          x[0] = Elem<CDT>::load(from, 0);
        } else {
          const u32x4 raw = __builtin_nontemporal_load((const u32x4*)from);
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            if constexpr (CDT == XLLM_HIP_INT8) {
#pragma unroll
              for (int e = 0; e < 4; ++e) x[4 * w + e] = (float)(int8_t)(raw[w] >> (8 * e));
            } else {
              const f32x2 lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[w], false);
              const f32x2 hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)raw[w], true);
              x[4 * w] = lo[0];
              x[4 * w + 1] = lo[1];
              x[4 * w + 2] = hi[0];
              x[4 * w + 3] = hi[1];
            }
          }
        }
        if (p.per_channel) {
          const float* s = p.scale[a] + (int64_t)h * p.head_dim + d;
#pragma unroll
          for (int e = 0; e < V; ++e) x[e] *= s[e];
        } else {
          const float s = p.scale[a][sc];
#pragma unroll
          for (int e = 0; e < V; ++e) x[e] *= s;
        }
        if constexpr (V == 1) {
          Elem<ODT>::store(dst, 0, x[0]);
        } else {
          store_converted<ODT, V>(dst, x);
        }
      }
    }
  }
}

template <int CDT, int ODT>
static void launch_gather(const GatherParams& p, bool vec, hipStream_t st) {
  const unsigned grid = (unsigned)((int64_t)p.batch * p.tiles * p.num_kv_heads);
  constexpr int V = CDT == XLLM_HIP_FP32 ? 4 : (CDT == XLLM_HIP_BF16 || CDT == XLLM_HIP_FP16) ? 8 : 16;
  if (vec) {
    gather_from_cache_kernel<CDT, ODT, V><<<grid, 256, 0, st>>>(p);
  } else {
    gather_from_cache_kernel<CDT, ODT, 1><<<grid, 256, 0, st>>>(p);
  }
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" int xllm_hip_gather_from_cache(const xllm_hip_kv_cache* c,
                                          void* key_out,
                                          void* value_out,
                                          int32_t out_dtype,
                                          int64_t key_token_stride,
                                          int64_t value_token_stride,
                                          const int32_t* context_lengths,
                                          const int32_t* context_seq_offset,
                                          const int32_t* cache_seq_offset,
                                          const int32_t* block_tables,
                                          int64_t block_table_stride,
                                          int32_t max_blocks_per_seq,
                                          int32_t batch,
                                          int32_t max_context_len,
                                          int32_t quant_mode,
                                          xllm_hip_stream_t stream) {
  XLLM_HIP_REQUIRE(c != nullptr, "cache is NULL");
  XLLM_HIP_REQUIRE(c->k_cache != nullptr, "k_cache is NULL");
  XLLM_HIP_REQUIRE(c->num_blocks > 0 && c->block_size > 0 && c->num_kv_heads > 0 && c->head_dim > 0,
                   "cache sizes must be positive");
  const int eb = elem_bytes(c->dtype);
  XLLM_HIP_REQUIRE(eb > 0, "unknown cache dtype %d", c->dtype);
  XLLM_HIP_REQUIRE(batch >= 0 && max_context_len >= 0, "batch or max_context_len is negative");
  if (batch == 0 || max_context_len == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(key_out != nullptr, "key output is NULL");
  XLLM_HIP_REQUIRE(value_out == nullptr || c->v_cache != nullptr, "value output given without a value cache");
  XLLM_HIP_REQUIRE(context_lengths != nullptr && block_tables != nullptr, "context_lengths or block_tables is NULL");
  XLLM_HIP_REQUIRE(max_blocks_per_seq >= 1 && block_table_stride >= max_blocks_per_seq, "bad block_tables shape");
  // the cache's own dtype as output: verbatim copy, also of a quantised cache (no scales involved)
  const bool quant = (c->dtype == XLLM_HIP_FP8_E4M3 || c->dtype == XLLM_HIP_INT8) && out_dtype != c->dtype;
  const int ob = elem_bytes(out_dtype);
  if (quant) {
    XLLM_HIP_REQUIRE(out_dtype == XLLM_HIP_BF16 || out_dtype == XLLM_HIP_FP16 || out_dtype == XLLM_HIP_FP32,
                     "a quantised cache dequantises to BF16/FP16/FP32, got dtype %d", out_dtype);
    XLLM_HIP_REQUIRE(c->k_scale != nullptr && (value_out == nullptr || c->v_scale != nullptr),
                     "a quantised cache needs its scale tensors");
    XLLM_HIP_REQUIRE(quant_mode == 0 || quant_mode == 1, "quant_mode must be 0 (per channel) or 1 (per token)");
  } else {
    XLLM_HIP_REQUIRE(out_dtype == c->dtype, "output dtype %d differs from the cache dtype %d", out_dtype, c->dtype);
  }
  const int64_t rowlen = (int64_t)c->num_kv_heads * c->head_dim;
  XLLM_HIP_REQUIRE(key_token_stride >= rowlen && (value_out == nullptr || value_token_stride >= rowlen),
                   "output token stride smaller than num_kv_heads*head_dim");
  const int tiles = (max_context_len + kGatherTile - 1) / kGatherTile;
  XLLM_HIP_REQUIRE((int64_t)batch * tiles * c->num_kv_heads <= 0x7fffffff, "too many workgroups");

  GatherParams p{};
  p.cache[0] = (const uint8_t*)c->k_cache;
  p.cache[1] = (const uint8_t*)c->v_cache;
  p.scale[0] = c->k_scale;
  p.scale[1] = c->v_scale;
  p.out[0] = (uint8_t*)key_out;
  p.out[1] = (uint8_t*)value_out;
  p.out_token_stride[0] = key_token_stride;
  p.out_token_stride[1] = value_token_stride;
  p.stride_block = c->stride_block;
  p.stride_head = c->stride_head;
  p.stride_slot = c->stride_slot;
  p.sc_stride_block = c->scale_stride_block;
  p.sc_stride_head = c->scale_stride_head;
  p.sc_stride_slot = c->scale_stride_slot;
  p.context_lengths = context_lengths;
  p.context_seq_offset = context_seq_offset;
  p.cache_seq_offset = cache_seq_offset;
  p.block_tables = block_tables;
  p.bt_stride = block_table_stride;
  p.num_blocks = c->num_blocks;
  p.max_blocks_per_seq = max_blocks_per_seq;
  p.batch = batch;
  p.tiles = tiles;
  p.num_kv_heads = c->num_kv_heads;
  p.head_dim = c->head_dim;
  p.block_size = c->block_size;
  p.arrays = value_out != nullptr ? 2 : 1;
  p.per_channel = quant && quant_mode == 0 ? 1 : 0;

  // 16-byte pieces of the cache per thread when every address allows it
  const int vin = 16 / eb;
  const uintptr_t in_mix = (uintptr_t)c->k_cache | (uintptr_t)(value_out ? c->v_cache : nullptr);
  const uintptr_t out_mix = (uintptr_t)key_out | (uintptr_t)value_out | (uintptr_t)(key_token_stride * ob) |
                            (uintptr_t)((value_out ? value_token_stride : 0) * ob);
  const bool vec = c->head_dim % vin == 0 && c->stride_block % vin == 0 && c->stride_head % vin == 0 &&
                   c->stride_slot % vin == 0 && (in_mix & 15) == 0 && (out_mix & 15) == 0;
  hipStream_t st = (hipStream_t)stream;
  switch (c->dtype) {
    case XLLM_HIP_BF16:
      launch_gather<XLLM_HIP_BF16, XLLM_HIP_BF16>(p, vec, st);
      break;
    case XLLM_HIP_FP16:
      launch_gather<XLLM_HIP_FP16, XLLM_HIP_FP16>(p, vec, st);
      break;
    case XLLM_HIP_FP32:
      launch_gather<XLLM_HIP_FP32, XLLM_HIP_FP32>(p, vec, st);
      break;
    case XLLM_HIP_INT8:
      if (out_dtype == XLLM_HIP_INT8) launch_gather<XLLM_HIP_INT8, XLLM_HIP_INT8>(p, vec, st);
      if (out_dtype == XLLM_HIP_BF16) launch_gather<XLLM_HIP_INT8, XLLM_HIP_BF16>(p, vec, st);
      if (out_dtype == XLLM_HIP_FP16) launch_gather<XLLM_HIP_INT8, XLLM_HIP_FP16>(p, vec, st);
      if (out_dtype == XLLM_HIP_FP32) launch_gather<XLLM_HIP_INT8, XLLM_HIP_FP32>(p, vec, st);
      break;
    default:
      if (out_dtype == XLLM_HIP_FP8_E4M3) launch_gather<XLLM_HIP_FP8_E4M3, XLLM_HIP_FP8_E4M3>(p, vec, st);
      if (out_dtype == XLLM_HIP_BF16) launch_gather<XLLM_HIP_FP8_E4M3, XLLM_HIP_BF16>(p, vec, st);
      if (out_dtype == XLLM_HIP_FP16) launch_gather<XLLM_HIP_FP8_E4M3, XLLM_HIP_FP16>(p, vec, st);
      if (out_dtype == XLLM_HIP_FP32) launch_gather<XLLM_HIP_FP8_E4M3, XLLM_HIP_FP32>(p, vec, st);
      break;
  }
  return check_launch("gather_from_cache_kernel");
}
