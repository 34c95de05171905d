// KV write through slot_mapping for gfx950: the verbatim scatter
// (reshape_paged_cache) and the per-token-per-head quantising scatter
// (quant_to_paged_cache).
//
// Index math follows reshape_paged_cache_kernel
// (xllm/core/kernels/cuda/reshape_paged_cache.cu:35-57): block = slot / bs,
// offset = slot % bs, then (block, offset, head, d) is resolved through the
// cache strides so that both the NHD and the HND block layouts are served.
#include "device_utils.h"
#include "host_utils.h"

#include <float.h>

namespace xllm_hip {

struct KvWriteParams {
  const uint8_t* key;
  const uint8_t* value;
  uint8_t* k_cache;
  uint8_t* v_cache;
  float* k_scale;
  float* v_scale;
  const int32_t* slots;
  int64_t key_token_stride;    // bytes (copy kernel) or elements (quant kernel)
  int64_t value_token_stride;
  int64_t stride_block;        // bytes (copy kernel) or elements (quant kernel)
  int64_t stride_head;
  int64_t stride_slot;
  int64_t scale_stride_block;  // elements
  int64_t scale_stride_head;
  int64_t scale_stride_slot;
  int64_t num_slots;
  int64_t num_tokens;
  int32_t row_bytes;  // head_dim * element size (copy kernel)
  int32_t head_dim;
  int32_t num_kv_heads;
  int32_t block_size;
};

// One workgroup per (token, K|V).  Every thread moves VEC bytes at a time; the
// host picks the widest VEC that all pointers and strides are aligned to.
template <typename VecT>
__global__ void __launch_bounds__(256) reshape_paged_cache_kernel(KvWriteParams p) {
  const int64_t t = blockIdx.x;
  const bool is_v = blockIdx.y != 0;
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t block = slot / p.block_size;
  const int64_t off = slot % p.block_size;
  const uint8_t* src = (is_v ? p.value : p.key) + t * (is_v ? p.value_token_stride : p.key_token_stride);
  uint8_t* dst = (is_v ? p.v_cache : p.k_cache) + block * p.stride_block + off * p.stride_slot;
  const int vec_per_row = p.row_bytes / (int)sizeof(VecT);
  const int total = p.num_kv_heads * vec_per_row;
  for (int i = threadIdx.x; i < total; i += blockDim.x) {
    const int h = i / vec_per_row;
    const int c = i - h * vec_per_row;
    const VecT v = *(const VecT*)(src + (int64_t)h * p.row_bytes + (int64_t)c * sizeof(VecT));
    *(VecT*)(dst + (int64_t)h * p.stride_head + (int64_t)c * sizeof(VecT)) = v;
  }
}

// One wave per (token, head, K|V): absmax over head_dim, scale, quantise, scatter.
template <int SRC_DT, int DST_DT>
__global__ void __launch_bounds__(256) quant_to_paged_cache_kernel(KvWriteParams p) {
  constexpr int kMaxPerLane = 8;  // head_dim <= 512
  const int lane = threadIdx.x & 63;
  const int64_t pair = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (pair >= p.num_tokens * p.num_kv_heads) return;
  const bool is_v = blockIdx.y != 0;
  const int64_t t = pair / p.num_kv_heads;
  const int h = (int)(pair - t * p.num_kv_heads);
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t block = slot / p.block_size;
  const int64_t off = slot % p.block_size;

  const void* src = is_v ? (const void*)p.value : (const void*)p.key;
  const int64_t src_base = t * (is_v ? p.value_token_stride : p.key_token_stride) + (int64_t)h * p.head_dim;

  float x[kMaxPerLane];
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + i * 64;
    x[i] = d < p.head_dim ? Elem<SRC_DT>::load(src, src_base + d) : 0.0f;
    amax = fmaxf(amax, fabsf(x[i]));
  }
  amax = wave_max(amax);

  constexpr float kQmax = DST_DT == XLLM_HIP_INT8 ? 127.0f : 448.0f;
  constexpr float kMinScale = DST_DT == XLLM_HIP_INT8 ? FLT_EPSILON : 1.0f / (448.0f * 512.0f);
  const float scale = fmaxf(amax / kQmax, kMinScale);

  uint8_t* dst = (is_v ? p.v_cache : p.k_cache) + block * p.stride_block + (int64_t)h * p.stride_head +
                 off * p.stride_slot;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + i * 64;
    if (d < p.head_dim) {
      const float y = x[i] / scale;
      dst[d] = DST_DT == XLLM_HIP_INT8 ? quantise_int8(y) : quantise_fp8_e4m3(y);
    }
  }
  if (lane == 0) {
    float* sc = is_v ? p.v_scale : p.k_scale;
    sc[block * p.scale_stride_block + (int64_t)h * p.scale_stride_head + off * p.scale_stride_slot] = scale;
  }
}

static int check_cache_common(const xllm_hip_kv_cache* c, bool need_v) {
  XLLM_HIP_REQUIRE(c != nullptr, "cache descriptor is NULL");
  XLLM_HIP_REQUIRE(c->k_cache != nullptr, "k_cache is NULL");
  XLLM_HIP_REQUIRE(!need_v || c->v_cache != nullptr, "value given but v_cache is NULL");
  XLLM_HIP_REQUIRE(c->num_blocks > 0 && c->block_size > 0 && c->num_kv_heads > 0 && c->head_dim > 0,
                   "cache sizes must be positive (blocks=%lld bs=%d heads=%d dim=%d)", (long long)c->num_blocks,
                   c->block_size, c->num_kv_heads, c->head_dim);
  XLLM_HIP_REQUIRE(elem_bytes(c->dtype) > 0, "unknown cache dtype %d", c->dtype);
  XLLM_HIP_REQUIRE(c->stride_block > 0 && c->stride_head > 0 && c->stride_slot > 0,
                   "cache strides must be positive");
  return XLLM_HIP_OK;
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" int xllm_hip_reshape_paged_cache(const xllm_hip_kv_cache* cache,
                                            const void* key,
                                            const void* value,
                                            const int32_t* slot_mapping,
                                            int64_t num_tokens,
                                            int64_t key_token_stride,
                                            int64_t value_token_stride,
                                            int32_t src_dtype,
                                            xllm_hip_stream_t stream) {
  if (int s = check_cache_common(cache, value != nullptr)) return s;
  XLLM_HIP_REQUIRE(num_tokens >= 0, "num_tokens is negative");
  if (num_tokens == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(key != nullptr && slot_mapping != nullptr, "key or slot_mapping is NULL");
  XLLM_HIP_REQUIRE(src_dtype == cache->dtype,
                   "reshape_paged_cache copies verbatim: key dtype %d != cache dtype %d "
                   "(use xllm_hip_quant_to_paged_cache for a quantised cache)",
                   src_dtype, cache->dtype);
  const int eb = elem_bytes(cache->dtype);
  const int64_t row = (int64_t)cache->num_kv_heads * cache->head_dim;
  XLLM_HIP_REQUIRE(key_token_stride >= row && (value == nullptr || value_token_stride >= row),
                   "token stride smaller than num_kv_heads*head_dim");

  KvWriteParams p{};
  p.key = (const uint8_t*)key;
  p.value = (const uint8_t*)value;
  p.k_cache = (uint8_t*)cache->k_cache;
  p.v_cache = (uint8_t*)cache->v_cache;
  p.slots = slot_mapping;
  p.key_token_stride = key_token_stride * eb;
  p.value_token_stride = value_token_stride * eb;
  p.stride_block = cache->stride_block * eb;
  p.stride_head = cache->stride_head * eb;
  p.stride_slot = cache->stride_slot * eb;
  p.num_slots = cache->num_blocks * cache->block_size;
  p.num_tokens = num_tokens;
  p.row_bytes = cache->head_dim * eb;
  p.head_dim = cache->head_dim;
  p.num_kv_heads = cache->num_kv_heads;
  p.block_size = cache->block_size;

  // Widest vector every address is a multiple of.
  uint64_t align = (uint64_t)(uintptr_t)p.key | (uint64_t)(uintptr_t)p.k_cache | (uint64_t)p.key_token_stride |
                   (uint64_t)p.stride_block | (uint64_t)p.stride_head | (uint64_t)p.stride_slot |
                   (uint64_t)p.row_bytes;
  if (value != nullptr) {
    align |= (uint64_t)(uintptr_t)p.value | (uint64_t)(uintptr_t)p.v_cache | (uint64_t)p.value_token_stride;
  }
  const dim3 grid((unsigned)num_tokens, value != nullptr ? 2 : 1);
  hipStream_t st = (hipStream_t)stream;
  if ((align & 15) == 0) {
    const int threads = (int)std::min<int64_t>(256, std::max<int64_t>(64, row * eb / 16));
    reshape_paged_cache_kernel<u32x4><<<grid, threads, 0, st>>>(p);
  } else if ((align & 3) == 0) {
    reshape_paged_cache_kernel<uint32_t><<<grid, 256, 0, st>>>(p);
  } else if ((align & 1) == 0) {
    reshape_paged_cache_kernel<uint16_t><<<grid, 256, 0, st>>>(p);
  } else {
    reshape_paged_cache_kernel<uint8_t><<<grid, 256, 0, st>>>(p);
  }
  return check_launch("reshape_paged_cache_kernel");
}

// head_dim 128 on aligned rows: sixteen lanes per (token, head, K|V), eight consecutive elements per
// lane (one 16-byte load for 2-byte sources, two for fp32), one 8-byte store.  Same arithmetic as
// above (a maximum does not depend on the order it is taken in).
template <int SRC_DT, int DST_DT>
__global__ void __launch_bounds__(256) quant_to_paged_cache_d128_kernel(KvWriteParams p) {
  const int sub = threadIdx.x & 15;
  const int64_t pair = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool live = pair < p.num_tokens * p.num_kv_heads;  // idle groups still take part in the shuffles
  const bool is_v = blockIdx.y != 0;
  const int64_t t = live ? pair / p.num_kv_heads : 0;
  const int h = live ? (int)(pair - t * p.num_kv_heads) : 0;
  const int64_t slot = live ? (int64_t)p.slots[t] : -1;
  const bool writes = slot >= 0 && slot < p.num_slots;
  const int64_t block = writes ? slot / p.block_size : 0;
  const int64_t off = writes ? slot % p.block_size : 0;
  const uint8_t* src = is_v ? p.value : p.key;
  const int64_t src_base = t * (is_v ? p.value_token_stride : p.key_token_stride) + (int64_t)h * 128 + 8 * sub;
  float x[8];
  if (SRC_DT == XLLM_HIP_FP32) {
    const f32x4 a = *(const f32x4*)(src + src_base * 4);
    const f32x4 b = *(const f32x4*)(src + src_base * 4 + 16);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      x[e] = a[e];
      x[4 + e] = b[e];
    }
  } else {
    const u32x4 raw = *(const u32x4*)(src + src_base * 2);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t w = raw[e >> 1];
      if (SRC_DT == XLLM_HIP_BF16) {
        x[e] = __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
      } else {
        x[e] = (float)__builtin_bit_cast(_Float16, (uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu)));
      }
    }
  }
  float amax = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[e]));
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o));
  if (!writes) return;
  constexpr float kQmax = DST_DT == XLLM_HIP_INT8 ? 127.0f : 448.0f;
  constexpr float kMinScale = DST_DT == XLLM_HIP_INT8 ? FLT_EPSILON : 1.0f / (448.0f * 512.0f);
  const float scale = fmaxf(amax / kQmax, kMinScale);
  uint32_t q2[2] = {0, 0};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float y = x[e] / scale;
    const uint32_t q = DST_DT == XLLM_HIP_INT8 ? quantise_int8(y) : quantise_fp8_e4m3(y);
    q2[e >> 2] |= q << (8 * (e & 3));
  }
  uint8_t* dst = (is_v ? p.v_cache : p.k_cache) + block * p.stride_block + (int64_t)h * p.stride_head +
                 off * p.stride_slot + 8 * sub;
  *(u32x2*)dst = u32x2{q2[0], q2[1]};
  if (sub == 0) {
    float* sc = is_v ? p.v_scale : p.k_scale;
    sc[block * p.scale_stride_block + (int64_t)h * p.scale_stride_head + off * p.scale_stride_slot] = scale;
  }
}

template <int SRC_DT>
static void launch_quant(int dst_dtype, const KvWriteParams& p, dim3 grid, hipStream_t st) {
  const int seb = SRC_DT == XLLM_HIP_FP32 ? 4 : 2;
  const bool d128 = p.head_dim == 128 &&
                    (((uintptr_t)p.key | (uintptr_t)p.value | (uintptr_t)(p.key_token_stride * seb) |
                      (uintptr_t)(p.value_token_stride * seb)) & 15) == 0 &&
                    (((uintptr_t)p.k_cache | (uintptr_t)p.v_cache | (uintptr_t)p.stride_block | (uintptr_t)p.stride_head |
                      (uintptr_t)p.stride_slot) & 7) == 0;
  if (d128) {
    const int64_t pairs = p.num_tokens * p.num_kv_heads;
    const dim3 g16((unsigned)((pairs + 15) / 16), grid.y);
    if (dst_dtype == XLLM_HIP_INT8) {
      quant_to_paged_cache_d128_kernel<SRC_DT, XLLM_HIP_INT8><<<g16, 256, 0, st>>>(p);
    } else {
      quant_to_paged_cache_d128_kernel<SRC_DT, XLLM_HIP_FP8_E4M3><<<g16, 256, 0, st>>>(p);
    }
    return;
  }
  if (dst_dtype == XLLM_HIP_INT8) {
    quant_to_paged_cache_kernel<SRC_DT, XLLM_HIP_INT8><<<grid, 256, 0, st>>>(p);
  } else {
    quant_to_paged_cache_kernel<SRC_DT, XLLM_HIP_FP8_E4M3><<<grid, 256, 0, st>>>(p);
  }
}

extern "C" int xllm_hip_quant_to_paged_cache(const xllm_hip_kv_cache* cache,
                                             const void* key,
                                             const void* value,
                                             const int32_t* slot_mapping,
                                             int64_t num_tokens,
                                             int64_t key_token_stride,
                                             int64_t value_token_stride,
                                             int32_t src_dtype,
                                             xllm_hip_stream_t stream) {
  if (int s = check_cache_common(cache, value != nullptr)) return s;
  XLLM_HIP_REQUIRE(num_tokens >= 0, "num_tokens is negative");
  if (num_tokens == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(key != nullptr && slot_mapping != nullptr, "key or slot_mapping is NULL");
  XLLM_HIP_REQUIRE(cache->dtype == XLLM_HIP_INT8 || cache->dtype == XLLM_HIP_FP8_E4M3,
                   "quant_to_paged_cache needs an INT8 or FP8_E4M3 cache, got dtype %d", cache->dtype);
  XLLM_HIP_REQUIRE(src_dtype == XLLM_HIP_BF16 || src_dtype == XLLM_HIP_FP16 || src_dtype == XLLM_HIP_FP32,
                   "quant_to_paged_cache source must be BF16/FP16/FP32, got dtype %d", src_dtype);
  XLLM_HIP_REQUIRE(cache->k_scale != nullptr, "k_cache_scale is required for quant_to_paged_cache");
  XLLM_HIP_REQUIRE(value == nullptr || cache->v_scale != nullptr, "value given but v_cache_scale is NULL");
  if (cache->head_dim > 512) {
    return fail(XLLM_HIP_UNSUPPORTED, "quant_to_paged_cache supports head_dim <= 512, got %d", cache->head_dim);
  }
  const int64_t row = (int64_t)cache->num_kv_heads * cache->head_dim;
  XLLM_HIP_REQUIRE(key_token_stride >= row && (value == nullptr || value_token_stride >= row),
                   "token stride smaller than num_kv_heads*head_dim");

  KvWriteParams p{};
  p.key = (const uint8_t*)key;
  p.value = (const uint8_t*)value;
  p.k_cache = (uint8_t*)cache->k_cache;
  p.v_cache = (uint8_t*)cache->v_cache;
  p.k_scale = cache->k_scale;
  p.v_scale = cache->v_scale;
  p.slots = slot_mapping;
  p.key_token_stride = key_token_stride;
  p.value_token_stride = value_token_stride;
  p.stride_block = cache->stride_block;
  p.stride_head = cache->stride_head;
  p.stride_slot = cache->stride_slot;
  p.scale_stride_block = cache->scale_stride_block;
  p.scale_stride_head = cache->scale_stride_head;
  p.scale_stride_slot = cache->scale_stride_slot;
  p.num_slots = cache->num_blocks * cache->block_size;
  p.num_tokens = num_tokens;
  p.head_dim = cache->head_dim;
  p.num_kv_heads = cache->num_kv_heads;
  p.block_size = cache->block_size;

  const int64_t pairs = num_tokens * cache->num_kv_heads;
  const dim3 grid((unsigned)((pairs + 3) / 4), value != nullptr ? 2 : 1);
  hipStream_t st = (hipStream_t)stream;
  switch (src_dtype) {
    case XLLM_HIP_BF16:
      launch_quant<XLLM_HIP_BF16>(cache->dtype, p, grid, st);
      break;
    case XLLM_HIP_FP16:
      launch_quant<XLLM_HIP_FP16>(cache->dtype, p, grid, st);
      break;
    default:
      launch_quant<XLLM_HIP_FP32>(cache->dtype, p, grid, st);
      break;
  }
  return check_launch("quant_to_paged_cache_kernel");
}
