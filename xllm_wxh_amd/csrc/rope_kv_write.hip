// The step in front of the decode path, in one pass over the fused qkv buffer: per-head RMSNorm of
// the query and key heads, rotary position embedding, and the scatter of the new K and V rows into
// the paged cache (verbatim or quantised per token and head).
//
//   norm + rotation, float arithmetic, one rounding   xllm/core/kernels/cuda/fused_qknorm_rope.cu:70-262
//   rotation alone, every operation rounded           xllm/core/kernels/cuda/rope.cu:26-52 (the
//                                                     arithmetic of scalar_t operands)
//   call sites                                        xllm/core/layers/common/qwen2_attention.cpp:147-189
//   cache write                                       the arithmetic of kv_write.hip
//
// General kernel: one wave per (token, head); the head's values go through LDS once so that a lane
// can pick up the rotation partner of each of its elements whatever head_dim, rotary_dim and style
// are.  head_dim 128 with 2-byte elements (every current model on this path) takes a kernel with
// sixteen lanes per head and 16-byte accesses instead.
#include "device_utils.h"
#include "host_utils.h"

#include <float.h>

namespace xllm_hip {

struct RopeParams {
  uint8_t* qkv;  // [tokens, (Hq + Hk + Hv) * D], q and k heads rewritten in place
  const void* q_weight;
  const void* k_weight;
  const void* cos_sin;  // [max_position, rotary_dim]: cos of the rotary_dim/2 frequencies, then sin
  const void* positions;
  int32_t positions_int32;  // nonzero: positions holds int32 entries, else int64
  const int32_t* slots;  // NULL: no cache write
  uint8_t* k_cache;
  uint8_t* v_cache;
  float* k_scale;
  float* v_scale;
  int64_t token_stride;  // elements
  int64_t stride_block;  // cache strides, elements
  int64_t stride_head;
  int64_t stride_slot;
  int64_t sc_stride_block;
  int64_t sc_stride_head;
  int64_t sc_stride_slot;
  int64_t num_tokens;
  int64_t num_slots;
  int64_t max_position;
  int32_t num_q_heads;
  int32_t num_k_heads;
  int32_t num_v_heads;
  int32_t head_dim;
  int32_t rotary_dim;
  int32_t block_size;
  int32_t cos_sin_dtype;
  int32_t interleave;   // pairs (2j, 2j+1) instead of (j, j + rotary_dim/2)
  int32_t per_op;       // round after every multiply and add, as arithmetic on scalar_t operands does
  float eps;
};

__device__ inline float load_any(const void* p, int64_t i, int dtype) {
  switch (dtype) {
    case XLLM_HIP_BF16:
      return Elem<XLLM_HIP_BF16>::load(p, i);
    case XLLM_HIP_FP16:
      return Elem<XLLM_HIP_FP16>::load(p, i);
    default:
      return Elem<XLLM_HIP_FP32>::load(p, i);
  }
}

// x as the element type DT holds it.
template <int DT>
__device__ inline float rounded(float x) {
  if (DT == XLLM_HIP_BF16) return bf16_bits_to_float(float_to_bf16_bits(x));
  if (DT == XLLM_HIP_FP16) return (float)(_Float16)x;
  return x;
}

enum { kNoCache = 0, kVerbatim = 1, kInt8 = 2, kFp8 = 3 };

template <int DT, int CACHE>
__global__ void __launch_bounds__(256) rope_kv_write_kernel(RopeParams p) {
  constexpr int kMaxPerLane = 8;  // head_dim <= 512
  __shared__ float stage[4][512];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int heads = p.num_q_heads + p.num_k_heads + p.num_v_heads;
  const int64_t unit = (int64_t)blockIdx.x * 4 + wave;
  if (unit >= p.num_tokens * heads) return;
  const int64_t t = unit / heads;
  const int hh = (int)(unit - t * heads);
  const bool is_q = hh < p.num_q_heads;
  const bool is_v = hh >= p.num_q_heads + p.num_k_heads;
  const int D = p.head_dim;
  const int R = p.rotary_dim;
  const int64_t base = t * p.token_stride + (int64_t)hh * D;

  float x[kMaxPerLane];
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + 64 * i;
    x[i] = d < D ? Elem<DT>::load(p.qkv, base + d) : 0.0f;
  }

  if (!is_v) {
    const void* w = is_q ? p.q_weight : p.k_weight;
    if (w != nullptr) {
      float ss = 0.0f;
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) ss += x[i] * x[i];
      ss = wave_sum(ss);
      const float rms = 1.0f / sqrtf(ss / (float)D + p.eps);
#pragma unroll
      for (int i = 0; i < kMaxPerLane; ++i) {
        const int d = lane + 64 * i;
        if (d < D) {
          x[i] *= rms * Elem<DT>::load(w, d);
          if (p.per_op) x[i] = rounded<DT>(x[i]);  // a separate norm layer hands over rounded values
        }
      }
    }
    // rotation
    float* mine = stage[wave];
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < D) mine[d] = x[i];
    }
    __builtin_amdgcn_wave_barrier();
    int64_t pos = p.positions_int32 ? (int64_t)((const int32_t*)p.positions)[t] : ((const int64_t*)p.positions)[t];
    pos = pos < 0 ? 0 : (pos >= p.max_position ? p.max_position - 1 : pos);  // never read outside the table
    const int half = R >> 1;
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < R) {
        int f, partner;
        bool first;  // this element is the x of its pair (else the y)
        if (p.interleave) {
          f = d >> 1;
          first = (d & 1) == 0;
          partner = d ^ 1;
        } else {
          first = d < half;
          f = first ? d : d - half;
          partner = first ? d + half : d - half;
        }
        float c = load_any(p.cos_sin, pos * R + f, p.cos_sin_dtype);
        float s = load_any(p.cos_sin, pos * R + half + f, p.cos_sin_dtype);
        const float a = x[i], b = mine[partner];
        if (p.per_op) {
          c = rounded<DT>(c);
          s = rounded<DT>(s);
          // x' = x cos - y sin ; y' = y cos + x sin, each product and the sum rounded
          const float ac = rounded<DT>(a * c), bs = rounded<DT>(b * s);
          x[i] = rounded<DT>(first ? ac - bs : ac + bs);
        } else {
          x[i] = first ? a * c - b * s : b * s + a * c;
        }
      }
    }
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < D) {
        Elem<DT>::store(p.qkv, base + d, x[i]);
        x[i] = rounded<DT>(x[i]);  // the cache receives what a reader of qkv would see
      }
    }
  }

  if (CACHE == kNoCache || is_q) return;
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t block = slot / p.block_size;
  const int64_t off = slot % p.block_size;
  const int h = is_v ? hh - p.num_q_heads - p.num_k_heads : hh - p.num_q_heads;
  const int64_t row = block * p.stride_block + (int64_t)h * p.stride_head + off * p.stride_slot;
  uint8_t* cache = is_v ? p.v_cache : p.k_cache;
  if (CACHE == kVerbatim) {
#pragma unroll
    for (int i = 0; i < kMaxPerLane; ++i) {
      const int d = lane + 64 * i;
      if (d < D) Elem<DT>::store(cache, row + d, x[i]);
    }
    return;
  }
  float amax = 0.0f;
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) amax = fmaxf(amax, fabsf(x[i]));
  amax = wave_max(amax);
  constexpr float kQmax = CACHE == kInt8 ? 127.0f : 448.0f;
  constexpr float kMinScale = CACHE == kInt8 ? FLT_EPSILON : 1.0f / (448.0f * 512.0f);
  const float scale = fmaxf(amax / kQmax, kMinScale);
#pragma unroll
  for (int i = 0; i < kMaxPerLane; ++i) {
    const int d = lane + 64 * i;
    if (d < D) {
      const float y = x[i] / scale;
      uint8_t q;
      if (CACHE == kInt8) {
        q = quantise_int8(y);
      } else {
        q = quantise_fp8_e4m3(y);
      }
      cache[row + d] = q;
    }
  }
  if (lane == 0) {
    float* sc = is_v ? p.v_scale : p.k_scale;
    sc[block * p.sc_stride_block + (int64_t)h * p.sc_stride_head + off * p.sc_stride_slot] = scale;
  }
}

// head_dim 128 with 2-byte elements: sixteen lanes per head, eight consecutive elements (16 bytes)
// per lane, four heads per wave.  The rotation partner of a lane's elements sits in the lane
// rotary_dim/16 further (NeoX pairs) or in the lane itself (interleaved pairs).  Same arithmetic as
// the general kernel except for the order in which the squares are summed.
template <int G>
__device__ inline float group_sum(float v) {  // over G consecutive lanes (G a power of two)
#pragma unroll
  for (int o = G / 2; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  return v;
}
template <int G>
__device__ inline float group_max(float v) {
#pragma unroll
  for (int o = G / 2; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}

template <int DT>
__device__ inline void unpack8(const u32x4 raw, float (&x)[8]) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const uint32_t w = raw[e >> 1];
    if (DT == XLLM_HIP_BF16) {
      x[e] = __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
    } else {
      x[e] = (float)__builtin_bit_cast(_Float16, (uint16_t)((e & 1) ? (w >> 16) : (w & 0xffffu)));
    }
  }
}
template <int DT>
__device__ inline u32x4 pack8(const float (&x)[8]) {
  u32x4 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t lo, hi;
    if (DT == XLLM_HIP_BF16) {
      lo = float_to_bf16_bits(x[2 * i]);
      hi = float_to_bf16_bits(x[2 * i + 1]);
    } else {
      lo = __builtin_bit_cast(uint16_t, (_Float16)x[2 * i]);
      hi = __builtin_bit_cast(uint16_t, (_Float16)x[2 * i + 1]);
    }
    r[i] = lo | (hi << 16);
  }
  return r;
}

// Eight consecutive cos (or sin) values starting at element `idx` of the table.
__device__ inline void load8_any(const void* p, int64_t idx, int dtype, float (&o)[8], int count) {
  if (dtype == XLLM_HIP_FP32) {
    const f32x4 a = *(const f32x4*)((const float*)p + idx);
    const f32x4 b = count > 4 ? *(const f32x4*)((const float*)p + idx + 4) : a;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] = a[e];
      o[4 + e] = b[e];
    }
  } else if (count > 4) {
    const u32x4 raw = *(const u32x4*)((const uint16_t*)p + idx);
    if (dtype == XLLM_HIP_BF16) {
      unpack8<XLLM_HIP_BF16>(raw, o);
    } else {
      unpack8<XLLM_HIP_FP16>(raw, o);
    }
  } else {
    const u32x2 r2 = *(const u32x2*)((const uint16_t*)p + idx);
    const u32x4 raw = {r2[0], r2[1], 0, 0};
    if (dtype == XLLM_HIP_BF16) {
      unpack8<XLLM_HIP_BF16>(raw, o);
    } else {
      unpack8<XLLM_HIP_FP16>(raw, o);
    }
  }
}

template <int DT, int CACHE>
__global__ void __launch_bounds__(256) rope_kv_write_d128_kernel(RopeParams p, int cache_vec_ok) {
  const int sub = threadIdx.x & 15;
  const int heads = p.num_q_heads + p.num_k_heads + p.num_v_heads;
  const int64_t unit = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool live = unit < p.num_tokens * heads;  // idle groups still take part in the shuffles
  const int64_t t = live ? unit / heads : 0;
  const int hh = live ? (int)(unit - t * heads) : 0;
  const bool is_q = hh < p.num_q_heads;
  const bool is_v = hh >= p.num_q_heads + p.num_k_heads;
  const int R = p.rotary_dim;
  const int64_t base = t * p.token_stride + (int64_t)hh * 128 + 8 * sub;

  float x[8];
  u32x4 raw = {0, 0, 0, 0};
  if (live) raw = *(const u32x4*)(p.qkv + base * 2);
  unpack8<DT>(raw, x);

  if (!is_v) {
    const void* w = is_q ? p.q_weight : p.k_weight;
    if (w != nullptr) {
      float ss = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += x[e] * x[e];
      ss = group_sum<16>(ss);
      const float rms = 1.0f / sqrtf(ss / 128.0f + p.eps);
      float wv[8];
      unpack8<DT>(*(const u32x4*)((const uint16_t*)w + 8 * sub), wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        x[e] *= rms * wv[e];
        if (p.per_op) x[e] = rounded<DT>(x[e]);
      }
    }
    int64_t pos = p.positions_int32 ? (int64_t)((const int32_t*)p.positions)[t] : ((const int64_t*)p.positions)[t];
    pos = pos < 0 ? 0 : (pos >= p.max_position ? p.max_position - 1 : pos);
    const int half = R >> 1;
    const int hl = R >> 4;  // lanes per half of the rotated range
    float y[8];             // rotation partners
    float c[8], sn[8];
    bool first[8];
    const bool rotates = 8 * sub < R;
    if (p.interleave) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y[e] = x[e ^ 1];
        first[e] = (e & 1) == 0;
      }
      float c4[8], s4[8];
      const int64_t f0 = pos * R + (rotates ? 4 * sub : 0);
      load8_any(p.cos_sin, f0, p.cos_sin_dtype, c4, 4);
      load8_any(p.cos_sin, f0 + half, p.cos_sin_dtype, s4, 4);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        c[e] = c4[e >> 1];
        sn[e] = s4[e >> 1];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y[e] = __shfl_xor(x[e], hl);
        first[e] = sub < hl;
      }
      const int fl = rotates ? (sub < hl ? sub : sub - hl) : 0;
      load8_any(p.cos_sin, pos * R + 8 * fl, p.cos_sin_dtype, c, 8);
      load8_any(p.cos_sin, pos * R + half + 8 * fl, p.cos_sin_dtype, sn, 8);
    }
    if (rotates) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float a = x[e], b = y[e];
        if (p.per_op) {
          const float cc = rounded<DT>(c[e]), ss2 = rounded<DT>(sn[e]);
          const float ac = rounded<DT>(a * cc), bs = rounded<DT>(b * ss2);
          x[e] = rounded<DT>(first[e] ? ac - bs : ac + bs);
        } else {
          x[e] = first[e] ? a * c[e] - b * sn[e] : b * sn[e] + a * c[e];
        }
      }
    }
    const u32x4 packed = pack8<DT>(x);
    if (live) *(u32x4*)(p.qkv + base * 2) = packed;
    unpack8<DT>(packed, x);  // the cache receives what a reader of qkv would see
  }

  if (CACHE == kNoCache) return;
  int64_t slot = -1;
  if (live && !is_q) slot = p.slots[t];
  const bool writes = slot >= 0 && slot < p.num_slots;
  const int64_t block = writes ? slot / p.block_size : 0;
  const int64_t off = writes ? slot % p.block_size : 0;
  const int h = is_v ? hh - p.num_q_heads - p.num_k_heads : hh - p.num_q_heads;
  const int64_t row = block * p.stride_block + (int64_t)h * p.stride_head + off * p.stride_slot + 8 * sub;
  uint8_t* cache = is_v ? p.v_cache : p.k_cache;
  if (CACHE == kVerbatim) {
    if (!writes) return;
    const u32x4 packed = is_v ? raw : pack8<DT>(x);  // value rows are copied bit for bit
    if (cache_vec_ok) {
      *(u32x4*)(cache + row * 2) = packed;
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) ((uint16_t*)cache)[row + e] = (uint16_t)(packed[e >> 1] >> (16 * (e & 1)));
    }
    return;
  }
  float amax = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[e]));
  amax = group_max<16>(amax);
  if (!writes) return;
  constexpr float kQmax = CACHE == kInt8 ? 127.0f : 448.0f;
  constexpr float kMinScale = CACHE == kInt8 ? FLT_EPSILON : 1.0f / (448.0f * 512.0f);
  const float scale = fmaxf(amax / kQmax, kMinScale);
  uint32_t q2[2] = {0, 0};
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float yv = x[e] / scale;
    uint32_t q;
    if (CACHE == kInt8) {
      q = quantise_int8(yv);
    } else {
      q = quantise_fp8_e4m3(yv);
    }
    q2[e >> 2] |= q << (8 * (e & 3));
  }
  if (cache_vec_ok) {
    *(u32x2*)(cache + row) = u32x2{q2[0], q2[1]};
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) cache[row + e] = (uint8_t)(q2[e >> 2] >> (8 * (e & 3)));
  }
  if (sub == 0) {
    float* sc = is_v ? p.v_scale : p.k_scale;
    sc[block * p.sc_stride_block + (int64_t)h * p.sc_stride_head + off * p.sc_stride_slot] = scale;
  }
}

template <int DT>
static void launch_rope_d128(int cache_kind, const RopeParams& p, int cache_vec_ok, unsigned grid, hipStream_t st) {
  switch (cache_kind) {
    case kNoCache:
      rope_kv_write_d128_kernel<DT, kNoCache><<<grid, 256, 0, st>>>(p, cache_vec_ok);
      break;
    case kVerbatim:
      rope_kv_write_d128_kernel<DT, kVerbatim><<<grid, 256, 0, st>>>(p, cache_vec_ok);
      break;
    case kInt8:
      rope_kv_write_d128_kernel<DT, kInt8><<<grid, 256, 0, st>>>(p, cache_vec_ok);
      break;
    default:
      rope_kv_write_d128_kernel<DT, kFp8><<<grid, 256, 0, st>>>(p, cache_vec_ok);
      break;
  }
}

template <int DT>
static void launch_rope(int cache_kind, const RopeParams& p, unsigned grid, hipStream_t st) {
  switch (cache_kind) {
    case kNoCache:
      rope_kv_write_kernel<DT, kNoCache><<<grid, 256, 0, st>>>(p);
      break;
    case kVerbatim:
      rope_kv_write_kernel<DT, kVerbatim><<<grid, 256, 0, st>>>(p);
      break;
    case kInt8:
      rope_kv_write_kernel<DT, kInt8><<<grid, 256, 0, st>>>(p);
      break;
    default:
      rope_kv_write_kernel<DT, kFp8><<<grid, 256, 0, st>>>(p);
      break;
  }
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" int xllm_hip_rope_kv_write(const xllm_hip_rope_args* a,
                                      const xllm_hip_kv_cache* cache,
                                      const int32_t* slot_mapping,
                                      xllm_hip_stream_t stream) {
  XLLM_HIP_REQUIRE(a != nullptr, "rope args are NULL");
  XLLM_HIP_REQUIRE(a->num_tokens >= 0, "num_tokens is negative");
  if (a->num_tokens == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(a->qkv != nullptr && a->cos_sin_cache != nullptr && a->positions != nullptr,
                   "qkv, cos_sin_cache or positions is NULL");
  XLLM_HIP_REQUIRE(a->dtype == XLLM_HIP_BF16 || a->dtype == XLLM_HIP_FP16 || a->dtype == XLLM_HIP_FP32,
                   "qkv must be BF16/FP16/FP32, got dtype %d", a->dtype);
  XLLM_HIP_REQUIRE(a->cos_sin_dtype == XLLM_HIP_BF16 || a->cos_sin_dtype == XLLM_HIP_FP16 ||
                       a->cos_sin_dtype == XLLM_HIP_FP32,
                   "cos_sin_cache must be BF16/FP16/FP32, got dtype %d", a->cos_sin_dtype);
  XLLM_HIP_REQUIRE(a->num_q_heads >= 0 && a->num_k_heads >= 0 && a->num_v_heads >= 0 &&
                       a->num_q_heads + a->num_k_heads + a->num_v_heads > 0,
                   "head counts must be non-negative and not all zero");
  XLLM_HIP_REQUIRE(a->head_dim > 0 && a->head_dim <= 512, "head_dim must be in 1..512, got %d", a->head_dim);
  XLLM_HIP_REQUIRE(a->rotary_dim >= 0 && a->rotary_dim <= a->head_dim && a->rotary_dim % 2 == 0,
                   "rotary_dim must be even and at most head_dim, got %d", a->rotary_dim);
  XLLM_HIP_REQUIRE(a->max_position > 0, "max_position must be positive");
  XLLM_HIP_REQUIRE((a->q_weight == nullptr) == (a->k_weight == nullptr), "q_weight and k_weight go together");
  const int64_t row = (int64_t)(a->num_q_heads + a->num_k_heads + a->num_v_heads) * a->head_dim;
  XLLM_HIP_REQUIRE(a->token_stride >= row, "token stride smaller than the heads it holds");

  RopeParams p{};
  p.qkv = (uint8_t*)a->qkv;
  p.q_weight = a->q_weight;
  p.k_weight = a->k_weight;
  p.cos_sin = a->cos_sin_cache;
  p.positions = a->positions;
  p.positions_int32 = a->positions_int32;
  p.token_stride = a->token_stride;
  p.num_tokens = a->num_tokens;
  p.max_position = a->max_position;
  p.num_q_heads = a->num_q_heads;
  p.num_k_heads = a->num_k_heads;
  p.num_v_heads = a->num_v_heads;
  p.head_dim = a->head_dim;
  p.rotary_dim = a->rotary_dim;
  p.cos_sin_dtype = a->cos_sin_dtype;
  p.interleave = a->interleave;
  p.per_op = a->round_each_op;
  p.eps = a->eps;

  int kind = kNoCache;
  if (cache != nullptr) {
    XLLM_HIP_REQUIRE(slot_mapping != nullptr, "a cache is given but slot_mapping is NULL");
    XLLM_HIP_REQUIRE(cache->k_cache != nullptr && cache->v_cache != nullptr, "k_cache or v_cache is NULL");
    XLLM_HIP_REQUIRE(cache->num_blocks > 0 && cache->block_size > 0, "cache sizes must be positive");
    XLLM_HIP_REQUIRE(cache->head_dim == a->head_dim && cache->num_kv_heads == a->num_k_heads &&
                         a->num_v_heads == a->num_k_heads,
                     "cache is [%d heads, dim %d], qkv holds %d k / %d v heads of dim %d", cache->num_kv_heads,
                     cache->head_dim, a->num_k_heads, a->num_v_heads, a->head_dim);
    XLLM_HIP_REQUIRE(cache->stride_block > 0 && cache->stride_head > 0 && cache->stride_slot > 0,
                     "cache strides must be positive");
    if (cache->dtype == XLLM_HIP_INT8 || cache->dtype == XLLM_HIP_FP8_E4M3) {
      XLLM_HIP_REQUIRE(cache->k_scale != nullptr && cache->v_scale != nullptr,
                       "a quantised cache needs k_scale and v_scale");
      kind = cache->dtype == XLLM_HIP_INT8 ? kInt8 : kFp8;
    } else {
      XLLM_HIP_REQUIRE(cache->dtype == a->dtype, "cache dtype %d differs from qkv dtype %d", cache->dtype, a->dtype);
      kind = kVerbatim;
    }
    p.slots = slot_mapping;
    p.k_cache = (uint8_t*)cache->k_cache;
    p.v_cache = (uint8_t*)cache->v_cache;
    p.k_scale = cache->k_scale;
    p.v_scale = cache->v_scale;
    p.stride_block = cache->stride_block;
    p.stride_head = cache->stride_head;
    p.stride_slot = cache->stride_slot;
    p.sc_stride_block = cache->scale_stride_block;
    p.sc_stride_head = cache->scale_stride_head;
    p.sc_stride_slot = cache->scale_stride_slot;
    p.num_slots = cache->num_blocks * cache->block_size;
    p.block_size = cache->block_size;
  }
  const int64_t units = a->num_tokens * (a->num_q_heads + a->num_k_heads + a->num_v_heads);
  XLLM_HIP_REQUIRE((units + 3) / 4 <= 0x7fffffff, "too many (token, head) pairs: %lld", (long long)units);
  hipStream_t st = (hipStream_t)stream;
  // The 16-lanes-per-head kernel: head_dim 128, 2-byte elements, rotary_dim a power of two from 16
  // (so that the rotation partner is a fixed lane away), everything it reads on 16-byte boundaries.
  // Whether it is used never depends on the cache, so a call with and one without a cache compute
  // identical values; a cache whose rows are not 16-byte aligned is written element by element.
  const int cs_eb = elem_bytes(a->cos_sin_dtype);
  const bool d128 = a->head_dim == 128 && (a->dtype == XLLM_HIP_BF16 || a->dtype == XLLM_HIP_FP16) &&
                    (a->rotary_dim == 16 || a->rotary_dim == 32 || a->rotary_dim == 64 || a->rotary_dim == 128) &&
                    (((uintptr_t)a->qkv | (uintptr_t)a->q_weight | (uintptr_t)a->k_weight |
                      (uintptr_t)a->cos_sin_cache) & 15) == 0 &&
                    a->token_stride % 8 == 0 && (a->rotary_dim / 2 * cs_eb) % (a->interleave ? 8 : 16) == 0 &&
                    (a->rotary_dim * cs_eb) % 16 == 0;
  if (d128) {
    int cache_vec_ok = 0;
    if (cache != nullptr) {
      const int ceb = elem_bytes(cache->dtype);
      const int need = ceb == 1 ? 8 : 16;  // bytes a lane stores at once
      cache_vec_ok = (((uintptr_t)cache->k_cache | (uintptr_t)cache->v_cache | (uintptr_t)(cache->stride_block * ceb) |
                       (uintptr_t)(cache->stride_head * ceb) | (uintptr_t)(cache->stride_slot * ceb)) &
                      (uintptr_t)(need - 1)) == 0;
    }
    XLLM_HIP_REQUIRE((units + 15) / 16 <= 0x7fffffff, "too many (token, head) pairs: %lld", (long long)units);
    const unsigned g16 = (unsigned)((units + 15) / 16);
    if (a->dtype == XLLM_HIP_BF16) {
      launch_rope_d128<XLLM_HIP_BF16>(kind, p, cache_vec_ok, g16, st);
    } else {
      launch_rope_d128<XLLM_HIP_FP16>(kind, p, cache_vec_ok, g16, st);
    }
    return check_launch("rope_kv_write_d128_kernel");
  }
  const unsigned grid = (unsigned)((units + 3) / 4);
  switch (a->dtype) {
    case XLLM_HIP_BF16:
      launch_rope<XLLM_HIP_BF16>(kind, p, grid, st);
      break;
    case XLLM_HIP_FP16:
      launch_rope<XLLM_HIP_FP16>(kind, p, grid, st);
      break;
    default:
      launch_rope<XLLM_HIP_FP32>(kind, p, grid, st);
      break;
  }
  return check_launch("rope_kv_write_kernel");
}
