// Device-side helpers shared by the gfx950 KV-write and paged-decode kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/xllm_hip_paged_kv.h"

namespace xllm_hip {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;

constexpr int kWave = 64;

__host__ __device__ inline int elem_bytes(int dtype) {
  switch (dtype) {
    case XLLM_HIP_BF16:
    case XLLM_HIP_FP16:
      return 2;
    case XLLM_HIP_FP32:
      return 4;
    case XLLM_HIP_FP8_E4M3:
    case XLLM_HIP_INT8:
      return 1;
    default:
      return 0;
  }
}

// ---- scalar element <-> float -------------------------------------------------

__device__ inline float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// Round-to-nearest-even float -> bf16 bits (NaN stays NaN): gfx950 converts in hardware
// (v_cvt_pk_bf16_f32), an eighth of the instructions of the integer form.
__device__ inline uint16_t float_to_bf16_bits(float f) {
  const __bf16 h = (__bf16)f;
  return __builtin_bit_cast(uint16_t, h);
}

__device__ inline float fp8_e4m3_to_float(uint8_t b) {
  f32x2 r = __builtin_amdgcn_cvt_pk_f32_fp8((int)b, false);
  return r[0];
}

template <int DT>
struct Elem;  // load(ptr, i) -> float ; store(ptr, i, float)

template <>
struct Elem<XLLM_HIP_BF16> {
  typedef uint16_t T;
  __device__ static float load(const void* p, int64_t i) {
    return bf16_bits_to_float(((const uint16_t*)p)[i]);
  }
  __device__ static void store(void* p, int64_t i, float v) {
    ((uint16_t*)p)[i] = float_to_bf16_bits(v);
  }
};
template <>
struct Elem<XLLM_HIP_FP16> {
  typedef uint16_t T;
  __device__ static float load(const void* p, int64_t i) {
    return (float)(((const _Float16*)p)[i]);
  }
  __device__ static void store(void* p, int64_t i, float v) {
    ((_Float16*)p)[i] = (_Float16)v;
  }
};
template <>
struct Elem<XLLM_HIP_FP32> {
  typedef float T;
  __device__ static float load(const void* p, int64_t i) { return ((const float*)p)[i]; }
  __device__ static void store(void* p, int64_t i, float v) { ((float*)p)[i] = v; }
};
template <>
struct Elem<XLLM_HIP_FP8_E4M3> {
  typedef uint8_t T;
  __device__ static float load(const void* p, int64_t i) {
    return fp8_e4m3_to_float(((const uint8_t*)p)[i]);
  }
};
template <>
struct Elem<XLLM_HIP_INT8> {
  typedef int8_t T;
  __device__ static float load(const void* p, int64_t i) {
    return (float)(((const int8_t*)p)[i]);
  }
};

// ---- saturating quantisers of the KV writes ------------------------------------------------------
// clamp(y, -m, m) = fmaxf(-m, fminf(y, m)), the order of xllm/core/kernels/cuda/fp8_quant_utils.cuh:121-122:
// fminf / fmaxf return their other operand for a NaN, so a NaN (a NaN element, or inf / inf in a row
// that holds an infinity) becomes +m.  The NaN case is spelled out because the compiler may fuse the
// two operations into one median instruction, which answers a NaN with the smallest operand.

// Round half to even, saturate to +-127.
__device__ inline uint8_t quantise_int8(float y) {
  const float r = y != y ? 127.0f : fmaxf(-127.0f, fminf(rintf(y), 127.0f));
  return (uint8_t)(int8_t)(int)r;
}

// Saturating round-to-nearest-even float -> OCP e4m3fn byte.
__device__ inline uint8_t quantise_fp8_e4m3(float y) {
  y = y != y ? 448.0f : fmaxf(-448.0f, fminf(y, 448.0f));
  const int packed = __builtin_amdgcn_cvt_pk_fp8_f32(y, y, 0, false);
  return (uint8_t)(packed & 0xff);
}

// ---- wave-level reductions ------------------------------------------------------

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

}  // namespace xllm_hip
