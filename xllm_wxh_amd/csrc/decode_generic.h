// The generic decode kernel (any head_dim <= 256, any supported type) and the CSR -> block_table kernel.
#pragma once

#include "decode_item.h"
#include "device_utils.h"

#include <math.h>

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Generic kernel: any head_dim <= 256, any supported dtype.  One wave per work item, one query
// row at a time; lanes are tokens for q.k and head-dim columns for p.v.  Not tuned: it exists
// so that every shape the operators accept is served and as an independent device-side check.
// ---------------------------------------------------------------------------------

// q . k over one cache row for the lane's token: 16-byte pieces when the rows allow it.
template <int KV_DT>
__device__ inline float dot_row(const uint8_t* cache, int64_t row, const float* qs, int D, bool vec_ok) {
  float dot = 0.0f;
  constexpr int kPer = KV_DT == XLLM_HIP_FP32 ? 4 : (KV_DT == XLLM_HIP_BF16 || KV_DT == XLLM_HIP_FP16) ? 8 : 16;
  if (vec_ok) {
    const u32x4* src = (const u32x4*)(cache + row * (16 / kPer));
    for (int d = 0; d < D; d += kPer) {
      const u32x4 raw = src[d / kPer];
#pragma unroll
      for (int e = 0; e < kPer; ++e) {
        float x;
        if (KV_DT == XLLM_HIP_FP32) {
          x = __uint_as_float(raw[e]);
        } else if (KV_DT == XLLM_HIP_BF16) {
          x = __uint_as_float((e & 1) ? (raw[e >> 1] & 0xffff0000u) : (raw[e >> 1] << 16));
        } else if (KV_DT == XLLM_HIP_FP16) {
          const uint16_t h = (uint16_t)((e & 1) ? (raw[e >> 1] >> 16) : (raw[e >> 1] & 0xffffu));
          x = (float)__builtin_bit_cast(_Float16, h);
        } else if (KV_DT == XLLM_HIP_INT8) {
          x = (float)(int8_t)((raw[e >> 2] >> (8 * (e & 3))) & 0xffu);
        } else {
          x = fp8_e4m3_to_float((uint8_t)((raw[e >> 2] >> (8 * (e & 3))) & 0xffu));
        }
        dot += qs[d + e] * x;
      }
    }
  } else {
    for (int d = 0; d < D; ++d) dot += qs[d] * Elem<KV_DT>::load(cache, row + d);
  }
  return dot;
}

template <int Q_DT, int KV_DT>
__global__ void __launch_bounds__(64) decode_generic_kernel(DecodeParams p) {
  __shared__ __attribute__((aligned(16))) float qs[256];
  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;
  const int lane = threadIdx.x;
  const int D = p.head_dim;
  const float neg_inf = -INFINITY;
  const bool quant = KV_DT == XLLM_HIP_FP8_E4M3 || KV_DT == XLLM_HIP_INT8;
  const int nhq = p.n * p.num_q_heads;
  const int row_end = min(it.n * p.group, (it.rg + 1) * p.rows_per_item);
  const int eb = KV_DT == XLLM_HIP_FP32 ? 4 : (KV_DT == XLLM_HIP_BF16 || KV_DT == XLLM_HIP_FP16) ? 2 : 1;
  // rows start on 16-byte boundaries and hold whole 16-byte pieces
  const bool vec_ok = (((uintptr_t)p.k_cache | (uintptr_t)(p.stride_block * eb) | (uintptr_t)(p.stride_head * eb) |
                        (uintptr_t)(p.stride_slot * eb) | (uintptr_t)(D * eb)) & 15) == 0;

  for (int r = it.rg * p.rows_per_item; r < row_end; ++r) {
    const int j = r / p.group;
    const int gq = r - j * p.group;
    const int head = it.hk * p.group + gq;
    const int64_t qbase = (int64_t)(it.q0 + j) * p.q_token_stride + (int64_t)head * D;
    __syncthreads();
    for (int d = lane; d < D; d += 64) qs[d] = Elem<Q_DT>::load(p.q, qbase + d) * p.scale_log2;
    __syncthreads();
    const int lim = it.len - (it.n - 1 - j);
    const int lo = p.window_left >= 0 ? lim - 1 - p.window_left : 0;

    float m_run = neg_inf, l_run = 0.0f;
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int tb = it.t_begin; tb < it.t_end; tb += 64) {
      const int tok = tb + lane;
      const bool vis = tok < it.t_end && tok < lim && tok >= lo;
      float x = neg_inf;
      float vscale = 0.0f;
      int64_t vrow = 0;  // invisible tokens point at the start of the cache and carry weight 0
      if (vis) {
        int bi = tok >> p.log2_bs;
        const int64_t blk = block_in_cache(p, it.ids[bi]);
        const int slot = tok & (p.block_size - 1);
        const int64_t row = blk * p.stride_block + (int64_t)it.hk * p.stride_head + (int64_t)slot * p.stride_slot;
        float dot = dot_row<KV_DT>(p.k_cache, row, qs, D, vec_ok);
        if (quant) {
          const int64_t srow = blk * p.sc_stride_block + (int64_t)it.hk * p.sc_stride_head +
                               (int64_t)slot * p.sc_stride_slot;
          dot *= p.k_scale[srow];
          vscale = p.v_scale[srow];
        } else {
          vscale = 1.0f;
        }
        x = dot;
        vrow = row;
      }
      const float mt = wave_max(x);
      const float m_new = fmaxf(m_run, mt);
      const float m_safe = m_new == neg_inf ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
      const float e = __builtin_amdgcn_exp2f(x - m_safe);
      l_run = l_run * alpha + wave_sum(e);
      m_run = m_new;
      const float pw = e * vscale;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] *= alpha;
      // p . V: lanes are head-dim columns; four tokens per step keep several loads in flight.  A
      // weight of exactly 0 (masked token) must not meet a garbage value: its row is skipped by select.
      const int cnt = min(64, it.t_end - tb);
      for (int tt = 0; tt < cnt; tt += 4) {
        float pt[4];
        int64_t rw[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          pt[u] = __shfl(pw, tt + u);  // lanes beyond cnt carry weight 0 and row 0
          rw[u] = __shfl(vrow, tt + u);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = lane + 64 * i;
          if (d < D) {
            float v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = Elem<KV_DT>::load(p.v_cache, rw[u] + d);
#pragma unroll
            for (int u = 0; u < 4; ++u) o[i] += pt[u] != 0.0f ? pt[u] * v[u] : 0.0f;
          }
        }
      }
    }
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    const float lse2 = l_run > 0.0f ? m_run + __builtin_amdgcn_logf(l_run) : neg_inf;
    if (p.implicit_plan) {
      // A step that is never split (more query rows per kv head than a split serves): every item is a whole
      // sequence, so the row is final and no partial is written (the workspace then holds none).
      const int64_t tok = (int64_t)it.q0 + j;
      if (lane == 0 && p.lse != nullptr) p.lse[tok * p.num_q_heads + head] = lse2;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        if (d < D) Elem<Q_DT>::store(p.out, tok * p.out_token_stride + (int64_t)head * D + d, o[i] * inv);
      }
      continue;
    }
    const int64_t prow = (int64_t)it.sc * nhq + (int64_t)j * p.num_q_heads + head;
    if (lane == 0) p.partial_lse[prow] = lse2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < D) p.partial_out[prow * D + d] = o[i] * inv;
    }
  }
}

// ---------------------------------------------------------------------------------
// CSR -> block_table / seq_lens.
// ---------------------------------------------------------------------------------

__global__ void __launch_bounds__(256) csr_to_block_table_kernel(const int32_t* indptr,
                                                                 const int32_t* indices,
                                                                 const int32_t* last_page_len,
                                                                 int batch,
                                                                 int block_size,
                                                                 int32_t* table,
                                                                 int64_t table_stride,
                                                                 int max_blocks,
                                                                 int32_t* seq_lens) {
  const int b = blockIdx.x;
  if (b >= batch) return;
  const int begin = indptr[b];
  const int nb = indptr[b + 1] - begin;
  for (int i = threadIdx.x; i < max_blocks; i += blockDim.x) {
    table[(int64_t)b * table_stride + i] = i < nb ? indices[begin + i] : 0;
  }
  if (threadIdx.x == 0) seq_lens[b] = nb > 0 ? (nb - 1) * block_size + last_page_len[b] : 0;
}

}  // namespace xllm_hip
