// Merge of the partial results of split sequences: the merge kernel and the fused form the 16-row
// attention kernel calls.
#pragma once

#include "decode_item.h"
#include "device_utils.h"

#include <math.h>
#include <type_traits>

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Merge of the sequences that were split into several chunks:
//   out = sum_i 2^(lse_i - lse) * partial_i,   lse = log2 sum_i 2^lse_i
// One wave per output row.  First the row's log-sum-exps, one chunk per lane, give the maximum and
// the denominator by wave reductions; then the partials are summed with their weights, the lanes
// covering the row's columns and the loads of several chunks in flight at a time — a long sequence
// of a small batch has hundreds of chunks per row, and a chunk-by-chunk running maximum would
// serialise that many memory latencies.
// ---------------------------------------------------------------------------------

constexpr int kMergeRowsPerBlock = 4;

// Partials that another workgroup of the same launch wrote are stored and loaded as device-scope
// atomics (relaxed): such accesses go past the caches that are not coherent across the XCDs, so the
// fused merge needs no cache write-back or invalidation, only the ordering its barrier and counter give.
__device__ inline void store_coherent(float* ptr, float v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <bool COHERENT>
__device__ inline float load_partial(const float* ptr) {
  if (COHERENT) return __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return *ptr;
}

// One wave merges the partials of output row (sequence b, query token j, head): all 64 lanes call.
// COLS: columns per lane (2 covers head_dim <= 128, 4 head_dim <= 256).
// (P: DecodeParams, or DecodeParams qualified with the constant address space when the caller reads
// its arguments straight from the kernel-argument segment.)
// `known_chunks`: the sequence's chunk count if the caller has it (a work item carries it), else -1.
template <int Q_DT, bool COHERENT, int COLS, int MAXB = 32, class P>
__device__ inline void merge_row_cols(const P& p, int b, int j, int head, int q0, int lane, int known_chunks = -1) {
  const int nhq = p.n * p.num_q_heads;
  const int rem = j * p.num_q_heads + head;
  const int cnt = known_chunks >= 0 ? known_chunks : chunks_of_sequence(p, b);
  const int D = p.head_dim;
  const float neg_inf = -INFINITY;
  // slot of the sequence's chunk i: its full chunks are consecutive, its tail lies among the tails; or
  // (no stored schedule) the sequence owns arith_chunks consecutive slots
  const bool arith = p.arith_chunks > 0;
  const int f0 = arith ? (b < p.arith_whole ? b * p.arith_first
                                              : p.arith_whole * p.arith_first + (b - p.arith_whole) * p.arith_chunks)
                       : p.full_prefix[b];
  const int nf = arith ? cnt : p.full_prefix[b + 1] - f0;
  const int tail_slot = arith ? 0 : p.hdr->total_full + p.tail_prefix[b];
  auto partial_row = [&](int i) { return (int64_t)(i < nf ? f0 + i : tail_slot) * nhq + rem; };

  // Columns lane, lane + 64, ... of the output row, summed over the chunks a batch at a time: the
  // loads of a batch are all issued before the first is used.  `weight(i)` is chunk i's factor.
  float o[COLS];
#pragma unroll
  for (int k = 0; k < COLS; ++k) o[k] = 0.0f;
  auto load_rows = [&](int i0, auto unroll, float (&v)[decltype(unroll)::value][COLS]) {
#pragma unroll
    for (int u = 0; u < decltype(unroll)::value; ++u) {
      if (u == 0 || i0 + u < cnt) {  // (uniform over the wave)
        const float* po = p.partial_out + partial_row(i0 + u) * D;
#pragma unroll
        for (int k = 0; k < COLS; ++k) v[u][k] = lane + 64 * k < D ? load_partial<COHERENT>(po + lane + 64 * k) : 0.0f;
      } else {
#pragma unroll
        for (int k = 0; k < COLS; ++k) v[u][k] = 0.0f;
      }
    }
  };
  auto add_rows = [&](int i0, auto unroll, const float (&v)[decltype(unroll)::value][COLS], auto weight) {
#pragma unroll
    for (int u = 0; u < decltype(unroll)::value; ++u) {
      const float w = i0 + u < cnt ? weight(i0 + u) : 0.0f;
#pragma unroll
      // (an empty chunk's row may hold anything; the fused multiply-add is spelled out so that every
      // instantiation of this function rounds alike and the two merges give the same bits)
      for (int k = 0; k < COLS; ++k) o[k] = w != 0.0f ? __builtin_fmaf(w, v[u][k], o[k]) : o[k];
    }
  };
  float m, ssum;
  if (cnt <= 256) {
    // The usual case.  Each lane keeps the log-sum-exps of chunks lane, lane + 64, ... in registers, and
    // the partial rows (up to MAXB of them — 8 at head_dim 256 —, then further batches) are on their way
    // while the maximum and the denominator are reduced: one memory round trip for a row of up to
    // that many chunks — these loads go to memory past the caches when the merge is fused, at more
    // than a microsecond each way.
    float l[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int i = lane + 64 * q;
      l[q] = i < cnt ? load_partial<COHERENT>(p.partial_lse + partial_row(i)) : neg_inf;
    }
    auto reduce_lse = [&](float (&e)[4]) {
      m = wave_max(fmaxf(fmaxf(l[0], l[1]), fmaxf(l[2], l[3])));
      const float m_safe = m == neg_inf ? 0.0f : m;
#pragma unroll
      for (int q = 0; q < 4; ++q) e[q] = __builtin_amdgcn_exp2f(l[q] - m_safe);  // 2^-inf = 0: empty or absent chunk
      ssum = wave_sum(e[0] + e[1] + e[2] + e[3]);
    };
    auto run = [&](auto batch) {
      constexpr int kB = decltype(batch)::value;
      float first[kB][COLS];
      load_rows(0, batch, first);
      float e[4];
      reduce_lse(e);
      auto weight = [&](int i) {
        const int q = i >> 6;
        const float mine = q == 0 ? e[0] : q == 1 ? e[1] : q == 2 ? e[2] : e[3];
        return __shfl(mine, i & 63);
      };
      add_rows(0, batch, first, weight);
      for (int i0 = kB; i0 < cnt; i0 += kB) {
        float v[kB][COLS];
        load_rows(i0, batch, v);
        add_rows(i0, batch, v, weight);
      }
    };
    if (cnt <= 8 || COLS > 2) {
      run(std::integral_constant<int, 8>{});
    } else if (cnt <= 16 || MAXB <= 16) {
      run(std::integral_constant<int, 16>{});
    } else {
      run(std::integral_constant<int, 32>{});
    }
  } else {
    m = neg_inf;
    for (int i = lane; i < cnt; i += 64) m = fmaxf(m, load_partial<COHERENT>(p.partial_lse + partial_row(i)));
    m = wave_max(m);
    const float m_safe = m == neg_inf ? 0.0f : m;
    ssum = 0.0f;
    for (int i = lane; i < cnt; i += 64) {
      ssum += __builtin_amdgcn_exp2f(load_partial<COHERENT>(p.partial_lse + partial_row(i)) - m_safe);
    }
    ssum = wave_sum(ssum);
    auto weight = [&](int i) {
      return __builtin_amdgcn_exp2f(load_partial<COHERENT>(p.partial_lse + partial_row(i)) - m_safe);
    };
    typedef std::integral_constant<int, 4> Four;
    for (int i0 = 0; i0 < cnt; i0 += 4) {
      float v[4][COLS];
      load_rows(i0, Four{}, v);
      add_rows(i0, Four{}, v, weight);
    }
  }
  const float inv = ssum > 0.0f ? 1.0f / ssum : 0.0f;
  const int64_t tok = (int64_t)q0 + j;
  if (p.lse != nullptr && lane == 0) {
    p.lse[tok * p.num_q_heads + head] = ssum > 0.0f ? m + __builtin_amdgcn_logf(ssum) : neg_inf;
  }
  const int64_t obase = tok * p.out_token_stride + (int64_t)head * D;
#pragma unroll
  for (int k = 0; k < COLS; ++k) {
    const int d = lane + 64 * k;
    if (d < D) Elem<Q_DT>::store(p.out, obase + d, o[k] * inv);
  }
}

template <int Q_DT, bool COHERENT>
__device__ inline void merge_row(const DecodeParams& p, int b, int j, int head, int q0, int lane) {
  // (the merge kernel's form: up to 16 rows in flight and so few enough registers for six waves per SIMD —
  // its loads are ordinary cached ones, and a row per wave wants many waves resident)
  if (p.head_dim <= 128) {
    merge_row_cols<Q_DT, COHERENT, 2, 16>(p, b, j, head, q0, lane);
  } else {
    merge_row_cols<Q_DT, COHERENT, 4>(p, b, j, head, q0, lane);
  }
}

template <int Q_DT>
__global__ void __launch_bounds__(64 * kMergeRowsPerBlock, 6) decode_merge_kernel(DecodeParams p) {
  const int nhq = p.n * p.num_q_heads;
  const int64_t row = (int64_t)blockIdx.x * kMergeRowsPerBlock + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= (int64_t)p.batch * nhq) return;
  const int b = (int)(row / nhq);
  int q0 = b * p.n, nb = p.n;
  if (p.q_indptr != nullptr) {
    q0 = p.q_indptr[b];
    nb = min(p.n, p.q_indptr[b + 1] - q0);
  }
  if (p.direct_single && chunks_of_sequence(p, b) == 1) return;  // already written by the attention kernel
  const int rem = (int)(row - (int64_t)b * nhq);  // j * Hq + head
  const int j = rem / p.num_q_heads;
  if (j >= nb) return;
  merge_row<Q_DT, false>(p, b, j, rem - j * p.num_q_heads, q0, lane);
}

// Fused merge, called by every thread of a workgroup (wave `wave`, lane `lane` of it: passed in, so
// that the caller need not keep its thread index in a register through its token loop) after it has
// written the partials of its item:
// the workgroup that finishes the last chunk of a (sequence, kv head, row group) combines that row
// group's partials, so no merge kernel follows.  Every wave waits until its partial stores (coherent,
// see store_coherent) have completed, the workgroup meets, and one thread counts the chunk in with a
// device-scope atomic; the workgroup that reads count - 1 knows that every other chunk's stores
// completed before its increment, resets the counter for the next launch and reads the partials with
// coherent loads.  (Device-scope fences instead — cache write-back and invalidation on every
// workgroup — made an 8 x 8192-token step three times slower.)
template <int Q_DT, int COLS, int MAXB, class P>
__device__ inline void merge_if_last(const P& p, const Item& it, int* lds_flag, int wave, int lane) {
  if (!p.fused_merge || p.implicit_plan) return;
  const int cnt = it.chunks;
  if (p.direct_single && cnt == 1) return;  // written directly
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's stores have completed
  __syncthreads();
  if (wave == 0 && lane == 0) {
    int32_t* c = p.counters + ((int64_t)it.b * p.num_kv_heads + it.hk) * p.row_groups + it.rg;
    const int old = __hip_atomic_fetch_add(c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const int last = old == cnt - 1;
    if (last) __hip_atomic_store(c, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *lds_flag = last;
  }
  __syncthreads();
  if (!*lds_flag) return;
  const int nwaves = blockDim.x >> 6;
  const int first = it.rg * p.rows_per_item;
  const int end = min(first + p.rows_per_item, it.n * p.group);
  for (int r = first + wave; r < end; r += nwaves) {
    const int j = r / p.group;
    merge_row_cols<Q_DT, true, COLS, MAXB>(p, it.b, j, it.hk * p.group + (r - j * p.group), it.q0, lane, cnt);
  }
}

}  // namespace xllm_hip
