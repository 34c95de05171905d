// Many query rows per kv head over a 16-bit cache, 256 rows per work item, through the 32x32x16 MFMA: the
// two-phase kernel of prefill_pingpong.h with half as many MFMA instructions per tile.
#pragma once

#include "prefill_pingpong.h"

namespace xllm_hip {

// Why the wider instruction.  A wave in its softmax phase shares its SIMD's issue slot with the wave in its matrix
// phase, and every MFMA that one issues takes about eight cycles of the slot whatever its size (two waves of a
// SIMD, 128 v_fma_f32 beside 32 v_mfma_f32_16x16x32: 794 cycles against 548 alone; beside the same work as 16
// v_mfma_f32_32x32x16: 668).  A 32-token tile against a wave's 32 query rows is 32 of the narrow MFMAs (two row
// tiles of 16) or 16 of the wide ones; the LDS traffic is the same.
//
// Layouts (lane l: n = l % 32, h = l / 32).  v_mfma_f32_32x32x16: A row l % 32 and B column l % 32, both with
// k = 8h .. 8h+7; D column n, rows 8(i / 4) + 4h + i % 4 for register i of 16.
//   S^T = K Q^T: A = K rows (tokens) of the LDS tile, 16-byte piece 2c + h of row n for chunk c of 16 elements;
//     B = the lane's query row, elements 16c + 8h .. +7, in registers for the whole item.  One accumulator: the lane
//     holds, of query row n, the scores of tokens 8(i / 4) + 4h + i % 4 — sixteen of the tile's 32, the other sixteen
//     being in lane l ^ 32.
//   O^T += V^T P^T, in two steps of 16 tokens: step s takes the weights of registers 8s .. 8s+7 as they lie (B:
//     k = 8h + e is token 8(2s + e / 4) + 4h + e % 4), and A = V^T through the transposing LDS read, which hands
//     lane i of a group of 16 the four tokens of one element: the group (l / 16) reads tokens 8j + 4h .. +3 for
//     j = 2s and 2s + 1 at elements 32dt + 16((l / 16) % 2) + i.  Four accumulators of 16 registers: O^T tile dt,
//     elements 32dt + 8(i / 4) + 4h + i % 4 of query row n.
// One query row per lane: the running maximum and the denominator are the lane's own (the two lanes of a row
// exchange their maxima once per tile, their partial denominators at the end), and the causal and window limits
// are per lane.
typedef __attribute__((ext_vector_type(16))) float f32x16;

template <bool F16>
struct WideMma {
  __device__ static inline f32x16 run(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <>
struct WideMma<true> {
  __device__ static inline f32x16 run(f16x8 a, f16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

template <int KV_DT>
struct WideRows {
  static_assert(!quant_of(KV_DT), "16-bit caches");
  typedef typename Mma<KV_DT>::Op Op;
  typedef f32x16 Scores;
  typedef Op Weights[2];

  Op qf[8];
  f32x16 acc[4];
  float m_run, l_run;
  int lim, lo;
  uint32_t k_off0;     // LDS offset of piece h of K row n        (chunk c: XOR c << 5)
  uint32_t v_off[4];   // LDS offsets of the transposing reads, token group j (tile dt: XOR dt << 6)
  int64_t out_off;     // element offset of the lane's output row (and of its elements 4h)
  int64_t lse_off;     // index of the row's log-sum-exp, or -1 for a lane without a row
  int h;

  __device__ inline void init(const DecodeParams& p, const Item& it, int row0, int lane) {
    const int n = lane & 31;
    h = lane >> 5;
    const int row = it.rg * p.rows_per_item + row0 + n;
    const bool valid = row < it.n * p.group;
    const int j = valid ? row / p.group : 0;
    const int gq = valid ? row - j * p.group : 0;
    lim = it.len - (it.n - 1 - j);
    lo = p.window_left >= 0 ? lim - 1 - p.window_left : 0;
    const int head = it.hk * p.group + gq;
    const uint16_t* qrow = (const uint16_t*)p.q + (int64_t)(it.q0 + j) * p.q_token_stride + (int64_t)head * 128;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      u32x4 raw = {0, 0, 0, 0};
      if (valid) raw = *(const u32x4*)(qrow + 16 * c + 8 * h);
      qf[c] = __builtin_bit_cast(Op, raw);
    }
    out_off = (int64_t)(it.q0 + j) * p.out_token_stride + (int64_t)head * 128 + 4 * h;
    lse_off = valid ? (int64_t)(it.q0 + j) * p.num_q_heads + head : -1;
    m_run = -INFINITY;
    l_run = 0.0f;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[dt][i] = 0.0f;
    }
    k_off0 = kLdsK + swz_k(n, h);
    const int i16 = lane & 15, half = (lane >> 4) & 1;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      v_off[g] = kLdsV + swz_v(8 * g + 4 * h + (i16 >> 2), 2 * half + ((i16 & 3) >> 1)) + (i16 & 1) * 8;
    }
  }

  // ---- S^T = K Q^T ----
  __device__ __forceinline__ Op k_fragment(const uint8_t* tile, int c) const {
    return *(const Op*)(tile + (k_off0 ^ (uint32_t)(c << 5)));
  }
  __device__ __forceinline__ void scores_step(int c, const Op& kf, Scores& s) const {
    s = WideMma<qf16_of(KV_DT)>::run(kf, qf[c], s);
  }
  // ---- V^T fragments and O^T += V^T P^T ----
  __device__ __forceinline__ Op v_fragment(const uint8_t* tile, int dt, int step) const {
    const s16x4 a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(tile + (v_off[2 * step] ^ (uint32_t)(dt << 6))));
    const s16x4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4*)(tile + (v_off[2 * step + 1] ^ (uint32_t)(dt << 6))));
    return __builtin_bit_cast(Op, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
  }
  __device__ __forceinline__ void accumulate_step(int dt, const Op& vf, const Op& w) { acc[dt] = WideMma<qf16_of(KV_DT)>::run(vf, w, acc[dt]); }

  // ---- softmax of the lane's sixteen scores ----
  __device__ static inline float pair_max(float v) {  // over the two lanes of a query row
    float a = v, b = v;
    lane_swap32(a, b);
    return max_of<true>(a, b);
  }
  __device__ __forceinline__ void rescale(float m_new) {
    const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    l_run *= alpha;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) acc[dt] *= alpha;
  }
  __device__ __forceinline__ void pack(const float (&e)[16], Weights& w) const {
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      const u32x4 pw = {Mma<KV_DT>::pack(e[8 * s], e[8 * s + 1]), Mma<KV_DT>::pack(e[8 * s + 2], e[8 * s + 3]),
                        Mma<KV_DT>::pack(e[8 * s + 4], e[8 * s + 5]), Mma<KV_DT>::pack(e[8 * s + 6], e[8 * s + 7])};
      w[s] = __builtin_bit_cast(Op, pw);
    }
  }
  // A tile every row sees in full.  The reference point of the exponents follows the running maximum lazily (see
  // RowTile::weights): whether any row's moves is asked first, and only then are new ones and the scaled accumulators
  // formed.
  __device__ __forceinline__ void plain_weights(const Scores& s, float scale, Weights& w) {
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) mt = fmaxf(mt, s[i]);
    mt = pair_max(mt) * scale;
    if (__builtin_amdgcn_ballot_w64(fmaxf(m_run, mt) > m_run + kLazyRescale) != 0) rescale(fmaxf(m_run, mt));
    const float m_safe = m_run == -INFINITY ? 0.0f : m_run;
    float e[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      e[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], scale, -m_safe));
      l_run += e[i];
    }
    pack(e, w);
  }
  // A tile at the causal edge, the sequence end or a window's lower edge: token tb + 8(i / 4) + 4h + i % 4.
  __device__ __forceinline__ void masked_weights(const Scores& s, int tb, float scale, Weights& w) {
    float x[16];
    float mt = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int tok = tb + 8 * (i >> 2) + 4 * h + (i & 3);
      x[i] = (tok < lim && tok >= lo) ? s[i] * scale : -INFINITY;
      mt = fmaxf(mt, x[i]);
    }
    mt = pair_max(mt);
    if (__builtin_amdgcn_ballot_w64(fmaxf(m_run, mt) > m_run + kLazyRescale) != 0) rescale(fmaxf(m_run, mt));
    const float m_safe = m_run == -INFINITY ? 0.0f : m_run;
    float e[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      e[i] = __builtin_amdgcn_exp2f(x[i] - m_safe);
      l_run += e[i];
    }
    pack(e, w);
  }

  // ---- end of the item: the rows are written as they are (a step of this many rows is never split) ----
  __device__ inline void finish(const DecodeParams& p) {
    float a = l_run, b = l_run;
    lane_swap32(a, b);
    const float l = a + b;
    if (lse_off < 0) return;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    if (p.lse != nullptr && h == 0) p.lse[lse_off] = l > 0.0f ? m_run + __builtin_amdgcn_logf(l) : -INFINITY;
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {  // elements 32dt + 8q + 4h .. +3
        const u32x2 o = {MmaOps<qf16_of(KV_DT)>::pack(acc[dt][4 * q] * inv, acc[dt][4 * q + 1] * inv),
                         MmaOps<qf16_of(KV_DT)>::pack(acc[dt][4 * q + 2] * inv, acc[dt][4 * q + 3] * inv)};
        *(u32x2*)((uint16_t*)p.out + out_off + 32 * dt + 8 * q) = o;
      }
    }
  }
};

template <int KV_DT>
__global__ void __launch_bounds__(512, 2) prefill_pingpong_wide_d128_kernel(DecodeParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t buf0[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf1[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf2[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf3[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf4[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf5[kPrefillTile];
  constexpr int kT = 32;
  constexpr int kNB = kPingPongBuffers;

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const bool late = wave >= 4;  // the group that runs one phase behind; waves w and w + 4 share a SIMD

  typedef WideRows<KV_DT> WR;
  typedef typename WR::Op Op;
  typedef typename WR::Scores Scores;
  typedef typename WR::Weights Weights;
  WR wr;
  wr.init(p, it, 32 * wave, lane);

  // What this wave's rows can see, and what every row of the item sees in full (see prefill_pingpong_d128_kernel).
  const int rows = it.n * p.group;
  const int r_first = it.rg * p.rows_per_item + 32 * wave;
  const bool has_rows = r_first < rows;
  const int r_last = min(r_first + 31, rows - 1);
  const int lim_first = it.len - (it.n - 1 - r_first / p.group);
  const int lim_last = has_rows ? it.len - (it.n - 1 - r_last / p.group) : 0;
  const int lo_first = p.window_left >= 0 ? lim_first - 1 - p.window_left : 0;
  const int lo_last = p.window_left >= 0 ? lim_last - 1 - p.window_left : 0;
  const int ri_first = it.rg * p.rows_per_item;
  const int lim_item = it.len - (it.n - 1 - ri_first / p.group);

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;
  int p1 = lim_item > w_begin ? (lim_item - w_begin) / kT : 0;
  p1 = p1 < iters ? p1 : iters;
  const int nfast = p1 >= 1 && p.window_left < 0 ? 1 + (p1 - 1) / kNB * kNB : 0;

  PingPongLoader<KV_DT, 1> ld;
  ld.init(p, wave, lane);
  const int mine = 4 * wave;

  auto buffer = [&](auto k) __attribute__((always_inline)) -> uint8_t* {
    constexpr int K = decltype(k)::value % kNB;
    if constexpr (K == 0) return buf0;
    if constexpr (K == 1) return buf1;
    if constexpr (K == 2) return buf2;
    if constexpr (K == 3) return buf3;
    if constexpr (K == 4) return buf4;
    return buf5;
  };
  auto barrier = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  Weights pf;  // the weights of the last pipelined tile: they wait for its V^T P^T in the next step
  Op vpre[2];  // ... with the first V fragments of that tile, read ahead of the step's barrier
  int blk = 0;

  // K Q^T of the tile in `cur`: eight chunks of 16 elements, the fragment of the next chunk on its way.
  auto scores_from = [&](const uint8_t* cur, Op (&kf)[2], Scores& s) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.0f;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if (c + 1 < 8) kf[(c + 1) & 1] = wr.k_fragment(cur, c + 1);
      wr.scores_step(c, kf[c & 1], s);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto scores = [&](const uint8_t* cur, Scores& s) __attribute__((always_inline)) {
    Op kf[2];
    kf[0] = wr.k_fragment(cur, 0);
    __builtin_amdgcn_sched_barrier(0);
    scores_from(cur, kf, s);
  };
  // O^T += V^T P^T with the V rows in `buf`: MFMA k = 0 .. 7 is (tile dt = k / 2, token step k % 2).  `pre`
  // (PRELOADED): the fragments of the first two, read before the step's barrier.  `then`: what to put in flight
  // with the last MFMAs.
  auto values_then = [&](const uint8_t* buf, const Weights& w, auto preloaded, const Op (&pre)[2], auto then) __attribute__((always_inline)) {
    Op vf[3];
#pragma unroll
    for (int k = 0; k < 2; ++k) vf[k] = decltype(preloaded)::value ? pre[k] : wr.v_fragment(buf, k >> 1, k & 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      if (k + 2 < 8) vf[(k + 2) % 3] = wr.v_fragment(buf, (k + 2) >> 1, (k + 2) & 1);
      if (k == 6) then();
      wr.accumulate_step(k >> 1, vf[k % 3], w[k & 1]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto values = [&](const uint8_t* buf, const Weights& w) __attribute__((always_inline)) {
    Op none[2];
    values_then(buf, w, std::false_type{}, none, [] {});
  };
  auto settle = [&](int tb, uint8_t* next) __attribute__((always_inline)) {
    blk = block_of_const(p, it, tb + (kNB - 1) * kT + mine);
    __builtin_amdgcn_s_waitcnt(0x0f76);  // vmcnt(6): the loads of three tiles may still be in flight
    if (tb + 2 * kT > it.len) ld.clear_tail(tb + kT, it.len, next);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  };

  auto whole = [&](auto ph, int i) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    uint8_t* cur = buffer(std::integral_constant<int, PH>{});
    const int tb = w_begin + i * kT;
    const bool visible = !(tb >= lim_last || tb + kT <= lo_first);
    Scores s;
    barrier();
    ld.issue(p, it, tb + (kNB - 2) * kT, blk, buffer(std::integral_constant<int, PH + kNB - 2>{}));
    if (visible) {
      XLLM_HIP_PINGPONG_SETPRIO(1);
      scores(cur, s);
      XLLM_HIP_PINGPONG_SETPRIO(0);
    }
    settle(tb, buffer(std::integral_constant<int, PH + 1>{}));
    barrier();
    if (visible) {
      Weights w;
      if (tb + kT > lim_first || tb < lo_last) {
        wr.masked_weights(s, tb, p.scale_log2, w);
      } else {
        wr.plain_weights(s, p.scale_log2, w);
      }
      values(cur, w);
    }
  };
  auto pipelined = [&](auto ph, auto first, int i) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    uint8_t* cur = buffer(std::integral_constant<int, PH>{});
    const int tb = w_begin + i * kT;
    Scores s;
    barrier();
    ld.issue(p, it, tb + (kNB - 2) * kT, blk, buffer(std::integral_constant<int, PH + kNB - 2>{}));
    XLLM_HIP_PINGPONG_SETPRIO(1);
    if constexpr (!decltype(first)::value) {
      Op kf[2];
      values_then(buffer(std::integral_constant<int, PH + kNB - 1>{}), pf, std::true_type{}, vpre,
                  [&]() __attribute__((always_inline)) { kf[0] = wr.k_fragment(cur, 0); });
      scores_from(cur, kf, s);
    } else {
      scores(cur, s);
    }
    XLLM_HIP_PINGPONG_SETPRIO(0);
    settle(tb, buffer(std::integral_constant<int, PH + 1>{}));
    barrier();
    wr.plain_weights(s, p.scale_log2, pf);
    __builtin_amdgcn_sched_barrier(0);
    vpre[0] = wr.v_fragment(cur, 0, 0);
    vpre[1] = wr.v_fragment(cur, 0, 1);
  };
  if (iters > 0) {
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the queries have arrived
    ld.issue(p, it, w_begin, block_of_const(p, it, w_begin + mine), buf0);
    ld.issue(p, it, w_begin + kT, block_of_const(p, it, w_begin + kT + mine), buf1);
    ld.issue(p, it, w_begin + 2 * kT, block_of_const(p, it, w_begin + 2 * kT + mine), buf2);
    ld.issue(p, it, w_begin + 3 * kT, block_of_const(p, it, w_begin + 3 * kT + mine), buf3);
    settle(w_begin - kT, buf0);
    if (late) barrier();
    int i = 0;
    if (nfast > 0) {
      pipelined(std::integral_constant<int, 0>{}, std::true_type{}, i);
      ++i;
      for (; i + kNB <= nfast; i += kNB) {
        pipelined(std::integral_constant<int, 1>{}, std::false_type{}, i);
        pipelined(std::integral_constant<int, 2>{}, std::false_type{}, i + 1);
        pipelined(std::integral_constant<int, 3>{}, std::false_type{}, i + 2);
        pipelined(std::integral_constant<int, 4>{}, std::false_type{}, i + 3);
        pipelined(std::integral_constant<int, 5>{}, std::false_type{}, i + 4);
        pipelined(std::integral_constant<int, 0>{}, std::false_type{}, i + 5);
      }
      values_then(buf0, pf, std::true_type{}, vpre, [] {});
    }
    if (nfast == 0) {
      whole(std::integral_constant<int, 0>{}, 0);
      i = 1;
    }
    while (i < iters) {
      whole(std::integral_constant<int, 1>{}, i);
      if (++i >= iters) break;
      whole(std::integral_constant<int, 2>{}, i);
      if (++i >= iters) break;
      whole(std::integral_constant<int, 3>{}, i);
      if (++i >= iters) break;
      whole(std::integral_constant<int, 4>{}, i);
      if (++i >= iters) break;
      whole(std::integral_constant<int, 5>{}, i);
      if (++i >= iters) break;
      whole(std::integral_constant<int, 0>{}, i);
      ++i;
    }
    if (!late) barrier();
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): nothing lands in LDS any more
  wr.finish(p);
}

}  // namespace xllm_hip
