// Many query rows per kv head over a 16-bit cache, 256 rows per work item: the two-phase ("ping-pong") form of
// prefill_mfma_d128_kernel.
#pragma once

#include "decode_mfma.h"

#include <type_traits>

namespace xllm_hip {

// A workgroup is eight waves and 256 query rows of one (sequence, kv head): wave w owns rows 32w .. 32w+31 as
// two row tiles, as in prefill_mfma_d128_kernel, and all eight walk the item's tokens over the same LDS tiles
// (global memory -> LDS directly, each wave four rows of K and of V per tile).  The eight waves are two to a
// SIMD, and what a wave does for a tile is two phases of about the same length that use different parts of the
// SIMD: the matrix phase (V^T P^T of the previous tile, then K Q^T of this one: 32 MFMAs fed from LDS) and the
// softmax phase (vector arithmetic only).  Waves 0-3 and waves 4-7 run these phases in opposite order — one
// group is in its matrix phase while the other is in its softmax phase — and a workgroup barrier at every
// phase change keeps them there, so that the two waves of a SIMD do not both wait for the same unit.  The
// second group starts one phase late (an extra barrier at its start, one at the first group's end).
//
// Phases and barriers.  Barrier number g of the workgroup: the first group passes 2t before the matrix phase of
// tile t and 2t+1 before its softmax phase; the second group 2t+1 and 2t+2.  Every wave waits for its own share
// of tile t+1 before the barrier that precedes its softmax phase of tile t, which for either group comes before
// any wave reads that tile.  Tile t's buffer is last read in the second group's matrix phase of tile t+1
// (its V rows), which ends before barrier 2t+4; a wave puts tile t+4 in flight into the buffer of tile t-2
// after the barrier before its matrix phase of tile t, i.e. after barrier 2t at the earliest.  Six buffers
// rotate; the loads of tiles t+2 .. t+4 are in flight while tile t+1 is waited for.
//
// The tiles every row of the item sees in full take the straight-line form above, six at a time (one per
// buffer, so that each LDS access names its buffer and the compiler can tell the loads in flight from the
// tile being read).  The others — the causal edge, the sequence end, a sliding window's lower edge, and up to
// five tiles that do not fill a group of six — take a form that keeps all three parts of a tile in one step
// (K Q^T in the matrix phase, softmax and V^T P^T in the other) and lets a wave skip a tile none of its rows
// sees; both forms pass the same barriers per tile.
// A wave in its matrix phase runs at a raised priority, so that its MFMAs are issued as soon as their operands
// are there rather than after the vector instructions of the SIMD's other wave.
#ifndef XLLM_HIP_PINGPONG_PRIO
#define XLLM_HIP_PINGPONG_PRIO 1
#endif
#if XLLM_HIP_PINGPONG_PRIO
#define XLLM_HIP_PINGPONG_SETPRIO(n) __builtin_amdgcn_s_setprio(n)
#else
#define XLLM_HIP_PINGPONG_SETPRIO(n) ((void)0)
#endif
// How the matrix phase reads its fragments (see the kernel).  XLLM_HIP_PP_ADDR_REGS: bit 0, the LDS offsets of the
// eight V fragments stay in registers; bit 1, those of the four K fragments do (otherwise they are formed anew
// for every read: two vector operations each, in a phase whose vector-issue slots the SIMD's other wave wants —
// 4 x 512 tokens on a 3584-token prefix: 147-150 us with none, 141 with either V or both).  XLLM_HIP_PP_VDEPTH /
// XLLM_HIP_PP_KDEPTH: V fragments / K chunks read ahead of the MFMAs that use them (3 or 4 and 2 measured the
// same as 2 and 1: the phase does not wait for LDS).
#ifndef XLLM_HIP_PP_ADDR_REGS
#define XLLM_HIP_PP_ADDR_REGS 3
#endif
#ifndef XLLM_HIP_PP_VDEPTH
#define XLLM_HIP_PP_VDEPTH 2
#endif
#ifndef XLLM_HIP_PP_KDEPTH
#define XLLM_HIP_PP_KDEPTH 1
#endif
constexpr int kPingPongRows = 256;
constexpr int kPingPongBuffers = 6;

template <int KV_DT, int TOK>
struct PingPongLoader {
  int wave, lane;
  uint32_t k_off, v_off;  // byte offset of the piece this lane fetches from the first of the wave's tokens
  int v_tok;              // ... and the token (within the wave's 4 * TOK) its V piece belongs to

  // The piece for position lane % 16 of row 4 * wave + lane / 16 of the tile: token (within the wave's 4 * TOK)
  // and byte offset.
  __device__ inline void piece(bool v, int& tok, int& byte) const {
    const int row4 = lane >> 4;
    const int row = 4 * wave + row4;
    const int pos = lane & 15;
    const int lp = v ? pos ^ (((row & 7) << 1) | ((row >> 3) & 1))  // see swz_v
                     : pos ^ (row & 15);                             // see swz_k
    constexpr int kPerTok = 16 / TOK;
    tok = row4 * TOK + lp / kPerTok;
    byte = (lp % kPerTok) * 16;
  }
  // The two offsets stay in registers of their own for the whole item: a register that addressed a load into LDS
  // may not be written again before that load has landed, so offsets formed anew for every tile would make
  // each tile wait for all the tiles in flight.
  __device__ inline void init(const DecodeParams& p, int wave_, int lane_) {
    wave = wave_;
    lane = lane_;
    int tok, byte;
    piece(false, tok, byte);
    k_off = (uint32_t)(tok * p.stride_slot * 2 + byte);
    piece(true, tok, byte);
    v_off = (uint32_t)(tok * p.stride_slot * 2 + byte);
    v_tok = tok;
  }
  // Loads of the wave's rows of the tile starting at token tb into `buf` (in flight on return): global memory ->
  // LDS, 16 bytes per lane, the wave's 64 pieces to consecutive LDS addresses from the one in M0.  Written as
  // asm so that the waits are this kernel's own (settle): the compiler, which cannot always tell which buffer a
  // load in flight writes, would otherwise put a wait for all of them in front of LDS reads.  (No "memory"
  // clobber, which brings those waits back: every read of a tile goes through an address the compiler cannot
  // see through — RowTile::opaque — and lies between the same two barriers as the wait for that tile, so no
  // read is merged with one of an earlier tile or moved ahead of its tile's arrival.)
  __device__ static inline void to_lds(const uint8_t* base, uint32_t offset, uint8_t* lds) {
    const uint32_t l = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)lds;
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(offset), "s"(base), "s"(l));
  }
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int blk, uint8_t* buf) const {
    const HalfBase b = half_base(p, it, tb + 4 * TOK * wave, blk);
    to_lds(p.k_cache + b.elem * 2, k_off, buf + kLdsK + 1024 * wave);
    to_lds(p.v_cache + b.elem * 2, v_off, buf + kLdsV + 1024 * wave);
  }
  // Zeros over the V pieces of tokens at or past the sequence end (after the loads have landed).
  __device__ inline void clear_tail(int tb, int len, uint8_t* buf) const {
    uint32_t z = 0;
    asm volatile("" : "+v"(z));  // made here, on the rare path, instead of living in registers through the loop
    if (tb + 4 * TOK * wave + v_tok >= len) *(u32x4*)(buf + kLdsV + 1024 * wave + lane * 16) = u32x4{z, z, z, z};
  }
};

template <int KV_DT, int TOK>
__global__ void __launch_bounds__(512, 2) prefill_pingpong_d128_kernel(DecodeParams p) {
  static_assert(!quant_of(KV_DT), "a 1-byte cache needs converting on the way into LDS");
  static_assert(TOK == 1, "head_dim 128: the scores and weights of a 64-token tile (head_dim 64) do not fit the registers");
  __shared__ __attribute__((aligned(16))) uint8_t buf0[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf1[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf2[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf3[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf4[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf5[kPrefillTile];
  __shared__ float lds_ml[8 * 16 * 2];
  constexpr int kT = 32 * TOK;  // tokens per tile
  constexpr int kNB = kPingPongBuffers;
  static_assert(2 * 16 * xch_row_bytes(TOK) <= kPrefillTile, "two waves' end-of-item exchanges must fit a tile buffer");

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  // The group that runs one phase behind.  Waves w and w + 4 of a workgroup share a SIMD.
  const bool late = (p.prefill_opts & 2) ? (wave & 1) != 0 : wave >= 4;

  typedef RowTile<KV_DT, TOK> RT;
  typedef typename RT::Op Op;
  RT rt[2];
  rt[0].init(p, it, 32 * wave, lane);
  rt[1].init(p, it, 32 * wave + 16, lane);

  // What this wave's rows can see (see prefill_mfma_d128_kernel), and what every row of the item sees in full.
  const int rows = it.n * p.group;
  const int r_first = it.rg * p.rows_per_item + 32 * wave;
  const bool has_rows = r_first < rows;
  const int r_last = min(r_first + 31, rows - 1);
  const int lim_first = it.len - (it.n - 1 - r_first / p.group);
  const int lim_last = has_rows ? it.len - (it.n - 1 - r_last / p.group) : 0;
  const int lo_first = p.window_left >= 0 ? lim_first - 1 - p.window_left : 0;
  const int lo_last = p.window_left >= 0 ? lim_last - 1 - p.window_left : 0;
  const int ri_first = it.rg * p.rows_per_item;
  const int lim_item = it.len - (it.n - 1 - ri_first / p.group);  // the item's first row sees the tokens below this

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;
  // tiles [0, nfast) take the straight-line form, nfast = 1 + 6k (none under a sliding window, whose lower edge
  // would put masked tiles in front of them)
  int p1 = lim_item > w_begin ? (lim_item - w_begin) / kT : 0;
  p1 = p1 < iters ? p1 : iters;
  const int nfast = p1 >= 1 && p.window_left < 0 ? 1 + (p1 - 1) / kNB * kNB : 0;

  PingPongLoader<KV_DT, TOK> ld;
  ld.init(p, wave, lane);
  const int mine = 4 * TOK * wave;  // first of the tokens this wave fetches, within a tile

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

  typedef typename RT::Scores Scores;
  typedef Op Weights[RT::kU];
  Weights pf0, pf1;  // the weights of the last pipelined tile: they wait for its V^T P^T in the next step
  Op vpre[XLLM_HIP_PP_VDEPTH];  // ... with the first V fragments of that tile, read ahead of the step's barrier
  int blk = 0;       // block id of this wave's rows of the tile that is put in flight next

  // Fragment reads run ahead of the MFMAs that use them: kVAhead head-dim tiles of V, kKAhead 32-element chunks
  // of K.  Nothing moves across the fences: the compiler would otherwise hoist a phase's 24 fragment reads to
  // its top and hold them all in registers.
  constexpr int kVAhead = XLLM_HIP_PP_VDEPTH, kKAhead = XLLM_HIP_PP_KDEPTH;
  auto frag_offset = [&](uint32_t v) __attribute__((always_inline)) { return (XLLM_HIP_PP_ADDR_REGS & 1) ? v : RT::opaque(v); };
  auto k_frag_offset = [&](uint32_t v) __attribute__((always_inline)) { return (XLLM_HIP_PP_ADDR_REGS & 2) ? v : RT::opaque(v); };
  auto k_fragments = [&](const uint8_t* cur, int c, Op (&kf)[2]) __attribute__((always_inline)) {
    const uint32_t ko = k_frag_offset(rt[0].k_off0) ^ (uint32_t)(c << 6);
    kf[0] = *(const Op*)(cur + ko);
    kf[1] = *(const Op*)(cur + ko + 4096);
  };
  // K Q^T of the tile in `cur` for both row tiles.  `kf`: the fragments of the first kKAhead chunks, already on their way.
  auto scores_from = [&](const uint8_t* cur, Op (&kf)[kKAhead + 1][2], Scores& s0, Scores& s1) __attribute__((always_inline)) {
    rt[0].scores_init(s0);
    rt[1].scores_init(s1);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (c + kKAhead < 4) k_fragments(cur, c + kKAhead, kf[(c + kKAhead) % (kKAhead + 1)]);
      rt[0].scores_step(c, kf[c % (kKAhead + 1)][0], kf[c % (kKAhead + 1)][1], s0);
      rt[1].scores_step(c, kf[c % (kKAhead + 1)][0], kf[c % (kKAhead + 1)][1], s1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto k_prologue = [&](const uint8_t* cur, Op (&kf)[kKAhead + 1][2]) __attribute__((always_inline)) {
#pragma unroll
    for (int c = 0; c < kKAhead; ++c) k_fragments(cur, c, kf[c]);
  };
  auto scores = [&](const uint8_t* cur, Scores& s0, Scores& s1) __attribute__((always_inline)) {
    Op kf[kKAhead + 1][2];
    k_prologue(cur, kf);
    __builtin_amdgcn_sched_barrier(0);
    scores_from(cur, kf, s0, s1);
  };
  // O^T += V^T P^T with the V rows in `buf`.  `then`: what to put in flight with the last tiles' MFMAs.
  // `pre` (PRELOADED): the fragments of the first kVAhead head-dim tiles, read before the step's barrier.
  auto values_then = [&](const uint8_t* buf, const Weights& w0, const Weights& w1, auto preloaded, const Op (&pre)[kVAhead],
                         auto then) __attribute__((always_inline)) {
    Op vf[kVAhead + 1];
#pragma unroll
    for (int dt = 0; dt < kVAhead; ++dt) {
      vf[dt] = decltype(preloaded)::value ? pre[dt] : rt[0].v_fragment(buf, dt, frag_offset(rt[0].v_off0));
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      if (dt + kVAhead < 8) vf[(dt + kVAhead) % (kVAhead + 1)] = rt[0].v_fragment(buf, dt + kVAhead, frag_offset(rt[0].v_off0));
      if (dt + kVAhead == 8) then();
      rt[0].template accumulate_step<false>(dt, vf[dt % (kVAhead + 1)], w0, 1.0f);
      rt[1].template accumulate_step<false>(dt, vf[dt % (kVAhead + 1)], w1, 1.0f);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto values = [&](const uint8_t* buf, const Weights& w0, const Weights& w1) __attribute__((always_inline)) {
    Op none[kVAhead];
    values_then(buf, w0, w1, std::false_type{}, none, [] {});
  };
  // The first V fragments of the tile in `buf`, put in flight ahead of the barrier behind which they are used.
  auto v_prologue = [&](const uint8_t* buf, Op (&pre)[kVAhead]) __attribute__((always_inline)) {
#pragma unroll
    for (int dt = 0; dt < kVAhead; ++dt) pre[dt] = rt[0].v_fragment(buf, dt, frag_offset(rt[0].v_off0));
  };
  // Softmax of both row tiles; the accumulators follow when a reference point moved (rare after the first tiles).
  auto weights = [&](auto masked, int tb, const Scores& s0, const Scores& s1, Weights& w0, Weights& w1) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked)::value;
    float kscl[RT::kN], lv[RT::kN], rvs[RT::kN];
    float alpha0, alpha1;
    const bool moved0 = rt[0].template softmax<MASKED>(s0, kscl, lv, rvs, tb, p.scale_log2, w0, alpha0);
    __builtin_amdgcn_sched_barrier(0);  // one softmax at a time: interleaving the two costs registers
    const bool moved1 = rt[1].template softmax<MASKED>(s1, kscl, lv, rvs, tb, p.scale_log2, w1, alpha1);
    if (moved0 || moved1) {  // (the factor of a tile whose maxima stayed is exactly 1)
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) {
        rt[0].acc[dt] *= alpha0;
        rt[1].acc[dt] *= alpha1;
      }
    }
  };
  // The same for a tile every row sees in full, with the common case — no reference point moves — as the straight
  // path: whether one moves is asked first (some row's tile maximum more than kLazyRescale above its reference
  // point: the condition of RowTile::weights), and only then are new reference points, factors and the scaled
  // accumulators formed.  Same operations on the same values as RowTile::softmax, so the same bits.
  auto plain_weights_of = [&](RT& r, const Scores& s, Weights& w) __attribute__((always_inline)) {
    static_assert(RT::kU == 1 && RT::kHalves == 2 && !RT::kQuant && !RT::kRowScale, "16-bit cache, head_dim 128");
    const float scale = p.scale_log2;
    float mt = -INFINITY;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) mt = fmaxf(mt, s[0][h][rr]);  // (a chain from -inf: the compiler forms three-input maxima)
    }
    mt = kg_max<true>(mt) * scale;
    if (__builtin_amdgcn_ballot_w64(fmaxf(r.m_run, mt) > r.m_run + kLazyRescale) != 0) {
      const float m_new = fmaxf(r.m_run, mt);
      const float m_safe = m_new == -INFINITY ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(r.m_run - m_safe);
      r.l_run *= alpha;
      r.m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) r.acc[dt] *= alpha;
    }
    const float m_safe = r.m_run == -INFINITY ? 0.0f : r.m_run;
    float e[8];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        e[4 * h + rr] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[0][h][rr], scale, -m_safe));
        r.l_run += e[4 * h + rr];
      }
    }
    const u32x4 pw = {Mma<KV_DT>::pack(e[0], e[1]), Mma<KV_DT>::pack(e[2], e[3]), Mma<KV_DT>::pack(e[4], e[5]),
                      Mma<KV_DT>::pack(e[6], e[7])};
    w[0] = __builtin_bit_cast(Op, pw);
  };
  auto plain_weights = [&](const Scores& s0, const Scores& s1, Weights& w0, Weights& w1) __attribute__((always_inline)) {
    plain_weights_of(rt[0], s0, w0);
    __builtin_amdgcn_sched_barrier(0);  // one softmax at a time: interleaving the two costs registers
    plain_weights_of(rt[1], s1, w1);
  };
  // Before the barrier that precedes a softmax phase: the block id for the loads issued after the next barrier
  // (a scalar load, which shares a counter with LDS: it is complete, and out of the way of the matrix phase's
  // LDS waits, when this returns), this wave's share of the next tile landed, its V rows past the sequence end zeroed.
  auto settle = [&](int tb, uint8_t* next) __attribute__((always_inline)) {
    blk = block_of_const(p, it, tb + (kNB - 1) * kT + mine);
    __builtin_amdgcn_s_waitcnt(0x0f76);  // vmcnt(6): the loads of three tiles may still be in flight
    if (tb + 2 * kT > it.len) ld.clear_tail(tb + kT, it.len, next);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  };

  // One tile, all of it in this step: K Q^T in the matrix phase; softmax and V^T P^T in the other.  (Scores and
  // weights are the step's own: nothing of a tile outlives its step here.)
  auto whole = [&](auto ph, int i) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    uint8_t* cur = buffer(std::integral_constant<int, PH>{});
    const int tb = w_begin + i * kT;
    const bool visible = !(tb >= lim_last || tb + kT <= lo_first);
    Scores s0, s1;
    barrier();
    ld.issue(p, it, tb + (kNB - 2) * kT, blk, buffer(std::integral_constant<int, PH + kNB - 2>{}));
    if (visible) {
      XLLM_HIP_PINGPONG_SETPRIO(1);
      scores(cur, s0, s1);
      XLLM_HIP_PINGPONG_SETPRIO(0);
    }
    settle(tb, buffer(std::integral_constant<int, PH + 1>{}));
    barrier();
    if (visible) {
      Weights w0, w1;
      if (tb + kT > lim_first || tb < lo_last) {
        weights(std::true_type{}, tb, s0, s1, w0, w1);
      } else {
        plain_weights(s0, s1, w0, w1);
      }
      values(cur, w0, w1);
    }
  };
  // A tile every row sees in full, after another such tile: V^T P^T of that one, K Q^T of this one, then the softmax.
  auto pipelined = [&](auto ph, auto first, int i) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    uint8_t* cur = buffer(std::integral_constant<int, PH>{});
    const int tb = w_begin + i * kT;
    Scores s0, s1;
    barrier();
    ld.issue(p, it, tb + (kNB - 2) * kT, blk, buffer(std::integral_constant<int, PH + kNB - 2>{}));
    XLLM_HIP_PINGPONG_SETPRIO(1);
    if constexpr (!decltype(first)::value) {
      Op kf[kKAhead + 1][2];
      values_then(buffer(std::integral_constant<int, PH + kNB - 1>{}), pf0, pf1, std::true_type{}, vpre,
                  [&]() __attribute__((always_inline)) { k_prologue(cur, kf); });
      scores_from(cur, kf, s0, s1);
    } else {
      scores(cur, s0, s1);
    }
    XLLM_HIP_PINGPONG_SETPRIO(0);
    settle(tb, buffer(std::integral_constant<int, PH + 1>{}));
    barrier();
    plain_weights(s0, s1, pf0, pf1);
    __builtin_amdgcn_sched_barrier(0);
    v_prologue(cur, vpre);  // (this tile's V rows have been in LDS since before its matrix phase)
  };
  if (iters > 0) {  // (an item without visible tokens touches no block: its table row may hold anything)
    // The queries have arrived (they are needed at once; and the compiler, which does not count the tile loads,
    // would otherwise carry a wait for them into every loop below)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    ld.issue(p, it, w_begin, block_of_const(p, it, w_begin + mine), buf0);
    ld.issue(p, it, w_begin + kT, block_of_const(p, it, w_begin + kT + mine), buf1);
    ld.issue(p, it, w_begin + 2 * kT, block_of_const(p, it, w_begin + 2 * kT + mine), buf2);
    ld.issue(p, it, w_begin + 3 * kT, block_of_const(p, it, w_begin + 3 * kT + mine), buf3);
    settle(w_begin - kT, buf0);  // tile 0 landed; the block id of tile 4
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
      values_then(buf0, pf0, pf1, std::true_type{}, vpre, [] {});  // the last pipelined tile's V^T P^T: that tile is in the first buffer
    }
    // The other tiles, from the second buffer on (or from the first, when no tile took the straight-line form),
    // again one step per buffer, so that what is in flight at each step is the same on every path to it.
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
  __syncthreads();  // all tiles consumed: the buffers become the exchange
  uint8_t* xch = (wave < 2 ? buf0 : wave < 4 ? buf1 : wave < 6 ? buf2 : buf3) + (wave & 1) * (16 * xch_row_bytes(TOK));
  finish_item<KV_DT, TOK, 1>(p, it, rt[0], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave);
  __syncthreads();
  finish_item<KV_DT, TOK, 1>(p, it, rt[1], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave + 1);
}

// The same over a 1-byte cache (head_dim 128): the two-phase form of prefill_quant_d128_kernel.  A tile's bytes go
// from global memory straight into a raw LDS buffer (one 16-byte load per lane and tile: lanes 0-31 the wave's four
// rows of K, lanes 32-63 its four rows of V; one 4-byte load for their fp32 scales), four raw buffers rotate, and
// the wave that fetched them converts them — it reads back exactly the bytes it fetched — into one of three
// converted tiles in the layout the MFMA operand reads expect, with the per-token factors of the softmax (see
// QuantPrefillLoader::convert).  The conversion is vector work and belongs to the softmax phase: in the softmax
// phase of tile t the first group converts its rows of tile t + 1, the second group, whose matrix phase of that
// tile comes a phase later but whose softmax phase of tile t comes after the first group has begun to read it,
// those of tile t + 2.  Tile t + 1 is thus whole before barrier 2t + 2, behind which it is first read, and its
// buffer's last occupant, tile t - 2, was last read before barrier 2t.  The three converted tiles are one LDS
// array and the loop is unrolled over them: their offsets are immediates of the LDS instructions.
constexpr int kPingPongRawTile = 8 * (1024 + 256);  // per wave: 512 bytes of K, 512 of V, a 256-byte scale load

template <int KV_DT>
struct PingPongQuantLoader {
  int wave, lane;
  uint32_t kv_off;  // byte offset of this lane's 16 bytes from the first of the wave's rows (K and V alike)
  uint32_t sc_off;  // byte offset of this lane's scale from the scale of the wave's first token

  // Row (of the wave's four) and 16-byte chunk of the row that this lane fetches and converts: lanes in quads, as
  // in QuantPrefillLoader::row_chunk.  (Formed where they are used: two registers fewer through the loop.)
  __device__ inline void row_chunk(int& row4, int& chunk) const {
    const int l5 = RowTile<KV_DT, 1>::opaque(lane) & 31;
    chunk = 4 * ((l5 >> 3) & 1) + (l5 & 3);
    row4 = 2 * (l5 >> 4) + ((l5 >> 2) & 1);
  }
  __device__ inline void init(const DecodeParams& p, int wave_, int lane_) {
    wave = wave_;
    lane = lane_;
    int row4, chunk;
    row_chunk(row4, chunk);
    kv_off = (uint32_t)(row4 * p.stride_slot + chunk * 16);
    sc_off = (uint32_t)((lane & 3) * p.sc_stride_slot * 4);
  }
  // Loads of the wave's rows of the tile starting at token tb into `raw` (in flight on return).
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int blk, uint8_t* raw) const {
    const HalfBase b = half_base(p, it, tb + 4 * wave, blk);
    const uint8_t* kv = (lane < 32 ? p.k_cache : p.v_cache) + b.elem + kv_off;
    const uint8_t* sc = (const uint8_t*)(((lane & 4) ? p.v_scale : p.k_scale) + b.scale) + sc_off;
    const uint32_t l = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)(raw + 1280 * wave);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(kv), "s"(l));
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" : : "v"(sc), "s"(l + 1024));
  }
  // What a lane holds of a raw tile between reading it back and converting it.
  struct Raw {
    u32x4 bytes;  // its 16 bytes of a K or V row
    float sc;     // lanes 0-3: the K scales of the wave's four tokens, lanes 4-7: their V scales
    float kfac;   // the factor of the K scales (LDS_SCALE: it is kept in LDS, see the kernel)
  };
  template <bool LDS_SCALE>
  __device__ inline Raw fetch(const uint8_t* raw, float scale_log2, const float* lds_scale) const {
    Raw r;
    r.bytes = *(const u32x4*)(raw + 1280 * wave + lane * 16);
    r.sc = *(const float*)(raw + 1280 * wave + 1024 + (lane & 7) * 4);
    r.kfac = LDS_SCALE ? *lds_scale : scale_log2;
    return r;
  }
  // The wave's rows of the tile at tb: converted (K, V, per-token factors) into `conv`.  `dst`: where in a
  // converted tile this lane's two 16-byte pieces go (conv_offset; it depends on the lane alone and is kept in a
  // register: formed anew for every tile it was a third of the conversion's instructions).
  __device__ inline uint32_t conv_offset() const {
    int row4, chunk;
    row_chunk(row4, chunk);
    const int row = 4 * wave + row4;
    return lane >= 32 ? kLdsV + swz_v(row, 2 * chunk) : kLdsK + swz_k(row, 2 * chunk);
  }
  template <bool MASKED>
  __device__ inline void store(const Raw& rw, uint8_t* conv, uint32_t dst, int tb, int len) const {
    u32x4 lo, hi;
    dequant16<KV_DT>(rw.bytes, lo, hi);
    if constexpr (kv_of(KV_DT) == XLLM_HIP_INT8) {  // V rows: 1152 + x -> x, exact in fp16 (see QuantPrefillLoader::convert)
      const _Float16 sub = lane >= 32 ? (_Float16)kInt8Offset : (_Float16)0.0f;
      lo = __builtin_bit_cast(u32x4, __builtin_bit_cast(f16x8, lo) - sub);
      hi = __builtin_bit_cast(u32x4, __builtin_bit_cast(f16x8, hi) - sub);
    }
    if (MASKED && lane >= 32) {
      int row4, chunk;
      row_chunk(row4, chunk);
      if (tb + 4 * wave + row4 >= len) lo = hi = u32x4{0, 0, 0, 0};
    }
    *(u32x4*)(conv + dst) = lo;
    *(u32x4*)(conv + (dst ^ 16)) = hi;
    if (lane < 8) {
      const int t = 4 * wave + (lane & 3);  // token of the tile
      const bool is_v = lane >= 4;
      const float vs = fmaxf(rw.sc, 0x1p-100f);
      float a = is_v ? __builtin_amdgcn_logf(vs) : rw.sc * rw.kfac;
      float r = __builtin_amdgcn_rcpf(vs);
      if (MASKED && tb + t >= len) a = r = 0.0f;
      *(float*)(conv + kLdsSc + (is_v ? 128 : 0) + t * 4) = a;
      if (is_v) *(float*)(conv + kLdsSc + 256 + t * 4) = r;
    }
  }
};

template <int KV_DT>
__global__ void __launch_bounds__(512, 2) prefill_pingpong_quant_d128_kernel(DecodeParams p) {
  static_assert(quant_of(KV_DT), "16-bit caches need no conversion: prefill_pingpong_d128_kernel");
  constexpr int kT = 32, kConv = 3, kRaw = 4;
  __shared__ __attribute__((aligned(16))) uint8_t lds[kConv * kLdsTile + kRaw * kPingPongRawTile];
  __shared__ float lds_ml[8 * 16 * 2];
  __shared__ float lds_q[16];
  static_assert(8 * 16 * xch_row_bytes(1) <= kConv * kLdsTile + kRaw * kPingPongRawTile, "the end-of-item exchanges must fit");
  uint8_t* const raws = lds + kConv * kLdsTile;

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  const bool late = wave >= 4;  // the group that runs one phase behind; waves w and w + 4 share a SIMD

  typedef RowTile<KV_DT, 1, false, false, kv_of(KV_DT) == XLLM_HIP_INT8, false, false> RT;
  typedef typename RT::Op Op;
  RT rt[2];
  int q_exp = 0;
  if constexpr (RT::kNormItem) {  // one factor for the queries of all eight waves: they share the converted tile's factors
    lds_q[wave] = fmaxf(RT::wave_q_absmax(p, it, 32 * wave, lane), RT::wave_q_absmax(p, it, 32 * wave + 16, lane));
    __syncthreads();
    float m = lds_q[0];
#pragma unroll
    for (int i = 1; i < 8; ++i) m = fmaxf(m, lds_q[i]);
    q_exp = RT::norm_exponent(m);
    __syncthreads();
  }
  rt[0].init(p, it, 32 * wave, lane, q_exp);
  rt[1].init(p, it, 32 * wave + 16, lane, q_exp);
  // (the factor of the K scales waits in LDS, a word per wave: no scalar register need hold it through the loop)
  if constexpr (RT::kNormItem) lds_q[8 + wave] = __builtin_amdgcn_ldexpf(p.scale_log2, q_exp);
  const float* lds_scale = lds_q + 8 + wave;

  const int rows = it.n * p.group;
  const int r_first = it.rg * p.rows_per_item + 32 * wave;
  const bool has_rows = r_first < rows;
  const int r_last = min(r_first + 31, rows - 1);
  const int lim_first = it.len - (it.n - 1 - r_first / p.group);
  const int lim_last = has_rows ? it.len - (it.n - 1 - r_last / p.group) : 0;
  const int lo_first = p.window_left >= 0 ? lim_first - 1 - p.window_left : 0;
  const int lo_last = p.window_left >= 0 ? lim_last - 1 - p.window_left : 0;
  const int ri_first = it.rg * p.rows_per_item;
  const int lim_item = it.len - (it.n - 1 - ri_first / p.group);  // the item's first row sees the tokens below this

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;
  // tiles [0, nfast) take the straight-line form, nfast = 1 + 3k (none under a sliding window)
  int p1 = lim_item > w_begin ? (lim_item - w_begin) / kT : 0;
  p1 = p1 < iters ? p1 : iters;
  const int nfast = p1 >= 1 && p.window_left < 0 ? 1 + (p1 - 1) / kConv * kConv : 0;

  PingPongQuantLoader<KV_DT> ld;
  ld.init(p, wave, lane);
  const uint32_t conv_dst = ld.conv_offset();
  const int mine = 4 * wave;  // first of the tokens this wave fetches, within a tile

  auto barrier = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  auto conv_tile = [&](auto k) __attribute__((always_inline)) -> uint8_t* { return lds + (decltype(k)::value % kConv) * kLdsTile; };

  typedef typename RT::Scores Scores;
  typedef Op Weights[RT::kU];
  Weights pf0, pf1;
  Op vpre[2];
  int blk = 0;  // block id of this wave's rows of the tile that is put in flight next

  auto k_fragments = [&](const uint8_t* cur, int c, Op (&kf)[2]) __attribute__((always_inline)) {
    const uint32_t ko = RT::opaque(rt[0].k_off0) ^ (uint32_t)(c << 6);
    kf[0] = *(const Op*)(cur + ko);
    kf[1] = *(const Op*)(cur + ko + 4096);
  };
  auto scores_from = [&](const uint8_t* cur, Op (&kf)[2][2], Scores& s0, Scores& s1) __attribute__((always_inline)) {
    rt[0].scores_init(s0);
    rt[1].scores_init(s1);
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      if (c + 1 < 4) k_fragments(cur, c + 1, kf[(c + 1) & 1]);
      rt[0].scores_step(c, kf[c & 1][0], kf[c & 1][1], s0);
      rt[1].scores_step(c, kf[c & 1][0], kf[c & 1][1], s1);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto scores = [&](const uint8_t* cur, Scores& s0, Scores& s1) __attribute__((always_inline)) {
    Op kf[2][2];
    k_fragments(cur, 0, kf[0]);
    __builtin_amdgcn_sched_barrier(0);
    scores_from(cur, kf, s0, s1);
  };
  auto values_then = [&](const uint8_t* buf, const Weights& w0, const Weights& w1, auto preloaded, const Op (&pre)[2],
                         auto mid, auto then) __attribute__((always_inline)) {
    Op vf[3];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt) vf[dt] = decltype(preloaded)::value ? pre[dt] : rt[0].v_fragment(buf, dt, RT::opaque(rt[0].v_off0));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      if (dt + 2 < 8) vf[(dt + 2) % 3] = rt[0].v_fragment(buf, dt + 2, RT::opaque(rt[0].v_off0));
      if (dt == 2) mid();
      if (dt == 6) then();
      rt[0].template accumulate_step<false>(dt, vf[dt % 3], w0, 1.0f);
      rt[1].template accumulate_step<false>(dt, vf[dt % 3], w1, 1.0f);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto values = [&](const uint8_t* buf, const Weights& w0, const Weights& w1) __attribute__((always_inline)) {
    Op none[2];
    values_then(buf, w0, w1, std::false_type{}, none, [] {}, [] {});
  };
  // Softmax of both row tiles over the converted tile `cur`, whose factors of the K scales and logarithms of the V
  // scales the caller has read (`kscl`, `lv`; the reciprocals of the V scales are read here, ahead of the
  // arithmetic that hides their latency); the accumulators follow when a reference point moved.
  auto weights_with = [&](auto masked, const uint8_t* cur, int tb, const Scores& s0, const Scores& s1, const float (&kscl)[RT::kN],
                          const float (&lv)[RT::kN], Weights& w0, Weights& w1) __attribute__((always_inline)) {
    constexpr bool MASKED = decltype(masked)::value;
    float rvs[RT::kN];
    float x0[RT::kN], x1[RT::kN];
    float alpha0, alpha1;
    rt[0].load_factor(cur, 2, rvs);
    rt[0].template scaled_scores<MASKED>(s0, kscl, lv, tb, p.scale_log2, x0);
    rt[1].template scaled_scores<MASKED>(s1, kscl, lv, tb, p.scale_log2, x1);
    __builtin_amdgcn_sched_barrier(0);
    const bool moved0 = rt[0].template weights<MASKED>(x0, rvs, p.scale_log2, w0, alpha0);
    __builtin_amdgcn_sched_barrier(0);
    const bool moved1 = rt[1].template weights<MASKED>(x1, rvs, p.scale_log2, w1, alpha1);
    if (moved0 || moved1) {
#pragma unroll
      for (int dt = 0; dt < 8; ++dt) {
        rt[0].acc[dt] *= alpha0;
        rt[1].acc[dt] *= alpha1;
      }
    }
  };
  auto weights = [&](auto masked, const uint8_t* cur, int tb, const Scores& s0, const Scores& s1, Weights& w0, Weights& w1)
      __attribute__((always_inline)) {
    float kscl[RT::kN], lv[RT::kN];
    rt[0].load_factor(cur, 0, kscl);
    rt[0].load_factor(cur, 1, lv);
    weights_with(masked, cur, tb, s0, s1, kscl, lv, w0, w1);
  };
  // In the matrix phase of tile i a wave converts its rows of tile i + 1.  fetch_next, right behind the phase's
  // barrier: they have landed (the loads of three tiles may still be in flight) and are on their way from the raw
  // buffer to registers.  store_next, among the phase's MFMAs: converted and written, and the raw buffer takes
  // the tile four further on.  (`ph`: i modulo the number of converted tiles.)
  typedef typename PingPongQuantLoader<KV_DT>::Raw Raw;
  auto fetch_next = [&](int i) __attribute__((always_inline)) -> Raw {
    __builtin_amdgcn_s_waitcnt(0x0f76);  // vmcnt(6)
    return ld.template fetch<RT::kNormItem>(raws + ((i + 1) & (kRaw - 1)) * kPingPongRawTile, p.scale_log2, lds_scale);
  };
  auto store_next = [&](auto ph, int i, const Raw& rw) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    const int tb = w_begin + (i + 1) * kT;
    uint8_t* conv = lds + ((PH + 1) % kConv) * kLdsTile;
    if (tb + kT > it.len) {
      ld.template store<true>(rw, conv, conv_dst, tb, it.len);
    } else {
      ld.template store<false>(rw, conv, conv_dst, tb, it.len);
    }
    __builtin_amdgcn_sched_barrier(0);  // (the raw bytes are in registers: their buffer may be written)
    ld.issue(p, it, tb + kRaw * kT, blk, raws + ((i + 1) & (kRaw - 1)) * kPingPongRawTile);
  };
  // The block id for the loads that the matrix phase of tile i issues (tile i + 5): a scalar load, which shares a
  // counter with LDS, so it is made where a wait for it delays nothing: ahead of the barrier before that phase.
  auto next_block = [&](int i) __attribute__((always_inline)) {
    blk = block_of_const(p, it, w_begin + (i + 1 + kRaw) * kT + mine);
  };

  auto whole = [&](auto ph, int i) __attribute__((always_inline)) {
    uint8_t* cur = conv_tile(ph);
    const int tb = w_begin + i * kT;
    const bool visible = !(tb >= lim_last || tb + kT <= lo_first);
    Scores s0, s1;
    barrier();
    const Raw rw = fetch_next(i);
    if (visible) {
      XLLM_HIP_PINGPONG_SETPRIO(1);
      scores(cur, s0, s1);
      XLLM_HIP_PINGPONG_SETPRIO(0);
    }
    store_next(ph, i, rw);
    barrier();
    if (visible) {
      Weights w0, w1;
      if (tb + kT > lim_first || tb < lo_last) {
        weights(std::true_type{}, cur, tb, s0, s1, w0, w1);
      } else {
        weights(std::false_type{}, cur, tb, s0, s1, w0, w1);
      }
      values(cur, w0, w1);
    }
    next_block(i + 1);
  };
  auto pipelined = [&](auto ph, auto first, int i) __attribute__((always_inline)) {
    constexpr int PH = decltype(ph)::value;
    uint8_t* cur = conv_tile(ph);
    const int tb = w_begin + i * kT;
    Scores s0, s1;
    barrier();
    const Raw rw = fetch_next(i);
    XLLM_HIP_PINGPONG_SETPRIO(1);
    if constexpr (!decltype(first)::value) {
      Op kf[2][2];
      values_then(conv_tile(std::integral_constant<int, PH + kConv - 1>{}), pf0, pf1, std::true_type{}, vpre,
                  [&]() __attribute__((always_inline)) { store_next(ph, i, rw); },
                  [&]() __attribute__((always_inline)) { k_fragments(cur, 0, kf[0]); });
      scores_from(cur, kf, s0, s1);
    } else {
      store_next(ph, i, rw);
      scores(cur, s0, s1);
    }
    float kscl[RT::kN], lv[RT::kN];  // on their way across the barrier
    rt[0].load_factor(cur, 0, kscl);
    rt[0].load_factor(cur, 1, lv);
    XLLM_HIP_PINGPONG_SETPRIO(0);
    barrier();
    weights_with(std::false_type{}, cur, tb, s0, s1, kscl, lv, pf0, pf1);
    __builtin_amdgcn_sched_barrier(0);
    vpre[0] = rt[0].v_fragment(cur, 0, RT::opaque(rt[0].v_off0));
    vpre[1] = rt[0].v_fragment(cur, 1, RT::opaque(rt[0].v_off0));
    next_block(i + 1);
    // (waited for here: behind the barrier it would make the first MFMA wait for the raw bytes' way to registers as well)
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
  };

  if (iters > 0) {  // (an item without visible tokens touches no block: its table row may hold anything)
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): the queries have arrived (see prefill_pingpong_d128_kernel)
    ld.issue(p, it, w_begin, block_of_const(p, it, w_begin + mine), raws);
    ld.issue(p, it, w_begin + kT, block_of_const(p, it, w_begin + kT + mine), raws + kPingPongRawTile);
    ld.issue(p, it, w_begin + 2 * kT, block_of_const(p, it, w_begin + 2 * kT + mine), raws + 2 * kPingPongRawTile);
    ld.issue(p, it, w_begin + 3 * kT, block_of_const(p, it, w_begin + 3 * kT + mine), raws + 3 * kPingPongRawTile);
    // tile 0 is converted before the first barrier (fetch_next(i) and store_next(.., i, ..) handle tile i + 1)
    {
      next_block(-1);
      const Raw rw = fetch_next(-1);
      store_next(std::integral_constant<int, kConv - 1>{}, -1, rw);
      next_block(0);
    }
    if (late) barrier();
    int i = 0;
    if (nfast > 0) {
      pipelined(std::integral_constant<int, 0>{}, std::true_type{}, i);
      ++i;
      for (; i + kConv <= nfast; i += kConv) {
        pipelined(std::integral_constant<int, 1>{}, std::false_type{}, i);
        pipelined(std::integral_constant<int, 2>{}, std::false_type{}, i + 1);
        pipelined(std::integral_constant<int, 0>{}, std::false_type{}, i + 2);
      }
      values_then(lds, pf0, pf1, std::true_type{}, vpre, [] {}, [] {});  // the last pipelined tile's V^T P^T: that tile is in the first buffer
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
      whole(std::integral_constant<int, 0>{}, i);
      ++i;
    }
    if (!late) barrier();
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): nothing lands in LDS any more
  __syncthreads();  // all tiles consumed: the buffers become the exchange
  uint8_t* xch = lds + wave * (16 * xch_row_bytes(1));
  finish_item<KV_DT, 1, 1>(p, it, rt[0], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave);
  __syncthreads();
  finish_item<KV_DT, 1, 1>(p, it, rt[1], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave + 1);
}

}  // namespace xllm_hip
