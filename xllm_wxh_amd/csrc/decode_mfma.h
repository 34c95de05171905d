// The MFMA attention kernels of the decode path (16-row, 32-row and 128-row forms).
#pragma once

#include "decode_item.h"
#include "decode_merge.h"
#include "device_utils.h"

#include <math.h>
#include <type_traits>

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// MFMA kernels, head_dim 128, bf16 or fp16 queries.  One workgroup per work item.
//
// A tile is 32 tokens.  Its K and V rows are fetched with fully coalesced 16-byte loads, parked
// in LDS (row-major, 16-byte pieces XOR-swizzled by row so that every access pattern below is
// bank-conflict free) and read back in MFMA operand order:
//   S^T[t][r]  = sum_d K[t][d] Q[r][d]      A = K tile (ds_read_b128), B = Q^T (registers)
//   O^T[d][r] += sum_t V[t][d] P[r][t]      A = V^T tile (ds_read_b64_tr_b16), B = P^T (registers)
// Computing the transposed products keeps a query row in one lane column for both MFMAs, so the
// probabilities leave the first MFMA already laid out as the second one's B operand and the
// softmax statistics are per-lane scalars.  Query rows r = j*g + gq (draft token j, head gq of
// the group) fill the 16 columns of an MFMA tile; a wave owns one such tile of rows.
//
// decode_mfma_d128_kernel        up to 16 rows per item, four waves: each takes a quarter of the
//                                item's tokens, stages its tiles privately, and they meet only
//                                at the end.
// decode_mfma_d128_rows32_kernel up to 32 rows per item, two waves: wave w owns rows 16w .. 16w+15,
//                                both walk all tokens of the item and share the LDS tile — each
//                                fetches and parks 16 of its 32 rows, then both read all of it —
//                                so K and V still cross HBM once.
// ---------------------------------------------------------------------------------

constexpr int kLdsK = 0;
constexpr int kLdsV = 8192;
constexpr int kLdsSc = 16384;    // per-token factors of a quantised tile: three arrays of up to 64 floats
constexpr int kLdsTile = 17152;  // one tile of K and V as 16-bit numbers (32 rows of 256 bytes each), plus the factors
constexpr int kWaves = 4;        // waves per work item of the 16-row kernel
constexpr float kLazyRescale = 8.0f;  // log2 of the largest softmax weight tolerated before the reference maximum moves

__device__ inline u32x4 ldg_stream(const void* p) {
  return __builtin_nontemporal_load((const u32x4*)p);
}

// LDS placement of a tile: 32 rows of 256 bytes, the sixteen 16-byte pieces of a row permuted by an
// XOR that depends on the row.  The LDS moves 128 bytes per clock, i.e. 8 lanes of a 16-byte access
// or 16 lanes of an 8-byte access at a time, and pieces s and s+8 of a row share banks; each access
// pattern of the kernel must therefore touch 8 different pieces (mod 8) per such group of lanes:
//   K rows are read 16 rows at a time, same piece (MFMA A operand)  -> XOR with the row number;
//   V rows are read 4 rows x 2 pieces at a time (transpose read)    -> XOR with twice the row number
//     (bit 3 of the row goes to bit 0 so that rows r and r+8 differ in parity, see KvHalfQuant).
__device__ inline uint32_t swz_k(int row, int piece) { return (uint32_t)(row * 256 + ((piece ^ (row & 15)) << 4)); }
__device__ inline uint32_t swz_v(int row, int piece) {
  return (uint32_t)(row * 256 + ((piece ^ (((row & 7) << 1) | ((row >> 3) & 1))) << 4));
}

// Physical block of token `tok` (any token up to the end of the chunk's last tile: the index is
// clamped to the sequence's block list).  The id comes back through a scalar load; callers fetch it
// a tile ahead of the loads that need it, so that its latency is off the critical path.
__device__ inline int block_of(const DecodeParams& p, const Item& it, int tok) {
  int bi = tok >> p.log2_bs;
  bi = bi < it.nblk ? bi : it.nblk - 1;
  return block_in_cache(p, __builtin_amdgcn_readfirstlane(it.ids[bi]));
}

// The same through the constant address space, which makes the load a scalar one whatever else the
// kernel does (after a global-to-LDS load the compiler no longer proves on its own that the table is
// unchanged, and a vector load here would make its wait cover every tile in flight).  The block
// lists are never written by these kernels.
__device__ inline int block_of_const(const DecodeParams& p, const Item& it, int tok) {
  int bi = tok >> p.log2_bs;
  bi = bi < it.nblk ? bi : it.nblk - 1;
  return block_in_cache(p, ((const __attribute__((address_space(4))) int32_t*)it.ids)[bi]);
}

// Uniform (scalar-register) part of the addresses of 16 consecutive tokens starting at `tok`
// (a multiple of 16, so they lie in one block, `blk`): element offset of (block, kv head, slot) in
// the cache and in the scale tensors.  The host admits only caches whose block and slot strides are
// below 2^31 elements to these kernels, so 32 x 32 -> 64 bit products suffice.
struct HalfBase {
  int64_t elem;
  int64_t scale;
};

__device__ inline HalfBase half_base(const DecodeParams& p, const Item& it, int tok, int blk) {
  const uint32_t slot = (uint32_t)(tok & (p.block_size - 1));
  HalfBase b;
  b.elem = (int64_t)((uint64_t)(uint32_t)blk * (uint32_t)p.stride_block) + it.head_off +
           (int64_t)(slot * (uint32_t)p.stride_slot);
  b.scale = (int64_t)((uint64_t)(uint32_t)blk * (uint32_t)p.sc_stride_block) + it.sc_head_off +
            (int64_t)(slot * (uint32_t)p.sc_stride_slot);
  return b;
}

// Template tag of the MFMA kernels: the cache dtype, plus kQF16 when the queries (and outputs) are
// fp16 rather than bf16.  An fp16 cache implies fp16 queries.
constexpr int kQF16 = 64;
constexpr int kv_of(int kt) { return kt & (kQF16 - 1); }
constexpr bool qf16_of(int kt) { return (kt & kQF16) != 0 || kv_of(kt) == XLLM_HIP_FP16; }
constexpr bool quant_of(int kt) { return kv_of(kt) == XLLM_HIP_FP8_E4M3 || kv_of(kt) == XLLM_HIP_INT8; }
// An int8 cache at head_dim 128 or 256: the K rows stay bytes in LDS and meet the queries in the int8 MFMA
// (v_mfma_i32_16x16x64_i8); see RowTile.  V is still converted to fp16 for the second MFMA.
#ifndef XLLM_HIP_RAW_K
#define XLLM_HIP_RAW_K 1
#endif
constexpr bool raw_k_of(int kt, int tok) { return XLLM_HIP_RAW_K && kv_of(kt) == XLLM_HIP_INT8 && tok != 2; }
// LDS placement of raw K rows: 128 bytes each, the eight 16-byte pieces of a row permuted by an XOR
// whose key takes all eight values over rows r .. r+7 (the MFMA operand read: 8 lanes, same piece,
// consecutive rows) and differs in bit 2 between rows r and r+1 (the park: 8 lanes write four
// neighbouring pieces of two neighbouring rows).
__device__ inline uint32_t swz_kraw(int row, int piece) {
  return (uint32_t)(row * 128 + ((piece ^ (((row & 1) << 2) | ((row >> 1) & 3))) << 4));
}
typedef __attribute__((ext_vector_type(4))) int i32x4;

// KvHalf<KV>: the registers that hold 16 tokens (half a tile) of K and V in flight, the per-lane
// geometry of their loads, and how they are parked in rows 16*h .. 16*h+15 of an LDS tile.
template <int KV_DT>
struct KvHalf;

// bf16 / fp16 cache: 8 loads of 16 bytes per lane (4 K + 4 V); a load instruction covers 4 rows:
// lane = (row-in-load, piece).
struct KvHalf16 {
  // Row 4j + lrow differs from row lrow only in bits the lane does not own, so its swizzled LDS
  // offset is the offset of row lrow with a j-dependent constant XORed in (plus j KiB): one register
  // per array instead of one per row.
  struct Geom {
    uint32_t g_off;  // byte offset of (row lrow, piece) from the first of the 16 rows
    uint32_t wk;     // LDS offset of K row lrow, piece
    uint32_t wv;     // LDS offset of V row lrow, piece
    int lrow;
    int tok;         // tokens per row
    int second;      // 1 if this lane's piece belongs to the second token of its row
    // `ptok`: DecodeParams::tok, which the kernels know at compile time (the offsets below that depend on it
    // alone then become immediates of the instructions that use them)
    __device__ inline void init(const DecodeParams& p, int lane, int ptok) {
      lrow = lane >> 4;
      const int piece = lane & 15;
      tok = ptok == 0 ? 1 : ptok;  // head_dim 256: rows are tokens here too; `plane` picks the half of the token
      second = tok == 2 && piece >= 8 ? 1 : 0;
      g_off = (uint32_t)(((lrow * tok + second) * p.stride_slot + (piece & (16 / tok - 1)) * 8) * 2);
      wk = kLdsK + swz_k(lrow, piece);
      wv = kLdsV + swz_v(lrow, piece);
    }
    // rows 4j + lrow (+16h): the K swizzle adds 4j; the V swizzle adds 8 for odd j, 1 for rows 8..15
    __device__ inline uint32_t k_row(int j, int h) const {
      return (wk ^ (uint32_t)((4 * j) << 4)) + j * 1024 + h * 4096;
    }
    __device__ inline uint32_t v_row(int j, int h) const {
      return (wv ^ (uint32_t)((((j & 1) << 3) | (j >> 1)) << 4)) + j * 1024 + h * 4096;
    }
  };
  u32x4 k[4];
  u32x4 v[4];

  // `plane` (head_dim 256 only): 0 = elements 0..127 of the 16 tokens, 1 = elements 128..255.
  template <bool KEEP = false>
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tok, int blk, const Geom& g, int plane = 0) {
    const HalfBase b = half_base(p, it, tok, blk);
    const uint8_t* kb = p.k_cache + b.elem * 2 + plane * 256;
    const uint8_t* vb = p.v_cache + b.elem * 2 + plane * 256;
    const int64_t step = 4 * p.stride_slot * g.tok * 2;  // four rows further, in bytes (uniform)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      k[j] = ldg_stream(kb + j * step + g.g_off);
      v[j] = ldg_stream(vb + j * step + g.g_off);
    }
  }
  // V rows at or beyond `len` may hold anything (unwritten slots); zero them so that 0 * x stays 0.
  // (K rows need no such care: their scores are replaced by -inf.)
  template <bool MASKED, bool RAWK = false>
  __device__ inline void park(uint8_t* tile, int h, int tok, int len, float, const Geom& g) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      u32x4 vv = v[j];
      if (MASKED && tok + g.tok * (4 * j + g.lrow) + g.second >= len) vv = u32x4{0, 0, 0, 0};
      *(u32x4*)(tile + g.k_row(j, h)) = k[j];
      *(u32x4*)(tile + g.v_row(j, h)) = vv;
    }
  }
};
template <>
struct KvHalf<XLLM_HIP_BF16> : KvHalf16 {};
template <>
struct KvHalf<XLLM_HIP_FP16> : KvHalf16 {};

// The 16-bit type the MFMAs compute in: that of the queries (bf16 and e4m3 cache values convert to
// either exactly) — except that an int8 cache always uses fp16, because a byte u = x + 128 becomes
// the fp16 number 1024 + u by a byte permute alone (0x6400 | u), 0.75 instructions per element
// instead of 1.75 through float; the kernel takes the offset 1152 = 1024 + 128 back out of the scores
// and of the output, and bf16 queries are converted once per work item.
template <bool F16>
struct MmaOps {
  typedef bf16x8 Op;
  __device__ static inline f32x4 run(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
  // K = 16: the first four elements of each operand
  __device__ static inline f32x4 run16(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(
        __builtin_bit_cast(s16x4, __builtin_shufflevector(a, a, 0, 1, 2, 3)),
        __builtin_bit_cast(s16x4, __builtin_shufflevector(b, b, 0, 1, 2, 3)), c, 0, 0, 0);
  }
  __device__ static inline uint32_t pack(float a, float b) {
    return __builtin_bit_cast(uint32_t, bf16x2{(__bf16)a, (__bf16)b});
  }
};
template <>
struct MmaOps<true> {
  typedef f16x8 Op;
  __device__ static inline f32x4 run(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
  __device__ static inline f32x4 run16(Op a, Op b, f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_shufflevector(a, a, 0, 1, 2, 3),
                                                 __builtin_shufflevector(b, b, 0, 1, 2, 3), c, 0, 0, 0);
  }
  __device__ static inline uint32_t pack(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
  }
};
constexpr bool f16_ops(int kt) { return kv_of(kt) == XLLM_HIP_INT8 || qf16_of(kt); }
template <int KV_DT>
struct Mma : MmaOps<f16_ops(KV_DT)> {};
constexpr float kInt8Offset = 1152.0f;

// Convert 16 quantised bytes to 16 numbers of the MFMA operand type (two 16-byte pieces).
template <int KV_DT>
__device__ inline void dequant16(const u32x4 raw, u32x4& lo, u32x4& hi) {
  uint32_t o[8];
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (kv_of(KV_DT) == XLLM_HIP_FP8_E4M3 && f16_ops(KV_DT)) {
      o[2 * w] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[w], 1.0f, false));
      o[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(raw[w], 1.0f, true));
    } else if (kv_of(KV_DT) == XLLM_HIP_FP8_E4M3) {
      o[2 * w] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)raw[w], 1.0f, false));
      o[2 * w + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)raw[w], 1.0f, true));
    } else {
      const uint32_t t = raw[w] ^ 0x80808080u;                         // bytes x + 128
      o[2 * w] = __builtin_amdgcn_perm(0x64646464u, t, 0x04010400u);      // (0x64, u1, 0x64, u0)
      o[2 * w + 1] = __builtin_amdgcn_perm(0x64646464u, t, 0x04030402u);  // (0x64, u3, 0x64, u2)
    }
  }
  lo = u32x4{o[0], o[1], o[2], o[3]};
  hi = u32x4{o[4], o[5], o[6], o[7]};
}

// 1-byte caches: 4 loads of 16 bytes per lane (2 K + 2 V).  A load instruction covers 8 rows of 128
// bytes; a lane holds 16 consecutive elements, which become two 16-byte pieces (2c, 2c+1) of one
// LDS row.  Lanes are assigned in quads so that the 8 lanes of an LDS write group hold pieces of
// two rows whose swizzles differ in parity — rows r, r+1 for K and rows r, r+8 for V — which makes
// the 8 pieces they write distinct mod 8.
// The fp32 scales of the 16 tokens travel beside them: lanes 0-15 fetch the K scales, lanes 16-31
// the V scales (one register).  What is parked after the tile is what the softmax wants per token,
// worked out once by the lane that holds the scale:
//   kscl = k_scale * sm_scale * log2(e)    score x = s * kscl + lv
//   lv   = log2(v_scale)                   weight w = 2^(x - max x) = p * v_scale / 2^max, never above 1
//   rvs  = 1 / v_scale                     denominator share p = w * rvs
// so the V scale rides inside the exponent: the weights given to the MFMA use the full range of a
// 16-bit float whatever the scales are, and no separate multiply by v_scale is needed.
template <int KV_DT>
struct KvHalfQuant {
  // Load j (0, 1): K rows krow + 8j, V rows vrow + 4j.  As for the bf16 cache the LDS offsets of the
  // further rows and of the second piece follow from one register by XOR.
  struct Geom {
    uint32_t gk_off;  // K: byte offset of (row krow, 16-byte chunk) from the first of the 16 rows
    uint32_t gv_off;  // V: same under the V lane assignment
    uint32_t wk;      // LDS offset of K row krow, piece 2 * chunk
    uint32_t wv;      // LDS offset of V row vrow, piece 2 * chunk
    uint32_t sc_g;    // byte offset of this lane's scale from the scale of the first of the 16 tokens
    uint32_t sc_lds;  // where kscl / lv is parked (before adding 64 bytes for the second half of the tile)
    uint32_t sc_half; // bytes between the two halves of a tile in each scale array
    uint32_t sc_next; // bytes from one scale array to the next
    int vrow;
    int tok;          // tokens per row
    int second;       // 1 if this lane's chunk belongs to the second token of its row
    int sc_tok;       // token (of the 16 * tok) whose scale this lane carries
    bool sc_on;       // lanes 0 .. 32 * tok - 1 carry a scale: first the K scales, then the V scales
    bool sc_is_v;
    uint32_t wkraw;   // LDS offset of raw K row krow, this lane's 16-byte piece (int8 cache, head_dim 128)
    __device__ inline void init(const DecodeParams& p, int lane, int ptok) {
      const int chunk = 4 * ((lane >> 3) & 1) + (lane & 3);
      const int pair = (lane >> 2) & 1;
      const int krow = 2 * (lane >> 4) + pair;  // rows r, r+1 alternate between quads (krow < 8)
      vrow = (lane >> 4) + 8 * pair;            // rows r, r+8 alternate between quads (vrow & 7 < 4)
      tok = ptok == 0 ? 1 : ptok;  // head_dim 256: rows are tokens here too; `plane` picks the half of the token
      second = tok == 2 && chunk >= 4 ? 1 : 0;
      const int in_tok = (chunk & (8 / tok - 1)) * 16;  // byte within the token's row
      gk_off = (uint32_t)((krow * tok + second) * p.stride_slot + in_tok);
      gv_off = (uint32_t)((vrow * tok + second) * p.stride_slot + in_tok);
      wk = kLdsK + swz_k(krow, 2 * chunk);
      wkraw = kLdsK + swz_kraw(krow, chunk);
      wv = kLdsV + swz_v(vrow, 2 * chunk);
      const int per_half = 16 * tok;  // tokens per half tile
      sc_tok = lane % per_half;
      sc_g = (uint32_t)(sc_tok * p.sc_stride_slot * 4);
      sc_is_v = ((lane / per_half) & 1) != 0;
      sc_on = lane < 2 * per_half;
      sc_half = (uint32_t)(per_half * 4);
      sc_next = 2 * sc_half;
      sc_lds = kLdsSc + (sc_is_v ? sc_next : 0) + sc_tok * 4;
    }
    // K row krow + 8j: swizzle adds 8; V row vrow + 4j: swizzle adds 8; second piece: XOR 1.
    __device__ inline uint32_t k_row(int j, int hi, int h) const {
      return (wk ^ (uint32_t)(((j << 3) | hi) << 4)) + j * 2048 + h * 4096;
    }
    __device__ inline uint32_t v_row(int j, int hi, int h) const {
      return (wv ^ (uint32_t)(((j << 3) | hi) << 4)) + j * 1024 + h * 4096;
    }
  };
  u32x4 k[2];
  u32x4 v[2];
  float sc;

  // `plane` (head_dim 256 only): 0 = elements 0..127 of the 16 tokens, 1 = elements 128..255.  Both
  // planes carry the tokens' scales (the second copy comes from the cache and lands in the unused
  // half of the factor arrays).
  // KEEP: ordinary loads, whose lines may stay in the CU's cache, for a workgroup whose other waves ask for the
  // rest of the same lines.
  template <bool KEEP = false>
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tok, int blk, const Geom& g, int plane = 0) {
    const HalfBase b = half_base(p, it, tok, blk);
    const uint8_t* kb = p.k_cache + b.elem + plane * 128;
    const uint8_t* vb = p.v_cache + b.elem + plane * 128;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if constexpr (KEEP) {
        k[j] = *(const u32x4*)(kb + j * 8 * p.stride_slot * g.tok + g.gk_off);
        v[j] = *(const u32x4*)(vb + j * 4 * p.stride_slot * g.tok + g.gv_off);
      } else {
        k[j] = ldg_stream(kb + j * 8 * p.stride_slot * g.tok + g.gk_off);
        v[j] = ldg_stream(vb + j * 4 * p.stride_slot * g.tok + g.gv_off);
      }
    }
    const float* sb = (g.sc_is_v ? p.v_scale : p.k_scale) + b.scale;
    if (g.sc_on) sc = *(const float*)((const uint8_t*)sb + g.sc_g);
  }

  // RAWK: the K rows are parked as they are (rows krow + 8j at 128 bytes each).
  template <bool MASKED, bool RAWK = false>
  __device__ inline void park(uint8_t* tile, int h, int tok, int len, float scale_log2, const Geom& g) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      u32x4 klo, khi, vlo, vhi;
      if constexpr (RAWK) {
        *(u32x4*)(tile + g.wkraw + j * 1024 + h * 2048) = k[j];
      } else {
        dequant16<KV_DT>(k[j], klo, khi);
        *(u32x4*)(tile + g.k_row(j, 0, h)) = klo;
        *(u32x4*)(tile + g.k_row(j, 1, h)) = khi;
      }
      dequant16<KV_DT>(v[j], vlo, vhi);
      if (MASKED && tok + g.tok * (g.vrow + 4 * j) + g.second >= len) vlo = vhi = u32x4{0, 0, 0, 0};
      *(u32x4*)(tile + g.v_row(j, 0, h)) = vlo;
      *(u32x4*)(tile + g.v_row(j, 1, h)) = vhi;
    }
    if (g.sc_on) {
      // A V scale of zero (an all-zero row) would put -inf into the exponent and lose the token's
      // share of the denominator; 2^-100 keeps it and still makes the row's contribution vanish.
      const float vs = fmaxf(sc, 0x1p-100f);
      float a = g.sc_is_v ? __builtin_amdgcn_logf(vs) : sc * scale_log2;
      float r = __builtin_amdgcn_rcpf(vs);
      if (MASKED && tok + g.sc_tok >= len) a = r = 0.0f;  // slots past the end may hold anything
      *(float*)(tile + g.sc_lds + h * g.sc_half) = a;
      if (g.sc_is_v) *(float*)(tile + g.sc_lds + g.sc_next + h * g.sc_half) = r;
    }
  }
};
template <>
struct KvHalf<XLLM_HIP_FP8_E4M3> : KvHalfQuant<XLLM_HIP_FP8_E4M3> {};
template <>
struct KvHalf<XLLM_HIP_INT8> : KvHalfQuant<XLLM_HIP_INT8> {};
template <>
struct KvHalf<XLLM_HIP_FP8_E4M3 | kQF16> : KvHalfQuant<XLLM_HIP_FP8_E4M3 | kQF16> {};
template <>
struct KvHalf<XLLM_HIP_INT8 | kQF16> : KvHalfQuant<XLLM_HIP_INT8 | kQF16> {};

// max / sum over the four lanes (kg = 0..3) that share a query row: lanes l, l^16, l^32, l^48.
// v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even rows of its
// second, v_permlane32_swap the upper half of the first with the lower half of the second; fed the
// same value twice they leave (rows 0,0,2,2 | rows 1,1,3,3) and (lower, lower | upper, upper).
// Written as asm because the compiler's builtin hands back the first result twice; the leading
// s_nop is the wait a VALU result needs before a lane permute may read it.
__device__ inline void lane_swap16(float& a, float& b) {
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ inline void lane_swap32(float& a, float& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
// The maximum over the four lanes that hold a query row's scores.  PLAIN: the maximum as the instruction alone
// (fmaxf first brings each operand to canonical form, an operation of its own; the same value for operands that
// are no signalling NaNs).  Only where it pays: it changes the register allocation of the kernels around it.
template <bool PLAIN>
__device__ inline float max_of(float a, float b) {
  if constexpr (PLAIN) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
  } else {
    return fmaxf(a, b);
  }
}
template <bool PLAIN = false>
__device__ inline float kg_max(float v) {
  float a = v, b = v;
  lane_swap16(a, b);
  a = b = max_of<PLAIN>(a, b);
  lane_swap32(a, b);
  return max_of<PLAIN>(a, b);
}
__device__ inline float kg_sum(float v) {
  float a = v, b = v;
  lane_swap16(a, b);
  a = b = a + b;
  lane_swap32(a, b);
  return a + b;
}

// State of one wave's tile of 16 query rows, and the attention over one parked tile.
//
// TOK = 1: head_dim 128, an LDS row is one token.  TOK = 2: head_dim 64; an LDS row is then two
// consecutive tokens (its first eight 16-byte pieces from one, the rest from the next), so parking
// and swizzles are those of head_dim 128, and the MFMAs split the row again:
//   scores of the first  token of row t:  K chunks 0, 1 of the row against the query's two chunks
//   scores of the second token of row t:  K chunks 2, 3 against the same query chunks
//   head-dim tiles 0..3 of V^T are the first token's values, tiles 4..7 the second's, so they take
//   the first / second tokens' weights as B operand and the two halves of O^T are added at the end.
// A tile is 32 rows either way, i.e. 32 * TOK tokens.
// TOK = 0: head_dim 256.  A token is two rows: row t of the tile's first half holds its elements
// 0..127, row t of the second half (row 16 + t) its elements 128..255, so a tile is 16 tokens.  The
// K fragments of the two halves then meet the query's chunks 0..3 and 4..7 and add up to one score
// tile; the V^T tiles of the first half are head-dim tiles 0..7 and those of the second 8..15, each
// against the 16 tokens' weights with the K = 16 form of the MFMA.
constexpr int tile_tokens_of(int tok) { return tok == 0 ? 16 : 32 * tok; }
constexpr int half_tokens_of(int tok) { return 16 * tok; }  // tokens between the tile's two halves (none at head_dim 256)
constexpr int head_dim_of(int tok) { return tok == 0 ? 256 : 128 / tok; }
constexpr int xch_row_bytes(int tok) { return head_dim_of(tok) * 4 + 16; }  // a query row in the end-of-item exchange

// RAWK: see kRawK.  OFFSET / OFFSET_K: int8 V / K rows sit in LDS with the offset 1152 (see kOffset); a
// caller that parks them as exact fp16 numbers passes false.
// FENCED: fragments and per-token factors are read where they are used and the LDS offsets of the
// fragments are formed every tile anew (scheduling fences; see kFenced), for a kernel with no register to spare.
// NORM_ROW: see kNormQ.
template <int KV_DT, int TOK, bool RAWK = raw_k_of(KV_DT, TOK), bool OFFSET = kv_of(KV_DT) == XLLM_HIP_INT8,
          bool OFFSET_K = OFFSET && !RAWK, bool FENCED = false, bool NORM_ROW = true>
struct RowTile {
  static constexpr bool kQuant = quant_of(KV_DT);
  // int8 rows sit in LDS as x + 1152.  With K' = K + 1152 and V' = V + 1152:
  //   q.K  = q.K' - 1152 * sum_d q_d                     the constant is the MFMA's initial C operand
  //   sum_t w_t V_t = sum_t w_t V'_t - 1152 * sum_t w_t   sum_t w_t comes from one more MFMA whose A
  //                                                       operand is all ones (wacc)
  // Rows zeroed because they lie past the sequence end carry weight 0 in both sums.
  static constexpr bool kOffset = OFFSET;     // V rows (costs an MFMA per tile and its accumulator, wacc)
  static constexpr bool kOffsetK = OFFSET_K;  // K rows (costs nothing per tile: the MFMA's initial C operand)
  // Raw K: the K rows are bytes in LDS and the scores come from the int8 MFMA.  The queries are held as
  // two int8 parts on one scale per query row, q = q_scale * (256 hi + lo) with q_scale a power of two,
  // 2^(e - 15) where 2^e is the first power of two above the row's largest magnitude: 16-bit fixed point
  // against that element, on a grid on which every bf16 query element within 2^7 of the row's largest is
  // exact (its own spacing is a multiple of the grid's).  A score is then
  // q_scale * k_scale * (256 S_hi + S_lo) with both sums exact in 32-bit integers (|S| <= 128 * 128 * 128);
  // q_scale is a per-lane factor, a query row living in one lane column of the score tile.
  static constexpr bool kRawK = RAWK;
  // bf16 queries that become fp16 operands are first brought to a largest magnitude in [2^14, 2^15) by a power of
  // two (exact), so that neither fp16's upper end (65504) nor its lower one (2^-14; nothing below 2^-24) cuts into
  // queries that bf16 holds well.  Row by row (NORM_ROW: the scores then take the row's factor back, like raw
  // K's), or, in a kernel with no register to spare for that, by the largest element of the whole work item,
  // which the caller hands to init and whose factor it folds into the per-token score factors it parks (rows
  // more than 2^28 below the item's largest element then lose bits).
  static constexpr bool kNormQ = !RAWK && f16_ops(KV_DT) && !qf16_of(KV_DT);
  static constexpr bool kNormItem = kNormQ && !NORM_ROW;
  // The scores carry a factor of their query row (q_scale).
  static constexpr bool kRowScale = RAWK || (kNormQ && NORM_ROW);
  static constexpr int kD = head_dim_of(TOK);
  static constexpr int kQC = kD / 32;    // 32-element chunks of a query row
  static constexpr int kDT = TOK == 0 ? 16 : 8;  // O^T accumulator tiles
  static constexpr int kU = TOK == 2 ? 2 : 1;    // tokens per row
  static constexpr int kHalves = TOK == 0 ? 1 : 2;  // halves of the tile that hold different tokens
  // head_dim 256 over a 1-byte cache fits two waves per SIMD (256 registers) only if fragments are read
  // as they are needed: without the fences the compiler hoists the reads of a tile's 8 K and 16 V
  // fragments and keeps the 12 XORed LDS offsets in registers through the loop (50 registers spilled).
  static constexpr bool kFenced = FENCED;
  typedef typename Mma<KV_DT>::Op Op;

  Op qf[kQC];      // Q^T fragments (B operand) of the lane's query row
  f32x4 acc[kDT];  // O^T accumulators: tile dt of the row elements, query rows 4*kg + rr
  f32x4 wacc;      // sum of the weights as the MFMA saw them (int8 only)
  float m_run;     // reference point of the exponents: follows the running maximum of the log2-scaled scores (of score + log2 v_scale if quantised) lazily, see softmax
  float l_run;     // this lane's share of the softmax denominator
  float s_init;    // initial value of the score accumulators: -1152 * sum_d q[r][d] (int8), else 0
  float q_scale;   // factor of the lane's query row on its scores (kRowScale); else 1
  int lim;         // tokens >= lim are invisible to the row (causal among draft tokens)
  int lo;          // tokens < lo are outside the sliding window
  uint32_t k_off0; // LDS offset of K row mi, piece kg        (piece 4c + kg: XOR c << 6)
  uint32_t v_off0; // LDS offset of the transpose read, tile 0 (tile dt: XOR dt << 5)
  int kg;

  // 16 query elements (two 16-byte loads) as floats.
  __device__ static inline void q_floats(const uint16_t* src, bool valid, float (&f)[16]) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      u32x4 raw = {0, 0, 0, 0};
      if (valid) raw = *(const u32x4*)(src + 8 * half);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (qf16_of(KV_DT)) {
          f[8 * half + e] = (float)__builtin_bit_cast(f16x8, raw)[e];
        } else {
          f[8 * half + e] = (float)__builtin_bit_cast(bf16x8, raw)[e];
        }
      }
    }
  }
  // Largest magnitude of the lane's query row (the four lanes that share a row get the same value).
  __device__ static inline float q_absmax(const uint16_t* qrow, bool valid, int kg) {
    float m = 0.0f;
#pragma unroll
    for (int c = 0; c < kD / 64; ++c) {
      float f[16];
      q_floats(qrow + 64 * c + 16 * kg, valid, f);
#pragma unroll
      for (int e = 0; e < 16; ++e) m = fmaxf(m, fabsf(f[e]));
    }
    return kg_max(m);
  }
  // kNormItem: exponent e of the power of two that brings the largest magnitude among the wave's 16 query rows at
  // `row_in_item` into [2^14, 2^15) (every lane gets the wave's value; waves that share parked per-token factors take the
  // largest of theirs).
  __device__ static inline float wave_q_absmax(const DecodeParams& p, const Item& it, int row_in_item, int lane) {
    const int row = it.rg * p.rows_per_item + row_in_item + (lane & 15);
    const bool valid = row < it.n * p.group;
    const int j = valid ? row / p.group : 0;
    const int gq = valid ? row - j * p.group : 0;
    const uint16_t* qrow = (const uint16_t*)p.q + (int64_t)(it.q0 + j) * p.q_token_stride +
                           (int64_t)(it.hk * p.group + gq) * kD;
    return wave_max(q_absmax(qrow, valid, lane >> 4));
  }
  __device__ static inline int norm_exponent(float absmax) {
    return __builtin_amdgcn_readfirstlane(pow2_above(absmax) - 15);
  }
  // The power of two 2^e with m < 2^e (m = f * 2^e, f in [0.5, 1)), as its exponent; within +-100 so that
  // both 2^e and its inverse times 2^15 are ordinary floats (a row of zeros gets the smallest).
  __device__ static inline int pow2_above(float m) {
    const int e = (int)((__builtin_bit_cast(uint32_t, m) >> 23) & 0xffu) - 126;
    return e < -100 ? -100 : (e > 100 ? 100 : e);
  }

  // `q_exp` (kNormItem): see norm_exponent; the caller folds 2^q_exp into the per-token score factors it parks.
  __device__ inline void init(const DecodeParams& p, const Item& it, int row_in_item, int lane, int q_exp = 0) {
    const int mi = lane & 15;  // MFMA row of A / column of B and D
    kg = lane >> 4;            // k-group of the operands; row block of D
    const int row = it.rg * p.rows_per_item + row_in_item + mi;
    const bool valid = row < it.n * p.group;
    const int j = valid ? row / p.group : 0;
    const int gq = valid ? row - j * p.group : 0;
    lim = it.len - (it.n - 1 - j);
    lo = p.window_left >= 0 ? lim - 1 - p.window_left : 0;
    const uint16_t* qrow = (const uint16_t*)p.q + (int64_t)(it.q0 + j) * p.q_token_stride +
                           (int64_t)(it.hk * p.group + gq) * kD;
    float sq = 0.0f;
    q_scale = 1.0f;
    if constexpr (kRawK) {
      // qf[c]: the high parts of elements 64c + 16kg .. + 15 (c = 0 .. kD/64 - 1), sixteen bytes in the
      // order the K bytes lie in memory; qf[kD/64 + c]: the low parts.
      const float top = q_absmax(qrow, valid, kg);
      int e2 = pow2_above(top);
      // (the few values whose grid number would pass 127 * 256 + 127 take the next power of two)
      if (top * __builtin_amdgcn_ldexpf(1.0f, 15 - e2) > 32639.0f) ++e2;
      const float inv = __builtin_amdgcn_ldexpf(1.0f, 15 - e2);
      q_scale = __builtin_amdgcn_ldexpf(1.0f, e2 - 15);
#pragma unroll
      for (int c = 0; c < kD / 64; ++c) {
        float f[16];
        q_floats(qrow + 64 * c + 16 * kg, valid, f);
        uint32_t hi4[4] = {0, 0, 0, 0}, lo4[4] = {0, 0, 0, 0};
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          int qi = (int)rintf(f[e] * inv);  // |qi| <= 32639
          qi = qi > 32639 ? 32639 : (qi < -32639 ? -32639 : qi);  // (a NaN or an infinity among the queries)
          const int h = (qi + 128) >> 8;    // -127 .. 127
          const int l = qi - (h << 8);      // -128 .. 127
          hi4[e >> 2] |= ((uint32_t)h & 0xffu) << (8 * (e & 3));
          lo4[e >> 2] |= ((uint32_t)l & 0xffu) << (8 * (e & 3));
        }
        qf[c] = __builtin_bit_cast(Op, u32x4{hi4[0], hi4[1], hi4[2], hi4[3]});
        qf[kD / 64 + c] = __builtin_bit_cast(Op, u32x4{lo4[0], lo4[1], lo4[2], lo4[3]});
      }
    }
    float down = 1.0f;
    if constexpr (kNormQ) {
      const int e2 = NORM_ROW ? pow2_above(q_absmax(qrow, valid, kg)) - 15 : q_exp;
      down = __builtin_amdgcn_ldexpf(1.0f, -e2);
      if (NORM_ROW) q_scale = __builtin_amdgcn_ldexpf(1.0f, e2);
    }
#pragma unroll
    for (int c = 0; c < (kRawK ? 0 : kQC); ++c) {
      u32x4 raw = {0, 0, 0, 0};
      if (valid) raw = *(const u32x4*)(qrow + c * 32 + kg * 8);
      if constexpr (qf16_of(KV_DT) || !f16_ops(KV_DT)) {
        qf[c] = __builtin_bit_cast(Op, raw);  // the queries already have the operand type
      } else {
        const bf16x8 qb = __builtin_bit_cast(bf16x8, raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) qf[c][e] = (_Float16)((float)qb[e] * down);
      }
      if constexpr (kOffsetK) {
#pragma unroll
        for (int e = 0; e < 8; ++e) sq += (float)qf[c][e];
      }
    }
    s_init = kOffsetK ? -kInt8Offset * kg_sum(sq) : 0.0f;
    m_run = -INFINITY;
    l_run = 0.0f;
    wacc = f32x4{0, 0, 0, 0};
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) acc[dt] = f32x4{0, 0, 0, 0};
    k_off0 = kLdsK + (kRawK ? swz_kraw(mi, kg) : swz_k(mi, kg));
    const int tau = 4 * kg + (mi >> 2);  // row (within 16) this lane points the transpose read at
    v_off0 = kLdsV + swz_v(tau, (mi & 3) >> 1) + (mi & 1) * 8;
  }

  static constexpr int kN = 4 * kU * kHalves;  // scores per lane and tile
  // (per-token factors of a quantised tile travel as three arrays in score order: as one struct
  // they cost registers to the point of spilling)
  // head_dim 256: the two halves' shares of one score tile.  Raw K: [part][half], the integer sums
  // S_hi and S_lo as bits.
  typedef f32x4 Scores[kRawK ? 2 : kU][2];

  __device__ __forceinline__ void load_factors(const uint8_t* tile, float (&kscl)[kN], float (&lv)[kN], float (&rvs)[kN]) const {
    if (!kQuant) return;
    // the factors of tokens kU * (16h + 4kg) .. + 4 * kU - 1 are contiguous in each array
    constexpr int kArr = 32 * kU * 4;  // bytes per array
#pragma unroll
    for (int h = 0; h < kHalves; ++h) {
      const int first = kU * (16 * h + 4 * kg) * 4;
#pragma unroll
      for (int v4 = 0; v4 < kU; ++v4) {
        const f32x4 a = *(const f32x4*)(tile + kLdsSc + first + 16 * v4);
        const f32x4 b = *(const f32x4*)(tile + kLdsSc + kArr + first + 16 * v4);
        const f32x4 c = *(const f32x4*)(tile + kLdsSc + 2 * kArr + first + 16 * v4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int t = 4 * v4 + e;  // token of the lane's 4 * kU: row rr = t / kU, u = t % kU
          const int i = ((t % kU) * kHalves + h) * 4 + t / kU;
          kscl[i] = a[e];
          lv[i] = b[e];
          rvs[i] = c[e];
        }
      }
    }
  }

  // One of the three factor arrays (0: kscl, 1: lv, 2: rvs) alone.
  __device__ __forceinline__ void load_factor(const uint8_t* tile, int which, float (&f)[kN]) const {
    constexpr int kArr = 32 * kU * 4;
#pragma unroll
    for (int h = 0; h < kHalves; ++h) {
      const int first = kU * (16 * h + 4 * kg) * 4;
#pragma unroll
      for (int v4 = 0; v4 < kU; ++v4) {
        const f32x4 a = *(const f32x4*)(tile + kLdsSc + which * kArr + first + 16 * v4);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int t = 4 * v4 + e;
          f[((t % kU) * kHalves + h) * 4 + t / kU] = a[e];
        }
      }
    }
  }

  // ---- S^T = K Q^T: chunk c of the rows' 128 elements, K fragments of the tile's two halves ----
  __device__ __forceinline__ void scores_init(Scores& s) const {
    if constexpr (kRawK) {
      s[0][0] = s[0][1] = s[1][0] = s[1][1] = f32x4{0, 0, 0, 0};  // (integer zeros)
      return;
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) s[u][0] = s[u][1] = f32x4{s_init, s_init, s_init, s_init};
    if (TOK == 0) s[0][1] = f32x4{0, 0, 0, 0};  // the halves are added: the offset term enters once
  }
  // Raw K: chunk c (0, 1) of the rows' 128 bytes against the queries' high and low parts.
  // head_dim 256: the tile's second half holds the same 16 tokens' bytes 128..255, which meet the
  // queries' chunks 2 and 3; both halves add into one pair of sums.
  __device__ __forceinline__ void scores_step_raw(int c, const i32x4& kf0, const i32x4& kf1, Scores& s) const {
    if constexpr (TOK == 0) {
      i32x4 hi = __builtin_bit_cast(i32x4, s[0][0]), lo = __builtin_bit_cast(i32x4, s[1][0]);
      hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf0, __builtin_bit_cast(i32x4, qf[c]), hi, 0, 0, 0);
      lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf0, __builtin_bit_cast(i32x4, qf[4 + c]), lo, 0, 0, 0);
      hi = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf1, __builtin_bit_cast(i32x4, qf[2 + c]), hi, 0, 0, 0);
      lo = __builtin_amdgcn_mfma_i32_16x16x64_i8(kf1, __builtin_bit_cast(i32x4, qf[6 + c]), lo, 0, 0, 0);
      s[0][0] = __builtin_bit_cast(f32x4, hi);
      s[1][0] = __builtin_bit_cast(f32x4, lo);
      return;
    }
    const i32x4 qh = __builtin_bit_cast(i32x4, qf[c]), ql = __builtin_bit_cast(i32x4, qf[2 + c]);
    s[0][0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_mfma_i32_16x16x64_i8(kf0, qh, __builtin_bit_cast(i32x4, s[0][0]), 0, 0, 0));
    s[0][1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_mfma_i32_16x16x64_i8(kf1, qh, __builtin_bit_cast(i32x4, s[0][1]), 0, 0, 0));
    s[1][0] = __builtin_bit_cast(f32x4, __builtin_amdgcn_mfma_i32_16x16x64_i8(kf0, ql, __builtin_bit_cast(i32x4, s[1][0]), 0, 0, 0));
    s[1][1] = __builtin_bit_cast(f32x4, __builtin_amdgcn_mfma_i32_16x16x64_i8(kf1, ql, __builtin_bit_cast(i32x4, s[1][1]), 0, 0, 0));
  }
  __device__ __forceinline__ void scores_step(int c, const Op& kf0, const Op& kf1, Scores& s) const {
    if constexpr (TOK == 0) {
      s[0][0] = Mma<KV_DT>::run(kf0, qf[c], s[0][0]);
      s[0][1] = Mma<KV_DT>::run(kf1, qf[4 + c], s[0][1]);
    } else {
      s[c / kQC][0] = Mma<KV_DT>::run(kf0, qf[c % kQC], s[c / kQC][0]);
      s[c / kQC][1] = Mma<KV_DT>::run(kf1, qf[c % kQC], s[c / kQC][1]);
    }
  }

  // ---- online softmax of the lane's query row over the tile starting at token tb ----
  // Score / weight index i = (u * kHalves + h) * 4 + rr: token kU * (16h + 4kg + rr) + u of the tile.
  // Leaves the weights as B operand of the second MFMA (k-slot e = 4h + rr) in pf and the factor
  // the accumulators are to be scaled by in alpha; returns whether any row's maximum moved.
  // First half: the scaled (and masked) scores x of the tile.  A plain tile of a 16-bit cache keeps the raw
  // scores here (the scale is not negative: the host sends other scales to the generic kernel) and the
  // scale rides in the FMA that forms the exponent, one operation per score less.
  template <bool MASKED>
  __device__ __forceinline__ void scaled_scores(const Scores& s, const float (&kscl)[kN], const float (&lv)[kN], int tb,
                                                float scale_log2, float (&x)[kN]) const {
    const float neg_inf = -INFINITY;
    constexpr bool kFold = !kQuant && !MASKED;
#pragma unroll
    for (int u = 0; u < kU; ++u) {
#pragma unroll
      for (int h = 0; h < kHalves; ++h) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          const int i = (u * kHalves + h) * 4 + rr;
          float raw;
          if constexpr (kRawK) {
            // (whole vectors are reinterpreted: a bit cast of one element of a vector reads element 0)
            const i32x4 both = (__builtin_bit_cast(i32x4, s[0][h]) << 8) + __builtin_bit_cast(i32x4, s[1][h]);
            raw = (float)both[rr];
          } else {
            raw = TOK == 0 ? s[0][0][rr] + s[0][1][rr] : s[u][h][rr];
          }
          if constexpr (kRowScale) raw *= q_scale;
          float v = kFold ? raw : kQuant ? __builtin_fmaf(raw, kscl[i], lv[i]) : raw * scale_log2;
          if (MASKED) {
            const int tok = tb + kU * (16 * h + 4 * kg + rr) + u;
            v = (tok < lim && tok >= lo) ? v : neg_inf;
          }
          x[i] = v;
        }
      }
    }
  }

  // Second half: running maximum, weights, denominator.
  template <bool MASKED>
  __device__ __forceinline__ bool weights(const float (&x)[kN], const float (&rvs)[kN], float scale_log2, Op (&pf)[kU],
                                          float& alpha) {
    const float neg_inf = -INFINITY;
    constexpr bool kFold = !kQuant && !MASKED;
    float mt = neg_inf;
#pragma unroll
    for (int i = 0; i < kN; ++i) mt = fmaxf(mt, x[i]);
    mt = kg_max(mt);
    if (kFold) mt *= scale_log2;
    // The reference point of the exponents follows the running maximum lazily: it moves (for every
    // row of the tile) only when some row's maximum has grown by more than kLazyRescale, i.e. when
    // weights above 2^kLazyRescale would appear.  Until then weights may exceed 1 by up to that
    // factor — harmless for the 16-bit weights (same relative precision) and the fp32 sums — and the
    // accumulators need no rescaling, which with 16 or 32 rows per wave is otherwise due on most
    // tiles of the first few thousand tokens.
    const float m_top = fmaxf(m_run, mt);
    const bool moved = __builtin_amdgcn_ballot_w64(m_top > m_run + kLazyRescale) != 0;
    const float m_new = moved ? m_top : m_run;
    const float m_safe = m_new == neg_inf ? 0.0f : m_new;
    alpha = __builtin_amdgcn_exp2f(m_run - m_safe);
    l_run *= alpha;
    m_run = m_new;
    float w[kN];
#pragma unroll
    for (int i = 0; i < kN; ++i) {
      const float e = __builtin_amdgcn_exp2f(kFold ? __builtin_fmaf(x[i], scale_log2, -m_safe) : x[i] - m_safe);
      w[i] = e;
      l_run = kQuant ? __builtin_fmaf(e, rvs[i], l_run) : l_run + e;
    }
    if constexpr (TOK == 0) {  // four weights: the B operand of the K = 16 MFMA
      const u32x4 pw = {Mma<KV_DT>::pack(w[0], w[1]), Mma<KV_DT>::pack(w[2], w[3]), 0u, 0u};
      pf[0] = __builtin_bit_cast(Op, pw);
    } else {
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const float* wu = w + 8 * u;
        const u32x4 pw = {Mma<KV_DT>::pack(wu[0], wu[1]), Mma<KV_DT>::pack(wu[2], wu[3]),
                          Mma<KV_DT>::pack(wu[4], wu[5]), Mma<KV_DT>::pack(wu[6], wu[7])};
        pf[u] = __builtin_bit_cast(Op, pw);
      }
    }
    return moved;
  }

  template <bool MASKED>
  __device__ __forceinline__ bool softmax(const Scores& s, const float (&kscl)[kN], const float (&lv)[kN], const float (&rvs)[kN], int tb, float scale_log2, Op (&pf)[kU],
                                 float& alpha) {
    float x[kN];
    scaled_scores<MASKED>(s, kscl, lv, tb, scale_log2, x);
    return weights<MASKED>(x, rvs, scale_log2, pf, alpha);
  }

  // ---- O^T = O^T * alpha + V^T P^T, tile dt of the rows' 128 elements ----
  __device__ __forceinline__ Op v_fragment(const uint8_t* tile, int dt) const { return v_fragment(tile, dt, v_off0); }
  // The offset of tile 0 made opaque: the XORs that give the other tiles' offsets are then computed where they
  // are used, every tile anew, instead of being held in registers through the token loop.
  __device__ __forceinline__ static uint32_t opaque(uint32_t v) {
    asm volatile("" : "+v"(v));
    return v;
  }
  __device__ __forceinline__ Op v_fragment(const uint8_t* tile, int dt, uint32_t v0) const {
    const uint32_t vo = v0 ^ (uint32_t)((dt & 7) << 5);
    if constexpr (TOK == 0) {  // tile dt of the 16 tokens: from the first half (dt < 8) or the second
      const s16x4 a = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)(tile + vo + (dt >> 3) * 4096));
      return __builtin_bit_cast(Op, __builtin_shufflevector(a, a, 0, 1, 2, 3, 0, 1, 2, 3));
    } else {
      const s16x4 a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)(tile + vo));
      const s16x4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)(tile + vo + 4096));
      return __builtin_bit_cast(Op, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
    }
  }
  template <bool RESCALE>
  __device__ __forceinline__ void accumulate_step(int dt, const Op& vf, const Op (&pf)[kU], float alpha) {
    f32x4 c = acc[dt];
    if (RESCALE) c *= alpha;
    if constexpr (TOK == 0) {
      acc[dt] = Mma<KV_DT>::run16(vf, pf[0], c);
    } else {
      acc[dt] = Mma<KV_DT>::run(vf, pf[dt * kU / 8], c);
    }
  }
  template <bool RESCALE>
  __device__ __forceinline__ void accumulate_weights(const Op (&pf)[kU], float alpha) {
    if (!kOffset) return;
    const u32x4 ones = {0x3c003c00u, 0x3c003c00u, 0x3c003c00u, 0x3c003c00u};  // fp16 1.0
    f32x4 c = wacc;
    if (RESCALE) c *= alpha;
    if constexpr (TOK == 0) {
      c = Mma<KV_DT>::run16(__builtin_bit_cast(Op, ones), pf[0], c);
    } else {
#pragma unroll
      for (int u = 0; u < kU; ++u) c = Mma<KV_DT>::run(__builtin_bit_cast(Op, ones), pf[u], c);
    }
    wacc = c;
  }
  template <bool RESCALE>
  __device__ __forceinline__ void accumulate(const uint8_t* tile, const Op (&pf)[kU], float alpha) {
    const uint32_t v0 = kFenced ? opaque(v_off0) : v_off0;
#pragma unroll
    for (int dt = 0; dt < kDT; ++dt) {
      accumulate_step<RESCALE>(dt, v_fragment(tile, dt, v0), pf, alpha);
      if (kFenced && (dt & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // (every 2, 8 or 16 tiles: the same time)
    }
    accumulate_weights<RESCALE>(pf, alpha);
  }

  // Attention of the 16 query rows over the 32 * TOK tokens parked in `tile` (first token tb).
  template <bool MASKED>
  __device__ __forceinline__ void attend(const uint8_t* tile, int tb, float scale_log2) {
    float kscl[kN], lv[kN], rvs[kN];
    if (!kFenced) load_factors(tile, kscl, lv, rvs);
    Scores s;
    scores_init(s);
    if constexpr (kRawK) {
      const uint32_t k0 = kFenced ? opaque(k_off0) : k_off0;
#pragma unroll
      for (int c = 0; c < 2; ++c) {
        const uint32_t ko = k0 ^ (uint32_t)(c << 6);
        scores_step_raw(c, *(const i32x4*)(tile + ko), *(const i32x4*)(tile + ko + 2048), s);
        if (kFenced && c < 1) __builtin_amdgcn_sched_barrier(0);
      }
    } else {
      const uint32_t k0 = kFenced ? opaque(k_off0) : k_off0;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const uint32_t ko = k0 ^ (uint32_t)(c << 6);
        scores_step(c, *(const Op*)(tile + ko), *(const Op*)(tile + ko + 4096), s);
        if (kFenced && c < 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
    Op pf[kU];
    float alpha;
    bool moved;
    if constexpr (kFenced && kQuant) {
      // the per-token factors are loaded when they are used: two for the exponents, then the third
      float x[kN];
      __builtin_amdgcn_sched_barrier(0);
      load_factor(tile, 0, kscl);
      load_factor(tile, 1, lv);
      scaled_scores<MASKED>(s, kscl, lv, tb, scale_log2, x);
      __builtin_amdgcn_sched_barrier(0);
      load_factor(tile, 2, rvs);
      moved = weights<MASKED>(x, rvs, scale_log2, pf, alpha);
      __builtin_amdgcn_sched_barrier(0);
    } else {
      if (kFenced) load_factors(tile, kscl, lv, rvs);
      moved = softmax<MASKED>(s, kscl, lv, rvs, tb, scale_log2, pf, alpha);
    }
    // The accumulators need rescaling only when some row's maximum moved, which becomes rare a few
    // tiles into a sequence.  Both variants of the product are written out, so that each path ends
    // in the MFMAs that define the accumulators (a branch around the multiplies alone makes the
    // compiler shuffle the accumulator registers on every tile).
    if (moved) {
      accumulate<true>(tile, pf, alpha);
    } else {
      accumulate<false>(tile, pf, alpha);
    }
  }
};

// The same for two row tiles held by one wave (32 query rows): every K and V fragment read from
// LDS feeds two MFMAs, which is what keeps a prefill-sized step from being bound by LDS bandwidth.
template <bool MASKED, class RT>
__device__ __forceinline__ void attend_pair(RT (&rt)[2], const uint8_t* tile, int tb, float scale_log2) {
  static_assert(!RT::kRawK, "two row tiles per wave read converted K rows");
  typedef typename RT::Op Op;
  float kscl[RT::kN], lv[RT::kN], rvs[RT::kN];
  if constexpr (!RT::kQuant) rt[0].load_factors(tile, kscl, lv, rvs);  // (nothing to load)
  typename RT::Scores s0, s1;
  rt[0].scores_init(s0);
  rt[1].scores_init(s1);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const uint32_t ko = rt[0].k_off0 ^ (uint32_t)(c << 6);
    const Op kf0 = *(const Op*)(tile + ko);
    const Op kf1 = *(const Op*)(tile + ko + 4096);
    rt[0].scores_step(c, kf0, kf1, s0);
    rt[1].scores_step(c, kf0, kf1, s1);
    if (RT::kQuant && c < 3) __builtin_amdgcn_sched_barrier(0);  // (the fragments are read as they are needed: no register to spare)
  }
  Op pf0[RT::kU], pf1[RT::kU];
  float alpha0, alpha1;
  bool moved0, moved1;
  if constexpr (RT::kQuant) {
    // The per-token factors live as briefly as they can (the kernel has no register to spare): the two
    // that turn scores into exponents are loaded, used for both row tiles and dropped; the third is
    // loaded for the sums.
    float x0[RT::kN], x1[RT::kN];
    rt[0].load_factor(tile, 0, kscl);
    rt[0].load_factor(tile, 1, lv);
    rt[0].template scaled_scores<MASKED>(s0, kscl, lv, tb, scale_log2, x0);
    rt[1].template scaled_scores<MASKED>(s1, kscl, lv, tb, scale_log2, x1);
    __builtin_amdgcn_sched_barrier(0);
    rt[0].load_factor(tile, 2, rvs);
    moved0 = rt[0].template weights<MASKED>(x0, rvs, scale_log2, pf0, alpha0);
    __builtin_amdgcn_sched_barrier(0);
    moved1 = rt[1].template weights<MASKED>(x1, rvs, scale_log2, pf1, alpha1);
  } else {
    moved0 = rt[0].template softmax<MASKED>(s0, kscl, lv, rvs, tb, scale_log2, pf0, alpha0);
    __builtin_amdgcn_sched_barrier(0);  // one softmax at a time: interleaving the two costs registers
    moved1 = rt[1].template softmax<MASKED>(s1, kscl, lv, rvs, tb, scale_log2, pf1, alpha1);
  }
  if (moved0 || moved1) {  // the factor of a tile whose maxima stayed is exactly 1
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      const Op vf = rt[0].v_fragment(tile, dt);
      rt[0].template accumulate_step<true>(dt, vf, pf0, alpha0);
      rt[1].template accumulate_step<true>(dt, vf, pf1, alpha1);
    }
    rt[0].template accumulate_weights<true>(pf0, alpha0);
    rt[1].template accumulate_weights<true>(pf1, alpha1);
  } else {
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      const Op vf = rt[0].v_fragment(tile, dt);
      rt[0].template accumulate_step<false>(dt, vf, pf0, alpha0);
      rt[1].template accumulate_step<false>(dt, vf, pf1, alpha1);
    }
    rt[0].template accumulate_weights<false>(pf0, alpha0);
    rt[1].template accumulate_weights<false>(pf1, alpha1);
  }
}

// The lane's index within its wave, counted afresh (after the token loop: threadIdx.x would otherwise
// hold a register through it).
__device__ inline int lane_id() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

// End of an item: the TW waves that share a set of 16 query rows exchange (m, l, acc) through LDS
// (each wave's own region `xch_base + wave * xch_stride` of 16 rows of head_dim floats + 16 bytes), then each finishes head_dim/TW columns:
// a sequence that is a single chunk gets its bf16 output rows (and LSE) written directly, a split
// sequence a normalised fp32 partial and its log2-sum-exp.  `row_set` says which 16 rows of the item
// these are.  All waves of the workgroup must call it.
template <int KV_DT, int TOK, int TW, class RT>
__device__ inline void finish_item(const DecodeParams& p, const Item& it, RT& rt, uint8_t* xch_base,
                                   int xch_stride, float* lds_ml, int wave, int rs, int tw, int lane, int row_set) {
  constexpr bool kOffset = RT::kOffset;
  constexpr int kD = head_dim_of(TOK);
  constexpr int kXchRow = xch_row_bytes(TOK);
  const float neg_inf = -INFINITY;
  const int mi = lane & 15, kg = lane >> 4;
  const int nhq = p.n * p.num_q_heads;
  const bool single = p.implicit_plan != 0 || (p.direct_single != 0 && it.chunks == 1);
  const float l = kg_sum(rt.l_run);
  uint8_t* mine = xch_base + wave * xch_stride;
#pragma unroll
  for (int dt = 0; dt < kD / 16; ++dt) {
    f32x4 o = rt.acc[dt];
    if (TOK == 2) o += rt.acc[dt + 4];  // the two tokens of a row accumulated into separate tiles
    if (kOffset) o -= kInt8Offset * rt.wacc[0];  // every element of wacc holds the row's sum
    *(f32x4*)(mine + mi * kXchRow + (dt * 16 + 4 * kg) * 4) = o;
  }
  if (kg == 0) {
    lds_ml[(wave * 16 + mi) * 2] = rt.m_run;
    lds_ml[(wave * 16 + mi) * 2 + 1] = l;
  }
  __syncthreads();

  const int col = mi;  // query row handled in the combine
  float m_all = neg_inf;
#pragma unroll
  for (int s = 0; s < TW; ++s) m_all = fmaxf(m_all, lds_ml[((rs * TW + s) * 16 + col) * 2]);
  const float m_safe = m_all == neg_inf ? 0.0f : m_all;
  float wgt[TW];
  float l_all = 0.0f;
#pragma unroll
  for (int s = 0; s < TW; ++s) {
    wgt[s] = __builtin_amdgcn_exp2f(lds_ml[((rs * TW + s) * 16 + col) * 2] - m_safe);
    l_all += wgt[s] * lds_ml[((rs * TW + s) * 16 + col) * 2 + 1];
  }
  const int r = it.rg * p.rows_per_item + row_set * 16 + col;
  if (r >= it.n * p.group) return;
  const int j = r / p.group;
  const int head = it.hk * p.group + (r - j * p.group);
  const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
  const float lse2 = l_all > 0.0f ? m_all + __builtin_amdgcn_logf(l_all) : neg_inf;
  const int64_t tok = (int64_t)it.q0 + j;
  const int64_t prow = (int64_t)it.sc * nhq + (int64_t)j * p.num_q_heads + head;
  constexpr int kCols = kD / TW;  // columns this wave finishes: 8 per lane and pass
  constexpr int kPasses = kCols >= 32 ? kCols / 32 : 1;
  if (kCols < 32 && 8 * kg >= kCols) return;
#pragma unroll
  for (int pass = 0; pass < kPasses; ++pass) {
    const int d0 = kCols * tw + 32 * pass + 8 * kg;
    f32x4 o_lo = {0, 0, 0, 0}, o_hi = {0, 0, 0, 0};
#pragma unroll
    for (int s = 0; s < TW; ++s) {
      const uint8_t* src = xch_base + (rs * TW + s) * xch_stride + col * kXchRow + d0 * 4;
      o_lo += wgt[s] * *(const f32x4*)(src);
      o_hi += wgt[s] * *(const f32x4*)(src + 16);
    }
    o_lo *= inv;
    o_hi *= inv;
    if (single) {
      typename MmaOps<qf16_of(KV_DT)>::Op ob;  // the output has the queries' type
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ob[e] = (decltype(ob[0] + ob[0]))o_lo[e];
        ob[4 + e] = (decltype(ob[0] + ob[0]))o_hi[e];
      }
      *(decltype(ob)*)((uint16_t*)p.out + tok * p.out_token_stride + (int64_t)head * kD + d0) = ob;
    } else if (p.fused_merge) {
      float* po = p.partial_out + prow * kD + d0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        store_coherent(po + e, o_lo[e]);
        store_coherent(po + 4 + e, o_hi[e]);
      }
    } else {
      float* po = p.partial_out + prow * kD + d0;
      *(f32x4*)(po) = o_lo;
      *(f32x4*)(po + 4) = o_hi;
    }
  }
  if (tw == 0 && kg == 0) {
    if (single) {
      if (p.lse != nullptr) p.lse[tok * p.num_q_heads + head] = lse2;
    } else if (p.fused_merge) {
      store_coherent(p.partial_lse + prow, lse2);
    } else {
      p.partial_lse[prow] = lse2;
    }
  }
}

// Token range of an item after the sliding window has removed the tiles no row can see.
__device__ inline int first_visible_tile(const DecodeParams& p, const Item& it) {
  int t0 = it.t_begin;
  if (p.window_left >= 0) {
    int first = it.len - it.n - p.window_left;  // window start of the earliest query row
    first = first > 0 ? first : 0;
    first &= ~(p.tile_tokens - 1);
    t0 = t0 > first ? t0 : first;
  }
  return t0;
}

// Waves per SIMD the 16-row kernel is compiled for: head_dim 256 needs the registers of one.
constexpr int decode_waves_per_simd(int tok) { return tok == 0 ? 1 : 2; }

// HEADS (with DecodeParams::wave_items: four neighbouring work items, one per wave, or two of two waves each; for steps
// that are not split, and the latter over any schedule, the merge kernel combining what is split): a work item covers kWaves neighbouring kv heads of a sequence chunk and wave w attends head
// it.hk + w over all of the chunk's tokens (instead of the four waves sharing one head's tokens).  For a
// cache whose kv heads lie side by side within a token (the NHD layout) the workgroup then reads runs of
// four rows — 512 bytes of a 1-byte cache — at about the same time, where a workgroup per head reads
// 128-byte rows at a 1 KiB stride; a plain streaming kernel measures 6.8 TB/s for the first pattern
// and 5.5 TB/s for the second on this part.  Every wave finishes its own 16 rows: no exchange between waves.
//
// WAVES: waves that share an item's tokens.  Four, two workgroups to a CU, when the launch has work items
// for that; eight (one such workgroup fills a CU: its tiles take 134 KiB of LDS) when a launch over a
// 1-byte cache has at most one item per CU, as a small batch cut into 32 chunks per sequence has: a wave
// has one tile in flight and converts it before it asks for the next, so four waves leave the CU's memory
// pipe idle much of the time, and cutting finer instead costs more in the merge than it gains.
//
// LOCK (with HEADS, for cache rows shorter than a 128-byte line whose neighbour in the line is the next kv head's
// row, which another wave of the workgroup attends): the four waves meet before every tile and load with ordinary
// loads, so that the two halves of a line are asked for at about the same time, the second finds it in the CU's
// cache, and the line crosses HBM once.
template <int KV_DT, int TOK, bool HEADS = false, int WAVES = kWaves, bool LOCK = false>
__global__ void __launch_bounds__(64 * WAVES, decode_waves_per_simd(TOK)) decode_mfma_d128_kernel(DecodeParams p) {
  static_assert(!(HEADS && WAVES != kWaves) && !(TOK == 0 && WAVES != kWaves), "eight waves: head_dim 64 and 128, one kv head per item");
  static_assert(!LOCK || HEADS, "in step: waves that attend neighbouring kv heads");
  __shared__ __attribute__((aligned(16))) uint8_t lds_all[WAVES * kLdsTile];
  __shared__ float lds_ml[WAVES * 16 * 2];  // (running max, denominator) per wave and query row
  __shared__ int lds_last;

  constexpr int kT = tile_tokens_of(TOK);  // tokens per tile
  constexpr int kH = half_tokens_of(TOK);  // tokens from the tile's first half to its second
  constexpr int kP1 = TOK == 0 ? 1 : 0;    // head_dim 256: the second half is the same tokens' second plane
  static_assert(16 * xch_row_bytes(TOK) <= kLdsTile, "the end-of-item exchange must fit a wave's tile");

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // uniform: keeps the loop scalar
  Item it;
  // (wave_items: 1 — every wave a work item of its own —, or 2: two waves share an item's tokens, two items to the workgroup)
  const int item_waves = HEADS ? __builtin_amdgcn_readfirstlane(p.wave_items) : 0;
  if (HEADS && item_waves) {
    // Neighbours in the order of the items (kv head fastest), whatever the head count.  A wave past the
    // last item keeps step with the others — they meet in a barrier at the end — as an item without rows
    // or tokens.
    const int vid = item_waves == 2 ? (int)blockIdx.x * 2 + (wave >> 1) : (int)blockIdx.x * kWaves + wave;
    if (!decode_item(p, vid, it)) {
      it = Item{};
      it.ids = p.block_ids;
      it.nblk = 1;
      it.chunks = 1;
    }
  } else {
    if (!decode_item(p, blockIdx.x, it)) return;
    if (HEADS) {
      it.hk += wave;
      it.head_off = (int64_t)it.hk * p.stride_head;
      it.sc_head_off = (int64_t)it.hk * p.sc_stride_head;
    }
  }
  const int lane = threadIdx.x & 63;
  uint8_t* tile = lds_all + wave * kLdsTile;  // this wave's private K/V tile

  constexpr bool kRawK = raw_k_of(KV_DT, TOK);
  typedef RowTile<KV_DT, TOK> RT;
  RT rt;
  rt.init(p, it, 0, lane);  // (the four waves hold the same rows, or each its head's)
  const float park_scale = p.scale_log2;

  // This wave's share of the item's tokens.
  const int t0 = first_visible_tile(p, it);
  const int span = it.t_end - t0;
  const int sharers = !HEADS ? WAVES : item_waves == 2 ? 2 : 1;  // waves that split the item's tokens
  const int share = span <= 0 ? 0 : (((span + sharers - 1) / sharers + kT - 1) & ~(kT - 1));
  const int w_begin = !HEADS ? t0 + wave * share : item_waves == 2 ? t0 + (wave & 1) * share : t0;
  const int w_end = min(it.t_end, w_begin + share);
  const int mask_hi_from = it.len - (it.n - 1);                                    // tiles reaching past this need masks
  const int mask_lo_until = p.window_left >= 0 ? it.len - 1 - p.window_left : 0;  // tiles starting below this too

  typename KvHalf<KV_DT>::Geom geom;
  geom.init(p, lane, TOK);
  // One register stage: the loads of tile i+1 are in flight while tile i is consumed.  (More stages were
  // slower wherever they were tried: two for the 1-byte caches of head_dim 256, which run one wave per
  // SIMD and so have few bytes in flight per CU, 458 against 367 us on 64 x 8192 tokens of fp8 — the
  // registers they take are paid for in copies between the two register files; two for 16-bit caches
  // at one wave per SIMD no better than one at two.)
  KvHalf<KV_DT> st[2];  // the two halves (16 rows each) of the tile in flight
  int blk[2];           // block ids of the halves loaded next, fetched a round earlier

  // Tile at tb: park it, put the next tile in flight, attend.  The scalar loads of the ids go out
  // before the tile is parked: they share a counter with the LDS traffic, so the next wait on LDS
  // also waits for them.
  auto step = [&](int tb) {
    const bool masked = (tb + kT > mask_hi_from) || (tb < mask_lo_until);
    const int nblk0 = block_of(p, it, tb + 2 * kT);
    const int nblk1 = block_of(p, it, tb + 2 * kT + kH);
    if (masked) {
      st[0].template park<true, kRawK>(tile, 0, tb, it.len, park_scale, geom);
      st[1].template park<true, kRawK>(tile, 1, tb + kH, it.len, park_scale, geom);
    } else {
      st[0].template park<false, kRawK>(tile, 0, tb, it.len, park_scale, geom);
      st[1].template park<false, kRawK>(tile, 1, tb + kH, it.len, park_scale, geom);
    }
    if (tb + kT < w_end) {
      st[0].template issue<LOCK>(p, it, tb + kT, blk[0], geom);
      st[1].template issue<LOCK>(p, it, tb + kT + kH, blk[1], geom, kP1);
    }
    blk[0] = nblk0;
    blk[1] = nblk1;
    if (masked) {
      rt.template attend<true>(tile, tb, p.scale_log2);
    } else {
      rt.template attend<false>(tile, tb, p.scale_log2);
    }
  };
  if constexpr (LOCK) {
    // In step: every wave walks as many tiles as the workgroup's longest share has, and the four meet before
    // each — every wave reaches every barrier, with or without a tile of its own.
    __shared__ int lds_tiles[kWaves];
    if (lane == 0) lds_tiles[wave] = w_begin < w_end ? (w_end - w_begin + kT - 1) / kT : 0;
    __syncthreads();
    const int tiles = __builtin_amdgcn_readfirstlane(max(max(lds_tiles[0], lds_tiles[1]), max(lds_tiles[2], lds_tiles[3])));
    if (w_begin < w_end) {
      st[0].template issue<LOCK>(p, it, w_begin, block_of(p, it, w_begin), geom);
      st[1].template issue<LOCK>(p, it, w_begin + kH, block_of(p, it, w_begin + kH), geom, kP1);
      blk[0] = block_of(p, it, w_begin + kT);
      blk[1] = block_of(p, it, w_begin + kT + kH);
    }
    int tb = w_begin;
    for (int i = 0; i < tiles; ++i, tb += kT) {
      __builtin_amdgcn_s_barrier();
      if (tb < w_end) step(tb);
    }
  } else if (w_begin < w_end) {
    st[0].template issue<LOCK>(p, it, w_begin, block_of(p, it, w_begin), geom);
    st[1].template issue<LOCK>(p, it, w_begin + kH, block_of(p, it, w_begin + kH), geom, kP1);
    blk[0] = block_of(p, it, w_begin + kT);
    blk[1] = block_of(p, it, w_begin + kT + kH);
    for (int tb = w_begin; tb < w_end; tb += kT) step(tb);
  }
  // The merge reads its arguments afresh from the kernel-argument segment (DecodeParams is the kernel's
  // only argument: it sits at the start of that segment), through a pointer the compiler cannot see
  // through: handed `p` itself, it loads every field the merge uses at the kernel's entry and keeps
  // them in scalar registers across the token loop, which then runs out of them (scalars get parked in
  // vector-register lanes and are fetched back with one vector operation each: 32 per tile in the
  // 1-byte kernels).  The pointer is formed here, ahead of the end-of-item exchange, so that the
  // loads are under way while the waves exchange their results.
  const __attribute__((address_space(4))) DecodeParams* pm =
      (const __attribute__((address_space(4))) DecodeParams*)__builtin_amdgcn_kernarg_segment_ptr();
  asm volatile("" : "+s"(pm));
  if constexpr (HEADS) {
    if (item_waves == 2) {
      finish_item<KV_DT, TOK, 2>(p, it, rt, lds_all, kLdsTile, lds_ml, wave, wave >> 1, wave & 1, lane_id(), 0);
    } else {
      finish_item<KV_DT, TOK, 1>(p, it, rt, lds_all, kLdsTile, lds_ml, wave, wave, 0, lane_id(), 0);
    }
  } else {
    finish_item<KV_DT, TOK, WAVES>(p, it, rt, lds_all, kLdsTile, lds_ml, wave, 0, wave, lane_id(), 0);
  }
  // (32 rows in flight make the int8 head_dim-64 instantiation spill)
  // (work items of several kv heads leave their split sequences to the merge kernel)
  if constexpr (!HEADS) {
    merge_if_last<qf16_of(KV_DT) ? XLLM_HIP_FP16 : XLLM_HIP_BF16, TOK == 0 ? 4 : 2, (TOK == 2 && quant_of(KV_DT)) ? 16 : 32>(*pm, it, &lds_last, wave, lane_id());
  }
}

// head_dim 256 over a 16-bit cache: one wave per SIMD (its two tile stages alone are 64 registers).
constexpr int rows32_waves_per_simd(int kv_dt, int tok) { return tok == 0 && !quant_of(kv_dt) ? 1 : 2; }

// PAIRS = 4: a work item of four kv heads whose rows lie side by side within a token (a 1-byte cache in the NHD
// layout), one pair of waves per head, eight waves to the workgroup and one such workgroup to a CU: the four pairs
// walk the same tokens in step (they meet at every tile's barrier), so that what the workgroup asks of memory at
// a time is a run of four rows, 512 bytes, instead of single rows a token's width apart.
template <int KV_DT, int TOK, int PAIRS = 1>
__global__ void __launch_bounds__(128 * PAIRS, rows32_waves_per_simd(KV_DT, TOK)) decode_mfma_d128_rows32_kernel(DecodeParams p) {
  // A pair of waves: wave w of it owns query rows 16w .. 16w+15 and fetches rows 16w ..
  // of every tile.  A tile is parked while both waves still read the previous one from the other
  // buffer, so one barrier per tile suffices.  Four such pairs share a CU.
  __shared__ __attribute__((aligned(16))) uint8_t lds_pairs[PAIRS * 2 * kLdsTile];
  __shared__ float lds_ml_pairs[PAIRS * 2 * 16 * 2];

  constexpr int kT = tile_tokens_of(TOK);  // tokens per tile
  constexpr int kH = half_tokens_of(TOK);  // tokens from the tile's first half to its second
  constexpr int kP1 = TOK == 0 ? 1 : 0;    // head_dim 256: the second half is the same tokens' second plane
  static_assert(16 * xch_row_bytes(TOK) <= kLdsTile, "the end-of-item exchange must fit a wave's tile");

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave_of_group = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int pair = PAIRS > 1 ? wave_of_group >> 1 : 0;
  const int wave = wave_of_group & 1;  // within the pair
  const int rs = wave;  // row set; also the tile half this wave fetches
  const int lane = threadIdx.x & 63;
  uint8_t* lds_all = lds_pairs + pair * (2 * kLdsTile);
  float* lds_ml = lds_ml_pairs + pair * (2 * 16 * 2);
  uint8_t* tiles = lds_all;
  if (PAIRS > 1) {  // (the item names the first of its kv heads)
    it.hk += pair;
    it.head_off = (int64_t)it.hk * p.stride_head;
    it.sc_head_off = (int64_t)it.hk * p.sc_stride_head;
  }

  constexpr bool kRawK = raw_k_of(KV_DT, TOK);
  constexpr bool kInt8 = kv_of(KV_DT) == XLLM_HIP_INT8;
  RowTile<KV_DT, TOK, kRawK, kInt8, kInt8 && !kRawK, rows32_waves_per_simd(KV_DT, TOK) == 2 && TOK == 0> rt;
  rt.init(p, it, 16 * rs, lane);
  const float park_scale = p.scale_log2;

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;
  const int mask_hi_from = it.len - (it.n - 1);
  const int mask_lo_until = p.window_left >= 0 ? it.len - 1 - p.window_left : 0;

  typename KvHalf<KV_DT>::Geom geom;
  geom.init(p, lane, TOK);
  // kDepth register stages, used in turn: the loads of tiles i+1 .. i+kDepth are in flight while tile
  // i is consumed (a wave fetches only half a tile, so one stage would leave too few bytes in flight
  // per CU to cover the HBM latency; four stages for head_dim 256, which runs one wave per SIMD,
  // were slower than two).  Both waves run the same iterations.
  constexpr int kDepth = 2;  // (the loop below is written out for two)
  KvHalf<KV_DT> mine[kDepth];  // the 16 rows this wave fetches: rows 16*rs .. of the tile
  int blk[kDepth];             // block id of the half each stage loads next, fetched a round earlier

  auto issue = [&](KvHalf<KV_DT>& m, int b, int tb) {
    if (tb < w_end) m.issue(p, it, tb + kH * rs, b, geom, kP1 * rs);
  };
  // `b`: block id of the half this wave fetches kDepth tiles on; replaced by that of the tile
  // 2 * kDepth on.  The scalar load goes out before the tile is parked: it shares a counter with the
  // LDS traffic, so the wait before the barrier also waits for it.
  auto step = [&](KvHalf<KV_DT>& m, int& b, int i) {
    const int tb = w_begin + i * kT;
    const int nblk = block_of(p, it, tb + 2 * kDepth * kT + kH * rs);
    uint8_t* tile = tiles + (i & 1) * kLdsTile;
    const bool masked = (tb + kT > mask_hi_from) || (tb < mask_lo_until);
    if (masked) {
      m.template park<true, kRawK>(tile, rs, tb + kH * rs, it.len, park_scale, geom);
    } else {
      m.template park<false, kRawK>(tile, rs, tb + kH * rs, it.len, park_scale, geom);
    }
    issue(m, b, tb + kDepth * kT);
    b = nblk;
    __syncthreads();  // both halves of tile i are parked; both waves are done with tile i-1
    if (masked) {
      rt.template attend<true>(tile, tb, p.scale_log2);
    } else {
      rt.template attend<false>(tile, tb, p.scale_log2);
    }
  };
  if (iters > 0) {  // (an item without visible tokens reads no block id: its list may be empty)
#pragma unroll
    for (int d = 0; d < kDepth; ++d) {
      issue(mine[d], block_of(p, it, w_begin + d * kT + kH * rs), w_begin + d * kT);
      blk[d] = block_of(p, it, w_begin + (kDepth + d) * kT + kH * rs);
    }
  }
  for (int i = 0; i < iters; i += kDepth) {
    step(mine[0], blk[0], i);
    if (i + 1 < iters) step(mine[1], blk[1], i + 1);
  }
  __syncthreads();  // all tiles consumed before the buffers are reused for the exchange
  finish_item<KV_DT, TOK, 1>(p, it, rt, lds_all, kLdsTile, lds_ml, wave, rs, 0, lane_id(), rs);
}

// Many query rows per kv head (prefill chunks, long verify steps) over a 16-bit cache: a workgroup is
// four waves and 128 query rows of one (sequence, kv head); wave w owns rows 32w .. 32w+31 as two row
// tiles, so every K and V fragment it reads from LDS feeds two MFMAs.  All four waves walk the
// item's tokens together, one tile per step.  The tile needs no conversion, so it goes from global
// memory straight into LDS (global_load_lds, 16 bytes per lane): no staging registers, no park.
// Such a load writes the wave's 64 pieces to consecutive LDS addresses, i.e. four whole rows; the
// swizzle is applied on the global side (lane = (row, position) fetches the piece that belongs at
// that position).  Wave w fetches rows 8w .. 8w+7 of K and of V.  Four tile buffers rotate: tiles
// i+1 .. i+3 are in flight while tile i is read.  Each buffer is an LDS array of its own and the
// loop is unrolled over them, so that the compiler can tell the loads in flight from the buffer
// being read and does not wait for them.  With causal rows a wave skips the tiles none of its rows
// can see.  Two such workgroups share a CU.
constexpr int kPrefillBuffers = 4;
constexpr int kPrefillTile = 16896;  // 16 KiB of K and V; as the end-of-item exchange 16 rows of 528 bytes

#define XLLM_HIP_GLOBAL_TO_LDS_16(gptr, lptr)                                                   \
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr),       \
                                   (__attribute__((address_space(3))) void*)(lptr), 16, 0, 0)

template <int KV_DT, int TOK>
struct PrefillLoader {
  int wave, lane;

  // Load q (0, 1) covers rows 4q .. 4q+3 of the wave's eight: token (within the wave's 8 * TOK)
  // and byte offset of the piece this lane fetches for position lane % 16 of its row.
  // Recomputed at every use — a few integer operations — rather than held in registers.
  __device__ inline void piece(int q, bool v, int& tok, int& byte) const {
    int lane = this->lane;
    asm volatile("" : "+v"(lane));  // keeps the compiler from hoisting these out of the loop and then spilling them
    const int row8 = 4 * q + (lane >> 4);
    const int row = 8 * wave + row8;  // row of the tile
    const int pos = lane & 15;
    const int lp = v ? pos ^ (((row & 7) << 1) | ((row >> 3) & 1))  // see swz_v
                     : pos ^ (row & 15);                             // see swz_k
    constexpr int kPerTok = 16 / TOK;  // pieces per token
    tok = row8 * TOK + lp / kPerTok;
    byte = (lp % kPerTok) * 16;
  }
  __device__ inline uint32_t offset(const DecodeParams& p, int q, bool v) const {
    int tok, byte;
    piece(q, v, tok, byte);
    return (uint32_t)(tok * p.stride_slot * 2 + byte);
  }

  // Loads of the wave's rows of the tile starting at token tb into `buf` (in flight on return).
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int blk, uint8_t* buf) const {
    const HalfBase b = half_base(p, it, tb + 8 * TOK * wave, blk);
    const uint8_t* kb = p.k_cache + b.elem * 2;
    const uint8_t* vb = p.v_cache + b.elem * 2;
    uint8_t* kl = buf + kLdsK + 2048 * wave;
    uint8_t* vl = buf + kLdsV + 2048 * wave;
    XLLM_HIP_GLOBAL_TO_LDS_16(kb + offset(p, 0, false), kl);
    XLLM_HIP_GLOBAL_TO_LDS_16(kb + offset(p, 1, false), kl + 1024);
    XLLM_HIP_GLOBAL_TO_LDS_16(vb + offset(p, 0, true), vl);
    XLLM_HIP_GLOBAL_TO_LDS_16(vb + offset(p, 1, true), vl + 1024);
  }

  // Zeros over the V pieces of tokens at or past the sequence end (after the loads have landed):
  // whatever those slots hold must not reach the MFMA, where even a weight of zero times NaN is NaN.
  __device__ inline void clear_tail(int tb, int len, uint8_t* buf) const {
    const int first = tb + 8 * TOK * wave;
    uint32_t z = 0;
    asm volatile("" : "+v"(z));  // made here, on the rare path, instead of living in registers through the loop
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      int tok, byte;
      piece(q, true, tok, byte);
      if (first + tok >= len) *(u32x4*)(buf + kLdsV + 2048 * wave + 1024 * q + lane * 16) = u32x4{z, z, z, z};
    }
  }
};

template <int KV_DT, int TOK>
__global__ void __launch_bounds__(256, 2) prefill_mfma_d128_kernel(DecodeParams p) {
  static_assert(!quant_of(KV_DT), "a 1-byte cache needs converting on the way into LDS");
  __shared__ __attribute__((aligned(16))) uint8_t buf0[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf1[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf2[kPrefillTile];
  __shared__ __attribute__((aligned(16))) uint8_t buf3[kPrefillTile];
  __shared__ float lds_ml[4 * 16 * 2];
  static_assert(TOK != 0, "head_dim 256 does not fit two row tiles per wave");
  constexpr int kT = 32 * TOK;  // tokens per tile

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;

  RowTile<KV_DT, TOK> rt[2];
  rt[0].init(p, it, 32 * wave, lane);
  rt[1].init(p, it, 32 * wave + 16, lane);

  // What this wave's rows can see: row r belongs to query token r / group, which sees the tokens
  // below lim(j) = len - (n - 1 - j) and, with a sliding window, from lim(j) - 1 - window_left on.
  const int rows = it.n * p.group;
  const int r_first = it.rg * p.rows_per_item + 32 * wave;
  const bool has_rows = r_first < rows;
  const int r_last = min(r_first + 31, rows - 1);
  const int lim_first = it.len - (it.n - 1 - r_first / p.group);
  const int lim_last = has_rows ? it.len - (it.n - 1 - r_last / p.group) : 0;
  const int lo_first = p.window_left >= 0 ? lim_first - 1 - p.window_left : 0;
  const int lo_last = p.window_left >= 0 ? lim_last - 1 - p.window_left : 0;

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;

  PrefillLoader<KV_DT, TOK> ld;
  ld.wave = wave;
  ld.lane = lane;
  const int mine = 8 * TOK * wave;  // first of the tokens this wave fetches, within a tile

  // Tile i: wait for this wave's share of it (tiles i+1 and i+2 stay in flight), meet the other
  // waves — their shares have landed too, and everyone is done with tile i-1, whose buffer `next`
  // is — then put tile i+3 in flight into `next` and attend tile i from `buf`.  Every step issues
  // its four loads, also past the end of the item (block_of keeps those inside the sequence's
  // blocks; nobody reads them): the count of loads in flight is then the same on every path, which
  // is what lets the compiler, too, wait for exactly the buffer it reads.
  auto step = [&](int i, uint8_t* buf, uint8_t* next, int& blk) {
    const int tb = w_begin + i * kT;
    const int nblk = block_of_const(p, it, tb + 4 * kT + mine);
    // (the builtin, not asm with a memory clobber: after such a clobber the block ids would no
    // longer come through scalar loads, and a vector load's wait would cover the tiles in flight)
    __builtin_amdgcn_s_waitcnt(0x0f78);  // vmcnt(8)
    if (tb + kT > it.len) ld.clear_tail(tb, it.len, buf);
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the zeros above are in LDS
    __builtin_amdgcn_s_barrier();
    ld.issue(p, it, tb + 3 * kT, blk, next);
    blk = nblk;
    if (!(tb >= lim_last || tb + kT <= lo_first)) {  // else: nothing here for this wave's rows
      if (tb + kT > lim_first || tb < lo_last) {
        attend_pair<true>(rt, buf, tb, p.scale_log2);
      } else {
        attend_pair<false>(rt, buf, tb, p.scale_log2);
      }
    }
  };
  if (iters > 0) {  // (an item without visible tokens touches no block: its table row may hold anything)
    ld.issue(p, it, w_begin, block_of_const(p, it, w_begin + mine), buf0);
    ld.issue(p, it, w_begin + kT, block_of_const(p, it, w_begin + kT + mine), buf1);
    ld.issue(p, it, w_begin + 2 * kT, block_of_const(p, it, w_begin + 2 * kT + mine), buf2);
    int blk = block_of_const(p, it, w_begin + 3 * kT + mine);
    int i = 0;
    for (; i + 4 <= iters; i += 4) {
      step(i, buf0, buf3, blk);
      step(i + 1, buf1, buf0, blk);
      step(i + 2, buf2, buf1, blk);
      step(i + 3, buf3, buf2, blk);
    }
    if (i < iters) step(i, buf0, buf3, blk);
    if (i + 1 < iters) step(i + 1, buf1, buf0, blk);
    if (i + 2 < iters) step(i + 2, buf2, buf1, blk);
  }
  __syncthreads();  // all tiles consumed before the buffers are reused for the exchange
  uint8_t* xch = wave == 0 ? buf0 : wave == 1 ? buf1 : wave == 2 ? buf2 : buf3;
  finish_item<KV_DT, TOK, 1>(p, it, rt[0], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave);
  __syncthreads();
  finish_item<KV_DT, TOK, 1>(p, it, rt[1], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave + 1);
}

// Many query rows per kv head over a 1-byte cache (head_dim 128): the structure of prefill_mfma_d128_kernel
// with a conversion stage.  A tile's bytes go from global memory straight into a raw LDS buffer (16 bytes
// per lane, each wave the eight rows of K and of V it owns, plus their fp32 scales), four raw buffers
// rotate (tiles i+1 .. i+3 in flight); a wave then converts its own rows — it reads back exactly the bytes
// it fetched — into one of two converted tiles in the layout the MFMA operand reads expect, with the
// per-token factors of the softmax, the waves meet, and all four attend the converted tile with two
// row tiles each.  The conversion is paid once per 128 query rows instead of once per 32.
constexpr int kQuantRawTile = 8192 + 1024;  // K and V bytes of 32 tokens, 4 x 256 bytes of scale loads

#define XLLM_HIP_GLOBAL_TO_LDS_4(gptr, lptr)                                                    \
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(gptr),       \
                                   (__attribute__((address_space(3))) void*)(lptr), 4, 0, 0)

template <int KV_DT>
struct QuantPrefillLoader {
  int wave, lane;

  // Row (of the wave's eight) and 16-byte chunk of the row this lane fetches and converts: lanes in
  // quads, so that the eight lanes of an LDS write group hold pieces of two neighbouring rows (the K
  // swizzle then spreads them over all banks).  Recomputed at every use rather than held in registers.
  __device__ inline void row_chunk(int& row8, int& chunk) const {
    int l = lane;
    asm volatile("" : "+v"(l));
    chunk = 4 * ((l >> 3) & 1) + (l & 3);
    row8 = 2 * (l >> 4) + ((l >> 2) & 1);
  }

  // Loads of the wave's rows of the tile starting at token tb into `raw` (in flight on return): three
  // instructions, K bytes, V bytes, scales (lanes 0-7 the K scales of the eight tokens, 8-15 the V scales).
  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int blk, uint8_t* raw) const {
    const HalfBase b = half_base(p, it, tb + 8 * wave, blk);
    int row8, chunk;
    row_chunk(row8, chunk);
    const uint32_t off = (uint32_t)(row8 * p.stride_slot + chunk * 16);
    XLLM_HIP_GLOBAL_TO_LDS_16(p.k_cache + b.elem + off, raw + 1024 * wave);
    XLLM_HIP_GLOBAL_TO_LDS_16(p.v_cache + b.elem + off, raw + 4096 + 1024 * wave);
    int l = lane;
    asm volatile("" : "+v"(l));
    const float* sp = ((l & 8) ? p.v_scale : p.k_scale) + b.scale + (int64_t)((l & 7) * p.sc_stride_slot);
    XLLM_HIP_GLOBAL_TO_LDS_4(sp, raw + 8192 + 256 * wave);
  }

  // The wave's rows of the tile at tb: raw -> converted (K, V, per-token factors); see KvHalfQuant::park.
  // `lds_scale` (LDS_SCALE): where the factor of the K scales is kept in LDS instead of in `scale_log2`, for a
  // kernel with no scalar register to spare for it through the token loop.
  template <bool MASKED, bool LDS_SCALE = false>
  __device__ inline void convert(const uint8_t* raw, uint8_t* conv, int tb, int len, float scale_log2,
                                 const float* lds_scale = nullptr) const {
    int row8, chunk;
    row_chunk(row8, chunk);
    const int row = 8 * wave + row8;
    const u32x4 kraw = *(const u32x4*)(raw + 1024 * wave + lane * 16);
    const u32x4 vraw = *(const u32x4*)(raw + 4096 + 1024 * wave + lane * 16);
    u32x4 klo, khi, vlo, vhi;
    dequant16<KV_DT>(kraw, klo, khi);
    dequant16<KV_DT>(vraw, vlo, vhi);
    if constexpr (kv_of(KV_DT) == XLLM_HIP_INT8) {
      // 1152 + x -> x, exact in fp16 (paid once per 128 query rows here, it saves every row tile the
      // bookkeeping of the offset: an MFMA per tile and its accumulator)
      // (V only: the offset of the K rows leaves the scores through the MFMA's initial C operand)
      auto exact = [](u32x4& v) { v = __builtin_bit_cast(u32x4, __builtin_bit_cast(f16x8, v) - (_Float16)kInt8Offset); };
      exact(vlo);
      exact(vhi);
    }
    if (MASKED && tb + row >= len) vlo = vhi = u32x4{0, 0, 0, 0};
    const uint32_t ko = kLdsK + swz_k(row, 2 * chunk), vo = kLdsV + swz_v(row, 2 * chunk);
    *(u32x4*)(conv + ko) = klo;
    *(u32x4*)(conv + (ko ^ 16)) = khi;
    *(u32x4*)(conv + vo) = vlo;
    *(u32x4*)(conv + (vo ^ 16)) = vhi;
    if (lane < 16) {
      if (LDS_SCALE) scale_log2 = *lds_scale;
      const float sc = *(const float*)(raw + 8192 + 256 * wave + lane * 4);
      const int t = 8 * wave + (lane & 7);  // token of the tile
      const bool is_v = lane >= 8;
      const float vs = fmaxf(sc, 0x1p-100f);
      float a = is_v ? __builtin_amdgcn_logf(vs) : sc * scale_log2;
      float r = __builtin_amdgcn_rcpf(vs);
      if (MASKED && tb + t >= len) a = r = 0.0f;
      *(float*)(conv + kLdsSc + (is_v ? 128 : 0) + t * 4) = a;
      if (is_v) *(float*)(conv + kLdsSc + 256 + t * 4) = r;
    }
  }
};

template <int KV_DT>
__global__ void __launch_bounds__(256, 2) prefill_quant_d128_kernel(DecodeParams p) {
  static_assert(quant_of(KV_DT), "16-bit caches need no conversion: prefill_mfma_d128_kernel");
  __shared__ __attribute__((aligned(16))) uint8_t raw0[kQuantRawTile];
  __shared__ __attribute__((aligned(16))) uint8_t raw1[kQuantRawTile];
  __shared__ __attribute__((aligned(16))) uint8_t raw2[kQuantRawTile];
  __shared__ __attribute__((aligned(16))) uint8_t raw3[kQuantRawTile];
  __shared__ __attribute__((aligned(16))) uint8_t conv0[kLdsTile];
  __shared__ __attribute__((aligned(16))) uint8_t conv1[kLdsTile];
  __shared__ float lds_ml[4 * 16 * 2];
  constexpr int kT = 32;
  static_assert(2 * 16 * xch_row_bytes(1) <= kLdsTile, "two waves' end-of-item exchanges must fit a converted tile");

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;

  typedef RowTile<KV_DT, 1, false, false, kv_of(KV_DT) == XLLM_HIP_INT8, false, false> RT;
  RT rt[2];
  int q_exp = 0;
  if constexpr (RT::kNormItem) {  // one factor for the queries of all four waves: they share the converted tile's factors
    lds_ml[wave] = fmaxf(RT::wave_q_absmax(p, it, 32 * wave, lane), RT::wave_q_absmax(p, it, 32 * wave + 16, lane));
    __syncthreads();
    q_exp = RT::norm_exponent(fmaxf(fmaxf(lds_ml[0], lds_ml[1]), fmaxf(lds_ml[2], lds_ml[3])));
    __syncthreads();
  }
  rt[0].init(p, it, 32 * wave, lane, q_exp);
  rt[1].init(p, it, 32 * wave + 16, lane, q_exp);
  // (the factor of the K scales waits in LDS, a word per wave: no scalar register is left to hold it through the loop)
  if constexpr (RT::kNormItem) lds_ml[4 + wave] = __builtin_amdgcn_ldexpf(p.scale_log2, q_exp);
  const float* lds_scale = lds_ml + 4 + wave;

  const int rows = it.n * p.group;
  const int r_first = it.rg * p.rows_per_item + 32 * wave;
  const bool has_rows = r_first < rows;
  const int r_last = min(r_first + 31, rows - 1);
  const int lim_first = it.len - (it.n - 1 - r_first / p.group);
  const int lim_last = has_rows ? it.len - (it.n - 1 - r_last / p.group) : 0;
  const int lo_first = p.window_left >= 0 ? lim_first - 1 - p.window_left : 0;
  const int lo_last = p.window_left >= 0 ? lim_last - 1 - p.window_left : 0;

  const int w_begin = first_visible_tile(p, it);
  const int w_end = it.t_end;
  const int iters = w_end > w_begin ? (w_end - w_begin + kT - 1) / kT : 0;

  QuantPrefillLoader<KV_DT> ld;
  ld.wave = wave;
  ld.lane = lane;
  const int mine = 8 * wave;  // first of the tokens this wave fetches, within a tile

  // Tile i: wait for this wave's three loads of it (tiles i+1 and i+2 stay in flight), convert its rows
  // from `raw` into `conv`, meet the other waves — their rows are converted too, and everyone is done
  // with the converted tile of step i-1 —, put tile i+3 in flight into `next` (which only this wave's
  // conversion of step i-1 read) and attend.  Every step issues its loads, also past the item's end.
  auto step = [&](int i, uint8_t* raw, uint8_t* next, uint8_t* conv, int& blk) {
    const int tb = w_begin + i * kT;
    const int nblk = block_of_const(p, it, tb + 4 * kT + mine);
    __builtin_amdgcn_s_waitcnt(0x0f76);  // vmcnt(6)
    if (tb + kT > it.len) {
      ld.template convert<true, RT::kNormItem>(raw, conv, tb, it.len, p.scale_log2, lds_scale);
    } else {
      ld.template convert<false, RT::kNormItem>(raw, conv, tb, it.len, p.scale_log2, lds_scale);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    ld.issue(p, it, tb + 3 * kT, blk, next);
    blk = nblk;
    if (!(tb >= lim_last || tb + kT <= lo_first)) {
      if (tb + kT > lim_first || tb < lo_last) {
        attend_pair<true>(rt, conv, tb, p.scale_log2);
      } else {
        attend_pair<false>(rt, conv, tb, p.scale_log2);
      }
    }
  };
  if (iters > 0) {
    ld.issue(p, it, w_begin, block_of_const(p, it, w_begin + mine), raw0);
    ld.issue(p, it, w_begin + kT, block_of_const(p, it, w_begin + kT + mine), raw1);
    ld.issue(p, it, w_begin + 2 * kT, block_of_const(p, it, w_begin + 2 * kT + mine), raw2);
    int blk = block_of_const(p, it, w_begin + 3 * kT + mine);
    int i = 0;
    for (; i + 4 <= iters; i += 4) {
      step(i, raw0, raw3, conv0, blk);
      step(i + 1, raw1, raw0, conv1, blk);
      step(i + 2, raw2, raw1, conv0, blk);
      step(i + 3, raw3, raw2, conv1, blk);
    }
    if (i < iters) step(i, raw0, raw3, conv0, blk);
    if (i + 1 < iters) step(i + 1, raw1, raw0, conv1, blk);
    if (i + 2 < iters) step(i + 2, raw2, raw1, conv0, blk);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): nothing lands in LDS any more
  __syncthreads();  // all tiles consumed before the buffers are reused for the exchange
  uint8_t* xch = (wave < 2 ? conv0 : conv1) + (wave & 1) * (16 * xch_row_bytes(1));
  finish_item<KV_DT, 1, 1>(p, it, rt[0], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave);
  __syncthreads();
  finish_item<KV_DT, 1, 1>(p, it, rt[1], xch, 0, lds_ml, wave, wave, 0, lane, 2 * wave + 1);
}

}  // namespace xllm_hip
