// Paged-attention decode for gfx950 (MI355X): split-KV ("flash decoding") over
// block_tables / seq_lens with GQA, bf16 / fp8-e4m3 / int8 KV caches.
//
// Three launches per call, none of which reads anything back to the host:
//   decode_plan_kernel   kv lengths -> chunk size, chunk table (once per step)
//   decode_*_kernel      one wave per (sequence chunk, kv head, row group): streams the
//                        chunk's K and V once and writes a normalised partial + log2-sum-exp
//   decode_merge_kernel  combines a sequence's partials into the output rows
//
// Semantics follow the reference's decode operators: head map kv = h / (Hq/Hkv)
// and fp32 softmax as in xllm/core/layers/cuda/flashinfer_attention.cpp:61-88, the
// block_table / seq_lens contract of xllm/core/kernels/mlu/mlu_ops_api.h:126-145,
// the CSR contract of xllm/core/kernels/cuda/cuda_ops_api.h:120-136, and the
// base-2 partial merge of xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73.
#include "decode_plan.h"
#include "device_utils.h"
#include "host_utils.h"

#include <math.h>
#include <stdlib.h>

#include <type_traits>

namespace xllm_hip {

struct DecodeParams {
  const void* q;
  void* out;
  float* lse;
  const uint8_t* k_cache;
  const uint8_t* v_cache;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_ids;  // block_table, or kv_indices in CSR form
  const int32_t* kv_indptr;  // non-NULL selects the CSR form
  const int32_t* seq_lens;
  const int32_t* kv_last_page_len;
  PlanHeader* hdr;
  int32_t* kv_len;
  int32_t* full_prefix;
  int32_t* tail_prefix;
  SeqChunk* seq_chunks;
  float* partial_lse;
  float* partial_out;
  int64_t q_token_stride;
  int64_t out_token_stride;
  int64_t stride_block;
  int64_t stride_head;
  int64_t stride_slot;
  int64_t sc_stride_block;
  int64_t sc_stride_head;
  int64_t sc_stride_slot;
  int64_t bt_stride;
  int32_t batch;
  int32_t n;  // query tokens per sequence
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t group;  // q heads per kv head
  int32_t rows;   // group * n
  int32_t row_groups;
  int32_t head_dim;
  int32_t block_size;
  int32_t log2_bs;
  int32_t max_blocks_per_seq;
  int32_t window_left;
  int32_t target_items;
  int32_t q_dtype;
  float scale_log2;  // sm_scale * log2(e)
};

// ---------------------------------------------------------------------------------
// Plan: one workgroup.  kv lengths -> total -> chunk size -> prefix sums -> chunk table.
// ---------------------------------------------------------------------------------

constexpr int kPlanThreads = 1024;

// Inclusive scan of (a, b) pairs over the workgroup; every thread gets its prefix and the totals.
__device__ inline void block_scan2(int a, int b, int* s_a, int* s_b, int& incl_a, int& incl_b, int& tot_a,
                                   int& tot_b) {
  const int tid = threadIdx.x;
  s_a[tid] = a;
  s_b[tid] = b;
  __syncthreads();
  for (int off = 1; off < kPlanThreads; off <<= 1) {
    int va = 0, vb = 0;
    if (tid >= off) {
      va = s_a[tid - off];
      vb = s_b[tid - off];
    }
    __syncthreads();
    s_a[tid] += va;
    s_b[tid] += vb;
    __syncthreads();
  }
  incl_a = s_a[tid];
  incl_b = s_b[tid];
  tot_a = s_a[kPlanThreads - 1];
  tot_b = s_b[kPlanThreads - 1];
  __syncthreads();
}

__global__ void __launch_bounds__(kPlanThreads) decode_plan_kernel(DecodeParams p) {
  __shared__ int s_a[kPlanThreads];
  __shared__ int s_b[kPlanThreads];
  __shared__ long long s_total[kPlanThreads / 64];
  __shared__ int s_chunk;
  const int tid = threadIdx.x;

  // 1. kv lengths and their sum.
  long long local = 0;
  for (int b = tid; b < p.batch; b += kPlanThreads) {
    int len;
    if (p.kv_indptr != nullptr) {
      const int nb = p.kv_indptr[b + 1] - p.kv_indptr[b];
      len = nb > 0 ? (nb - 1) * p.block_size + p.kv_last_page_len[b] : 0;
    } else {
      len = p.seq_lens[b];
    }
    len = len > 0 ? len : 0;
    p.kv_len[b] = len;
    local += len;
  }
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) local += __shfl_xor(local, o);
  if ((tid & 63) == 0) s_total[tid >> 6] = local;
  __syncthreads();
  if (tid == 0) {
    long long total = 0;
    for (int i = 0; i < kPlanThreads / 64; ++i) total += s_total[i];
    // 2. Chunk size: split so that about target_items work items exist.
    const long long work = total * p.num_kv_heads * p.row_groups;
    long long c = (work + p.target_items - 1) / p.target_items;
    c = (c + kTileTokens - 1) / kTileTokens * kTileTokens;
    if (c < kMinChunkTokens) c = kMinChunkTokens;
    if (c > (1 << 30)) c = 1 << 30;
    s_chunk = (int)c;
  }
  __syncthreads();
  const int chunk = s_chunk;

  // 3. Prefix sums of the full-chunk and tail-chunk counts.
  int run_full = 0, run_tail = 0;
  for (int base = 0; base < p.batch; base += kPlanThreads) {
    const int b = base + tid;
    int nf = 0, nt = 0;
    if (b < p.batch) {
      const int len = p.kv_len[b];
      nf = len / chunk;
      nt = (len - nf * chunk) > 0 ? 1 : 0;
    }
    int incl_f, incl_t, tot_f, tot_t;
    block_scan2(nf, nt, s_a, s_b, incl_f, incl_t, tot_f, tot_t);
    if (b < p.batch) {
      p.full_prefix[b] = run_full + incl_f - nf;
      p.tail_prefix[b] = run_tail + incl_t - nt;
    }
    run_full += tot_f;
    run_tail += tot_t;
  }
  if (tid == 0) {
    p.full_prefix[p.batch] = run_full;
    p.tail_prefix[p.batch] = run_tail;
    PlanHeader h{};
    h.total_full = run_full;
    h.total_tail = run_tail;
    h.chunk_tokens = chunk;
    h.total_items = (run_full + run_tail) * p.num_kv_heads * p.row_groups;
    *p.hdr = h;
  }
  __syncthreads();  // prefix arrays written by this workgroup are visible to it below

  // 4. Chunk table: full chunks first, then the tails.
  for (int b = tid; b < p.batch; b += kPlanThreads) {
    const int len = p.kv_len[b];
    const int nf = len / chunk;
    const int f0 = p.full_prefix[b];
    for (int c = 0; c < nf; ++c) p.seq_chunks[f0 + c] = SeqChunk{b, c};
    if (len - nf * chunk > 0) p.seq_chunks[run_full + p.tail_prefix[b]] = SeqChunk{b, nf};
  }
}

// ---------------------------------------------------------------------------------
// Work-item decoding shared by the attention kernels.
// ---------------------------------------------------------------------------------

struct Item {
  int sc;       // sequence-chunk slot (indexes the partial arrays)
  int b;        // sequence
  int hk;       // kv head
  int rg;       // row group
  int len;      // kv length of the sequence
  int t_begin;  // first token of the chunk (multiple of kTileTokens)
  int t_end;    // one past the last token of the chunk (<= len)
  const int32_t* ids;  // block list of the sequence
  int nblk;     // valid entries in ids (>= 1)
};

__device__ inline bool decode_item(const DecodeParams& p, int item_id, Item& it) {
  const PlanHeader hdr = *p.hdr;
  if (item_id >= hdr.total_items) return false;
  it.rg = item_id % p.row_groups;
  const int rest = item_id / p.row_groups;
  it.hk = rest % p.num_kv_heads;
  it.sc = rest / p.num_kv_heads;
  const SeqChunk s = p.seq_chunks[it.sc];
  it.b = s.seq;
  it.len = p.kv_len[it.b];
  it.t_begin = s.chunk * hdr.chunk_tokens;
  const long long end = (long long)it.t_begin + hdr.chunk_tokens;
  it.t_end = end < it.len ? (int)end : it.len;
  if (p.kv_indptr != nullptr) {
    it.ids = p.block_ids + p.kv_indptr[it.b];
  } else {
    it.ids = p.block_ids + (int64_t)it.b * p.bt_stride;
  }
  it.nblk = (it.len + p.block_size - 1) >> p.log2_bs;
  if (it.nblk < 1) it.nblk = 1;
  return true;
}

// ---------------------------------------------------------------------------------
// MFMA kernel, head_dim 128, bf16 queries.  One wave per work item.
//
// Per 32-token tile the wave loads K and V rows with fully coalesced 16-byte
// loads, parks them in its private 16 KiB of LDS (row-major, 16-byte pieces
// XOR-swizzled by row so that the fragment reads below are bank-conflict free),
// and reads them back in MFMA operand order:
//   S^T[t][r]  = sum_d K[t][d] Q[r][d]      A = K tile (ds_read_b128), B = Q^T (registers)
//   O^T[d][r] += sum_t V[t][d] P[r][t]      A = V^T tile (ds_read_b64_tr_b16), B = P^T (registers)
// Computing the transposed products keeps a query row in one lane column for
// both MFMAs, so the probabilities leave the first MFMA already laid out as the
// second one's B operand and the softmax statistics are per-lane scalars.
// Query rows r = j*g + gq (draft token j, head gq of the group) fill the 16
// columns of an MFMA tile; NT tiles cover up to 16*NT rows.
// ---------------------------------------------------------------------------------

constexpr int kLdsK = 0;
constexpr int kLdsV = 8192;
constexpr int kLdsWave = 16384;

template <int KV_DT>
struct KvStage;  // registers holding one tile in flight + how to park it in LDS

__device__ inline u32x4 ldg_stream(const void* p) {
  return __builtin_nontemporal_load((const u32x4*)p);
}

__device__ inline uint32_t swz(int row, int piece) { return (uint32_t)(row * 256 + ((piece ^ (row & 15)) << 4)); }

// bf16 cache: 16 loads of 16 bytes per lane and tile (8 K + 8 V); lane = (row-in-load, piece).
template <>
struct KvStage<XLLM_HIP_BF16> {
  u32x4 k[8];
  u32x4 v[8];

  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int lane) {
    const int lrow = lane >> 4, piece = lane & 15;
    const int bs_mask = p.block_size - 1;
    int bi0 = tb >> p.log2_bs, bi1 = (tb + 16) >> p.log2_bs;
    bi0 = bi0 < it.nblk ? bi0 : it.nblk - 1;
    bi1 = bi1 < it.nblk ? bi1 : it.nblk - 1;
    const int64_t blk0 = it.ids[bi0], blk1 = it.ids[bi1];
    const int64_t head_off = (int64_t)it.hk * p.stride_head + piece * 8;
    const int64_t base0 = blk0 * p.stride_block + head_off + (int64_t)((tb & bs_mask) + lrow) * p.stride_slot;
    const int64_t base1 = blk1 * p.stride_block + head_off + (int64_t)(((tb + 16) & bs_mask) + lrow) * p.stride_slot;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t o0 = (base0 + (int64_t)(4 * j) * p.stride_slot) * 2;
      const int64_t o1 = (base1 + (int64_t)(4 * j) * p.stride_slot) * 2;
      k[j] = ldg_stream(p.k_cache + o0);
      k[j + 4] = ldg_stream(p.k_cache + o1);
      v[j] = ldg_stream(p.v_cache + o0);
      v[j + 4] = ldg_stream(p.v_cache + o1);
    }
  }

  // Rows at or beyond `len` may hold anything (unwritten slots); zero them so that 0 * x stays 0.
  template <bool MASKED>
  __device__ inline void park(uint8_t* lds, int tb, int len, int lane) {
    const int lrow = lane >> 4, piece = lane & 15;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = 4 * j + lrow;
      u32x4 kk = k[j], vv = v[j];
      if (MASKED && tb + row >= len) {
        kk = u32x4{0, 0, 0, 0};
        vv = u32x4{0, 0, 0, 0};
      }
      const uint32_t off = swz(row, piece);
      *(u32x4*)(lds + kLdsK + off) = kk;
      *(u32x4*)(lds + kLdsV + off) = vv;
    }
  }

  __device__ inline void take_scales(f32x4 (&)[2], f32x4 (&)[2]) const {}
};

// Convert 16 quantised bytes to 16 bf16 (exact for both e4m3 and int8).
template <int KV_DT>
__device__ inline void dequant16(const u32x4 raw, bf16x8& lo, bf16x8& hi) {
  union {
    bf16x2 h[8];
    bf16x8 v[2];
  } u;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (KV_DT == XLLM_HIP_FP8_E4M3) {
      u.h[2 * w] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)raw[w], 1.0f, false);
      u.h[2 * w + 1] = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8((int)raw[w], 1.0f, true);
    } else {
      const uint32_t t = raw[w] ^ 0x80808080u;  // int8 + 128 as unsigned bytes
      const float f0 = (float)(t & 0xffu) - 128.0f;
      const float f1 = (float)((t >> 8) & 0xffu) - 128.0f;
      const float f2 = (float)((t >> 16) & 0xffu) - 128.0f;
      const float f3 = (float)(t >> 24) - 128.0f;
      u.h[2 * w] = bf16x2{(__bf16)f0, (__bf16)f1};
      u.h[2 * w + 1] = bf16x2{(__bf16)f2, (__bf16)f3};
    }
  }
  lo = u.v[0];
  hi = u.v[1];
}

// 1-byte caches: 8 loads of 16 bytes per lane and tile (4 K + 4 V); lane = (row-in-load, 16-element piece),
// plus the fp32 scales of the tile's tokens in the layout of the score registers.
template <int KV_DT>
struct KvStageQuant {
  u32x4 k[4];
  u32x4 v[4];
  f32x4 ks[2];
  f32x4 vs[2];

  __device__ inline void issue(const DecodeParams& p, const Item& it, int tb, int lane) {
    const int lrow = lane >> 3, piece = lane & 7;
    const int kg = lane >> 4;
    const int bs_mask = p.block_size - 1;
    int bi0 = tb >> p.log2_bs, bi1 = (tb + 16) >> p.log2_bs;
    bi0 = bi0 < it.nblk ? bi0 : it.nblk - 1;
    bi1 = bi1 < it.nblk ? bi1 : it.nblk - 1;
    const int64_t blk0 = it.ids[bi0], blk1 = it.ids[bi1];
    const int slot0 = tb & bs_mask, slot1 = (tb + 16) & bs_mask;
    const int64_t head_off = (int64_t)it.hk * p.stride_head + piece * 16;
    const int64_t base0 = blk0 * p.stride_block + head_off + (int64_t)(slot0 + lrow) * p.stride_slot;
    const int64_t base1 = blk1 * p.stride_block + head_off + (int64_t)(slot1 + lrow) * p.stride_slot;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t o0 = base0 + (int64_t)(8 * j) * p.stride_slot;
      const int64_t o1 = base1 + (int64_t)(8 * j) * p.stride_slot;
      k[j] = ldg_stream(p.k_cache + o0);
      k[j + 2] = ldg_stream(p.k_cache + o1);
      v[j] = ldg_stream(p.v_cache + o0);
      v[j + 2] = ldg_stream(p.v_cache + o1);
    }
    // Scales of tokens tb + 16*s + 4*kg + rr, the tokens of this lane's score registers.
    const int64_t s0 = blk0 * p.sc_stride_block + (int64_t)it.hk * p.sc_stride_head +
                       (int64_t)(slot0 + 4 * kg) * p.sc_stride_slot;
    const int64_t s1 = blk1 * p.sc_stride_block + (int64_t)it.hk * p.sc_stride_head +
                       (int64_t)(slot1 + 4 * kg) * p.sc_stride_slot;
    if (p.sc_stride_slot == 1) {
      ks[0] = *(const f32x4*)(p.k_scale + s0);
      ks[1] = *(const f32x4*)(p.k_scale + s1);
      vs[0] = *(const f32x4*)(p.v_scale + s0);
      vs[1] = *(const f32x4*)(p.v_scale + s1);
    } else {
#pragma unroll
      for (int rr = 0; rr < 4; ++rr) {
        ks[0][rr] = p.k_scale[s0 + rr * p.sc_stride_slot];
        ks[1][rr] = p.k_scale[s1 + rr * p.sc_stride_slot];
        vs[0][rr] = p.v_scale[s0 + rr * p.sc_stride_slot];
        vs[1][rr] = p.v_scale[s1 + rr * p.sc_stride_slot];
      }
    }
  }

  template <bool MASKED>
  __device__ inline void park(uint8_t* lds, int tb, int len, int lane) {
    const int lrow = lane >> 3, piece = lane & 7;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = 8 * j + lrow;
      bf16x8 klo, khi, vlo, vhi;
      dequant16<KV_DT>(k[j], klo, khi);
      dequant16<KV_DT>(v[j], vlo, vhi);
      if (MASKED && tb + row >= len) {
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        klo = khi = vlo = vhi = z;
      }
      const uint32_t o_lo = swz(row, 2 * piece), o_hi = swz(row, 2 * piece + 1);
      *(bf16x8*)(lds + kLdsK + o_lo) = klo;
      *(bf16x8*)(lds + kLdsK + o_hi) = khi;
      *(bf16x8*)(lds + kLdsV + o_lo) = vlo;
      *(bf16x8*)(lds + kLdsV + o_hi) = vhi;
    }
  }

  __device__ inline void take_scales(f32x4 (&kss)[2], f32x4 (&vss)[2]) const {
    kss[0] = ks[0];
    kss[1] = ks[1];
    vss[0] = vs[0];
    vss[1] = vs[1];
  }
};
template <>
struct KvStage<XLLM_HIP_FP8_E4M3> : KvStageQuant<XLLM_HIP_FP8_E4M3> {};
template <>
struct KvStage<XLLM_HIP_INT8> : KvStageQuant<XLLM_HIP_INT8> {};

template <int KV_DT, int NT>
__global__ void __launch_bounds__(64) decode_mfma_d128_kernel(DecodeParams p) {
  constexpr bool kQuant = KV_DT != XLLM_HIP_BF16;
  __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsWave];

  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;

  const int lane = threadIdx.x;
  const int mi = lane & 15;  // MFMA row of A / column of B and D
  const int kg = lane >> 4;  // k-group of the operands; row block of D
  const float neg_inf = -INFINITY;

  // Query rows of this lane's column, one per N tile.
  int lim[NT];  // tokens >= lim are invisible to the row (causal among draft tokens)
  int lo[NT];   // tokens < lo are outside the sliding window
  bool valid[NT];
  bf16x8 qf[NT][4];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int r = it.rg * kMaxRowsPerItem + nt * 16 + mi;
    valid[nt] = r < p.rows;
    const int j = valid[nt] ? r / p.group : 0;
    const int gq = valid[nt] ? r - j * p.group : 0;
    lim[nt] = it.len - (p.n - 1 - j);
    lo[nt] = p.window_left >= 0 ? lim[nt] - 1 - p.window_left : 0;
    const uint16_t* qrow = (const uint16_t*)p.q + (int64_t)(it.b * p.n + j) * p.q_token_stride +
                           (int64_t)(it.hk * p.group + gq) * 128;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      u32x4 raw = {0, 0, 0, 0};
      if (valid[nt]) raw = *(const u32x4*)(qrow + c * 32 + kg * 8);
      qf[nt][c] = __builtin_bit_cast(bf16x8, raw);
    }
  }

  // Tile range.  With a sliding window, tiles wholly below every row's window are skipped.
  int t0 = it.t_begin;
  if (p.window_left >= 0) {
    int first = it.len - p.n - p.window_left;  // window start of the earliest query row
    first = first > 0 ? first : 0;
    first &= ~(kTileTokens - 1);
    t0 = t0 > first ? t0 : first;
  }
  const int mask_hi_from = it.len - (p.n - 1);                                // tiles reaching past this need masks
  const int mask_lo_until = p.window_left >= 0 ? it.len - 1 - p.window_left : 0;  // tiles starting below this too

  f32x4 acc[NT][8];
  float m_run[NT], l_run[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    m_run[nt] = neg_inf;
    l_run[nt] = 0.0f;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) acc[nt][dt] = f32x4{0, 0, 0, 0};
  }

  // Per-lane LDS read offsets.
  uint32_t k_off[4];
#pragma unroll
  for (int c = 0; c < 4; ++c) k_off[c] = kLdsK + swz(mi, c * 4 + kg);
  const int tau = 4 * kg + (mi >> 2);  // token row (within a 16-token half) this lane points the transpose read at
  uint32_t v_off[8];
#pragma unroll
  for (int dt = 0; dt < 8; ++dt) v_off[dt] = kLdsV + swz(tau, dt * 2 + ((mi & 3) >> 1)) + (mi & 1) * 8;

  KvStage<KV_DT> stage;

  auto tile = [&](int tb, const f32x4 (&ksc)[2], const f32x4 (&vsc)[2], auto masked_tag) {
    constexpr bool MASKED = decltype(masked_tag)::value;
    // ---- S^T = K Q^T ----
    f32x4 s[2][NT];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) s[h][nt] = f32x4{0, 0, 0, 0};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const bf16x8 kf = *(const bf16x8*)(lds + k_off[c] + h * 4096);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          s[h][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[nt][c], s[h][nt], 0, 0, 0);
        }
      }
    }
    // ---- online softmax, per query row (lane column) ----
    bf16x8 pf[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      float x[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
          float v = s[h][nt][rr] * p.scale_log2;
          if (kQuant) v *= ksc[h][rr];
          if (MASKED) {
            const int tok = tb + 16 * h + 4 * kg + rr;
            v = (tok < lim[nt] && tok >= lo[nt]) ? v : neg_inf;
          }
          x[4 * h + rr] = v;
        }
      }
      float mt = fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(x[4], x[5]), fmaxf(x[6], x[7])));
      mt = fmaxf(mt, __shfl_xor(mt, 16));
      mt = fmaxf(mt, __shfl_xor(mt, 32));
      const float m_new = fmaxf(m_run[nt], mt);
      const float m_safe = m_new == neg_inf ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run[nt] - m_safe);
      float psum = 0.0f;
      float pv[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float e = __builtin_amdgcn_exp2f(x[i] - m_safe);
        psum += e;
        pv[i] = e;
      }
      if (kQuant) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) {
            float w = vsc[h][rr];
            if (MASKED) {
              const int tok = tb + 16 * h + 4 * kg + rr;
              w = tok < it.len ? w : 0.0f;
            }
            pv[4 * h + rr] *= w;
          }
        }
      }
      l_run[nt] = l_run[nt] * alpha + psum;
      m_run[nt] = m_new;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) acc[nt][dt] *= alpha;
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) pf[nt][i] = (__bf16)pv[i];
    }
    // ---- O^T += V^T P^T ----
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      const s16x4 a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)(lds + v_off[dt]));
      const s16x4 a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) s16x4*)(lds + v_off[dt] + 4096));
      const bf16x8 vf = __builtin_bit_cast(bf16x8, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc[nt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[nt], acc[nt][dt], 0, 0, 0);
      }
    }
  };

  if (t0 < it.t_end) {
    stage.issue(p, it, t0, lane);
    for (int tb = t0; tb < it.t_end; tb += kTileTokens) {
      const bool masked = (tb + kTileTokens > mask_hi_from) || (tb < mask_lo_until);
      if (masked) {
        stage.template park<true>(lds, tb, it.len, lane);
      } else {
        stage.template park<false>(lds, tb, it.len, lane);
      }
      // The scales of the tile being consumed must outlive the next issue.
      f32x4 ksc[2] = {}, vsc[2] = {};
      stage.take_scales(ksc, vsc);
      if (tb + kTileTokens < it.t_end) stage.issue(p, it, tb + kTileTokens, lane);
      if (masked) {
        tile(tb, ksc, vsc, std::true_type{});
      } else {
        tile(tb, ksc, vsc, std::false_type{});
      }
    }
  }

  // ---- normalised partial + base-2 log-sum-exp ----
  const int nhq = p.n * p.num_q_heads;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float l = l_run[nt];
    l += __shfl_xor(l, 16);
    l += __shfl_xor(l, 32);
    if (!valid[nt]) continue;
    const int r = it.rg * kMaxRowsPerItem + nt * 16 + mi;
    const int j = r / p.group;
    const int gq = r - j * p.group;
    const int64_t prow = (int64_t)it.sc * nhq + (int64_t)j * p.num_q_heads + it.hk * p.group + gq;
    const float inv = l > 0.0f ? 1.0f / l : 0.0f;
    if (kg == 0) p.partial_lse[prow] = l > 0.0f ? m_run[nt] + __builtin_amdgcn_logf(l) : neg_inf;
    float* po = p.partial_out + prow * 128 + 4 * kg;
#pragma unroll
    for (int dt = 0; dt < 8; ++dt) {
      *(f32x4*)(po + dt * 16) = acc[nt][dt] * inv;
    }
  }
}

// ---------------------------------------------------------------------------------
// Generic kernel: any head_dim <= 256, any supported dtype.  One wave per work item, one query
// row at a time; lanes are tokens for q.k and head-dim columns for p.v.  Not tuned: it exists
// so that every shape the operators accept is served and as an independent device-side check.
// ---------------------------------------------------------------------------------

template <int Q_DT, int KV_DT>
__global__ void __launch_bounds__(64) decode_generic_kernel(DecodeParams p) {
  __shared__ float qs[256];
  Item it;
  if (!decode_item(p, blockIdx.x, it)) return;
  const int lane = threadIdx.x;
  const int D = p.head_dim;
  const float neg_inf = -INFINITY;
  const bool quant = KV_DT == XLLM_HIP_FP8_E4M3 || KV_DT == XLLM_HIP_INT8;
  const int nhq = p.n * p.num_q_heads;
  const int row_end = min(p.rows, (it.rg + 1) * kMaxRowsPerItem);

  for (int r = it.rg * kMaxRowsPerItem; r < row_end; ++r) {
    const int j = r / p.group;
    const int gq = r - j * p.group;
    const int head = it.hk * p.group + gq;
    const int64_t qbase = (int64_t)(it.b * p.n + j) * p.q_token_stride + (int64_t)head * D;
    __syncthreads();
    for (int d = lane; d < D; d += 64) qs[d] = Elem<Q_DT>::load(p.q, qbase + d) * p.scale_log2;
    __syncthreads();
    const int lim = it.len - (p.n - 1 - j);
    const int lo = p.window_left >= 0 ? lim - 1 - p.window_left : 0;

    float m_run = neg_inf, l_run = 0.0f;
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int tb = it.t_begin; tb < it.t_end; tb += 64) {
      const int tok = tb + lane;
      const bool vis = tok < it.t_end && tok < lim && tok >= lo;
      float x = neg_inf;
      float vscale = 0.0f;
      int64_t vrow = 0;
      if (vis) {
        int bi = tok >> p.log2_bs;
        const int64_t blk = it.ids[bi];
        const int slot = tok & (p.block_size - 1);
        const int64_t row = blk * p.stride_block + (int64_t)it.hk * p.stride_head + (int64_t)slot * p.stride_slot;
        float dot = 0.0f;
        for (int d = 0; d < D; ++d) dot += qs[d] * Elem<KV_DT>::load(p.k_cache, row + d);
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
      const int cnt = min(64, it.t_end - tb);
      for (int tt = 0; tt < cnt; ++tt) {
        const float pt = __shfl(pw, tt);
        const int64_t row = __shfl(vrow, tt);
        if (pt != 0.0f) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int d = lane + 64 * i;
            if (d < D) o[i] += pt * Elem<KV_DT>::load(p.v_cache, row + d);
          }
        }
      }
    }
    const int64_t prow = (int64_t)it.sc * nhq + (int64_t)j * p.num_q_heads + head;
    const float inv = l_run > 0.0f ? 1.0f / l_run : 0.0f;
    if (lane == 0) p.partial_lse[prow] = l_run > 0.0f ? m_run + __builtin_amdgcn_logf(l_run) : neg_inf;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < D) p.partial_out[prow * D + d] = o[i] * inv;
    }
  }
}

// ---------------------------------------------------------------------------------
// Merge: out = sum_i 2^(lse_i - lse) * partial_i,  lse = log2 sum_i 2^lse_i.
// 32 threads per output row, 8 rows per workgroup.
// ---------------------------------------------------------------------------------

template <int Q_DT>
__global__ void __launch_bounds__(256) decode_merge_kernel(DecodeParams p) {
  const int nhq = p.n * p.num_q_heads;
  const int64_t row = (int64_t)blockIdx.x * 8 + (threadIdx.x >> 5);
  const int sub = threadIdx.x & 31;
  if (row >= (int64_t)p.batch * nhq) return;
  const int b = (int)(row / nhq);
  const int rem = (int)(row - (int64_t)b * nhq);  // j * Hq + head
  const int j = rem / p.num_q_heads;
  const int head = rem - j * p.num_q_heads;
  const int D = p.head_dim;
  const float neg_inf = -INFINITY;

  const int f0 = p.full_prefix[b];
  const int nf = p.full_prefix[b + 1] - f0;
  const int has_tail = p.tail_prefix[b + 1] - p.tail_prefix[b];
  const int tail_slot = p.hdr->total_full + p.tail_prefix[b];
  const int cnt = nf + has_tail;

  float mx = neg_inf;
  for (int i = 0; i < cnt; ++i) {
    const int sc = i < nf ? f0 + i : tail_slot;
    mx = fmaxf(mx, p.partial_lse[(int64_t)sc * nhq + rem]);
  }
  float denom = 0.0f;
  if (mx != neg_inf) {
    for (int i = 0; i < cnt; ++i) {
      const int sc = i < nf ? f0 + i : tail_slot;
      denom += __builtin_amdgcn_exp2f(p.partial_lse[(int64_t)sc * nhq + rem] - mx);
    }
  }
  const float lse = mx != neg_inf ? mx + __builtin_amdgcn_logf(denom) : neg_inf;
  if (p.lse != nullptr && sub == 0) p.lse[(int64_t)(b * p.n + j) * p.num_q_heads + head] = lse;

  const int64_t obase = (int64_t)(b * p.n + j) * p.out_token_stride + (int64_t)head * D;
  for (int d4 = sub * 4; d4 < D; d4 += 128) {
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (mx != neg_inf) {
      for (int i = 0; i < cnt; ++i) {
        const int sc = i < nf ? f0 + i : tail_slot;
        const int64_t prow = (int64_t)sc * nhq + rem;
        const float w = __builtin_amdgcn_exp2f(p.partial_lse[prow] - lse);
        const float* po = p.partial_out + prow * D + d4;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if (d4 + e < D) o[e] += w * po[e];
        }
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (d4 + e < D) Elem<Q_DT>::store(p.out, obase + d4 + e, o[e]);
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

// ---------------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------------

enum Variant { kNone = 0, kMfmaD128 = 1, kGeneric = 2 };

// Split target: about this many work items per launch.  One wave of the attention kernel occupies
// one SIMD, and the chip has 256 CUs x 4 SIMDs.
static int target_items() {
  int v = 1024;
  if (const char* e = getenv("XLLM_HIP_DECODE_TARGET_ITEMS")) {
    const int t = atoi(e);
    if (t > 0) v = t;
  }
  return v > kMaxTargetItems ? kMaxTargetItems : v;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static Variant pick_variant(const xllm_hip_kv_cache* c, const xllm_hip_decode_args* a) {
  const int eb = elem_bytes(c->dtype);
  const bool kv_ok = c->dtype == XLLM_HIP_BF16 || c->dtype == XLLM_HIP_FP8_E4M3 || c->dtype == XLLM_HIP_INT8;
  const bool force_generic = getenv("XLLM_HIP_DECODE_FORCE_GENERIC") != nullptr;
  if (!force_generic && c->head_dim == 128 && a->q_dtype == XLLM_HIP_BF16 && kv_ok && c->block_size >= 16 &&
      is_pow2(c->block_size)) {
    const int vec = 16 / eb;  // elements per 16-byte load
    const bool strides_ok = c->stride_block % vec == 0 && c->stride_head % vec == 0 && c->stride_slot % vec == 0 &&
                            a->q_token_stride % 8 == 0;
    const bool ptrs_ok = aligned16(c->k_cache) && aligned16(c->v_cache) && aligned16(a->q);
    bool scales_ok = true;
    if (eb == 1) {
      scales_ok = c->k_scale != nullptr && c->v_scale != nullptr &&
                  (c->scale_stride_slot != 1 ||
                   (c->scale_stride_block % 4 == 0 && c->scale_stride_head % 4 == 0 && aligned16(c->k_scale) &&
                    aligned16(c->v_scale)));
    }
    if (strides_ok && ptrs_ok && scales_ok) return kMfmaD128;
  }
  if (c->head_dim <= 256 && is_pow2(c->block_size)) return kGeneric;
  return kNone;
}

static int fill_params(const xllm_hip_kv_cache* c,
                       const xllm_hip_decode_args* a,
                       void* workspace,
                       size_t workspace_bytes,
                       DecodeParams& p) {
  XLLM_HIP_REQUIRE(c != nullptr && a != nullptr, "cache or args is NULL");
  XLLM_HIP_REQUIRE(c->k_cache != nullptr && c->v_cache != nullptr, "k_cache or v_cache is NULL");
  XLLM_HIP_REQUIRE(c->num_blocks > 0 && c->block_size > 0 && c->num_kv_heads > 0 && c->head_dim > 0,
                   "cache sizes must be positive");
  XLLM_HIP_REQUIRE(elem_bytes(c->dtype) > 0, "unknown cache dtype %d", c->dtype);
  XLLM_HIP_REQUIRE(a->batch >= 0 && a->q_per_seq >= 1 && a->num_q_heads >= 1, "bad batch/q_per_seq/num_q_heads");
  XLLM_HIP_REQUIRE(a->num_q_heads % c->num_kv_heads == 0, "num_q_heads %d is not a multiple of num_kv_heads %d",
                   a->num_q_heads, c->num_kv_heads);
  XLLM_HIP_REQUIRE(a->q_dtype == XLLM_HIP_BF16 || a->q_dtype == XLLM_HIP_FP16 || a->q_dtype == XLLM_HIP_FP32,
                   "query dtype must be BF16/FP16/FP32, got %d", a->q_dtype);
  const bool quant = c->dtype == XLLM_HIP_FP8_E4M3 || c->dtype == XLLM_HIP_INT8;
  XLLM_HIP_REQUIRE(!quant || (c->k_scale != nullptr && c->v_scale != nullptr),
                   "a quantised cache needs k_scale and v_scale");
  if (a->batch > 0) {
    XLLM_HIP_REQUIRE(a->q != nullptr && a->out != nullptr, "q or out is NULL");
    if (a->block_table != nullptr) {
      XLLM_HIP_REQUIRE(a->seq_lens != nullptr, "block_table form needs seq_lens");
      XLLM_HIP_REQUIRE(a->max_blocks_per_seq >= 1 && a->block_table_stride >= a->max_blocks_per_seq,
                       "bad block_table shape");
    } else {
      XLLM_HIP_REQUIRE(a->kv_indptr != nullptr && a->kv_indices != nullptr && a->kv_last_page_len != nullptr,
                       "neither block_table nor the CSR arrays were given");
    }
    const int64_t rowlen = (int64_t)a->num_q_heads * c->head_dim;
    XLLM_HIP_REQUIRE(a->q_token_stride >= rowlen && a->out_token_stride >= rowlen,
                     "q/out token stride smaller than num_q_heads*head_dim");
  }
  const WorkspaceLayout w =
      workspace_layout(a->batch, a->q_per_seq, a->num_q_heads, c->num_kv_heads, c->head_dim);
  if (workspace == nullptr || workspace_bytes < w.total_bytes) {
    return fail(XLLM_HIP_WORKSPACE_TOO_SMALL, "workspace has %zu bytes, need %zu", workspace_bytes, w.total_bytes);
  }
  XLLM_HIP_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");

  uint8_t* ws = (uint8_t*)workspace;
  p = DecodeParams{};
  p.q = a->q;
  p.out = a->out;
  p.lse = a->lse;
  p.k_cache = (const uint8_t*)c->k_cache;
  p.v_cache = (const uint8_t*)c->v_cache;
  p.k_scale = c->k_scale;
  p.v_scale = c->v_scale;
  if (a->block_table != nullptr) {
    p.block_ids = a->block_table;
    p.kv_indptr = nullptr;
    p.seq_lens = a->seq_lens;
  } else {
    p.block_ids = a->kv_indices;
    p.kv_indptr = a->kv_indptr;
    p.kv_last_page_len = a->kv_last_page_len;
  }
  p.hdr = (PlanHeader*)(ws + w.header);
  p.kv_len = (int32_t*)(ws + w.kv_len);
  p.full_prefix = (int32_t*)(ws + w.full_prefix);
  p.tail_prefix = (int32_t*)(ws + w.tail_prefix);
  p.seq_chunks = (SeqChunk*)(ws + w.seq_chunks);
  p.partial_lse = (float*)(ws + w.partial_lse);
  p.partial_out = (float*)(ws + w.partial_out);
  p.q_token_stride = a->q_token_stride;
  p.out_token_stride = a->out_token_stride;
  p.stride_block = c->stride_block;
  p.stride_head = c->stride_head;
  p.stride_slot = c->stride_slot;
  p.sc_stride_block = c->scale_stride_block;
  p.sc_stride_head = c->scale_stride_head;
  p.sc_stride_slot = c->scale_stride_slot;
  p.bt_stride = a->block_table_stride;
  p.batch = a->batch;
  p.n = a->q_per_seq;
  p.num_q_heads = a->num_q_heads;
  p.num_kv_heads = c->num_kv_heads;
  p.group = a->num_q_heads / c->num_kv_heads;
  p.rows = p.group * p.n;
  p.row_groups = row_groups(a->q_per_seq, a->num_q_heads, c->num_kv_heads);
  p.head_dim = c->head_dim;
  p.block_size = c->block_size;
  p.log2_bs = is_pow2(c->block_size) ? ilog2(c->block_size) : 0;
  p.max_blocks_per_seq = a->max_blocks_per_seq;
  p.window_left = a->window_left;
  p.target_items = target_items();
  p.q_dtype = a->q_dtype;
  p.scale_log2 = a->sm_scale * 1.4426950408889634f;
  return XLLM_HIP_OK;
}

// Upper bound of the work-item count for any lengths (see workspace_layout).
static int64_t max_items(const DecodeParams& p) {
  const int64_t per = (int64_t)p.num_kv_heads * p.row_groups;
  return ((int64_t)p.target_items / per + p.batch + 1) * per;
}

template <int KV_DT>
static void launch_mfma(const DecodeParams& p, unsigned grid, hipStream_t st) {
  const int rows_per_item = p.rows < kMaxRowsPerItem ? p.rows : kMaxRowsPerItem;
  if (rows_per_item <= 16) {
    decode_mfma_d128_kernel<KV_DT, 1><<<grid, 64, 0, st>>>(p);
  } else {
    decode_mfma_d128_kernel<KV_DT, 2><<<grid, 64, 0, st>>>(p);
  }
}

template <int Q_DT>
static int launch_generic(int kv_dtype, const DecodeParams& p, unsigned grid, hipStream_t st) {
  switch (kv_dtype) {
    case XLLM_HIP_BF16:
      decode_generic_kernel<Q_DT, XLLM_HIP_BF16><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP16:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP16><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP32:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP32><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP8_E4M3:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP8_E4M3><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_INT8:
      decode_generic_kernel<Q_DT, XLLM_HIP_INT8><<<grid, 64, 0, st>>>(p);
      break;
    default:
      return fail(XLLM_HIP_UNSUPPORTED, "no decode kernel for cache dtype %d", kv_dtype);
  }
  return XLLM_HIP_OK;
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" size_t xllm_hip_paged_decode_workspace_bytes(int32_t batch,
                                                        int32_t q_per_seq,
                                                        int32_t num_q_heads,
                                                        int32_t num_kv_heads,
                                                        int32_t head_dim) {
  if (batch < 0 || q_per_seq < 1 || num_q_heads < 1 || num_kv_heads < 1 || head_dim < 1) return 0;
  return workspace_layout(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim).total_bytes;
}

extern "C" const char* xllm_hip_paged_decode_variant(const xllm_hip_kv_cache* cache,
                                                     const xllm_hip_decode_args* args) {
  if (cache == nullptr || args == nullptr) return "";
  switch (pick_variant(cache, args)) {
    case kMfmaD128:
      return "mfma_d128";
    case kGeneric:
      return "generic";
    default:
      return "";
  }
}

extern "C" int xllm_hip_paged_decode_plan(const xllm_hip_kv_cache* cache,
                                          const xllm_hip_decode_args* args,
                                          void* workspace,
                                          size_t workspace_bytes,
                                          xllm_hip_stream_t stream) {
  DecodeParams p;
  if (int s = fill_params(cache, args, workspace, workspace_bytes, p)) return s;
  if (p.batch == 0) return XLLM_HIP_OK;
  decode_plan_kernel<<<1, kPlanThreads, 0, (hipStream_t)stream>>>(p);
  return check_launch("decode_plan_kernel");
}

extern "C" int xllm_hip_paged_decode_run(const xllm_hip_kv_cache* cache,
                                         const xllm_hip_decode_args* args,
                                         void* workspace,
                                         size_t workspace_bytes,
                                         xllm_hip_stream_t stream) {
  return xllm_hip_paged_decode_run_timed(cache, args, workspace, workspace_bytes, stream, nullptr, nullptr);
}

extern "C" int xllm_hip_paged_decode_run_timed(const xllm_hip_kv_cache* cache,
                                               const xllm_hip_decode_args* args,
                                               void* workspace,
                                               size_t workspace_bytes,
                                               xllm_hip_stream_t stream,
                                               void* ev_begin,
                                               void* ev_end) {
  DecodeParams p;
  if (int s = fill_params(cache, args, workspace, workspace_bytes, p)) return s;
  if (p.batch == 0) return XLLM_HIP_OK;
  const Variant v = pick_variant(cache, args);
  if (v == kNone) {
    return fail(XLLM_HIP_UNSUPPORTED,
                "no decode kernel for head_dim=%d block_size=%d (head_dim <= 256 and a power-of-two block_size "
                "are required)",
                cache->head_dim, cache->block_size);
  }
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)max_items(p);
  if (ev_begin != nullptr && hipEventRecord((hipEvent_t)ev_begin, st) != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipEventRecord(ev_begin) failed");
  }
  if (v == kMfmaD128) {
    switch (cache->dtype) {
      case XLLM_HIP_BF16:
        launch_mfma<XLLM_HIP_BF16>(p, grid, st);
        break;
      case XLLM_HIP_FP8_E4M3:
        launch_mfma<XLLM_HIP_FP8_E4M3>(p, grid, st);
        break;
      default:
        launch_mfma<XLLM_HIP_INT8>(p, grid, st);
        break;
    }
  } else {
    int s;
    switch (args->q_dtype) {
      case XLLM_HIP_BF16:
        s = launch_generic<XLLM_HIP_BF16>(cache->dtype, p, grid, st);
        break;
      case XLLM_HIP_FP16:
        s = launch_generic<XLLM_HIP_FP16>(cache->dtype, p, grid, st);
        break;
      default:
        s = launch_generic<XLLM_HIP_FP32>(cache->dtype, p, grid, st);
        break;
    }
    if (s) return s;
  }
  if (int s = check_launch("decode attention kernel")) return s;
  if (ev_end != nullptr && hipEventRecord((hipEvent_t)ev_end, st) != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipEventRecord(ev_end) failed");
  }

  const int64_t rows = (int64_t)p.batch * p.n * p.num_q_heads;
  const unsigned mgrid = (unsigned)((rows + 7) / 8);
  switch (args->q_dtype) {
    case XLLM_HIP_BF16:
      decode_merge_kernel<XLLM_HIP_BF16><<<mgrid, 256, 0, st>>>(p);
      break;
    case XLLM_HIP_FP16:
      decode_merge_kernel<XLLM_HIP_FP16><<<mgrid, 256, 0, st>>>(p);
      break;
    default:
      decode_merge_kernel<XLLM_HIP_FP32><<<mgrid, 256, 0, st>>>(p);
      break;
  }
  return check_launch("decode_merge_kernel");
}

extern "C" int xllm_hip_paged_decode(const xllm_hip_kv_cache* cache,
                                     const xllm_hip_decode_args* args,
                                     void* workspace,
                                     size_t workspace_bytes,
                                     xllm_hip_stream_t stream) {
  if (int s = xllm_hip_paged_decode_plan(cache, args, workspace, workspace_bytes, stream)) return s;
  return xllm_hip_paged_decode_run(cache, args, workspace, workspace_bytes, stream);
}

extern "C" int xllm_hip_csr_to_block_table(const int32_t* kv_indptr,
                                           const int32_t* kv_indices,
                                           const int32_t* kv_last_page_len,
                                           int32_t batch,
                                           int32_t block_size,
                                           int32_t* block_table,
                                           int64_t block_table_stride,
                                           int32_t max_blocks_per_seq,
                                           int32_t* seq_lens,
                                           xllm_hip_stream_t stream) {
  XLLM_HIP_REQUIRE(batch >= 0 && block_size > 0 && max_blocks_per_seq >= 1, "bad sizes");
  if (batch == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(kv_indptr && kv_indices && kv_last_page_len && block_table && seq_lens, "NULL argument");
  XLLM_HIP_REQUIRE(block_table_stride >= max_blocks_per_seq, "block_table_stride < max_blocks_per_seq");
  csr_to_block_table_kernel<<<(unsigned)batch, 256, 0, (hipStream_t)stream>>>(
      kv_indptr, kv_indices, kv_last_page_len, batch, block_size, block_table, block_table_stride,
      max_blocks_per_seq, seq_lens);
  return check_launch("csr_to_block_table_kernel");
}
