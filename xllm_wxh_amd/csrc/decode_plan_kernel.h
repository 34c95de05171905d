// Device-side plan of a decode step: kv lengths -> chunk size -> chunk table (see decode_plan.h).
#pragma once

#include "decode_params.h"
#include "device_utils.h"

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Plan: one workgroup.  kv lengths -> total -> chunk size -> prefix sums -> chunk table.
// ---------------------------------------------------------------------------------

// Inclusive scan of (a, b) over the wave, in the data-parallel-primitive form (shifts within rows of 16
// lanes, then the row broadcasts): six dependent register operations per value, where shuffles through
// the LDS crossbar cost the plan's one wave some 700 cycles per 64 sequences.
__device__ inline int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, false);  // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, false);  // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, false);  // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, false);  // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1 and 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2 and 3
  return v;
}
__device__ inline void wave_scan2(int& a, int& b, int lane) {
  (void)lane;
  a = wave_inclusive_scan(a);
  b = wave_inclusive_scan(b);
}

// The finished-chunk counters of the fused merge at the start of a step that stores no schedule.
__global__ void __launch_bounds__(256) decode_zero_counters_kernel(int32_t* counters, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) counters[i] = 0;
}

constexpr int kPlanLens = 8192;  // sequences whose lengths the plan keeps in LDS (32 KiB)

__global__ void __launch_bounds__(64) decode_plan_kernel(DecodeParams p) {
  const int lane = threadIdx.x;
  // tails by size class: how many there are, then how many have been placed
  __shared__ int tail_hist[64];
  __shared__ int tail_fill[64];
  tail_hist[lane] = 0;
  tail_fill[lane] = 0;
  // the finished-chunk counters of the fused merge start every step at zero (the attention kernel
  // leaves them at zero again, so one plan serves every layer of the step)
  if (p.fused_merge) {
    const int ncounters = p.batch * p.num_kv_heads * p.row_groups;
    for (int i = lane; i < ncounters; i += 64) p.counters[i] = 0;
  }

  // 1. kv lengths, their sum and their maximum.  Four loads per lane are in flight at a time, and the
  //    lengths of up to kPlanLens sequences stay in LDS for the two passes below (each pass otherwise waits
  //    for memory once per 64 sequences: 20 us for 1024 sequences, 7 from LDS).
  __shared__ int lens[kPlanLens];
  __shared__ int first_full[kPlanLens];  // first full-chunk slot of a sequence (pass 3 then needs no second scan)
  const bool in_lds = p.batch <= kPlanLens;
  long long total = 0;
  int max_len = 0;
  for (int base = 0; base < p.batch; base += 256) {
    int l[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = base + 64 * u + lane;
      l[u] = b < p.batch ? kv_length(p, b) : 0;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int b = base + 64 * u + lane;
      if (b < p.batch) {
        p.kv_len[b] = l[u];
        if (in_lds) lens[b] = l[u];
        total += l[u];
        max_len = l[u] > max_len ? l[u] : max_len;
      }
    }
  }
  __syncthreads();
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    total += __shfl_xor(total, o);
    const int other = __shfl_xor(max_len, o);
    max_len = other > max_len ? other : max_len;
  }

  // 2. Chunk size.
  const int chunk = p.fixed_chunk > 0
                        ? p.fixed_chunk
                        : choose_chunk(total, max_len, p.batch, p.item_heads, p.row_groups, p.target_items,
                                       p.target_small, p.min_chunk, p.tile_tokens);

  // 3. Prefix sums of the full-chunk and tail-chunk counts (lengths are re-derived rather than
  //    re-read so that no lane depends on another lane's global store).
  auto length_of = [&](int b) { return in_lds ? lens[b] : kv_length(p, b); };
  // The tail chunks differ in size.  They are dispatched after the (equal) full chunks, longest
  // first — in 64 size classes — so that the launch ends with the shortest work items.
  // (in single precision: a 64-bit division costs this one wave a hundred instructions per sequence, and the
  // classes only order the tails; both passes below compute them alike)
  const float classes_per_token = 64.0f / (float)chunk;
  auto tail_class = [&](int tail_len) {  // tail_len < chunk
    const int c = (int)((float)tail_len * classes_per_token);
    return c > 63 ? 63 : c;
  };
  int total_full = 0, total_tail = 0;
  for (int base = 0; base < p.batch; base += 64) {
    const int b = base + lane;
    int nf = 0, nt = 0;
    if (b < p.batch) {
      const int len = length_of(b);
      nf = (int)((unsigned)len / (unsigned)chunk);
      nt = ((len - nf * chunk) > 0 || len == 0) ? 1 : 0;  // an empty sequence keeps one (empty) chunk: it writes zeros
      if (nt) atomicAdd(&tail_hist[tail_class(len - nf * chunk)], 1);
    }
    int sf = nf, st = nt;
    wave_scan2(sf, st, lane);
    if (b < p.batch) {
      p.full_prefix[b] = total_full + sf - nf;
      if (in_lds) first_full[b] = total_full + sf - nf;
      p.num_chunks[b] = nf + nt;
    }
    total_full += __shfl(sf, 63);
    total_tail += __shfl(st, 63);
  }
  // first slot of size class `lane`: the number of tails in larger classes
  int class_start = 0;
  {
    const int mine = tail_hist[lane];
    int incl = mine;  // inclusive scan from the top: lanes 63, 62, ...
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int up = __shfl_down(incl, o);
      if (lane + o < 64) incl += up;
    }
    class_start = incl - mine;
  }
  tail_hist[lane] = class_start;  // reused as the class offsets
  if (lane == 0) {
    p.full_prefix[p.batch] = total_full;
    p.tail_prefix[p.batch] = total_tail;
    PlanHeader h{};
    h.total_full = total_full;
    h.total_tail = total_tail;
    h.chunk_tokens = chunk;
    h.total_items = (total_full + total_tail) * p.item_heads * p.row_groups;
    *p.hdr = h;
  }

  // 4. Chunk table: full chunks first, then the tails by decreasing size class.
  int run_full = 0, run_tail = 0;
  for (int base = 0; base < p.batch; base += 64) {
    const int b = base + lane;
    int nf = 0, nt = 0, len_b = 0;
    if (b < p.batch) {
      len_b = length_of(b);
      nf = (int)((unsigned)len_b / (unsigned)chunk);
      nt = ((len_b - nf * chunk) > 0 || len_b == 0) ? 1 : 0;  // an empty sequence keeps one (empty) chunk: it writes zeros
    }
    int sf = nf, st = nt;
    if (!in_lds) wave_scan2(sf, st, lane);
    if (b < p.batch) {
      const int f0 = in_lds ? first_full[b] : run_full + sf - nf;
      // (the table holds every chunk any lengths can produce — see workspace_layout —; the bound is
      // checked here all the same, so that nothing is ever written outside it)
      for (int ci = 0; ci < nf; ++ci) {
        if (f0 + ci < p.max_seq_chunks) {
          p.seq_chunks[f0 + ci] = SeqChunk{b, ci, len_b, nf + nt, ci * chunk, (ci + 1) * chunk, f0 + ci, 0};
        }
      }
      if (nt) {
        const int cls = tail_class(len_b - nf * chunk);
        const int slot = tail_hist[cls] + atomicAdd(&tail_fill[cls], 1);
        p.tail_prefix[b] = slot;
        if (total_full + slot < p.max_seq_chunks) {
          p.seq_chunks[total_full + slot] = SeqChunk{b, nf, len_b, nf + nt, nf * chunk, len_b, total_full + slot, 0};
        }
      }
    }
    if (!in_lds) {
      run_full += __shfl(sf, 63);
      run_tail += __shfl(st, 63);
    }
  }
}

}  // namespace xllm_hip
