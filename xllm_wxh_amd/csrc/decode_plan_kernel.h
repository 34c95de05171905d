// Device-side plan of a decode step: kv lengths -> chunk size -> chunk table (see decode_plan.h).
#pragma once

#include "decode_params.h"
#include "device_utils.h"

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Plan: one workgroup.  kv lengths -> total -> chunk size -> prefix sums -> chunk table.
// ---------------------------------------------------------------------------------

// Inclusive scan of (a, b) over the wave.
__device__ inline void wave_scan2(int& a, int& b, int lane) {
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int ua = __shfl_up(a, o), ub = __shfl_up(b, o);
    if (lane >= o) {
      a += ua;
      b += ub;
    }
  }
}

// The finished-chunk counters of the fused merge at the start of a step that stores no schedule.
__global__ void __launch_bounds__(256) decode_zero_counters_kernel(int32_t* counters, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) counters[i] = 0;
}

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

  // 1. kv lengths, their sum and their maximum.
  long long total = 0;
  int max_len = 0;
  for (int b = lane; b < p.batch; b += 64) {
    const int len = kv_length(p, b);
    p.kv_len[b] = len;
    total += len;
    max_len = len > max_len ? len : max_len;
  }
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
  auto length_of = [&](int b) { return kv_length(p, b); };
  // The tail chunks differ in size.  They are dispatched after the (equal) full chunks, longest
  // first — in 64 size classes — so that the launch ends with the shortest work items.
  auto tail_class = [&](int tail_len) { return (int)(((long long)tail_len * 64) / chunk); };  // tail_len < chunk
  int total_full = 0, total_tail = 0;
  for (int base = 0; base < p.batch; base += 64) {
    const int b = base + lane;
    int nf = 0, nt = 0;
    if (b < p.batch) {
      const int len = length_of(b);
      nf = len / chunk;
      nt = ((len - nf * chunk) > 0 || len == 0) ? 1 : 0;  // an empty sequence keeps one (empty) chunk: it writes zeros
      if (nt) atomicAdd(&tail_hist[tail_class(len - nf * chunk)], 1);
    }
    int sf = nf, st = nt;
    wave_scan2(sf, st, lane);
    if (b < p.batch) {
      p.full_prefix[b] = total_full + sf - nf;
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
      nf = len_b / chunk;
      nt = ((len_b - nf * chunk) > 0 || len_b == 0) ? 1 : 0;  // an empty sequence keeps one (empty) chunk: it writes zeros
    }
    int sf = nf, st = nt;
    wave_scan2(sf, st, lane);
    if (b < p.batch) {
      const int f0 = run_full + sf - nf;
      // (the table holds every chunk any lengths can produce — see workspace_layout —; the bound is
      // checked here all the same, so that nothing is ever written outside it)
      for (int ci = 0; ci < nf; ++ci) {
        if (f0 + ci < p.max_seq_chunks) p.seq_chunks[f0 + ci] = SeqChunk{b, ci, len_b, nf + nt};
      }
      if (nt) {
        const int cls = tail_class(len_b - nf * chunk);
        const int slot = tail_hist[cls] + atomicAdd(&tail_fill[cls], 1);
        p.tail_prefix[b] = slot;
        if (total_full + slot < p.max_seq_chunks) p.seq_chunks[total_full + slot] = SeqChunk{b, nf, len_b, nf + nt};
      }
    }
    run_full += __shfl(sf, 63);
    run_tail += __shfl(st, 63);
  }
}

}  // namespace xllm_hip
