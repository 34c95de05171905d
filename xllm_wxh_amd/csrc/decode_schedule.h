// The split-KV schedule of a decode step, made on the host from the kv lengths the engine holds there
// (the reference re-plans on the host before every step, also before every replay of a captured graph:
// xllm/core/runtime/cuda_graph_executor_impl.cpp:586-668, xllm/core/layers/cuda/flashinfer_planinfo.cpp:215-324;
// the lengths: xllm/core/framework/model/model_input_params.h:341 kv_seq_lens_vec).
//
// It fills the same tables as decode_plan_kernel (decode_plan.h), in a host buffer laid out like the head of the
// workspace, and differs from the device-side plan in what full knowledge of the lengths allows:
//   * every sequence is cut into chunks of its own, nearly equal size (no short tail behind full chunks);
//   * how finely to cut is chosen among a few targets by the finishing time a list schedule of the step's work
//     items predicts (each workgroup slot takes the next item when it falls free, which is what the hardware
//     dispatcher does with workgroups in index order);
//   * the chunks are dispatched longest first across all sequences.
// Host code only: no HIP types.
#pragma once

#include "decode_plan.h"

#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <functional>
#include <queue>
#include <vector>

namespace xllm_hip {

// The thresholds by which the host shapes a decode step (fill_params in paged_decode.hip reads them here; the
// reasoning stands beside each use), each with the measurement it came from — per layer on an existing schedule,
// one MI355X, 8 kv heads of 128 elements unless noted.  `bench.py --schedule-audit` times every choice they lead
// to against the forced alternatives.
struct ShapeRules {
  // Lengths count as nearly equal when max_len * batch <= total * 5 / 4: every sequence then owns the same number
  // of chunk slots and at most a fifth of the launch's workgroups find nothing to do (fixed-length buckets; the
  // ragged workload, lognormal sigma 0.8, has max * batch = 4 x total and keeps the stored schedule).
  int nearly_equal_num = 5, nearly_equal_den = 4;
  // One wave per kv head (work items of four heads, or four items to a workgroup) up to this mean length:
  // 1-byte cache 2048 x 256 tokens 242 -> 203 us, 256 x 6144 499 -> 492, 128 x 8192 326 -> 333 (not those);
  // 16-bit cache 4096 x 64 tokens 264 -> 193, 2048 x 128 202 -> 182, 256 tokens and more the same;
  // head_dim 64 over a 16-bit cache 4096 x 128 69 -> 51, 2048 x 768 130 -> 127, 2048 tokens the same.
  int wave_per_head_max_mean_quant = 8192, wave_per_head_max_mean_d64 = 2048, wave_per_head_max_mean_16bit = 192;
  // Its gain over four waves per head, as k / mean length up to a cap (fitted to the rows above): 1-byte rows of
  // 128 bytes 100 / L (19 % at 256 tokens, 5 % at 2048), of 64 bytes 200 / L; 16-bit rows of 256 bytes 16 / L, of
  // 128 bytes 25 / L.
  double wave_per_head_k_quant = 100.0, wave_per_head_k_quant_d64 = 200.0, wave_per_head_k_16bit = 16.0, wave_per_head_k_16bit_d64 = 25.0;
  double wave_per_head_cap_quant = 0.2, wave_per_head_cap_quant_d64 = 0.4, wave_per_head_cap_16bit = 0.3;
  // Four-head items over a 1-byte cache whose heads lie side by side gain this much from the layout alone
  // (fp8, 128 x 8192 tokens, NHD: 391 -> 338 us).
  double side_by_side_gain = 0.16;
  // The same where the rows are 64 bytes and two kv heads share a 128-byte line (head_dim 64, 1-byte cache, NHD):
  // waves that attend neighbouring heads in step, against four waves to a head (int8, 14q/2kv, 512 x 8192 tokens
  // 259 -> 209 us; 32q/8kv, 64 x 16384 tokens 314 -> 232).
  double short_rows_gain = 0.24;
  // Narrow items whose last round's sequences are cut fill their rounds but for the merges; the wider form must
  // beat the narrow one by this factor to be taken (192 sequences of 2048 fp8 tokens, 1.5 rounds of four-head
  // workgroups: 148 us against 134).
  double cut_rounds_filled = 0.97, wider_items_hurdle = 1.01;
  // Eight waves per item (1-byte caches) when the launch has at most one item per CU and at least three quarters
  // of the CUs get one (20 x 8192 fp8 tokens: 69 us as 160 eight-wave items, 65 as 480 four-wave items), and
  // while the items are at most a quarter more than the CUs, the sequences past a round being cut (33 sequences x
  // 8192 fp8 tokens: 105 -> 100 us, 40: 122 -> 116).
  int eight_waves_min_num = 3, eight_waves_min_den = 4, eight_waves_over_num = 5, eight_waves_over_den = 4;
  // The fused merge loads 32 partials in one batch: no sequence is cut finer by the rules that rely on it (one
  // 32768-token fp8 sequence: 31 us at 256 items, 38 at 512).
  int fused_merge_max_chunks = 32;
  // The sequences of a partly filled last round are cut while the step is under four rounds (288 x 2048 fp8
  // tokens, 4.5 rounds: 202 us whole, 206 cut); an even cut that fills under nine tenths of a round is taken one
  // finer first (1-byte caches); cut in two throughout, the last round's sequences must get at least three times
  // the others' chunks (fp8, 8192 tokens: 40 sequences 132 -> 122 us, 48, four chunks each, 136 -> 144).
  int cut_last_round_below_rounds = 4, round_fill_num = 9, round_fill_den = 10, last_round_min_ratio = 3;
};
constexpr ShapeRules kShapeRules{};

struct HostScheduleInput {
  const int32_t* kv_lens;  // [batch], as the kernels will see them (cut to 0 .. len_cap here)
  int32_t batch;
  int32_t len_cap;         // tokens a sequence's block list can hold (INT32_MAX: unknown)
  int32_t per;             // work items per sequence chunk: kv heads (or head groups) x row groups
  int32_t slots;           // workgroups the GPU runs at once
  int32_t tile;            // chunk sizes are multiples of it
  int32_t min_chunk;       // no chunk of a cut sequence is shorter
  int64_t max_seq_chunks;  // records and partial rows the workspace holds, and the launch covers
  int32_t max_per_seq;     // chunks a sequence is cut into at most
  double item_overhead;    // fixed cost of a work item, in tokens of streaming (prologue, epilogue, partial rows)
  double solo_speedup;     // rate of a workgroup that has its CU to itself, against one that shares it (a CU holds
                           // two slots: over a 16-bit cache one workgroup already streams at the CU's full rate)
  double merge_base;       // what a step that cuts sequences ends with: the merge of the last one, in tokens ...
  double merge_per_chunk;  // ... plus this much per chunk of the sequence with the most
};

struct HostScheduleResult {
  int32_t chunk_target = 0;    // the chunk size the cut was made for (0: nothing is cut)
  int64_t total_chunks = 0;
  double predicted_span = 0;   // finishing time of the list schedule, in tokens
  size_t bytes = 0;            // bytes of the host buffer that hold the schedule (header .. last record)
};

inline int32_t schedule_clamped_len(int32_t len, int32_t cap) {
  len = len < cap ? len : cap;
  return len > 0 ? len : 0;
}

// Chunk size and count of a sequence of `len` tokens cut for chunks of about `target` tokens: n nearly equal
// chunks, tile-aligned, none below min_chunk unless the sequence is whole.
inline void schedule_cut(int32_t len, int64_t target, const HostScheduleInput& in, int32_t& n, int32_t& chunk) {
  n = 1;
  chunk = len;
  if (target <= 0 || len <= target + target / 4) return;  // (a sequence that would only shed a small piece stays whole)
  int64_t parts = (len + target - 1) / target;
  if (parts > in.max_per_seq) parts = in.max_per_seq;
  int64_t c = (len + parts - 1) / parts;
  c = (c + in.tile - 1) / in.tile * in.tile;
  if (c < in.min_chunk) c = in.min_chunk;
  const int64_t cnt = (len + c - 1) / c;
  if (cnt <= 1) return;
  n = (int32_t)cnt;
  chunk = (int32_t)c;
}

// Finishing time of the step if its sequence chunks, `per` equal work items each, are handed to `slots` slots
// longest first.  Items of one sequence chunk start together on `per` slots, so the slots are simulated in
// groups of `per` (the last group may be narrower; it is treated as a full one: an upper estimate).  A step
// with no more items than slots runs them all at once, the faster the more CUs hold a single workgroup.
inline double schedule_span(std::vector<int32_t>& sizes, const HostScheduleInput& in) {
  std::sort(sizes.begin(), sizes.end(), std::greater<int32_t>());
  int64_t lanes = in.slots / (in.per > 0 ? in.per : 1);
  if (lanes < 1) lanes = 1;
  if (sizes.empty()) return 0.0;
  if ((int64_t)sizes.size() <= lanes) {
    const double spare = (double)(lanes - (int64_t)sizes.size()) / (0.5 * (double)lanes);
    const double rate = 1.0 + (in.solo_speedup - 1.0) * (spare < 1.0 ? spare : 1.0);
    return sizes[0] / rate + in.item_overhead;
  }
  std::priority_queue<double, std::vector<double>, std::greater<double>> free_at;
  for (int64_t i = 0; i < lanes; ++i) free_at.push(0.0);
  double span = 0.0;
  for (int32_t s : sizes) {
    const double t = free_at.top() + s + in.item_overhead;
    free_at.pop();
    free_at.push(t);
    span = t > span ? t : span;
  }
  return span;
}

// Builds the schedule into `host` (laid out by `w`, the workspace's own layout: header, kv_len, full_prefix,
// tail_prefix, num_chunks, seq_chunks).  `host_bytes` must cover w.seq_chunks + max_seq_chunks records.
inline bool host_schedule(const HostScheduleInput& in, const WorkspaceLayout& w, uint8_t* host, size_t host_bytes,
                          HostScheduleResult& out) {
  const int64_t room = in.max_seq_chunks < w.max_seq_chunks ? in.max_seq_chunks : w.max_seq_chunks;
  if (in.batch < 0 || room < in.batch || host_bytes < w.seq_chunks + sizeof(SeqChunk) * (size_t)room) return false;
  int64_t total = 0;
  int32_t longest = 0;
  for (int32_t b = 0; b < in.batch; ++b) {
    const int32_t l = schedule_clamped_len(in.kv_lens[b], in.len_cap);
    total += l;
    longest = l > longest ? l : longest;
  }
  // Candidate chunk sizes: nothing cut; then the work spread over 0.5, 1, 1.5, 2, 3 and 4 times the slots.
  const int64_t lanes = std::max<int64_t>(1, in.slots / (in.per > 0 ? in.per : 1));
  int64_t best_target = 0;
  double best_span = -1.0;
  int64_t best_count = in.batch;
  std::vector<int32_t> sizes;
  sizes.reserve((size_t)room);
  const int kNum[7] = {0, 1, 2, 3, 4, 6, 8};  // halves of the slots
  for (int k = 0; k < 7; ++k) {
    // (a cut aimed at a quarter as many chunks as there are sequences changes nothing that matters — a batch of
    // that many rounds is balanced by its number — so a large batch ends here, after one pass over its lengths)
    if (kNum[k] > 0 && 2 * lanes * kNum[k] <= in.batch) continue;
    int64_t target = 0;
    if (kNum[k] > 0) {
      target = (2 * total + lanes * kNum[k] - 1) / (lanes * kNum[k]);
      target = (target + in.tile - 1) / in.tile * in.tile;
      if (target < in.min_chunk) target = in.min_chunk;
      if (target >= longest) continue;  // cuts nothing
    }
    // (rounding up sequence by sequence may leave a few chunks more than the slots' multiple that was aimed
    // for, and those few would take a round of their own: the target grows until they are gone)
    const int64_t aim = kNum[k] > 0 ? std::max<int64_t>(lanes * kNum[k] / 2, in.batch) : in.batch;
    int64_t count = 0;
    for (int attempt = 0; attempt < 12; ++attempt) {
      count = 0;
      for (int32_t b = 0; b < in.batch; ++b) {
        int32_t n, c;
        schedule_cut(schedule_clamped_len(in.kv_lens[b], in.len_cap), target, in, n, c);
        count += n;
      }
      if (kNum[k] == 0 || count <= aim || target >= longest) break;
      target += std::max<int64_t>(in.tile, target / 32 / in.tile * in.tile);
    }
    const bool fits = count <= room;
    if (kNum[k] == 0 && fits && 2 * lanes * kNum[6] <= in.batch) {  // (the only candidate: its finishing time is not asked for)
      best_span = 0.0;
      continue;
    }
    if (fits && (target == best_target && best_span >= 0.0)) continue;  // (the same cut as the best so far)
    int32_t most = 1;
    sizes.clear();
    for (int32_t b = 0; b < in.batch && fits; ++b) {
      const int32_t l = schedule_clamped_len(in.kv_lens[b], in.len_cap);
      int32_t n, c;
      schedule_cut(l, target, in, n, c);
      for (int32_t i = 0; i < n; ++i) sizes.push_back(std::min(c, l - i * c));
      most = n > most ? n : most;
    }
    if (!fits) continue;
    const double span = schedule_span(sizes, in) + (most > 1 ? in.merge_base + in.merge_per_chunk * most : 0.0);
    if (best_span < 0.0 || span < best_span * 0.98) {  // (a finer cut must gain at least 2 %: it costs partial rows)
      best_span = span;
      best_target = target;
      best_count = count;
    }
  }
  // Tables.  Partial slots in sequence order (full_prefix), dispatch longest first.
  PlanHeader hdr;
  memset(&hdr, 0, sizeof(hdr));
  int32_t* kv_len = (int32_t*)(host + w.kv_len);
  int32_t* full_prefix = (int32_t*)(host + w.full_prefix);
  int32_t* tail_prefix = (int32_t*)(host + w.tail_prefix);
  int32_t* num_chunks = (int32_t*)(host + w.num_chunks);
  SeqChunk* table = (SeqChunk*)(host + w.seq_chunks);
  int32_t slot = 0;
  for (int32_t b = 0; b < in.batch; ++b) {
    const int32_t l = schedule_clamped_len(in.kv_lens[b], in.len_cap);
    int32_t n, c;
    schedule_cut(l, best_target, in, n, c);
    kv_len[b] = l;
    full_prefix[b] = slot;
    tail_prefix[b] = 0;
    num_chunks[b] = n;
    for (int32_t i = 0; i < n; ++i) {
      SeqChunk r;
      r.seq = b;
      r.chunk = i;
      r.len = l;
      r.chunks = n;
      r.t_begin = i * c;
      r.t_end = std::min<int64_t>((int64_t)(i + 1) * c, l);
      r.slot = slot + i;
      r.pad = 0;
      table[slot + i] = r;
    }
    slot += n;
  }
  full_prefix[in.batch] = slot;
  tail_prefix[in.batch] = 0;
  std::stable_sort(table, table + slot, [](const SeqChunk& a, const SeqChunk& b) {
    return a.t_end - a.t_begin > b.t_end - b.t_begin;
  });
  hdr.total_full = slot;
  hdr.total_tail = 0;
  hdr.chunk_tokens = (int32_t)best_target;
  hdr.total_items = slot * in.per;
  memcpy(host + w.header, &hdr, sizeof(hdr));
  out.chunk_target = (int32_t)best_target;
  out.total_chunks = best_count;
  out.predicted_span = best_span;
  out.bytes = w.seq_chunks + sizeof(SeqChunk) * (size_t)slot;
  return true;
}

}  // namespace xllm_hip
