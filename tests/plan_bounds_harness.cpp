// Host-side harness for tests/test_plan_bounds.py: the chunk choice and the workspace bound of the
// decode plan, as plain C functions over the header the kernels are built from.
#include "decode_plan.h"
#include "decode_schedule.h"

#include <vector>

extern "C" {

int harness_choose_chunk(long long total, long long max_len, int batch, int num_kv_heads, int row_groups, int target,
                         int target_small, int min_chunk, int tile) {
  return xllm_hip::choose_chunk(total, max_len, batch, num_kv_heads, row_groups, target, target_small, min_chunk, tile);
}

long long harness_max_seq_chunks(int batch, int q_per_seq, int num_q_heads, int num_kv_heads, int head_dim) {
  return xllm_hip::workspace_layout(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim).max_seq_chunks;
}

int harness_row_groups(int q_per_seq, int num_q_heads, int num_kv_heads, int rows_per_item) {
  return xllm_hip::row_groups(q_per_seq, num_q_heads, num_kv_heads, rows_per_item);
}

int harness_max_target_items() { return xllm_hip::kMaxTargetItems; }

// The schedule made on the host for `lens`: the records (8 ints each) into `records`, the per-sequence arrays into
// kv_len / first_slot / num_chunks; returns the number of records, or -1 when the step does not fit.
// out[0..2]: chunk size the cut was made for, total items of the header, predicted span.
long long harness_host_schedule(const int* lens, int batch, int len_cap, int per, int slots, int tile, int min_chunk,
                                long long max_seq_chunks, int max_per_seq, double item_overhead, double solo_speedup, int q_per_seq,
                                int num_q_heads, int num_kv_heads, int head_dim, int* records, int* kv_len,
                                int* first_slot, int* num_chunks, long long* out) {
  using namespace xllm_hip;
  const WorkspaceLayout w = workspace_layout(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim);
  std::vector<uint8_t> host(w.partial_lse);
  HostScheduleInput in;
  in.kv_lens = lens;
  in.batch = batch;
  in.len_cap = len_cap;
  in.per = per;
  in.slots = slots;
  in.tile = tile;
  in.min_chunk = min_chunk;
  in.max_seq_chunks = max_seq_chunks;
  in.max_per_seq = max_per_seq;
  in.item_overhead = item_overhead;
  in.solo_speedup = solo_speedup;
  in.merge_base = item_overhead;
  in.merge_per_chunk = item_overhead * 0.03;
  HostScheduleResult r;
  if (!host_schedule(in, w, host.data(), host.size(), r)) return -1;
  const PlanHeader* hdr = (const PlanHeader*)(host.data() + w.header);
  const long long n = hdr->total_full + hdr->total_tail;
  memcpy(records, host.data() + w.seq_chunks, sizeof(SeqChunk) * (size_t)n);
  memcpy(kv_len, host.data() + w.kv_len, sizeof(int) * (size_t)batch);
  memcpy(first_slot, host.data() + w.full_prefix, sizeof(int) * ((size_t)batch + 1));
  memcpy(num_chunks, host.data() + w.num_chunks, sizeof(int) * (size_t)batch);
  out[0] = r.chunk_target;
  out[1] = hdr->total_items;
  out[2] = (long long)r.predicted_span;
  out[3] = (long long)w.max_seq_chunks;
  return n;
}
}
