// Host-side harness for tests/test_plan_bounds.py: the chunk choice and the workspace bound of the
// decode plan, as plain C functions over the header the kernels are built from.
#include "decode_plan.h"

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
}
