// Batch-level attention inputs shared by every layer of a step: the fields of
// xllm::layer::AttentionMetadata (xllm/core/layers/common/attention_metadata.h:68-153) that the
// decode path reads, built from cumulative lengths the way
// xllm/core/layers/common/attention_metadata_builder.cpp:29-124 does.
#pragma once

#include <algorithm>

#include <torch/torch.h>

#include <memory>

#include "host_index.h"
#include "ops_api.h"

namespace xllm::layer {

using PlanInfo = xllm::kernel::hip::PlanInfo;

struct AttentionMetadata {
  torch::Tensor q_cu_seq_lens;
  torch::Tensor kv_cu_seq_lens;
  torch::Tensor kv_seq_lens;  // per sequence (diff of the cumulative lengths)
  torch::Tensor q_seq_lens;
  torch::Tensor block_table;   // [batch, max_blocks] int32, padded with 0
  torch::Tensor slot_mapping;  // [num_tokens] int32
  int64_t max_query_len = 0;
  int64_t max_seq_len = 0;
  int64_t total_kv_len = 0;
  bool is_prefill = false;
  bool is_chunked_prefill = false;
  bool is_dummy = false;
  bool is_causal = false;
  // Split-KV schedule of the step, built at layer 0 and shared by every layer
  // (attention_metadata.h:112-117).  Null: every call builds its own.
  std::shared_ptr<PlanInfo> plan_info;
  // CSR form of the block lists (the CUDA backend's inputs).
  torch::Tensor paged_kv_indptr;
  torch::Tensor paged_kv_indices;
  torch::Tensor paged_kv_last_page_len;
};

// Decode-step metadata from the batch builder's tensors: cumulative kv/q lengths [batch+1],
// new_cache_slots, block_tables.  kv_seq_lens = diff(cumulative) (attention_metadata_builder.cpp:105);
// a dummy batch (q_max_seq_len == 0) writes slot 1 only (:120-124).
inline AttentionMetadata build_decode_metadata(const torch::Tensor& q_cu_seq_lens,
                                               const torch::Tensor& kv_cu_seq_lens,
                                               const torch::Tensor& new_cache_slots,
                                               const torch::Tensor& block_tables,
                                               int64_t q_max_seq_len,
                                               int64_t kv_max_seq_len,
                                               int64_t total_kv_len) {
  AttentionMetadata m;
  m.plan_info = std::make_shared<PlanInfo>();  // layer_id -1 until the layer loop sets it (attention_metadata_builder.cpp:60)
  m.q_cu_seq_lens = q_cu_seq_lens;
  m.kv_cu_seq_lens = kv_cu_seq_lens;
  m.max_query_len = q_max_seq_len;
  m.max_seq_len = kv_max_seq_len;
  m.total_kv_len = total_kv_len;
  m.slot_mapping = new_cache_slots;
  m.block_table = block_tables;
  m.kv_seq_lens = torch::diff(kv_cu_seq_lens).contiguous();
  m.q_seq_lens = torch::diff(q_cu_seq_lens).contiguous();
  m.is_dummy = q_max_seq_len == 0;
  if (m.is_dummy) m.slot_mapping = torch::tensor({1}, new_cache_slots.options());
  return m;
}

// The same from the host-side batch arrays: their int32 tensors are created on `device` the way
// BatchInputBuilder::state_to_forward_input (xllm/core/framework/batch/batch_input_builder.cpp:500-560)
// creates them (block tables padded with 0), CSR arrays included.
inline AttentionMetadata build_decode_metadata(const host_index::DecodeBatchInputs& in, const torch::Device& device) {
  auto i32 = [&](const std::vector<int32_t>& v) {
    return torch::tensor(v, torch::TensorOptions().dtype(torch::kInt32)).to(device);
  };
  int32_t max_blocks = 0;
  const std::vector<int32_t> flat = in.pad_block_tables(max_blocks);
  torch::Tensor table = i32(flat).view({(int64_t)in.num_sequences(), (int64_t)max_blocks});
  AttentionMetadata m = build_decode_metadata(i32(in.q_seq_lens), i32(in.kv_seq_lens), i32(in.new_cache_slots), table,
                                              in.q_max_seq_len, in.kv_max_seq_len, in.total_kv_len());
  m.paged_kv_indptr = i32(in.paged_kv_indptr);
  m.paged_kv_indices = i32(in.paged_kv_indices);
  m.paged_kv_last_page_len = i32(in.paged_kv_last_page_len);
  // The lengths are on the host here, as in the reference's engine (model_input_params.h:341 kv_seq_lens_vec),
  // whose plan is made from them.  A ragged batch takes the schedule made on the host, which cuts every long
  // sequence by its own length (3-17 % per layer on 16 to 64 sequences of lognormal lengths); nearly equal
  // lengths keep the device-side plan with the two aggregates, whose work-item shapes may follow the lengths
  // (many short sequences: a wave per kv head, 20-30 % there).
  const size_t batch = in.kv_seq_lens.size() > 0 ? in.kv_seq_lens.size() - 1 : 0;
  int64_t longest = 0;
  for (size_t b = 0; b < batch; ++b) longest = std::max<int64_t>(longest, in.kv_seq_lens[b + 1] - in.kv_seq_lens[b]);
  if (batch > 0 && longest * (int64_t)batch * 4 > in.total_kv_len() * 5) {
    m.plan_info->kv_lens_host.resize(batch);
    for (size_t b = 0; b < batch; ++b) m.plan_info->kv_lens_host[b] = in.kv_seq_lens[b + 1] - in.kv_seq_lens[b];
  }
  return m;
}

}  // namespace xllm::layer
