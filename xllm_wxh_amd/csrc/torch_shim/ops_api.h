// libtorch host side of the HIP backend: the operators of xllm/core/kernels/ops_api.h that lie on
// the paged-KV decode path, plus the backend's batch_decode in both reference argument lists.
// Every function only checks the tensor contract and forwards pointers, sizes and strides to the
// C ABI (include/xllm_hip_paged_kv.h) on torch's current HIP stream; outputs are pre-allocated by
// the caller and mutated in place.  A contract violation throws through TORCH_CHECK (the reference
// aborts through glog CHECK: xllm/core/kernels/cuda/reshape_paged_cache.cu:68-69,
// xllm/core/kernels/ops_api.cpp:198-199).
#pragma once

#include <torch/torch.h>

#include <optional>
#include <vector>
#include <string>

#include "param.h"

namespace xllm::kernel {

// xllm/core/kernels/ops_api.h:31 — verbatim KV write through slot_mapping.
void reshape_paged_cache(ReshapePagedCacheParams& params);

// xllm/core/kernels/ops_api.h:35-37 — per-token-per-head quantising KV write (int8 / fp8-e4m3).
void quant_to_paged_cache(ReshapePagedCacheParams& params);

// xllm/core/kernels/ops_api.h:33 — cached sequences copied verbatim into dense tensors (paged mode).
void reshape_from_cache(ReshapeFromCacheParams& params);

// xllm/core/kernels/ops_api.h:41 — the same gather out of a quantised cache, dequantising on the way
// (what xllm/core/layers/mlu/attention.cpp:196-214 runs before a chunked prefill).
void dequant_from_paged_cache(ReshapeFromCacheParams& params);

namespace hip {

// The role of xllm::layer::PlanInfo (xllm/core/layers/common/attention_metadata.h:31-35): one per step,
// shared by every layer.  The model's layer loop sets layer_id before each layer
// (xllm/models/llm/llm_model_base.h:115); layer 0 builds the split-KV schedule of the step in the
// stream's workspace and the later layers reuse it (the reference plans at layer 0 only,
// xllm/core/layers/cuda/flashinfer_planinfo.cpp:252-253).  The schedule depends on the lengths, the
// block lists' addresses and the sizes, not on q, out or the cache's contents; `key` records what
// it was built for, and a later layer whose inputs differ is refused.
// host_plan (no counterpart in the reference, whose plan is always made on the host): the kernel and its work
// items follow from the step's sizes alone and the schedule always comes from the workspace
// (xllm_hip_decode_args::host_plan), so that a forward captured in a graph serves later steps of other lengths:
// captured, layer 0's device-side plan is part of the graph and reads the lengths of each replay.  kv_lens_host,
// if not empty (the engine's kv_seq_lens_vec, xllm/core/framework/model/model_input_params.h:341), makes layer 0
// plan on the host instead (xllm_hip_paged_decode_plan_host) when the stream is not being captured.
struct PlanInfo {
  int32_t layer_id = -1;
  const void* workspace = nullptr;  // where layer 0 left the schedule
  uint64_t key = 0;
  bool host_plan = false;
  std::vector<int32_t> kv_lens_host;
};

// Argument list of xllm::kernel::mlu::batch_decode (xllm/core/kernels/mlu/mlu_ops_api.h:126-145).
// query/output: [batch, q_len, Hq, D]; q_len > 1 = speculative verify, causal among the q_len tokens.
void batch_decode(const torch::Tensor& query,
                  const torch::Tensor& k_cache,
                  torch::Tensor& output,
                  const torch::Tensor& block_table,
                  const torch::Tensor& seq_lens,
                  const std::optional<torch::Tensor>& v_cache,
                  std::optional<torch::Tensor>& output_lse,
                  const std::optional<torch::Tensor>& q_quant_scale,
                  const std::optional<torch::Tensor>& k_cache_quant_scale,
                  const std::optional<torch::Tensor>& v_cache_quant_scale,
                  const std::optional<torch::Tensor>& out_quant_scale,
                  const std::optional<torch::Tensor>& alibi_slope,
                  const std::optional<torch::Tensor>& mask,
                  const std::string& compute_dtype,
                  int64_t max_seq_len,
                  int64_t window_size_left,
                  int64_t window_size_right,
                  float scale,
                  bool return_lse,
                  int64_t kv_cache_quant_bit_size,
                  int64_t total_kv_len = 0,
                  PlanInfo* plan_info = nullptr);

// Chunked prefill / mixed steps over the paged cache: the block_tables form of
// xllm::kernel::mlu::batch_prefill (xllm/core/kernels/mlu/mlu_ops_api.h:103-124, called with the caches
// as key/value in xllm/core/layers/mlu/attention.cpp:179-250).  query/output: [tokens, Hq, D]; sequence b
// owns rows q_cu_seq_lens[b] .. q_cu_seq_lens[b+1], the last tokens of its kv_seq_lens[b] cached tokens
// (already written), causal.  A quantised cache is attended directly (the reference dequantises it to
// a dense copy first, attention.cpp:182-222).
void batch_prefill_paged(const torch::Tensor& query,
                         const torch::Tensor& k_cache,
                         const torch::Tensor& v_cache,
                         torch::Tensor& output,
                         std::optional<torch::Tensor>& output_lse,
                         const torch::Tensor& q_cu_seq_lens,
                         const torch::Tensor& kv_seq_lens,
                         const std::optional<torch::Tensor>& k_cache_quant_scale,
                         const std::optional<torch::Tensor>& v_cache_quant_scale,
                         const torch::Tensor& block_tables,
                         int64_t max_query_len,
                         int64_t max_seq_len,
                         float scale,
                         int64_t window_size_left,
                         bool return_lse,
                         int64_t total_kv_len = 0,
                         PlanInfo* plan_info = nullptr);

// Tensor arguments of xllm::kernel::cuda::batch_decode (xllm/core/kernels/cuda/cuda_ops_api.h:120-136)
// without the FlashInfer uri / plan / workspaces, which have no counterpart here.
// query/output: [tokens, Hq, D]; caches in the CUDA backend's NHD shape [blocks, block_size, Hkv, D].
void batch_decode_csr(torch::Tensor query,
                      torch::Tensor k_cache,
                      torch::Tensor v_cache,
                      torch::Tensor paged_kv_indptr,
                      torch::Tensor paged_kv_indices,
                      torch::Tensor paged_kv_last_page_len,
                      int64_t window_left,
                      double sm_scale,
                      torch::Tensor output,
                      std::optional<torch::Tensor>& output_lse,
                      PlanInfo* plan_info = nullptr,
                      // a quantised cache (fp8 KV is what the CUDA-shaped caller anticipates,
                      // xllm/core/kernels/cuda/utils.cpp:275-293): fp32 scales [blocks, block_size, Hkv]
                      const std::optional<torch::Tensor>& k_cache_scale = std::nullopt,
                      const std::optional<torch::Tensor>& v_cache_scale = std::nullopt);

// xllm::kernel::cuda::fused_qk_norm_rope (xllm/core/kernels/cuda/cuda_ops_api.h:227-241): per-head RMSNorm
// and rotary embedding of the q and k heads of the fused buffer, in place.
void fused_qk_norm_rope(torch::Tensor& qkv,
                        int64_t num_heads_q,
                        int64_t num_heads_k,
                        int64_t num_heads_v,
                        int64_t head_dim,
                        double eps,
                        const torch::Tensor& q_weight,
                        const torch::Tensor& k_weight,
                        const torch::Tensor& cos_sin_cache,
                        bool interleaved,
                        const torch::Tensor& position_ids);

// xllm::kernel::cuda::rotary_embedding (xllm/core/kernels/cuda/rope.cu:152-249): rotation of query
// [tokens, heads * head_size] and, if given, key, in place, every operation rounded to the element type.
void rotary_embedding(torch::Tensor& positions,
                      torch::Tensor& query,
                      std::optional<torch::Tensor> key,
                      torch::Tensor& cos_sin_cache,
                      bool is_neox);

// Steps 2-5 of Qwen2AttentionImpl::forward up to the attention call
// (xllm/core/layers/common/qwen2_attention.cpp:147-189) in one launch: norm (when the weights are
// given) and rotation of q and k in place in qkv, then the KV write of the rotated k and of v through
// slot_mapping — quantising iff the scale tensors are given.
void rope_kv_write(torch::Tensor& qkv,
                   int64_t num_heads_q,
                   int64_t num_heads_kv,
                   int64_t head_dim,
                   const std::optional<torch::Tensor>& q_weight,
                   const std::optional<torch::Tensor>& k_weight,
                   double eps,
                   const torch::Tensor& cos_sin_cache,
                   bool interleaved,
                   bool round_each_op,
                   const torch::Tensor& position_ids,
                   const torch::Tensor& k_cache,
                   const torch::Tensor& v_cache,
                   const std::optional<torch::Tensor>& k_cache_scale,
                   const std::optional<torch::Tensor>& v_cache_scale,
                   const torch::Tensor& slot_mapping);

// Whole-block movement inside one layer's cache (K, V and the scale tensors together).
// swap_blocks: what KVCache::swap_blocks does (xllm/core/framework/kv_cache/kv_cache.cpp:104-125):
// blocks src[i] -> dst[i], int64 index tensors on the device, all sources read before any
// destination is written (a staging tensor is allocated for the call, as index_select does).
void swap_blocks(const torch::Tensor& k_cache,
                 const torch::Tensor& v_cache,
                 const std::optional<torch::Tensor>& k_cache_scale,
                 const std::optional<torch::Tensor>& v_cache_scale,
                 const torch::Tensor& src,
                 const torch::Tensor& dst);
// copy_blocks: the block-copy step on the batch builder's arrays
// (xllm/core/framework/batch/batch_input_builder.cpp:691-720, xllm/models/llm/npu/llm_model_base.h:69-75):
// block src_block_indices[g] -> blocks dst_block_indices[cum_sum[g-1] .. cum_sum[g]), int32 tensors.
void copy_blocks(const torch::Tensor& k_cache,
                 const torch::Tensor& v_cache,
                 const std::optional<torch::Tensor>& k_cache_scale,
                 const std::optional<torch::Tensor>& v_cache_scale,
                 const torch::Tensor& src_block_indices,
                 const torch::Tensor& dst_block_indices,
                 const torch::Tensor& cum_sum);

// Scratch of the decode kernels — the role of the reference's FlashinferWorkspace singleton
// (xllm/core/layers/cuda/flashinfer_workspace.cpp:24-38, sized by FLAGS_flashinfer_workspace_buffer_size,
// default 128 MiB: xllm/core/common/global_flags.cpp:564-567).  One buffer per (device, stream),
// allocated at the capacity in force when that stream first decodes and never reallocated: a captured
// HIP graph keeps the buffer's address, so a later, larger step must not move it, and steps on two
// streams must not share the plan, counters and partials.  A step that needs more than the buffer
// holds fails (TORCH_CHECK) instead of growing it.  `stream` is the hipStream_t the step runs on.
void set_decode_workspace_bytes(size_t bytes);  // capacity of buffers created from now on
size_t decode_workspace_capacity();
torch::Tensor decode_workspace(const torch::Device& device, void* stream);

}  // namespace hip
}  // namespace xllm::kernel
