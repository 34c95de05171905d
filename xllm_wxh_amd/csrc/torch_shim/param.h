// Parameter blocks of the KV-write and cache read-back operators, field for field the reference's
// xllm::kernel::ReshapePagedCacheParams (xllm/core/kernels/param.h:122-157) and
// xllm::kernel::ReshapeFromCacheParams (xllm/core/kernels/param.h:160-215).
#pragma once

#include <torch/torch.h>

#include <optional>

namespace xllm::kernel {

struct ReshapePagedCacheParams {
  // [num_tokens, num_kv_heads, head_dim]; last two dimensions contiguous, token stride free.
  torch::Tensor key;
  std::optional<torch::Tensor> value;
  // Paged caches.  Native shape [num_blocks, num_kv_heads, block_size, head_dim]; a tensor with
  // permuted strides (e.g. an NHD buffer viewed through permute(0, 2, 1, 3)) is accepted as is.
  torch::Tensor k_cache;
  std::optional<torch::Tensor> v_cache;
  // [num_tokens] int32, contiguous.
  torch::Tensor slot_mapping;
  // false = context to cache.  true (cache to context) is not part of the decode path.
  bool direction = false;
  // [num_blocks, num_kv_heads, block_size] float32; required by quant_to_paged_cache.
  std::optional<torch::Tensor> k_cache_scale;
  std::optional<torch::Tensor> v_cache_scale;
};

struct ReshapeFromCacheParams {
  // Outputs [total_length, num_kv_heads, head_dim], last two dimensions contiguous.
  // reshape_from_cache: the cache's dtype.  dequant_from_paged_cache: bf16 / fp16 / fp32.
  torch::Tensor key;
  std::optional<torch::Tensor> value;
  // Paged caches [num_blocks, num_kv_heads, block_size, head_dim] (permuted strides accepted).
  torch::Tensor key_cache;
  std::optional<torch::Tensor> value_cache;
  // [batch] int32: cached tokens of each sequence; none may exceed max_context_len.
  torch::Tensor context_lengths;
  int64_t max_context_len = 0;
  // [batch] int32: first output row of each sequence (default: packed in order).
  std::optional<torch::Tensor> context_seq_offset;
  // [batch, max_blocks] int32.  Required: the linear (unpaged) cache mode is not part of this path.
  std::optional<torch::Tensor> block_tables;
  // [batch] int32: first cached position of each sequence (default 0).
  std::optional<torch::Tensor> cache_seq_offset;
  // dequant_from_paged_cache only: float32 scales [num_blocks, num_kv_heads, block_size]
  // (quant_mode 1, per token) or [num_kv_heads, head_dim] (quant_mode 0, per channel).
  std::optional<torch::Tensor> key_cache_quant_scale;
  std::optional<torch::Tensor> value_cache_quant_scale;
  int64_t quant_mode = 1;
  int64_t quant_bit = 8;
};

}  // namespace xllm::kernel
