// Parameter block of the KV-write operators, field for field the reference's
// xllm::kernel::ReshapePagedCacheParams (xllm/core/kernels/param.h:122-157).
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

}  // namespace xllm::kernel
