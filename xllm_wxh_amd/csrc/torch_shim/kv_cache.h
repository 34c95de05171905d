// Per-layer KV cache holder of the HIP backend — the role of xllm::KVCache
// (xllm/core/framework/kv_cache/kv_cache.h:27-77) restricted to what the decode path touches.
#pragma once

#include <torch/torch.h>

#include <optional>

#include "ops_api.h"

namespace xllm {

class KVCache final {
 public:
  KVCache() = default;
  // key/value cache: [num_blocks, num_kv_heads, block_size, head_dim] (HND, the native layout of the
  // HIP backend; an NHD buffer is passed as buffer.permute({0, 2, 1, 3})).
  KVCache(torch::Tensor key_cache, torch::Tensor value_cache)
      : key_cache_(std::move(key_cache)), value_cache_(std::move(value_cache)) {}
  // Quantised cache (int8 / float8_e4m3fn) with fp32 scales [num_blocks, num_kv_heads, block_size].
  KVCache(torch::Tensor key_cache, torch::Tensor value_cache, torch::Tensor key_cache_scale,
          torch::Tensor value_cache_scale)
      : key_cache_(std::move(key_cache)),
        value_cache_(std::move(value_cache)),
        key_cache_scale_(std::move(key_cache_scale)),
        value_cache_scale_(std::move(value_cache_scale)) {}

  torch::Tensor get_k_cache() const { return key_cache_; }
  torch::Tensor get_v_cache() const { return value_cache_; }

  // nullopt when the cache is not quantised: this is the switch between reshape_paged_cache and
  // quant_to_paged_cache (xllm/core/framework/kv_cache/kv_cache.cpp:56-67,
  // xllm/core/layers/mlu/attention.cpp:96-117).
  std::optional<torch::Tensor> get_k_cache_scale() const {
    if (!key_cache_scale_.defined() || key_cache_scale_.numel() == 0) return std::nullopt;
    return key_cache_scale_;
  }
  std::optional<torch::Tensor> get_v_cache_scale() const {
    if (!value_cache_scale_.defined() || value_cache_scale_.numel() == 0) return std::nullopt;
    return value_cache_scale_;
  }

  bool empty() const { return !key_cache_.defined() || !value_cache_.defined(); }

  // Batched block copy src_tensor[i] -> dst_tensor[i] over K, V and the scales, sources read first
  // (xllm/core/framework/kv_cache/kv_cache.cpp:104-125).
  void swap_blocks(torch::Tensor& src_tensor, torch::Tensor& dst_tensor) {
    kernel::hip::swap_blocks(key_cache_, value_cache_, get_k_cache_scale(), get_v_cache_scale(), src_tensor,
                             dst_tensor);
  }

 private:
  torch::Tensor key_cache_;
  torch::Tensor value_cache_;
  torch::Tensor key_cache_scale_;
  torch::Tensor value_cache_scale_;
};

}  // namespace xllm
