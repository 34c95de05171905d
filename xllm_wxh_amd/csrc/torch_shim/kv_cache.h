// Per-layer KV cache holder of the HIP backend — the role of xllm::KVCache
// (xllm/core/framework/kv_cache/kv_cache.h:27-77) restricted to what the decode path touches.
#pragma once

#include <torch/torch.h>

#include <optional>
#include <utility>
#include <vector>

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

  // Allocates the K and V pools of one layer (and, if `with_scales`, their fp32 scale tensors of the
  // cache shape minus its last dimension) — what xllm/core/runtime/worker_impl.cpp:229-313 does with
  // one torch::zeros per tensor.  Here K and V are carved from ONE buffer, V starting kSkewBytes past a
  // 2 MiB boundary behind K: a decode work item reads block b of K and block b of V together, and
  // when the two pools are separate allocations (whose addresses differ by a multiple of 2 MiB) those
  // two reads meet in the same DRAM channel.  Measured on one MI355X: Llama-3-8B decode, batch 64 x
  // 4096 tokens, 162.4 -> 158.8 us per step (82.7 -> 84.6 % of 8 TB/s); fp8 cache 333 -> 326 us.
  // `shape` is the cache shape in either layout ([blocks, heads, slots, dim] or [blocks, slots, heads, dim]).
  static constexpr int64_t kSkewBytes = 4096;
  static constexpr int64_t kPageBytes = 2 << 20;
  static KVCache allocate(const std::vector<int64_t>& shape, torch::ScalarType dtype, const torch::Device& device,
                          bool with_scales = false) {
    TORCH_CHECK(shape.size() == 4, "cache shape must have four dimensions");
    auto pair = [&](const std::vector<int64_t>& shp, torch::ScalarType dt) {
      int64_t numel = 1;
      for (int64_t d : shp) numel *= d;
      const int64_t bytes = numel * (int64_t)torch::elementSize(dt);
      const int64_t v_at = (bytes + kPageBytes - 1) / kPageBytes * kPageBytes + kSkewBytes;
      torch::Tensor buf = torch::zeros({v_at + bytes}, torch::TensorOptions().dtype(torch::kUInt8).device(device));
      return std::make_pair(buf.narrow(0, 0, bytes).view(dt).view(shp), buf.narrow(0, v_at, bytes).view(dt).view(shp));
    };
    auto kv = pair(shape, dtype);
    if (!with_scales) return KVCache(kv.first, kv.second);
    auto sc = pair(std::vector<int64_t>(shape.begin(), shape.end() - 1), torch::kFloat32);
    return KVCache(kv.first, kv.second, sc.first, sc.second);
  }

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
