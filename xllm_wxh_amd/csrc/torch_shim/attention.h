// Attention dispatch of the HIP backend: KV write, then attention over the paged cache (decode,
// speculative verify, and prefill chunks / mixed steps through the same kernels) — the role of
// xllm::layer::AttentionImpl (xllm/core/layers/cuda/attention.h:41-46,
// xllm/core/layers/mlu/attention.h:47-52; same constructor and forward signature on every backend).
#pragma once

#include <torch/torch.h>

#include <optional>
#include <tuple>

#include "attention_metadata.h"
#include "kv_cache.h"

namespace xllm::layer {

class AttentionImpl {
 public:
  AttentionImpl(int64_t num_heads, int64_t head_size, float scale, int64_t num_kv_heads, int64_t sliding_window);

  // query [T, Hq*D], key/value [T, Hkv*D] (slices of the fused qkv buffer are fine).
  // Returns (output [T, Hq*D], lse = nullopt).
  std::tuple<torch::Tensor, std::optional<torch::Tensor>> forward(const AttentionMetadata& attn_metadata,
                                                                   torch::Tensor& query,
                                                                   torch::Tensor& key,
                                                                   torch::Tensor& value,
                                                                   KVCache& kv_cache);

  // The same step fed from the fused qkv buffer before norm and rotation — what
  // Qwen2AttentionImpl::forward does between the qkv projection and the output projection
  // (xllm/core/layers/common/qwen2_attention.cpp:147-189): one launch for q/k norm (when the weights
  // are given), rotary embedding and the KV write, then the decode.  qkv [T, (Hq + 2 Hkv) * D] is
  // updated in place; returns (output [T, Hq*D], lse = nullopt).
  std::tuple<torch::Tensor, std::optional<torch::Tensor>> forward_qkv(const AttentionMetadata& attn_metadata,
                                                                       const torch::Tensor& positions,
                                                                       torch::Tensor& qkv,
                                                                       const torch::Tensor& cos_sin_cache,
                                                                       bool interleaved,
                                                                       const std::optional<torch::Tensor>& q_norm_weight,
                                                                       const std::optional<torch::Tensor>& k_norm_weight,
                                                                       double eps,
                                                                       KVCache& kv_cache);

  // Prefill chunks over a quantised cache are attended in place (the many-row kernel converts each
  // tile once per 128 query rows).  From this many query rows per kv head on (averaged over the step's
  // sequences: 4096 = chunks of 1024 tokens at four query heads per kv head) the cached ranges are
  // instead dequantised once into a dense 16-bit copy, which the 16-bit many-row kernel then attends —
  // the order of operations of the reference's MLU layer (xllm/core/layers/mlu/attention.cpp:179-228);
  // with that many row groups per sequence one conversion is cheaper than one per row group
  // (2 x 2048 tokens on 6144: 710 us against 840 us in place; 4 x 512 on 3584: 261 against 256).
  // The copy lives in buffers shared by all layers, one set per (device, stream), grown outside stream capture to
  // the largest step seen and then reused; with AttentionMetadata::plan_info, layer 0 makes the copy's block table
  // and the step's schedule and later layers reuse both.
  // 0 disables the dense route.
  void set_prefill_dequant_rows(int64_t rows) { prefill_dequant_rows_ = rows; }

 private:
  void decoder_forward(const AttentionMetadata& attn_metadata,
                       torch::Tensor& query,
                       torch::Tensor& output,
                       const torch::Tensor& k_cache,
                       const torch::Tensor& v_cache,
                       const std::optional<torch::Tensor>& k_cache_scale,
                       const std::optional<torch::Tensor>& v_cache_scale);

  int64_t num_heads_;
  int64_t head_size_;
  float scale_;
  int64_t num_kv_heads_;
  int64_t sliding_window_;
  int64_t prefill_dequant_rows_ = 4096;
};

}  // namespace xllm::layer
