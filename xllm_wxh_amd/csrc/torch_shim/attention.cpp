#include "attention.h"

#include "ops_api.h"

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <map>
#include <mutex>
#include <tuple>

namespace xllm::layer {

namespace {

// The dense 16-bit copy of a step's cached K/V ranges (decoder_forward's route for very many query rows over a
// 1-byte cache) and the block table over it.  One per (device, stream, element type), kept for the life of the
// process and only ever grown — outside stream capture: a captured graph holds the addresses.
struct DenseCopy {
  torch::Tensor k, v;        // flat, in the queries' type
  torch::Tensor table;       // [batch, blocks of the longest sequence]: consecutive blocks of the copy
  torch::Tensor row_offset;  // [batch]: first row of each sequence in the copy
};

DenseCopy& dense_copy(const torch::Device& device, const torch::TensorOptions& options, int64_t elements) {
  static std::mutex mu;
  static std::map<std::tuple<int, int64_t, int>, DenseCopy> copies;
  const auto stream = c10::hip::getCurrentHIPStream(device.index());
  std::lock_guard<std::mutex> lock(mu);
  DenseCopy& dc = copies[std::make_tuple((int)device.index(), (int64_t)stream.id(), (int)c10::typeMetaToScalarType(options.dtype()))];
  if (!dc.k.defined() || dc.k.numel() < elements) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing(stream.stream(), &capturing);
    TORCH_CHECK(capturing == hipStreamCaptureStatusNone,
                "the dense copy of the cached K/V must grow to ", elements, " elements: run the largest step of the "
                "bucket once on this stream before capturing it");
    // (a quarter more than asked for: steps of a serving loop grow token by token)
    const int64_t n = elements + elements / 4;
    dc.k = torch::Tensor();
    dc.v = torch::Tensor();
    dc.k = torch::empty({n}, options);
    dc.v = torch::empty({n}, options);
  }
  return dc;
}

}  // namespace

AttentionImpl::AttentionImpl(int64_t num_heads, int64_t head_size, float scale, int64_t num_kv_heads,
                             int64_t sliding_window)
    : num_heads_(num_heads), head_size_(head_size), scale_(scale), num_kv_heads_(num_kv_heads),
      // window_left = sliding_window - 1; -1 disables it (xllm/core/layers/mlu/attention.cpp:60-63)
      sliding_window_(sliding_window > -1 ? sliding_window - 1 : sliding_window) {}

std::tuple<torch::Tensor, std::optional<torch::Tensor>> AttentionImpl::forward(
    const AttentionMetadata& attn_metadata, torch::Tensor& query, torch::Tensor& key, torch::Tensor& value,
    KVCache& kv_cache) {
  std::optional<torch::Tensor> output_lse = std::nullopt;
  torch::Tensor output = torch::empty_like(query);
  // dummy batches and empty steps return the untouched buffer
  // (xllm/core/layers/mlu/attention.cpp:80-82, xllm/core/layers/cuda/flashinfer_attention.cpp:120-123)
  if (attn_metadata.is_dummy || attn_metadata.max_seq_len == 0) {
    return {output.view({-1, num_heads_ * head_size_}), output_lse};
  }
  torch::Tensor k_cache = kv_cache.get_k_cache();
  torch::Tensor v_cache = kv_cache.get_v_cache();
  std::optional<torch::Tensor> k_cache_scale = kv_cache.get_k_cache_scale();
  std::optional<torch::Tensor> v_cache_scale = kv_cache.get_v_cache_scale();

  // 1. KV write of the step's new tokens (write, then attend).
  xllm::kernel::ReshapePagedCacheParams write;
  write.key = key.view({-1, num_kv_heads_, head_size_});
  write.value = value.view({-1, num_kv_heads_, head_size_});
  write.k_cache = k_cache;
  write.v_cache = v_cache;
  write.slot_mapping = attn_metadata.slot_mapping;
  if (k_cache_scale.has_value()) {
    write.k_cache_scale = k_cache_scale;
    write.v_cache_scale = v_cache_scale;
    xllm::kernel::quant_to_paged_cache(write);
  } else {
    xllm::kernel::reshape_paged_cache(write);
  }

  // 2. Decode.
  decoder_forward(attn_metadata, query, output, k_cache, v_cache, k_cache_scale, v_cache_scale);
  return {output.view({-1, num_heads_ * head_size_}), output_lse};
}

std::tuple<torch::Tensor, std::optional<torch::Tensor>> AttentionImpl::forward_qkv(
    const AttentionMetadata& attn_metadata, const torch::Tensor& positions, torch::Tensor& qkv,
    const torch::Tensor& cos_sin_cache, bool interleaved, const std::optional<torch::Tensor>& q_norm_weight,
    const std::optional<torch::Tensor>& k_norm_weight, double eps, KVCache& kv_cache) {
  std::optional<torch::Tensor> output_lse = std::nullopt;
  const int64_t q_size = num_heads_ * head_size_;
  torch::Tensor output = torch::empty({qkv.size(0), q_size}, qkv.options());
  if (attn_metadata.is_dummy || attn_metadata.max_seq_len == 0) {
    return {output, output_lse};
  }
  TORCH_CHECK(qkv.dim() == 2 && qkv.size(1) == (num_heads_ + 2 * num_kv_heads_) * head_size_,
              "qkv must be [tokens, (num_heads + 2 * num_kv_heads) * head_size]");
  torch::Tensor k_cache = kv_cache.get_k_cache();
  torch::Tensor v_cache = kv_cache.get_v_cache();
  std::optional<torch::Tensor> k_cache_scale = kv_cache.get_k_cache_scale();
  std::optional<torch::Tensor> v_cache_scale = kv_cache.get_v_cache_scale();
  // the fused CUDA kernel serves 1-D positions with the norm weights; without them the reference
  // rotates with rope.cu, whose arithmetic rounds every operation
  const bool with_norm = q_norm_weight.has_value() && q_norm_weight->defined();
  // int32 positions (what the reference's modules pass) and int64 ones are both read as they are
  torch::Tensor pos = positions.scalar_type() == torch::kInt || positions.scalar_type() == torch::kLong
                          ? positions.contiguous()
                          : positions.to(torch::kLong).contiguous();
  xllm::kernel::hip::rope_kv_write(qkv, num_heads_, num_kv_heads_, head_size_, q_norm_weight, k_norm_weight, eps,
                                   cos_sin_cache, interleaved, /*round_each_op=*/!with_norm, pos, k_cache, v_cache,
                                   k_cache_scale, v_cache_scale, attn_metadata.slot_mapping);
  torch::Tensor query = qkv.slice(/*dim=*/-1, 0, q_size);
  decoder_forward(attn_metadata, query, output, k_cache, v_cache, k_cache_scale, v_cache_scale);
  return {output, output_lse};
}

void AttentionImpl::decoder_forward(const AttentionMetadata& attn_metadata, torch::Tensor& query,
                                    torch::Tensor& output, const torch::Tensor& k_cache,
                                    const torch::Tensor& v_cache, const std::optional<torch::Tensor>& k_cache_scale,
                                    const std::optional<torch::Tensor>& v_cache_scale) {
  std::optional<torch::Tensor> output_lse = std::nullopt;
  if (attn_metadata.is_prefill || attn_metadata.is_chunked_prefill) {
    // Prefill chunks and mixed steps: the step's K/V are in the cache already (write, then attend), so
    // every sequence attends its cached range with its own number of query tokens
    // (xllm/core/layers/mlu/attention.cpp:179-250, xllm/core/layers/cuda/flashinfer_attention.cpp:224-284).
    TORCH_CHECK(attn_metadata.block_table.defined() && attn_metadata.kv_seq_lens.defined() &&
                    attn_metadata.q_cu_seq_lens.defined(),
                "prefill over the paged cache needs block_table, kv_seq_lens and q_cu_seq_lens");
    torch::Tensor q3 = query.view({-1, num_heads_, head_size_});
    torch::Tensor o3 = output.view({-1, num_heads_, head_size_});
    const int64_t batch = attn_metadata.block_table.size(0);
    const int64_t rows_avg = batch > 0 ? q3.size(0) * (num_heads_ / num_kv_heads_) / batch : 0;
    if (k_cache_scale.has_value() && prefill_dequant_rows_ > 0 && rows_avg >= prefill_dequant_rows_ &&
        attn_metadata.total_kv_len > 0) {
      // Very many query rows per kv head over a 1-byte cache.  Attended in place, every 128 rows stream
      // and convert a sequence's K/V again; instead the cached ranges are dequantised once into a dense
      // copy in the queries' type (sequence b at a block-aligned row offset, found on the device: no
      // length is read back) and the 16-bit many-row kernel runs over that copy through a block table
      // of consecutive blocks.
      const int64_t bs = k_cache.size(2);
      const int64_t total_blocks = (attn_metadata.total_kv_len + batch * (bs - 1)) / bs + 1;
      // The copy and its block table live in buffers that every layer of the process shares, one set per
      // (device, stream), grown to the largest step seen and then reused: layer after layer on a stream consumes
      // its copy before the next one overwrites it.  The table and the rows' offsets depend on the lengths alone:
      // layer 0 of a step makes them (plan_info.layer_id; every call if the metadata carries no plan_info).
      PlanInfo* plan_info = attn_metadata.plan_info.get();
      DenseCopy& dc = dense_copy(query.device(), query.options(), total_blocks * bs * num_kv_heads_ * head_size_);
      if (plan_info == nullptr || plan_info->layer_id == 0 || !dc.table.defined()) {
        const auto i32 = torch::TensorOptions().dtype(torch::kInt32).device(query.device());
        torch::Tensor blocks_per_seq = torch::div(attn_metadata.kv_seq_lens + (bs - 1), bs, "floor").to(torch::kInt32);
        torch::Tensor first_block = (torch::cumsum(blocks_per_seq, 0) - blocks_per_seq).to(torch::kInt32);
        const int64_t max_blocks = (attn_metadata.max_seq_len + bs - 1) / bs;
        dc.table = torch::clamp_max(first_block.unsqueeze(1) + torch::arange(max_blocks, i32).unsqueeze(0), total_blocks - 1)
                       .to(torch::kInt32)
                       .contiguous();
        dc.row_offset = (first_block * bs).to(torch::kInt32);
      }
      TORCH_CHECK(dc.table.size(0) == batch, "the dense copy's block table was made for another batch: layer 0 of the step must come first");
      torch::Tensor dk = dc.k.narrow(0, 0, total_blocks * bs * num_kv_heads_ * head_size_).view({total_blocks, bs, num_kv_heads_, head_size_});
      torch::Tensor dv = dc.v.narrow(0, 0, total_blocks * bs * num_kv_heads_ * head_size_).view({total_blocks, bs, num_kv_heads_, head_size_});
      xllm::kernel::ReshapeFromCacheParams g;
      g.key = dk.view({-1, num_kv_heads_, head_size_});
      g.value = dv.view({-1, num_kv_heads_, head_size_});
      g.key_cache = k_cache;
      g.value_cache = v_cache;
      g.context_lengths = attn_metadata.kv_seq_lens;
      g.max_context_len = attn_metadata.max_seq_len;
      g.context_seq_offset = dc.row_offset;
      g.block_tables = attn_metadata.block_table;
      g.key_cache_quant_scale = k_cache_scale;
      g.value_cache_quant_scale = v_cache_scale;
      xllm::kernel::dequant_from_paged_cache(g);
      // the dense copy is token-major ([blocks, slots, heads, dim]); the kernels take its HND view
      xllm::kernel::hip::batch_prefill_paged(q3, dk.permute({0, 2, 1, 3}), dv.permute({0, 2, 1, 3}), o3, output_lse,
                                             attn_metadata.q_cu_seq_lens, attn_metadata.kv_seq_lens, std::nullopt,
                                             std::nullopt, dc.table, attn_metadata.max_query_len,
                                             attn_metadata.max_seq_len, scale_, sliding_window_, false,
                                             attn_metadata.total_kv_len, plan_info);
      return;
    }
    xllm::kernel::hip::batch_prefill_paged(q3, k_cache, v_cache, o3, output_lse, attn_metadata.q_cu_seq_lens,
                                           attn_metadata.kv_seq_lens, k_cache_scale, v_cache_scale,
                                           attn_metadata.block_table, attn_metadata.max_query_len,
                                           attn_metadata.max_seq_len, scale_, sliding_window_, false,
                                           attn_metadata.total_kv_len, attn_metadata.plan_info.get());
    return;
  }
  // One decode row per query token by default (speculative verify arrives expanded into rows,
  // xllm/core/runtime/speculative_worker_impl.cpp:230-243); a batch whose sequences all carry
  // max_query_len > 1 tokens against one block-table row each is the multi-token form.
  int64_t q_len = 1;
  if (attn_metadata.max_query_len > 1 && attn_metadata.block_table.defined() &&
      attn_metadata.block_table.size(0) * attn_metadata.max_query_len == query.size(0)) {
    q_len = attn_metadata.max_query_len;
  }
  torch::Tensor q4 = query.view({-1, q_len, num_heads_, head_size_});
  torch::Tensor o4 = output.view({-1, q_len, num_heads_, head_size_});
  if (attn_metadata.block_table.defined() && attn_metadata.kv_seq_lens.defined()) {
    xllm::kernel::hip::batch_decode(q4, k_cache, o4, attn_metadata.block_table, attn_metadata.kv_seq_lens, v_cache,
                                    output_lse, std::nullopt, k_cache_scale, v_cache_scale, std::nullopt,
                                    std::nullopt, std::nullopt, "float", attn_metadata.max_seq_len, sliding_window_,
                                    -1, scale_, false, k_cache_scale.has_value() ? 8 : -1,
                                    attn_metadata.total_kv_len, attn_metadata.plan_info.get());
  } else {
    TORCH_CHECK(attn_metadata.paged_kv_indptr.defined(), "neither block_table nor the CSR arrays are set");
    torch::Tensor q3 = query.view({-1, num_heads_, head_size_});
    torch::Tensor o3 = output.view({-1, num_heads_, head_size_});
    // the CSR entry point takes the CUDA backend's NHD shape: hand it the NHD view of our HND cache (and scales)
    std::optional<torch::Tensor> ks, vs;
    if (k_cache_scale.has_value()) {
      ks = k_cache_scale->permute({0, 2, 1});
      vs = v_cache_scale->permute({0, 2, 1});
    }
    xllm::kernel::hip::batch_decode_csr(q3, k_cache.permute({0, 2, 1, 3}), v_cache.permute({0, 2, 1, 3}),
                                        attn_metadata.paged_kv_indptr, attn_metadata.paged_kv_indices,
                                        attn_metadata.paged_kv_last_page_len, sliding_window_, scale_, o3, output_lse,
                                        attn_metadata.plan_info.get(), ks, vs);
  }
}

}  // namespace xllm::layer
