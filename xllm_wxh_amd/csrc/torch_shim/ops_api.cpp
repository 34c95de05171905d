#include "ops_api.h"

#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <utility>

#include "../../../include/xllm_hip_paged_kv.h"

namespace xllm::kernel {
namespace {

int32_t dtype_code(const torch::Tensor& t) {
  switch (t.scalar_type()) {
    case torch::kBFloat16:
      return XLLM_HIP_BF16;
    case torch::kHalf:
      return XLLM_HIP_FP16;
    case torch::kFloat:
      return XLLM_HIP_FP32;
    case torch::kFloat8_e4m3fn:
      return XLLM_HIP_FP8_E4M3;
    case torch::kChar:
      return XLLM_HIP_INT8;
    default:
      TORCH_CHECK(false, "unsupported dtype ", t.scalar_type());
  }
}

xllm_hip_stream_t current_stream(const torch::Tensor& t) {
  return (xllm_hip_stream_t)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void check_status(int status) {
  TORCH_CHECK(status == XLLM_HIP_OK, "xllm_hip status ", status, ": ", xllm_hip_last_error());
}

// Cache descriptor from [blocks, heads, slots, dim]-shaped tensors of any strides.
xllm_hip_kv_cache make_cache(const torch::Tensor& k,
                             const std::optional<torch::Tensor>& v,
                             const std::optional<torch::Tensor>& k_scale,
                             const std::optional<torch::Tensor>& v_scale) {
  TORCH_CHECK(k.defined() && k.dim() == 4, "k_cache must be [num_blocks, num_kv_heads, block_size, head_dim]");
  TORCH_CHECK(k.is_cuda(), "k_cache must live on the GPU");
  TORCH_CHECK(k.stride(3) == 1, "head_dim of k_cache must be contiguous");
  xllm_hip_kv_cache c{};
  c.k_cache = k.data_ptr();
  if (v.has_value() && v->defined()) {
    TORCH_CHECK(v->sizes() == k.sizes() && v->strides() == k.strides() && v->scalar_type() == k.scalar_type(),
                "v_cache must match k_cache in shape, strides and dtype");
    c.v_cache = v->data_ptr();
  }
  c.num_blocks = k.size(0);
  c.num_kv_heads = (int32_t)k.size(1);
  c.block_size = (int32_t)k.size(2);
  c.head_dim = (int32_t)k.size(3);
  c.dtype = dtype_code(k);
  c.stride_block = k.stride(0);
  c.stride_head = k.stride(1);
  c.stride_slot = k.stride(2);
  if (k_scale.has_value() && k_scale->defined()) {
    TORCH_CHECK(k_scale->scalar_type() == torch::kFloat && k_scale->dim() == 3 && k_scale->size(0) == k.size(0) &&
                    k_scale->size(1) == k.size(1) && k_scale->size(2) == k.size(2),
                "k_cache_scale must be float32 [num_blocks, num_kv_heads, block_size]");
    c.k_scale = k_scale->data_ptr<float>();
    c.scale_stride_block = k_scale->stride(0);
    c.scale_stride_head = k_scale->stride(1);
    c.scale_stride_slot = k_scale->stride(2);
    if (v_scale.has_value() && v_scale->defined()) {
      TORCH_CHECK(v_scale->sizes() == k_scale->sizes() && v_scale->strides() == k_scale->strides() &&
                      v_scale->scalar_type() == torch::kFloat,
                  "v_cache_scale must match k_cache_scale");
      c.v_scale = v_scale->data_ptr<float>();
    }
  }
  return c;
}

void check_write_inputs(const ReshapePagedCacheParams& p) {
  TORCH_CHECK(p.key.defined() && p.k_cache.defined() && p.slot_mapping.defined(),
              "key, k_cache and slot_mapping are required");
  TORCH_CHECK(!p.direction, "direction=true (cache to context) is not part of the decode path");
  TORCH_CHECK(p.key.dim() == 3, "key must be [num_tokens, num_kv_heads, head_dim]");
  // keys and values should be continuous at n_kv_heads and head_dim dims
  TORCH_CHECK(p.key.stride(-1) == 1 && p.key.stride(-2) == p.key.size(-1),
              "key must be contiguous in its last two dimensions");
  if (p.value.has_value()) {
    TORCH_CHECK(p.value->sizes() == p.key.sizes() && p.value->scalar_type() == p.key.scalar_type(),
                "value must match key");
    TORCH_CHECK(p.value->stride(-1) == 1 && p.value->stride(-2) == p.value->size(-1),
                "value must be contiguous in its last two dimensions");
    TORCH_CHECK(p.v_cache.has_value(), "value given without v_cache");
  } else {
    TORCH_CHECK(!p.v_cache.has_value(), "v_cache given without value");
  }
  TORCH_CHECK(p.slot_mapping.scalar_type() == torch::kInt && p.slot_mapping.dim() == 1 &&
                  p.slot_mapping.is_contiguous() && p.slot_mapping.numel() == p.key.size(0),
              "slot_mapping must be a contiguous int32 vector with one entry per token");
  TORCH_CHECK(p.key.size(1) == p.k_cache.size(1) && p.key.size(2) == p.k_cache.size(3),
              "key heads/head_dim do not match the cache");
}

}  // namespace

void reshape_paged_cache(ReshapePagedCacheParams& params) {
  check_write_inputs(params);
  const xllm_hip_kv_cache cache = make_cache(params.k_cache, params.v_cache, std::nullopt, std::nullopt);
  const bool has_v = params.value.has_value();
  check_status(xllm_hip_reshape_paged_cache(&cache, params.key.data_ptr(), has_v ? params.value->data_ptr() : nullptr,
                                            params.slot_mapping.data_ptr<int32_t>(), params.key.size(0),
                                            params.key.stride(0), has_v ? params.value->stride(0) : 0,
                                            dtype_code(params.key), current_stream(params.key)));
}

void quant_to_paged_cache(ReshapePagedCacheParams& params) {
  check_write_inputs(params);
  TORCH_CHECK(params.k_cache_scale.has_value(), "k_cache_scale is required for quant_to_paged_cache");
  const xllm_hip_kv_cache cache =
      make_cache(params.k_cache, params.v_cache, params.k_cache_scale, params.v_cache_scale);
  const bool has_v = params.value.has_value();
  check_status(xllm_hip_quant_to_paged_cache(&cache, params.key.data_ptr(), has_v ? params.value->data_ptr() : nullptr,
                                             params.slot_mapping.data_ptr<int32_t>(), params.key.size(0),
                                             params.key.stride(0), has_v ? params.value->stride(0) : 0,
                                             dtype_code(params.key), current_stream(params.key)));
}

namespace {

void gather_from_cache(ReshapeFromCacheParams& p, bool dequant) {
  TORCH_CHECK(p.key.defined() && p.key_cache.defined() && p.context_lengths.defined(),
              "key, key_cache and context_lengths are required");
  TORCH_CHECK(p.block_tables.has_value() && p.block_tables->defined() && p.block_tables->dim() == 2,
              "block_tables [batch, max_blocks] is required (the linear cache mode is not part of the paged path)");
  TORCH_CHECK(p.key.dim() == 3 && p.key.stride(-1) == 1 && p.key.stride(-2) == p.key.size(-1),
              "key must be [total_length, num_kv_heads, head_dim], contiguous in its last two dimensions");
  const bool has_v = p.value.has_value() && p.value->defined();
  if (has_v) {
    TORCH_CHECK(p.value_cache.has_value() && p.value_cache->defined(), "value given without value_cache");
    TORCH_CHECK(p.value->dim() == 3 && p.value->scalar_type() == p.key.scalar_type() &&
                    p.value->size(1) == p.key.size(1) && p.value->size(2) == p.key.size(2) &&
                    p.value->stride(-1) == 1 && p.value->stride(-2) == p.value->size(-1),
                "value must match key in dtype and row shape");
  }
  TORCH_CHECK(p.key.size(1) == p.key_cache.size(1) && p.key.size(2) == p.key_cache.size(3),
              "key heads/head_dim do not match the cache");
  auto i32 = [](const torch::Tensor& t) { return t.scalar_type() == torch::kInt && t.is_cuda(); };
  TORCH_CHECK(i32(p.context_lengths) && i32(*p.block_tables) && p.block_tables->stride(1) == 1,
              "context_lengths and block_tables must be int32 tensors on the GPU");
  const int64_t batch = p.context_lengths.numel();
  TORCH_CHECK(p.block_tables->size(0) >= batch, "one block_tables row per sequence");
  torch::Tensor lens = p.context_lengths.contiguous(), rows, starts;
  if (p.context_seq_offset.has_value() && p.context_seq_offset->defined()) {
    TORCH_CHECK(i32(*p.context_seq_offset) && p.context_seq_offset->numel() == batch, "bad context_seq_offset");
    rows = p.context_seq_offset->contiguous();
  }
  if (p.cache_seq_offset.has_value() && p.cache_seq_offset->defined()) {
    TORCH_CHECK(i32(*p.cache_seq_offset) && p.cache_seq_offset->numel() == batch, "bad cache_seq_offset");
    starts = p.cache_seq_offset->contiguous();
  }
  const std::optional<torch::Tensor> vc = has_v ? p.value_cache : std::nullopt;
  xllm_hip_kv_cache cache;
  if (!dequant) {
    TORCH_CHECK(p.key.scalar_type() == p.key_cache.scalar_type(),
                "reshape_from_cache copies verbatim: key and key_cache dtypes differ");
    cache = make_cache(p.key_cache, vc, std::nullopt, std::nullopt);
  } else {
    TORCH_CHECK(p.quant_bit == 8, "only 8-bit caches exist on this path");
    TORCH_CHECK(p.key_cache_quant_scale.has_value() && p.key_cache_quant_scale->defined(),
                "key_cache_quant_scale is required for dequant_from_paged_cache");
    TORCH_CHECK(p.key_cache.element_size() == 1 && p.key.element_size() > 1,
                "dequant_from_paged_cache reads a 1-byte cache into bf16/fp16/fp32 tensors");
    if (p.quant_mode == 1) {
      cache = make_cache(p.key_cache, vc, p.key_cache_quant_scale, has_v ? p.value_cache_quant_scale : std::nullopt);
      TORCH_CHECK(!has_v || cache.v_scale != nullptr, "value needs value_cache_quant_scale");
    } else {
      TORCH_CHECK(p.quant_mode == 0, "quant_mode must be 0 (per channel) or 1 (per token)");
      cache = make_cache(p.key_cache, vc, std::nullopt, std::nullopt);
      auto channel = [&](const std::optional<torch::Tensor>& s) {
        TORCH_CHECK(s.has_value() && s->defined() && s->scalar_type() == torch::kFloat && s->is_contiguous() &&
                        s->dim() == 2 && s->size(0) == cache.num_kv_heads && s->size(1) == cache.head_dim,
                    "per-channel scales must be contiguous float32 [num_kv_heads, head_dim]");
        return s->data_ptr<float>();
      };
      cache.k_scale = channel(p.key_cache_quant_scale);
      if (has_v) cache.v_scale = channel(p.value_cache_quant_scale);
    }
  }
  check_status(xllm_hip_gather_from_cache(
      &cache, p.key.data_ptr(), has_v ? p.value->data_ptr() : nullptr, dtype_code(p.key), p.key.stride(0),
      has_v ? p.value->stride(0) : 0, lens.data_ptr<int32_t>(), rows.defined() ? rows.data_ptr<int32_t>() : nullptr,
      starts.defined() ? starts.data_ptr<int32_t>() : nullptr, p.block_tables->data_ptr<int32_t>(),
      p.block_tables->stride(0), (int32_t)p.block_tables->size(1), (int32_t)batch, (int32_t)p.max_context_len,
      (int32_t)p.quant_mode, current_stream(p.key)));
}

}  // namespace

void reshape_from_cache(ReshapeFromCacheParams& params) { gather_from_cache(params, false); }

void dequant_from_paged_cache(ReshapeFromCacheParams& params) { gather_from_cache(params, true); }

namespace hip {

namespace {
std::mutex workspace_mu;
size_t workspace_capacity = 128u << 20;  // FLAGS_flashinfer_workspace_buffer_size's default
std::map<std::pair<int, void*>, torch::Tensor> workspaces;  // (device, stream) -> buffer
}  // namespace

void set_decode_workspace_bytes(size_t bytes) {
  std::lock_guard<std::mutex> lock(workspace_mu);
  workspace_capacity = bytes;
}

size_t decode_workspace_capacity() {
  std::lock_guard<std::mutex> lock(workspace_mu);
  return workspace_capacity;
}

torch::Tensor decode_workspace(const torch::Device& device, xllm_hip_stream_t stream) {
  std::lock_guard<std::mutex> lock(workspace_mu);
  torch::Tensor& ws = workspaces[{(int)device.index(), stream}];
  if (!ws.defined()) {
    ws = torch::empty({(int64_t)workspace_capacity}, torch::TensorOptions().dtype(torch::kUInt8).device(device));
  }
  return ws;
}

namespace {

// Pinned host buffers of the schedules made on the host, two per (device, stream) used in turn, each with the
// event recorded behind its last copy to the device.
struct HostStaging {
  torch::Tensor buffer[2];
  hipEvent_t event[2] = {nullptr, nullptr};
  int turn = 0;
};
HostStaging& host_staging(const torch::Device& device, xllm_hip_stream_t stream) {
  static std::mutex mu;
  static std::map<std::pair<int, xllm_hip_stream_t>, HostStaging> all;
  std::lock_guard<std::mutex> lock(mu);
  return all[{(int)device.index(), stream}];
}

// What a schedule depends on (FNV-1a over the fields): a later layer must present the same.
uint64_t plan_key(const xllm_hip_kv_cache& c, const xllm_hip_decode_args& a) {
  const uint64_t fields[] = {(uint64_t)a.batch,
                             (uint64_t)a.q_per_seq,
                             (uint64_t)a.num_q_heads,
                             (uint64_t)a.q_dtype,
                             (uint64_t)(uintptr_t)a.block_table,
                             (uint64_t)a.block_table_stride,
                             (uint64_t)a.max_blocks_per_seq,
                             (uint64_t)(uintptr_t)a.seq_lens,
                             (uint64_t)(uintptr_t)a.kv_indptr,
                             (uint64_t)(uintptr_t)a.kv_indices,
                             (uint64_t)(uintptr_t)a.kv_last_page_len,
                             (uint64_t)(uintptr_t)a.q_indptr,
                             (uint64_t)a.max_seq_len,
                             (uint64_t)a.total_kv_len,
                             (uint64_t)a.host_plan,
                             (uint64_t)c.dtype,
                             (uint64_t)c.num_kv_heads,
                             (uint64_t)c.head_dim,
                             (uint64_t)c.block_size,
                             (uint64_t)c.num_blocks,
                             // the layout decides the shape of the work items (kv heads side by side: four to an item)
                             (uint64_t)c.stride_block,
                             (uint64_t)c.stride_head,
                             (uint64_t)c.stride_slot,
                             (uint64_t)c.scale_stride_block,
                             (uint64_t)c.scale_stride_head,
                             (uint64_t)c.scale_stride_slot,
                             // the kernel family chosen (it also depends on alignments)
                             (uint64_t)(uintptr_t)xllm_hip_paged_decode_variant(&c, &a)};
  uint64_t h = 1469598103934665603ull;
  auto mix = [&](uint64_t f) {
    for (int i = 0; i < 8; ++i) {
      h ^= (f >> (8 * i)) & 0xff;
      h *= 1099511628211ull;
    }
  };
  // ... and so do the library's diagnostic switches: one toggled between two layers changes it under the schedule
  for (int32_t o = 0; o < XLLM_HIP_OPTION_COUNT; ++o) mix((uint64_t)xllm_hip_get_option(o));
  for (uint64_t f : fields) mix(f);
  return h;
}

void run_decode(const xllm_hip_kv_cache& cache, xllm_hip_decode_args& a, const torch::Tensor& q3, PlanInfo* plan) {
  const size_t need =
      xllm_hip_paged_decode_workspace_bytes(a.batch, a.q_per_seq, a.num_q_heads, cache.num_kv_heads, cache.head_dim);
  const xllm_hip_stream_t stream = current_stream(q3);
  torch::Tensor ws = decode_workspace(q3.device(), stream);
  // Never grown: a captured graph keeps the buffer's address, and a step under capture must not allocate.
  TORCH_CHECK(need <= (size_t)ws.numel(), "this decode step needs ", need, " bytes of workspace; the buffer of this ",
              "stream holds ", ws.numel(), " (raise it with set_decode_workspace_bytes before the first decode call ",
              "on a stream)");
  if (plan == nullptr) {
    check_status(xllm_hip_paged_decode(&cache, &a, ws.data_ptr(), (size_t)ws.numel(), stream));
    return;
  }
  TORCH_CHECK(plan->layer_id != -1, "Need to set layer_id to PlanInfo.");
  a.host_plan = plan->host_plan || !plan->kv_lens_host.empty() ? 1 : 0;
  const uint64_t key = plan_key(cache, a);
  if (plan->layer_id == 0) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    (void)hipStreamIsCapturing((hipStream_t)stream, &capturing);
    if (!plan->kv_lens_host.empty() && capturing == hipStreamCaptureStatusNone) {
      TORCH_CHECK((int64_t)plan->kv_lens_host.size() == a.batch, "kv_lens_host has ", plan->kv_lens_host.size(),
                  " entries, the step has ", a.batch, " sequences");
      HostStaging& st = host_staging(q3.device(), stream);
      const size_t bytes = xllm_hip_paged_decode_plan_host_bytes(a.batch, a.q_per_seq, a.num_q_heads, cache.num_kv_heads,
                                                                 cache.head_dim);
      const int turn = st.turn;
      st.turn = 1 - turn;
      if (!st.buffer[turn].defined() || (size_t)st.buffer[turn].numel() < bytes) {
        st.buffer[turn] = torch::empty({(int64_t)std::max<size_t>(bytes, 1 << 16)},
                                       torch::TensorOptions().dtype(torch::kUInt8).pinned_memory(true));
        if (st.event[turn] == nullptr) TORCH_CHECK(hipEventCreateWithFlags(&st.event[turn], hipEventDisableTiming) == hipSuccess);
      } else {
        TORCH_CHECK(hipEventSynchronize(st.event[turn]) == hipSuccess);  // its last copy to the device has run
      }
      check_status(xllm_hip_paged_decode_plan_host(&cache, &a, plan->kv_lens_host.data(), ws.data_ptr(), (size_t)ws.numel(),
                                                   st.buffer[turn].data_ptr(), (size_t)st.buffer[turn].numel(), stream,
                                                   nullptr));
      TORCH_CHECK(hipEventRecord(st.event[turn], (hipStream_t)stream) == hipSuccess);
    } else {
      check_status(xllm_hip_paged_decode_plan(&cache, &a, ws.data_ptr(), (size_t)ws.numel(), stream));
    }
    plan->workspace = ws.data_ptr();
    plan->key = key;
  } else {
    TORCH_CHECK(plan->workspace == ws.data_ptr() && plan->key == key,
                "layer ", plan->layer_id, " presents other lengths, block lists, sizes or another stream than the ",
                "ones the step's schedule was built for at layer 0");
  }
  check_status(xllm_hip_paged_decode_run(&cache, &a, ws.data_ptr(), (size_t)ws.numel(), stream));
}

void fill_q_out(xllm_hip_decode_args& a, const torch::Tensor& q3, torch::Tensor& o3, int64_t q_per_seq) {
  TORCH_CHECK(q3.dim() == 3 && o3.dim() == 3 && o3.sizes() == q3.sizes() && o3.scalar_type() == q3.scalar_type(),
              "output must match query [tokens, heads, head_dim]");
  TORCH_CHECK(q3.stride(2) == 1 && q3.stride(1) == q3.size(2) && o3.stride(2) == 1 && o3.stride(1) == o3.size(2),
              "query/output heads and head_dim must be contiguous");
  TORCH_CHECK(q_per_seq >= 1 && q3.size(0) % q_per_seq == 0, "query tokens not divisible by q_len");
  a.q = q3.data_ptr();
  a.out = o3.data_ptr();
  a.q_token_stride = q3.stride(0);
  a.out_token_stride = o3.stride(0);
  a.q_dtype = dtype_code(q3);
  a.batch = (int32_t)(q3.size(0) / q_per_seq);
  a.q_per_seq = (int32_t)q_per_seq;
  a.num_q_heads = (int32_t)q3.size(1);
}

}  // namespace

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
                  const std::string& /*compute_dtype*/,
                  int64_t max_seq_len,
                  int64_t window_size_left,
                  int64_t window_size_right,
                  float scale,
                  bool return_lse,
                  int64_t kv_cache_quant_bit_size,
                  int64_t total_kv_len,
                  PlanInfo* plan_info) {
  TORCH_CHECK(v_cache.has_value(), "v_cache is required (single-cache MLA decode is outside this path)");
  TORCH_CHECK(!q_quant_scale.has_value() && !out_quant_scale.has_value() && !alibi_slope.has_value() &&
                  !mask.has_value(),
              "q/out quantisation, alibi and custom masks are not supported by the HIP decode path");
  TORCH_CHECK(window_size_right < 0, "window_size_right must be -1 for decode");
  const bool quant = k_cache_quant_scale.has_value();
  TORCH_CHECK(kv_cache_quant_bit_size == -1 || (kv_cache_quant_bit_size == 8 && quant),
              "kv_cache_quant_bit_size must be -1, or 8 together with k/v_cache_quant_scale");
  TORCH_CHECK(!quant || v_cache_quant_scale.has_value(), "v_cache_quant_scale is required with k_cache_quant_scale");
  TORCH_CHECK(query.dim() == 4 && output.dim() == 4, "query/output must be [batch, q_len, heads, head_dim]");
  const xllm_hip_kv_cache cache = make_cache(k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale);

  torch::Tensor q3 = query.view({-1, query.size(2), query.size(3)});
  torch::Tensor o3 = output.view({-1, output.size(2), output.size(3)});
  xllm_hip_decode_args a{};
  fill_q_out(a, q3, o3, query.size(1));
  TORCH_CHECK(q3.size(2) == cache.head_dim, "query head_dim does not match the cache");
  a.sm_scale = scale;
  a.window_left = (int32_t)window_size_left;
  TORCH_CHECK(block_table.scalar_type() == torch::kInt && block_table.dim() == 2 && block_table.stride(1) == 1 &&
                  block_table.size(0) == a.batch,
              "block_table must be int32 [batch, max_blocks]");
  TORCH_CHECK(seq_lens.scalar_type() == torch::kInt && seq_lens.is_contiguous() && seq_lens.numel() == a.batch,
              "seq_lens must be contiguous int32 [batch]");
  a.block_table = block_table.data_ptr<int32_t>();
  // (the row stride of a one-row table is arbitrary in torch: such a table is its one row)
  a.block_table_stride = block_table.size(0) > 1 ? block_table.stride(0) : block_table.size(1);
  a.max_blocks_per_seq = (int32_t)block_table.size(1);
  a.seq_lens = seq_lens.data_ptr<int32_t>();
  a.max_seq_len = (int32_t)max_seq_len;
  a.total_kv_len = total_kv_len;
  if (return_lse) {
    TORCH_CHECK(output_lse.has_value(), "return_lse needs a pre-allocated output_lse");
  }
  if (output_lse.has_value() && output_lse->defined()) {
    TORCH_CHECK(output_lse->scalar_type() == torch::kFloat && output_lse->is_contiguous() &&
                    output_lse->numel() == q3.size(0) * q3.size(1),
                "output_lse must be contiguous float32 [tokens, heads]");
    a.lse = output_lse->data_ptr<float>();
  }
  run_decode(cache, a, q3, plan_info);
}

void batch_prefill_paged(const torch::Tensor& query, const torch::Tensor& k_cache, const torch::Tensor& v_cache,
                         torch::Tensor& output, std::optional<torch::Tensor>& output_lse,
                         const torch::Tensor& q_cu_seq_lens, const torch::Tensor& kv_seq_lens,
                         const std::optional<torch::Tensor>& k_cache_quant_scale,
                         const std::optional<torch::Tensor>& v_cache_quant_scale, const torch::Tensor& block_tables,
                         int64_t max_query_len, int64_t max_seq_len, float scale, int64_t window_size_left,
                         bool return_lse, int64_t total_kv_len, PlanInfo* plan_info) {
  TORCH_CHECK(query.dim() == 3 && output.dim() == 3, "query/output must be [tokens, heads, head_dim]");
  TORCH_CHECK(max_query_len >= 1, "max_query_len must be at least 1");
  const bool quant = k_cache_quant_scale.has_value();
  TORCH_CHECK(!quant || v_cache_quant_scale.has_value(), "v_cache_quant_scale is required with k_cache_quant_scale");
  const xllm_hip_kv_cache cache = make_cache(k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale);
  xllm_hip_decode_args a{};
  torch::Tensor o3 = output;
  fill_q_out(a, query, o3, 1);
  TORCH_CHECK(query.size(2) == cache.head_dim, "query head_dim does not match the cache");
  TORCH_CHECK(q_cu_seq_lens.scalar_type() == torch::kInt && q_cu_seq_lens.is_contiguous() &&
                  q_cu_seq_lens.numel() >= 1,
              "q_cu_seq_lens must be contiguous int32 [batch + 1]");
  a.batch = (int32_t)(q_cu_seq_lens.numel() - 1);
  a.q_per_seq = (int32_t)max_query_len;
  a.q_indptr = q_cu_seq_lens.data_ptr<int32_t>();
  a.sm_scale = scale;
  a.window_left = (int32_t)window_size_left;
  TORCH_CHECK(block_tables.scalar_type() == torch::kInt && block_tables.dim() == 2 && block_tables.stride(1) == 1 &&
                  block_tables.size(0) == a.batch,
              "block_tables must be int32 [batch, max_blocks]");
  TORCH_CHECK(kv_seq_lens.scalar_type() == torch::kInt && kv_seq_lens.is_contiguous() && kv_seq_lens.numel() == a.batch,
              "kv_seq_lens must be contiguous int32 [batch]");
  a.block_table = block_tables.data_ptr<int32_t>();
  a.block_table_stride = block_tables.size(0) > 1 ? block_tables.stride(0) : block_tables.size(1);
  a.max_blocks_per_seq = (int32_t)block_tables.size(1);
  a.seq_lens = kv_seq_lens.data_ptr<int32_t>();
  a.max_seq_len = (int32_t)max_seq_len;
  a.total_kv_len = total_kv_len;
  if (return_lse) {
    TORCH_CHECK(output_lse.has_value(), "return_lse needs a pre-allocated output_lse");
  }
  if (output_lse.has_value() && output_lse->defined()) {
    TORCH_CHECK(output_lse->scalar_type() == torch::kFloat && output_lse->is_contiguous() &&
                    output_lse->numel() == query.size(0) * query.size(1),
                "output_lse must be contiguous float32 [tokens, heads]");
    a.lse = output_lse->data_ptr<float>();
  }
  run_decode(cache, a, query, plan_info);
}

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
                      PlanInfo* plan_info,
                      const std::optional<torch::Tensor>& k_cache_scale,
                      const std::optional<torch::Tensor>& v_cache_scale) {
  TORCH_CHECK(k_cache_scale.has_value() == v_cache_scale.has_value(), "k_cache_scale and v_cache_scale come together");
  // NHD [blocks, block_size, Hkv, D] -> logical [blocks, Hkv, block_size, D] view (scales likewise)
  std::optional<torch::Tensor> ks, vs;
  if (k_cache_scale.has_value()) {
    ks = k_cache_scale->permute({0, 2, 1});
    vs = v_cache_scale->permute({0, 2, 1});
  }
  const xllm_hip_kv_cache cache = make_cache(k_cache.permute({0, 2, 1, 3}), v_cache.permute({0, 2, 1, 3}), ks, vs);
  xllm_hip_decode_args a{};
  fill_q_out(a, query, output, 1);
  a.sm_scale = (float)sm_scale;
  a.window_left = (int32_t)window_left;
  for (const torch::Tensor* t : {&paged_kv_indptr, &paged_kv_indices, &paged_kv_last_page_len}) {
    TORCH_CHECK(t->scalar_type() == torch::kInt && t->is_contiguous(), "CSR arrays must be contiguous int32");
  }
  TORCH_CHECK(paged_kv_indptr.numel() == a.batch + 1 && paged_kv_last_page_len.numel() == a.batch,
              "CSR arrays do not match the batch");
  a.kv_indptr = paged_kv_indptr.data_ptr<int32_t>();
  a.kv_indices = paged_kv_indices.data_ptr<int32_t>();
  a.kv_last_page_len = paged_kv_last_page_len.data_ptr<int32_t>();
  if (output_lse.has_value() && output_lse->defined()) a.lse = output_lse->data_ptr<float>();
  run_decode(cache, a, query, plan_info);
}

namespace {

void rope_call(torch::Tensor& qkv, int64_t hq, int64_t hk, int64_t hv, int64_t head_dim, double eps,
               const std::optional<torch::Tensor>& q_weight, const std::optional<torch::Tensor>& k_weight,
               const torch::Tensor& cos_sin_cache, bool interleaved, bool round_each_op,
               const torch::Tensor& position_ids, const xllm_hip_kv_cache* cache, const torch::Tensor* slot_mapping) {
  TORCH_CHECK(qkv.is_cuda() && qkv.dim() == 2 && qkv.stride(1) == 1, "qkv must be a 2-D GPU tensor, rows contiguous");
  TORCH_CHECK((position_ids.scalar_type() == torch::kLong || position_ids.scalar_type() == torch::kInt) &&
                  position_ids.dim() == 1 && position_ids.is_contiguous() && position_ids.numel() == qkv.size(0),
              "position_ids must be contiguous int64 or int32 [num_tokens]");
  TORCH_CHECK(cos_sin_cache.dim() == 2 && cos_sin_cache.is_contiguous(),
              "cos_sin_cache must be contiguous [max_position, rotary_dim]");
  xllm_hip_rope_args a{};
  a.qkv = qkv.data_ptr();
  a.token_stride = qkv.stride(0);
  a.num_tokens = qkv.size(0);
  a.dtype = dtype_code(qkv);
  a.num_q_heads = (int32_t)hq;
  a.num_k_heads = (int32_t)hk;
  a.num_v_heads = (int32_t)hv;
  a.head_dim = (int32_t)head_dim;
  a.rotary_dim = (int32_t)cos_sin_cache.size(1);
  if (q_weight.has_value() && q_weight->defined()) {
    TORCH_CHECK(k_weight.has_value() && k_weight->defined(), "q_weight and k_weight go together");
    for (const torch::Tensor* w : {&*q_weight, &*k_weight}) {
      TORCH_CHECK(w->scalar_type() == qkv.scalar_type() && w->dim() == 1 && w->numel() == head_dim &&
                      w->is_contiguous(),
                  "norm weights must be [head_dim] of qkv's dtype");
    }
    a.q_weight = q_weight->data_ptr();
    a.k_weight = k_weight->data_ptr();
  }
  a.eps = (float)eps;
  a.cos_sin_dtype = dtype_code(cos_sin_cache);
  a.cos_sin_cache = cos_sin_cache.data_ptr();
  a.max_position = cos_sin_cache.size(0);
  a.positions = position_ids.data_ptr();
  a.positions_int32 = position_ids.scalar_type() == torch::kInt ? 1 : 0;
  a.interleave = interleaved ? 1 : 0;
  a.round_each_op = round_each_op ? 1 : 0;
  const int32_t* slots = nullptr;
  if (cache != nullptr) {
    TORCH_CHECK(slot_mapping->scalar_type() == torch::kInt && slot_mapping->is_contiguous() &&
                    slot_mapping->numel() == qkv.size(0),
                "slot_mapping must be contiguous int32 [num_tokens]");
    slots = slot_mapping->data_ptr<int32_t>();
  }
  check_status(xllm_hip_rope_kv_write(&a, cache, slots, current_stream(qkv)));
}

}  // namespace

void fused_qk_norm_rope(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_k, int64_t num_heads_v,
                        int64_t head_dim, double eps, const torch::Tensor& q_weight, const torch::Tensor& k_weight,
                        const torch::Tensor& cos_sin_cache, bool interleaved, const torch::Tensor& position_ids) {
  rope_call(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved,
            false, position_ids, nullptr, nullptr);
}

void rotary_embedding(torch::Tensor& positions, torch::Tensor& query, std::optional<torch::Tensor> key,
                      torch::Tensor& cos_sin_cache, bool is_neox) {
  const int64_t head_size = cos_sin_cache.size(-1);  // as the reference derives it (rope.cu:169)
  auto one = [&](torch::Tensor t) {
    torch::Tensor flat = t.dim() == 3 ? t.view({t.size(0), -1}) : t;
    TORCH_CHECK(flat.size(1) % head_size == 0, "hidden size is not a multiple of head_size");
    rope_call(flat, flat.size(1) / head_size, 0, 0, head_size, 0.0, std::nullopt, std::nullopt, cos_sin_cache,
              !is_neox, true, positions, nullptr, nullptr);
  };
  one(query);
  if (key.has_value() && key->defined()) one(*key);
}

void rope_kv_write(torch::Tensor& qkv, int64_t num_heads_q, int64_t num_heads_kv, int64_t head_dim,
                   const std::optional<torch::Tensor>& q_weight, const std::optional<torch::Tensor>& k_weight, double eps,
                   const torch::Tensor& cos_sin_cache, bool interleaved, bool round_each_op,
                   const torch::Tensor& position_ids, const torch::Tensor& k_cache, const torch::Tensor& v_cache,
                   const std::optional<torch::Tensor>& k_cache_scale, const std::optional<torch::Tensor>& v_cache_scale,
                   const torch::Tensor& slot_mapping) {
  xllm_hip_kv_cache cache = make_cache(k_cache, v_cache, k_cache_scale, v_cache_scale);
  rope_call(qkv, num_heads_q, num_heads_kv, num_heads_kv, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved,
            round_each_op, position_ids, &cache, &slot_mapping);
}

void swap_blocks(const torch::Tensor& k_cache,
                 const torch::Tensor& v_cache,
                 const std::optional<torch::Tensor>& k_cache_scale,
                 const std::optional<torch::Tensor>& v_cache_scale,
                 const torch::Tensor& src,
                 const torch::Tensor& dst) {
  TORCH_CHECK(src.defined() && dst.defined() && src.scalar_type() == torch::kLong &&
                  dst.scalar_type() == torch::kLong && src.is_cuda() && dst.is_cuda(),
              "swap_blocks takes int64 index tensors on the GPU");
  TORCH_CHECK(src.numel() == dst.numel(), "src and dst must name the same number of blocks");
  const int64_t n = src.numel();
  if (n == 0) return;
  xllm_hip_kv_cache cache = make_cache(k_cache, v_cache, k_cache_scale, v_cache_scale);
  const torch::Tensor s = src.contiguous(), d = dst.contiguous();
  const size_t bytes = xllm_hip_swap_blocks_staging_bytes(&cache, n);
  torch::Tensor staging =
      torch::empty({(int64_t)bytes}, torch::TensorOptions().dtype(torch::kUInt8).device(k_cache.device()));
  check_status(xllm_hip_swap_blocks(&cache, s.data_ptr<int64_t>(), d.data_ptr<int64_t>(), n, staging.data_ptr(), bytes,
                                    current_stream(k_cache)));
}

void copy_blocks(const torch::Tensor& k_cache,
                 const torch::Tensor& v_cache,
                 const std::optional<torch::Tensor>& k_cache_scale,
                 const std::optional<torch::Tensor>& v_cache_scale,
                 const torch::Tensor& src_block_indices,
                 const torch::Tensor& dst_block_indices,
                 const torch::Tensor& cum_sum) {
  for (const torch::Tensor* t : {&src_block_indices, &dst_block_indices, &cum_sum}) {
    TORCH_CHECK(t->defined() && t->scalar_type() == torch::kInt && t->is_cuda(),
                "copy_blocks takes int32 index tensors on the GPU");
  }
  TORCH_CHECK(src_block_indices.numel() == cum_sum.numel(), "one cum_sum entry per source block");
  if (src_block_indices.numel() == 0 || dst_block_indices.numel() == 0) return;
  xllm_hip_kv_cache cache = make_cache(k_cache, v_cache, k_cache_scale, v_cache_scale);
  const torch::Tensor s = src_block_indices.contiguous(), d = dst_block_indices.contiguous(), c = cum_sum.contiguous();
  check_status(xllm_hip_copy_blocks(&cache, s.data_ptr<int32_t>(), d.data_ptr<int32_t>(), c.data_ptr<int32_t>(),
                                    (int32_t)s.numel(), (int32_t)d.numel(), current_stream(k_cache)));
}

}  // namespace hip
}  // namespace xllm::kernel
