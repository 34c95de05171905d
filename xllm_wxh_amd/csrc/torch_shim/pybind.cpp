// Python binding of the libtorch host side, so that pytest can drive the C++ operators and the
// AttentionImpl twin on the GPU box.
#include <pybind11/stl.h>
#include <torch/extension.h>

#include "attention.h"
#include "ops_api.h"

namespace py = pybind11;
using xllm::KVCache;
using xllm::kernel::ReshapeFromCacheParams;
using xllm::kernel::ReshapePagedCacheParams;
using xllm::layer::AttentionImpl;
using xllm::layer::AttentionMetadata;

PYBIND11_MODULE(_xllm_hip_torch, m) {
  py::class_<ReshapePagedCacheParams>(m, "ReshapePagedCacheParams")
      .def(py::init<>())
      .def_readwrite("key", &ReshapePagedCacheParams::key)
      .def_readwrite("value", &ReshapePagedCacheParams::value)
      .def_readwrite("k_cache", &ReshapePagedCacheParams::k_cache)
      .def_readwrite("v_cache", &ReshapePagedCacheParams::v_cache)
      .def_readwrite("slot_mapping", &ReshapePagedCacheParams::slot_mapping)
      .def_readwrite("direction", &ReshapePagedCacheParams::direction)
      .def_readwrite("k_cache_scale", &ReshapePagedCacheParams::k_cache_scale)
      .def_readwrite("v_cache_scale", &ReshapePagedCacheParams::v_cache_scale);
  py::class_<ReshapeFromCacheParams>(m, "ReshapeFromCacheParams")
      .def(py::init<>())
      .def_readwrite("key", &ReshapeFromCacheParams::key)
      .def_readwrite("value", &ReshapeFromCacheParams::value)
      .def_readwrite("key_cache", &ReshapeFromCacheParams::key_cache)
      .def_readwrite("value_cache", &ReshapeFromCacheParams::value_cache)
      .def_readwrite("context_lengths", &ReshapeFromCacheParams::context_lengths)
      .def_readwrite("max_context_len", &ReshapeFromCacheParams::max_context_len)
      .def_readwrite("context_seq_offset", &ReshapeFromCacheParams::context_seq_offset)
      .def_readwrite("block_tables", &ReshapeFromCacheParams::block_tables)
      .def_readwrite("cache_seq_offset", &ReshapeFromCacheParams::cache_seq_offset)
      .def_readwrite("key_cache_quant_scale", &ReshapeFromCacheParams::key_cache_quant_scale)
      .def_readwrite("value_cache_quant_scale", &ReshapeFromCacheParams::value_cache_quant_scale)
      .def_readwrite("quant_mode", &ReshapeFromCacheParams::quant_mode)
      .def_readwrite("quant_bit", &ReshapeFromCacheParams::quant_bit);
  m.def("reshape_from_cache", &xllm::kernel::reshape_from_cache);
  m.def("dequant_from_paged_cache", &xllm::kernel::dequant_from_paged_cache);
  m.def("reshape_paged_cache", &xllm::kernel::reshape_paged_cache);
  m.def("quant_to_paged_cache", &xllm::kernel::quant_to_paged_cache);
  py::class_<xllm::layer::PlanInfo, std::shared_ptr<xllm::layer::PlanInfo>>(m, "PlanInfo")
      .def(py::init<>())
      .def_readwrite("layer_id", &xllm::layer::PlanInfo::layer_id)
      .def_readwrite("host_plan", &xllm::layer::PlanInfo::host_plan)
      .def_readwrite("kv_lens_host", &xllm::layer::PlanInfo::kv_lens_host);
  m.def("batch_decode",
        [](const torch::Tensor& query, const torch::Tensor& k_cache, torch::Tensor output,
           const torch::Tensor& block_table, const torch::Tensor& seq_lens, const std::optional<torch::Tensor>& v_cache,
           std::optional<torch::Tensor> output_lse, const std::optional<torch::Tensor>& k_scale,
           const std::optional<torch::Tensor>& v_scale, int64_t max_seq_len, int64_t window_size_left, float scale,
           bool return_lse, int64_t kv_cache_quant_bit_size, std::shared_ptr<xllm::layer::PlanInfo> plan_info) {
          xllm::kernel::hip::batch_decode(query, k_cache, output, block_table, seq_lens, v_cache, output_lse,
                                          std::nullopt, k_scale, v_scale, std::nullopt, std::nullopt, std::nullopt,
                                          "float", max_seq_len, window_size_left, -1, scale, return_lse,
                                          kv_cache_quant_bit_size, 0, plan_info.get());
        },
        py::arg("query"), py::arg("k_cache"), py::arg("output"), py::arg("block_table"), py::arg("seq_lens"),
        py::arg("v_cache"), py::arg("output_lse"), py::arg("k_scale"), py::arg("v_scale"), py::arg("max_seq_len"),
        py::arg("window_size_left"), py::arg("scale"), py::arg("return_lse"), py::arg("kv_cache_quant_bit_size"),
        py::arg("plan_info") = nullptr);
  m.def("batch_decode_csr",
        [](torch::Tensor query, torch::Tensor k_cache, torch::Tensor v_cache, torch::Tensor indptr, torch::Tensor indices,
           torch::Tensor last_page_len, int64_t window_left, double sm_scale, torch::Tensor output,
           std::optional<torch::Tensor> k_cache_scale, std::optional<torch::Tensor> v_cache_scale) {
          std::optional<torch::Tensor> lse = std::nullopt;
          xllm::kernel::hip::batch_decode_csr(query, k_cache, v_cache, indptr, indices, last_page_len, window_left,
                                              sm_scale, output, lse, nullptr, k_cache_scale, v_cache_scale);
        },
        py::arg("query"), py::arg("k_cache"), py::arg("v_cache"), py::arg("paged_kv_indptr"), py::arg("paged_kv_indices"),
        py::arg("paged_kv_last_page_len"), py::arg("window_left"), py::arg("sm_scale"), py::arg("output"),
        py::arg("k_cache_scale") = std::nullopt, py::arg("v_cache_scale") = std::nullopt);

  py::class_<KVCache>(m, "KVCache")
      .def(py::init<>())
      .def(py::init<torch::Tensor, torch::Tensor>())
      .def(py::init<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor>())
      .def_static("allocate",
                  [](const std::vector<int64_t>& shape, py::object dtype, const std::string& device, bool with_scales) {
                    return KVCache::allocate(shape, torch::python::detail::py_object_to_dtype(dtype),
                                             torch::Device(device), with_scales);
                  },
                  py::arg("shape"), py::arg("dtype"), py::arg("device"), py::arg("with_scales") = false)
      .def("get_k_cache", &KVCache::get_k_cache)
      .def("get_v_cache", &KVCache::get_v_cache)
      .def("get_k_cache_scale", &KVCache::get_k_cache_scale)
      .def("get_v_cache_scale", &KVCache::get_v_cache_scale)
      .def("empty", &KVCache::empty)
      .def("swap_blocks", [](KVCache& self, torch::Tensor src, torch::Tensor dst) { self.swap_blocks(src, dst); });
  m.def("copy_blocks", &xllm::kernel::hip::copy_blocks);

  py::class_<AttentionMetadata>(m, "AttentionMetadata")
      .def(py::init<>())
      .def_readwrite("plan_info", &AttentionMetadata::plan_info)
      .def_readwrite("kv_seq_lens", &AttentionMetadata::kv_seq_lens)
      .def_readwrite("q_seq_lens", &AttentionMetadata::q_seq_lens)
      .def_readwrite("block_table", &AttentionMetadata::block_table)
      .def_readwrite("slot_mapping", &AttentionMetadata::slot_mapping)
      .def_readwrite("max_query_len", &AttentionMetadata::max_query_len)
      .def_readwrite("max_seq_len", &AttentionMetadata::max_seq_len)
      .def_readwrite("total_kv_len", &AttentionMetadata::total_kv_len)
      .def_readwrite("is_prefill", &AttentionMetadata::is_prefill)
      .def_readwrite("is_chunked_prefill", &AttentionMetadata::is_chunked_prefill)
      .def_readwrite("is_dummy", &AttentionMetadata::is_dummy)
      .def_readwrite("paged_kv_indptr", &AttentionMetadata::paged_kv_indptr)
      .def_readwrite("paged_kv_indices", &AttentionMetadata::paged_kv_indices)
      .def_readwrite("paged_kv_last_page_len", &AttentionMetadata::paged_kv_last_page_len);
  m.def("build_decode_metadata",
        py::overload_cast<const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, const torch::Tensor&, int64_t,
                          int64_t, int64_t>(&xllm::layer::build_decode_metadata));
  m.def("build_decode_metadata", [](const xllm::host_index::DecodeBatchInputs& in, const std::string& device) {
    return xllm::layer::build_decode_metadata(in, torch::Device(device));
  });

  // host-side index producers
  namespace hi = xllm::host_index;
  m.def("kv_cache_slots", &hi::kv_cache_slots);
  m.def("calc_slot_id", &hi::calc_slot_id);
  m.def("calc_kv_len", &hi::calc_kv_len);
  py::class_<hi::DecodeBatchInputs>(m, "DecodeBatchInputs")
      .def(py::init<int32_t>())
      .def("add_sequence", &hi::DecodeBatchInputs::add_sequence)
      .def("pad_decode_batch", &hi::DecodeBatchInputs::pad_decode_batch)
      .def("num_sequences", &hi::DecodeBatchInputs::num_sequences)
      .def("total_kv_len", &hi::DecodeBatchInputs::total_kv_len)
      .def("padded_block_tables",
           [](const hi::DecodeBatchInputs& self) {
             int32_t width = 0;
             const std::vector<int32_t> flat = self.pad_block_tables(width);
             std::vector<std::vector<int32_t>> rows(self.block_tables.size());
             for (size_t b = 0; b < rows.size(); ++b) rows[b].assign(flat.begin() + b * width, flat.begin() + (b + 1) * width);
             return rows;
           })
      .def_readonly("positions", &hi::DecodeBatchInputs::positions)
      .def_readonly("new_cache_slots", &hi::DecodeBatchInputs::new_cache_slots)
      .def_readonly("q_seq_lens", &hi::DecodeBatchInputs::q_seq_lens)
      .def_readonly("kv_seq_lens", &hi::DecodeBatchInputs::kv_seq_lens)
      .def_readonly("paged_kv_indptr", &hi::DecodeBatchInputs::paged_kv_indptr)
      .def_readonly("paged_kv_indices", &hi::DecodeBatchInputs::paged_kv_indices)
      .def_readonly("paged_kv_last_page_len", &hi::DecodeBatchInputs::paged_kv_last_page_len)
      .def_readonly("write_block_ids", &hi::DecodeBatchInputs::write_block_ids)
      .def_readonly("q_max_seq_len", &hi::DecodeBatchInputs::q_max_seq_len)
      .def_readonly("kv_max_seq_len", &hi::DecodeBatchInputs::kv_max_seq_len);
  py::class_<hi::ExpandedDecodeRows>(m, "ExpandedDecodeRows")
      .def_readonly("positions", &hi::ExpandedDecodeRows::positions)
      .def_readonly("new_cache_slots", &hi::ExpandedDecodeRows::new_cache_slots)
      .def_readonly("kv_seq_lens", &hi::ExpandedDecodeRows::kv_seq_lens)
      .def_readonly("block_tables", &hi::ExpandedDecodeRows::block_tables)
      .def_readonly("kv_max_seq_len", &hi::ExpandedDecodeRows::kv_max_seq_len);
  m.def("expand_decode_rows", &hi::expand_decode_rows);
  m.def("decode_rows", [](const std::vector<int32_t>& positions, const std::vector<int32_t>& kv_cu,
                          const std::vector<std::vector<int32_t>>& block_tables, int32_t block_size,
                          const std::vector<std::pair<int32_t, int32_t>>& rows) {
    hi::ExpandedDecodeRows out;
    for (const auto& r : rows) hi::append_decode_row(positions, kv_cu, block_tables, block_size, r.first, r.second, out);
    return out;
  });

  py::class_<AttentionImpl>(m, "AttentionImpl")
      .def(py::init<int64_t, int64_t, float, int64_t, int64_t>())
      .def("set_prefill_dequant_rows", &AttentionImpl::set_prefill_dequant_rows)
      .def("forward", [](AttentionImpl& self, const AttentionMetadata& md, torch::Tensor query, torch::Tensor key,
                         torch::Tensor value, KVCache& kv) { return self.forward(md, query, key, value, kv); })
      .def("forward_qkv", [](AttentionImpl& self, const AttentionMetadata& md, torch::Tensor positions,
                             torch::Tensor qkv, torch::Tensor cos_sin_cache, bool interleaved,
                             std::optional<torch::Tensor> q_norm_weight, std::optional<torch::Tensor> k_norm_weight,
                             double eps, KVCache& kv) {
        return self.forward_qkv(md, positions, qkv, cos_sin_cache, interleaved, q_norm_weight, k_norm_weight, eps, kv);
      });
  m.def("set_decode_workspace_bytes", [](int64_t bytes) { xllm::kernel::hip::set_decode_workspace_bytes((size_t)bytes); });
  m.def("decode_workspace_capacity", []() { return (int64_t)xllm::kernel::hip::decode_workspace_capacity(); });
  m.def("decode_workspace_ptr", [](const std::string& device, int64_t stream) {
    return (int64_t)(intptr_t)xllm::kernel::hip::decode_workspace(torch::Device(device), (void*)(intptr_t)stream).data_ptr();
  });
  m.def("fused_qk_norm_rope", [](torch::Tensor qkv, int64_t hq, int64_t hk, int64_t hv, int64_t head_dim, double eps,
                                 torch::Tensor q_weight, torch::Tensor k_weight, torch::Tensor cos_sin_cache,
                                 bool interleaved, torch::Tensor position_ids) {
    xllm::kernel::hip::fused_qk_norm_rope(qkv, hq, hk, hv, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved,
                                          position_ids);
  });
  m.def("rotary_embedding", [](torch::Tensor positions, torch::Tensor query, std::optional<torch::Tensor> key,
                               torch::Tensor cos_sin_cache, bool is_neox) {
    xllm::kernel::hip::rotary_embedding(positions, query, key, cos_sin_cache, is_neox);
  });
}
