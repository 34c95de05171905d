// Host-side producers of the integer inputs of the paged-KV path: slot ids of the tokens written in
// a step, padded block tables, cumulative lengths and the CSR form of the block lists, plus the row
// expansion of a speculative step.  Plain C++ over std::vector — the scheduler side of the engine
// runs on the host, once per step, and hands these arrays to the device as int32 tensors.
//
// Restated from the reference:
//   kv_cache_slots          KVCacheState::kv_cache_slots       xllm/core/framework/request/sequence_kv_state.cpp:120-134
//   DecodeBatchInputs       BatchInputBuilder::setup_kv_cache_info / padding_decode_batch_size /
//                           state_to_forward_input             xllm/core/framework/batch/batch_input_builder.cpp:438-560
//   calc_slot_id, calc_kv_len, append_decode_row               xllm/core/runtime/spec_input_builder.cpp:76-161
// A violated precondition throws std::invalid_argument / std::out_of_range where the reference's
// CHECK aborts the process.
#pragma once

#include <algorithm>
#include <cstdint>
#include <set>
#include <stdexcept>
#include <string>
#include <vector>

namespace xllm::host_index {

inline void require(bool ok, const char* what) {
  if (!ok) throw std::invalid_argument(what);
}

// Slot ids of positions [pos_start, pos_end) of a sequence whose blocks are `block_ids`:
// slot = block_id * block_size + position % block_size.
inline std::vector<int32_t> kv_cache_slots(const std::vector<int32_t>& block_ids, int32_t block_size, int32_t pos_start,
                                           int32_t pos_end) {
  require(!block_ids.empty(), "no cache blocks available");
  require(block_size > 0, "invalid block_size");
  std::vector<int32_t> slots;
  slots.reserve(pos_end > pos_start ? pos_end - pos_start : 0);
  for (int32_t i = pos_start; i < pos_end; ++i) {
    require(i >= 0, "invalid position");
    const size_t block_idx = (size_t)(i / block_size);
    if (block_idx >= block_ids.size()) throw std::out_of_range("position beyond the sequence's blocks");
    slots.push_back(block_ids[block_idx] * block_size + i % block_size);
  }
  return slots;
}

// Slot of one position through a (padded) block-table row.
inline int32_t calc_slot_id(int32_t position, const std::vector<int32_t>& block_table_row, int32_t block_size) {
  require(block_size > 0, "invalid block_size");
  require(position >= 0, "invalid position");
  const int32_t block_idx = position / block_size;
  if ((size_t)block_idx >= block_table_row.size()) throw std::out_of_range("block table index out of range");
  const int32_t block_id = block_table_row[block_idx];
  require(block_id >= 0, "invalid block_id");
  return block_id * block_size + position % block_size;
}

// kv length of sequence seq_id from the cumulative lengths [batch + 1], plus `offset`.
inline int32_t calc_kv_len(const std::vector<int32_t>& kv_seq_lens_cumulative, int32_t seq_id, int32_t offset) {
  require(seq_id >= 0, "invalid seq_id");
  if ((size_t)(seq_id + 1) >= kv_seq_lens_cumulative.size()) throw std::out_of_range("seq_id out of range for cumulative layout");
  return kv_seq_lens_cumulative[seq_id + 1] - kv_seq_lens_cumulative[seq_id] + offset;
}

// The integer inputs of one step, accumulated sequence by sequence.
struct DecodeBatchInputs {
  std::vector<int32_t> positions;           // one per token of the step
  std::vector<int32_t> new_cache_slots;     // one per token of the step
  std::vector<int32_t> q_seq_lens = {0};    // cumulative, [batch + 1]
  std::vector<int32_t> kv_seq_lens = {0};   // cumulative, [batch + 1]
  std::vector<int32_t> paged_kv_indptr = {0};
  std::vector<int32_t> paged_kv_indices;
  std::vector<int32_t> paged_kv_last_page_len;
  std::vector<std::vector<int32_t>> block_tables;  // ragged until pad_block_tables()
  std::set<int32_t> write_block_ids;               // blocks that receive tokens in this step
  int32_t q_max_seq_len = 0;
  int32_t kv_max_seq_len = 0;
  int32_t block_size = 0;

  explicit DecodeBatchInputs(int32_t block_size_) : block_size(block_size_) {
    require(block_size_ > 0, "invalid block_size");
  }

  int32_t num_sequences() const { return (int32_t)block_tables.size(); }
  int64_t total_kv_len() const { return kv_seq_lens.back(); }

  // A sequence that holds n_kv_cache_tokens tokens in `block_ids` already and receives the tokens at
  // positions [n_kv_cache_tokens, seq_len) in this step.
  void add_sequence(const std::vector<int32_t>& block_ids, int32_t n_kv_cache_tokens, int32_t seq_len) {
    require(n_kv_cache_tokens >= 0 && seq_len > n_kv_cache_tokens, "a sequence needs at least one new token");
    const int32_t q_len = seq_len - n_kv_cache_tokens;
    const std::vector<int32_t> slots = kv_cache_slots(block_ids, block_size, n_kv_cache_tokens, seq_len);
    new_cache_slots.insert(new_cache_slots.end(), slots.begin(), slots.end());
    for (int32_t p = n_kv_cache_tokens; p < seq_len; ++p) positions.push_back(p);
    q_seq_lens.push_back(q_seq_lens.back() + q_len);
    kv_seq_lens.push_back(kv_seq_lens.back() + seq_len);
    q_max_seq_len = std::max(q_max_seq_len, q_len);
    kv_max_seq_len = std::max(kv_max_seq_len, seq_len);
    paged_kv_indices.insert(paged_kv_indices.end(), block_ids.begin(), block_ids.end());
    paged_kv_indptr.push_back(paged_kv_indptr.back() + (int32_t)block_ids.size());
    paged_kv_last_page_len.push_back(seq_len % block_size == 0 ? block_size : seq_len % block_size);
    for (size_t i = (size_t)(n_kv_cache_tokens / block_size); i < block_ids.size(); ++i) write_block_ids.insert(block_ids[i]);
    block_tables.push_back(block_ids);
  }

  // Padding rows up to a fixed decode batch size (graph replay wants fixed shapes): each writes slot 0
  // and owns the one reserved block 0 with a single token in it.
  void pad_decode_batch(int32_t num_decoding_tokens, int32_t min_decoding_batch_size) {
    const int32_t n = num_sequences();
    if (n >= min_decoding_batch_size) return;
    const bool same = q_max_seq_len == num_decoding_tokens && (int64_t)positions.size() == (int64_t)n * num_decoding_tokens;
    if (!same) return;
    for (int32_t i = n; i < min_decoding_batch_size; ++i) {
      for (int32_t k = 0; k < num_decoding_tokens; ++k) {
        positions.push_back(0);
        new_cache_slots.push_back(0);
      }
      kv_seq_lens.push_back(kv_seq_lens.back() + num_decoding_tokens);
      q_seq_lens.push_back(q_seq_lens.back() + num_decoding_tokens);
      block_tables.emplace_back();
      paged_kv_indices.push_back(0);
      paged_kv_indptr.push_back(paged_kv_indptr.back() + 1);
      paged_kv_last_page_len.push_back(1);
    }
  }

  // Block tables as a dense [batch, max_blocks] array, padded with `pad_value` (0: the reserved block).
  std::vector<int32_t> pad_block_tables(int32_t& max_blocks, int32_t pad_value = 0) const {
    size_t width = 0;
    for (const auto& row : block_tables) width = std::max(width, row.size());
    max_blocks = (int32_t)width;
    std::vector<int32_t> flat(block_tables.size() * width, pad_value);
    for (size_t b = 0; b < block_tables.size(); ++b) {
      std::copy(block_tables[b].begin(), block_tables[b].end(), flat.begin() + b * width);
    }
    return flat;
  }
};

// Rows of a speculative step: sequence s (last position positions[s], block-table row s) contributes
// one row per offset, at position positions[s] + offset, with kv length len(s) + offset and its own
// copy of the block-table row.
struct ExpandedDecodeRows {
  std::vector<int32_t> positions;
  std::vector<int32_t> new_cache_slots;
  std::vector<int32_t> kv_seq_lens;  // per row, not cumulative
  std::vector<std::vector<int32_t>> block_tables;
  int32_t kv_max_seq_len = 0;
};

// One row of a speculative step (append_decode_row, xllm/core/runtime/spec_input_builder.cpp:112-147):
// sequence seq_id at position positions[seq_id] + position_offset, appended to `out`.
inline void append_decode_row(const std::vector<int32_t>& positions, const std::vector<int32_t>& kv_seq_lens_cumulative,
                              const std::vector<std::vector<int32_t>>& block_tables, int32_t block_size, int32_t seq_id,
                              int32_t position_offset, ExpandedDecodeRows& out) {
  require(seq_id >= 0, "invalid seq_id");
  if ((size_t)seq_id >= positions.size() || (size_t)seq_id >= block_tables.size()) throw std::out_of_range("seq_id out of range");
  const int32_t pos = positions[seq_id] + position_offset;
  require(pos >= 0, "invalid decode position");
  out.positions.push_back(pos);
  out.new_cache_slots.push_back(calc_slot_id(pos, block_tables[seq_id], block_size));
  const int32_t kv_len = calc_kv_len(kv_seq_lens_cumulative, seq_id, position_offset);
  out.kv_max_seq_len = std::max(out.kv_max_seq_len, kv_len);
  out.kv_seq_lens.push_back(kv_len);
  out.block_tables.push_back(block_tables[seq_id]);
}

inline ExpandedDecodeRows expand_decode_rows(const std::vector<int32_t>& positions,
                                             const std::vector<int32_t>& kv_seq_lens_cumulative,
                                             const std::vector<std::vector<int32_t>>& block_tables, int32_t block_size,
                                             const std::vector<int32_t>& position_offsets) {
  require(positions.size() == block_tables.size(), "one position and one block-table row per sequence");
  ExpandedDecodeRows out;
  for (size_t s = 0; s < positions.size(); ++s) {
    for (const int32_t off : position_offsets) {
      append_decode_row(positions, kv_seq_lens_cumulative, block_tables, block_size, (int32_t)s, off, out);
    }
  }
  return out;
}

}  // namespace xllm::host_index
