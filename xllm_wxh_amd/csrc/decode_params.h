// Arguments of the decode kernels: one struct, passed by value, filled by fill_params on the host.
#pragma once

#include "decode_plan.h"

#include <stdint.h>

namespace xllm_hip {

struct DecodeParams {
  const void* q;
  void* out;
  float* lse;
  const uint8_t* k_cache;
  const uint8_t* v_cache;
  const float* k_scale;
  const float* v_scale;
  const int32_t* block_ids;  // block_table, or kv_indices in CSR form
  const int32_t* kv_indptr;  // non-NULL selects the CSR form
  const int32_t* seq_lens;
  const int32_t* kv_last_page_len;
  const int32_t* q_indptr;  // [batch+1] first query token of each sequence; NULL: n tokens each
  PlanHeader* hdr;
  int32_t* kv_len;
  int32_t* full_prefix;
  int32_t* tail_prefix;
  int32_t* num_chunks;
  SeqChunk* seq_chunks;
  float* partial_lse;
  float* partial_out;
  int32_t* counters;  // per (sequence, kv head, row group): chunks finished so far (fused merge)
  int64_t q_token_stride;
  int64_t out_token_stride;
  int64_t stride_block;
  int64_t stride_head;
  int64_t stride_slot;
  int64_t sc_stride_block;
  int64_t sc_stride_head;
  int64_t sc_stride_slot;
  int64_t bt_stride;
  int32_t max_seq_chunks;  // entries of seq_chunks
  int32_t batch;
  int32_t n;  // query tokens per sequence (the largest count when q_indptr is set)
  int32_t num_q_heads;
  int32_t num_kv_heads;
  int32_t heads_per_item;  // kv heads one work item covers: 1, or 4 (one per wave of the 16-row kernel; see fill_params)
  int32_t item_heads;      // num_kv_heads / heads_per_item: work items per sequence chunk and row group
  int32_t eight_waves;     // != 0: the 16-row kernel runs eight waves per work item whatever the launch's size (1-byte caches)
  int32_t wave_items;      // 1: every wave of a 16-row workgroup is a work item of its own (item 4 * workgroup + wave); 2: two waves to an item, two items to a workgroup; steps that are not split, and (2 only) a 1-byte cache of 64-byte rows with an even number of kv heads, whose split sequences the merge kernel combines
  int32_t lockstep;        // != 0: the 16-row kernel's waves, each attending a kv head of its own, walk their tokens in step (its LOCK form; 1-byte caches at head_dim 64 whose kv heads lie side by side)
  int32_t group;  // q heads per kv head
  int32_t rows;   // group * n
  int32_t row_groups;
  int32_t cluster;        // neighbouring work items kept on one XCD (see decode_item)
  int32_t rows_per_item;  // query rows one work item handles (32, 128 or 256 MFMA, 1 generic)
  int32_t prefill_opts;   // XLLM_HIP_OPTION_PREFILL_KERNEL as the 256-row kernel reads it
  int32_t min_chunk;      // smallest chunk the plan may choose
  int32_t head_dim;
  int32_t tok;          // tokens per 256-byte LDS row of the MFMA kernels: 1 (head_dim 128), 2 (head_dim 64),
                        // 0 (head_dim 256: a token is two rows, one in each half of the tile)
  int32_t tile_tokens;  // tokens per tile: 32 * tok (16 at head_dim 256); chunk sizes are multiples of it
  int32_t block_size;
  int32_t log2_bs;
  int32_t max_blocks_per_seq;
  int32_t last_block;  // num_blocks - 1: block ids are taken within 0 .. last_block
  int32_t len_cap;  // block_table form: tokens a table row can hold (a longer seq_lens entry is cut to it)
  int32_t window_left;
  int32_t target_items;   // workgroup slots of the launch (see choose_chunk)
  int32_t target_small;   // ... and the item budget of a batch with fewer (sequence, kv head, row group) triples
  int32_t fixed_chunk;    // > 0: chunk size chosen on the host (1 << 30 = never split)
  int32_t arith_chunks;   // > 0: no schedule is stored.  Every sequence owns this many chunk slots of fixed_chunk
                          // tokens (slot = sequence * arith_chunks + chunk); a work item derives its chunk, and a
                          // merge the row's partials, from the sequence's length alone
  int32_t arith_whole;    // ... except the first arith_whole sequences, which own arith_first slots each, for chunks
  int32_t arith_first;    // of first_chunk tokens (one slot and no cut: first_chunk = 2^30): slot = sequence *
  int32_t first_chunk;    // arith_first + chunk; then arith_whole * arith_first + (sequence - arith_whole) * arith_chunks + chunk
  int32_t direct_single;  // the attention kernel writes the output rows of single-chunk sequences itself
  int32_t implicit_plan;  // nothing is split and nothing is merged: item = (sequence, kv head, row group),
                          // lengths come straight from the inputs and no plan kernel runs
  int32_t fused_merge;    // the attention kernel merges a split sequence itself: the workgroup that finishes the
                          // last chunk of a (sequence, kv head, row group) combines the partials
  int32_t q_dtype;
  float scale_log2;  // sm_scale * log2(e)
};

// kv length of sequence b as every kernel uses it: never negative and never beyond what the
// sequence's block list holds, so that no block id is read from outside the list.
// (P: DecodeParams, possibly qualified with the constant address space)
template <class P>
__device__ inline int kv_length(const P& p, int b) {
  int len;
  if (p.kv_indptr != nullptr) {
    const int nb = p.kv_indptr[b + 1] - p.kv_indptr[b];
    int last = p.kv_last_page_len[b];
    last = last < p.block_size ? last : p.block_size;
    len = nb > 0 ? (nb - 1) * p.block_size + (last > 0 ? last : 0) : 0;
  } else {
    len = p.seq_lens[b];
    len = len < p.len_cap ? len : p.len_cap;
  }
  return len > 0 ? len : 0;
}

// Chunks of a sequence of `len` tokens cut every `chunk` tokens: the full ones and a tail; an empty
// sequence keeps one (empty) chunk, which writes zeros.
__device__ inline int chunks_of_length(int len, int chunk) {
  const int full = len / chunk;
  return full + ((len - full * chunk) > 0 || len == 0 ? 1 : 0);
}

// Chunks sequence b was cut into.  Without a stored schedule: never more than the slots a sequence
// owns (the last slot's chunk then runs to the end of the sequence, see decode_item).
template <class P>
__device__ inline int chunks_of_sequence(const P& p, int b) {
  if (p.arith_chunks > 0) {
    const bool first = b < p.arith_whole;
    const int slots = first ? p.arith_first : p.arith_chunks;
    const int cnt = chunks_of_length(kv_length(p, b), first ? p.first_chunk : p.fixed_chunk);
    return cnt < slots ? cnt : slots;
  }
  return p.num_chunks[b];
}

// A block id as the kernels use it: within the cache, whatever the table holds.
__device__ inline int block_in_cache(const DecodeParams& p, int id) {
  id = id > 0 ? id : 0;
  return id < p.last_block ? id : p.last_block;
}

}  // namespace xllm_hip
