// What a workgroup of an attention kernel works on, decoded from its index.
#pragma once

#include "decode_params.h"

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Work-item decoding shared by the attention kernels.
// ---------------------------------------------------------------------------------

struct Item {
  int sc;       // sequence-chunk slot (indexes the partial arrays)
  int b;        // sequence
  int hk;       // kv head
  int rg;       // row group
  int len;      // kv length of the sequence
  int t_begin;  // first token of the chunk (multiple of kTileTokens)
  int t_end;    // one past the last token of the chunk (<= len)
  const int32_t* ids;  // block list of the sequence
  int nblk;     // valid entries in ids (>= 1)
  int n;        // query tokens of the sequence
  int q0;       // index of its first query token
  int chunks;   // chunks the sequence was cut into (1: this item writes the output rows itself)
  int64_t head_off;     // hk * stride_head (cache elements)
  int64_t sc_head_off;  // hk * sc_stride_head (scale elements)
};

constexpr int kXcds = 8;  // workgroup x runs on XCD x % 8, each with its own L2

__device__ inline bool decode_item(const DecodeParams& p, int item_id, Item& it) {
  // Work items in their natural order are (sequence chunk, kv head, row group), row group fastest.
  // Some neighbours in that order read the same memory: the row groups of one (chunk, kv head) stream
  // the same K/V, and with small blocks the scale rows of neighbouring kv heads share cache lines.
  // Consecutive workgroup ids land on different XCDs, so a cluster of `p.cluster` neighbours is
  // given ids that are congruent mod 8 and consecutive on that XCD: its members then run there at
  // about the same time, and all but the first find the shared lines in that XCD's L2.
  int linear = item_id;
  if (p.cluster > 1) {
    const int on_xcd = item_id / kXcds;
    linear = ((on_xcd / p.cluster) * kXcds + item_id % kXcds) * p.cluster + on_xcd % p.cluster;
  }
  it.rg = linear % p.row_groups;
  const int rest = linear / p.row_groups;
  // (an item that covers several kv heads gets the first of them here; its waves take one each)
  it.hk = (rest % p.item_heads) * p.heads_per_item;
  it.sc = rest / p.item_heads;
  int chunk = 0, chunk_tokens = 1 << 30;
  it.chunks = 1;
  bool to_the_end = false;  // the chunk runs to the end of the sequence whatever its length
  int stored_begin = -1, stored_end = 0;  // the chunk's token range as a stored schedule gives it
  if (p.implicit_plan) {
    if (it.sc >= p.batch) return false;
    it.b = it.sc;
  } else if (p.arith_chunks > 0) {
    // No stored schedule: slot = sequence * arith_chunks + chunk.  The block list, the queries and the
    // length are then independent loads.  A sequence longer than its slots hold (a host-side
    // max_seq_len that was too small) gives the rest to its last chunk.
    // The first arith_whole sequences own arith_first slots each (one, when they are not cut), ahead of the
    // others': they are the long items of the launch, and run first.
    const int first_slots = p.arith_whole * p.arith_first;
    const bool first = it.sc < first_slots;
    const int rest_sc = it.sc - first_slots;
    const int slots = first ? p.arith_first : p.arith_chunks;
    it.b = first ? it.sc / slots : p.arith_whole + rest_sc / slots;
    chunk = first ? it.sc - it.b * slots : rest_sc - (it.b - p.arith_whole) * slots;
    if (it.b >= p.batch) return false;
    it.len = kv_length(p, it.b);
    chunk_tokens = first ? p.first_chunk : p.fixed_chunk;
    const int cnt = chunks_of_length(it.len, chunk_tokens);
    it.chunks = cnt < slots ? cnt : slots;
    if (chunk >= it.chunks) return false;
    to_the_end = chunk == slots - 1;
  } else {
    // The header and the item's record are independent loads (the record's index is clamped to the
    // table, whose last entries the plan may not have written: such a record is not used).
    const SeqChunk s = p.seq_chunks[it.sc < p.max_seq_chunks ? it.sc : 0];
    const PlanHeader hdr = *p.hdr;
    if (rest * p.row_groups >= hdr.total_items || it.sc >= p.max_seq_chunks) return false;
    // (a record no plan wrote — a run on a workspace that was planned with other host-side lengths —
    // names no sequence outside the batch)
    if ((unsigned)s.seq >= (unsigned)p.batch || s.chunk < 0) return false;
    // (nor a partial slot outside the workspace, nor a token range outside the sequence)
    if ((unsigned)s.slot >= (unsigned)p.max_seq_chunks || s.t_begin < 0 || s.len < 0) return false;
    it.b = s.seq;
    it.len = s.len;
    it.chunks = s.chunks;
    it.sc = s.slot;
    stored_begin = s.t_begin;
    stored_end = s.t_end < s.len ? s.t_end : s.len;
  }
  if (p.q_indptr != nullptr) {
    it.q0 = p.q_indptr[it.b];
    const int cnt = p.q_indptr[it.b + 1] - it.q0;
    it.n = cnt < 0 ? 0 : (cnt > p.n ? p.n : cnt);  // never beyond what the launch and the workspace were sized for
  } else {
    it.q0 = it.b * p.n;
    it.n = p.n;
  }
  if (it.rg * p.rows_per_item >= it.n * p.group) return false;  // this sequence has no rows in the group
  if (p.implicit_plan) it.len = kv_length(p, it.b);
  if (stored_begin >= 0) {
    it.t_begin = stored_begin;
    it.t_end = stored_end;
  } else {
    it.t_begin = chunk * chunk_tokens;
    const long long end = (long long)it.t_begin + chunk_tokens;
    it.t_end = end < it.len && !to_the_end ? (int)end : it.len;
  }
  {  // no row of the item sees beyond the causal limit of its last row
    const int rows = it.n * p.group;
    const int last = min((it.rg + 1) * p.rows_per_item, rows) - 1;
    const int lim = it.len - (it.n - 1 - last / p.group);
    it.t_end = it.t_end < lim ? it.t_end : lim;
  }
  if (p.kv_indptr != nullptr) {
    it.ids = p.block_ids + p.kv_indptr[it.b];
  } else {
    it.ids = p.block_ids + (int64_t)it.b * p.bt_stride;
  }
  it.nblk = (it.len + p.block_size - 1) >> p.log2_bs;
  if (p.kv_indptr != nullptr) {  // (a stored length that the sequence's list cannot hold reads no id outside the list)
    const int listed = p.kv_indptr[it.b + 1] - p.kv_indptr[it.b];
    it.nblk = it.nblk < listed ? it.nblk : listed;
  }
  if (it.nblk < 1) it.nblk = 1;
  it.head_off = (int64_t)it.hk * p.stride_head;
  it.sc_head_off = (int64_t)it.hk * p.sc_stride_head;
  return true;
}

}  // namespace xllm_hip
