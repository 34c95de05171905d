// Split-KV schedule of one decode step and the workspace layout that carries it.
//
// A sequence of kv length L is cut into chunks of `chunk_tokens` tokens (a
// multiple of the 32-token tile): floor(L/C) full chunks and, if L % C != 0,
// one tail chunk (an empty sequence keeps one empty chunk).  One work item =
// (sequence chunk, kv head, row group), run by one workgroup.  A sequence that
// is a single chunk has its output rows written by that workgroup; a split
// sequence gets one normalised partial output and its base-2 log-sum-exp per
// chunk and row, and the merge kernel combines them with
// w_i = 2^(lse_i - lse_total) — the algebra of the reference's two-partial merge
// (xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73), extended to any
// number of partials.
//
// Full chunks are numbered before tail chunks so that the hardware dispatcher,
// which starts workgroups in index order, runs the equal-sized long items first
// and fills the end of the launch with the short tails.
#pragma once

#include <stddef.h>
#include <stdint.h>

namespace xllm_hip {

constexpr int kTileTokens = 32;       // rows per MFMA tile (one token each, two at head_dim 64); chunk sizes are multiples of a tile
constexpr int kMinChunkTokens = 512;  // smallest split worth a partial round trip (128 tokens per wave)
constexpr int kMinChunkTokensGeneric = 64;  // the one-wave kernel: one 64-token step
constexpr int kMaxTargetItems = 2048; // largest split target of any kernel: eight one-wave items of the generic kernel per CU
constexpr int kMaxRowsPerItem = 32;   // query rows (g * n) one work item of the MFMA decode kernels handles
constexpr int kPrefillRowsPerItem = 128;  // ... and of the many-row (prefill) kernel, used above kPrefillMinRows rows
constexpr int kPrefillMinRows = 32;
constexpr int kPrefillWideRows = 256;  // ... and of its eight-wave form, used above kPrefillRowsPerItem rows (16-bit caches)

#if defined(__HIPCC__)
#define XLLM_HIP_HD __host__ __device__
#else
#define XLLM_HIP_HD
#endif

// Chunk size for a batch whose kv lengths sum to `total` with maximum `max_len`.  Shared by the
// device-side plan and by the host's check that nothing is split, so it uses these aggregates only.
//
// `target` is the number of work items the GPU holds at once (workgroup slots).  A batch with at least
// that many (sequence, kv head, row group) triples is cut so that about `target` items exist — a quarter
// more when it is ragged (longest sequence above 1.5x the mean): the tail chunks then differ in size,
// and although they are dispatched longest first a little slack helps the last ones pack.  (Measured on
// the ragged workload: 320 to 900 items are equally good, 2000 items cost 4 %.)
//
// A smaller batch is cut against `target_small`, for the 16-row kernel one workgroup per CU: a split
// launch is bound by HBM from about 150 equal items on, and what more items add is partials for the
// merge and workgroups whose prologue and epilogue nothing overlaps.  Measured, one sequence of 32768
// tokens x 8 kv heads: 192 to 256 items 33-34 us, 320 and more 40-43 us; 3 x 20000 tokens: 47 us at 192
// items, 53-58 us at 264 to 504.
//   equal lengths   the item count is exact: k = target_small / triples chunks per sequence (at least
//                   one: 24 x 8192 tokens x 8 kv heads run unsplit as 192 items in 119 us, cut in three
//                   for 512 slots — 576 items, a second round — 145 us; 20 x 8192 tokens: 104 us as 160
//                   items, 107 as 480);
//   else            items <= triples + work / chunk, so chunk = work / (target_small - triples) keeps them
//                   within target_small; but no coarser than work / (9/16 target_small) — below about 144
//                   equal items the longest one, streaming alone at some 50 GB/s, would set the time
//                   (one long sequence in a batch of short ones); and a sequence that would only shed a
//                   tail under a quarter of a chunk is left whole.
XLLM_HIP_HD inline int choose_chunk(long long total, long long max_len, int batch, int num_kv_heads,
                                    int row_groups, int target, int target_small, int min_chunk,
                                    int tile = kTileTokens) {
  const long long triples = (long long)batch * num_kv_heads * row_groups;
  const long long work = total * num_kv_heads * row_groups;
  long long c;
  if (max_len * batch == total) {
    long long k = triples > 0 ? target_small / triples : 1;
    if (k < 1) k = 1;
    c = (max_len + k - 1) / k;
  } else if (triples < target_small) {
    const long long within = target_small - triples;
    const long long enough = (long long)target_small * 9 / 16;
    const long long c_within = (work + within - 1) / within;
    const long long c_enough = (work + enough - 1) / enough;
    c = c_within < c_enough ? c_within : c_enough;
    if (max_len <= c + c / 4) c = max_len;
  } else {
    long long t = target;
    if (max_len * batch * 2 > total * 3) t += t / 4;
    if (t > kMaxTargetItems) t = kMaxTargetItems;
    c = (work + t - 1) / t;
  }
  c = (c + tile - 1) / tile * tile;
  if (c < min_chunk) c = min_chunk;
  if (c > (1 << 30)) c = 1 << 30;
  return (int)c;
}

struct PlanHeader {
  int32_t total_full;    // number of full sequence-chunks
  int32_t total_tail;    // number of tail sequence-chunks
  int32_t chunk_tokens;  // C (the device-side plan; a plan made on the host cuts every sequence to its own size)
  int32_t total_items;   // (total_full + total_tail) * num_kv_heads * row_groups
  int32_t pad[12];
};

// One sequence chunk of the stored schedule, in the order the work items are dispatched.
struct SeqChunk {
  int32_t seq;      // sequence index b
  int32_t chunk;    // chunk index within the sequence
  int32_t len;      // kv length of the sequence
  int32_t chunks;   // chunks of the sequence: one record tells a work item all it needs
  int32_t t_begin;  // token range of the chunk: [t_begin, t_end), t_begin a multiple of the tile
  int32_t t_end;
  int32_t slot;     // where the chunk's partial rows live: full_prefix[seq] + chunk for a full chunk, total_full +
                    // tail_prefix[seq] for a tail (the device-side plan dispatches in slot order: slot = index)
  int32_t pad;
};

struct WorkspaceLayout {
  size_t header;        // PlanHeader
  size_t kv_len;        // int32 [B]
  size_t full_prefix;   // int32 [B+1]  first full-chunk slot of sequence b
  size_t tail_prefix;   // int32 [B+1]  tail-chunk slot (relative to total_full) of sequence b
  size_t num_chunks;    // int32 [B]    chunks of sequence b (full + tail)
  size_t seq_chunks;    // SeqChunk [max_seq_chunks]
  size_t partial_lse;   // float [max_seq_chunks][n][Hq]
  size_t partial_out;   // float [max_seq_chunks][n][Hq][D]
  size_t counters;      // int32 [B][Hkv][row groups]  chunks of a (sequence, kv head, row group) that have finished
  size_t total_bytes;
  int64_t max_seq_chunks;
};

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

inline int row_groups(int q_per_seq, int num_q_heads, int num_kv_heads, int rows_per_item = kMaxRowsPerItem) {
  const int rows = q_per_seq * (num_q_heads / num_kv_heads);
  return (rows + rows_per_item - 1) / rows_per_item;
}

// More than four row groups per kv head (over 128 query rows: chunked prefill rather than decode or
// speculative verify): sequences are never split into chunks.
constexpr int kMaxRowGroupsForSplit = 4;
inline bool never_split(int q_per_seq, int num_q_heads, int num_kv_heads) {
  return row_groups(q_per_seq, num_q_heads, num_kv_heads) > kMaxRowGroupsForSplit;
}

// Split target of each kernel: about this many work items (workgroups) per launch.  A workgroup of the
// 16-row and the 128-row MFMA kernels is four waves, one per SIMD of a CU, and two fit on a CU (256
// VGPRs, < 80 KiB of LDS); four two-wave workgroups of the 32-row kernel do; the generic kernel runs
// one wave per item, eight per CU.  head_dim 256 runs one wave per SIMD: half as many workgroups.
// CUs of the device the sizes are for: the callers pass what the device reports (hipDeviceAttributeMultiprocessorCount,
// read once per device); this is the MI355X's count, for code that sizes things with no device at hand.
constexpr int kDefaultCUs = 256;
// Up to 16 query rows per kv head, over a cache whose kv heads lie side by side within a token, a work item
// covers four kv heads (one per wave of the 16-row kernel) when the head count allows it.
constexpr int kHeadsPerItem = 4;
// (17 to 32 rows: the 32-row kernel's form of the same, a pair of waves per head; `rows32` says that the caller means it)
inline int item_heads_of(int rows, int num_kv_heads, bool heads_side_by_side, bool rows32 = false) {
  return heads_side_by_side && (rows <= 16 || (rows32 && rows <= 32)) && num_kv_heads % kHeadsPerItem == 0
             ? num_kv_heads / kHeadsPerItem
             : num_kv_heads;
}
inline int natural_target_items(bool mfma, int rows, bool one_wave_per_simd, int cus = kDefaultCUs) {
  int v = !mfma ? 8 * cus : (rows > 16 && rows <= kPrefillMinRows) ? 4 * cus : 2 * cus;
  if (one_wave_per_simd) v /= 2;
  return v;
}

// Sequence chunks any lengths can produce, for any kernel that may serve the shape (the workspace is
// sized before the kernel is chosen).  Sum_b ceil(L_b / C) <= sum(L)/C + B, and choose_chunk keeps
// C >= sum(L) * Hkv * RG / t with t at most the kernel's target plus a quarter, so a kernel with
// target T and RG row groups yields at most 1.25 T / (Hkv * RG) + B chunks:
//   generic kernel   T = 2048, one row per item: RG = rows
//   MFMA kernels     up to 16 rows T = 512, 17..32 rows T = 1024 (RG = 1); more rows T = 512 with 128
//                    (16-bit cache) or 32 (1-byte cache) rows per item: RG >= ceil(rows / 128)
//   16-row MFMA kernel over a cache whose heads lie side by side (work items of kHeadsPerItem kv heads): Hkv / 4 in place of Hkv
inline int64_t max_seq_chunks_for(int batch, int rows, int num_kv_heads, int cus = kDefaultCUs) {
  auto bound = [&](int64_t target, int64_t rg, int64_t heads) { return (target + target / 4 + heads * rg - 1) / (heads * rg); };
  const int64_t generic = bound(natural_target_items(false, rows, false, cus), rows, num_kv_heads);
  const int64_t mfma = bound(natural_target_items(true, rows, false, cus),
                             rows <= kPrefillMinRows ? 1 : (rows + kPrefillRowsPerItem - 1) / kPrefillRowsPerItem,
                             item_heads_of(rows, num_kv_heads, true));
  return (generic > mfma ? generic : mfma) + batch + 1;
}

inline WorkspaceLayout workspace_layout(int batch, int q_per_seq, int num_q_heads, int num_kv_heads, int head_dim,
                                        int cus = kDefaultCUs) {
  WorkspaceLayout w;
  w.max_seq_chunks = max_seq_chunks_for(batch, q_per_seq * (num_q_heads / num_kv_heads), num_kv_heads, cus);
  // A step that is never split writes its output rows directly, whichever kernel serves it: no chunk
  // records and no partial rows (at 4096 query tokens they would be 64 MiB that nothing touches).
  const bool whole = never_split(q_per_seq, num_q_heads, num_kv_heads);
  if (whole) w.max_seq_chunks = 0;
  size_t off = 0;
  w.header = off;
  off += sizeof(PlanHeader);
  w.kv_len = off;
  off = align_up(off + sizeof(int32_t) * (size_t)batch, 64);
  w.full_prefix = off;
  off = align_up(off + sizeof(int32_t) * ((size_t)batch + 1), 64);
  w.tail_prefix = off;
  off = align_up(off + sizeof(int32_t) * ((size_t)batch + 1), 64);
  w.num_chunks = off;
  off = align_up(off + sizeof(int32_t) * (size_t)batch, 64);
  w.seq_chunks = off;
  off = align_up(off + sizeof(SeqChunk) * (size_t)w.max_seq_chunks, 256);
  w.partial_lse = off;
  off = align_up(off + sizeof(float) * (size_t)w.max_seq_chunks * q_per_seq * num_q_heads, 256);
  w.partial_out = off;
  off = align_up(off + sizeof(float) * (size_t)w.max_seq_chunks * q_per_seq * num_q_heads * head_dim, 256);
  w.counters = off;
  off = align_up(off + sizeof(int32_t) * (size_t)batch * num_kv_heads * row_groups(q_per_seq, num_q_heads, num_kv_heads), 256);
  w.total_bytes = off;
  return w;
}

}  // namespace xllm_hip
