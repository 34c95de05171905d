// Paged-attention decode for gfx950 (MI355X): split-KV ("flash decoding") over
// block_tables / seq_lens with GQA, bf16 / fp16 / fp8-e4m3 / int8 KV caches, one or several query
// tokens per sequence (decode, speculative verify, prefill chunks).
//
// Launches per call, none of which reads anything back to the host:
//   decode_plan_kernel   kv lengths -> chunk size, chunk table (one wave; once per step)
//   decode_*_kernel      one workgroup per (sequence chunk, kv head, row group): its waves stream
//                        the chunk's K and V once; a sequence that is a single chunk gets its
//                        output rows written directly, otherwise a normalised partial +
//                        log2-sum-exp is written, and (16-row MFMA kernel) the workgroup that finishes
//                        the last chunk of a (sequence, kv head) combines its partials
//   decode_merge_kernel  combines the partials of the sequences that were split (the other kernels)
// When the host-side length hints show that no sequence needs splitting, only the middle one is
// launched: a work item is then (sequence, kv head, row group) and needs no schedule.
//
// Semantics follow the reference's decode operators: head map kv = h / (Hq/Hkv)
// and fp32 softmax as in xllm/core/layers/cuda/flashinfer_attention.cpp:61-88, the
// block_table / seq_lens contract of xllm/core/kernels/mlu/mlu_ops_api.h:126-145,
// the CSR contract of xllm/core/kernels/cuda/cuda_ops_api.h:120-136, and the
// base-2 partial merge of xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73.
#include "decode_plan.h"
#include "decode_schedule.h"
#include "device_utils.h"
#include "host_utils.h"
// the device side, in the order a decode step uses it
#include "decode_params.h"
#include "decode_plan_kernel.h"
#include "decode_item.h"
#include "decode_merge.h"
#include "decode_mfma.h"
#include "prefill_pingpong.h"
#include "decode_generic.h"

#include <math.h>
#include <stdlib.h>

#include <atomic>
#include <mutex>
#include <type_traits>

// Workspace of xllm_hip_paged_decode_static: one array per GPU, part of the loaded code object (it is
// never allocated or freed).  In host code the name is only a handle for hipGetSymbolAddress; kernels
// get the address that call returns, like any caller-owned workspace.
static __device__ __align__(256) unsigned char scratch[XLLM_HIP_STATIC_WORKSPACE_BYTES];

namespace xllm_hip {

// ---------------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------------

enum Variant { kNone = 0, kMfmaD128 = 1, kGeneric = 2, kMfmaD64 = 3, kMfmaD256 = 4 };
static bool is_mfma(Variant v) { return v == kMfmaD128 || v == kMfmaD64 || v == kMfmaD256; }

// Process-wide diagnostic switches (xllm_hip_set_option).  Their initial values come from the
// environment, read once, when the first of them is used.
struct Options {
  std::atomic<int64_t> v[XLLM_HIP_OPTION_COUNT];
  Options() {
    static const char* const names[XLLM_HIP_OPTION_COUNT] = {
        "XLLM_HIP_DECODE_FORCE_GENERIC", "XLLM_HIP_DECODE_TARGET_ITEMS", "XLLM_HIP_DECODE_SEPARATE_MERGE",
        "XLLM_HIP_DECODE_STORED_SCHEDULE", "XLLM_HIP_DECODE_ITEM_PER_HEAD", "XLLM_HIP_DECODE_FOUR_WAVE_ITEMS",
        "XLLM_HIP_PREFILL_KERNEL"};
    for (int i = 0; i < XLLM_HIP_OPTION_COUNT; ++i) {
      const char* e = getenv(names[i]);
      v[i].store(e != nullptr ? atoll(e) : 0, std::memory_order_relaxed);
    }
  }
};
static Options& options() {
  static Options o;  // (initialisation of a function-local static is thread-safe)
  return o;
}
static int64_t option(int which) { return options().v[which].load(std::memory_order_relaxed); }

// CUs of the current device, as the runtime reports them (asked once per device; kDefaultCUs where there is no
// device to ask: the size functions are also called on hosts without a GPU).
static int device_cus() {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    (void)hipGetLastError();
    return kDefaultCUs;
  }
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = kDefaultCUs;
    }
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Work items to aim for (natural_target_items), or fewer when the diagnostic option says so: the
// workspace is sized for the natural targets, so the option can only lower them.
static int target_items(int variant_is_mfma, int rows, bool one_wave_per_simd) {
  const int v = natural_target_items(variant_is_mfma != 0, rows, one_wave_per_simd, device_cus());
  const int64_t t = option(XLLM_HIP_OPTION_DECODE_TARGET_ITEMS);
  return t > 0 && t < v ? (int)t : v;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

static Variant pick_variant(const xllm_hip_kv_cache* c, const xllm_hip_decode_args* a) {
  const int eb = elem_bytes(c->dtype);
  // 16-bit queries; a 16-bit cache must have the queries' type
  const bool q16 = a->q_dtype == XLLM_HIP_BF16 || a->q_dtype == XLLM_HIP_FP16;
  const bool kv_ok = q16 && (c->dtype == a->q_dtype || c->dtype == XLLM_HIP_FP8_E4M3 || c->dtype == XLLM_HIP_INT8);
  const bool force_generic = option(XLLM_HIP_OPTION_DECODE_FORCE_GENERIC) != 0;
  // head_dim 64 rides on the head_dim-128 kernels with two tokens per tile row: half a tile
  // (32 tokens) must then lie in one block.
  // head_dim 256 rides on them with two tile rows per token: a tile is 16 tokens.
  const bool d128 = c->head_dim == 128 && c->block_size >= 16;
  const bool d64 = c->head_dim == 64 && c->block_size >= 32;
  const bool d256 = c->head_dim == 256 && c->block_size >= 16;
  if (!force_generic && (d128 || d64 || d256) && kv_ok && is_pow2(c->block_size) && a->sm_scale >= 0.0f) {
    const int vec = 16 / eb;  // elements per 16-byte load
    const bool strides_ok = c->stride_block % vec == 0 && c->stride_head % vec == 0 && c->stride_slot % vec == 0 &&
                            a->q_token_stride % 8 == 0 && a->out_token_stride % 8 == 0;
    // (the output rows are written as 16-byte vectors, like the query rows are read)
    const bool ptrs_ok = aligned16(c->k_cache) && aligned16(c->v_cache) && aligned16(a->q) && aligned16(a->out);
    const int64_t lim32 = (int64_t)1 << 31;  // the kernels form block and slot offsets from 32-bit factors
    bool scales_ok = true;
    if (eb == 1) {
      scales_ok = c->k_scale != nullptr && c->v_scale != nullptr && c->scale_stride_block >= 0 &&
                  c->scale_stride_block < lim32 && c->scale_stride_slot >= 0 &&
                  c->scale_stride_slot * c->block_size < lim32;
    }
    const bool range_ok = c->stride_block >= 0 && c->stride_block < lim32 && c->stride_slot >= 0 &&
                          c->stride_slot * c->block_size < lim32;
    if (strides_ok && range_ok && ptrs_ok && scales_ok) return d128 ? kMfmaD128 : d64 ? kMfmaD64 : kMfmaD256;
  }
  if (c->head_dim <= 256 && is_pow2(c->block_size)) return kGeneric;
  return kNone;
}

static int fill_params(const xllm_hip_kv_cache* c,
                       const xllm_hip_decode_args* a,
                       void* workspace,
                       size_t workspace_bytes,
                       DecodeParams& p) {
  XLLM_HIP_REQUIRE(c != nullptr && a != nullptr, "cache or args is NULL");
  // A step whose schedule comes from xllm_hip_paged_decode_plan_host: the kernel and the shape of its work items
  // follow from sizes alone — never from the host-side lengths, which a captured graph would freeze — and the
  // schedule is always the stored one, which that call (or the device-side plan) rewrites before every step.
  xllm_hip_decode_args sized;
  if (a->host_plan != 0) {
    sized = *a;
    sized.max_seq_len = 0;
    sized.total_kv_len = 0;
    a = &sized;
  }
  XLLM_HIP_REQUIRE(c->k_cache != nullptr && c->v_cache != nullptr, "k_cache or v_cache is NULL");
  XLLM_HIP_REQUIRE(c->num_blocks > 0 && c->block_size > 0 && c->num_kv_heads > 0 && c->head_dim > 0,
                   "cache sizes must be positive");
  XLLM_HIP_REQUIRE(elem_bytes(c->dtype) > 0, "unknown cache dtype %d", c->dtype);
  XLLM_HIP_REQUIRE(a->batch >= 0 && a->q_per_seq >= 1 && a->num_q_heads >= 1, "bad batch/q_per_seq/num_q_heads");
  XLLM_HIP_REQUIRE(a->num_q_heads % c->num_kv_heads == 0, "num_q_heads %d is not a multiple of num_kv_heads %d",
                   a->num_q_heads, c->num_kv_heads);
  XLLM_HIP_REQUIRE(a->q_dtype == XLLM_HIP_BF16 || a->q_dtype == XLLM_HIP_FP16 || a->q_dtype == XLLM_HIP_FP32,
                   "query dtype must be BF16/FP16/FP32, got %d", a->q_dtype);
  const bool quant = c->dtype == XLLM_HIP_FP8_E4M3 || c->dtype == XLLM_HIP_INT8;
  XLLM_HIP_REQUIRE(!quant || (c->k_scale != nullptr && c->v_scale != nullptr),
                   "a quantised cache needs k_scale and v_scale");
  if (a->batch > 0) {
    XLLM_HIP_REQUIRE(a->q != nullptr && a->out != nullptr, "q or out is NULL");
    if (a->block_table != nullptr) {
      XLLM_HIP_REQUIRE(a->seq_lens != nullptr, "block_table form needs seq_lens");
      XLLM_HIP_REQUIRE(a->max_blocks_per_seq >= 1 && a->block_table_stride >= a->max_blocks_per_seq,
                       "bad block_table shape");
    } else {
      XLLM_HIP_REQUIRE(a->kv_indptr != nullptr && a->kv_indices != nullptr && a->kv_last_page_len != nullptr,
                       "neither block_table nor the CSR arrays were given");
    }
    const int64_t rowlen = (int64_t)a->num_q_heads * c->head_dim;
    XLLM_HIP_REQUIRE(a->q_token_stride >= rowlen && a->out_token_stride >= rowlen,
                     "q/out token stride smaller than num_q_heads*head_dim");
  }
  const WorkspaceLayout w =
      workspace_layout(a->batch, a->q_per_seq, a->num_q_heads, c->num_kv_heads, c->head_dim, device_cus());
  if (workspace == nullptr || workspace_bytes < w.total_bytes) {
    return fail(XLLM_HIP_WORKSPACE_TOO_SMALL, "workspace has %zu bytes, need %zu", workspace_bytes, w.total_bytes);
  }
  XLLM_HIP_REQUIRE(((uintptr_t)workspace & 255) == 0, "workspace must be 256-byte aligned");

  uint8_t* ws = (uint8_t*)workspace;
  p = DecodeParams{};
  p.q = a->q;
  p.out = a->out;
  p.lse = a->lse;
  p.k_cache = (const uint8_t*)c->k_cache;
  p.v_cache = (const uint8_t*)c->v_cache;
  p.k_scale = c->k_scale;
  p.v_scale = c->v_scale;
  if (a->block_table != nullptr) {
    p.block_ids = a->block_table;
    p.kv_indptr = nullptr;
    p.seq_lens = a->seq_lens;
  } else {
    p.block_ids = a->kv_indices;
    p.kv_indptr = a->kv_indptr;
    p.kv_last_page_len = a->kv_last_page_len;
  }
  p.q_indptr = a->q_indptr;
  p.hdr = (PlanHeader*)(ws + w.header);
  p.kv_len = (int32_t*)(ws + w.kv_len);
  p.full_prefix = (int32_t*)(ws + w.full_prefix);
  p.tail_prefix = (int32_t*)(ws + w.tail_prefix);
  p.num_chunks = (int32_t*)(ws + w.num_chunks);
  p.seq_chunks = (SeqChunk*)(ws + w.seq_chunks);
  p.max_seq_chunks = (int32_t)w.max_seq_chunks;
  p.partial_lse = (float*)(ws + w.partial_lse);
  p.partial_out = (float*)(ws + w.partial_out);
  p.counters = (int32_t*)(ws + w.counters);
  p.q_token_stride = a->q_token_stride;
  p.out_token_stride = a->out_token_stride;
  p.stride_block = c->stride_block;
  p.stride_head = c->stride_head;
  p.stride_slot = c->stride_slot;
  p.sc_stride_block = c->scale_stride_block;
  p.sc_stride_head = c->scale_stride_head;
  p.sc_stride_slot = c->scale_stride_slot;
  p.bt_stride = a->block_table_stride;
  p.batch = a->batch;
  p.n = a->q_per_seq;
  p.num_q_heads = a->num_q_heads;
  p.num_kv_heads = c->num_kv_heads;
  p.group = a->num_q_heads / c->num_kv_heads;
  p.rows = p.group * p.n;
  const Variant variant = pick_variant(c, a);
  // the many-row kernel moves tiles from global memory to LDS as they are: 16-bit caches only
  // (nor does head_dim 256: two row tiles of 256 elements per wave do not fit the registers)
  // (a 1-byte cache at head_dim 128 has a many-row kernel of its own, which converts the tiles in LDS)
  p.rows_per_item = !is_mfma(variant) ? 1
                    : (p.rows > kPrefillMinRows && variant != kMfmaD256 && (!quant || variant == kMfmaD128))
                        ? kPrefillRowsPerItem
                        : kMaxRowsPerItem;
  // More rows than one such item: 256 rows per item, eight waves in two groups that alternate between their
  // matrix and softmax phases (prefill_pingpong_d128_kernel; prefill_pingpong_quant_d128_kernel over a 1-byte cache).
  p.prefill_opts = (int32_t)option(XLLM_HIP_OPTION_PREFILL_KERNEL);
  // (head_dim 128: at head_dim 64 a tile is 64 tokens, and its scores and weights do not fit that kernel's registers)
  if (p.rows_per_item == kPrefillRowsPerItem && p.rows > kPrefillRowsPerItem && variant == kMfmaD128 &&
      (p.prefill_opts & 1) == 0) {
    p.rows_per_item = kPrefillWideRows;
  }
  p.min_chunk = is_mfma(variant) ? kMinChunkTokens : kMinChunkTokensGeneric;
  p.tok = variant == kMfmaD64 ? 2 : variant == kMfmaD256 ? 0 : 1;
  p.tile_tokens = variant == kMfmaD256 ? kTileTokens / 2 : kTileTokens * p.tok;
  p.row_groups = row_groups(a->q_per_seq, a->num_q_heads, c->num_kv_heads, p.rows_per_item);
  // The kv heads of a token lie side by side (the NHD layout: a head's row is followed by the next head's)
  // and a row is 128 bytes (1-byte cache): the 16-row kernel at head_dim 128 then takes work items of four
  // kv heads, one per wave, so that a workgroup reads runs of four rows instead of single rows a token's
  // width apart (fp8, 128 x 8192 tokens: 391 -> 338 us; HND 325).  Over a 16-bit cache, whose rows are 256
  // bytes, it measured the same as one head per item (166 us), so those keep the simpler form.
  // At head_dim 64 such rows are 64 bytes, two kv heads to a 128-byte line: there the waves of a workgroup should
  // attend neighbouring heads wherever they can, and walk their tokens in step (see DecodeParams::lockstep
  // below), whatever the sequences' lengths (int8, 14q/2kv, 512 x 16384 tokens: 542 us with four waves to a
  // head, against 349 in HND).
  const bool short_rows = variant == kMfmaD64 && quant && c->stride_head == c->head_dim && c->num_kv_heads > 1 &&
                          c->stride_slot >= (int64_t)c->num_kv_heads * c->head_dim;
  const bool side_by_side = ((variant == kMfmaD128 && quant && c->stride_head == c->head_dim &&
                              c->stride_slot >= (int64_t)c->num_kv_heads * c->head_dim) ||
                             short_rows) &&
                            option(XLLM_HIP_OPTION_DECODE_ITEM_PER_HEAD) == 0;
  // The same work items serve a large batch of short sequences in any layout, when the host-side lengths say
  // so: a wave that has a kv head's whole sequence to itself runs four times as many tiles between its
  // prologue and its epilogue as a wave with a quarter of it, and ends without the exchange between the four.
  // As long as such items fill every workgroup slot: over a 1-byte cache up to 8192 tokens per sequence in
  // the mean (fp8, 64 q heads: 2048 x 256 tokens 242 -> 203 us, 1024 x 512 211 -> 186, 256 x 2048 177 -> 167,
  // 256 x 6144 499 -> 492; int8 512 x 1024 198 -> 176; 128 x 8192, which gives 256 such items, 326 -> 333:
  // not those), over a 16-bit cache up to 192 (4096 x 64 tokens 264 -> 193 us, 2048 x 128 202 -> 182, 256 and more the same).
  // head_dim 64 likewise, a 16-bit cache up to 2048 tokens (14q/2kv: int8 2048 x 1024 tokens 112 -> 95 us, 4096 x 256
  // 88 -> 62; bf16 4096 x 128 69 -> 51, 2048 x 768 130 -> 127, 2048 tokens the same).
  // A ragged batch, whose long sequences are cut, has more of them to cut and to merge when an item is four
  // heads wide: it takes these items from four times as many on (lognormal lengths, fp8, per layer on an
  // existing schedule: 1024 sequences around 512 tokens 286 -> 243 us, 2048 around 256 336 -> 268, 1024 around
  // 1024 508 -> 454; 512 sequences around 1024 the same; 256 around 2048, 243 -> 270: not those).
  // Equal items run in rounds of as many workgroups as there are slots, and a workgroup that does the work of
  // four makes the last, partly filled round four times as long: 288 sequences of 2048 fp8 tokens x 8 kv heads
  // are 576 such workgroups, 1.125 rounds, 258 us against 202 as 2304 workgroups of one head each (4.5 rounds);
  // 320 sequences 261 against 219, 640 (2.5 rounds against 10) 443 against 432.  So for nearly equal lengths
  // the wider items are taken when (filled share of their rounds) x (their measured gain for the step's mean
  // length) beats the filled share of the narrow items' rounds.
  const int64_t four_head_items = (int64_t)p.batch * item_heads_of(p.rows, c->num_kv_heads, true);
  const int cus = device_cus();
  const int64_t slots = natural_target_items(true, p.rows, false, cus);
  const ShapeRules& R = kShapeRules;
  const bool nearly_equal = (int64_t)a->max_seq_len * p.batch * R.nearly_equal_den <= a->total_kv_len * R.nearly_equal_num;
  auto wider_items_pay = [&](int64_t narrow_items, int per_workgroup, double layout_gain = 0.0, bool narrow_cut = false) {
    auto filled = [&](int64_t workgroups) {
      if (workgroups <= 0) return 1.0;
      // (fewer than the slots: equal sequences are cut into as many chunks each as still fit)
      if (workgroups < slots) return (double)(workgroups * (slots / workgroups)) / (double)slots;
      const int64_t rounds = (workgroups + slots - 1) / slots;
      return (double)workgroups / (double)(rounds * slots);
    };
    const double mean = (double)a->total_kv_len / (double)(p.batch > 0 ? p.batch : 1);
    // gain of one wave per item over four, by mean length: 1-byte rows of 128 bytes 100 / L (19 % at 256 tokens,
    // 5 % at 2048), of 64 bytes 200 / L; 16-bit rows of 256 bytes 16 / L, of 128 bytes 25 / L
    const double k = variant == kMfmaD64 ? (quant ? R.wave_per_head_k_quant_d64 : R.wave_per_head_k_16bit_d64)
                                         : (quant ? R.wave_per_head_k_quant : R.wave_per_head_k_16bit);
    double gain = k / (mean > 1.0 ? mean : 1.0);
    const double cap = quant ? (variant == kMfmaD64 ? R.wave_per_head_cap_quant_d64 : R.wave_per_head_cap_quant) : R.wave_per_head_cap_16bit;
    gain = gain < cap ? gain : cap;
    if (per_workgroup == 2) gain *= 0.5;
    gain += layout_gain;
    // (narrow items whose last round's sequences are cut fill their rounds but for the merges)
    const double narrow_filled = narrow_cut ? R.cut_rounds_filled : filled(narrow_items);
    return filled((narrow_items + per_workgroup - 1) / per_workgroup) * (1.0 + gain) > narrow_filled * R.wider_items_hurdle;
  };
  const bool short_sequences = (variant == kMfmaD128 || variant == kMfmaD64) && a->max_seq_len > 0 && a->total_kv_len > 0 &&
                               four_head_items >= (nearly_equal ? slots : 4 * slots) &&
                               (short_rows || a->total_kv_len <= (int64_t)p.batch * (quant ? R.wave_per_head_max_mean_quant : variant == kMfmaD64 ? R.wave_per_head_max_mean_d64 : R.wave_per_head_max_mean_16bit)) &&
                               (!nearly_equal || wider_items_pay((int64_t)p.batch * c->num_kv_heads, kHeadsPerItem)) &&
                               option(XLLM_HIP_OPTION_DECODE_ITEM_PER_HEAD) == 0;
  // (the four-head items of a 1-byte cache with its heads side by side gain 16 % from the layout alone, 391 -> 338
  // us: they too give way where their rounds would be poorly filled and the host-side lengths show it)
  const bool side_by_side_pays = !(a->max_seq_len > 0 && a->total_kv_len > 0 && nearly_equal) ||
                                 wider_items_pay((int64_t)p.batch * c->num_kv_heads, kHeadsPerItem, short_rows ? R.short_rows_gain : R.side_by_side_gain);
  p.item_heads = item_heads_of(p.rows, c->num_kv_heads, (side_by_side && side_by_side_pays) || short_sequences);
  // 17 to 32 rows per kv head over such a cache (the heads side by side, rows of 128 bytes): the 32-row kernel's
  // form of the four-head item, eight waves to the workgroup and one workgroup to a CU.
  const bool side_by_side32 = side_by_side && variant == kMfmaD128 && p.rows > 16 && p.rows <= kMaxRowsPerItem && p.rows_per_item == kMaxRowsPerItem;
  if (side_by_side32) p.item_heads = item_heads_of(p.rows, c->num_kv_heads, true, true);
  p.heads_per_item = c->num_kv_heads / p.item_heads;
  p.head_dim = c->head_dim;
  p.block_size = c->block_size;
  p.log2_bs = is_pow2(c->block_size) ? ilog2(c->block_size) : 0;
  p.max_blocks_per_seq = a->max_blocks_per_seq;
  p.last_block = c->num_blocks - 1 < INT32_MAX ? (int32_t)(c->num_blocks - 1) : INT32_MAX;
  {
    const int64_t cap = (int64_t)a->max_blocks_per_seq * c->block_size;
    p.len_cap = a->block_table != nullptr && cap < INT32_MAX ? (int32_t)cap : INT32_MAX;
  }
  p.window_left = a->window_left;
  // head_dim 256 runs one wave per SIMD (registers), so half as many workgroups are resident — except the
  // 32-row kernel over a 1-byte cache, which fits two
  const bool one_wave_per_simd = variant == kMfmaD256 && !(p.rows > 16 && quant);
  p.target_items = target_items(is_mfma(variant), p.rows, one_wave_per_simd);
  // (the 32-row kernel's four-head items: one workgroup of eight waves per CU where four of two waves are)
  if (side_by_side32 && p.heads_per_item > 1) p.target_items = p.target_items / kHeadsPerItem > 0 ? p.target_items / kHeadsPerItem : 1;
  // A small batch on the 16-row kernel: one of the two workgroups a CU holds (the 32-row kernel wants
  // all its slots filled: 4 x 32768 tokens of int8 with 4 draft tokens, 65 us at 1024 items, 84 at 512).
  // (work items of four kv heads keep every slot as the target: each of their waves streams a head of its own,
  // so one workgroup per CU would leave half of the loads in flight that two do)
  p.target_small = is_mfma(variant) && p.rows <= 16 && !one_wave_per_simd && p.heads_per_item == 1 ? p.target_items / 2
                                                                                                : p.target_items;
  // ... except over a 1-byte cache, where four waves have half as many bytes in flight per tile and do not
  // saturate a CU's share of HBM (fp8, 16 x 8192 tokens: 65 us at 256 items, 55 at 512): every slot, as long
  // as that cuts a sequence into at most the 32 chunks the in-kernel merge loads in one batch (one
  // 32768-token sequence: 31 us at 256 items, 38 at 512).  Better still is one workgroup of eight waves per
  // CU (wide_items below), which needs the launch's size to be known here.
  const int32_t target_one_per_cu = p.target_small;
  if (quant && p.target_small < p.target_items) {
    const int64_t triples = (int64_t)p.batch * p.item_heads * p.row_groups;
    const int64_t cap = R.fused_merge_max_chunks * triples;
    p.target_small = (int32_t)(cap >= p.target_items ? p.target_items : cap > p.target_small ? cap : p.target_small);
  }
  // Only the MFMA kernel finishes single-chunk sequences itself.  When the caller's host-side
  // lengths (the reference keeps both in AttentionMetadata) show that the chunk the plan would
  // pick covers the longest sequence, no sequence is split: the plan is told never to split
  // (which stays correct even if the hints were wrong) and the merge launch is dropped.
  p.direct_single = is_mfma(variant) ? 1 : 0;
  // Up to 16 rows per kv head the attention kernel merges split sequences itself (no merge launch).
  // With more rows the work of a merge is large enough to want the whole GPU: fused into the 32-row
  // kernel it made the int8 verify workload 7 % slower (401 against 377 us), the tails of all row
  // groups ending together.
  // Nor with work items of four kv heads: the workgroup that finishes last would merge four heads' rows, each
  // wave its head's one after the other (fp8, 8 rows per kv head: 356 us fused against 338 with the merge kernel).
  p.fused_merge = is_mfma(variant) && p.rows <= 16 && p.heads_per_item == 1 &&
                          option(XLLM_HIP_OPTION_DECODE_SEPARATE_MERGE) == 0
                      ? 1
                      : 0;
  const bool hints = a->max_seq_len > 0 && a->total_kv_len > 0;
  const bool stay_whole = never_split(a->q_per_seq, a->num_q_heads, c->num_kv_heads);
  auto decide = [&]() {
    p.fixed_chunk = 0;
    // (not a ragged batch of more items than run at once: as whole sequences in index order its long sequences
    // start whenever their turn comes, the last of them alone at the end; the stored schedule runs them first —
    // lognormal lengths, sigma 0.8, per layer: 256 sequences around 8192 fp8 tokens 1125 us whole in index order,
    // 830 from the stored schedule; around 2048 bf16 tokens 495 against 422; 1024 around 2048 int8 1153 against 884)
    const int64_t triples = (int64_t)p.batch * p.item_heads * p.row_groups;
    if (p.direct_single && hints && (nearly_equal || triples <= p.target_items) &&
        a->max_seq_len <= choose_chunk(a->total_kv_len, a->max_seq_len, p.batch, p.item_heads, p.row_groups,
                                       p.target_items, p.target_small, p.min_chunk, p.tile_tokens)) {
      p.fixed_chunk = 1 << 30;
    }
    // Many query rows per kv head (chunked prefill): the row groups supply the parallelism, and one
    // partial per chunk and row would be large, so nothing is split.
    if (stay_whole) p.fixed_chunk = 1 << 30;
    // (a step that is never split is whole sequences for the generic kernel too: it then writes the rows itself)
    p.implicit_plan = (p.direct_single || stay_whole) && p.fixed_chunk == (1 << 30) ? 1 : 0;
    // A split step whose host-side lengths are (nearly) equal needs no stored schedule: with the chunk
    // size the device-side plan would choose from the same aggregates, every sequence owns
    // ceil(max_seq_len / chunk) chunk slots and a work item finds its chunk from its index and the
    // sequence's length.  No plan kernel runs, and the item's block list, queries and length are
    // independent loads.  Not for ragged batches: the slots of the shorter sequences would be empty
    // workgroups (at most a quarter of them may be), and the tails would not be ordered by size.
    p.arith_chunks = 0;
    if (p.fixed_chunk == 0 && hints && option(XLLM_HIP_OPTION_DECODE_STORED_SCHEDULE) == 0) {
      const int c = choose_chunk(a->total_kv_len, a->max_seq_len, p.batch, p.item_heads, p.row_groups, p.target_items,
                                 p.target_small, p.min_chunk, p.tile_tokens);
      const int64_t per_seq = ((int64_t)a->max_seq_len + c - 1) / c;
      if (per_seq * p.batch <= w.max_seq_chunks && per_seq * p.batch <= INT32_MAX &&
          (int64_t)a->max_seq_len * p.batch * 4 <= a->total_kv_len * 5) {
        p.fixed_chunk = c;
        p.arith_chunks = (int32_t)per_seq;
      }
    }
  };
  // Over a 1-byte cache the 16-row kernel also comes with eight waves per work item, one such workgroup to a
  // CU (launch_mfma_tok): with the host-side lengths the launch's size is known here, and a step that can be
  // cut into at most one item per CU is (fp8, 64 q heads: 32 x 8192 tokens 94 -> 87 us, 2 x 32768 40 -> 33,
  // 3 x 20000 36 -> 31; int8 with two draft tokens, 32 x 32768: 341 -> 326) — unless that leaves over a
  // quarter of the CUs without an item (20 x 8192 tokens of fp8: 69 us as 160 items, 65 as 480 in every slot).
  const bool wide_items = quant && is_mfma(variant) && variant != kMfmaD256 && p.rows <= 16 && p.heads_per_item == 1 &&
                          hints && option(XLLM_HIP_OPTION_DECODE_FOUR_WAVE_ITEMS) == 0;
  bool decided = false;
  if (wide_items && target_one_per_cu < p.target_small) {
    const int32_t every_slot = p.target_small;
    p.target_small = target_one_per_cu;
    decide();
    const int64_t items = (p.implicit_plan ? (int64_t)p.batch : (int64_t)p.batch * p.arith_chunks) * p.item_heads * p.row_groups;
    decided = (p.implicit_plan || p.arith_chunks > 0) && items <= cus && items * R.eight_waves_min_den >= (int64_t)cus * R.eight_waves_min_num;
    if (!decided) p.target_small = every_slot;
  }
  if (!decided) decide();
  // Equal items beyond whole rounds of the slots: 66 sequences x 8 kv heads are 528 work items for 512 slots,
  // and the 16 of the second round take as long as the 512 of the first (fp8, 8192 tokens: 255 us against 167
  // for 64 sequences).  The sequences of the last, partly filled round are therefore cut into as many chunks
  // as fill the slots once more — 2 sequences x 8 heads x 32 chunks — while the others stay whole (arith_whole):
  // the last round then takes a fraction of a whole one.
  p.arith_whole = 0;
  p.arith_first = 0;
  p.first_chunk = 1 << 30;
  p.eight_waves = 0;
  // (the 32-row kernel over a 1-byte cache as well — int8, four draft tokens, 32768 tokens x 8 kv heads: 66 sequences
  // 996 us where 64 take 709 —, there also from a step that is already cut evenly, `uniform` chunks a sequence)
  const bool rows32 = p.rows > 16 && p.rows <= kMaxRowsPerItem && p.rows_per_item == kMaxRowsPerItem;
  const int64_t uniform = p.implicit_plan ? 1 : (rows32 && p.arith_chunks > 0 ? p.arith_chunks : 0);
  if (is_mfma(variant) && ((p.rows <= 16 && p.fused_merge && p.implicit_plan) || (rows32 && uniform > 0)) &&
      p.heads_per_item == 1 && hints && nearly_equal && option(XLLM_HIP_OPTION_DECODE_STORED_SCHEDULE) == 0) {
    const int64_t per = (int64_t)p.item_heads * p.row_groups;
    const int64_t items = (int64_t)p.batch * per;
    // A round: an item per CU for a 16-bit cache.  What has to balance there is the bytes a CU streams, not
    // the slots it fills: 33 sequences x 8 kv heads, 264 items of 8192 bf16 tokens, all resident at once, take
    // 228 us where 256 take 159 — eight CUs stream two items.  Over a 1-byte cache a CU wants two workgroups
    // to stream at its full rate, so a round is every slot, and a step of fewer items than slots (but more
    // than the 256 that eight-wave workgroups serve) is first cut in two throughout.
    // ... or, while the items are at most a quarter more than the CUs, runs eight waves per item like a step of
    // up to 256 items: a round is then an item per CU, the sequences past it are cut, and their chunks follow the
    // whole items onto the CUs (fp8, 8192 tokens x 8 kv heads: 33 sequences 105 us cut in two throughout)
    const bool eight = quant && p.rows <= 16 && p.tok != 0 && uniform == 1 && items > cus && items * R.eight_waves_over_den <= (int64_t)cus * R.eight_waves_over_num &&
                       option(XLLM_HIP_OPTION_DECODE_FOUR_WAVE_ITEMS) == 0;
    const int64_t round = eight ? cus : quant || one_wave_per_simd ? p.target_items : cus;
    // chunks of the sequences that stay as they are: the even cut the step has, or one more when that cut fills
    // less than nine tenths of a round
    const int64_t first = !eight && quant && uniform * items < round && uniform * items * R.round_fill_den < round * R.round_fill_num ? uniform + 1 : uniform;
    const int64_t whole_rounds = first * items / round;
    // (from 2048 items on the last round weighs little: 288 x 2048 fp8 tokens x 8 kv heads 202 us whole, 206 cut)
    if (whole_rounds >= 1 && items < (int64_t)R.cut_last_round_below_rounds * p.target_items && (first * items) % round != 0) {
      const int64_t whole_seqs = whole_rounds * round / (per * first);
      const int64_t cut_seqs = p.batch - whole_seqs;
      int64_t k = round / (cut_seqs * per);
      k = k > R.fused_merge_max_chunks ? R.fused_merge_max_chunks : k;  // (what the fused merge loads in one batch)
      // (bf16, 4096 tokens x 8 kv heads: 66 sequences 192 -> 167 us, 72 196 -> 185, 80, two chunks, 204 -> 206;
      // 8192 tokens: 33 sequences 228 -> 168, 40 237 -> 203, 44 242 -> 220, 48 247 -> 240.  fp8, 8192 tokens: 66
      // sequences 255 -> 179, 80 260 -> 217, 96 277 -> 258, 136 413 -> 359)
      auto chunk_for = [&](int64_t parts) {
        int64_t c = ((int64_t)a->max_seq_len + parts - 1) / parts;
        c = (c + p.tile_tokens - 1) / p.tile_tokens * p.tile_tokens;
        return c < p.min_chunk ? (int64_t)p.min_chunk : c;
      };
      const int64_t chunk1 = first > 1 ? chunk_for(first) : (int64_t)1 << 30;
      const int64_t k1 = first > 1 ? ((int64_t)a->max_seq_len + chunk1 - 1) / chunk1 : 1;
      // (no more chunks than the workspace holds partial rows for)
      const int64_t room = (w.max_seq_chunks - whole_seqs * k1) / cut_seqs;
      k = k > room ? room : k;
      const int64_t chunk = chunk_for(k > 1 ? k : 1);
      k = ((int64_t)a->max_seq_len + chunk - 1) / chunk;
      // (cut in two throughout, every sequence is merged: that pays while the last round's are few — fp8, 8192 tokens
      // x 8 kv heads, 33 sequences 129 -> 105 us, 40 132 -> 122, but 48, whose last 16 get four chunks each, 136 -> 144)
      if (k > k1 && (first == 1 || k >= R.last_round_min_ratio * k1) && whole_seqs * k1 + cut_seqs * k <= w.max_seq_chunks) {
        p.fixed_chunk = (int32_t)chunk;
        p.arith_chunks = (int32_t)k;
        p.arith_whole = (int32_t)whole_seqs;
        p.arith_first = (int32_t)k1;
        p.first_chunk = (int32_t)chunk1;
        p.implicit_plan = 0;
        p.eight_waves = eight ? 1 : 0;
      }
    }
  }
  // Many short sequences when the kv heads are no multiple of four (a tensor-parallel shard's one or two):
  // four neighbouring work items to a workgroup, one per wave, for the same reason as the four-head items
  // above.  The step is then not split at all (its items fill every slot four times over), which is why
  // nearly equal lengths are asked for.  With half as many items (from 1024 on, any head count) two waves
  // share an item and a workgroup takes two (fp8, 128 sequences of 2048 tokens x 8 kv heads: 89.5 -> 86.4 us;
  // 192 sequences, 1.5 rounds of such workgroups, would take 148 against 134: see wider_items_pay).
  p.wave_items = 0;
  if ((variant == kMfmaD128 || variant == kMfmaD64) && p.rows <= 16 && p.heads_per_item == 1 && hints && nearly_equal &&
      (short_rows || a->total_kv_len <= (int64_t)p.batch * (quant ? R.wave_per_head_max_mean_quant : variant == kMfmaD64 ? R.wave_per_head_max_mean_d64 : R.wave_per_head_max_mean_16bit)) &&
      option(XLLM_HIP_OPTION_DECODE_ITEM_PER_HEAD) == 0) {
    const int64_t items = (int64_t)p.batch * c->num_kv_heads;
    // (64-byte rows, see short_rows: two waves to an item from one round of items on, if that leaves more workgroups than
    // CUs — int8, 14q/2kv over NHD, 400 x 4096 tokens 111 -> 102 us, 500 x 2048 65 -> 59; 256 x 8192, a workgroup per CU, 130 -> 133)
    const int per_group = items >= kHeadsPerItem * slots ? 1
                          : items >= 2 * slots || (short_rows && items >= slots && items / 2 > cus) ? 2
                                                                                                     : 0;
    if (per_group != 0 && wider_items_pay(items, per_group == 1 ? kWaves : 2, short_rows ? R.short_rows_gain : 0.0, p.arith_whole > 0)) {
      p.wave_items = per_group;
      p.fixed_chunk = 1 << 30;
      p.implicit_plan = 1;
      p.arith_chunks = 0;
      p.arith_whole = 0;
    }
  }
  // 64-byte rows whose kv heads come in pairs but not in fours (short_rows; a tensor-parallel shard's two), in a
  // step that keeps its schedule, split or ragged: the same workgroups of two items, two waves each, over the
  // schedule's items as they are — neighbours 2j and 2j + 1 in their order are a chunk's kv heads 2j and 2j + 1, the
  // two halves of the same lines — and split sequences go to the merge kernel, as those of four-head items do.
  // From a round of items on, more workgroups than CUs (a small batch keeps eight waves to an item).  int8, 14q/2kv
  // over NHD: 300 x 12000 tokens 235 -> 216 us (HND 163), 272 x 8192 150 -> 144, 260 x 16384 277 -> 268; lognormal
  // lengths, 512 sequences around 4096 tokens 194 -> 192, 1024 around 512 75 -> 73.
  if (p.wave_items == 0 && short_rows && p.rows <= 16 && p.heads_per_item == 1 && c->num_kv_heads % 2 == 0 &&
      (int64_t)p.batch * c->num_kv_heads >= slots && (int64_t)p.batch * c->num_kv_heads / 2 > cus &&
      option(XLLM_HIP_OPTION_DECODE_ITEM_PER_HEAD) == 0) {
    p.wave_items = 2;
    p.fused_merge = 0;
    p.eight_waves = 0;
  }
  // XCD clusters: the row groups of a (chunk, kv head); and the kv heads whose rows share 128-byte
  // lines — scale rows shorter than a line (HND: block_size * 4 bytes per head; NHD: the heads of a
  // slot are adjacent floats) or cache rows shorter than a line (NHD with 64 one-byte elements).
  int heads_per_line = 1;
  {
    auto shared_by = [](int64_t head_stride_bytes) {
      return head_stride_bytes > 0 && head_stride_bytes < 128 ? (int)(128 / head_stride_bytes) : 1;
    };
    heads_per_line = shared_by(c->stride_head * elem_bytes(c->dtype));
    if (quant) heads_per_line = max(heads_per_line, shared_by(c->scale_stride_head * 4));
    // Cache rows shorter than a line, and waves of a workgroup that attend neighbouring kv heads (1-byte caches at
    // head_dim 64 over NHD): the waves walk their tokens in step, a barrier per tile, and load with ordinary loads
    // instead of streaming ones, so that the halves of a line are asked for together — the second from the CU's
    // cache — and cross HBM once.  int8, 2 kv heads, 512 x 8192 tokens: 1.60x the algorithmic bytes fetched and
    // 265 us as independent waves, 225 us in step (1.13x), 209 us with ordinary loads as well (HND 173); fp8
    // 266 -> 206; 8 kv heads, 128 x 8192 tokens 314 -> 253 us, 1024 x 1024 tokens 268 -> 237.  Rows of a whole
    // line gain nothing from it and lose the waves' independence (fp8, head_dim 128, 128 x 8192 tokens over
    // NHD: 350 -> 365 us): not those.
    p.lockstep = (p.wave_items || p.heads_per_item > 1) && short_rows ? 1 : 0;
    if (heads_per_line > c->num_kv_heads) heads_per_line = c->num_kv_heads;
    while (heads_per_line > 1 && c->num_kv_heads % heads_per_line != 0) --heads_per_line;
  }
  // (in work items: an item of four heads covers that many of the line's heads itself)
  int items_per_line = (heads_per_line + p.heads_per_item - 1) / p.heads_per_item;
  while (items_per_line > 1 && p.item_heads % items_per_line != 0) --items_per_line;
  p.cluster = p.wave_items ? 1 : p.row_groups * items_per_line;
  p.q_dtype = a->q_dtype;
  p.scale_log2 = a->sm_scale * 1.4426950408889634f;
  return XLLM_HIP_OK;
}

// Upper bound of the work-item count for any lengths (see workspace_layout).
static int64_t max_items(const DecodeParams& p) {
  const int64_t per = (int64_t)p.item_heads * p.row_groups;
  int64_t seq_chunks = p.batch;
  if (p.arith_chunks > 0) {
    seq_chunks = (int64_t)p.arith_whole * p.arith_first + (int64_t)(p.batch - p.arith_whole) * p.arith_chunks;
  } else if (p.fixed_chunk != (1 << 30)) {
    int64_t t = 2 * (int64_t)p.target_items;  // choose_chunk may raise the target (by a quarter)
    if (t > kMaxTargetItems) t = kMaxTargetItems;
    seq_chunks = t / per + p.batch + 1;
  }
  int64_t items = seq_chunks * per;
  if (p.cluster > 1) {  // whole clusters, eight at a time (see decode_item)
    const int64_t clusters = (items + p.cluster - 1) / p.cluster;
    items = (clusters + kXcds - 1) / kXcds * kXcds * p.cluster;
  }
  if (p.wave_items == 1) items = (items + kWaves - 1) / kWaves;  // four of them to a workgroup
  if (p.wave_items == 2) items = (items + 1) / 2;
  return items;
}

template <int KV_DT, int TOK>
static void launch_mfma_tok(const DecodeParams& p, unsigned grid, hipStream_t st) {
  if (p.rows_per_item == kPrefillWideRows) {
    if constexpr (!quant_of(KV_DT) && TOK == 1) prefill_pingpong_d128_kernel<KV_DT, TOK><<<grid, 512, 0, st>>>(p);
    if constexpr (quant_of(KV_DT) && TOK == 1) prefill_pingpong_quant_d128_kernel<KV_DT><<<grid, 512, 0, st>>>(p);
  } else if (p.rows_per_item == kPrefillRowsPerItem) {
    if constexpr (!quant_of(KV_DT) && TOK != 0) prefill_mfma_d128_kernel<KV_DT, TOK><<<grid, 256, 0, st>>>(p);
    if constexpr (quant_of(KV_DT) && TOK == 1) prefill_quant_d128_kernel<KV_DT><<<grid, 256, 0, st>>>(p);
  } else if (p.rows <= 16) {
    if constexpr (TOK != 0) {
      if (p.heads_per_item > 1 || p.wave_items) {
        if constexpr (TOK == 2 && quant_of(KV_DT)) {  // (the one shape whose rows are shorter than a line)
          if (p.lockstep) {
            decode_mfma_d128_kernel<KV_DT, TOK, true, kWaves, true><<<grid, 64 * kWaves, 0, st>>>(p);
            return;
          }
        }
        decode_mfma_d128_kernel<KV_DT, TOK, true><<<grid, 64 * kWaves, 0, st>>>(p);
        return;
      }
    }
    if constexpr (TOK != 0 && quant_of(KV_DT)) {
      // At most one work item per CU over a 1-byte cache: eight waves share it (one 32768-token sequence:
      // 25 us against 31 for fp8, 26 against 32 for int8; over a 16-bit cache, whose tiles take no
      // conversion, 31.7 against 31.0).
      if ((grid <= (unsigned)device_cus() || p.eight_waves) && option(XLLM_HIP_OPTION_DECODE_FOUR_WAVE_ITEMS) == 0) {
        decode_mfma_d128_kernel<KV_DT, TOK, false, 2 * kWaves><<<grid, 128 * kWaves, 0, st>>>(p);
        return;
      }
    }
    decode_mfma_d128_kernel<KV_DT, TOK><<<grid, 64 * kWaves, 0, st>>>(p);
  } else {
    if constexpr (TOK == 1 && quant_of(KV_DT)) {
      if (p.heads_per_item > 1) {
        decode_mfma_d128_rows32_kernel<KV_DT, TOK, kHeadsPerItem><<<grid, 128 * kHeadsPerItem, 0, st>>>(p);
        return;
      }
    }
    decode_mfma_d128_rows32_kernel<KV_DT, TOK><<<grid, 128, 0, st>>>(p);
  }
}

template <int KV_DT>
static void launch_mfma(const DecodeParams& p, unsigned grid, hipStream_t st) {
  if (p.tok == 2) {
    launch_mfma_tok<KV_DT, 2>(p, grid, st);
  } else if (p.tok == 0) {
    launch_mfma_tok<KV_DT, 0>(p, grid, st);
  } else {
    launch_mfma_tok<KV_DT, 1>(p, grid, st);
  }
}

template <int Q_DT>
static int launch_generic(int kv_dtype, const DecodeParams& p, unsigned grid, hipStream_t st) {
  switch (kv_dtype) {
    case XLLM_HIP_BF16:
      decode_generic_kernel<Q_DT, XLLM_HIP_BF16><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP16:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP16><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP32:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP32><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_FP8_E4M3:
      decode_generic_kernel<Q_DT, XLLM_HIP_FP8_E4M3><<<grid, 64, 0, st>>>(p);
      break;
    case XLLM_HIP_INT8:
      decode_generic_kernel<Q_DT, XLLM_HIP_INT8><<<grid, 64, 0, st>>>(p);
      break;
    default:
      return fail(XLLM_HIP_UNSUPPORTED, "no decode kernel for cache dtype %d", kv_dtype);
  }
  return XLLM_HIP_OK;
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" int xllm_hip_paged_decode_describe(const xllm_hip_kv_cache* cache,
                                              const xllm_hip_decode_args* args,
                                              size_t workspace_bytes,
                                              int64_t* out,
                                              int32_t count) {
  XLLM_HIP_REQUIRE(out != nullptr && count >= 0, "out is NULL or count negative");
  XLLM_HIP_REQUIRE(cache != nullptr && args != nullptr, "cache or args is NULL");
  if (workspace_bytes == 0) {
    workspace_bytes = workspace_layout(args->batch, args->q_per_seq, args->num_q_heads, cache->num_kv_heads,
                                       cache->head_dim, device_cus()).total_bytes;
  }
  DecodeParams p;
  // (a workspace address that is never read: every field of it the host forms is an offset from it)
  if (int s = fill_params(cache, args, (void*)(uintptr_t)4096, workspace_bytes, p)) return s;
  const Variant v = pick_variant(cache, args);
  XLLM_HIP_REQUIRE(v != kNone, "no decode kernel for head_dim=%d block_size=%d", cache->head_dim, cache->block_size);
  const int64_t grid = p.batch == 0 ? 0 : max_items(p);
  const bool quant = cache->dtype == XLLM_HIP_FP8_E4M3 || cache->dtype == XLLM_HIP_INT8;
  int64_t waves = 1, per_workgroup = 1;
  if (is_mfma(v)) {
    if (p.rows_per_item == kPrefillWideRows) {
      waves = 8;
    } else if (p.rows_per_item == kPrefillRowsPerItem) {
      waves = 4;
    } else if (p.rows > 16) {
      waves = p.heads_per_item > 1 ? 2 * kHeadsPerItem : 2;
    } else if (p.heads_per_item > 1 || p.wave_items) {
      waves = 4;
      per_workgroup = p.wave_items == 2 ? 2 : (p.wave_items == 1 ? 4 : 1);
    } else {
      const bool eight = quant && p.tok != 0 && (grid <= device_cus() || p.eight_waves) &&
                         option(XLLM_HIP_OPTION_DECODE_FOUR_WAVE_ITEMS) == 0;
      waves = eight ? 8 : 4;
    }
  }
  const bool stored = !p.implicit_plan && p.arith_chunks == 0;
  const int64_t slots_used = p.implicit_plan ? 0
                             : p.arith_chunks > 0
                                 ? (int64_t)p.arith_whole * p.arith_first + (int64_t)(p.batch - p.arith_whole) * p.arith_chunks
                                 : (int64_t)p.max_seq_chunks;
  const int64_t values[14] = {grid,
                              waves,
                              p.implicit_plan,
                              stored ? 1 : 0,
                              p.implicit_plan || p.fixed_chunk == (1 << 30) ? 0 : p.fixed_chunk,
                              p.arith_chunks,
                              p.arith_whole,
                              p.arith_whole > 0 ? p.arith_first : 0,
                              p.arith_whole > 0 && p.first_chunk != (1 << 30) ? p.first_chunk : 0,
                              p.heads_per_item,
                              per_workgroup,
                              p.fused_merge && !p.implicit_plan ? 1 : 0,
                              p.max_seq_chunks,
                              slots_used};
  for (int i = 0; i < count && i < 14; ++i) out[i] = values[i];
  return XLLM_HIP_OK;
}

extern "C" size_t xllm_hip_paged_decode_workspace_bytes(int32_t batch,
                                                        int32_t q_per_seq,
                                                        int32_t num_q_heads,
                                                        int32_t num_kv_heads,
                                                        int32_t head_dim) {
  if (batch < 0 || q_per_seq < 1 || num_q_heads < 1 || num_kv_heads < 1 || head_dim < 1) return 0;
  return workspace_layout(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim, device_cus()).total_bytes;
}

extern "C" int xllm_hip_set_option(int32_t which, int64_t value) {
  XLLM_HIP_REQUIRE(which >= 0 && which < XLLM_HIP_OPTION_COUNT, "unknown option %d", which);
  options().v[which].store(value, std::memory_order_relaxed);
  return XLLM_HIP_OK;
}

extern "C" int64_t xllm_hip_get_option(int32_t which) {
  return which >= 0 && which < XLLM_HIP_OPTION_COUNT ? option(which) : -1;
}

extern "C" const char* xllm_hip_paged_decode_variant(const xllm_hip_kv_cache* cache,
                                                     const xllm_hip_decode_args* args) {
  if (cache == nullptr || args == nullptr) return "";
  switch (pick_variant(cache, args)) {
    case kMfmaD128:
      return "mfma_d128";
    case kMfmaD64:
      return "mfma_d64";
    case kMfmaD256:
      return "mfma_d256";
    case kGeneric:
      return "generic";
    default:
      return "";
  }
}

extern "C" int xllm_hip_paged_decode_plan(const xllm_hip_kv_cache* cache,
                                          const xllm_hip_decode_args* args,
                                          void* workspace,
                                          size_t workspace_bytes,
                                          xllm_hip_stream_t stream) {
  DecodeParams p;
  if (int s = fill_params(cache, args, workspace, workspace_bytes, p)) return s;
  if (p.batch == 0 || p.implicit_plan) return XLLM_HIP_OK;  // an unsplit step needs no schedule
  if (p.arith_chunks > 0) {
    // nor does one whose work items find their chunks themselves; the counters of the fused merge
    // still start the step at zero
    if (!p.fused_merge) return XLLM_HIP_OK;
    const int ncounters = p.batch * p.num_kv_heads * p.row_groups;
    decode_zero_counters_kernel<<<(unsigned)((ncounters + 255) / 256), 256, 0, (hipStream_t)stream>>>(p.counters,
                                                                                                   ncounters);
    return check_launch("decode_zero_counters_kernel");
  }
  decode_plan_kernel<<<1, 64, 0, (hipStream_t)stream>>>(p);
  return check_launch("decode_plan_kernel");
}

extern "C" size_t xllm_hip_paged_decode_plan_host_bytes(int32_t batch,
                                                        int32_t q_per_seq,
                                                        int32_t num_q_heads,
                                                        int32_t num_kv_heads,
                                                        int32_t head_dim) {
  if (batch < 0 || q_per_seq < 1 || num_q_heads < 1 || num_kv_heads < 1 || head_dim < 1) return 0;
  return workspace_layout(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim, device_cus()).partial_lse;  // header .. last record
}

extern "C" int xllm_hip_paged_decode_plan_host(const xllm_hip_kv_cache* cache,
                                               const xllm_hip_decode_args* args,
                                               const int32_t* host_kv_lens,
                                               void* workspace,
                                               size_t workspace_bytes,
                                               void* host_staging,
                                               size_t host_staging_bytes,
                                               xllm_hip_stream_t stream,
                                               int64_t* info) {
  XLLM_HIP_REQUIRE(args != nullptr && args->host_plan != 0, "args->host_plan must be set for a plan made on the host");
  DecodeParams p;
  if (int s = fill_params(cache, args, workspace, workspace_bytes, p)) return s;
  if (info != nullptr) info[0] = info[1] = info[2] = 0;
  if (p.batch == 0 || p.implicit_plan) return XLLM_HIP_OK;  // a step that is never split needs no schedule
  XLLM_HIP_REQUIRE(host_kv_lens != nullptr && host_staging != nullptr, "host_kv_lens or host_staging is NULL");
  XLLM_HIP_REQUIRE(p.arith_chunks == 0 && p.fixed_chunk == 0, "a step with a plan made on the host keeps a stored schedule");
  const WorkspaceLayout w =
      workspace_layout(args->batch, args->q_per_seq, args->num_q_heads, cache->num_kv_heads, cache->head_dim, device_cus());
  if (host_staging_bytes < w.partial_lse) {
    return fail(XLLM_HIP_WORKSPACE_TOO_SMALL, "host_staging has %zu bytes, need %zu", host_staging_bytes, w.partial_lse);
  }
  const bool quant = cache->dtype == XLLM_HIP_FP8_E4M3 || cache->dtype == XLLM_HIP_INT8;
  const Variant v = pick_variant(cache, args);
  HostScheduleInput in;
  in.kv_lens = host_kv_lens;
  in.batch = p.batch;
  in.len_cap = p.len_cap;
  in.per = p.item_heads * p.row_groups;
  in.slots = p.target_items;  // the workgroups the GPU holds at once
  in.tile = p.tile_tokens;
  in.min_chunk = p.min_chunk;
  in.max_seq_chunks = max_items(p) / in.per;  // what the launch covers
  in.max_per_seq = p.fused_merge ? 32 : 256;  // what a merge loads in one batch
  {
    // Costs in tokens of a slot's streaming (6.5 TB/s over the slots; a token of one kv head is K, V and scales):
    // four microseconds per work item; a step that cuts sequences ends with a merge of five microseconds and
    // 0.15 per chunk.  A CU holds two workgroups of the 16-row kernel: over a 16-bit cache one of them alone
    // already streams at the CU's full rate, over a 1-byte cache at about two thirds of it (see choose_chunk).
    const double bytes_per_token = 2.0 * cache->head_dim * elem_bytes(cache->dtype) * p.heads_per_item + (quant ? 8.0 : 0.0);
    const double tokens_per_us = 6.5e6 / ((double)in.slots * bytes_per_token);
    in.item_overhead = 4.0 * tokens_per_us;
    in.merge_base = 5.0 * tokens_per_us;
    in.merge_per_chunk = 0.15 * tokens_per_us;
    in.solo_speedup = !is_mfma(v) || p.rows > 16 ? 1.0 : quant ? 1.3 : 2.0;
  }
  HostScheduleResult r;
  if (!host_schedule(in, w, (uint8_t*)host_staging, host_staging_bytes, r)) {
    return fail(XLLM_HIP_INVALID_ARGUMENT, "the step's chunks do not fit the workspace (batch %d, %lld records)", p.batch,
                (long long)in.max_seq_chunks);
  }
  if (info != nullptr) {
    info[0] = r.chunk_target;
    info[1] = r.total_chunks;
    info[2] = (int64_t)r.predicted_span;
  }
  if (hipMemcpyAsync(workspace, host_staging, r.bytes, hipMemcpyHostToDevice, (hipStream_t)stream) != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipMemcpyAsync of the schedule failed");
  }
  if (p.fused_merge) {
    const int ncounters = p.batch * p.num_kv_heads * p.row_groups;
    decode_zero_counters_kernel<<<(unsigned)((ncounters + 255) / 256), 256, 0, (hipStream_t)stream>>>(p.counters, ncounters);
    return check_launch("decode_zero_counters_kernel");
  }
  return XLLM_HIP_OK;
}

extern "C" int xllm_hip_paged_decode_run(const xllm_hip_kv_cache* cache,
                                         const xllm_hip_decode_args* args,
                                         void* workspace,
                                         size_t workspace_bytes,
                                         xllm_hip_stream_t stream) {
  return xllm_hip_paged_decode_run_timed(cache, args, workspace, workspace_bytes, stream, nullptr, nullptr);
}

extern "C" int xllm_hip_paged_decode_run_timed(const xllm_hip_kv_cache* cache,
                                               const xllm_hip_decode_args* args,
                                               void* workspace,
                                               size_t workspace_bytes,
                                               xllm_hip_stream_t stream,
                                               void* ev_begin,
                                               void* ev_end) {
  DecodeParams p;
  if (int s = fill_params(cache, args, workspace, workspace_bytes, p)) return s;
  if (p.batch == 0) return XLLM_HIP_OK;
  const Variant v = pick_variant(cache, args);
  if (v == kNone) {
    return fail(XLLM_HIP_UNSUPPORTED,
                "no decode kernel for head_dim=%d block_size=%d (head_dim <= 256 and a power-of-two block_size "
                "are required)",
                cache->head_dim, cache->block_size);
  }
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = (unsigned)max_items(p);
  if (ev_begin != nullptr && hipEventRecord((hipEvent_t)ev_begin, st) != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipEventRecord(ev_begin) failed");
  }
  if (is_mfma(v)) {
    const bool qf16 = args->q_dtype == XLLM_HIP_FP16;
    switch (cache->dtype) {
      case XLLM_HIP_BF16:
        launch_mfma<XLLM_HIP_BF16>(p, grid, st);
        break;
      case XLLM_HIP_FP16:
        launch_mfma<XLLM_HIP_FP16>(p, grid, st);
        break;
      case XLLM_HIP_FP8_E4M3:
        if (qf16) {
          launch_mfma<XLLM_HIP_FP8_E4M3 | kQF16>(p, grid, st);
        } else {
          launch_mfma<XLLM_HIP_FP8_E4M3>(p, grid, st);
        }
        break;
      default:
        if (qf16) {
          launch_mfma<XLLM_HIP_INT8 | kQF16>(p, grid, st);
        } else {
          launch_mfma<XLLM_HIP_INT8>(p, grid, st);
        }
        break;
    }
  } else {
    int s;
    switch (args->q_dtype) {
      case XLLM_HIP_BF16:
        s = launch_generic<XLLM_HIP_BF16>(cache->dtype, p, grid, st);
        break;
      case XLLM_HIP_FP16:
        s = launch_generic<XLLM_HIP_FP16>(cache->dtype, p, grid, st);
        break;
      default:
        s = launch_generic<XLLM_HIP_FP32>(cache->dtype, p, grid, st);
        break;
    }
    if (s) return s;
  }
  if (int s = check_launch("decode attention kernel")) return s;
  if (ev_end != nullptr && hipEventRecord((hipEvent_t)ev_end, st) != hipSuccess) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipEventRecord(ev_end) failed");
  }
  if (p.implicit_plan || p.fused_merge) return XLLM_HIP_OK;  // nothing was split, or the attention kernel merged

  const int64_t rows = (int64_t)p.batch * p.n * p.num_q_heads;
  const unsigned mgrid = (unsigned)((rows + kMergeRowsPerBlock - 1) / kMergeRowsPerBlock);
  switch (args->q_dtype) {
    case XLLM_HIP_BF16:
      decode_merge_kernel<XLLM_HIP_BF16><<<mgrid, 64 * kMergeRowsPerBlock, 0, st>>>(p);
      break;
    case XLLM_HIP_FP16:
      decode_merge_kernel<XLLM_HIP_FP16><<<mgrid, 64 * kMergeRowsPerBlock, 0, st>>>(p);
      break;
    default:
      decode_merge_kernel<XLLM_HIP_FP32><<<mgrid, 64 * kMergeRowsPerBlock, 0, st>>>(p);
      break;
  }
  return check_launch("decode_merge_kernel");
}

extern "C" int xllm_hip_paged_decode(const xllm_hip_kv_cache* cache,
                                     const xllm_hip_decode_args* args,
                                     void* workspace,
                                     size_t workspace_bytes,
                                     xllm_hip_stream_t stream) {
  if (int s = xllm_hip_paged_decode_plan(cache, args, workspace, workspace_bytes, stream)) return s;
  return xllm_hip_paged_decode_run(cache, args, workspace, workspace_bytes, stream);
}

// Device address of `scratch` on the current device, looked up once per device.
static int static_workspace(void** out) {
  constexpr int kMaxDevices = 64;
  static std::mutex mu;
  static void* ptrs[kMaxDevices] = {nullptr};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    return fail(XLLM_HIP_RUNTIME_ERROR, "hipGetDevice failed or device index beyond %d", kMaxDevices - 1);
  }
  std::lock_guard<std::mutex> lock(mu);
  if (ptrs[dev] == nullptr) {
    void* ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      return fail(XLLM_HIP_RUNTIME_ERROR, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    }
    ptrs[dev] = ptr;
  }
  *out = ptrs[dev];
  return XLLM_HIP_OK;
}

extern "C" int xllm_hip_paged_decode_static(const xllm_hip_kv_cache* cache,
                                            const xllm_hip_decode_args* args,
                                            xllm_hip_stream_t stream) {
  XLLM_HIP_REQUIRE(cache != nullptr && args != nullptr, "cache or args is NULL");
  XLLM_HIP_REQUIRE(args->batch >= 0 && args->q_per_seq >= 1 && args->num_q_heads >= 1 && cache->num_kv_heads >= 1 &&
                       cache->head_dim >= 1,
                   "bad batch/q_per_seq/num_q_heads/num_kv_heads/head_dim");
  const size_t need =
      workspace_layout(args->batch, args->q_per_seq, args->num_q_heads, cache->num_kv_heads, cache->head_dim, device_cus())
          .total_bytes;
  if (need > (size_t)XLLM_HIP_STATIC_WORKSPACE_BYTES) {
    return fail(XLLM_HIP_WORKSPACE_TOO_SMALL,
                "these sizes need %zu bytes of workspace, the built-in one holds %zu: call xllm_hip_paged_decode "
                "with a caller-owned workspace",
                need, (size_t)XLLM_HIP_STATIC_WORKSPACE_BYTES);
  }
  void* ws = nullptr;
  if (int s = static_workspace(&ws)) return s;
  return xllm_hip_paged_decode(cache, args, ws, (size_t)XLLM_HIP_STATIC_WORKSPACE_BYTES, stream);
}

extern "C" int xllm_hip_csr_to_block_table(const int32_t* kv_indptr,
                                           const int32_t* kv_indices,
                                           const int32_t* kv_last_page_len,
                                           int32_t batch,
                                           int32_t block_size,
                                           int32_t* block_table,
                                           int64_t block_table_stride,
                                           int32_t max_blocks_per_seq,
                                           int32_t* seq_lens,
                                           xllm_hip_stream_t stream) {
  XLLM_HIP_REQUIRE(batch >= 0 && block_size > 0 && max_blocks_per_seq >= 1, "bad sizes");
  if (batch == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(kv_indptr && kv_indices && kv_last_page_len && block_table && seq_lens, "NULL argument");
  XLLM_HIP_REQUIRE(block_table_stride >= max_blocks_per_seq, "block_table_stride < max_blocks_per_seq");
  csr_to_block_table_kernel<<<(unsigned)batch, 256, 0, (hipStream_t)stream>>>(
      kv_indptr, kv_indices, kv_last_page_len, batch, block_size, block_table, block_table_stride,
      max_blocks_per_seq, seq_lens);
  return check_launch("csr_to_block_table_kernel");
}
