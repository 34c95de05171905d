/*
 * C ABI of the MI355X (gfx950) paged-KV decode path: the KV write through
 * slot_mapping and paged-attention decode over block_tables / seq_lens.
 *
 * Every entry point takes plain device pointers, sizes and strides and returns
 * an int status (0 = ok).  Nothing here allocates, frees or synchronises: work
 * is enqueued on the hipStream_t the caller passes (NULL = the null stream), so
 * every call is legal under HIP graph capture.  All pointers are device
 * pointers unless a comment says "host".
 *
 * Reference interfaces these replace (paths relative to the xLLM tree):
 *   xllm/core/kernels/ops_api.h:31-37          reshape_paged_cache / quant_to_paged_cache
 *   xllm/core/kernels/param.h:122-157          ReshapePagedCacheParams (tensor contract)
 *   xllm/core/kernels/cuda/cuda_ops_api.h:43-48,120-136   cuda::reshape_paged_cache, cuda::batch_decode (CSR form)
 *   xllm/core/kernels/mlu/mlu_ops_api.h:66-77,126-145     quant_to_paged_cache, batch_decode (block_table form)
 */
#ifndef XLLM_HIP_PAGED_KV_H_
#define XLLM_HIP_PAGED_KV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XLLM_HIP_ABI_VERSION 4

/* A hipStream_t, passed as an opaque pointer so that C callers need no HIP headers. */
typedef void* xllm_hip_stream_t;

/* Element types.  Values are part of the ABI. */
enum xllm_hip_dtype {
  XLLM_HIP_BF16 = 0,
  XLLM_HIP_FP16 = 1,
  XLLM_HIP_FP32 = 2,
  XLLM_HIP_FP8_E4M3 = 3, /* OCP e4m3fn, the encoding of torch.float8_e4m3fn */
  XLLM_HIP_INT8 = 4
};

enum xllm_hip_status {
  XLLM_HIP_OK = 0,
  XLLM_HIP_INVALID_ARGUMENT = 1,    /* a size, stride, pointer or dtype violates the contract */
  XLLM_HIP_UNSUPPORTED = 2,         /* valid request that no kernel here implements */
  XLLM_HIP_WORKSPACE_TOO_SMALL = 3, /* see xllm_hip_paged_decode_workspace_bytes */
  XLLM_HIP_RUNTIME_ERROR = 4        /* a HIP launch failed; see xllm_hip_last_error */
};

/*
 * One layer's paged KV cache.  Logical coordinates are (block, slot, head, d);
 * the element (block, slot, head, d) of K lives at
 *   k_cache + block*stride_block + head*stride_head + slot*stride_slot + d      (elements)
 * so both reference layouts are expressible without a copy:
 *   NHD [n_blocks, block_size, Hkv, D] (xllm/core/distributed_runtime/llm_engine.cpp:574-577):
 *        stride_block = bs*Hkv*D, stride_slot = Hkv*D, stride_head = D
 *   HND [n_blocks, Hkv, block_size, D] (llm_engine.cpp:595-612, kernels/param.h:133-143):
 *        stride_block = Hkv*bs*D, stride_head = bs*D, stride_slot = D
 * HND is the native (fastest) layout of the decode kernel.  V uses the same
 * strides as K.  head_dim is always contiguous.
 *
 * Quantised caches (dtype FP8_E4M3 or INT8) carry one fp32 scale per
 * (block, slot, head) for K and for V (xllm/core/runtime/worker_impl.cpp:276-287:
 * the cache shape minus its last dimension); element (block, slot, head) lives at
 *   k_scale + block*scale_stride_block + head*scale_stride_head + slot*scale_stride_slot.
 * A dequantised element is  (float)q * scale.
 */
typedef struct xllm_hip_kv_cache {
  void* k_cache;
  void* v_cache;  /* may be NULL for the write path when value is NULL */
  float* k_scale; /* NULL unless dtype is FP8_E4M3 / INT8 */
  float* v_scale;
  int64_t num_blocks;
  int32_t block_size;
  int32_t num_kv_heads;
  int32_t head_dim;
  int32_t dtype; /* xllm_hip_dtype of the cache elements */
  int64_t stride_block;
  int64_t stride_head;
  int64_t stride_slot;
  int64_t scale_stride_block;
  int64_t scale_stride_head;
  int64_t scale_stride_slot;
} xllm_hip_kv_cache;

/*
 * KV write through slot_mapping: for every token t with slot = slot_mapping[t],
 *   block = slot / block_size, off = slot % block_size,
 *   k_cache[block][off][h][d] = key[t*key_token_stride + h*head_dim + d]   (same for V)
 * — the index math of reshape_paged_cache_kernel
 * (xllm/core/kernels/cuda/reshape_paged_cache.cu:35-57), behind
 * xllm::kernel::reshape_paged_cache (xllm/core/kernels/ops_api.cpp:150-180).
 * Elements are copied verbatim (src_dtype must equal cache->dtype; BF16, FP16,
 * FP32 or 1-byte types).  key/value are [num_tokens, Hkv, D] with the last two
 * dimensions contiguous and a free token stride (they are slices of the fused
 * qkv buffer).  value == NULL writes K only.  A negative slot or a slot beyond
 * num_blocks*block_size is skipped (the reference would write out of bounds).
 * Duplicate slots (padding rows all map to slot 0,
 * xllm/core/framework/batch/batch_input_builder.cpp:517) are legal; which
 * duplicate wins is unspecified, as in the reference.
 */
int xllm_hip_reshape_paged_cache(const xllm_hip_kv_cache* cache,
                                 const void* key,
                                 const void* value,
                                 const int32_t* slot_mapping,
                                 int64_t num_tokens,
                                 int64_t key_token_stride,
                                 int64_t value_token_stride,
                                 int32_t src_dtype,
                                 xllm_hip_stream_t stream);

/*
 * Quantising KV write: per token and per head, symmetric quantisation of the
 * head_dim values followed by the same scatter as above, plus the scale store —
 * xllm::kernel::quant_to_paged_cache (xllm/core/kernels/ops_api.cpp:196-210,
 * xllm/core/kernels/mlu/mlu_ops_api.h:66-77).  src_dtype is BF16, FP16 or FP32;
 * cache->dtype is INT8 (qmax 127) or FP8_E4M3 (qmax 448).
 *   absmax = max_d |x_d|                     (fmaxf: a NaN element does not take part)
 *   scale  = max(absmax / qmax, min_scale)   min_scale = FLT_EPSILON (int8), 1/(448*512) (fp8)
 *            (xllm/core/kernels/cuda/fp8_quant_utils.cuh:38-53)
 *   q_d    = int8: clamp(rint(x_d / scale), -127, 127)   (round half to even)
 *            fp8 : e4m3fn_rne(clamp(x_d / scale, -448, 448))  (fp8_quant_utils.cuh:112-131)
 *   clamp(y, -m, m) = fmaxf(-m, fminf(y, m)) as in fp8_quant_utils.cuh:121-122, so a NaN quotient (a NaN
 *   element, or an infinite one: inf / inf) becomes +m; an all-zero row gets scale = min_scale and zeros.
 */
int xllm_hip_quant_to_paged_cache(const xllm_hip_kv_cache* cache,
                                  const void* key,
                                  const void* value,
                                  const int32_t* slot_mapping,
                                  int64_t num_tokens,
                                  int64_t key_token_stride,
                                  int64_t value_token_stride,
                                  int32_t src_dtype,
                                  xllm_hip_stream_t stream);

/*
 * Paged-attention decode.
 *
 *   out[b*n + j, h, :] = sum_t softmax_t(sm_scale * q[b*n + j, h] . K[b, t, h/g]) * V[b, t, h/g]
 *   t < seq_lens[b] - (n - 1 - j),   g = num_q_heads / num_kv_heads
 *
 * with K[b, t] found through the block table: block = table[b][t / block_size],
 * slot = t % block_size.  n = q_per_seq query tokens per sequence; n = 1 is
 * plain decode (xllm/core/kernels/mlu/mlu_ops_api.h:126-145 batch_decode,
 * xllm/core/kernels/cuda/batch_decode.cpp:26-86).  n > 1 is speculative verify:
 * the n draft tokens are the LAST n tokens of the sequence (already written to
 * the cache) and token j sees seq_lens[b] - (n-1-j) keys, which is what the
 * reference expresses by expanding every draft token into its own decode row
 * with its own kv length (xllm/core/runtime/speculative_worker_impl.cpp:230-243).
 * With q_indptr != NULL the sequences carry different numbers of query tokens — a chunked-prefill or
 * mixed step (xllm/core/layers/cuda/flashinfer_attention.cpp:224-284, q_cu_seq_lens / qo_indptr of
 * xllm/core/layers/common/attention_metadata.h): the tokens of sequence b are rows
 * q_indptr[b] .. q_indptr[b+1] of q/out, n_b = q_indptr[b+1] - q_indptr[b] of them, again the LAST
 * n_b tokens of the sequence, token j seeing seq_lens[b] - (n_b-1-j) keys (causal, aligned to the end
 * of the kv range).  q_per_seq must then be at least max_b n_b (the reference's max_query_len); it
 * sizes the launch and the workspace, and tokens beyond it are ignored.  Above 128 query rows per kv
 * head (q_per_seq * num_q_heads / num_kv_heads) sequences are never split into chunks.
 *
 * The block list of sequence b is given in one of two forms:
 *   block_table form (mlu_ops_api.h:130-131): block_table != NULL, row b starts at
 *       block_table + b*block_table_stride, padded with any valid block id;
 *       seq_lens[b] is the kv length (an entry above max_blocks_per_seq*block_size, which the row
 *       cannot hold, is cut to that: no block id is read from outside the row).
 *   CSR form (cuda_ops_api.h:129-131): block_table == NULL; the list is
 *       kv_indices[kv_indptr[b] .. kv_indptr[b+1]) and the kv length is
 *       (kv_indptr[b+1]-kv_indptr[b]-1)*block_size + kv_last_page_len[b]
 *       (kv_last_page_len is taken within 0 .. block_size).
 *
 * Block ids are expected within 0 .. num_blocks-1; one outside is taken as the nearest valid block
 * (the result for that sequence is then meaningless, but nothing outside the cache is read).
 *
 * q/out are [batch*n, num_q_heads, head_dim] of q_dtype (BF16, FP16 or FP32),
 * head_dim contiguous, head stride = head_dim, token strides free.
 * lse, if not NULL, receives the base-2 log-sum-exp of the scaled scores,
 *   lse[row, h] = log2(sum_t 2^(log2(e) * sm_scale * q.k_t)),
 * fp32 [batch*n, num_q_heads] — the quantity the reference's merge consumes
 * (xllm/core/kernels/cuda/xattention/lse_combine.cu:61-73).
 * A sequence with kv length 0 yields zeros (lse = -inf).
 * window_left < 0 disables the sliding window; otherwise query at position p
 * sees keys p - window_left .. p.
 */
typedef struct xllm_hip_decode_args {
  const void* q;
  void* out;
  float* lse; /* may be NULL */
  int64_t q_token_stride;
  int64_t out_token_stride;
  int32_t q_dtype;
  int32_t batch;
  int32_t q_per_seq;
  int32_t num_q_heads;
  float sm_scale;
  int32_t window_left;
  /* block_table form */
  const int32_t* block_table;
  int64_t block_table_stride;
  int32_t max_blocks_per_seq; /* row length of block_table */
  const int32_t* seq_lens;
  /* CSR form (used when block_table == NULL) */
  const int32_t* kv_indptr;
  const int32_t* kv_indices;
  const int32_t* kv_last_page_len;
  /* Host-side hints, as the reference keeps them in AttentionMetadata
   * (xllm/core/layers/common/attention_metadata.h:75-77).  max_seq_len must be
   * >= every kv length; total_kv_len (0 = unknown) only tunes the split. */
  int32_t max_seq_len;
  int64_t total_kv_len;
  /* Query token offsets [batch+1] for sequences with different numbers of query tokens; NULL: every
   * sequence has q_per_seq of them. */
  const int32_t* q_indptr;
  /* != 0: the step's schedule is the one xllm_hip_paged_decode_plan_host (or, from the same arguments,
   * xllm_hip_paged_decode_plan) stores in the workspace before the step.  Which kernel runs and how its work
   * items are shaped then follows from the sizes alone and max_seq_len / total_kv_len are ignored, so that a
   * xllm_hip_paged_decode_run captured in a graph serves every later step of the same sizes: what changes from
   * step to step lives in the workspace. */
  int32_t host_plan;
} xllm_hip_decode_args;

/*
 * Bytes of scratch xllm_hip_paged_decode needs for these sizes (split-KV
 * partial results and the per-step schedule).  Depends on sizes only, never on
 * the lengths, so one allocation serves every step.
 */
size_t xllm_hip_paged_decode_workspace_bytes(int32_t batch,
                                             int32_t q_per_seq,
                                             int32_t num_q_heads,
                                             int32_t num_kv_heads,
                                             int32_t head_dim);

/*
 * Build the per-step split-KV schedule from the kv lengths, on the device
 * (no host read-back, unlike the reference's layer-0 plan,
 * xllm/core/layers/cuda/flashinfer_planinfo.cpp:252-253,299-300).  The schedule
 * is stored at the head of `workspace` and depends only on args' block
 * list/length fields, batch, q_per_seq, num_q_heads and the cache's
 * num_kv_heads/head_dim/block_size: it may be built once per step and reused
 * by every layer's xllm_hip_paged_decode_run with the same workspace.
 */
int xllm_hip_paged_decode_plan(const xllm_hip_kv_cache* cache,
                               const xllm_hip_decode_args* args,
                               void* workspace,
                               size_t workspace_bytes,
                               xllm_hip_stream_t stream);

/*
 * The same schedule made on the host, from the kv lengths the engine holds there
 * (xllm/core/framework/model/model_input_params.h:341 kv_seq_lens_vec) — what the reference does before every
 * step, also before every replay of a captured graph (xllm/core/runtime/cuda_graph_executor_impl.cpp:586-668,
 * CudaGraphPersistentParam::update -> update_decode_plan_info; xllm/core/layers/cuda/flashinfer_planinfo.cpp:215-324).
 * With every length known, each sequence is cut into chunks of its own, nearly equal size, how finely is chosen
 * by the finishing time a list schedule of the step's work items predicts, and the chunks are dispatched longest
 * first.  args->host_plan must be set (see there); host_kv_lens[b] must be the kv length the device-side arrays
 * give for sequence b.  The schedule is written into host_staging (xllm_hip_paged_decode_plan_host_bytes bytes,
 * best pinned) and copied to the head of `workspace` with one hipMemcpyAsync on `stream`; host_staging must stay
 * untouched until that copy has run.  Nothing is allocated and nothing is read back; the call is made outside a
 * captured graph, the runs it serves may be inside one.  info, if not NULL, receives {chunk size the cut was made
 * for (0: nothing is cut), sequence chunks, predicted finishing time in tokens}.
 */
size_t xllm_hip_paged_decode_plan_host_bytes(int32_t batch,
                                             int32_t q_per_seq,
                                             int32_t num_q_heads,
                                             int32_t num_kv_heads,
                                             int32_t head_dim);
int xllm_hip_paged_decode_plan_host(const xllm_hip_kv_cache* cache,
                                    const xllm_hip_decode_args* args,
                                    const int32_t* host_kv_lens,
                                    void* workspace,
                                    size_t workspace_bytes,
                                    void* host_staging,
                                    size_t host_staging_bytes,
                                    xllm_hip_stream_t stream,
                                    int64_t* info);

/* Attention proper; requires a schedule built by xllm_hip_paged_decode_plan in `workspace` from the same
 * sizes, block list / length arrays and host-side lengths (max_seq_len, total_kv_len): with host-side
 * lengths that are nearly equal (max_seq_len * batch <= 1.25 * total_kv_len) a split step stores no
 * schedule — every work item derives its chunk from its index and its sequence's length — and the plan
 * call only zeroes the counters of the in-kernel combine, so a run with other host-side lengths than its
 * plan finds no schedule (its result is then undefined; nothing outside the arguments is read).
 * Split sequences leave normalised partial results in the workspace; up to 16 query rows per kv
 * head the attention kernel combines them itself (the workgroup that finishes a sequence's last
 * chunk; it counts in counters that the plan zeroes and every run leaves at zero), otherwise a merge
 * kernel follows.  Two runs must not share a workspace concurrently.
 * The in-kernel combine rests on how gfx950 treats device-scope atomic accesses, not on the HIP
 * memory model alone: partials are stored and loaded as relaxed device-scope atomics (which go to
 * memory past the caches that are private to an XCD), a wave waits for its stores to complete
 * (s_waitcnt vmcnt(0)) before the workgroup's thread 0 increments the counter, and the workgroup that
 * reads the final count reads the partials.  No release/acquire fence pair is issued (it was
 * measured three times slower).  XLLM_HIP_OPTION_DECODE_SEPARATE_MERGE selects the separate merge
 * kernel, which depends on stream order alone, for every shape. */
int xllm_hip_paged_decode_run(const xllm_hip_kv_cache* cache,
                              const xllm_hip_decode_args* args,
                              void* workspace,
                              size_t workspace_bytes,
                              xllm_hip_stream_t stream);

/*
 * xllm_hip_paged_decode_run that also records two caller-created hipEvent_t on `stream`: ev_begin
 * just before the attention kernel (the launch that streams the KV cache) and ev_end just after
 * it, before the merge kernel if one follows.  A measurement hook for benchmarks; it has no counterpart in the
 * reference.  Either event may be NULL.
 */
int xllm_hip_paged_decode_run_timed(const xllm_hip_kv_cache* cache,
                                    const xllm_hip_decode_args* args,
                                    void* workspace,
                                    size_t workspace_bytes,
                                    xllm_hip_stream_t stream,
                                    void* ev_begin,
                                    void* ev_end);

/* plan + run in one call. */
int xllm_hip_paged_decode(const xllm_hip_kv_cache* cache,
                          const xllm_hip_decode_args* args,
                          void* workspace,
                          size_t workspace_bytes,
                          xllm_hip_stream_t stream);

/*
 * xllm_hip_paged_decode without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops and harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The schedule, the split partials and the merge counters live in an
 * array of XLLM_HIP_STATIC_WORKSPACE_BYTES bytes that is part of the library's device code: each GPU
 * the library runs on holds its own copy from the first launch until the process ends, and this
 * call neither allocates nor frees anything.  Sizes for which xllm_hip_paged_decode_workspace_bytes
 * exceeds that constant are refused with XLLM_HIP_WORKSPACE_TOO_SMALL and a message (with
 * r = min(q_per_seq * num_q_heads / num_kv_heads, 128) query rows per kv head the need is at most
 * 2560 * r * head_dim * 4 bytes for r <= 16 and 1280 * r * head_dim * 4 bytes above, plus
 * r * num_kv_heads * head_dim * 4 bytes per sequence: 20 MiB + 128 KiB per sequence for 32 query rows
 * per kv head at head_dim 128 and 8 kv heads, 20 MiB + 64 KiB per sequence for 16).
 * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (two streams, two
 * threads) race; calls ordered on a stream, or by events, do not.  Nothing needs clearing between
 * calls: each call rebuilds the schedule and zeroes the counters it uses with a kernel, not a memset.
 * The device current at the call must be the one `stream` belongs to.  The array's address is looked
 * up on the first call per device (hipGetSymbolAddress): make one call on each device before
 * capturing a graph that contains this entry point.
 */
#define XLLM_HIP_STATIC_WORKSPACE_BYTES (48u << 20)
int xllm_hip_paged_decode_static(const xllm_hip_kv_cache* cache,
                                 const xllm_hip_decode_args* args,
                                 xllm_hip_stream_t stream);

/*
 * Index-only conversion between the two block-list forms
 * (xllm/core/framework/batch/batch_input_builder.cpp:438-494 builds both from
 * the same sequences): fills block_table rows (padding with 0) and seq_lens
 * from the CSR arrays.
 */
int xllm_hip_csr_to_block_table(const int32_t* kv_indptr,
                                const int32_t* kv_indices,
                                const int32_t* kv_last_page_len,
                                int32_t batch,
                                int32_t block_size,
                                int32_t* block_table,
                                int64_t block_table_stride,
                                int32_t max_blocks_per_seq,
                                int32_t* seq_lens,
                                xllm_hip_stream_t stream);

/*
 * The step in front of the KV write, fused with it: per-head RMSNorm of the query and key heads
 * (optional), rotary position embedding of both, and the scatter of the new K and V rows into the
 * paged cache, in one pass over the fused qkv buffer
 * (call sites: xllm/core/layers/common/qwen2_attention.cpp:147-189 — fused_qk_norm_rope or
 * q_norm/k_norm + rotary_emb, then AttentionImpl::forward's cache write).
 *
 * Norm and rotation follow xllm::kernel::cuda::fused_qk_norm_rope
 * (xllm/core/kernels/cuda/cuda_ops_api.h:227-241, kernel fused_qknorm_rope.cu:70-262): per head,
 *   x_d <- x_d * rsqrt(mean_d(x_d^2) + eps) * weight_d        (skipped when q_weight == NULL)
 *   pairs (j, j + rotary_dim/2) [interleave: (2j, 2j+1)], frequency j, position pos = positions[t]:
 *   x' = x cos - y sin,  y' = y cos + x sin,   cos = cache[pos][j], sin = cache[pos][rotary_dim/2 + j]
 * in float with one rounding to the element type at the end; elements beyond rotary_dim pass
 * through.  round_each_op != 0 rounds to the element type after the norm, after each product and
 * after the sum instead, which is what xllm::kernel::cuda::rotary_embedding computes on scalar_t
 * operands (xllm/core/kernels/cuda/rope.cu:26-52, used when the fused kernel is not).
 * q and k heads are rewritten in place in qkv.  positions outside [0, max_position) are clamped
 * (the reference would read outside the table).
 *
 * With cache != NULL the rotated K heads and the V heads of every token are then written to
 * slot_mapping[t] exactly as xllm_hip_reshape_paged_cache (cache->dtype == dtype) or
 * xllm_hip_quant_to_paged_cache (INT8 / FP8_E4M3 cache) would write them from the updated buffer;
 * num_k_heads and num_v_heads must equal cache->num_kv_heads.  cache == NULL: norm and rotation only.
 */
typedef struct xllm_hip_rope_args {
  void* qkv;            /* [num_tokens, (Hq + Hk + Hv) * head_dim], last dimension contiguous */
  int64_t token_stride; /* elements between consecutive tokens */
  int64_t num_tokens;
  int32_t dtype;        /* BF16 / FP16 / FP32: qkv and the norm weights */
  int32_t num_q_heads;
  int32_t num_k_heads;
  int32_t num_v_heads;
  int32_t head_dim;     /* <= 512 */
  int32_t rotary_dim;   /* even, <= head_dim */
  const void* q_weight; /* [head_dim] or NULL (no norm; then k_weight is NULL too) */
  const void* k_weight;
  float eps;
  int32_t cos_sin_dtype;     /* BF16 / FP16 / FP32 */
  const void* cos_sin_cache; /* [max_position, rotary_dim] */
  int64_t max_position;
  const void* positions;     /* [num_tokens], int64 (or int32, see positions_int32) */
  int32_t interleave;        /* 0: NeoX pairs (j, j + rotary_dim/2); 1: GPT-J pairs (2j, 2j+1) */
  int32_t round_each_op;
  int32_t positions_int32;   /* nonzero: positions is const int32_t* (the type the reference's attention
                              * modules pass, xllm/core/layers/common/tests/qwen2_attention_tests.cpp:226) */
} xllm_hip_rope_args;

int xllm_hip_rope_kv_write(const xllm_hip_rope_args* args,
                           const xllm_hip_kv_cache* cache,
                           const int32_t* slot_mapping,
                           xllm_hip_stream_t stream);

/*
 * Batched block swap — KVCache::swap_blocks
 * (xllm/core/framework/kv_cache/kv_cache.cpp:104-125; called per layer from
 * xllm/core/runtime/worker_impl.cpp:584-606 with int64 index tensors): for every pair i the whole
 * block src_blocks[i] of K, of V and, for a quantised cache, of both scale tensors is copied to
 * block dst_blocks[i].  The reference gathers all sources first (index_select) and scatters
 * afterwards (index_copy_), so a block that is both a destination and a source still supplies its
 * old contents.  With a staging buffer of xllm_hip_swap_blocks_staging_bytes(cache, num_pairs)
 * bytes (16-byte aligned) this call does exactly that, in two launches.  With staging == NULL it
 * copies in place in one pass, which is the same result whenever no destination block is also a
 * source (the block manager hands out fresh blocks as destinations).  Pairs with an id outside
 * [0, num_blocks) are skipped (the reference would throw).  Duplicate destinations: one of the
 * writers wins per 16-byte piece, as with index_copy_.
 */
size_t xllm_hip_swap_blocks_staging_bytes(const xllm_hip_kv_cache* cache, int64_t num_pairs);
int xllm_hip_swap_blocks(const xllm_hip_kv_cache* cache,
                         const int64_t* src_blocks,
                         const int64_t* dst_blocks,
                         int64_t num_pairs,
                         void* staging,
                         size_t staging_bytes,
                         xllm_hip_stream_t stream);

/*
 * One-to-many block copy in the form the batch builder emits for the block-copy kernel
 * (xllm/core/framework/batch/batch_input_builder.cpp:691-720; fields
 * xllm/core/framework/model/model_input_params.h:542-545; consumed by
 * xllm/models/llm/npu/llm_model_base.h:69-75): source block src_block_indices[g] is copied to the
 * destination blocks dst_block_indices[cum_sum[g-1] .. cum_sum[g]) (cum_sum[-1] = 0), for
 * g < num_groups; num_dst = cum_sum[num_groups-1].  K, V and the scale tensors move together.
 * Destinations must not be sources of the same call.
 */
int xllm_hip_copy_blocks(const xllm_hip_kv_cache* cache,
                         const int32_t* src_block_indices,
                         const int32_t* dst_block_indices,
                         const int32_t* cum_sum,
                         int32_t num_groups,
                         int32_t num_dst,
                         xllm_hip_stream_t stream);

/*
 * Process-wide diagnostic switches; none is needed in service and none has a counterpart in the
 * reference.  Each starts at the integer value of the environment variable of the same name with
 * the prefix XLLM_HIP_ (XLLM_HIP_DECODE_FORCE_GENERIC, ...), read once when the first decode call or
 * option call is made, or 0.  Safe to call from any thread; a change applies to calls made after it.
 */
enum xllm_hip_option {
  XLLM_HIP_OPTION_DECODE_FORCE_GENERIC = 0,  /* != 0: every decode call takes the generic kernel */
  XLLM_HIP_OPTION_DECODE_TARGET_ITEMS = 1,   /* > 0: work items a split decode step is cut for, if that is fewer
                                              * than the kernel's own target (256 to 2048) */
  XLLM_HIP_OPTION_DECODE_SEPARATE_MERGE = 2, /* != 0: split sequences are always combined by the merge kernel */
  XLLM_HIP_OPTION_DECODE_STORED_SCHEDULE = 3, /* != 0: a split step always stores its schedule in the workspace
                                               * (the plan kernel), also when the host-side lengths would let
                                               * every work item derive its chunk by itself */
  XLLM_HIP_OPTION_DECODE_ITEM_PER_HEAD = 4, /* != 0: a work item is always one kv head, also over a cache whose kv
                                             * heads lie side by side within a token (NHD) and for a large batch of
                                             * short sequences, where the 16-row kernel otherwise gives an item four
                                             * kv heads, one per wave */
  XLLM_HIP_OPTION_DECODE_FOUR_WAVE_ITEMS = 5, /* != 0: the 16-row kernel always runs four waves per work item, also
                                               * when the launch has at most one item per CU (where it otherwise
                                               * runs eight) */
  XLLM_HIP_OPTION_PREFILL_KERNEL = 6, /* bit 0: steps of more than 128 query rows per kv head at head_dim 128
                                       * take the 128-row kernels (four waves per work item) instead of the
                                       * 256-row ones (eight waves in two groups that alternate between their
                                       * matrix and softmax phases); bit 1: the late group of the 256-row kernel
                                       * for 16-bit caches is the odd waves instead of waves 4-7 (two waves of
                                       * different SIMDs: for measurements) */
  XLLM_HIP_OPTION_COUNT = 7
};
int xllm_hip_set_option(int32_t which, int64_t value);
int64_t xllm_hip_get_option(int32_t which); /* -1 for an unknown option */

/* Message of the last non-OK status returned on this host thread ("" if none). */
const char* xllm_hip_last_error(void);

/*
 * Sequences read back out of the paged cache into dense tensors: the paged mode of
 * xllm::kernel::reshape_from_cache (xllm/core/kernels/ops_api.cpp:182-196, arguments
 * xllm/core/kernels/param.h:160-215, xllm/core/kernels/mlu/mlu_ops_api.h:56-64) and
 * xllm::kernel::dequant_from_paged_cache (xllm/core/kernels/ops_api.cpp:214-232,
 * xllm/core/kernels/mlu/mlu_ops_api.h:79-101; run before a chunked-prefill step over a quantised
 * cache, xllm/core/layers/mlu/attention.cpp:179-214).  For every sequence b < batch and token
 * t < context_lengths[b]:
 *   pos = (cache_seq_offset ? cache_seq_offset[b] : 0) + t
 *   blk = block_tables[b * block_table_stride + pos / block_size],  slot = pos % block_size
 *   row = (context_seq_offset ? context_seq_offset[b] : context_lengths[0] + .. + context_lengths[b-1]) + t
 *   key_out[row][h][d] = k_cache[blk][slot][h][d]            (same for value_out; NULL: keys only)
 * key_out/value_out are [rows, num_kv_heads, head_dim] with a free token stride (elements).
 * out_dtype == cache->dtype copies the elements verbatim (any dtype).  For an FP8_E4M3/INT8 cache
 * out_dtype BF16/FP16/FP32 dequantises: (float)q * scale, rounded once to out_dtype, where the scale
 * is the cache's per-(block, head, slot) one (quant_mode 1, per token) or k_scale/v_scale read as
 * a dense [num_kv_heads, head_dim] array (quant_mode 0, per channel).  max_context_len bounds
 * context_lengths (it sizes the grid; longer sequences are cut there).  Tokens whose block index
 * lies beyond max_blocks_per_seq or whose block id is outside [0, num_blocks) are skipped.
 */
int xllm_hip_gather_from_cache(const xllm_hip_kv_cache* cache,
                               void* key_out,
                               void* value_out,
                               int32_t out_dtype,
                               int64_t key_token_stride,
                               int64_t value_token_stride,
                               const int32_t* context_lengths,
                               const int32_t* context_seq_offset,
                               const int32_t* cache_seq_offset,
                               const int32_t* block_tables,
                               int64_t block_table_stride,
                               int32_t max_blocks_per_seq,
                               int32_t batch,
                               int32_t max_context_len,
                               int32_t quant_mode,
                               xllm_hip_stream_t stream);

/* XLLM_HIP_ABI_VERSION the library was built with. */
int xllm_hip_abi_version(void);

/* Name of the kernel variant xllm_hip_paged_decode_run would pick for these
 * arguments ("mfma_d128", "mfma_d64", "mfma_d256", "generic", or "" if unsupported); host-only, launches nothing. */
const char* xllm_hip_paged_decode_variant(const xllm_hip_kv_cache* cache,
                                          const xllm_hip_decode_args* args);

/* How xllm_hip_paged_decode_plan / _run would run these arguments on a workspace of `workspace_bytes` (0: of
 * xllm_hip_paged_decode_workspace_bytes): host-only, launches nothing, reads no device memory (pointers are only
 * checked for NULL).  No counterpart in the reference; it exists so that the step's schedule can be inspected,
 * and tested, without a GPU.  Writes up to `count` of
 *   out[0]  workgroups of the attention launch          out[1]  waves per workgroup (1, 2, 4 or 8)
 *   out[2]  1: nothing is split (no plan, no merge)     out[3]  1: the schedule is stored by the plan kernel
 *   out[4]  chunk tokens of the cut sequences (0: chosen on the device)
 *   out[5]  chunk slots per cut sequence (schedule-free split; else 0)
 *   out[6]  leading sequences that keep out[7] slots each of out[8] tokens (0: whole); the others are cut finer
 *   out[9]  kv heads per work item                      out[10] work items per workgroup (1, 2 or 4)
 *   out[11] 1: split sequences are merged inside the attention kernel
 *   out[12] sequence-chunk slots the workspace holds    out[13] sequence-chunk slots the launch addresses
 * and returns XLLM_HIP_OK, or the error the same arguments would get. */
int xllm_hip_paged_decode_describe(const xllm_hip_kv_cache* cache,
                                   const xllm_hip_decode_args* args,
                                   size_t workspace_bytes,
                                   int64_t* out,
                                   int32_t count);

#ifdef __cplusplus
}
#endif

#endif /* XLLM_HIP_PAGED_KV_H_ */
