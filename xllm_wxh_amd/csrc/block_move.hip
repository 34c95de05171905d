// Whole-block movement inside a paged KV cache for gfx950: the batched block swap
// (xllm/core/framework/kv_cache/kv_cache.cpp:104-125) and the one-to-many block copy that the
// scheduler's copy-on-write emits (xllm/core/framework/batch/batch_input_builder.cpp:685-720,
// consumed in xllm/models/llm/npu/llm_model_base.h:69-75).  K, V and, for quantised caches, the
// two fp32 scale tensors of a block move together.
//
// A block of one array is `rows = num_kv_heads * block_size` rows of `row_bytes`; row r sits at
// head (r / block_size) * stride_head + slot (r % block_size) * stride_slot, so both block layouts
// are served.  Pure HBM traffic: bytes read = bytes written = what the blocks hold.
#include "device_utils.h"
#include "host_utils.h"

namespace xllm_hip {

struct BlockMoveParams {
  // array a: 0 = K, 1 = V, 2 = K scales, 3 = V scales
  uint8_t* base[4];
  int64_t stride_block[4];  // bytes
  int64_t stride_head[4];
  int64_t stride_slot[4];
  int32_t row_bytes[4];
  int64_t staging_off[4];   // byte offset of the array inside a staged block
  uint8_t* staging;         // dense copies of whole blocks, one per pair (NULL: none)
  int64_t staging_block_bytes;
  const void* src_ids;      // per pair, or per group when cum_sum is set
  const void* dst_ids;      // per pair
  const int32_t* cum_sum;   // group g serves pairs [cum_sum[g-1], cum_sum[g]); NULL: src_ids is per pair
  int64_t num_pairs;
  int64_t num_blocks;
  int32_t num_groups;
  int32_t ids64;            // ids are int64 (else int32)
  int32_t rows;             // num_kv_heads * block_size
  int32_t block_size;
  int32_t mode;             // 0: cache[src] -> cache[dst]; 1: cache[src] -> staging; 2: staging -> cache[dst]
};

__device__ inline int64_t load_id(const void* ids, int64_t i, int ids64) {
  return ids64 ? ((const int64_t*)ids)[i] : (int64_t)((const int32_t*)ids)[i];
}

// grid (pair, piece of the block, array).  VecT: widest type every address is a multiple of.
template <typename VecT>
__global__ void __launch_bounds__(256) block_move_kernel(BlockMoveParams p) {
  const int64_t pair = blockIdx.x;
  const int a = blockIdx.z;
  int64_t src_blk = 0, dst_blk = 0;
  if (p.mode != 2) {
    int64_t si = pair;
    if (p.cum_sum != nullptr) {  // first group whose end lies beyond this pair
      int lo = 0, hi = p.num_groups - 1;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        if ((int64_t)p.cum_sum[mid] > pair) {
          hi = mid;
        } else {
          lo = mid + 1;
        }
      }
      if ((int64_t)p.cum_sum[lo] <= pair) return;  // beyond the last group
      si = lo;
    }
    src_blk = load_id(p.src_ids, si, p.ids64);
    if (src_blk < 0 || src_blk >= p.num_blocks) return;
  }
  if (p.mode != 1) {
    dst_blk = load_id(p.dst_ids, pair, p.ids64);
    if (dst_blk < 0 || dst_blk >= p.num_blocks) return;
    // a pair that names an invalid source moves nothing in either phase
    if (p.mode == 2) {
      const int64_t s = load_id(p.src_ids, pair, p.ids64);
      if (s < 0 || s >= p.num_blocks) return;
    }
  }
  const int vec_per_row = p.row_bytes[a] / (int)sizeof(VecT);
  const int64_t total = (int64_t)p.rows * vec_per_row;
  const uint8_t* src_base;
  uint8_t* dst_base;
  const bool src_dense = p.mode == 2, dst_dense = p.mode == 1;
  src_base = src_dense ? p.staging + pair * p.staging_block_bytes + p.staging_off[a]
                       : p.base[a] + src_blk * p.stride_block[a];
  dst_base = dst_dense ? p.staging + pair * p.staging_block_bytes + p.staging_off[a]
                       : p.base[a] + dst_blk * p.stride_block[a];
  for (int64_t i = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.y * blockDim.x) {
    const int r = (int)(i / vec_per_row);
    const int c = (int)(i - (int64_t)r * vec_per_row);
    const int h = r / p.block_size;
    const int s = r - h * p.block_size;
    const int64_t strided = (int64_t)h * p.stride_head[a] + (int64_t)s * p.stride_slot[a] + (int64_t)c * sizeof(VecT);
    const int64_t dense = (int64_t)r * p.row_bytes[a] + (int64_t)c * sizeof(VecT);
    const VecT v = *(const VecT*)(src_base + (src_dense ? dense : strided));
    *(VecT*)(dst_base + (dst_dense ? dense : strided)) = v;
  }
}

static bool quantised(const xllm_hip_kv_cache* c) {
  return c->dtype == XLLM_HIP_INT8 || c->dtype == XLLM_HIP_FP8_E4M3;
}

// Bytes one block occupies in the staging buffer (K, V, then the scales), each part 16-byte aligned.
static int64_t staged_block_bytes(const xllm_hip_kv_cache* c, int64_t off[4]) {
  const int64_t rows = (int64_t)c->num_kv_heads * c->block_size;
  const int64_t kv = (rows * c->head_dim * elem_bytes(c->dtype) + 15) & ~(int64_t)15;
  const int64_t sc = quantised(c) ? ((rows * 4 + 15) & ~(int64_t)15) : 0;
  off[0] = 0;
  off[1] = kv;
  off[2] = 2 * kv;
  off[3] = 2 * kv + sc;
  return 2 * kv + 2 * sc;
}

static int check_cache(const xllm_hip_kv_cache* c) {
  XLLM_HIP_REQUIRE(c != nullptr, "cache descriptor is NULL");
  XLLM_HIP_REQUIRE(c->k_cache != nullptr, "k_cache is NULL");
  XLLM_HIP_REQUIRE(c->num_blocks > 0 && c->block_size > 0 && c->num_kv_heads > 0 && c->head_dim > 0,
                   "cache sizes must be positive (blocks=%lld bs=%d heads=%d dim=%d)", (long long)c->num_blocks,
                   c->block_size, c->num_kv_heads, c->head_dim);
  XLLM_HIP_REQUIRE(elem_bytes(c->dtype) > 0, "unknown cache dtype %d", c->dtype);
  XLLM_HIP_REQUIRE(c->stride_block > 0 && c->stride_head > 0 && c->stride_slot > 0, "cache strides must be positive");
  if (quantised(c)) {
    XLLM_HIP_REQUIRE(c->k_scale != nullptr && (c->v_cache == nullptr || c->v_scale != nullptr),
                     "a quantised cache moves its scales with its blocks: k_scale / v_scale is NULL");
    XLLM_HIP_REQUIRE(c->scale_stride_block > 0 && c->scale_stride_head > 0 && c->scale_stride_slot > 0,
                     "scale strides must be positive");
  }
  return XLLM_HIP_OK;
}

static int launch(const xllm_hip_kv_cache* c, BlockMoveParams& p, hipStream_t st) {
  const int eb = elem_bytes(c->dtype);
  p.base[0] = (uint8_t*)c->k_cache;
  p.base[1] = (uint8_t*)c->v_cache;
  p.base[2] = (uint8_t*)c->k_scale;
  p.base[3] = (uint8_t*)c->v_scale;
  for (int a = 0; a < 2; ++a) {
    p.stride_block[a] = c->stride_block * eb;
    p.stride_head[a] = c->stride_head * eb;
    p.stride_slot[a] = c->stride_slot * eb;
    p.row_bytes[a] = c->head_dim * eb;
  }
  for (int a = 2; a < 4; ++a) {
    p.stride_block[a] = c->scale_stride_block * 4;
    p.stride_head[a] = c->scale_stride_head * 4;
    p.stride_slot[a] = c->scale_stride_slot * 4;
    p.row_bytes[a] = 4;
  }
  p.staging_block_bytes = staged_block_bytes(c, p.staging_off);
  p.num_blocks = c->num_blocks;
  p.rows = c->num_kv_heads * c->block_size;
  p.block_size = c->block_size;
  XLLM_HIP_REQUIRE(p.num_pairs <= 0x7fffffff, "too many blocks in one call (%lld)", (long long)p.num_pairs);

  // K and V (arrays 0, 1): widest vector all addresses are multiples of.
  const uintptr_t mix = (uintptr_t)p.base[0] | (uintptr_t)p.base[1] | (uintptr_t)p.stride_block[0] |
                        (uintptr_t)p.stride_head[0] | (uintptr_t)p.stride_slot[0] | (uintptr_t)p.row_bytes[0] |
                        (uintptr_t)p.staging;
  const int arrays_kv = c->v_cache != nullptr ? 2 : 1;
  const int64_t block_bytes = (int64_t)p.rows * p.row_bytes[0];
  auto pieces = [](int64_t vecs) {
    int64_t n = (vecs + 256 * 8 - 1) / (256 * 8);  // about eight vectors per thread
    return (unsigned)(n < 1 ? 1 : n > 64 ? 64 : n);
  };
  if ((mix & 15) == 0) {
    block_move_kernel<u32x4><<<dim3((unsigned)p.num_pairs, pieces(block_bytes / 16), arrays_kv), 256, 0, st>>>(p);
  } else if ((mix & 3) == 0) {
    block_move_kernel<uint32_t><<<dim3((unsigned)p.num_pairs, pieces(block_bytes / 4), arrays_kv), 256, 0, st>>>(p);
  } else if ((mix & 1) == 0) {
    block_move_kernel<uint16_t><<<dim3((unsigned)p.num_pairs, pieces(block_bytes / 2), arrays_kv), 256, 0, st>>>(p);
  } else {
    block_move_kernel<uint8_t><<<dim3((unsigned)p.num_pairs, pieces(block_bytes), arrays_kv), 256, 0, st>>>(p);
  }
  if (int s = check_launch("block_move_kernel")) return s;
  if (quantised(c)) {
    // the scale arrays (2, 3) ride in a second launch of the 4-byte variant
    BlockMoveParams q = p;
    q.base[0] = p.base[2];
    q.base[1] = p.base[3];
    for (int a = 0; a < 2; ++a) {
      q.stride_block[a] = p.stride_block[2];
      q.stride_head[a] = p.stride_head[2];
      q.stride_slot[a] = p.stride_slot[2];
      q.row_bytes[a] = 4;
      q.staging_off[a] = p.staging_off[2 + a];
    }
    block_move_kernel<uint32_t><<<dim3((unsigned)p.num_pairs, 1, arrays_kv), 256, 0, st>>>(q);
    if (int s = check_launch("block_move_kernel (scales)")) return s;
  }
  return XLLM_HIP_OK;
}

}  // namespace xllm_hip

using namespace xllm_hip;

extern "C" size_t xllm_hip_swap_blocks_staging_bytes(const xllm_hip_kv_cache* cache, int64_t num_pairs) {
  if (cache == nullptr || num_pairs <= 0 || elem_bytes(cache->dtype) <= 0) return 0;
  int64_t off[4];
  return (size_t)(staged_block_bytes(cache, off) * num_pairs);
}

extern "C" int xllm_hip_swap_blocks(const xllm_hip_kv_cache* cache,
                                    const int64_t* src_blocks,
                                    const int64_t* dst_blocks,
                                    int64_t num_pairs,
                                    void* staging,
                                    size_t staging_bytes,
                                    xllm_hip_stream_t stream) {
  if (int s = check_cache(cache)) return s;
  XLLM_HIP_REQUIRE(num_pairs >= 0, "num_pairs is negative");
  if (num_pairs == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(src_blocks != nullptr && dst_blocks != nullptr, "src_blocks or dst_blocks is NULL");
  BlockMoveParams p{};
  p.src_ids = src_blocks;
  p.dst_ids = dst_blocks;
  p.ids64 = 1;
  p.num_pairs = num_pairs;
  hipStream_t st = (hipStream_t)stream;
  if (staging == nullptr) {
    p.mode = 0;
    return launch(cache, p, st);
  }
  XLLM_HIP_REQUIRE(((uintptr_t)staging & 15) == 0, "staging must be 16-byte aligned");
  XLLM_HIP_REQUIRE(staging_bytes >= xllm_hip_swap_blocks_staging_bytes(cache, num_pairs),
                   "staging holds %zu bytes, %zu needed", staging_bytes,
                   xllm_hip_swap_blocks_staging_bytes(cache, num_pairs));
  p.staging = (uint8_t*)staging;
  p.mode = 1;
  if (int s = launch(cache, p, st)) return s;
  p.mode = 2;
  return launch(cache, p, st);
}

extern "C" int xllm_hip_copy_blocks(const xllm_hip_kv_cache* cache,
                                    const int32_t* src_block_indices,
                                    const int32_t* dst_block_indices,
                                    const int32_t* cum_sum,
                                    int32_t num_groups,
                                    int32_t num_dst,
                                    xllm_hip_stream_t stream) {
  if (int s = check_cache(cache)) return s;
  XLLM_HIP_REQUIRE(num_groups >= 0 && num_dst >= 0, "num_groups or num_dst is negative");
  if (num_groups == 0 || num_dst == 0) return XLLM_HIP_OK;
  XLLM_HIP_REQUIRE(src_block_indices != nullptr && dst_block_indices != nullptr && cum_sum != nullptr,
                   "src_block_indices, dst_block_indices or cum_sum is NULL");
  BlockMoveParams p{};
  p.src_ids = src_block_indices;
  p.dst_ids = dst_block_indices;
  p.cum_sum = cum_sum;
  p.num_groups = num_groups;
  p.ids64 = 0;
  p.num_pairs = num_dst;
  p.mode = 0;
  return launch(cache, p, (hipStream_t)stream);
}
