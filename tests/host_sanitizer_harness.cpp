// Host-code harness built with -fsanitize=address,undefined by tests/test_host_sanitizers.py: the plan
// arithmetic the decode kernels share with the host, a serial restatement of the plan kernel's chunk
// table writes into a heap array of exactly the workspace's size, the host index producers and the
// argument checks of the libtorch operators (which throw before anything is launched).  Any
// out-of-bounds access, signed overflow or misaligned access aborts the run; otherwise it prints
// "sanitizer harness ok".
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "decode_plan.h"
#include "torch_shim/host_index.h"
#include "torch_shim/ops_api.h"

namespace {

uint64_t rng_state = 0x9E3779B97F4A7C15ull;
uint64_t next_u64() {  // SplitMix64
  uint64_t z = (rng_state += 0x9E3779B97F4A7C15ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
int64_t uniform(int64_t lo, int64_t hi) { return lo + (int64_t)(next_u64() % (uint64_t)(hi - lo + 1)); }

int failures = 0;
void expect(bool ok, const char* what) {
  if (!ok) {
    std::printf("FAILED: %s\n", what);
    ++failures;
  }
}

// The chunk table as decode_plan_kernel fills it (full chunks in sequence order, then the tails by
// decreasing size class), written through a raw pointer into an allocation of max_seq_chunks records.
void plan_sweep() {
  using namespace xllm_hip;
  struct Kernel { int target, small, rows_per_item, min_chunk, tile; };
  const int hkvs[] = {1, 2, 4, 8, 16}, groups[] = {1, 2, 4, 7, 8, 16}, ns[] = {1, 1, 2, 4, 8};
  const int batches[] = {1, 2, 3, 7, 24, 64, 200, 1000};
  for (int iter = 0; iter < 4000; ++iter) {
    const int hkv = hkvs[uniform(0, 4)], g = groups[uniform(0, 5)], n = ns[uniform(0, 4)];
    const int rows = g * n;
    if (never_split(n, hkv * g, hkv)) continue;
    // the kernels that can serve this many rows per kv head: generic, or the MFMA kernel for the row count
    const Kernel mfma = rows <= 16 ? Kernel{512, 256, 32, 512, 32}
                        : rows <= 32 ? Kernel{1024, 1024, 32, 512, 32}
                                     : Kernel{512, 512, uniform(0, 1) ? 128 : 32, 512, 32};
    const Kernel k = uniform(0, 2) == 0 ? Kernel{2048, 2048, 1, 64, 32} : mfma;
    const int rg = row_groups(n, hkv * g, hkv, k.rows_per_item);
    const int batch = batches[uniform(0, 7)];
    std::vector<int> lens(batch);
    const int kind = (int)uniform(0, 3);
    for (int b = 0; b < batch; ++b) {
      lens[b] = kind == 0 ? 0 : kind == 1 ? (int)uniform(0, 40000) : (int)uniform(1, 300);
    }
    if (kind == 0) {
      const int same = (int)uniform(1, 200000);
      for (int& l : lens) l = same;
    }
    if (kind == 2) lens[uniform(0, batch - 1)] = (int)uniform(1000, 1000000);
    long long total = 0, max_len = 0;
    for (int l : lens) {
      total += l;
      max_len = l > max_len ? l : max_len;
    }
    const int chunk = choose_chunk(total, max_len, batch, hkv, rg, k.target, k.small, k.min_chunk, k.tile);
    const WorkspaceLayout w = workspace_layout(batch, n, hkv * g, hkv, 128);
    SeqChunk* table = (SeqChunk*)std::malloc(sizeof(SeqChunk) * (size_t)w.max_seq_chunks);
    int total_full = 0;
    std::vector<int> hist(64, 0), fill(64, 0), start(64, 0);
    for (int l : lens) {
      const int nf = l / chunk, rest = l - nf * chunk;
      total_full += nf;
      if (rest > 0 || l == 0) ++hist[(int)(((long long)rest * 64) / chunk)];
    }
    for (int c = 62; c >= 0; --c) start[c] = start[c + 1] + hist[c + 1];
    int f0 = 0, written = 0;
    for (int b = 0; b < batch; ++b) {
      const int l = lens[b], nf = l / chunk, rest = l - nf * chunk, nt = (rest > 0 || l == 0) ? 1 : 0;
      for (int ci = 0; ci < nf; ++ci) table[f0 + ci] = SeqChunk{b, ci, l, nf + nt};  // (checked by ASan)
      f0 += nf;
      written += nf + nt;
      if (nt) {
        const int cls = (int)(((long long)rest * 64) / chunk);
        table[total_full + start[cls] + fill[cls]++] = SeqChunk{b, nf, l, nf + nt};
      }
    }
    expect(written <= w.max_seq_chunks, "chunk count within the workspace");
    std::free(table);
  }
}

void host_index_checks() {
  namespace hi = xllm::host_index;
  // golden values of the reference's batch test (xllm/core/framework/batch/batch_test.cpp:176-204)
  hi::DecodeBatchInputs in(4);
  in.add_sequence({1, 2, 3}, 0, 9);
  in.add_sequence({4, 5, 6, 7}, 15, 16);
  in.add_sequence({8, 9, 10, 11, 12}, 19, 20);
  in.add_sequence({13, 14, 15}, 4, 8);
  expect(in.new_cache_slots == std::vector<int32_t>({4, 5, 6, 7, 8, 9, 10, 11, 12, 31, 51, 56, 57, 58, 59}), "golden slots");
  expect(in.kv_seq_lens == std::vector<int32_t>({0, 9, 25, 45, 53}), "cumulative kv lengths");
  int32_t width = 0;
  const std::vector<int32_t> flat = in.pad_block_tables(width);
  expect(width == 5 && flat.size() == 20 && flat[3] == 0 && flat[14] == 12, "padded block tables");
  in.pad_decode_batch(1, 8);
  const hi::ExpandedDecodeRows rows =
      hi::expand_decode_rows({8, 15}, {0, 9, 25}, {{1, 2, 3}, {4, 5, 6, 7, 8}}, 4, {0, 1, 2});
  expect(rows.new_cache_slots.size() == 6 && rows.kv_max_seq_len == 18, "expanded rows");
  int thrown = 0;
  try { hi::kv_cache_slots({}, 4, 0, 1); } catch (const std::invalid_argument&) { ++thrown; }
  try { hi::kv_cache_slots({1}, 4, 0, 9); } catch (const std::out_of_range&) { ++thrown; }
  try { hi::calc_slot_id(40, {1, 2}, 4); } catch (const std::out_of_range&) { ++thrown; }
  try { hi::calc_kv_len({0, 5}, 1, 0); } catch (const std::out_of_range&) { ++thrown; }
  try { hi::calc_slot_id(-1, {1, 2}, 4); } catch (const std::invalid_argument&) { ++thrown; }
  expect(thrown == 5, "host index preconditions throw");
}

template <typename F>
bool throws(F&& f) {
  try {
    f();
  } catch (const c10::Error&) {
    return true;
  }
  return false;
}

// Contract violations of the operators: each is caught by a check on the host, before any launch
// (the tensors here live on the CPU, so even a passing check could launch nothing).
void shim_argument_checks() {
  using namespace xllm::kernel;
  ReshapePagedCacheParams p;
  p.key = torch::zeros({3, 2, 8});
  p.value = torch::zeros({3, 2, 8});
  p.k_cache = torch::zeros({2, 2, 4, 8});
  p.v_cache = torch::zeros({2, 2, 4, 8});
  p.slot_mapping = torch::zeros({3}, torch::kLong);
  expect(throws([&] { reshape_paged_cache(p); }), "int64 slot_mapping is refused");
  p.slot_mapping = torch::zeros({3}, torch::kInt);
  expect(throws([&] { quant_to_paged_cache(p); }), "quantising write without scales is refused");
  expect(throws([&] { reshape_paged_cache(p); }), "a cache on the CPU is refused");
  p.direction = true;
  expect(throws([&] { reshape_paged_cache(p); }), "direction = true is refused");
  p.direction = false;
  p.key = torch::zeros({3, 8, 2}).transpose(1, 2);
  expect(throws([&] { reshape_paged_cache(p); }), "a key that is not contiguous in its last two dimensions is refused");
  ReshapeFromCacheParams g;
  g.key = torch::zeros({3, 2, 8});
  g.key_cache = torch::zeros({2, 2, 4, 8});
  g.context_lengths = torch::zeros({1}, torch::kInt);
  expect(throws([&] { reshape_from_cache(g); }), "the linear cache mode is refused");
  std::optional<torch::Tensor> lse;
  torch::Tensor q = torch::zeros({1, 1, 4, 8}), out = torch::zeros({1, 1, 4, 8});
  expect(throws([&] {
           hip::batch_decode(q, p.k_cache, out, torch::zeros({1, 1}, torch::kInt), torch::zeros({1}, torch::kInt),
                             std::nullopt, lse, std::nullopt, std::nullopt, std::nullopt, std::nullopt, std::nullopt,
                             std::nullopt, "float", 0, -1, -1, 1.0f, false, -1);
         }),
         "decode without v_cache is refused");
  expect(throws([&] {
           hip::batch_decode(q, p.k_cache, out, torch::zeros({1, 1}, torch::kLong), torch::zeros({1}, torch::kInt),
                             p.v_cache, lse, std::nullopt, std::nullopt, std::nullopt, std::nullopt, std::nullopt,
                             std::nullopt, "float", 0, -1, -1, 1.0f, false, -1);
         }),
         "an int64 block table is refused");
}

}  // namespace

int main() {
  plan_sweep();
  host_index_checks();
  shim_argument_checks();
  if (failures == 0) std::printf("sanitizer harness ok\n");
  return failures == 0 ? 0 : 1;
}
