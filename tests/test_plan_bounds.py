"""The split-KV plan on the host: whatever the lengths, the chunk size `choose_chunk` picks yields no
more sequence chunks than the workspace holds records and partial rows for (the plan kernel writes one
record per chunk, the attention kernels one partial per chunk and row), and the choices it is meant to
make for small batches.  The header the kernels are built from is compiled with g++ into a small
library; no GPU is involved."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(REPO, "xllm_wxh_amd", "csrc")


@pytest.fixture(scope="module")
def plan(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("plan") / "libplan_harness.so")
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-I", CSRC,
                    os.path.join(REPO, "tests", "plan_bounds_harness.cpp"), "-o", out], check=True)
    lib = ctypes.CDLL(out)
    lib.harness_choose_chunk.argtypes = [ctypes.c_longlong, ctypes.c_longlong] + [ctypes.c_int] * 7
    lib.harness_max_seq_chunks.restype = ctypes.c_longlong
    return lib


def _chunks(lens, c):
    lens = np.asarray(lens, np.int64)
    return int(np.maximum(1, -(-lens // c)).sum())  # an empty sequence keeps one (empty) chunk


def kernels_for(rows, rng):
    """(workgroup slots, budget of a small batch, rows per item, smallest chunk, tile) of the kernels
    that can serve `rows` query rows per kv head: the generic kernel, the MFMA kernel for that row
    count at head_dim 128 / 64 / 256, and a target lowered by the diagnostic option."""
    out = [(2048, 2048, 1, 64, 32)]
    if rows <= 16:
        out += [(512, 256, 32, 512, 32), (512, 256, 32, 512, 64), (256, 256, 32, 512, 16)]
        out += [(512, 256, 32, 512, 32, 4)]  # work items of four kv heads (a cache whose heads lie side by side)
        out += [(512, 256, 32, 512, 64, 4), (512, 512, 32, 512, 64, 4)]  # ... at head_dim 64 (1-byte rows of 64 bytes)
        out += [(512, 512, 32, 512, 32), (512, 384, 32, 512, 32)]  # 1-byte caches: small batches are cut for more slots
    elif rows <= 32:
        out += [(1024, 1024, 32, 512, 32), (1024, 1024, 32, 512, 64), (512, 512, 32, 512, 16)]
    else:
        out += [(512, 512, 128, 512, 32), (512, 512, 32, 512, 32), (256, 256, 32, 512, 16)]
    lowered = int(rng.choice([1, 64, 200]))
    out += [(lowered, lowered // 2, 32, 512, 32)]
    return out


@pytest.mark.parametrize("seed", range(6))
def test_chunk_count_never_exceeds_the_workspace(plan, seed):
    rng = np.random.default_rng(seed)
    for _ in range(3000):
        hkv = int(rng.choice([1, 2, 4, 8, 16]))
        g = int(rng.choice([1, 2, 4, 7, 8, 16]))
        n = int(rng.choice([1, 1, 2, 4, 8]))
        choices = kernels_for(g * n, rng)
        choice = choices[int(rng.integers(len(choices)))]
        target, small, rows_per_item, min_chunk, tile = choice[:5]
        heads_per_item = choice[5] if len(choice) > 5 and hkv % choice[5] == 0 else 1
        rg = plan.harness_row_groups(n, hkv * g, hkv, rows_per_item)
        if plan.harness_row_groups(n, hkv * g, hkv, 32) > 4:
            continue  # never split
        batch = int(rng.choice([1, 2, 3, 7, 24, 64, 200, 1000]))
        kind = rng.random()
        if kind < 0.25:
            lens = np.full(batch, int(rng.integers(1, 200000)))
        elif kind < 0.5:
            lens = rng.integers(0, 40000, size=batch)
        elif kind < 0.75:
            lens = rng.integers(1, 300, size=batch)
            lens[int(rng.integers(batch))] = int(rng.integers(1000, 1000000))  # one long among short
        else:
            lens = np.clip(np.round(rng.lognormal(np.log(2048), 0.8, size=batch)), 16, 32768).astype(np.int64)
        total, max_len = int(lens.sum()), int(lens.max())
        c = plan.harness_choose_chunk(total, max_len, batch, hkv // heads_per_item, rg, target, small, min_chunk, tile)
        assert c >= min_chunk and c % tile == 0
        bound = plan.harness_max_seq_chunks(batch, n, hkv * g, hkv, 128)
        assert _chunks(lens, c) <= bound, (target, small, hkv, rg, batch, total, max_len, c)


def test_workspace_stays_within_the_shared_buffer_of_the_reference():
    """The reference reserves 128 MiB for split-KV partials (FLAGS_flashinfer_workspace_buffer_size,
    xllm/core/common/global_flags.cpp:564-567): every shape up to 128 query rows per kv head and
    head_dim 256 fits a buffer of that size at batch 64."""
    from xllm_wxh_amd import _lib

    lib = _lib.load()
    for rows, hkv, d in ((1, 8, 128), (4, 8, 128), (16, 8, 128), (32, 8, 128), (96, 8, 256), (128, 4, 256)):
        need = lib.xllm_hip_paged_decode_workspace_bytes(64, rows, hkv, hkv, d)
        assert 0 < need <= 128 << 20, (rows, hkv, d, need)


def test_never_split_steps_need_no_partial_rows():
    """Chunked-prefill and mixed steps (more than 128 query rows per kv head) are never split: their rows are
    written directly and the workspace holds neither chunk records nor partial rows, so ordinary chunks fit
    the 128 MiB the libtorch layer reserves (xllm/core/common/global_flags.cpp:564-567) — 1 x 4096 query
    tokens of 32 heads x 128 would otherwise need 129 MiB of partial rows that nothing touches."""
    from xllm_wxh_amd import _lib

    lib = _lib.load()
    for batch, n in ((1, 4096), (1, 8192), (4, 2048), (8, 1024), (16, 512), (64, 512), (256, 128)):
        need = lib.xllm_hip_paged_decode_workspace_bytes(batch, n, 32, 8, 128)
        assert 0 < need <= 1 << 20, (batch, n, need)
    # 128 rows per kv head are still split (and sized for it)
    assert lib.xllm_hip_paged_decode_workspace_bytes(8, 32, 32, 8, 128) > 1 << 20


def test_small_batch_choices(plan):
    def chunk(lens, hkv=8, rg=1, target=512, small=256):
        lens = np.asarray(lens, np.int64)
        return plan.harness_choose_chunk(int(lens.sum()), int(lens.max()), len(lens), hkv, rg, target, small, 512, 32)

    # equal lengths: 256 / (batch * kv heads) chunks per sequence, each a whole number of tiles
    assert chunk([32768]) == 1024                       # 32 chunks x 8 heads = 256 items
    assert chunk([8192] * 8) == 2048                    # 4 chunks each
    assert chunk([8192] * 16) == 4096                   # 2 chunks each
    assert chunk([8192] * 24) >= 8192                   # 192 (sequence, head) pairs: unsplit
    assert chunk([4096] * 48) >= 4096                   # more pairs than the budget: unsplit
    assert chunk([4096] * 64) >= 4096                   # the Llama-3-8B shape: one item per pair
    assert chunk([20000] * 3) == 2016                   # 10 chunks each, 240 items
    # ragged small batch: the item count stays within the budget ...
    lens = [4000, 2500, 900, 3300, 1700, 2900]
    c = chunk(lens)
    assert _chunks(lens, c) * 8 <= 256
    # ... except that one long sequence among short ones is still cut finely enough to fill the GPU
    lens = [100000] + [1000] * 30
    c = chunk(lens)
    assert 100 <= _chunks(lens, c) * 8 and c <= 100000 // 12
    # lengths so close that a split would only shed short tails: left whole
    lens = [2500 + 16 * i for i in range(20)]
    assert chunk(lens) >= max(lens)
    # the 32-row kernel keeps all its slots as the budget
    assert chunk([32768] * 32, target=1024, small=1024) == 8192
    # a large ragged batch: about 640 items' worth of work per chunk
    rng = np.random.default_rng(0)
    lens = np.clip(np.round(rng.lognormal(np.log(2048), 0.8, size=256)), 16, 32768).astype(np.int64)
    c = chunk(lens)
    assert abs(c - int(lens.sum()) * 8 / 640) <= 32
