"""The decode schedule made on the host from the kv lengths (csrc/decode_schedule.h, behind
xllm_hip_paged_decode_plan_host): compiled with g++ and checked on the CPU.  Whatever the lengths, the records
cover every token of every sequence exactly once with tile-aligned chunks, a sequence's partial slots are
consecutive and in sequence order, the dispatch order is longest first, no sequence has more chunks than a merge
loads, and nothing exceeds the records the workspace holds and the launch covers."""
import ctypes
import os
import subprocess

import numpy as np
import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(REPO, "xllm_wxh_amd", "csrc")


@pytest.fixture(scope="module")
def harness(tmp_path_factory):
    out = str(tmp_path_factory.mktemp("sched") / "libsched_harness.so")
    subprocess.run(["g++", "-O1", "-std=c++17", "-shared", "-fPIC", "-I", CSRC,
                    os.path.join(REPO, "tests", "plan_bounds_harness.cpp"), "-o", out], check=True)
    lib = ctypes.CDLL(out)
    ip, llp = ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_longlong)
    lib.harness_host_schedule.argtypes = [ip] + [ctypes.c_int] * 6 + [ctypes.c_longlong, ctypes.c_int, ctypes.c_double, ctypes.c_double] + \
        [ctypes.c_int] * 4 + [ip, ip, ip, ip, llp]
    lib.harness_host_schedule.restype = ctypes.c_longlong
    return lib


def schedule(lib, lens, per=8, slots=512, tile=32, min_chunk=512, cap=None, max_per_seq=32, overhead=200.0, len_cap=2**31 - 1,
             q_per_seq=1, hq=32, hkv=8, d=128, solo=2.0):
    lens = np.ascontiguousarray(lens, np.int32)
    B = len(lens)
    room = 4096 + B
    rec = np.zeros((room, 8), np.int32)
    kv_len, first, cnt = np.zeros(B, np.int32), np.zeros(B + 1, np.int32), np.zeros(B, np.int32)
    out = np.zeros(4, np.int64)
    ptr = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int))
    n = lib.harness_host_schedule(ptr(lens), B, len_cap, per, slots, tile, min_chunk, cap if cap is not None else room,
                                  max_per_seq, overhead, solo, q_per_seq, hq, hkv, d, ptr(rec), ptr(kv_len), ptr(first), ptr(cnt),
                                  out.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)))
    return n, rec[:max(n, 0)], kv_len, first, cnt, out


def check(lens, n, rec, kv_len, first, cnt, out, per, tile, min_chunk, max_per_seq, len_cap=2**31 - 1):
    lens = np.clip(np.asarray(lens, np.int64), 0, len_cap)
    B = len(lens)
    assert n == cnt.sum() == first[B] and out[1] == n * per
    assert np.array_equal(kv_len, lens)
    assert np.array_equal(first[:B], np.concatenate([[0], np.cumsum(cnt)[:-1]]))
    seq, chunk, ln, chunks, t0, t1, slot = (rec[:, i] for i in range(7))
    assert np.array_equal(np.sort(slot), np.arange(n))                # every partial slot once
    assert np.array_equal(slot, first[seq] + chunk)                  # ... at its sequence's place
    assert np.array_equal(ln, lens[seq]) and np.array_equal(chunks, cnt[seq])
    assert np.all(t0 % tile == 0) and np.all(t1 <= ln) and np.all((t1 > t0) | (ln == 0))
    size = t1 - t0
    assert np.all(size[:-1] >= size[1:])                             # longest first
    assert cnt.max() <= max_per_seq
    for b in range(B):
        mine = np.nonzero(seq == b)[0]
        order = mine[np.argsort(chunk[mine])]
        assert np.array_equal(chunk[order], np.arange(cnt[b]))
        assert t0[order][0] == 0 and t1[order][-1] == lens[b]
        assert np.array_equal(t0[order][1:], t1[order][:-1])         # the chunks tile the sequence
        if cnt[b] > 1:
            assert size[order][:-1].min() >= min_chunk               # only a sequence's last chunk may be short
            assert size[order][:-1].max() - size[order][:-1].min() == 0


@pytest.mark.parametrize("seed", range(4))
def test_records_cover_every_sequence_once(harness, seed):
    rng = np.random.default_rng(seed)
    for _ in range(300):
        B = int(rng.choice([1, 2, 3, 8, 33, 48, 64, 136, 256, 700]))
        kind = rng.integers(4)
        if kind == 0:
            lens = np.full(B, int(rng.integers(1, 40000)))
        elif kind == 1:
            lens = np.clip(np.round(rng.lognormal(np.log(rng.choice([300, 2048, 8192])), 0.8, B)), 1, 200000)
        elif kind == 2:
            lens = rng.integers(0, 600, B)
        else:
            lens = np.concatenate([[int(rng.integers(20000, 300000))], rng.integers(0, 3000, B - 1)])
        per = int(rng.choice([1, 2, 8, 16]))
        slots = int(rng.choice([256, 512, 1024, 2048]))
        tile = int(rng.choice([16, 32, 64]))
        min_chunk = int(rng.choice([64, 512]))
        max_per_seq = int(rng.choice([32, 256]))
        cap = B + int(rng.choice([1, 50, 400, 3000]))
        len_cap = int(rng.choice([2**31 - 1, 50000]))
        n, rec, kv_len, first, cnt, out = schedule(harness, lens, per, slots, tile, min_chunk, cap, max_per_seq,
                                                   float(rng.choice([0.0, 100.0, 400.0])), len_cap)
        assert 0 <= n <= cap, (n, cap)
        check(lens, n, rec, kv_len, first, cnt, out, per, tile, min_chunk, max_per_seq, len_cap)


def test_the_cut_follows_the_lengths(harness):
    # one long sequence among short ones: only the long one is cut, into equal chunks
    lens = [40000] + [300] * 63
    n, rec, kv_len, first, cnt, out = schedule(harness, lens)
    assert cnt[0] > 1 and np.all(cnt[1:] == 1)
    # equal sequences that fill the slots exactly stay whole
    n, rec, kv_len, first, cnt, out = schedule(harness, [4096] * 64)
    assert n == 64 and out[0] == 0
    # a small batch is cut for the slots: 8 sequences x 8 heads over 512 slots -> a workgroup per CU (4 chunks each)
    # where one workgroup streams at its CU's full rate, every slot (8 chunks) where it takes two
    n, rec, kv_len, first, cnt, out = schedule(harness, [8192] * 8, solo=2.0)
    assert np.all(cnt == 4)
    n, rec, kv_len, first, cnt, out = schedule(harness, [8192] * 8, solo=1.3)
    assert np.all(cnt == 8)
    # ragged: a lognormal batch ends within a fifth of the even share of the work
    rng = np.random.default_rng(3)
    lens = np.clip(np.round(rng.lognormal(np.log(8192), 0.8, 48)), 16, 65536).astype(np.int64)
    n, rec, kv_len, first, cnt, out = schedule(harness, lens)
    even = lens.sum() / (512 / 8)
    assert out[2] <= 1.2 * even + 2000, (out[2], even)
    # an empty batch entry keeps one empty record
    n, rec, kv_len, first, cnt, out = schedule(harness, [0, 5, 0])
    assert n == 3 and np.all(cnt == 1)
