"""Pins for the oracle's attention, KV write and quantisers: closed forms, invariants, library
routines and brute force on tiny inputs, chosen so that a dropped term, a wrong head map, an
off-by-one in the causal limit or a transposed operand fails at least one of them."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc


def _case(seed, B, Hq, Hkv, D, bs, lens, n=1, layout="HND", extra_blocks=2):
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, np.int32)
    need = (lens + bs - 1) // bs
    nblocks = int(need.sum()) + extra_blocks
    perm = rng.permutation(nblocks)
    table = np.zeros((B, int(need.max())), np.int32)
    o = 0
    for b in range(B):
        table[b, : need[b]] = perm[o:o + need[b]]
        o += need[b]
    shape = (nblocks, Hkv, bs, D) if layout == "HND" else (nblocks, bs, Hkv, D)
    k = rng.standard_normal(shape).astype(np.float32)
    v = rng.standard_normal(shape).astype(np.float32)
    q = rng.standard_normal((B * n, Hq, D)).astype(np.float32)
    return q, k, v, table, lens


def test_vectorised_equals_scalar_loops():
    q, k, v, table, lens = _case(0, 3, 6, 2, 8, 4, [1, 7, 10], n=2)
    lens = np.maximum(lens, 2)
    a, la = orc.paged_decode_loops(q, k, v, table, lens, 0.37, q_per_seq=2)
    b, lb = orc.paged_decode(q, k, v, table, lens, 0.37, q_per_seq=2)
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-12)
    np.testing.assert_allclose(la, lb, rtol=0, atol=1e-12)
    a, la = orc.paged_decode_loops(q, k, v, table, lens, 0.37, q_per_seq=2, window_left=3)
    b, lb = orc.paged_decode(q, k, v, table, lens, 0.37, q_per_seq=2, window_left=3)
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-12)
    np.testing.assert_allclose(la, lb, rtol=0, atol=1e-12)


def test_nhd_and_hnd_layouts_agree():
    q, k, v, table, lens = _case(1, 2, 4, 2, 8, 4, [5, 9])
    a, _ = orc.paged_decode(q, k, v, table, lens, 0.5)
    b, _ = orc.paged_decode(q, k.transpose(0, 2, 1, 3).copy(), v.transpose(0, 2, 1, 3).copy(), table, lens, 0.5,
                            layout="NHD")
    np.testing.assert_array_equal(a, b)


def test_kv_len_one_returns_value_row():
    # "For kv_len=1, attention output equals value exactly" (xllm/core/runtime/cuda_graph_executor_test.cpp:150-151)
    q, k, v, table, lens = _case(2, 3, 8, 2, 16, 4, [1, 1, 1])
    out, lse = orc.paged_decode(q, k, v, table, lens, 0.25)
    for b in range(3):
        for h in range(8):
            np.testing.assert_array_equal(out[b, h], v[table[b, 0], h // 4, 0].astype(np.float64))
            s = 0.25 * float(np.dot(q[b, h].astype(np.float64), k[table[b, 0], h // 4, 0].astype(np.float64)))
            assert abs(lse[b, h] - s / np.log(2.0)) < 1e-12


def test_identical_keys_give_mean_of_values():
    q, k, v, table, lens = _case(3, 2, 4, 2, 8, 4, [6, 11])
    k[:] = k[0, 0, 0]  # every key row identical -> uniform softmax
    out, lse = orc.paged_decode(q, k, v, table, lens, 1.0)
    for b in range(2):
        L = lens[b]
        for h in range(4):
            rows = np.stack([v[table[b, t // 4], h // 2, t % 4] for t in range(L)]).astype(np.float64)
            np.testing.assert_allclose(out[b, h], rows.mean(0), atol=1e-12)
            s = float(np.dot(q[b, h].astype(np.float64), k[0, 0, 0].astype(np.float64)))
            assert abs(lse[b, h] - (s + np.log(L)) / np.log(2.0)) < 1e-10


def test_matches_torch_softmax_on_dense_copy():
    # Library routine: gather the sequence densely, then torch.softmax + matmul per head.
    q, k, v, table, lens = _case(4, 2, 6, 3, 16, 8, [13, 40])
    out, _ = orc.paged_decode(q, k, v, table, lens, 0.3)
    for b in range(2):
        L = int(lens[b])
        K = torch.from_numpy(np.stack([k[table[b, t // 8], :, t % 8] for t in range(L)])).double()  # [L, Hkv, D]
        V = torch.from_numpy(np.stack([v[table[b, t // 8], :, t % 8] for t in range(L)])).double()
        for h in range(6):
            s = (K[:, h // 2] @ torch.from_numpy(q[b, h]).double()) * 0.3
            o = torch.softmax(s, 0) @ V[:, h // 2]
            np.testing.assert_allclose(out[b, h], o.numpy(), atol=1e-12)


def test_wrong_head_map_is_detected():
    # With g=2, head h must read kv head h // 2, not h % Hkv: the two maps differ for h=1.
    q, k, v, table, lens = _case(5, 1, 4, 2, 8, 4, [9])
    out, _ = orc.paged_decode(q, k, v, table, lens, 0.3)
    L = 9
    K1 = np.stack([k[table[0, t // 4], 1, t % 4] for t in range(L)]).astype(np.float64)
    V1 = np.stack([v[table[0, t // 4], 1, t % 4] for t in range(L)]).astype(np.float64)
    s = K1 @ q[0, 1].astype(np.float64) * 0.3
    p = np.exp(s - s.max())
    wrong = (p / p.sum()) @ V1  # h % Hkv map
    assert np.abs(out[0, 1] - wrong).max() > 1e-3


def test_block_table_permutation_invariance_and_garbage_isolation():
    q, k, v, table, lens = _case(6, 2, 4, 2, 8, 4, [7, 10], extra_blocks=6)
    out, lse = orc.paged_decode(q, k, v, table, lens, 0.4)
    # move every used block somewhere else
    nblocks = k.shape[0]
    perm = np.random.default_rng(0).permutation(nblocks)
    k2, v2 = np.empty_like(k), np.empty_like(v)
    k2[perm] = k
    v2[perm] = v
    table2 = perm[table].astype(np.int32)
    out2, lse2 = orc.paged_decode(q, k2, v2, table2, lens, 0.4)
    np.testing.assert_array_equal(out, out2)
    np.testing.assert_array_equal(lse, lse2)
    # slots beyond seq_len and padded table entries (0) must not matter
    k3, v3 = k.copy(), v.copy()
    for b in range(2):
        L = int(lens[b])
        last_blk = table[b, (L - 1) // 4]
        k3[last_blk, :, L % 4 if L % 4 else 4:] = 1e30
        v3[last_blk, :, L % 4 if L % 4 else 4:] = np.nan
    out3, _ = orc.paged_decode(q, k3, v3, table, lens, 0.4)
    np.testing.assert_array_equal(out, out3)


def test_multi_token_verify_equals_expanded_rows():
    # n draft tokens with a causal mask == n separate decode rows with kv lens L-n+1..L and a
    # duplicated block-table row (xllm/core/runtime/speculative_worker_impl.cpp:230-243).
    n = 3
    q, k, v, table, lens = _case(7, 2, 4, 2, 8, 4, [9, 14], n=n)
    out, lse = orc.paged_decode(q, k, v, table, lens, 0.4, q_per_seq=n)
    table_x = np.repeat(table, n, axis=0)
    lens_x = np.concatenate([[L - (n - 1 - j) for j in range(n)] for L in lens]).astype(np.int32)
    out_x, lse_x = orc.paged_decode(q, k, v, table_x, lens_x, 0.4, q_per_seq=1)
    np.testing.assert_allclose(out, out_x, rtol=0, atol=1e-13)
    np.testing.assert_allclose(lse, lse_x, rtol=0, atol=1e-13)


def test_split_merge_identity():
    # Attention over [0, L) == lse_combine(attention over [0, s), attention over [s, L)).
    q, k, v, table, lens = _case(8, 1, 4, 2, 8, 4, [23])
    full, lse_full = orc.paged_decode(q, k, v, table, lens, 0.6)
    s = 12
    a, lse_a = orc.paged_decode(q, k, v, table, np.array([s], np.int32), 0.6)
    # second half: rebuild a table that starts at token s (s is a multiple of the block size)
    table_b = table[:, s // 4:]
    b, lse_b = orc.paged_decode(q, k, v, table_b, np.array([23 - s], np.int32), 0.6)
    merged, lse_m = orc.lse_combine(a, lse_a, b, lse_b)
    np.testing.assert_allclose(merged, full, atol=1e-12)
    np.testing.assert_allclose(lse_m, lse_full, atol=1e-12)


def test_lse_combine_two_element_closed_form():
    o_a, o_b = np.array([[[1.0, 2.0]]]), np.array([[[3.0, -2.0]]])
    out, lse = orc.lse_combine(o_a, np.array([[1.0]]), o_b, np.array([[3.0]]))
    w_a, w_b = 2.0 / (2.0 + 8.0), 8.0 / (2.0 + 8.0)
    np.testing.assert_allclose(out, w_a * o_a + w_b * o_b, atol=1e-15)
    assert abs(lse[0, 0] - np.log2(10.0)) < 1e-15


def test_sliding_window_keeps_last_keys_only():
    q, k, v, table, lens = _case(9, 1, 2, 1, 8, 4, [20])
    w = 5
    out, _ = orc.paged_decode(q, k, v, table, lens, 0.4, window_left=w)
    # same as attention over a sequence made of the last w+1 tokens only
    toks = range(20 - 1 - w, 20)
    K = np.stack([k[table[0, t // 4], 0, t % 4] for t in toks]).astype(np.float64)
    V = np.stack([v[table[0, t // 4], 0, t % 4] for t in toks]).astype(np.float64)
    for h in range(2):
        s = K @ q[0, h].astype(np.float64) * 0.4
        p = np.exp(s - s.max())
        np.testing.assert_allclose(out[0, h], (p / p.sum()) @ V, atol=1e-12)


def test_zero_length_sequence_gives_zeros():
    q, k, v, table, lens = _case(10, 2, 2, 1, 8, 4, [0, 5])
    out, lse = orc.paged_decode(q, k, v, table, lens, 0.4)
    assert (out[0] == 0).all() and np.isneginf(lse[0]).all()
    assert np.isfinite(lse[1]).all()


# ---- KV write -------------------------------------------------------------------------------


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_reshape_paged_cache_vectorised_equals_literal_loops(layout):
    rng = np.random.default_rng(0)
    nb, bs, H, D, T = 6, 4, 2, 8, 5
    shape = (nb, bs, H, D) if layout == "NHD" else (nb, H, bs, D)
    slots = np.array([4, 23, 0, 9, 10], np.int32)
    keys = rng.standard_normal((T, H, D)).astype(np.float32)
    vals = rng.standard_normal((T, H, D)).astype(np.float32)
    kc1, vc1 = np.full(shape, -7.0, np.float32), np.full(shape, -9.0, np.float32)
    kc2, vc2 = kc1.copy(), vc1.copy()
    orc.reshape_paged_cache_loops(slots, keys, vals, kc1, vc1, layout)
    orc.reshape_paged_cache(slots, keys, vals, kc2, vc2, layout)
    np.testing.assert_array_equal(kc1, kc2)
    np.testing.assert_array_equal(vc1, vc2)
    # closed form on the flat NHD buffer: dst = slot * H * D + h * D + d (reshape_paged_cache.cu:41-56)
    if layout == "NHD":
        flat = kc1.reshape(-1)
        for t, s in enumerate(slots):
            np.testing.assert_array_equal(flat[s * H * D:(s + 1) * H * D], keys[t].reshape(-1))
    # untouched slots keep the poison value
    untouched = np.ones(nb * bs, bool)
    untouched[slots] = False
    kview = kc1 if layout == "NHD" else kc1.transpose(0, 2, 1, 3)
    assert (kview.reshape(nb * bs, -1)[untouched] == -7.0).all()


def test_reshape_paged_cache_duplicate_slot_zero():
    # padding rows all write slot 0 (xllm/core/framework/batch/batch_input_builder.cpp:517): legal.
    nb, bs, H, D = 2, 4, 1, 4
    kc, vc = np.zeros((nb, bs, H, D), np.float32), np.zeros((nb, bs, H, D), np.float32)
    keys = np.arange(3 * H * D, dtype=np.float32).reshape(3, H, D)
    orc.reshape_paged_cache_loops(np.array([0, 0, 5]), keys, keys, kc, vc, "NHD")
    np.testing.assert_array_equal(kc[0, 0], keys[1])  # sequential loops: the last duplicate wins
    np.testing.assert_array_equal(kc[1, 1], keys[2])


# ---- quantisers -----------------------------------------------------------------------------


def test_e4m3_decode_matches_torch_for_every_byte():
    b = np.arange(256, dtype=np.uint8)
    ref = torch.from_numpy(b).view(torch.float8_e4m3fn).float().numpy()
    mine = orc.e4m3fn_to_float(b)
    np.testing.assert_array_equal(np.isnan(ref), np.isnan(mine))
    np.testing.assert_array_equal(ref[~np.isnan(ref)], mine[~np.isnan(mine)])
    assert mine[0x7E] == 448.0 and mine[0x08] == 2.0 ** -6 and mine[0x01] == 2.0 ** -9


def test_e4m3_encode_matches_torch_round_to_nearest_even():
    b = np.arange(256, dtype=np.uint8)
    vals = orc.e4m3fn_to_float(b)
    finite = np.sort(vals[~np.isnan(vals)])
    # every representable value, every midpoint between neighbours, and points just off the midpoints
    mids = (finite[:-1].astype(np.float64) + finite[1:].astype(np.float64)) / 2
    probes = np.concatenate([finite, mids, np.nextafter(mids.astype(np.float32), np.float32(1e9)),
                             np.nextafter(mids.astype(np.float32), np.float32(-1e9)),
                             np.random.default_rng(0).uniform(-448, 448, 20000)]).astype(np.float32)
    probes = probes[np.abs(probes) <= 448.0]
    ref = torch.from_numpy(probes).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = orc.float_to_e4m3fn(probes)
    # +0 and -0 both decode to zero; compare decoded values and the sign bit of non-zeros
    np.testing.assert_array_equal(orc.e4m3fn_to_float(ref), orc.e4m3fn_to_float(mine))
    nz = orc.e4m3fn_to_float(ref) != 0
    np.testing.assert_array_equal(ref[nz], mine[nz])


@pytest.mark.parametrize("kind,qmax", [("int8", 127.0), ("fp8", 448.0)])
def test_quantiser_scale_and_roundtrip(kind, qmax):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 3, 128)).astype(np.float32)
    x[0, 0] = 0.0  # an all-zero row must not divide by zero
    q, s = orc.quantize_per_token_head(x, kind)
    amax = np.abs(x).max(-1)
    np.testing.assert_array_equal(s[amax > 1e-3], (amax / np.float32(qmax)).astype(np.float32)[amax > 1e-3])
    assert s[0, 0] > 0 and np.all(orc.dequantize(q, s, kind)[0, 0] == 0)
    deq = orc.dequantize(q, s, kind)
    # error bound: half a quantisation step (int8) / 2^-4 relative (e4m3: 3 mantissa bits)
    if kind == "int8":
        assert np.all(np.abs(deq - x) <= 0.5 * s[..., None] * (1 + 1e-6))
        assert q.dtype == np.int8 and q.min() >= -127
        # the element holding the absmax maps to +-127 exactly
        assert np.all(np.abs(q[1:]).max(-1) == 127)
    else:
        assert np.all(np.abs(deq - x) <= np.maximum(np.abs(x) * 2.0 ** -4, s[..., None] * 2.0 ** -10) * (1 + 1e-6))
        assert np.all(np.abs(orc.e4m3fn_to_float(q[1:])).max(-1) == 448.0)


def test_int8_round_half_even_and_saturation():
    x = np.zeros((1, 4), np.float32)
    x[0] = [127.0, 0.5, 1.5, -2.5]  # scale = 1 -> y = x
    q, s = orc.quantize_per_token_head(x, "int8")
    assert s[0] == 1.0 and q[0].tolist() == [127, 0, 2, -2]


def test_quant_to_paged_cache_scatter():
    rng = np.random.default_rng(2)
    nb, bs, H, D, T = 4, 4, 2, 16, 3
    keys = rng.standard_normal((T, H, D)).astype(np.float32)
    vals = rng.standard_normal((T, H, D)).astype(np.float32)
    kc, vc = np.zeros((nb, H, bs, D), np.int8), np.zeros((nb, H, bs, D), np.int8)
    ks, vs = np.zeros((nb, H, bs), np.float32), np.zeros((nb, H, bs), np.float32)
    slots = np.array([5, 14, 3])
    orc.quant_to_paged_cache(slots, keys, vals, kc, vc, ks, vs, "int8")
    qk, sk = orc.quantize_per_token_head(keys, "int8")
    for t, s in enumerate(slots):
        np.testing.assert_array_equal(kc[s // bs, :, s % bs], qk[t])
        np.testing.assert_array_equal(ks[s // bs, :, s % bs], sk[t])
    assert np.count_nonzero(ks) == T * H


# ---- torch-CPU restatement (the timed CPU baseline) -------------------------------------------


@pytest.mark.parametrize("n", [1, 3])
def test_torch_cpu_path_matches_numpy_oracle(n):
    from oracle import torch_cpu_path as tcp

    q, k, v, table, lens = _case(20, 3, 8, 2, 16, 4, [5, 9, 30], n=n)
    ref, _ = orc.paged_decode(q, k, v, table, lens, 0.3, q_per_seq=n)
    got = tcp.paged_decode(torch.from_numpy(q), torch.from_numpy(k), torch.from_numpy(v), torch.from_numpy(table),
                           torch.from_numpy(lens), 0.3, q_per_seq=n)
    np.testing.assert_allclose(got.numpy(), ref, atol=2e-5)


def test_torch_cpu_path_quantised_and_write():
    from oracle import torch_cpu_path as tcp

    q, k, v, table, lens = _case(21, 2, 4, 2, 16, 4, [7, 12])
    qk, sk = orc.quantize_per_token_head(k, "int8")
    qv, sv = orc.quantize_per_token_head(v, "int8")
    ref, _ = orc.paged_decode(q, qk, qv, table, lens, 0.3, k_scale=sk, v_scale=sv, kind="int8")
    got = tcp.paged_decode(torch.from_numpy(q), torch.from_numpy(qk), torch.from_numpy(qv), torch.from_numpy(table),
                           torch.from_numpy(lens), 0.3, k_scale=torch.from_numpy(sk), v_scale=torch.from_numpy(sv))
    np.testing.assert_allclose(got.numpy(), ref, atol=2e-5)
    # KV write by advanced indexing == the literal loops
    slots = np.array([3, 17, 9], np.int32)
    keys = np.random.default_rng(0).standard_normal((3, 2, 16)).astype(np.float32)
    kc1, vc1 = k.copy(), v.copy()
    orc.reshape_paged_cache_loops(slots, keys, keys * 2, kc1, vc1, "HND")
    kc2, vc2 = torch.from_numpy(k.copy()), torch.from_numpy(v.copy())
    tcp.reshape_paged_cache(torch.from_numpy(slots), torch.from_numpy(keys), torch.from_numpy(keys * 2), kc2, vc2)
    np.testing.assert_array_equal(kc2.numpy(), kc1)
    np.testing.assert_array_equal(vc2.numpy(), vc1)


def test_quantisers_on_non_finite_rows_follow_c_fmaxf_fminf(tmp_path):
    """NaN, +-Inf and all-zero rows: the oracle's quantiser against the clamp of
    xllm/core/kernels/cuda/fp8_quant_utils.cuh:121-122 compiled as C (fmaxf / fminf return the other
    operand for a NaN, so a NaN quotient saturates to +max and absmax skips NaN elements), with the
    e4m3 encoding of the clamped value taken from torch."""
    import ctypes
    import os
    import subprocess

    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quant_clamp_ref.c")
    so = str(tmp_path / "libquant_clamp_ref.so")
    subprocess.run(["gcc", "-O1", "-shared", "-fPIC", src, "-lm", "-o", so], check=True)
    lib = ctypes.CDLL(so)
    lib.ref_absmax.restype = ctypes.c_float
    lib.ref_absmax.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.ref_scaled_clamp.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                     ctypes.c_void_p]
    rng = np.random.default_rng(5)
    rows = rng.standard_normal((6, 64)).astype(np.float32)
    rows[0, 3] = np.nan
    rows[1, 0], rows[1, 9] = np.inf, -np.inf
    rows[2] = 0.0
    rows[3] = np.nan
    rows[4, 5], rows[4, 6] = np.nan, -np.inf
    for kind, qmax, min_scale in (("int8", 127.0, np.finfo(np.float32).eps), ("fp8", 448.0, 1.0 / (448.0 * 512.0))):
        q, s = orc.quantize_per_token_head(rows, kind)
        for r in range(rows.shape[0]):
            row = np.ascontiguousarray(rows[r])
            amax = lib.ref_absmax(row.ctypes.data, row.size)
            scale = np.float32(max(np.float32(amax) / np.float32(qmax), np.float32(min_scale)))
            assert s[r] == scale or (np.isinf(s[r]) and np.isinf(scale))
            y = np.empty_like(row)
            lib.ref_scaled_clamp(row.ctypes.data, row.size, ctypes.c_float(float(scale)), ctypes.c_float(qmax),
                                 int(kind == "int8"), y.ctypes.data)
            assert not np.isnan(y).any()
            if kind == "int8":
                np.testing.assert_array_equal(q[r], y.astype(np.int8))
            else:
                want = torch.from_numpy(y).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
                same = (q[r] == want) | (((q[r] & 0x7F) == 0) & ((want & 0x7F) == 0))
                assert same.all()
        top = 127 if kind == "int8" else 0x7E
        assert q[0, 3] == top and q[1, 0] == top and q[1, 9] == top and (q[3] == top).all() and (q[2] == 0).all()
