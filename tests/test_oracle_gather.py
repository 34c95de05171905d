"""Pins of the oracle's reshape_from_cache / dequant_from_paged_cache (CPU only)."""
import numpy as np

from oracle import paged_kv_oracle as orc


def _pool(rng, nb=12, H=2, bs=4, D=8):
    k = rng.standard_normal((nb, H, bs, D)).astype(np.float32)
    v = rng.standard_normal((nb, H, bs, D)).astype(np.float32)
    return k, v


def test_reshape_from_cache_is_the_inverse_of_the_kv_write():
    rng = np.random.default_rng(0)
    nb, H, bs, D = 12, 2, 4, 8
    lens = [7, 1, 9]
    tables = [[3, 8, 0], [5, 0, 0], [1, 10, 2]]
    keys = rng.standard_normal((sum(lens), H, D)).astype(np.float32)
    values = rng.standard_normal((sum(lens), H, D)).astype(np.float32)
    slots = np.concatenate([orc.kv_cache_slots(tables[b], bs, 0, n) for b, n in enumerate(lens)])
    kc = np.zeros((nb, H, bs, D), np.float32)
    vc = np.zeros((nb, H, bs, D), np.float32)
    orc.reshape_paged_cache(slots, keys, values, kc, vc, layout="HND")
    k, v = orc.reshape_from_cache(kc, vc, lens, tables)
    assert np.array_equal(k, keys) and np.array_equal(v, values)
    # the NHD layout holds the same values
    k2, _ = orc.reshape_from_cache(kc.transpose(0, 2, 1, 3).copy(), None, lens, tables, layout="NHD")
    assert np.array_equal(k2, keys)


def test_reshape_from_cache_agrees_with_the_attention_oracles_gather():
    rng = np.random.default_rng(1)
    kc, vc = _pool(rng)
    lens = [6, 11]
    tables = [[4, 9, 0], [7, 2, 11]]
    k, v = orc.reshape_from_cache(kc, vc, lens, tables)
    row = 0
    for b, n in enumerate(lens):
        assert np.array_equal(k[row:row + n], orc.gather_sequence(kc, tables[b], n).transpose(1, 0, 2))
        assert np.array_equal(v[row:row + n], orc.gather_sequence(vc, tables[b], n).transpose(1, 0, 2))
        row += n


def test_offsets_known_answer():
    # one head, one channel: the cache element is its own (block, slot) label
    nb, bs = 5, 4
    kc = (np.arange(nb)[:, None] * 10 + np.arange(bs)[None, :]).astype(np.float32).reshape(nb, 1, bs, 1)
    # sequence 0: positions 2..6 of blocks [3, 1]; sequence 1: positions 0..1 of block [4]
    k, _ = orc.reshape_from_cache(kc, None, [5, 2], [[3, 1], [4, 0]], context_seq_offset=[4, 0],
                                  cache_seq_offset=[2, 0], total_rows=10, fill=-1)
    assert k[:, 0, 0].tolist() == [40, 41, -1, -1, 32, 33, 10, 11, 12, -1]


def test_dequant_round_trip_through_the_quantising_write():
    rng = np.random.default_rng(2)
    nb, H, bs, D = 10, 3, 4, 16
    lens = [5, 8]
    tables = [[2, 7], [9, 4]]
    x = (rng.standard_normal((sum(lens), H, D)) * 3).astype(np.float32)
    slots = np.concatenate([orc.kv_cache_slots(tables[b], bs, 0, n) for b, n in enumerate(lens)])
    for kind, dt in (("int8", np.int8), ("fp8", np.uint8)):
        kc = np.zeros((nb, H, bs, D), dt)
        vc = np.zeros((nb, H, bs, D), dt)
        ks = np.zeros((nb, H, bs), np.float32)
        vs = np.zeros((nb, H, bs), np.float32)
        orc.quant_to_paged_cache(slots, x, -x, kc, vc, ks, vs, kind)
        k, v = orc.dequant_from_paged_cache(kc, vc, ks, vs, lens, tables, kind)
        q, s = orc.quantize_per_token_head(x, kind)
        want = orc.dequantize(q, s, kind)
        assert np.array_equal(k, want) and np.array_equal(v, -want)
        assert np.abs(k - x).max() <= np.abs(x).max() / (254 if kind == "int8" else 16) + 1e-6
        # 16-bit outputs are the fp32 values rounded once
        kb, _ = orc.dequant_from_paged_cache(kc, None, ks, None, lens, tables, kind, out_kind="bf16")
        assert np.array_equal(kb, orc.round_to_dtype(want, "bf16").astype(np.float32))


def test_per_channel_mode():
    rng = np.random.default_rng(3)
    nb, H, bs, D = 4, 2, 4, 8
    kc = rng.integers(-127, 128, size=(nb, H, bs, D)).astype(np.int8)
    sc = rng.uniform(0.01, 0.1, size=(H, D)).astype(np.float32)
    k, _ = orc.dequant_from_paged_cache(kc, None, sc, None, [6], [[1, 3]], "int8", quant_mode=0)
    for t in range(6):
        blk = [1, 3][t // bs]
        for h in range(H):
            for d in range(D):
                assert k[t, h, d] == np.float32(kc[blk, h, t % bs, d]) * sc[h, d]
