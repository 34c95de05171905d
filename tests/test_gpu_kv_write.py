"""KV write through slot_mapping on the GPU, bit-exact against the oracle, through the C ABI."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "index_math.json")))
TDT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _bits(t):
    """Bit pattern of a tensor as an integer numpy array (bit-exact comparison, NaN-safe)."""
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()]).numpy()


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("dt", ["bf16", "fp16", "fp32"])
def test_reshape_paged_cache_bit_exact(gpu, layout, dt):
    print("case reshape", layout, dt, flush=True)
    rng = np.random.default_rng(0)
    nb, bs, H, D, T = 37, 16, 8, 128, 29
    slots = rng.choice(nb * bs, size=T, replace=False).astype(np.int32)
    g = torch.Generator().manual_seed(1)
    # key/value are slices of one fused qkv buffer: token stride != H*D (qwen2_attention.cpp:140-142)
    qkv = torch.randn(T, (4 * H + 2 * H) * D, generator=g).to(TDT[dt])
    key = qkv[:, 4 * H * D:5 * H * D].view(T, H, D)
    val = qkv[:, 5 * H * D:].view(T, H, D)
    shape = (nb, bs, H, D) if layout == "NHD" else (nb, H, bs, D)
    kc0 = torch.full(shape, -3.0, dtype=TDT[dt])
    vc0 = torch.full(shape, -5.0, dtype=TDT[dt])
    # oracle on the host copy (numpy has no bf16: run it on the bit patterns)
    kc_ref, vc_ref = _bits(kc0).copy(), _bits(vc0).copy()
    orc.reshape_paged_cache_loops(slots, _bits(key), _bits(val), kc_ref, vc_ref, layout)

    qkv_d = qkv.to(gpu)
    p = ops.ReshapePagedCacheParams(
        key=qkv_d[:, 4 * H * D:5 * H * D].view(T, H, D), value=qkv_d[:, 5 * H * D:].view(T, H, D),
        k_cache=kc0.to(gpu), v_cache=vc0.to(gpu), slot_mapping=torch.from_numpy(slots).to(gpu), kv_layout=layout)
    assert p.key.stride(0) == 6 * H * D
    ops.reshape_paged_cache(p)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(_bits(p.k_cache), kc_ref)
    np.testing.assert_array_equal(_bits(p.v_cache), vc_ref)


def test_reshape_paged_cache_golden_slots(gpu):
    """Slots from the reference's own batch test land where its index math says."""
    print("case reshape golden", flush=True)
    g = GOLDEN["batch_test_basic"]
    bs, H, D = g["block_size"], 2, 8
    slots = np.asarray(g["expected_new_cache_slots"], np.int32)
    T = len(slots)
    key = torch.arange(T * H * D, dtype=torch.float32).view(T, H, D)
    kc = torch.zeros(20, bs, H, D)
    p = ops.ReshapePagedCacheParams(key=key.to(gpu), value=(key + 0.5).to(gpu), k_cache=kc.to(gpu),
                                    v_cache=kc.clone().to(gpu), slot_mapping=torch.from_numpy(slots).to(gpu),
                                    kv_layout="NHD")
    ops.reshape_paged_cache(p)
    torch.cuda.synchronize()
    got = p.k_cache.cpu().view(20 * bs, H, D)
    for t, s in enumerate(slots):
        assert torch.equal(got[s], key[t])
    untouched = np.setdiff1d(np.arange(20 * bs), slots)
    assert float(got[untouched].abs().max()) == 0.0
    assert torch.equal(p.v_cache.cpu().view(20 * bs, H, D)[slots.astype(np.int64)], key + 0.5)


def test_reshape_paged_cache_edge_cases(gpu):
    print("case reshape edges", flush=True)
    nb, bs, H, D = 4, 16, 2, 64
    kc = torch.full((nb, H, bs, D), 9.0, dtype=torch.bfloat16, device=gpu)
    vc = kc.clone()
    # empty input
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(
        key=torch.empty(0, H, D, dtype=torch.bfloat16, device=gpu), value=torch.empty(0, H, D, dtype=torch.bfloat16, device=gpu),
        k_cache=kc, v_cache=vc, slot_mapping=torch.empty(0, dtype=torch.int32, device=gpu)))
    # duplicates of slot 0 (padding rows), a negative slot and an out-of-range slot
    key = torch.arange(5 * H * D, dtype=torch.float32).view(5, H, D).to(torch.bfloat16).to(gpu)
    slots = torch.tensor([0, 0, -1, nb * bs, 17], dtype=torch.int32, device=gpu)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key, value=key, k_cache=kc, v_cache=vc, slot_mapping=slots))
    torch.cuda.synchronize()
    # Two writers to one slot race (the reference's kernel has the same property); each 16-byte piece
    # comes from one of them, so every element equals one of the two candidates.
    row0 = kc[0, :, 0, :]
    assert bool(((row0 == key[0]) | (row0 == key[1])).all())
    assert torch.equal(kc[1, :, 1, :], key[4])
    mask = torch.ones(nb, bs, dtype=torch.bool)
    mask[0, 0] = mask[1, 1] = False
    assert bool((kc.cpu().permute(0, 2, 1, 3)[mask] == 9.0).all())
    # K only
    kc2 = torch.zeros_like(kc)
    ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key[:1], k_cache=kc2,
                                                        slot_mapping=torch.tensor([5], dtype=torch.int32, device=gpu)))
    torch.cuda.synchronize()
    assert torch.equal(kc2[0, :, 5, :], key[0])


def test_reshape_paged_cache_contract_errors(gpu):
    H, D = 2, 64
    kc = torch.zeros(4, H, 16, D, dtype=torch.bfloat16, device=gpu)
    key = torch.zeros(3, H, D, dtype=torch.bfloat16, device=gpu)
    with pytest.raises(_lib.XllmHipError):  # slot_mapping must be int32 (param.h:144-147)
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key, value=key, k_cache=kc, v_cache=kc,
                                                            slot_mapping=torch.zeros(3, dtype=torch.int64, device=gpu)))
    with pytest.raises(_lib.XllmHipError):  # last two dims must be contiguous (reshape_paged_cache.cu:68-69)
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key.transpose(1, 2).contiguous().transpose(1, 2), value=key,
                                                            k_cache=kc, v_cache=kc,
                                                            slot_mapping=torch.zeros(3, dtype=torch.int32, device=gpu)))
    with pytest.raises(_lib.XllmHipError):  # dtype mismatch between key and cache
        ops.reshape_paged_cache(ops.ReshapePagedCacheParams(key=key.float(), value=key.float(), k_cache=kc, v_cache=kc,
                                                            slot_mapping=torch.zeros(3, dtype=torch.int32, device=gpu)))
    with pytest.raises(_lib.XllmHipError):  # quant without scales (ops_api.cpp:198-199)
        ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(key=key, value=key, k_cache=kc.to(torch.int8),
                                                             v_cache=kc.to(torch.int8),
                                                             slot_mapping=torch.zeros(3, dtype=torch.int32, device=gpu)))


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("src", ["bf16", "fp32"])
def test_quant_to_paged_cache_bit_exact(gpu, layout, kind, src):
    print("case quant", layout, kind, src, flush=True)
    rng = np.random.default_rng(3)
    nb, bs, H, D, T = 19, 16, 8, 128, 41
    slots = rng.choice(nb * bs, size=T, replace=False).astype(np.int32)
    g = torch.Generator().manual_seed(2)
    key = (torch.randn(T, H, D, generator=g) * 1.7).to(TDT[src])
    val = (torch.randn(T, H, D, generator=g) * 0.3).to(TDT[src])
    key[3, 1] = 0.0          # all-zero row: scale falls back to the minimum, values stay 0
    key[4, 0] *= 1e-9        # tiny row
    val[5, 2, 7] = 300.0     # one dominant element
    cdt = torch.int8 if kind == "int8" else torch.float8_e4m3fn
    cshape = (nb, H, bs, D) if layout == "HND" else (nb, bs, H, D)
    sshape = cshape[:3]
    kc = torch.zeros(cshape, dtype=torch.int8).view(cdt).to(gpu)
    vc = torch.zeros(cshape, dtype=torch.int8).view(cdt).to(gpu)
    ks = torch.full(sshape, -1.0, device=gpu)
    vs = torch.full(sshape, -1.0, device=gpu)
    ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(
        key=key.to(gpu), value=val.to(gpu), k_cache=kc, v_cache=vc, slot_mapping=torch.from_numpy(slots).to(gpu),
        k_cache_scale=ks, v_cache_scale=vs, kv_layout=layout))
    torch.cuda.synchronize()

    np_dt = np.int8 if kind == "int8" else np.uint8
    kc_ref, vc_ref = np.zeros(cshape, np_dt), np.zeros(cshape, np_dt)
    ks_ref, vs_ref = np.full(sshape, -1.0, np.float32), np.full(sshape, -1.0, np.float32)
    orc.quant_to_paged_cache(slots, key.float().numpy(), val.float().numpy(), kc_ref, vc_ref, ks_ref, vs_ref, kind, layout)
    np.testing.assert_array_equal(ks.cpu().numpy(), ks_ref)
    np.testing.assert_array_equal(vs.cpu().numpy(), vs_ref)
    got_k, got_v = _bits(kc).view(np_dt), _bits(vc).view(np_dt)
    if kind == "fp8":  # +0 and -0 are the same value; compare bytes up to the sign of zero
        for got, ref in ((got_k, kc_ref), (got_v, vc_ref)):
            same = (got == ref) | (((got & 0x7F) == 0) & ((ref & 0x7F) == 0))
            assert same.all(), int((~same).sum())
    else:
        np.testing.assert_array_equal(got_k, kc_ref)
        np.testing.assert_array_equal(got_v, vc_ref)


@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("fused", [False, True])
def test_quantisers_on_nan_inf_and_zero_rows(gpu, kind, fused):
    """Rows holding NaN, +-Inf or only zeros through both quantisers (quant_to_paged_cache and the
    write fused behind the rotary embedding, here with an identity rotation), bit-exact against the
    oracle: absmax skips NaN, and the clamp — in the reference's order,
    xllm/core/kernels/cuda/fp8_quant_utils.cuh:121-122 — turns a NaN quotient into +max."""
    print("case quant non-finite", kind, fused, flush=True)
    nb, bs, H, D, T = 4, 16, 2, 128, 6
    g = torch.Generator().manual_seed(8)
    key = torch.randn(T, H, D, generator=g)
    val = torch.randn(T, H, D, generator=g)
    key[0, 0, 5] = float("nan")
    key[1, 1, 0] = float("inf")
    key[1, 1, 9] = float("-inf")
    key[2, 0] = 0.0
    val[3, 1, 100] = float("nan")
    val[3, 1, 101] = float("-inf")
    val[4, 0] = float("nan")  # nothing finite in the row
    val[5, 1] = 0.0
    key, val = key.to(torch.bfloat16), val.to(torch.bfloat16)
    slots = np.array([3, 17, 40, 5, 63, 22], np.int32)
    cdt = torch.int8 if kind == "int8" else torch.float8_e4m3fn
    cshape, sshape = (nb, H, bs, D), (nb, H, bs)
    kc = torch.zeros(cshape, dtype=torch.int8).view(cdt).to(gpu)
    vc = torch.zeros(cshape, dtype=torch.int8).view(cdt).to(gpu)
    ks = torch.full(sshape, -1.0, device=gpu)
    vs = torch.full(sshape, -1.0, device=gpu)
    sm = torch.from_numpy(slots).to(gpu)
    if fused:
        # one query head of zeros in front, cos = 1 and sin = 0: the rotation leaves K as it is
        qkv = torch.cat([torch.zeros(T, D, dtype=torch.bfloat16), key.reshape(T, -1), val.reshape(T, -1)], 1).to(gpu)
        cos_sin = torch.cat([torch.ones(4, D // 2), torch.zeros(4, D // 2)], 1).to(torch.bfloat16).to(gpu)
        pos = torch.zeros(T, dtype=torch.int32, device=gpu)
        ops.rope_kv_write(qkv, 1, H, D, cos_sin, pos, kc, vc, sm, k_cache_scale=ks, v_cache_scale=vs)
    else:
        ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(key=key.to(gpu), value=val.to(gpu), k_cache=kc, v_cache=vc,
                                                             slot_mapping=sm, k_cache_scale=ks, v_cache_scale=vs))
    torch.cuda.synchronize()
    np_dt = np.int8 if kind == "int8" else np.uint8
    kc_ref, vc_ref = np.zeros(cshape, np_dt), np.zeros(cshape, np_dt)
    ks_ref, vs_ref = np.full(sshape, -1.0, np.float32), np.full(sshape, -1.0, np.float32)
    kf, vf = key.float().numpy(), val.float().numpy()
    if fused:
        # NaN * 0 of the rotation's sine term: a row's NaN reaches its rotation partner too
        half = D // 2
        part = np.concatenate([kf[..., half:], kf[..., :half]], -1)
        kf = np.where(np.isnan(part) | np.isinf(part), np.float32("nan"), kf)
    orc.quant_to_paged_cache(slots, kf, vf, kc_ref, vc_ref, ks_ref, vs_ref, kind, "HND")
    np.testing.assert_array_equal(ks.cpu().numpy(), ks_ref)
    np.testing.assert_array_equal(vs.cpu().numpy(), vs_ref)
    for got, ref in ((_bits(kc).view(np_dt), kc_ref), (_bits(vc).view(np_dt), vc_ref)):
        if kind == "fp8":  # +0 and -0 are the same value
            same = (got == ref) | (((got & 0x7F) == 0) & ((ref & 0x7F) == 0))
            assert same.all(), int((~same).sum())
        else:
            np.testing.assert_array_equal(got, ref)
    # the saturated codes are where the oracle's docstring says they are
    top = 127 if kind == "int8" else 0x7E
    assert int(_bits(kc).view(np_dt)[0, 0, 3, 5]) == top      # NaN element
    assert int(_bits(kc).view(np_dt)[1, 1, 1, 9]) == top      # -inf / inf = NaN -> +max
    assert (_bits(vc).view(np_dt)[3, 0, 15, :] == top).all()  # a row of NaN
