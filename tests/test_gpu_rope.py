"""RMSNorm + rotary embedding + KV write in one launch, on the GPU, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu

TDT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}
# one unit in the last place of the element type, relative (plus the smallest step near zero); for
# fp32 the element type is the arithmetic type, so the bound is that of a few float operations with
# cancellation in x cos - y sin
ULP = {"bf16": (2.0 ** -7, 1e-30), "fp16": (2.0 ** -10, 6.0e-8), "fp32": (1e-5, 2e-6)}


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()]).numpy()


def _inputs(T, hq, hk, hv, D, R, maxpos, kind, seed, cache_kind="fp32", scale=0.2):
    g = torch.Generator().manual_seed(seed)
    dt = TDT[kind]
    qkv = (torch.randn(T, (hq + hk + hv) * D, generator=g) * scale).to(dt)
    qw, kw = torch.randn(D, generator=g).to(dt), torch.randn(D, generator=g).to(dt)
    theta = torch.rand(maxpos, R // 2, generator=g) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(TDT[cache_kind])
    pos = torch.randint(0, maxpos, (T,), generator=g)
    return qkv, qw, kw, cos_sin, pos


@pytest.mark.parametrize("T,hq,hk,hv,D,R,maxpos,interleaved,kind", [
    (17, 8, 4, 4, 128, 128, 512, False, "fp16"),   # fused_qknorm_rope_test.cpp MatchesReferenceNeoX
    (11, 6, 2, 2, 64, 64, 256, True, "bf16"),      # fused_qknorm_rope_test.cpp MatchesReferenceInterleaved
    (33, 32, 8, 8, 128, 128, 4096, False, "bf16"),  # Llama-3-8B / Qwen3 head counts
    (5, 4, 2, 2, 128, 64, 64, False, "bf16"),      # partial rotary
    (5, 4, 2, 2, 256, 128, 64, True, "fp32"),
    (3, 2, 1, 1, 192, 96, 64, False, "fp16"),      # head_dim not a power of two
])
def test_fused_qk_norm_rope_matches_oracle(gpu, T, hq, hk, hv, D, R, maxpos, interleaved, kind):
    print("case fused_qk_norm_rope", T, hq, hk, hv, D, R, interleaved, kind, flush=True)
    qkv, qw, kw, cos_sin, pos = _inputs(T, hq, hk, hv, D, R, maxpos, kind, seed=2026)
    want = orc.fused_qk_norm_rope(qkv.float().numpy(), hq, hk, hv, D, 1e-6, qw.float().numpy(), kw.float().numpy(),
                                  cos_sin.numpy(), interleaved, pos.numpy(), kind)
    d = qkv.to(gpu)
    ops.fused_qk_norm_rope(d, hq, hk, hv, D, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), interleaved, pos.to(gpu))
    torch.cuda.synchronize()
    got = d.float().cpu().numpy().astype(np.float64)
    rel, tiny = ULP[kind]
    # float arithmetic in another order than the oracle's float64: one unit in the last place
    assert np.all(np.abs(got - want) <= rel * np.abs(want) + tiny), float(np.abs(got - want).max())
    # the reference's own tolerance for its kernel (fused_qknorm_rope_test.cpp:186,240)
    assert np.allclose(got, want, rtol=2e-3 if kind != "bf16" else 2e-2, atol=2e-3 if kind != "bf16" else 2e-2)
    assert np.array_equal(_bits(d[:, (hq + hk) * D:]), _bits(qkv[:, (hq + hk) * D:]))  # v untouched


@pytest.mark.parametrize("kind", ["bf16", "fp16"])
@pytest.mark.parametrize("is_neox", [True, False])
def test_rotary_embedding_every_op_rounded_is_bit_exact(gpu, kind, is_neox):
    print("case rotary_embedding", kind, is_neox, flush=True)
    T, hq, hk, D = 19, 8, 2, 128
    qkv, _, _, cos_sin, pos = _inputs(T, hq, hk, hk, D, D, 300, kind, seed=8, cache_kind=kind, scale=1.0)
    want = orc.fused_qk_norm_rope(qkv.float().numpy(), hq, hk, hk, D, 0.0, None, None, cos_sin.float().numpy(),
                                  not is_neox, pos.numpy(), kind, round_each_op=True)
    d = qkv.to(gpu)
    q = d[:, :hq * D]                      # slices of the fused buffer, as in qwen2_attention.cpp:140-142
    k = d[:, hq * D:(hq + hk) * D]
    ops.rotary_embedding(pos.to(gpu), q, k, cos_sin.to(gpu), is_neox)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(d), _bits(torch.from_numpy(want).to(TDT[kind])))


@pytest.mark.parametrize("cache_kind", ["bf16", "int8", "fp8"])
@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("norm", [True, False])
def test_rope_kv_write_equals_the_two_steps(gpu, cache_kind, layout, norm):
    print("case rope_kv_write", cache_kind, layout, norm, flush=True)
    T, hq, hk, D, nb, bs = 29, 8, 2, 128, 9, 16
    qkv, qw, kw, cos_sin, pos = _inputs(T, hq, hk, hk, D, D, 128, "bf16", seed=11, scale=1.0)
    if not norm:
        qw = kw = None
    rng = np.random.default_rng(2)
    slots = rng.choice(nb * bs, size=T, replace=False).astype(np.int32)
    slots[3], slots[7] = -1, nb * bs + 5  # skipped
    slots = torch.from_numpy(slots).to(gpu)
    shape = (nb, hk, bs, D) if layout == "HND" else (nb, bs, hk, D)
    cdt = {"bf16": torch.bfloat16, "int8": torch.int8, "fp8": torch.float8_e4m3fn}[cache_kind]

    def fresh():
        if cache_kind == "bf16":
            return (torch.full(shape, 7.0, dtype=cdt, device=gpu), torch.full(shape, 9.0, dtype=cdt, device=gpu),
                    None, None)
        z = torch.full(shape, 3, dtype=torch.int8, device=gpu).view(cdt)
        return z.clone(), z.clone(), torch.full(shape[:3], -1.0, device=gpu), torch.full(shape[:3], -2.0, device=gpu)

    gw = (qw.to(gpu), kw.to(gpu)) if norm else (None, None)
    # two steps: norm + rotation, then the KV write from the updated buffer
    a = qkv.to(gpu)
    ka, va, ksa, vsa = fresh()
    if norm:
        ops.fused_qk_norm_rope(a, hq, hk, hk, D, 1e-6, gw[0], gw[1], cos_sin.to(gpu), False, pos.to(gpu))
    else:
        ops._rope_call(a, hq, hk, hk, D, 0.0, None, None, cos_sin.to(gpu), False, pos.to(gpu), False)
    key = a[:, hq * D:(hq + hk) * D].view(T, hk, D)
    val = a[:, (hq + hk) * D:].view(T, hk, D)
    params = ops.ReshapePagedCacheParams(key=key, value=val, k_cache=ka, v_cache=va, slot_mapping=slots,
                                         k_cache_scale=ksa, v_cache_scale=vsa, kv_layout=layout)
    (ops.reshape_paged_cache if cache_kind == "bf16" else ops.quant_to_paged_cache)(params)
    # one launch
    b = qkv.to(gpu)
    kb, vb, ksb, vsb = fresh()
    ops.rope_kv_write(b, hq, hk, D, cos_sin.to(gpu), pos.to(gpu), kb, vb, slots, q_weight=gw[0], k_weight=gw[1],
                      eps=1e-6, k_cache_scale=ksb, v_cache_scale=vsb, kv_layout=layout)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(a), _bits(b))
    assert np.array_equal(_bits(ka), _bits(kb)) and np.array_equal(_bits(va), _bits(vb))
    if ksa is not None:
        assert np.array_equal(_bits(ksa), _bits(ksb)) and np.array_equal(_bits(vsa), _bits(vsb))
    # and the cache holds the rotated keys: check one token against the oracle's dequantised row
    if cache_kind == "bf16":
        t = 0
        s = int(slots[t])
        row = kb[s // bs, :, s % bs, :] if layout == "HND" else kb[s // bs, s % bs, :, :]
        assert np.array_equal(_bits(row), _bits(b[t, hq * D:(hq + hk) * D].view(hk, D)))


@pytest.mark.parametrize("cache_kind", ["bf16", "int8"])
def test_prefill_sized_launch(gpu, cache_kind):
    """A prefill-sized launch (3001 tokens x 48 heads, a ragged last workgroup): the rotation bit-exact
    against the oracle, and the cache rows and scales equal to those of the separate KV write."""
    print("case rope many tokens", cache_kind, flush=True)
    T, hq, hk, D, bs = 3001, 32, 8, 128, 16
    nb = (T + bs - 1) // bs + 2
    qkv, _, _, cos_sin, pos = _inputs(T, hq, hk, hk, D, D, 4096, "bf16", seed=5, cache_kind="bf16", scale=1.0)
    want = orc.fused_qk_norm_rope(qkv.float().numpy(), hq, hk, hk, D, 0.0, None, None, cos_sin.float().numpy(),
                                  False, pos.numpy(), "bf16", round_each_op=True)
    slots = torch.from_numpy(np.random.default_rng(4).permutation(nb * bs)[:T].astype(np.int32)).to(gpu)
    shape = (nb, hk, bs, D)
    if cache_kind == "bf16":
        kc, vc = torch.zeros(shape, dtype=torch.bfloat16, device=gpu), torch.zeros(shape, dtype=torch.bfloat16, device=gpu)
        ks = vs = None
    else:
        kc, vc = torch.zeros(shape, dtype=torch.int8, device=gpu), torch.zeros(shape, dtype=torch.int8, device=gpu)
        ks, vs = torch.zeros(shape[:3], device=gpu), torch.zeros(shape[:3], device=gpu)
    d = qkv.to(gpu)
    ops.rope_kv_write(d, hq, hk, D, cos_sin.to(gpu), pos.to(gpu), kc, vc, slots, round_each_op=True,
                      k_cache_scale=ks, v_cache_scale=vs)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(d), _bits(torch.from_numpy(want).to(torch.bfloat16)))
    # the separate write of the rotated keys and the values
    k2, v2 = torch.zeros_like(kc), torch.zeros_like(vc)
    ks2 = vs2 = None
    if ks is not None:
        ks2, vs2 = torch.zeros_like(ks), torch.zeros_like(vs)
    params = ops.ReshapePagedCacheParams(key=d[:, hq * D:(hq + hk) * D].view(T, hk, D), value=d[:, (hq + hk) * D:].view(T, hk, D),
                                         k_cache=k2, v_cache=v2, slot_mapping=slots, k_cache_scale=ks2, v_cache_scale=vs2)
    (ops.reshape_paged_cache if cache_kind == "bf16" else ops.quant_to_paged_cache)(params)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(kc), _bits(k2)) and np.array_equal(_bits(vc), _bits(v2))
    if ks is not None:
        assert np.array_equal(_bits(ks), _bits(ks2)) and np.array_equal(_bits(vs), _bits(vs2))


def test_rope_edge_cases_and_errors(gpu):
    print("case rope edges", flush=True)
    qkv, qw, kw, cos_sin, pos = _inputs(4, 2, 1, 1, 128, 128, 16, "bf16", seed=1)
    d = qkv.to(gpu)
    ops.fused_qk_norm_rope(d[:0], 2, 1, 1, 128, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False, pos[:0].to(gpu))
    # positions outside the table are clamped to its ends rather than read out of bounds
    far = torch.tensor([-5, 0, 15, 10 ** 9], dtype=torch.int64)
    ops.fused_qk_norm_rope(d, 2, 1, 1, 128, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False, far.to(gpu))
    e = qkv.to(gpu)
    ops.fused_qk_norm_rope(e, 2, 1, 1, 128, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False,
                           torch.tensor([0, 0, 15, 15]).to(gpu))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(d), _bits(e))
    with pytest.raises(_lib.XllmHipError):  # odd rotary_dim
        ops.fused_qk_norm_rope(e, 2, 1, 1, 128, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin[:, :127].contiguous().to(gpu),
                               False, pos.to(gpu))
    with pytest.raises(_lib.XllmHipError):  # more heads than the row holds
        ops.fused_qk_norm_rope(e, 4, 1, 1, 128, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False, pos.to(gpu))


@pytest.mark.parametrize("D,kind", [(128, "bf16"), (192, "fp16")])  # the 16-lanes-per-head kernel and the general one
def test_int32_positions_are_read_as_they_are(gpu, D, kind):
    """The reference's attention modules hand int32 positions over
    (xllm/core/layers/common/tests/qwen2_attention_tests.cpp:226,549): same bits as with int64."""
    print("case rope int32 positions", D, kind, flush=True)
    T, hq, hk = 13, 4, 2
    qkv, qw, kw, cos_sin, pos = _inputs(T, hq, hk, hk, D, D, 700, kind, seed=31)
    a, b = qkv.to(gpu), qkv.to(gpu)
    ops.fused_qk_norm_rope(a, hq, hk, hk, D, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False, pos.to(gpu))
    ops.fused_qk_norm_rope(b, hq, hk, hk, D, 1e-6, qw.to(gpu), kw.to(gpu), cos_sin.to(gpu), False,
                           pos.to(torch.int32).to(gpu))
    torch.cuda.synchronize()
    assert not np.array_equal(_bits(a), _bits(qkv))
    assert np.array_equal(_bits(a), _bits(b))
