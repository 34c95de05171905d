"""Pins of the oracle's RMSNorm + rotary-embedding restatement (CPU only)."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc

TDT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def torch_reference(qkv, hq, hk, hv, D, eps, qw, kw, cos_sin, interleaved, pos):
    """The formula the reference's own test holds its kernel to
    (xllm/core/kernels/cuda/fused_qknorm_rope_test.cpp:28-109), in torch on the CPU."""
    T = qkv.size(0)
    R = cos_sin.size(1)
    half = R // 2
    out = qkv.clone()
    sel = cos_sin.index_select(0, pos)
    cos, sin = sel[:, :half].view(T, 1, half), sel[:, half:R].view(T, 1, half)

    def rope(x):
        xf = x.float()
        rot, rest = xf[..., :R], xf[..., R:]
        if interleaved:
            r = rot.reshape(T, -1, half, 2)
            e, o = r[..., 0], r[..., 1]
            rot = torch.stack([e * cos - o * sin, e * sin + o * cos], -1).reshape(T, -1, R)
        else:
            a, b = rot[..., :half], rot[..., half:]
            rot = torch.cat([a * cos - b * sin, b * cos + a * sin], -1)
        return torch.cat([rot, rest], -1).to(x.dtype)

    for lo, n, w in ((0, hq, qw), (hq * D, hk, kw)):
        x = out[:, lo:lo + n * D].view(T, n, D)
        xf = x.float()
        rms = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
        x.copy_(rope((xf * rms * w.float().view(1, 1, D)).to(x.dtype)))
    return out


@pytest.mark.parametrize("T,hq,hk,hv,D,maxpos,interleaved,kind,tol", [
    (17, 8, 4, 4, 128, 512, False, "fp16", 2e-3),   # MatchesReferenceNeoX
    (11, 6, 2, 2, 64, 256, True, "bf16", 2e-2),     # MatchesReferenceInterleaved
])
def test_matches_the_reference_tests_formula(T, hq, hk, hv, D, maxpos, interleaved, kind, tol):
    g = torch.Generator().manual_seed(2026)
    dt = TDT[kind]
    qkv = (torch.randn(T, (hq + hk + hv) * D, generator=g) * 0.2).to(dt)
    qw, kw = torch.randn(D, generator=g).to(dt), torch.randn(D, generator=g).to(dt)
    cos_sin = torch.randn(maxpos, D, generator=g)
    pos = torch.randint(0, maxpos, (T,), generator=g)
    want = torch_reference(qkv, hq, hk, hv, D, 1e-6, qw, kw, cos_sin, interleaved, pos).float().numpy()
    got = orc.fused_qk_norm_rope(qkv.float().numpy(), hq, hk, hv, D, 1e-6, qw.float().numpy(), kw.float().numpy(),
                                 cos_sin.numpy(), interleaved, pos.numpy(), kind)
    assert np.allclose(got, want, rtol=tol, atol=tol)
    # the v heads pass through untouched
    assert np.array_equal(got[:, (hq + hk) * D:], qkv.float().numpy()[:, (hq + hk) * D:])


def test_norm_alone_is_torch_rms_norm():
    g = torch.Generator().manual_seed(1)
    T, H, D = 5, 3, 128
    x = torch.randn(T, H * D, generator=g)
    w = torch.randn(D, generator=g)
    ident = torch.cat([torch.ones(4, D // 2), torch.zeros(4, D // 2)], 1)  # cos = 1, sin = 0
    got = orc.fused_qk_norm_rope(x.numpy(), H, 0, 0, D, 1e-5, w.numpy(), w.numpy(), ident.numpy(), False,
                                 np.zeros(T, dtype=np.int64), "fp32")
    want = torch.nn.functional.rms_norm(x.view(T, H, D), (D,), w, 1e-5).view(T, H * D)
    assert np.allclose(got, want.numpy(), rtol=2e-6, atol=2e-6)


@pytest.mark.parametrize("interleaved", [False, True])
def test_rotation_is_complex_multiplication(interleaved):
    rng = np.random.default_rng(3)
    T, H, D, R, maxpos = 6, 2, 64, 32, 50
    x = rng.standard_normal((T, H * D))
    theta = rng.uniform(0, 2 * np.pi, size=(maxpos, R // 2))
    cache = np.concatenate([np.cos(theta), np.sin(theta)], axis=1)
    pos = rng.integers(0, maxpos, size=T)
    got = orc.fused_qk_norm_rope(x, H, 0, 0, D, 0.0, None, None, cache, interleaved, pos, "fp32").reshape(T, H, D)
    xi, yi = orc.rope_pairs(R, interleaved)
    xr = x.reshape(T, H, D)
    z = (xr[..., xi] + 1j * xr[..., yi]) * np.exp(1j * theta[pos])[:, None, :]
    assert np.allclose(got[..., xi], z.real, atol=1e-6) and np.allclose(got[..., yi], z.imag, atol=1e-6)
    assert np.allclose(got[..., R:], xr[..., R:].astype(np.float32))  # partial rotary: the rest passes through
    # a rotation keeps the length of every pair
    assert np.allclose(got[..., xi] ** 2 + got[..., yi] ** 2, xr[..., xi] ** 2 + xr[..., yi] ** 2, rtol=1e-5)


def test_identity_angle_and_rounding_helpers():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 2 * 64, generator=g).to(torch.bfloat16)
    ident = np.concatenate([np.ones((2, 32)), np.zeros((2, 32))], axis=1)
    for per_op in (False, True):
        got = orc.fused_qk_norm_rope(x.float().numpy(), 1, 1, 0, 64, 0.0, None, None, ident, False, [0, 1, 1], "bf16",
                                     round_each_op=per_op)
        assert np.array_equal(got, x.float().numpy())
    v = torch.randn(4096, generator=g, dtype=torch.float64) * 3
    assert np.array_equal(orc.round_to_dtype(v.numpy(), "bf16"), v.float().to(torch.bfloat16).double().numpy())
    assert np.array_equal(orc.round_to_dtype(v.numpy(), "fp16"), v.to(torch.float16).double().numpy())
    # ties go to even: 1 + 2^-8 is halfway between bf16 neighbours 1 and 1 + 2^-7
    assert orc.round_to_dtype(np.array([1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8]), "bf16").tolist() == [1.0, 1.0 + 2.0 ** -6]


def test_round_each_op_differs_only_in_the_last_place():
    g = torch.Generator().manual_seed(7)
    T, H, D = 9, 4, 128
    x = torch.randn(T, H * D, generator=g).to(torch.bfloat16).float().numpy()
    theta = np.random.default_rng(0).uniform(0, 6.28, size=(64, D // 2))
    cache = orc.round_to_dtype(np.concatenate([np.cos(theta), np.sin(theta)], 1), "bf16")
    pos = np.arange(T) * 3
    a = orc.fused_qk_norm_rope(x, H, 0, 0, D, 0.0, None, None, cache, False, pos, "bf16")
    b = orc.fused_qk_norm_rope(x, H, 0, 0, D, 0.0, None, None, cache, False, pos, "bf16", round_each_op=True)
    assert not np.array_equal(a, b)
    assert np.all(np.abs(a - b) <= 2.0 ** -6 * np.maximum(np.abs(a), np.abs(b)) + 2.0 ** -8)
