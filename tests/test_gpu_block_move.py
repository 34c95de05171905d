"""Whole-block swap / copy on the GPU, bit-exact against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()]).numpy()


def _make_cache(kind, layout, nb, H, bs, D, seed):
    g = torch.Generator().manual_seed(seed)
    shape = (nb, H, bs, D) if layout == "HND" else (nb, bs, H, D)
    sshape = shape[:3]
    if kind in ("int8", "fp8"):
        k = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
        v = torch.randint(-128, 128, shape, generator=g, dtype=torch.int8)
        if kind == "fp8":
            k, v = k.view(torch.float8_e4m3fn), v.view(torch.float8_e4m3fn)
        ks = torch.rand(sshape, generator=g) + 0.01
        vs = torch.rand(sshape, generator=g) + 0.01
    else:
        dt = {"bf16": torch.bfloat16, "fp32": torch.float32}[kind]
        k = torch.randn(shape, generator=g).to(dt)
        v = torch.randn(shape, generator=g).to(dt)
        ks = vs = None
    return k, v, ks, vs


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("kind", ["bf16", "fp32", "int8", "fp8"])
@pytest.mark.parametrize("exact", [True, False])
def test_swap_blocks_bit_exact(gpu, kind, layout, exact):
    print("case swap_blocks", kind, layout, exact, flush=True)
    nb, H, bs, D = 23, 4, 16, 128
    k, v, ks, vs = _make_cache(kind, layout, nb, H, bs, D, seed=3)
    src = [1, 1, 4, 9, 22]
    dst = [0, 2, 5, 10, 3]
    if exact:  # destinations that are sources too: the gather must come first
        src += [10, 5]
        dst += [11, 12]
    ref = [_bits(t).copy() if t is not None else None for t in (k, v, ks, vs)]
    orc.swap_blocks(ref, src, dst)
    dk, dv = k.to(gpu), v.to(gpu)
    dks = ks.to(gpu) if ks is not None else None
    dvs = vs.to(gpu) if vs is not None else None
    ops.swap_blocks(dk, dv, torch.tensor(src, device=gpu), torch.tensor(dst, device=gpu), dks, dvs,
                    kv_layout=layout, exact=exact)
    torch.cuda.synchronize()
    for got, want in zip((dk, dv, dks, dvs), ref):
        if want is not None:
            assert np.array_equal(_bits(got), want)


def test_swap_blocks_edge_cases(gpu):
    print("case swap_blocks edges", flush=True)
    nb, H, bs, D = 8, 2, 16, 64
    k, v, _, _ = _make_cache("bf16", "HND", nb, H, bs, D, seed=5)
    dk, dv = k.to(gpu), v.to(gpu)
    e = torch.empty(0, dtype=torch.int64, device=gpu)
    ops.swap_blocks(dk, dv, e, e)  # empty list
    # ids outside the pool are skipped; the valid pair still moves
    ops.swap_blocks(dk, dv, torch.tensor([-1, nb, 3], device=gpu), torch.tensor([1, 2, nb + 4], device=gpu))
    ops.swap_blocks(dk, dv, torch.tensor([6], device=gpu), torch.tensor([7], device=gpu))
    torch.cuda.synchronize()
    want_k = _bits(k).copy()
    want_k[7] = want_k[6]
    assert np.array_equal(_bits(dk), want_k)
    # a strided cache view (every other block of a larger pool, odd head_dim of 2-byte elements)
    big = torch.randn(2 * nb, H, bs, 33).to(torch.bfloat16).to(gpu)
    view = big[::2]
    ref = _bits(view).copy()
    orc.swap_blocks([ref], [0, 2], [1, 3])
    ops.swap_blocks(view, None, torch.tensor([0, 2], device=gpu), torch.tensor([1, 3], device=gpu))
    torch.cuda.synchronize()
    assert np.array_equal(_bits(view), ref)
    with pytest.raises(_lib.XllmHipError):
        ki, vi, _, _ = _make_cache("int8", "HND", nb, H, bs, D, seed=6)
        ops.swap_blocks(ki.to(gpu), vi.to(gpu), torch.tensor([0], device=gpu), torch.tensor([1], device=gpu))


@pytest.mark.parametrize("kind", ["bf16", "int8"])
def test_copy_blocks_group_form(gpu, kind):
    print("case copy_blocks", kind, flush=True)
    nb, H, bs, D = 40, 8, 128, 128
    k, v, ks, vs = _make_cache(kind, "HND", nb, H, bs, D, seed=9)
    pairs = [(5, 20), (2, 21), (5, 22), (2, 23), (3, 24), (5, 25), (30, 39)]
    src, dst, cum = orc.build_block_copy_groups(pairs)
    ref = [_bits(t).copy() if t is not None else None for t in (k, v, ks, vs)]
    orc.copy_blocks(ref, src, dst, cum)
    dk, dv = k.to(gpu), v.to(gpu)
    dks = ks.to(gpu) if ks is not None else None
    dvs = vs.to(gpu) if vs is not None else None
    i32 = dict(dtype=torch.int32, device=gpu)
    ops.copy_blocks(dk, dv, torch.tensor(src, **i32), torch.tensor(dst, **i32), torch.tensor(cum, **i32), dks, dvs)
    torch.cuda.synchronize()
    for got, want in zip((dk, dv, dks, dvs), ref):
        if want is not None:
            assert np.array_equal(_bits(got), want)
