"""The allocation policy of the KV pools (ops.allocate_kv_cache and its C++ twin KVCache::allocate):
K and V carved from one buffer, V displaced 4 KiB from a 2 MiB boundary behind K."""
import os

import numpy as np
import pytest
import torch

from xllm_wxh_amd import build as xbuild
from xllm_wxh_amd import ops

PAGE = 2 << 20


def _check(k, v, ks, vs, shape, dtype, with_scales):
    assert tuple(k.shape) == tuple(shape) == tuple(v.shape) and k.dtype == dtype == v.dtype
    assert k.is_contiguous() and v.is_contiguous()
    nbytes = k.numel() * k.element_size()
    dist = v.data_ptr() - k.data_ptr()
    assert dist >= nbytes  # disjoint
    assert dist % PAGE == ops.KV_SKEW_BYTES and v.data_ptr() % 16 == 0
    assert float(k.float().abs().sum()) == 0.0 and float(v.float().abs().sum()) == 0.0
    k.view(torch.uint8).fill_(1)
    assert float(v.view(torch.uint8).float().sum()) == 0.0  # writing all of K leaves V alone
    if with_scales:
        assert tuple(ks.shape) == tuple(shape[:3]) == tuple(vs.shape) and ks.dtype == torch.float32
        assert (vs.data_ptr() - ks.data_ptr()) % PAGE == ops.KV_SKEW_BYTES
    else:
        assert ks is None and vs is None


@pytest.mark.parametrize("shape,dtype,with_scales", [
    ((10, 8, 16, 128), torch.bfloat16, False),
    ((300, 16, 8, 128), torch.int8, True),          # NHD, more than one 2 MiB page per pool
    ((7, 2, 16, 64), torch.float32, False),
    ((33, 8, 16, 128), torch.float8_e4m3fn, True),
])
def test_python_allocation(shape, dtype, with_scales):
    _check(*ops.allocate_kv_cache(shape, dtype, "cpu", with_scales), shape, dtype, with_scales)


def test_cpp_allocation_matches():
    if not os.path.exists(xbuild.TORCH_SHIM_PATH):
        xbuild.build_torch_shim(verbose=False)
    from xllm_wxh_amd import _xllm_hip_torch as shim

    for shape, dtype, with_scales in [((10, 8, 16, 128), torch.bfloat16, False), ((300, 16, 8, 128), torch.int8, True)]:
        kv = shim.KVCache.allocate(list(shape), dtype, "cpu", with_scales)
        _check(kv.get_k_cache(), kv.get_v_cache(), kv.get_k_cache_scale(), kv.get_v_cache_scale(), shape, dtype,
               with_scales)
    with pytest.raises(RuntimeError):
        shim.KVCache.allocate([4, 4, 4], torch.bfloat16, "cpu", False)


@pytest.mark.gpu
@pytest.mark.parametrize("kv", ["bf16", "int8"])
def test_decode_on_allocated_pools_equals_separate_pools(gpu, kv):
    """Same values in pools from the allocator and in separately allocated tensors: bitwise equal outputs,
    bit-exact writes."""
    from tests.helpers import Case

    print("case allocate_kv_cache", kv, flush=True)
    c = Case(3, 32, 8, 128, 16, [700, 33, 2000], kv=kv, seed=41)
    out_a, _ = c.run()
    k, v, ks, vs = ops.allocate_kv_cache(tuple(c.k_cache.shape), c.k_cache.dtype, gpu, with_scales=c.k_scale is not None)
    k.copy_(c.k_cache)
    v.copy_(c.v_cache)
    if ks is not None:
        ks.copy_(c.k_scale)
        vs.copy_(c.v_scale)
        c.k_scale, c.v_scale = ks, vs
    c.k_cache, c.v_cache = k, v
    out_b, _ = c.run()
    assert torch.equal(out_a, out_b)
