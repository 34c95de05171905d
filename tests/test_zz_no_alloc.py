"""xllm_hip_paged_decode_static (the decode entry point that takes no workspace and allocates
nothing) against xllm_hip_paged_decode with a caller-owned workspace: same kernels, same schedule,
so the outputs and log-sum-exps must be the same bits.  Every case makes two calls in a row, the
second on a smaller input, because every call on a GPU shares one built-in array that keeps the
previous call's schedule, partials and counters."""
import ctypes

import pytest
import torch

from helpers import Case
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _args(case, out, lse):
    desc = ops._cache_desc(case.k_cache, case.v_cache, case.k_scale, case.v_scale, case.layout)
    args, keep = ops._decode_args(case.q, out, lse, case.block_table, case.seq_lens, None, case.n, case.scale, -1, 0,
                                  desc)
    return desc, args, keep


def _both(case):
    lib = _lib.load()
    dev = case.q.device
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    res = []
    for static in (False, True):
        out = torch.full_like(case.q, float("nan"))
        lse = torch.full((case.q.size(0), case.Hq), float("nan"), dtype=torch.float32, device=dev)
        desc, args, keep = _args(case, out, lse)
        if static:
            _lib.check(lib.xllm_hip_paged_decode_static(ctypes.byref(desc), ctypes.byref(args), stream))
        else:
            need = lib.xllm_hip_paged_decode_workspace_bytes(args.batch, args.q_per_seq, args.num_q_heads,
                                                             desc.num_kv_heads, desc.head_dim)
            assert need <= _lib.STATIC_WORKSPACE_BYTES
            ws = torch.empty(need, dtype=torch.uint8, device=dev)
            _lib.check(lib.xllm_hip_paged_decode(ctypes.byref(desc), ctypes.byref(args), ctypes.c_void_p(ws.data_ptr()),
                                                 need, stream))
        torch.cuda.synchronize()
        res.append((out, lse))
    return res


CASES = {
    # split sequences, partials merged inside the 16-row kernel (counters in the workspace)
    "bf16_fused_merge": (dict(Hq=32, Hkv=8, D=128, bs=16, kv="bf16"), [[8192, 5000], [3000]]),
    # 32 query rows per kv head: partials in the workspace, merged by the merge kernel
    "int8_rows32_merge_kernel": (dict(Hq=32, Hkv=4, D=64, bs=32, kv="int8", n=4), [[6000, 4096, 777], [2500, 90]]),
    # generic kernel (fp32 queries): always through the partials
    "fp32_generic": (dict(Hq=14, Hkv=2, D=64, bs=16, kv="fp32", qdt="fp32"), [[500, 37, 1, 260], [129, 64]]),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_static_workspace_decode_equals_caller_workspace_decode(gpu, name):
    shape, calls = CASES[name]
    for i, lens in enumerate(calls):  # the second call is the smaller one
        case = Case(len(lens), lens=lens, seed=11 + i, **shape)
        (out_ws, lse_ws), (out_st, lse_st) = _both(case)
        assert not torch.isnan(out_st.float()).any()
        assert torch.equal(out_ws.view(torch.uint8), out_st.view(torch.uint8)), (name, i)
        assert torch.equal(lse_ws.view(torch.int32), lse_st.view(torch.int32)), (name, i)
        # and against the oracle, like every other decode test
        ref, _ = case.oracle()
        assert float((out_st.float().cpu().numpy() - ref).__abs__().max()) <= case.tol


def test_sizes_beyond_the_built_in_workspace_are_refused(gpu):
    case = Case(1, 64, 4, 256, 16, lens=[64], n=8, kv="bf16")  # 128 rows per kv head at head_dim 256: about 85 MB
    out = torch.zeros_like(case.q)
    desc, args, keep = _args(case, out, None)
    lib = _lib.load()
    rc = lib.xllm_hip_paged_decode_static(ctypes.byref(desc), ctypes.byref(args), None)
    assert rc == _lib.WORKSPACE_TOO_SMALL
    assert b"caller-owned workspace" in lib.xllm_hip_last_error()
    torch.cuda.synchronize()
    assert float(out.abs().max()) == 0.0  # nothing was launched
