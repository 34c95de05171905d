"""reshape_from_cache / dequant_from_paged_cache on the GPU, bit-exact against the oracle, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.test_gpu_block_move import _bits, _make_cache
from xllm_wxh_amd import _lib, ops

pytestmark = pytest.mark.gpu

OUT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def _tables(nb, bs, lens, seed, extra=0):
    rng = np.random.default_rng(seed)
    need = [(n + extra + bs - 1) // bs for n in lens]
    perm = rng.permutation(nb - 1)[: sum(need)] + 1
    width = max(need) + 1
    table = np.zeros((len(lens), width), np.int32)
    at = 0
    for b, n in enumerate(need):
        table[b, :n] = perm[at:at + n]
        at += n
    return table


def _np_cache(t, layout):
    """HND numpy view of a cache tensor's raw values (int8 / uint8 e4m3 bits / float32)."""
    t = t.detach().cpu()
    if t.dtype == torch.float8_e4m3fn:
        a = t.view(torch.uint8).numpy()
    elif t.dtype == torch.bfloat16:
        a = t.float().numpy()
    else:
        a = t.numpy()
    return a if layout == "HND" else a.transpose(0, 2, 1, 3)


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("kind", ["bf16", "fp32", "int8"])
@pytest.mark.parametrize("D", [128, 20])
def test_reshape_from_cache_bit_exact(gpu, kind, layout, D):
    print("case reshape_from_cache", kind, layout, D, flush=True)
    nb, H, bs = 40, 4, 16
    lens = [70, 1, 0, 129, 16]
    k, v, _, _ = _make_cache(kind, layout, nb, H, bs, D, seed=7)
    table = _tables(nb, bs, lens, seed=8)
    want_k, want_v = orc.reshape_from_cache(_np_cache(k, layout), _np_cache(v, layout), lens, table)
    total = sum(lens)
    out_k = torch.zeros(total, H, D, dtype=k.dtype, device=gpu)
    out_v = torch.zeros(total, H, D, dtype=k.dtype, device=gpu)
    ops.reshape_from_cache(out_k, out_v, k.to(gpu), v.to(gpu), torch.tensor(lens, dtype=torch.int32, device=gpu),
                           max(lens), None, torch.from_numpy(table).to(gpu), None, kv_layout=layout)
    torch.cuda.synchronize()
    conv = (lambda t: t.float().cpu().numpy()) if kind == "bf16" else (lambda t: t.cpu().numpy())
    assert np.array_equal(conv(out_k), want_k) and np.array_equal(conv(out_v), want_v)


def test_reshape_from_cache_offsets_and_strided_outputs(gpu):
    print("case reshape_from_cache offsets", flush=True)
    nb, H, bs, D = 30, 2, 16, 64
    lens = [20, 33, 5]
    start = [3, 0, 11]      # first cached position of each sequence
    rows_at = [40, 0, 70]   # first output row of each sequence
    k, _, _, _ = _make_cache("bf16", "HND", nb, H, bs, D, seed=9)
    table = _tables(nb, bs, lens, seed=10, extra=16)
    want, _ = orc.reshape_from_cache(k.float().numpy(), None, lens, table, context_seq_offset=rows_at,
                                     cache_seq_offset=start, total_rows=80, fill=-7)
    wide = torch.full((80, H * D + 32), -7, dtype=torch.bfloat16, device=gpu)  # rows of a wider buffer
    out = wide[:, : H * D].view(80, H, D)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    ops.reshape_from_cache(out, None, k.to(gpu), None, i32(lens), max(lens), i32(rows_at), torch.from_numpy(table).to(gpu),
                           i32(start))
    torch.cuda.synchronize()
    assert np.array_equal(out.float().cpu().numpy(), want)
    assert (wide[:, H * D:] == -7).all()


@pytest.mark.parametrize("layout", ["HND", "NHD"])
@pytest.mark.parametrize("kind", ["int8", "fp8"])
@pytest.mark.parametrize("out_kind", ["bf16", "fp16", "fp32"])
def test_dequant_from_paged_cache_bit_exact(gpu, kind, layout, out_kind):
    print("case dequant_from_paged_cache", kind, layout, out_kind, flush=True)
    nb, H, bs, D = 40, 4, 16, 128
    lens = [70, 1, 129, 16]
    k, v, ks, vs = _make_cache(kind, layout, nb, H, bs, D, seed=11)
    if out_kind == "fp16":
        ks, vs = ks * 0.1, vs * 0.1  # keep |q * scale| inside fp16's range
    table = _tables(nb, bs, lens, seed=12)
    sc = (lambda s: s.numpy()) if layout == "HND" else (lambda s: s.numpy().transpose(0, 2, 1))
    want_k, want_v = orc.dequant_from_paged_cache(_np_cache(k, layout), _np_cache(v, layout), sc(ks), sc(vs), lens,
                                                  table, kind, out_kind=out_kind)
    total = sum(lens)
    out_k = torch.zeros(total, H, D, dtype=OUT[out_kind], device=gpu)
    out_v = torch.zeros(total, H, D, dtype=OUT[out_kind], device=gpu)
    ops.dequant_from_paged_cache(out_k, out_v, k.to(gpu), v.to(gpu), ks.to(gpu), vs.to(gpu),
                                 torch.tensor(lens, dtype=torch.int32, device=gpu), max(lens), None,
                                 torch.from_numpy(table).to(gpu), 1, 8, kv_layout=layout)
    torch.cuda.synchronize()
    assert np.array_equal(out_k.float().cpu().numpy(), want_k, equal_nan=True)
    assert np.array_equal(out_v.float().cpu().numpy(), want_v, equal_nan=True)


def test_dequant_per_channel_and_odd_head_dim(gpu):
    print("case dequant per channel", flush=True)
    nb, H, bs, D = 12, 3, 8, 20  # head_dim 20: the element-wise kernel
    lens = [13, 30]
    k, _, ks, _ = _make_cache("int8", "HND", nb, H, bs, D, seed=13)
    table = _tables(nb, bs, lens, seed=14)
    want, _ = orc.dequant_from_paged_cache(k.numpy(), None, ks.numpy(), None, lens, table, "int8", out_kind="bf16")
    out = torch.zeros(sum(lens), H, D, dtype=torch.bfloat16, device=gpu)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=gpu)
    ops.dequant_from_paged_cache(out, None, k.to(gpu), None, ks.to(gpu), None, i32(lens), max(lens), None,
                                 torch.from_numpy(table).to(gpu))
    assert np.array_equal(out.float().cpu().numpy(), want)
    # per channel
    g = torch.Generator().manual_seed(15)
    ch = torch.rand(H, D, generator=g) * 0.1 + 0.01
    want, _ = orc.dequant_from_paged_cache(k.numpy(), None, ch.numpy(), None, lens, table, "int8", out_kind="fp32",
                                           quant_mode=0)
    out = torch.zeros(sum(lens), H, D, dtype=torch.float32, device=gpu)
    ops.dequant_from_paged_cache(out, None, k.to(gpu), None, ch.to(gpu), None, i32(lens), max(lens), None,
                                 torch.from_numpy(table).to(gpu), 0)
    assert np.array_equal(out.cpu().numpy(), want)


def test_dequant_then_dense_attention_equals_paged_decode(gpu):
    """The reference's MLU route for a quantised cache (dequantise, then attend) and the direct
    paged decode see the same numbers."""
    print("case dequant + attention", flush=True)
    from tests.helpers import Case, max_abs_err
    case = Case(2, 32, 8, 128, 16, [300, 77], kv="int8", seed=31)
    out, _ = case.run()
    lens = [300, 77]
    kd = torch.zeros(sum(lens), 8, 128, dtype=torch.float32, device=gpu)
    vd = torch.zeros_like(kd)
    ops.dequant_from_paged_cache(kd, vd, case.k_cache, case.v_cache, case.k_scale, case.v_scale, case.seq_lens,
                                 max(lens), None, case.block_table)
    row = 0
    for b, n in enumerate(lens):
        q = case.q[b].float().view(8, 4, 128)
        kk, vv = kd[row:row + n], vd[row:row + n]
        p = torch.softmax(torch.einsum("hgd,thd->hgt", q, kk) * case.scale, dim=-1)
        ref = torch.einsum("hgt,thd->hgd", p, vv).reshape(32, 128)
        assert max_abs_err(out[b], ref.cpu().numpy()) <= 2.5e-2
        row += n


def test_errors(gpu):
    k = torch.zeros(4, 2, 16, 64, dtype=torch.bfloat16, device=gpu)
    lens = torch.tensor([3], dtype=torch.int32, device=gpu)
    bt = torch.zeros(1, 2, dtype=torch.int32, device=gpu)
    with pytest.raises(_lib.XllmHipError):  # dtype differs
        ops.reshape_from_cache(torch.zeros(3, 2, 64, device=gpu), None, k, None, lens, 3, None, bt)
    with pytest.raises(_lib.XllmHipError):  # no block tables: the linear mode is not served
        ops.reshape_from_cache(torch.zeros(3, 2, 64, dtype=torch.bfloat16, device=gpu), None, k, None, lens, 3)
    with pytest.raises(_lib.XllmHipError):  # head count differs
        ops.reshape_from_cache(torch.zeros(3, 4, 64, dtype=torch.bfloat16, device=gpu), None, k, None, lens, 3, None, bt)
    q = torch.zeros(4, 2, 16, 64, dtype=torch.int8, device=gpu)
    with pytest.raises(_lib.XllmHipError):  # scales missing
        ops.dequant_from_paged_cache(torch.zeros(3, 2, 64, dtype=torch.bfloat16, device=gpu), None, q, None, None, None,
                                     lens, 3, None, bt)
    # empty batch and max_context_len 0 are no-ops
    ops.reshape_from_cache(torch.zeros(0, 2, 64, dtype=torch.bfloat16, device=gpu), None, k, None,
                           torch.zeros(0, dtype=torch.int32, device=gpu), 0, None, bt)
