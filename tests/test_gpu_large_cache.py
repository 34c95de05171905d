"""Caches larger than 4 GiB per tensor (an MI355X holds 288 GB: one layer's K cache of a long-context
deployment passes 2^31 elements and 2^32 bytes): every kernel of the path on blocks that straddle
those offsets and on the last blocks of the pool, against the oracle run on a compact copy of the
same blocks.  The big tensors are allocated uninitialised; only the blocks in use are written."""

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import ops

pytestmark = pytest.mark.gpu

HQ, HKV, D, BS = 32, 8, 128, 16
TDT = {"bf16": torch.bfloat16, "int8": torch.int8}
BIG_BLOCKS = {"bf16": 170000, "int8": 300000}  # 5.2 GiB of bf16, 4.6 GiB of int8 per cache tensor


def _bits(t):
    t = t.detach().cpu().contiguous()
    return t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()]).numpy()


class BigCase:
    """A compact cache of `nb` blocks on the host (block 0 unused) and its image inside a big pool on
    the device: compact block i lives in physical block phys[i]."""

    def __init__(self, kind, lens, gpu, seed):
        self.kind, self.gpu = kind, gpu
        self.lens = np.asarray(lens, np.int32)
        need = (self.lens + BS - 1) // BS
        self.nb = int(need.sum()) + 10  # block 0, the sequences' blocks, 9 spare blocks for the block moves
        nbig = BIG_BLOCKS[kind]
        block_bytes = HKV * BS * D * (2 if kind == "bf16" else 1)
        rng = np.random.default_rng(seed)
        # physical ids: around the 2^31- and 2^32-byte offsets, the end of the pool, a few low ones
        edges = [(1 << 31) // block_bytes, (1 << 32) // block_bytes]
        pool = [1, 2, 3]
        for e in edges:
            pool += list(range(e - 3, e + 4))
        pool += list(range(nbig - 8, nbig))
        rest = rng.choice(np.arange(edges[1] + 8, nbig - 8), self.nb - 1 - len(pool), replace=False).tolist()
        phys = np.array(pool + rest, np.int64)
        rng.shuffle(phys)
        self.phys = np.concatenate([[0], phys]).astype(np.int64)  # compact 0 -> physical 0
        assert len(set(self.phys.tolist())) == self.nb and self.phys.max() == nbig - 1
        # compact tables
        perm = rng.permutation(self.nb - 10) + 1
        self.table = np.zeros((len(lens), int(need.max())), np.int32)
        o = 0
        for b in range(len(lens)):
            self.table[b, : need[b]] = perm[o:o + need[b]]
            o += int(need[b])
        self.spare = np.arange(self.nb - 9, self.nb)  # compact ids not in any table
        self.big_table = self.phys[self.table].astype(np.int32)
        g = torch.Generator().manual_seed(seed)
        shape = (self.nb, HKV, BS, D)
        if kind == "int8":
            self.k = torch.randint(-127, 128, shape, generator=g, dtype=torch.int8)
            self.v = torch.randint(-127, 128, shape, generator=g, dtype=torch.int8)
            self.ks = (torch.rand(shape[:3], generator=g) * 0.02 + 0.002)
            self.vs = (torch.rand(shape[:3], generator=g) * 0.02 + 0.002)
        else:
            self.k = torch.randn(shape, generator=g).to(torch.bfloat16)
            self.v = torch.randn(shape, generator=g).to(torch.bfloat16)
            self.ks = self.vs = None
        idx = torch.from_numpy(self.phys).to(gpu)
        self.big_k = torch.empty((nbig, HKV, BS, D), dtype=TDT[kind], device=gpu)
        self.big_v = torch.empty((nbig, HKV, BS, D), dtype=TDT[kind], device=gpu)
        assert self.big_k.numel() > (1 << 31) and self.big_k.numel() * self.big_k.element_size() > (1 << 32)
        self.big_k.index_copy_(0, idx, self.k.to(gpu))
        self.big_v.index_copy_(0, idx, self.v.to(gpu))
        self.big_ks = self.big_vs = None
        if self.ks is not None:
            self.big_ks = torch.empty((nbig, HKV, BS), dtype=torch.float32, device=gpu)
            self.big_vs = torch.empty((nbig, HKV, BS), dtype=torch.float32, device=gpu)
            self.big_ks.index_copy_(0, idx, self.ks.to(gpu))
            self.big_vs.index_copy_(0, idx, self.vs.to(gpu))
        self.idx = idx

    def compact_from_device(self):
        """The in-use blocks of the big pool, read back in compact order."""
        out = [self.big_k.index_select(0, self.idx).cpu(), self.big_v.index_select(0, self.idx).cpu()]
        if self.big_ks is not None:
            out += [self.big_ks.index_select(0, self.idx).cpu(), self.big_vs.index_select(0, self.idx).cpu()]
        return out

    def host(self):
        return [t for t in (self.k, self.v, self.ks, self.vs) if t is not None]

    def float_caches(self):
        if self.kind == "int8":
            return (orc.dequantize(self.k.numpy(), self.ks.numpy(), "int8"),
                    orc.dequantize(self.v.numpy(), self.vs.numpy(), "int8"))
        return self.k.float().numpy(), self.v.float().numpy()

    def dev(self, a, dtype=torch.int32):
        return torch.tensor(np.asarray(a), dtype=dtype, device=self.gpu)


@pytest.fixture(scope="module", params=["bf16", "int8"])
def big(request, gpu):
    print("case large cache: building", request.param, flush=True)
    case = BigCase(request.param, [700, 41, 2000, 48], gpu, seed=17)
    yield case
    del case
    torch.cuda.empty_cache()


def _assert_pool_equals_host(big):
    for got, want in zip(big.compact_from_device(), big.host()):
        assert np.array_equal(_bits(got)[1:], _bits(want)[1:])  # (block 0 is never written)


def test_kv_write_lands_in_high_blocks(big):
    print("case large cache: write", big.kind, flush=True)
    B = len(big.lens)
    g = torch.Generator().manual_seed(3)
    nk = torch.randn(B, HKV, D, generator=g).to(torch.bfloat16)
    nv = torch.randn(B, HKV, D, generator=g).to(torch.bfloat16)
    pos = big.lens - 1
    slots_c = np.array([big.table[b, pos[b] // BS] * BS + pos[b] % BS for b in range(B)], np.int64)
    slots_p = np.array([big.phys[big.table[b, pos[b] // BS]] * BS + pos[b] % BS for b in range(B)], np.int64)
    assert slots_p.max() < (1 << 31)
    if big.kind == "int8":
        k, v, ks, vs = (t.numpy() for t in big.host())
        orc.quant_to_paged_cache(slots_c, nk.float().numpy(), nv.float().numpy(), k, v, ks, vs, "int8", "HND")
    else:
        k, v = (t.view(torch.int16).numpy() for t in big.host())
        orc.reshape_paged_cache(slots_c, nk.view(torch.int16).numpy(), nv.view(torch.int16).numpy(), k, v, "HND")
    params = ops.ReshapePagedCacheParams(key=nk.to(big.gpu), value=nv.to(big.gpu), k_cache=big.big_k,
                                         v_cache=big.big_v, slot_mapping=big.dev(slots_p),
                                         k_cache_scale=big.big_ks, v_cache_scale=big.big_vs)
    (ops.quant_to_paged_cache if big.kind == "int8" else ops.reshape_paged_cache)(params)
    torch.cuda.synchronize()
    _assert_pool_equals_host(big)


@pytest.mark.parametrize("n,generic", [(1, False), (5, False), (40, False), (1, True)])
def test_decode_reads_high_blocks(big, n, generic):
    print("case large cache: decode", big.kind, n, generic, flush=True)
    B = len(big.lens)
    lens = big.lens  # all at least 40: every query token has a position
    g = torch.Generator().manual_seed(5 + n)
    q = torch.randn(B * n, HQ, D, generator=g).to(torch.bfloat16)
    kf, vf = big.float_caches()
    ref, _ = orc.paged_decode(q.float().numpy(), kf, vf, big.table, lens, 1.0 / np.sqrt(D), q_per_seq=n)
    out = torch.full((B * n, HQ, D), float("nan"), dtype=torch.bfloat16, device=big.gpu)
    with ops.option("force_generic", int(bool(generic))):
        ops.batch_decode(q.to(big.gpu), big.big_k, out, big.dev(big.big_table), big.dev(lens), big.big_v,
                         k_cache_quant_scale=big.big_ks, v_cache_quant_scale=big.big_vs, scale=1.0 / float(np.sqrt(D)),
                         q_per_seq=n, kv_cache_quant_bit_size=8 if big.kind == "int8" else -1)
        torch.cuda.synchronize()
    err = float(np.abs(out.float().cpu().numpy() - ref).max())
    assert err <= (5e-2 if big.kind == "int8" else 2e-2), err


def test_gather_reads_high_blocks(big):
    print("case large cache: gather", big.kind, flush=True)
    lens = [int(x) for x in big.lens]
    total = sum(lens)
    i32 = lambda a: big.dev(a)
    if big.kind == "int8":
        want_k, want_v = orc.dequant_from_paged_cache(big.k.numpy(), big.v.numpy(), big.ks.numpy(), big.vs.numpy(), lens,
                                                      big.table, "int8", out_kind="bf16")
        out_k = torch.zeros(total, HKV, D, dtype=torch.bfloat16, device=big.gpu)
        out_v = torch.zeros(total, HKV, D, dtype=torch.bfloat16, device=big.gpu)
        ops.dequant_from_paged_cache(out_k, out_v, big.big_k, big.big_v, big.big_ks, big.big_vs, i32(lens), max(lens),
                                     None, i32(big.big_table))
        torch.cuda.synchronize()
        assert np.array_equal(out_k.float().cpu().numpy(), want_k) and np.array_equal(out_v.float().cpu().numpy(), want_v)
    else:
        want_k, want_v = orc.reshape_from_cache(big.k.float().numpy(), big.v.float().numpy(), lens, big.table)
        out_k = torch.zeros(total, HKV, D, dtype=torch.bfloat16, device=big.gpu)
        out_v = torch.zeros(total, HKV, D, dtype=torch.bfloat16, device=big.gpu)
        ops.reshape_from_cache(out_k, out_v, big.big_k, big.big_v, i32(lens), max(lens), None, i32(big.big_table))
        torch.cuda.synchronize()
        assert np.array_equal(out_k.float().cpu().numpy(), want_k) and np.array_equal(out_v.float().cpu().numpy(), want_v)


@pytest.mark.parametrize("exact", [True, False])
def test_block_moves_between_high_blocks(big, exact):
    print("case large cache: block moves", big.kind, exact, flush=True)
    src_c = [int(big.table[0, 0]), int(big.table[2, 5]), int(big.table[2, 100]), int(big.table[0, 0])]
    dst_c = [int(x) for x in big.spare[:4]]
    if not exact:
        dst_c = [int(x) for x in big.spare[4:8]]
    ref = [_bits(t).copy() for t in big.host()]
    orc.swap_blocks(ref, src_c, dst_c)
    i64 = lambda a: big.dev(big.phys[np.asarray(a)], torch.int64)
    ops.swap_blocks(big.big_k, big.big_v, i64(src_c), i64(dst_c), big.big_ks, big.big_vs, exact=exact)
    torch.cuda.synchronize()
    for got, want in zip(big.compact_from_device(), ref):
        assert np.array_equal(_bits(got)[1:], want[1:])
    # keep the host copy in step with the pool for the tests that follow
    for t, want in zip(big.host(), ref):
        _bits_view = t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()])
        _bits_view.copy_(torch.from_numpy(want))


def test_copy_blocks_group_form_high_blocks(big):
    print("case large cache: copy_blocks", big.kind, flush=True)
    pairs = [(int(big.table[2, 7]), int(big.spare[8])), (int(big.table[1, 0]), int(big.spare[0])),
             (int(big.table[2, 7]), int(big.spare[1]))]
    src, dst, cum = orc.build_block_copy_groups(pairs)
    ref = [_bits(t).copy() for t in big.host()]
    orc.copy_blocks(ref, src, dst, cum)
    i32p = lambda a: big.dev(big.phys[np.asarray(a)])
    ops.copy_blocks(big.big_k, big.big_v, i32p(src), i32p(dst), big.dev(cum), big.big_ks, big.big_vs)
    torch.cuda.synchronize()
    for got, want in zip(big.compact_from_device(), ref):
        assert np.array_equal(_bits(got)[1:], want[1:])
    for t, want in zip(big.host(), ref):
        t.view({1: torch.uint8, 2: torch.int16, 4: torch.int32}[t.element_size()]).copy_(torch.from_numpy(want))


def test_rope_kv_write_into_high_blocks(big):
    print("case large cache: rope + write", big.kind, flush=True)
    B = len(big.lens)
    g = torch.Generator().manual_seed(23)
    qkv = torch.randn(B, (HQ + 2 * HKV) * D, generator=g).to(torch.bfloat16)
    theta = torch.rand(4096, D // 2, generator=g) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(torch.bfloat16)
    pos = (big.lens - 1).astype(np.int64)
    slots_c = np.array([big.table[b, pos[b] // BS] * BS + pos[b] % BS for b in range(B)], np.int64)
    slots_p = np.array([big.phys[big.table[b, pos[b] // BS]] * BS + pos[b] % BS for b in range(B)], np.int64)
    # the two-step route on a compact device copy is the reference here (bit-equal by another test)
    small = [t.clone().to(big.gpu) for t in big.host()]
    a = qkv.to(big.gpu)
    ops.rope_kv_write(a, HQ, HKV, D, cos_sin.to(big.gpu), big.dev(pos, torch.int64), small[0], small[1],
                      big.dev(slots_c), k_cache_scale=small[2] if len(small) > 2 else None,
                      v_cache_scale=small[3] if len(small) > 2 else None)
    b = qkv.to(big.gpu)
    ops.rope_kv_write(b, HQ, HKV, D, cos_sin.to(big.gpu), big.dev(pos, torch.int64), big.big_k, big.big_v,
                      big.dev(slots_p), k_cache_scale=big.big_ks, v_cache_scale=big.big_vs)
    torch.cuda.synchronize()
    assert np.array_equal(_bits(a), _bits(b))
    for got, want in zip(big.compact_from_device(), small):
        assert np.array_equal(_bits(got)[1:], _bits(want)[1:])
