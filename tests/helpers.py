"""Shared builders for the GPU parity tests: seeded inputs on the device, the same inputs for the
CPU oracle, and the comparison itself."""
import numpy as np
import torch

from oracle import paged_kv_oracle as orc
from xllm_wxh_amd import ops

# Tolerances of the path (max-abs error of the attention output against the fp32 oracle).
TOL_BF16_KV = 2e-2
TOL_QUANT_KV = 5e-2

TORCH_KV_DTYPE = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32,
                  "fp8": torch.float8_e4m3fn, "int8": torch.int8}
TORCH_Q_DTYPE = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def make_tables(batch, block_size, lens, seed, extra_blocks=3, reserve_block0=True):
    """Disjoint shuffled block lists; block 0 is left unused (it is the padding block of the
    reference's block manager, xllm/core/framework/block/block_manager_impl.cpp:43-45)."""
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, np.int32)
    need = (lens.astype(np.int64) + block_size - 1) // block_size
    nblocks = int(need.sum()) + extra_blocks + (1 if reserve_block0 else 0)
    perm = rng.permutation(nblocks - 1) + 1 if reserve_block0 else rng.permutation(nblocks)
    table = np.zeros((batch, max(int(need.max()), 1)), np.int32)
    o = 0
    for b in range(batch):
        table[b, : need[b]] = perm[o:o + need[b]]
        o += int(need[b])
    return table, nblocks


class Case:
    """One decode problem: host copies for the oracle and device tensors for the HIP path."""

    def __init__(self, B, Hq, Hkv, D, bs, lens, n=1, kv="bf16", qdt="bf16", layout="HND", seed=0, std=1.0,
                 device="cuda", value_seed=None):
        self.B, self.Hq, self.Hkv, self.D, self.bs, self.n = B, Hq, Hkv, D, bs, n
        self.kv, self.qdt, self.layout = kv, qdt, layout
        self.lens = np.asarray(lens, np.int32)
        self.table, self.nblocks = make_tables(B, bs, self.lens, seed)
        g = torch.Generator().manual_seed(seed if value_seed is None else value_seed)
        shape = (self.nblocks, Hkv, bs, D)
        kf = torch.randn(shape, generator=g) * std
        vf = torch.randn(shape, generator=g) * std
        q = torch.randn(B * n, Hq, D, generator=g).to(TORCH_Q_DTYPE[qdt])
        self.scale = 1.0 / float(np.sqrt(D))
        if kv in ("fp8", "int8"):
            qk, sk = orc.quantize_per_token_head(kf.numpy(), kv)
            qv, sv = orc.quantize_per_token_head(vf.numpy(), kv)
            self.k_ref, self.v_ref = orc.dequantize(qk, sk, kv), orc.dequantize(qv, sv, kv)
            kc = torch.from_numpy(qk.view(np.uint8)).view(TORCH_KV_DTYPE[kv])
            vc = torch.from_numpy(qv.view(np.uint8)).view(TORCH_KV_DTYPE[kv])
            ks, vs = torch.from_numpy(sk), torch.from_numpy(sv)
        else:
            kc, vc = kf.to(TORCH_KV_DTYPE[kv]), vf.to(TORCH_KV_DTYPE[kv])
            self.k_ref, self.v_ref = kc.float().numpy(), vc.float().numpy()
            ks = vs = None
        self.q_ref = q.float().numpy()
        if layout == "NHD":
            kc, vc = kc.permute(0, 2, 1, 3).contiguous(), vc.permute(0, 2, 1, 3).contiguous()
            if ks is not None:
                ks, vs = ks.permute(0, 2, 1).contiguous(), vs.permute(0, 2, 1).contiguous()
        self.k_cache, self.v_cache = kc.to(device), vc.to(device)
        self.k_scale = ks.to(device) if ks is not None else None
        self.v_scale = vs.to(device) if vs is not None else None
        self.q = q.to(device)
        self.block_table = torch.from_numpy(self.table).to(device)
        self.seq_lens = torch.from_numpy(self.lens).to(device)

    @property
    def tol(self):
        return TOL_QUANT_KV if self.kv in ("fp8", "int8") else TOL_BF16_KV

    def oracle(self, window_left=-1):
        return orc.paged_decode(self.q_ref, self.k_ref, self.v_ref, self.table, self.lens, self.scale,
                                q_per_seq=self.n, window_left=window_left)

    def run(self, window_left=-1, lse=True, hints=False, **kw):
        if hints:  # host-side lengths, as the reference's AttentionMetadata carries them
            kw.setdefault("max_seq_len", int(self.lens.max()))
            kw.setdefault("total_kv_len", int(self.lens.sum()))
        out = torch.full_like(self.q, float("nan"))
        lse_t = torch.full((self.q.size(0), self.Hq), float("nan"), dtype=torch.float32, device=self.q.device) \
            if lse else None
        ops.batch_decode(self.q, self.k_cache, out, self.block_table, self.seq_lens, self.v_cache, lse_t, None,
                         self.k_scale, self.v_scale, scale=self.scale, return_lse=lse, q_per_seq=self.n,
                         kv_layout=self.layout, window_size_left=window_left,
                         kv_cache_quant_bit_size=8 if self.k_scale is not None else -1, **kw)
        torch.cuda.synchronize()
        return out, lse_t

    def variant(self):
        return ops.decode_variant(self.q, self.k_cache, self.v_cache, self.block_table, self.seq_lens,
                                  self.k_scale, self.v_scale, q_per_seq=self.n, kv_layout=self.layout)


def max_abs_err(out, ref):
    return float(np.abs(out.float().cpu().numpy().astype(np.float64) - ref).max())


def max_rel_err_per_seq(out, ref, q_per_seq=1):
    """Largest, over the sequences, of (max-abs error of the sequence's output rows) / (RMS of its
    reference rows).  Long sequences of zero-mean values have outputs of a few hundredths, where an
    absolute bound alone would let a wrong V scale or a dropped chunk through."""
    got = out.float().cpu().numpy().astype(np.float64)
    got = got.reshape(-1, q_per_seq, *got.shape[1:])
    want = np.asarray(ref, np.float64).reshape(got.shape)
    worst = 0.0
    for b in range(got.shape[0]):
        rms = float(np.sqrt(np.mean(want[b] ** 2)))
        if rms > 0.0:
            worst = max(worst, float(np.abs(got[b] - want[b]).max()) / rms)
    return worst


def lse_err(lse, ref):
    got = lse.cpu().numpy().astype(np.float64)
    fin = np.isfinite(ref)
    assert np.array_equal(np.isneginf(got), np.isneginf(ref))
    return float(np.abs(got[fin] - ref[fin]).max()) if fin.any() else 0.0


def max_rel_err_ragged(got, ref, q_indptr):
    """max_rel_err_per_seq for sequences with different numbers of query rows (rows q_indptr[b] ..
    q_indptr[b+1] belong to sequence b)."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    worst = 0.0
    for b in range(len(q_indptr) - 1):
        lo, hi = int(q_indptr[b]), int(q_indptr[b + 1])
        if hi > lo:
            rms = float(np.sqrt(np.mean(ref[lo:hi] ** 2)))
            if rms > 0.0:
                worst = max(worst, float(np.abs(got[lo:hi] - ref[lo:hi]).max()) / rms)
    return worst
