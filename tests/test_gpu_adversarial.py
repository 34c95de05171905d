"""Paged-attention decode on inputs chosen to stress the range-dependent devices of the kernels, against
the fp32 oracle, through the C ABI: per-token scales that span 2^±20 inside one sequence, scores that
grow along the sequence (the softmax's reference point moves on every tile, or jumps by just under / just
over the 2^8 the kernels tolerate before they move it), one dominant key late in a long sequence,
identical keys (the output is then the mean of the values: a closed form), values with a large common
offset, query heads of one GQA group whose magnitudes differ by 2^10 and 2^14, a softmax scale of zero
and a large one over tiny queries.

The i.i.d. N(0, 1) inputs of the other tests never reach these.  Bounds here are per query row and head
and relative to what that row can resolve:
  lse      |got - ref| <= E = 1e-4 * max(1, S / 16),  S = max_t sum_d |q_d k_td| * scale * log2(e)  (fp32
           accumulation of the scores; 1e-4 is the bound of the other decode tests),
  output   |got - ref| <= (c + 2 ln 2 * E) * A,  A = max_d sum_t p_t |v_td|  (the attention over |V|: 16-bit
           weights and a 16-bit output carry a relative error of 2^-9 each against the terms of that sum; the
           second term is what scores off by E do to the weights).
"""
import math

import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.helpers import TORCH_KV_DTYPE, TORCH_Q_DTYPE, Case, make_tables
from xllm_wxh_amd import ops

pytestmark = pytest.mark.gpu

OUT_TOL = {"bf16": 1.2e-2, "fp16": 1.2e-2, "fp8": 2.5e-2, "int8": 2.5e-2}
LSE_TOL = 1e-4


class AdvCase(Case):
    """A decode problem built from explicit per-sequence K / V ([L, Hkv, D] fp32 each) and queries
    ([B * n, Hq, D] fp32), laid into a shuffled paged cache whose unused slots hold large garbage."""

    def __init__(self, Hq, Hkv, D, bs, K, V, q, n=1, kv="bf16", qdt="bf16", scale=None, seed=0, device="cuda"):
        B = len(K)
        self.B, self.Hq, self.Hkv, self.D, self.bs, self.n = B, Hq, Hkv, D, bs, n
        self.kv, self.qdt, self.layout = kv, qdt, "HND"
        self.lens = np.asarray([k.shape[0] for k in K], np.int32)
        self.table, self.nblocks = make_tables(B, bs, self.lens, seed)
        rng = np.random.default_rng(seed + 1)
        kf = (rng.standard_normal((self.nblocks, Hkv, bs, D)) * 37.0).astype(np.float32)
        vf = (rng.standard_normal((self.nblocks, Hkv, bs, D)) * 37.0).astype(np.float32)
        for b in range(B):
            L = int(self.lens[b])
            t = np.arange(L)
            blk, slot = self.table[b, t // bs], t % bs
            kf[blk, :, slot, :] = K[b]
            vf[blk, :, slot, :] = V[b]
        qt = torch.from_numpy(np.asarray(q, np.float32)).to(TORCH_Q_DTYPE[qdt])
        self.scale = 1.0 / float(np.sqrt(D)) if scale is None else float(scale)
        if kv in ("fp8", "int8"):
            qk, sk = orc.quantize_per_token_head(kf, kv)
            qv, sv = orc.quantize_per_token_head(vf, kv)
            self.k_ref, self.v_ref = orc.dequantize(qk, sk, kv), orc.dequantize(qv, sv, kv)
            kc = torch.from_numpy(qk.view(np.uint8)).view(TORCH_KV_DTYPE[kv])
            vc = torch.from_numpy(qv.view(np.uint8)).view(TORCH_KV_DTYPE[kv])
            ks, vs = torch.from_numpy(sk), torch.from_numpy(sv)
        else:
            kc = torch.from_numpy(kf).to(TORCH_KV_DTYPE[kv])
            vc = torch.from_numpy(vf).to(TORCH_KV_DTYPE[kv])
            self.k_ref, self.v_ref = kc.float().numpy(), vc.float().numpy()
            ks = vs = None
        self.q_ref = qt.float().numpy()
        self.k_cache, self.v_cache = kc.to(device), vc.to(device)
        self.k_scale = ks.to(device) if ks is not None else None
        self.v_scale = vs.to(device) if vs is not None else None
        self.q = qt.to(device)
        self.block_table = torch.from_numpy(self.table).to(device)
        self.seq_lens = torch.from_numpy(self.lens).to(device)

    def reference(self):
        """(out, lse, A, S): the oracle's output and base-2 log-sum-exp, the attention over |V| reduced to
        its largest column (per row and head) and the largest sum_d |q_d k_td| * scale * log2(e) of a row."""
        out, lse = orc.paged_decode(self.q_ref, self.k_ref, self.v_ref, self.table, self.lens, self.scale,
                                    q_per_seq=self.n)
        a_out, _ = orc.paged_decode(self.q_ref, self.k_ref, np.abs(self.v_ref), self.table, self.lens, self.scale,
                                    q_per_seq=self.n)
        g = self.Hq // self.Hkv
        S = np.zeros((self.B * self.n, self.Hq))
        for b in range(self.B):
            L = int(self.lens[b])
            Kb = np.abs(orc.gather_sequence(self.k_ref, self.table[b], L).astype(np.float64))  # [Hkv, L, D]
            qb = np.abs(self.q_ref[b * self.n:(b + 1) * self.n].astype(np.float64)).reshape(self.n, self.Hkv, g, self.D)
            s = np.einsum("jkgd,ktd->jkgt", qb, Kb).max(-1)
            S[b * self.n:(b + 1) * self.n] = s.reshape(self.n, self.Hq)
        return out, lse, a_out.max(-1), S * abs(self.scale) * math.log2(math.e)


def check(case, out_tol=None, lse_tol=LSE_TOL, hints=False):
    ref, lse_ref, A, S = case.reference()
    got, lse = case.run(hints=hints)
    got = got.float().cpu().numpy().astype(np.float64)
    lse = lse.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    c = OUT_TOL[case.kv] if out_tol is None else out_tol
    err = np.abs(got - ref).max(-1)                      # [rows, heads]
    worst = float((err / np.maximum(A, 1e-300)).max())
    fin = np.isfinite(lse_ref)
    assert np.array_equal(np.isfinite(lse), fin)
    if case.kv == "int8" and case.qdt == "fp16":
        # An int8 cache meets the queries as 16-bit fixed point against each row's largest element.  bf16 elements
        # within 2^7 of that element lie on the grid; fp16 ones (11 bits) only within 2^5, the rest are rounded.
        lse_tol = 2.0 * lse_tol
    lse_bound = lse_tol * np.maximum(1.0, S / 16.0)
    lerr = np.where(fin, np.abs(np.where(fin, lse - lse_ref, 0.0)), 0.0)
    lworst = float((lerr / lse_bound).max())
    print("   variant=%s out err / A = %.3e (tol %.1e)   lse err / bound = %.3f" % (case.variant(), worst, c, lworst),
          flush=True)
    # (a score off by e changes a weight by the factor 2^e, the output by up to 2 e ln 2 of A: visible where the
    # scores are so large that fp32 no longer resolves them, as with keys of magnitude 2^20)
    assert (err <= (c + 2.0 * math.log(2.0) * lse_bound) * A + 1e-30).all(), worst
    assert (lerr <= lse_bound).all(), lworst
    return got, lse


# kernels: (heads per kv head, query tokens) -> rows per kv head 4 (16-row kernel), 32 (32-row kernel), 64 (128-row
# kernel at head_dim 128 and over 16-bit caches at head_dim 64; two row groups of 32 elsewhere)
KERNELS = [(4, 1), (8, 4), (4, 16)]
DIMS = [(128, 16), (64, 32), (256, 16)]
CACHES = [("bf16", "bf16"), ("fp16", "fp16"), ("fp8", "bf16"), ("int8", "bf16"), ("int8", "fp16")]
GRID = [(kv, qdt, g, n, D, bs) for kv, qdt in CACHES for g, n in KERNELS for D, bs in DIMS]
grid = pytest.mark.parametrize("kv,qdt,g,n,D,bs", GRID, ids=lambda v: str(v))
HKV = 2


def _base(rng, lens, g, n, D):
    K = [rng.standard_normal((L, HKV, D)).astype(np.float32) for L in lens]
    V = [rng.standard_normal((L, HKV, D)).astype(np.float32) for L in lens]
    q = rng.standard_normal((len(lens) * n, HKV * g, D)).astype(np.float32)
    return K, V, q


@grid
def test_scales_spanning_forty_binary_orders(gpu, kv, qdt, g, n, D, bs):
    """K and V rows scaled by 2^u, u uniform in [-20, 20], token by token: per-token scales of a quantised
    cache span 2^40 inside every tile.  Twice: queries as they are (the large keys decide), and queries 2^-17
    smaller so that the large keys' scores are ordinary and the small ones' all but zero."""
    print("case adversarial scale span", kv, qdt, g, n, D, bs, flush=True)
    rng = np.random.default_rng(101)
    lens = [700, 2077]
    K, V, q = _base(rng, lens, g, n, D)
    for b, L in enumerate(lens):
        K[b] *= np.exp2(rng.uniform(-20, 20, size=(L, HKV, 1))).astype(np.float32)
        V[b] *= np.exp2(rng.uniform(-20, 20, size=(L, HKV, 1))).astype(np.float32)
    if qdt == "fp16":  # (keep cache values and outputs inside fp16's range)
        K = [np.clip(k, -6e4, 6e4) for k in K]
        V = [np.clip(v, -6e4, 6e4) for v in V]
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, seed=3))
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q * 2.0 ** -17, n=n, kv=kv, qdt=qdt, seed=4))


def _directed(rng, lens, g, n, D, x_of_t):
    """Keys and queries sharing one direction per kv head so that the log2-scaled score of token t is close to
    x_of_t(b, t) for every row (plus a little noise)."""
    K, V, q = _base(rng, lens, g, n, D)
    u = rng.standard_normal((HKV, D))
    u /= np.linalg.norm(u, axis=-1, keepdims=True)
    scale = 1.0 / math.sqrt(D)
    c = 1.0 / (scale * math.log2(math.e))
    for b, L in enumerate(lens):
        x = np.asarray([x_of_t(b, t) for t in range(L)], np.float64)
        K[b] = (0.05 * K[b] + (x[:, None, None] * c) * u[None]).astype(np.float32)
    q = 0.05 * q + np.repeat(u, g, axis=0)[None]
    return K, V, q.astype(np.float32), scale


@grid
@pytest.mark.parametrize("per_tile", [2.5, 9.0])
def test_scores_that_grow_along_the_sequence(gpu, kv, qdt, g, n, D, bs, per_tile):
    """log2-scaled scores rising by `per_tile` every 32 tokens: at 9 the reference point of the exponents moves
    on every tile (more than 2^8 per tile), at 2.5 every fourth; every weight but the last few underflows."""
    print("case adversarial growing scores", kv, qdt, g, n, D, bs, per_tile, flush=True)
    rng = np.random.default_rng(102)
    lens = [330, 1500]
    K, V, q, scale = _directed(rng, lens, g, n, D, lambda b, t: per_tile * t / 32.0)
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, scale=scale, seed=5))


@grid
@pytest.mark.parametrize("jump", [7.9, 8.1])
def test_one_score_jumps_by_about_two_to_the_eighth(gpu, kv, qdt, g, n, D, bs, jump):
    """Flat scores but for one token, `jump` above the rest in log2 terms, in the middle of a tile late in the
    sequence: 7.9 stays under the threshold at which the reference point moves (the weight 2^7.9 is kept
    against the old one), 8.1 is over it."""
    print("case adversarial jump", kv, qdt, g, n, D, bs, jump, flush=True)
    rng = np.random.default_rng(103)
    lens = [611, 1203]
    at = [400, 1100]
    K, V, q, scale = _directed(rng, lens, g, n, D, lambda b, t: jump if t == at[b] else 0.0)
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, scale=scale, seed=6))


@grid
def test_one_dominant_key_late_in_a_long_sequence(gpu, kv, qdt, g, n, D, bs):
    """5000 tokens (split into chunks and merged), one key 40 binary orders above the others at token 4700:
    the output is that token's value row."""
    print("case adversarial dominant key", kv, qdt, g, n, D, bs, flush=True)
    rng = np.random.default_rng(104)
    lens = [5000, 900]
    at = [4700, 3]
    K, V, q, scale = _directed(rng, lens, g, n, D, lambda b, t: 40.0 if t == at[b] else 0.0)
    case = AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, scale=scale, seed=7)
    got, _ = check(case)
    for b in range(2):
        L = int(case.lens[b])
        want = orc.gather_sequence(case.v_ref, case.table[b], L)[:, at[b], :]  # [Hkv, D]
        rows = got[b * n:(b + 1) * n].reshape(n, HKV, g, D)
        assert np.abs(rows - want[None, :, None, :]).max() <= OUT_TOL[kv] * np.abs(want).max()


@grid
def test_identical_keys_give_the_mean_of_the_values(gpu, kv, qdt, g, n, D, bs):
    """Every key of a sequence the same row: all weights are equal whatever the queries, so the output is
    the mean of the visible value rows and the log-sum-exp is score + log2(count) — closed forms."""
    print("case adversarial identical keys", kv, qdt, g, n, D, bs, flush=True)
    rng = np.random.default_rng(105)
    lens = [257, 1999]
    K, V, q = _base(rng, lens, g, n, D)
    K = [np.broadcast_to(k[:1], k.shape).copy() for k in K]
    case = AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, seed=8)
    got, lse = check(case)
    for b, L in enumerate(lens):
        Vb = orc.gather_sequence(case.v_ref, case.table[b], L).astype(np.float64)  # [Hkv, L, D]
        Kb = orc.gather_sequence(case.k_ref, case.table[b], L).astype(np.float64)
        for j in range(n):
            vis = L - (n - 1 - j)
            want = Vb[:, :vis].mean(1)  # [Hkv, D]
            rows = got[b * n + j].reshape(HKV, g, D)
            assert np.abs(rows - want[:, None, :]).max() <= OUT_TOL[kv] * np.abs(Vb).mean() * 4
            x = np.einsum("kgd,kd->kg", case.q_ref[b * n + j].astype(np.float64).reshape(HKV, g, D), Kb[:, 0]) \
                * case.scale * math.log2(math.e)
            assert np.abs(lse[b * n + j].reshape(HKV, g) - (x + math.log2(vis))).max() <= 2e-4


@grid
def test_values_with_a_large_common_offset(gpu, kv, qdt, g, n, D, bs):
    """V = 1000 + N(0, 1): the output is 1000 and a little; the bound is relative to it."""
    print("case adversarial value offset", kv, qdt, g, n, D, bs, flush=True)
    rng = np.random.default_rng(106)
    lens = [300, 1100]
    K, V, q = _base(rng, lens, g, n, D)
    V = [v + 1000.0 for v in V]
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, seed=9))


@grid
@pytest.mark.parametrize("ratio", [10, 14])
def test_query_heads_of_very_different_magnitude(gpu, kv, qdt, g, n, D, bs, ratio):
    """One head of each GQA group carries queries 2^ratio larger than the others (its attention is one-hot),
    and two other heads' queries of one draft token are 2^8 larger: the ordinary heads beside them — same
    work item, same K tile — must keep their precision.  Checked per head.  (The kernel that serves more
    than 32 rows per kv head over an int8 cache scales its bf16 queries by the work item, not by the row,
    before they become fp16 numbers: rows more than 2^28 below the item's largest element would lose bits.)"""
    print("case adversarial head magnitudes", kv, qdt, g, n, D, bs, ratio, flush=True)
    rng = np.random.default_rng(107)
    lens = [130, 901]
    K, V, q = _base(rng, lens, g, n, D)
    q = q.reshape(len(lens), n, HKV, g, D)
    q[:, :, :, 1] *= 2.0 ** ratio
    if n > 1:
        q[:, 1, :, 2:] *= 2.0 ** 8
    q = q.reshape(len(lens) * n, HKV * g, D)
    if qdt == "fp16":  # (inside fp16's range)
        q = np.clip(q, -6e4, 6e4)
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, seed=10))


@grid
def test_softmax_scale_zero_and_large(gpu, kv, qdt, g, n, D, bs):
    """scale 0: uniform weights, the mean of the values, lse = log2(count).  A scale of 2^12 / sqrt(D) over
    queries 2^-12 smaller: the same scores as the ordinary problem."""
    print("case adversarial softmax scale", kv, qdt, g, n, D, bs, flush=True)
    rng = np.random.default_rng(108)
    lens = [77, 1300]
    K, V, q = _base(rng, lens, g, n, D)
    case = AdvCase(HKV * g, HKV, D, bs, K, V, q, n=n, kv=kv, qdt=qdt, scale=0.0, seed=11)
    got, lse = check(case)
    for b, L in enumerate(lens):
        for j in range(n):
            assert np.abs(lse[b * n + j] - math.log2(L - (n - 1 - j))).max() <= 1e-5
    check(AdvCase(HKV * g, HKV, D, bs, K, V, q * 2.0 ** -12, n=n, kv=kv, qdt=qdt, scale=2.0 ** 12 / math.sqrt(D), seed=12))
