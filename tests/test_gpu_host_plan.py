"""The decode schedule made on the host (xllm_hip_paged_decode_plan_host) through the C ABI, against the oracle:
ragged batches on every kernel that splits sequences, both block-list forms, and a run captured once in a graph
and replayed on other lengths, each replay behind a new plan — what the reference's graph executor does before
every replay (xllm/core/runtime/cuda_graph_executor_impl.cpp:586-668)."""
import numpy as np
import pytest
import torch

from oracle import paged_kv_oracle as orc
from tests.helpers import Case, lse_err, max_abs_err, max_rel_err_per_seq
from xllm_wxh_amd import ops

pytestmark = pytest.mark.gpu


def ragged(B, mean, seed, extremes=True):
    rng = np.random.default_rng(seed)
    lens = np.clip(np.round(rng.lognormal(np.log(mean), 0.8, B)), 1, 40000).astype(np.int32)
    if extremes and B >= 5:
        lens[0], lens[1], lens[2] = 0, 1, 33
    return lens


@pytest.mark.parametrize("kv,layout", [("bf16", "HND"), ("fp8", "HND"), ("int8", "HND"), ("fp8", "NHD"), ("bf16", "NHD")])
@pytest.mark.parametrize("B,mean,Hq,Hkv,D,bs,n", [(5, 6000, 32, 8, 128, 16, 1), (40, 1500, 64, 8, 128, 16, 1),
                                                  (9, 3000, 64, 8, 128, 128, 2), (6, 5000, 64, 8, 128, 16, 4),
                                                  (7, 4000, 14, 2, 64, 32, 1), (4, 5000, 16, 4, 256, 16, 1)])
def test_host_plan_matches_oracle(gpu, kv, layout, B, mean, Hq, Hkv, D, bs, n):
    print("case host plan", kv, layout, B, mean, Hq, Hkv, D, bs, n, flush=True)
    c = Case(B, Hq, Hkv, D, bs, ragged(B, mean, seed=B + n), n=n, kv=kv, layout=layout, seed=50 + B)
    ref, ref_lse = c.oracle()
    out, lse = c.run(host_kv_lens=c.lens)
    err, rel = max_abs_err(out, ref), max_rel_err_per_seq(out, ref, n)
    print("   err %.3e rel %.3e" % (err, rel), flush=True)
    assert err <= c.tol and rel <= (3e-2 if kv == "bf16" else 8e-2)
    assert lse_err(lse, ref_lse) <= (1e-2 if kv == "bf16" else 5e-2)
    # the device-side plan serves the same arguments (host_plan without lengths): same schedule format
    out2, _ = c.run(host_plan=True)
    assert max_abs_err(out2, ref) <= c.tol


def test_host_plan_generic_kernel_and_csr_form(gpu):
    print("case host plan generic / csr", flush=True)
    c = Case(6, 14, 2, 64, 16, [700, 0, 3000, 1, 64, 129], kv="fp32", qdt="fp32", seed=61)
    assert c.variant() == "generic"
    ref, _ = c.oracle()
    out, _ = c.run(host_kv_lens=c.lens)
    assert max_abs_err(out, ref) <= 1e-4
    # CSR form over an NHD fp8 cache, lengths from the same host vector
    c = Case(7, 32, 8, 128, 16, ragged(7, 5000, 3), kv="fp8", layout="NHD", seed=62)
    ref, _ = c.oracle()
    need = (c.lens.astype(np.int64) + c.bs - 1) // c.bs
    indptr = np.concatenate([[0], np.cumsum(need)]).astype(np.int32)
    indices = np.concatenate([c.table[b, : need[b]] for b in range(c.B)]).astype(np.int32)
    last = np.where(c.lens > 0, (c.lens - 1) % c.bs + 1, 0).astype(np.int32)
    out = torch.full_like(c.q, float("nan"))
    dev = c.q.device
    ops.batch_decode_csr(c.q, c.k_cache, c.v_cache, torch.from_numpy(indptr).to(dev), torch.from_numpy(indices).to(dev),
                         torch.from_numpy(last).to(dev), -1, c.scale, out, k_cache_scale=c.k_scale, v_cache_scale=c.v_scale,
                         kv_layout="NHD", host_kv_lens=c.lens)
    torch.cuda.synchronize()
    assert max_abs_err(out, ref) <= c.tol


def test_host_plan_cuts_by_length(gpu):
    """What the plan reports: one long sequence among short ones is the only one cut; equal sequences that fill
    the GPU stay whole."""
    c = Case(33, 32, 8, 128, 16, [30000] + [200] * 32, seed=63)
    out = torch.empty_like(c.q)
    info = ops.batch_decode(c.q, c.k_cache, out, c.block_table, c.seq_lens, c.v_cache, scale=c.scale, run=False,
                            host_kv_lens=c.lens)
    assert info["chunk_tokens"] > 0 and 33 < info["sequence_chunks"] <= 33 + 32
    ref, _ = c.oracle()
    got, _ = c.run(host_kv_lens=c.lens)
    assert max_abs_err(got, ref) <= c.tol
    c = Case(64, 32, 8, 128, 16, [1024] * 64, seed=64)
    info = ops.batch_decode(c.q, c.k_cache, torch.empty_like(c.q), c.block_table, c.seq_lens, c.v_cache, scale=c.scale,
                            run=False, host_kv_lens=c.lens)
    assert info["chunk_tokens"] == 0 and info["sequence_chunks"] == 64


@pytest.mark.parametrize("kv,n", [("bf16", 1), ("fp8", 1), ("int8", 4)])
def test_captured_run_replayed_behind_new_host_plans(gpu, kv, n):
    """One xllm_hip_paged_decode_run captured in a graph, replayed three times on other lengths: before each
    replay the lengths on the device are rewritten and the plan is made again on the host, outside the graph.
    Every replay is checked against the oracle and against the eager call on the same lengths."""
    print("case replay", kv, n, flush=True)
    B, Hq, Hkv, D, bs = 12, 64, 8, 128, 16
    cap = ragged(B, 6000, seed=7, extremes=False)
    cap[:] = cap.max()
    c = Case(B, Hq, Hkv, D, bs, cap, n=n, kv=kv, seed=70)
    dev = c.q.device
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)  # one workspace for the plan's stream and the graph's
    seq_lens = c.seq_lens.clone()
    out = torch.zeros_like(c.q)
    kw = dict(scale=c.scale, q_per_seq=n, kv_cache_quant_bit_size=8 if c.k_scale is not None else -1, workspace=ws)

    def decode(plan, run, lens=None):
        return ops.batch_decode(c.q, c.k_cache, out, c.block_table, seq_lens, c.v_cache, None, None, c.k_scale, c.v_scale,
                                plan=plan, run=run, host_plan=True, host_kv_lens=lens, **kw)

    first = ragged(B, 3000, seed=8, extremes=False)
    seq_lens.copy_(torch.from_numpy(np.minimum(first, cap)))
    decode(True, True, np.minimum(first, cap))  # warm-up, eager
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            decode(False, True)
    torch.cuda.current_stream().wait_stream(side)
    for step, seed in enumerate((11, 12, 13)):
        lens = np.minimum(ragged(B, [1500, 6000, 300][step], seed=seed), cap)
        seq_lens.copy_(torch.from_numpy(lens))
        decode(True, False, lens)
        out.fill_(float("nan"))
        torch.cuda.synchronize()  # (eager work and a synchronisation between the replays)
        graph.replay()
        torch.cuda.synchronize()
        ref, _ = orc.paged_decode(c.q_ref, c.k_ref, c.v_ref, c.table, lens, c.scale, q_per_seq=n)
        err = max_abs_err(out, ref)
        print("   replay %d err %.3e" % (step, err), flush=True)
        assert err <= c.tol
        replayed = out.clone()
        decode(True, True, lens)
        torch.cuda.synchronize()
        assert torch.equal(replayed.view(torch.int16), out.view(torch.int16))
