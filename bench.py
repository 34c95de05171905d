#!/usr/bin/env python3
"""Benchmark of the paged-KV decode hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one decode-attention call (split schedule + attention + merge) over one batch of the
workload, with q, the paged KV cache, the block table and the lengths already resident in HBM.
Several disjoint KV pools are rotated from step to step so that the 256 MiB Infinity Cache cannot
serve a repeat.  Prints ONE JSON line: the step time, the achieved HBM rate on the algorithmic
bytes, the roofline of the dominant kernel and a CPU baseline (the torch-CPU restatement of the
same path on the host cores).  The KV write of the step's new tokens is timed separately
(`kv_write_us`).

Two back-to-back regions of K steps each are run after the warm-up.  The first is bracketed by
synchronisations only and gives `value`.  The second repeats the same K steps with a pair of HIP
events recorded (by the library, on the launch stream) around the attention kernel of every step
and gives the kernel's average duration for the roofline; the events cost a few microseconds per
step, which is why they stay out of the region `value` is taken from.
"""
import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBPS = 8000.0
DEFAULT_WORKLOAD = "cfg2_llama3_8b_b64_ctx4k"


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD)
    ap.add_argument("--pools", type=int, default=3, help="disjoint KV pools rotated between steps")
    ap.add_argument("--kv-layout", choices=["HND", "NHD"], default="HND",
                    help="HND [blocks, heads, slots, dim] is the path's native layout; NHD [blocks, slots, heads, dim] "
                         "is what the reference's CUDA backend allocates")
    ap.add_argument("--set", action="append", default=[], metavar="FIELD=VALUE",
                    help="replace a field of the workload (e.g. --set block_size=128 --set batch=16): a variation "
                         "of the named workload, reported under the name <workload>+<field>=<value>")
    ap.add_argument("--kv-skew-bytes", type=int, default=None,
                    help="bytes (a multiple of 16) by which a V pool is displaced from a 2 MiB boundary behind its K "
                         "pool; default: the library's allocation policy (ops.allocate_kv_cache, 4096).  -1 allocates "
                         "K and V separately, as torch.empty per tensor does")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-engine-step", action="store_true",
                    help="skip the write_plus_attend_us leg (the step through the C++ AttentionImpl under a HIP graph)")
    ap.add_argument("--engine-layers", type=int, default=32,
                    help="attention layers per captured model forward in the write_plus_attend_us leg")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="budget of the CPU baseline leg")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 1 GiB device-to-device copy a few times and exit: the known-size "
                         "kernel against which the rocprofv3 FETCH_SIZE / WRITE_SIZE counters are scaled")
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="untimed steps run for this long before the warm-up steps (clock and TLB settling)")
    ap.add_argument("--no-sustained", action="store_true",
                    help="skip the interleaved and sustained timing legs (profiling runs: fewer dispatches to trace)")
    ap.add_argument("--schedule-audit", action="store_true",
                    help="time the scheduling rules' choice against each forced alternative over a grid of shapes "
                         "(cache type x batch x length, equal and lognormal lengths); one JSON line per cell")
    ap.add_argument("--audit-cells", default="", help="comma-separated substrings: only cells whose name holds one")
    ap.add_argument("--aux", action="store_true",
                    help="time the kernels around the decode path instead (KV writes, norm + rotary embedding + "
                         "write, block copy, a chunked-prefill step) and print one JSON line of their own")
    return ap.parse_args()


def build_pools(w, torch, ops, num_blocks, npools, device, layout="HND", skew_bytes=None):
    """KV pools (HND is the native layout), allocated by the library's policy (ops.allocate_kv_cache).
    Quantised pools are produced by the path's own quantising KV write from N(0,1) fp32 values, as
    the workloads define them (generated in fp32, then quantised per token and head)."""
    def allocate(dt, with_scales):
        if skew_bytes is not None and skew_bytes < 0:  # separate allocations
            k, v = torch.empty(shape, device=device, dtype=dt), torch.empty(shape, device=device, dtype=dt)
            if not with_scales:
                return k, v, None, None
            return (k, v, torch.empty(shape[:3], device=device, dtype=torch.float32),
                    torch.empty(shape[:3], device=device, dtype=torch.float32))
        kw = {} if skew_bytes is None else {"skew_bytes": skew_bytes}
        return ops.allocate_kv_cache(shape, dt, device, with_scales, **kw)

    pools = []
    gen = torch.Generator(device=device)
    gen.manual_seed(1234)
    shape = (num_blocks, w.num_kv_heads, w.block_size, w.head_dim) if layout == "HND" else \
        (num_blocks, w.block_size, w.num_kv_heads, w.head_dim)
    for _ in range(npools):
        if w.kv_dtype in ("bf16", "fp32"):
            dt = torch.bfloat16 if w.kv_dtype == "bf16" else torch.float32
            k, v, _, _ = allocate(dt, False)
            for t in (k, v):  # generated in slices: a whole-pool temporary would double the footprint
                flat = t.view(-1)
                for s0 in range(0, flat.numel(), 1 << 28):
                    part = flat[s0:s0 + (1 << 28)]
                    part.copy_(torch.randn(part.numel(), device=device, dtype=dt, generator=gen) * w.value_std)
            pools.append((k, v, None, None))
            continue
        cdt = torch.int8 if w.kv_dtype == "int8" else torch.float8_e4m3fn
        k, v, ks, vs = allocate(cdt, True)
        total_slots = num_blocks * w.block_size
        chunk = 1 << 16
        for s0 in range(0, total_slots, chunk):
            t = min(chunk, total_slots - s0)
            src_k = torch.randn(t, w.num_kv_heads, w.head_dim, device=device, dtype=torch.float32, generator=gen)
            src_v = torch.randn(t, w.num_kv_heads, w.head_dim, device=device, dtype=torch.float32, generator=gen)
            if w.value_std != 1.0:
                src_k *= w.value_std
                src_v *= w.value_std
            slots = torch.arange(s0, s0 + t, device=device, dtype=torch.int32)
            ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(
                key=src_k, value=src_v, k_cache=k, v_cache=v, slot_mapping=slots, k_cache_scale=ks,
                v_cache_scale=vs, kv_layout=layout))
        torch.cuda.synchronize()
        pools.append((k, v, ks, vs))
    return pools


def engine_step_us(torch, w, pools, table, seq_lens, lists, layout, steps, device, hints, layers):
    """The step as the engine runs it, per layer: xllm::layer::AttentionImpl::forward_qkv of the C++
    libtorch shim (rotary embedding + KV write of the step's new tokens in one launch, then the decode
    attention), captured once in a HIP graph and replayed — graph mode of the reference,
    xllm/core/runtime/cuda_graph_executor_impl.cpp:129-180,548-601.  One graph holds one model forward:
    `layers` attention layers (layer i on KV pool i mod pools) that share one AttentionMetadata, the
    layer loop setting plan_info.layer_id (xllm/models/llm/llm_model_base.h:115) so that the split-KV
    schedule is built at layer 0 only, as the reference plans (flashinfer_planinfo.cpp:252-253).
    Returns microseconds per layer over at least `steps` replayed layers.  `hints`: the metadata carries
    the host-side max_seq_len / total_kv_len of the step (the engine knows them when it captures a
    batch-size bucket); without them the kernel choice is independent of host values."""
    import numpy as np

    from xllm_wxh_amd import _xllm_hip_torch as shim
    from xllm_wxh_amd import workloads

    T = w.batch * w.q_per_seq
    Hq, Hkv, D = w.num_q_heads, w.num_kv_heads, w.head_dim
    gen = torch.Generator(device=device)
    gen.manual_seed(7)
    qkv = (torch.randn(T, (Hq + 2 * Hkv) * D, device=device, dtype=torch.float32, generator=gen) * w.q_std).to(torch.bfloat16)
    max_pos = int(seq_lens.max()) + 1
    theta = torch.rand(max_pos, D // 2, device=device, generator=gen) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(torch.bfloat16)
    positions = torch.from_numpy(np.concatenate(
        [np.arange(L - w.q_per_seq, L) for L in seq_lens.astype(np.int64)]).astype(np.int32)).to(device)
    slots = torch.from_numpy(workloads.decode_slots(w, seq_lens, lists)).to(device)
    i32 = lambda a: torch.from_numpy(np.asarray(a, np.int32)).to(device)
    q_cu = i32(np.arange(w.batch + 1) * w.q_per_seq)
    kv_cu = i32(np.concatenate([[0], np.cumsum(seq_lens.astype(np.int64))]))
    md = shim.build_decode_metadata(q_cu, kv_cu, slots, i32(table), w.q_per_seq, int(seq_lens.max()),
                                    int(seq_lens.sum()) if hints else 0)
    md.plan_info.layer_id = 0
    if not hints:
        md.max_seq_len = max_pos  # non-zero (zero means an empty step) but not a tight bound
    hnd = (lambda t: t) if layout == "HND" else (lambda t: t.permute(0, 2, 1, 3))
    hnd_s = (lambda t: t) if layout == "HND" else (lambda t: t.permute(0, 2, 1))
    caches = [shim.KVCache(hnd(k), hnd(v)) if ks is None else shim.KVCache(hnd(k), hnd(v), hnd_s(ks), hnd_s(vs))
              for k, v, ks, vs in pools]
    attn = shim.AttentionImpl(Hq, D, w.sm_scale, Hkv, -1)

    def run_all():
        for layer in range(layers):
            md.plan_info.layer_id = layer
            attn.forward_qkv(md, positions, qkv, cos_sin, False, None, None, 0.0, caches[layer % len(caches)])

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_all()  # also creates the capture stream's decode workspace before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run_all()
    replays = max(3, (steps + layers - 1) // layers)
    for _ in range(max(2, replays // 5)):
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e6 / (replays * layers)


def host_plan_graph_us(torch, ops, w, pools, q, out, block_table, seq_lens_t, seq_lens, layout, steps, layers, bound_lens=None):
    """Graph mode with a plan made on the host before every replay (the reference's
    CudaGraphPersistentParam::update, xllm/core/runtime/cuda_graph_executor_impl.cpp:586-668): `layers`
    xllm_hip_paged_decode_run launches (layer i on KV pool i mod pools) captured once with
    xllm_hip_decode_args::host_plan — at `bound_lens`, other lengths than the replays' when given, as a graph
    captured for a batch-size bucket is —, then replayed; before each replay xllm_hip_paged_decode_plan_host makes the
    schedule from the step's host-side lengths, outside the graph.  Returns (microseconds per layer, microseconds of
    host time per plan call)."""
    ws = torch.empty(ops.WORKSPACE_BYTES, dtype=torch.uint8, device=q.device)
    lens_dev = seq_lens_t.clone()
    quant = pools[0][2] is not None

    def call(i, plan, run, lens=None):
        k, v, ks, vs = pools[i % len(pools)]
        return ops.batch_decode(q, k, out, block_table, lens_dev, v, None, None, ks, vs, scale=w.sm_scale, q_per_seq=w.q_per_seq,
                                kv_layout=layout, kv_cache_quant_bit_size=8 if quant else -1, workspace=ws, plan=plan, run=run,
                                host_plan=True, host_kv_lens=lens)

    import numpy as np
    if bound_lens is not None:
        lens_dev.copy_(torch.from_numpy(np.asarray(bound_lens, np.int32)))
    call(0, True, True, bound_lens if bound_lens is not None else seq_lens)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for i in range(layers):
                call(i, False, True)
    torch.cuda.current_stream().wait_stream(side)
    lens_dev.copy_(seq_lens_t)
    replays = max(3, (steps + layers - 1) // layers)
    for _ in range(2):
        call(0, True, False, seq_lens)
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(replays):
        call(0, True, False, seq_lens)
        graph.replay()
    torch.cuda.synchronize()
    per_layer = (time.perf_counter() - t0) * 1e6 / (replays * layers)
    # the plan call by itself, on an idle stream (in the loop above it also waits for the copy of the plan before
    # last, which stands in the stream behind a whole replay)
    host = 0.0
    for _ in range(20):
        torch.cuda.synchronize()
        h0 = time.perf_counter()
        call(0, True, False, seq_lens)
        host += time.perf_counter() - h0
    torch.cuda.synchronize()
    return per_layer, host * 1e6 / 20


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.stderr.write("bench.py measures the decode path on ONE GPU; --gpus %d is not supported "
                         "(the path has no cross-GPU step, each GPU would run this same kernel on its own "
                         "KV-head or sequence shard).\n" % args.gpus)
        sys.exit(2)

    import numpy as np
    import torch

    from xllm_wxh_amd import ops, workloads

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py needs a GPU (torch.cuda.is_available() is False)\n")
        sys.exit(2)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.copy_calibration:
        src = torch.randn(1 << 29, device=device, dtype=torch.bfloat16)  # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": True, "bytes_read_per_launch": src.numel() * 2,
                          "bytes_written_per_launch": src.numel() * 2, "launches": 10}))
        return
    if args.aux:
        print(json.dumps(aux_kernels(torch, ops, device)), flush=True)
        return
    if args.schedule_audit:
        schedule_audit(torch, ops, device, args.audit_cells)
        return
    w = workloads.WORKLOADS[args.workload]
    if args.set:
        import dataclasses

        changes = {}
        for item in args.set:
            field, _, value = item.partition("=")
            current = getattr(w, field)
            changes[field] = type(current)(value) if not isinstance(current, str) else value
        w = dataclasses.replace(w, name=w.name + "+" + ",".join(args.set), **changes)
    io_dtype = torch.float32 if w.kv_dtype == "fp32" else torch.bfloat16  # query, output, new K/V rows
    seq_lens = workloads.make_seq_lens(w, seed=0)
    table, num_blocks, lists = workloads.make_block_tables(w, seq_lens, seed=0)
    pools = build_pools(w, torch, ops, num_blocks, args.pools, device, args.kv_layout, args.kv_skew_bytes)
    T = w.batch * w.q_per_seq
    gen = torch.Generator(device=device)
    gen.manual_seed(99)
    q = (torch.randn(T, w.num_q_heads, w.head_dim, device=device, dtype=torch.float32, generator=gen) * w.q_std).to(io_dtype)
    out = torch.empty_like(q)
    block_table = torch.from_numpy(table).to(device)
    seq_lens_d = torch.from_numpy(seq_lens).to(device)
    ws = torch.empty(ops.decode_workspace_bytes(w.batch, w.q_per_seq, w.num_q_heads, w.num_kv_heads, w.head_dim),
                     dtype=torch.uint8, device=device)
    quant_bits = 8 if w.kv_dtype in ("fp8", "int8") else -1

    def step(i, events=None):
        k, v, ks, vs = pools[i % len(pools)]
        ops.batch_decode(q, k, out, block_table, seq_lens_d, v, None, None, ks, vs, scale=w.sm_scale,
                         q_per_seq=w.q_per_seq, workspace=ws, kv_cache_quant_bit_size=quant_bits,
                         max_seq_len=int(seq_lens.max()), total_kv_len=int(seq_lens.sum()), events=events,
                         kv_layout=args.kv_layout)

    variant = ops.decode_variant(q, pools[0][0], pools[0][1], block_table, seq_lens_d, pools[0][2], pools[0][3],
                                 q_per_seq=w.q_per_seq, kv_layout=args.kv_layout)
    schedule = ops.decode_describe(q, pools[0][0], pools[0][1], block_table, seq_lens_d, pools[0][2], pools[0][3],
                                   q_per_seq=w.q_per_seq, kv_layout=args.kv_layout, max_seq_len=int(seq_lens.max()),
                                   total_kv_len=int(seq_lens.sum()))

    # HIP events around the attention kernel of every timed step (recorded on the launch stream by
    # the library itself).  torch creates the handles; the first record materialises them.
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    for a, b in ev:
        a.record()
        b.record()
    handles = [(a.cuda_event, b.cuda_event) for a, b in ev]

    # Let clocks and address translation settle first: right after the pools are generated the first
    # ~100 launches of a step run up to 30 % slower than the steady state a serving loop sees.
    t_settle = time.perf_counter()
    i = 0
    while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
        step(i)
        i += 1
        if i % 16 == 0:
            torch.cuda.synchronize()
    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    us_per_step = (t1 - t0) * 1e6 / args.steps
    for i in range(args.steps):
        step(i, handles[i])
    torch.cuda.synchronize()
    us_per_step_with_events = (time.perf_counter() - t1) * 1e6 / args.steps
    kern_us = sorted(a.elapsed_time(b) * 1e3 for a, b in ev)
    kern_avg_us = sum(kern_us) / len(kern_us)

    # the step's KV write, timed on its own
    src_dt = io_dtype
    new_k = torch.randn(T, w.num_kv_heads, w.head_dim, device=device, dtype=src_dt, generator=gen)
    new_v = torch.randn(T, w.num_kv_heads, w.head_dim, device=device, dtype=src_dt, generator=gen)
    slots = torch.from_numpy(workloads.decode_slots(w, seq_lens, lists)).to(device)

    def kv_write(i):
        k, v, ks, vs = pools[i % len(pools)]
        p = ops.ReshapePagedCacheParams(key=new_k, value=new_v, k_cache=k, v_cache=v, slot_mapping=slots,
                                        k_cache_scale=ks, v_cache_scale=vs, kv_layout=args.kv_layout)
        if ks is not None:
            ops.quant_to_paged_cache(p)
        else:
            ops.reshape_paged_cache(p)

    for i in range(5):
        kv_write(i)
    torch.cuda.synchronize()
    t2 = time.perf_counter()
    for i in range(args.steps):
        kv_write(i)
    torch.cuda.synchronize()
    kv_write_us = (time.perf_counter() - t2) * 1e6 / args.steps

    def kv_write_graph_us(reps=50):
        # the kernel itself: 50 writes (rotating pools) captured in a HIP graph, replayed
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for i in range(reps):
                kv_write(i)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e6 / (10 * reps)

    kv_write_in_graph_us = kv_write_graph_us()

    # the schedule (plan) and the attention proper (run) on their own: an engine builds the schedule once per
    # step, at layer 0, and every layer runs on it
    def plan_or_run(i, plan):
        k, v, ks, vs = pools[i % len(pools)]
        ops.batch_decode(q, k, out, block_table, seq_lens_d, v, None, None, ks, vs, scale=w.sm_scale,
                         q_per_seq=w.q_per_seq, workspace=ws, kv_cache_quant_bit_size=quant_bits,
                         max_seq_len=int(seq_lens.max()), total_kv_len=int(seq_lens.sum()), kv_layout=args.kv_layout,
                         plan=plan, run=not plan)

    def run_loop_us():
        # (the legs before this one end in host-side pauses — graph captures, synchronisations — after which the
        # first few hundred launches run up to 15 % slower: settle as before the main leg)
        t_settle = time.perf_counter()
        i = 0
        while (time.perf_counter() - t_settle) * 1e3 < args.settle_ms:
            plan_or_run(i, False)
            i += 1
            if i % 16 == 0:
                torch.cuda.synchronize()
        for i in range(max(3, args.warmup // 2)):
            plan_or_run(i, False)
        torch.cuda.synchronize()
        t = time.perf_counter()
        for i in range(args.steps):
            plan_or_run(i, False)
        torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e6 / args.steps

    def plan_graph_us(reps=50):
        # a plan is a few microseconds of GPU time, less than the binding's launch cost: 50 of them in a graph
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        graph = torch.cuda.CUDAGraph()
        anchor = torch.zeros(64, device=device)
        with torch.cuda.graph(graph, stream=side):
            anchor.add_(1.0)  # (a plan may launch nothing: the graph is never empty)
            for i in range(reps):
                plan_or_run(i, True)
        for _ in range(3):
            graph.replay()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(10):
            graph.replay()
        torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e6 / (10 * reps)

    plan_or_run(0, True)
    run_us = run_loop_us()
    plan_us = plan_graph_us()
    plan_or_run(0, True)

    def interleaved_us(rounds=4, per=50):
        # `value` (plan + run per call) and `run_us` (runs on an existing schedule) in alternating legs, so that a
        # drift of the clocks over the benchmark's run shows in both series instead of between them
        full, runs = [], []
        for i in range(per):  # (settled: see run_loop_us)
            step(i)
        for _ in range(rounds):
            torch.cuda.synchronize()
            t = time.perf_counter()
            for i in range(per):
                step(i)
            torch.cuda.synchronize()
            full.append(round((time.perf_counter() - t) * 1e6 / per, 2))
            plan_or_run(0, True)
            torch.cuda.synchronize()
            t = time.perf_counter()
            for i in range(per):
                plan_or_run(i, False)
            torch.cuda.synchronize()
            runs.append(round((time.perf_counter() - t) * 1e6 / per, 2))
        return full, runs

    def sustained_us(seconds=1.0):
        # back-to-back steps for at least a second (the queue is drained every 256 steps, so that the clock below
        # follows the GPU and not the enqueueing)
        n = 0
        torch.cuda.synchronize()
        t = time.perf_counter()
        while time.perf_counter() - t < seconds:
            for i in range(256):
                step(n + i)
            n += 256
            torch.cuda.synchronize()
        return (time.perf_counter() - t) * 1e6 / n, n

    interleaved_full = interleaved_runs = sustained = sustained_steps = None
    if not args.no_sustained:
        interleaved_full, interleaved_runs = interleaved_us()
        sustained, sustained_steps = sustained_us()

    engine_us = engine_no_hints_us = None
    if io_dtype == torch.bfloat16 and not args.no_engine_step:
        engine_us = engine_step_us(torch, w, pools, table, seq_lens, lists, args.kv_layout, args.steps, device, True,
                                   args.engine_layers)
        engine_no_hints_us = engine_step_us(torch, w, pools, table, seq_lens, lists, args.kv_layout, args.steps, device,
                                            False, args.engine_layers)

    host_plan_us = host_plan_call_us = None
    if not args.no_engine_step:
        # captured at the bucket's bounds (every sequence at the longest length), replayed on the step's own lengths
        bound = np.full(w.batch, int(seq_lens.max()), np.int32)
        host_plan_us, host_plan_call_us = host_plan_graph_us(torch, ops, w, pools, q, out, block_table, seq_lens_d, seq_lens,
                                                             args.kv_layout, args.steps, args.engine_layers, bound)

    alg_bytes = workloads.algorithmic_bytes(w, seq_lens)
    achieved_gbps = alg_bytes / us_per_step / 1e3
    kern_gbps = alg_bytes / kern_avg_us / 1e3

    rows_per_kv_head = w.q_per_seq * (w.num_q_heads // w.num_kv_heads)
    kernel_name = ("decode_generic_kernel" if not variant.startswith("mfma") else
                   "decode_mfma_d128_kernel" if rows_per_kv_head <= 16 else "decode_mfma_d128_rows32_kernel")
    # figures of the committed rocprofv3 runs of this same command (profiles/): HBM bytes per launch from
    # the FETCH_SIZE / WRITE_SIZE counters, and the kernel's average duration in the kernel trace
    traffic = rocprof_avg = rocprof_commit = None
    tpath = os.path.join(REPO, "profiles", "hbm_traffic.json")
    # (they were taken in the default configuration: HND pools with the library's K/V placement)
    if os.path.exists(tpath) and args.kv_layout == "HND" and args.kv_skew_bytes is None:
        entry = json.load(open(tpath)).get(w.name, {})
        traffic = entry.get("traffic_bytes_per_launch")
        rocprof_avg = entry.get("kernel_avg_us")
        rocprof_commit = entry.get("commit", json.load(open(tpath)).get("_commit"))

    result = {
        "metric": "decode-attn us/step + achieved HBM GB/s (% of 8 TB/s), Llama-3-8B shape b64 ctx4k",
        "value": round(us_per_step, 2),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(us_per_step / 1e3, 5),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": w.kv_dtype if w.kv_dtype in ("bf16", "fp32") else "bf16 (KV %s)" % w.kv_dtype,
        "data": "synthetic",
        "config": {
            "workload": w.name,
            "description": w.description,
            "batch": w.batch,
            "q_per_seq": w.q_per_seq,
            "num_q_heads": w.num_q_heads,
            "num_kv_heads": w.num_kv_heads,
            "head_dim": w.head_dim,
            "block_size": w.block_size,
            "kv_dtype": w.kv_dtype,
            "sum_seq_len": int(seq_lens.sum()),
            "max_seq_len": int(seq_lens.max()),
            "kv_layout": args.kv_layout,
            "kv_allocation": ("separate K and V allocations" if (args.kv_skew_bytes or 0) < 0 else
                              "ops.allocate_kv_cache: one buffer, V %d bytes past a 2 MiB boundary behind K"
                              % (ops.KV_SKEW_BYTES if args.kv_skew_bytes is None else args.kv_skew_bytes)),
            "kv_pools_rotated": len(pools),
            "kernel_variant": variant,
            "schedule": schedule,
        },
        "achieved_gbps": round(achieved_gbps, 1),
        "pct_of_hbm_peak": round(100.0 * achieved_gbps / HBM_PEAK_GBPS, 2),
        "algorithmic_bytes": int(alg_bytes),
        "kv_write_us": round(kv_write_us, 2),
        "kv_write_in_graph_us": round(kv_write_in_graph_us, 2),
        "kv_write_us_note": "KV write of the step's new tokens issued through the Python (ctypes) binding, one call per "
                            "step: dominated by the binding's launch cost, not by the kernel; kv_write_in_graph_us: "
                            "the same launches captured in a HIP graph (50 per graph) and replayed",
        "plan_us": round(plan_us, 2),
        "run_us": round(run_us, 2),
        "run_pct_of_hbm_peak": round(100.0 * alg_bytes / run_us / 1e3 / HBM_PEAK_GBPS, 2),
        "plan_run_note": "value = plan + run of every step (xllm_hip_paged_decode); plan_us: the schedule alone "
                         "(xllm_hip_paged_decode_plan; no launch at all when the host-side lengths show that nothing "
                         "is split), run_us: attention (+ merge) on an existing schedule (xllm_hip_paged_decode_run), "
                         "what every layer after layer 0 costs an engine that plans once per step",
        "interleaved_value_us": interleaved_full,
        "interleaved_run_us": interleaved_runs,
        "sustained_us": None if sustained is None else round(sustained, 2),
        "sustained_steps": sustained_steps,
        "timing_note": "interleaved_*: four alternating legs of 50 steps each of plan + run (what `value` times) and "
                       "of runs on an existing schedule (run_us), in the order they ran; sustained_us: plan + run per "
                       "step over at least a second of back-to-back steps",
        "engine_layers": args.engine_layers,
        "write_plus_attend_us": None if engine_us is None else round(engine_us, 2),
        "write_plus_attend_no_hints_us": None if engine_no_hints_us is None else round(engine_no_hints_us, 2),
        "write_plus_attend_note": "per layer, as the engine runs the step: C++ AttentionImpl::forward_qkv (rotary "
                                  "embedding + KV write in one launch, then decode attention) of engine_layers "
                                  "layers sharing one AttentionMetadata, captured once in a HIP graph and replayed "
                                  "(layer i on pool i mod pools; the schedule is built at layer 0 only); no_hints: "
                                  "metadata without the host-side total_kv_len",
        "host_plan_graph_us": None if host_plan_us is None else round(host_plan_us, 2),
        "host_plan_call_us": None if host_plan_call_us is None else round(host_plan_call_us, 1),
        "host_plan_graph_note": "per layer: engine_layers xllm_hip_paged_decode_run launches captured once in a HIP graph "
                                "with xllm_hip_decode_args::host_plan at the bucket's bounds (every sequence at the "
                                "longest length) and replayed on the step's own lengths; before each replay "
                                "xllm_hip_paged_decode_plan_host makes the schedule from the host-side lengths, outside "
                                "the graph (host_plan_call_us: host time of that call through the Python binding). "
                                "Compare with run_us, the eager run with the step's own hints",
        "roofline": {
            "bound": "hbm",
            "kernel": kernel_name,
            "achieved": round(kern_gbps, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(kern_gbps / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "kernel_avg_us": round(kern_avg_us, 2),
            "kernel_min_us": round(kern_us[0], 2),
            "kernel_max_us": round(kern_us[-1], 2),
            "measured": "achieved and frac use kernel_avg_us: the average over HIP events that the library records "
                        "around the attention kernel on its launch stream in %d further steps (%.2f us/step with the "
                        "events); an event pair adds about 2 us of command-processor time to the kernel's own "
                        "duration, which is rocprof_kernel_avg_us" % (args.steps, us_per_step_with_events),
            "rocprof_kernel_avg_us": rocprof_avg,
            "rocprof_commit": rocprof_commit,
            "rocprof_note": "traffic and rocprof_kernel_avg_us are stored figures, read from profiles/hbm_traffic.json: "
                            "they were measured by rocprofv3 on the tree of rocprof_commit, not in this run",
        },
    }

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(w, torch, pools[0], q, block_table, seq_lens, out, step, args)
    print(json.dumps(result), flush=True)


def aux_kernels(torch, ops, device):
    """Average duration (torch events on the launch stream, 50 launches after 5) and algorithmic
    bandwidth of the kernels around the decode path, Llama-3-8B head shape (32 q / 8 kv heads, D 128)."""
    Hq, Hkv, D, bs, nb = 32, 8, 128, 16, 40000  # 40000 blocks of 16 tokens: 2.6 GB of bf16 K+V
    gen = torch.Generator(device=device)
    gen.manual_seed(5)
    kc = torch.randn(nb, Hkv, bs, D, device=device, dtype=torch.bfloat16, generator=gen)
    vc = torch.randn(nb, Hkv, bs, D, device=device, dtype=torch.bfloat16, generator=gen)
    kq = torch.empty(nb, Hkv, bs, D, device=device, dtype=torch.int8)
    vq = torch.empty_like(kq)
    ksc = torch.empty(nb, Hkv, bs, device=device, dtype=torch.float32)
    vsc = torch.empty_like(ksc)
    theta = torch.rand(8192, D // 2, device=device, generator=gen) * 6.283
    cos_sin = torch.cat([torch.cos(theta), torch.sin(theta)], 1).to(torch.bfloat16)

    def timed(fn, n=50, settle_ms=100.0):
        # (settled like the main workload's legs: right after a host-side pause the first launches of a kernel run
        # up to 15 % slower than the steady state a serving loop sees; at least five launches, at most settle_ms)
        t_settle = time.perf_counter()
        i = 0
        while i < 5 or (time.perf_counter() - t_settle) * 1e3 < settle_ms:
            fn()
            i += 1
            if i % 16 == 0:
                torch.cuda.synchronize()
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n

    res = {"aux_kernels": True, "shape": "32 q / 8 kv heads, head_dim 128, bf16 activations", "entries": []}

    def add(name, us, nbytes, note=""):
        res["entries"].append({"kernel": name, "us": round(us, 2), "algorithmic_bytes": int(nbytes),
                               "gbps": round(nbytes / us / 1e3, 1), "note": note})

    for T in (64, 8192):
        qkv = torch.randn(T, (Hq + 2 * Hkv) * D, device=device, dtype=torch.bfloat16, generator=gen)
        key = qkv[:, Hq * D:(Hq + Hkv) * D].view(T, Hkv, D)
        val = qkv[:, (Hq + Hkv) * D:].view(T, Hkv, D)
        slots = torch.randperm(nb * bs, device=device, generator=gen)[:T].to(torch.int32)
        pos = torch.randint(0, 8192, (T,), device=device, generator=gen)
        p16 = ops.ReshapePagedCacheParams(key=key, value=val, k_cache=kc, v_cache=vc, slot_mapping=slots)
        p8 = ops.ReshapePagedCacheParams(key=key, value=val, k_cache=kq, v_cache=vq, slot_mapping=slots,
                                         k_cache_scale=ksc, v_cache_scale=vsc)
        kvb = T * Hkv * D * 2
        add("reshape_paged_cache T=%d" % T, timed(lambda: ops.reshape_paged_cache(p16)), 2 * kvb * 2)
        add("quant_to_paged_cache int8 T=%d" % T, timed(lambda: ops.quant_to_paged_cache(p8)),
            2 * kvb + 2 * kvb // 2 + 2 * T * Hkv * 4)
        add("rope_kv_write bf16 cache T=%d" % T,
            timed(lambda: ops.rope_kv_write(qkv, Hq, Hkv, D, cos_sin, pos, kc, vc, slots, round_each_op=True)),
            T * ((2 * Hq + 2 * Hkv) * D * 2 + Hkv * D * 2 + 2 * Hkv * D * 2), "q,k read+written, v read, cache written")
        add("rope_kv_write int8 cache T=%d" % T,
            timed(lambda: ops.rope_kv_write(qkv, Hq, Hkv, D, cos_sin, pos, kq, vq, slots, round_each_op=True,
                                            k_cache_scale=ksc, v_cache_scale=vsc)),
            T * ((2 * Hq + 2 * Hkv) * D * 2 + Hkv * D * 2 + 2 * Hkv * D + 2 * Hkv * 4))
    for nblk in (64, 4096):
        perm = torch.randperm(nb, device=device, generator=gen)
        src, dst = perm[:nblk].contiguous(), perm[nblk:2 * nblk].contiguous()
        blk_bytes = 2 * Hkv * bs * D * 2
        add("swap_blocks in place, %d blocks of 16 tokens" % nblk,
            timed(lambda: ops.swap_blocks(kc, vc, src, dst, exact=False)), 2 * nblk * blk_bytes, "read + write")
        add("swap_blocks gather-then-scatter, %d blocks" % nblk,
            timed(lambda: ops.swap_blocks(kc, vc, src, dst, exact=True)), 4 * nblk * blk_bytes,
            "two passes through a staging buffer allocated per call")
    # sequences read back out of the cache: 32 sequences of 4096 tokens
    B, L = 32, 4096
    table = torch.randperm(nb, device=device, generator=gen)[: B * (L // bs)].to(torch.int32).view(B, L // bs)
    lens = torch.full((B,), L, device=device, dtype=torch.int32)
    dk = torch.empty(B * L, Hkv, D, device=device, dtype=torch.bfloat16)
    dv = torch.empty_like(dk)
    kvb = B * L * Hkv * D * 2  # elements of K and V
    add("reshape_from_cache bf16, 32 x 4096 tokens", timed(lambda: ops.reshape_from_cache(dk, dv, kc, vc, lens, L, None, table)),
        2 * kvb * 2, "read + write")
    ops.quant_to_paged_cache(ops.ReshapePagedCacheParams(
        key=dk[:4096], value=dv[:4096], k_cache=kq, v_cache=vq, k_cache_scale=ksc, v_cache_scale=vsc,
        slot_mapping=torch.arange(4096, device=device, dtype=torch.int32)))
    add("dequant_from_paged_cache int8 -> bf16, 32 x 4096 tokens",
        timed(lambda: ops.dequant_from_paged_cache(dk, dv, kq, vq, ksc, vsc, lens, L, None, table)),
        kvb + B * L * Hkv * 4 * 2 + kvb * 2, "1-byte cache and scales read, bf16 written")
    del dk, dv
    # a chunked-prefill step: 4 sequences, 512 new tokens each on top of a 3584-token prefix
    B, n, L = 4, 512, 4096
    q = torch.randn(B * n, Hq, D, device=device, dtype=torch.bfloat16, generator=gen)
    out = torch.empty_like(q)
    table = torch.randperm(nb, device=device, generator=gen)[: B * (L // bs)].to(torch.int32).view(B, L // bs)
    lens = torch.full((B,), L, device=device, dtype=torch.int32)
    q_indptr = (torch.arange(B + 1, device=device) * n).to(torch.int32)
    us = timed(lambda: ops.batch_decode(q, kc, out, table, lens, vc, scale=D ** -0.5, q_per_seq=n, q_indptr=q_indptr,
                                        max_seq_len=L, total_kv_len=B * L), n=10)
    flops = 4.0 * B * Hq * D * sum(L - n + 1 + j for j in range(n))
    res["entries"].append({"kernel": "chunked prefill (256-row kernel), 4 x 512 tokens on a 3584-token prefix, bf16",
                           "us": round(us, 1), "tflops": round(flops / us / 1e6, 1),
                           "frac_of_mfma_peak": round(flops / us / 1e6 / 2500.0, 3),
                           "note": "flops of the visible (causal) part only; every 256 query rows stream the "
                                   "sequence's K/V again, from the L2 of their XCD"})
    with ops.option("prefill_kernel", 1):
        us128 = timed(lambda: ops.batch_decode(q, kc, out, table, lens, vc, scale=D ** -0.5, q_per_seq=n, q_indptr=q_indptr,
                                               max_seq_len=L, total_kv_len=B * L), n=10)
    res["entries"].append({"kernel": "the same through the 128-row kernel (XLLM_HIP_OPTION_PREFILL_KERNEL = 1)",
                           "us": round(us128, 1), "tflops": round(flops / us128 / 1e6, 1),
                           "frac_of_mfma_peak": round(flops / us128 / 1e6 / 2500.0, 3), "note": ""})
    # a plain prefill: 4 sequences of 4096 tokens from an empty cache (the whole sequence is the chunk)
    n2 = 4096
    q2 = torch.randn(B * n2, Hq, D, device=device, dtype=torch.bfloat16, generator=gen)
    out2 = torch.empty_like(q2)
    q_indptr2 = (torch.arange(B + 1, device=device) * n2).to(torch.int32)
    us2 = timed(lambda: ops.batch_decode(q2, kc, out2, table, lens, vc, scale=D ** -0.5, q_per_seq=n2, q_indptr=q_indptr2,
                                         max_seq_len=L, total_kv_len=B * L), n=5)
    flops2 = 4.0 * B * Hq * D * sum(j + 1 for j in range(n2))
    res["entries"].append({"kernel": "prefill (256-row kernel), 4 x 4096 tokens from an empty cache, bf16",
                           "us": round(us2, 1), "tflops": round(flops2 / us2 / 1e6, 1),
                           "frac_of_mfma_peak": round(flops2 / us2 / 1e6 / 2500.0, 3),
                           "note": "causal: flops of the visible part only"})
    del q2, out2
    def int8_in_place():
        ops.batch_decode(q, kq, out, table, lens, vq, None, None, ksc, vsc, scale=D ** -0.5, q_per_seq=n,
                         q_indptr=q_indptr, max_seq_len=L, total_kv_len=B * L, kv_cache_quant_bit_size=8)

    us = timed(int8_in_place, n=10)
    res["entries"].append({"kernel": "chunked prefill over an int8 cache in place (256-row kernel for 1-byte caches), 4 x 512 tokens on a 3584-token prefix",
                           "us": round(us, 1), "tflops": round(flops / us / 1e6, 1),
                           "frac_of_mfma_peak": round(flops / us / 1e6 / 2500.0, 3),
                           "note": "every 256 query rows stream the sequence's K/V bytes and convert them to fp16 tiles in LDS again"})
    with ops.option("prefill_kernel", 1):
        us128 = timed(int8_in_place, n=10)
    res["entries"].append({"kernel": "the same through the 128-row kernel for 1-byte caches (XLLM_HIP_OPTION_PREFILL_KERNEL = 1)",
                           "us": round(us128, 1), "tflops": round(flops / us128 / 1e6, 1),
                           "frac_of_mfma_peak": round(flops / us128 / 1e6 / 2500.0, 3), "note": ""})
    # speculative verify with 64 query rows per kv head (64 q heads, 8 draft tokens)
    B, n, L, Hq2 = 32, 8, 8192, 64
    q = torch.randn(B * n, Hq2, D, device=device, dtype=torch.bfloat16, generator=gen)
    out = torch.empty_like(q)
    table = torch.randperm(nb, device=device, generator=gen)[: B * (L // bs)].to(torch.int32).view(B, L // bs)
    lens = torch.full((B,), L, device=device, dtype=torch.int32)
    us = timed(lambda: ops.batch_decode(q, kc, out, table, lens, vc, scale=D ** -0.5, q_per_seq=n, max_seq_len=L,
                                        total_kv_len=B * L), n=20)
    add("verify, 64 rows per kv head (128-row kernel, half of its waves idle), 32 x 8192 tokens bf16", us,
        B * L * Hkv * D * 2 * 2, "K/V bytes")
    return res


def schedule_audit(torch, ops, device, only=""):
    """For every cell of a fixed grid, the decode step as the library's rules shape it (hints = the true lengths)
    against the same step with each rule forced the other way (xllm_hip_set_option), without hints, and with the
    schedule made on the host.  Timed per layer on an existing schedule (plan once, then runs), the figure
    `run_us` is; a cell's `loss_pct` is how far the rules' choice is behind the fastest alternative."""
    import numpy as np

    Hq, Hkv, D, bs = 32, 8, 128, 16
    max_tokens = 4 << 20
    nb = max_tokens // bs + 4096
    gen = torch.Generator(device=device)
    gen.manual_seed(11)
    rng = np.random.default_rng(11)
    caches = {}

    def cache(kind):
        if kind not in caches:
            caches.clear()  # one pool at a time
            torch.cuda.empty_cache()
            if kind == "bf16":
                k = torch.randn(nb, Hkv, bs, D, device=device, dtype=torch.bfloat16, generator=gen)
                v = torch.randn(nb, Hkv, bs, D, device=device, dtype=torch.bfloat16, generator=gen)
                caches[kind] = (k, v, None, None)
            else:
                raw = torch.randint(-100, 100, (2, nb, Hkv, bs, D), device=device, dtype=torch.int8, generator=gen)
                if kind == "fp8":
                    raw = (raw.to(torch.float32) / 16).to(torch.float8_e4m3fn)
                sc = torch.rand(2, nb, Hkv, bs, device=device, generator=gen) * 0.01 + 0.005
                caches[kind] = (raw[0], raw[1], sc[0], sc[1])
        return caches[kind]

    def timed(fn, n):
        for _ in range(3):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(n):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e3 / n

    alternatives = [("no_hints", {}, "nohints"), ("host_plan", {}, "host"), ("stored_schedule", {"stored_schedule": 1}, None),
                    ("item_per_head", {"item_per_head": 1}, None), ("four_wave_items", {"four_wave_items": 1}, None),
                    ("separate_merge", {"separate_merge": 1}, None), ("target_256", {"target_items": 256}, None)]
    wanted = [t for t in only.split(",") if t]
    worst, host_wins = [], []
    for kind in ("bf16", "fp8", "int8"):
        for B in (16, 64, 256, 1024):
            for mean in (256, 2048, 8192, 32768):
                for dist in ("equal", "lognormal"):
                    name = "%s_b%d_l%d_%s" % (kind, B, mean, dist)
                    if B * mean > max_tokens // 2 or (wanted and not any(t in name for t in wanted)):
                        continue
                    if dist == "equal":
                        lens = np.full(B, mean, dtype=np.int64)
                    else:
                        lens = np.clip(rng.lognormal(np.log(mean), 0.8, B), 16, 4 * mean).astype(np.int64)
                        lens = np.minimum(lens, max(16, (max_tokens - 16 * B) // B * 4))
                        while lens.sum() > max_tokens - 16 * B:
                            lens = np.maximum(lens * 9 // 10, 16)
                    k, v, ks, vs = cache(kind)
                    blocks = (lens + bs - 1) // bs
                    table = torch.zeros(B, int(blocks.max()), dtype=torch.int32, device=device)
                    perm = torch.randperm(nb, device=device, generator=gen).to(torch.int32)
                    o = 0
                    for b in range(B):
                        table[b, : blocks[b]] = perm[o: o + blocks[b]]
                        o += int(blocks[b])
                    seq_lens = torch.from_numpy(lens.astype(np.int32)).to(device)
                    q = torch.randn(B, Hq, D, device=device, dtype=torch.bfloat16, generator=gen)
                    out = torch.empty_like(q)
                    ws = torch.empty(ops.WORKSPACE_BYTES, dtype=torch.uint8, device=device)
                    host_lens = [int(x) for x in lens]

                    base = dict(scale=D ** -0.5, q_per_seq=1, workspace=ws, kv_cache_quant_bit_size=8 if ks is not None else -1)
                    by_mode = {"host": dict(base, host_plan=True), "nohints": base,
                               None: dict(base, max_seq_len=int(lens.max()), total_kv_len=int(lens.sum()))}

                    def step(mode, plan, run):
                        # (the same host-side work in every mode: a step of under 20 us is timed by its launch)
                        kw = by_mode[mode]
                        if mode == "host" and plan:
                            kw = dict(kw, host_kv_lens=host_lens)
                        ops.batch_decode(q, k, out, table, seq_lens, v, None, None, ks, vs, plan=plan, run=run, **kw)

                    def measure(mode, opts):
                        import contextlib
                        with contextlib.ExitStack() as st:
                            for key, val in opts.items():
                                st.enter_context(ops.option(key, val))
                            step(mode, True, False)
                            n = max(5, min(50, int(20000 / max(20.0, B * mean / 4000.0))))
                            return timed(lambda: step(mode, False, True), n)

                    measure(None, {})  # (the cell's first measurement runs on cold caches and a ramping clock)
                    rule = measure(None, {})
                    res = {alt: round(measure(mode, opts), 1) for alt, opts, mode in alternatives}
                    rule = min(rule, measure(None, {}))  # (and once more behind the alternatives: the smaller counts)
                    # the forced alternatives (and the call without hints) against the rules' choice; the schedule made
                    # on the host is another entry point, which needs every length on the host: reported beside them
                    host_us = res.pop("host_plan")
                    best_name = min(res, key=res.get)
                    best = min(res[best_name], rule)
                    loss = (rule - best) / best * 100.0
                    kv_bytes = float(lens.sum()) * Hkv * D * 2 * (2 if kind == "bf16" else 1)
                    line = {"cell": name, "rule_us": round(rule, 1), "frac_of_8TBs": round(kv_bytes / rule / 8e6, 3),
                            "alternatives_us": res, "best": best_name if res[best_name] < rule else "rule",
                            "loss_pct": round(loss, 1), "host_plan_us": host_us,
                            "host_plan_gain_pct": round((rule - host_us) / host_us * 100.0, 1)}
                    print(json.dumps(line), flush=True)
                    if loss > 3.0:
                        worst.append((name, round(loss, 1), best_name))
                    if rule > host_us * 1.03:
                        host_wins.append((name, line["host_plan_gain_pct"]))
                    del table, seq_lens, q, out, ws
    print(json.dumps({"schedule_audit_summary": True, "cells_where_a_forced_alternative_wins_by_over_3_pct": worst,
                      "cells_where_the_host_plan_wins_by_over_3_pct": host_wins}), flush=True)


def cpu_baseline(w, torch, pool, q, block_table, seq_lens, out, step, args):
    """The torch-CPU restatement of the same step on the host cores (baseline only).  Runs on a
    bounded sample: the first `nseq` sequences of the batch, chosen so that the leg stays within
    --cpu-seconds; the per-step figure is scaled to the whole batch by kv tokens."""
    import numpy as np

    from oracle import torch_cpu_path as tcp

    cores = torch.get_num_threads()
    k, v, ks, vs = pool
    if args.kv_layout == "NHD":  # the CPU path reads [blocks, heads, slots, dim] views
        k, v = k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3)
        if ks is not None:
            ks, vs = ks.permute(0, 2, 1), vs.permute(0, 2, 1)
    total_tokens = int(seq_lens.sum())
    # sample: whole batch unless it is very large
    nseq = w.batch
    budget_tokens = 400_000
    if total_tokens > budget_tokens:
        csum = np.cumsum(seq_lens.astype(np.int64))
        nseq = max(1, int(np.searchsorted(csum, budget_tokens)))
    sample_tokens = int(seq_lens[:nseq].sum())
    tbl = block_table[:nseq].cpu()
    used = torch.unique(tbl.flatten())
    remap = torch.zeros(int(k.size(0)), dtype=torch.long)
    remap[used.long()] = torch.arange(used.numel())
    tbl_c = remap[tbl.long()].to(torch.int32)
    kc, vc = k[used.to(k.device).long()].cpu(), v[used.to(k.device).long()].cpu()
    ksc = ks[used.to(k.device).long()].cpu() if ks is not None else None
    vsc = vs[used.to(k.device).long()].cpu() if vs is not None else None
    if ks is None:
        kc, vc = kc.float(), vc.float()
    qc = q[: nseq * w.q_per_seq].cpu().float()
    lens_c = torch.from_numpy(seq_lens[:nseq].copy())

    def run():
        return tcp.paged_decode(qc, kc, vc, tbl_c, lens_c, w.sm_scale, q_per_seq=w.q_per_seq, k_scale=ksc,
                                v_scale=vsc)

    ref = run()  # warm-up, also the check below
    times = []
    t_start = time.perf_counter()
    runs = 20 if w.kv_dtype == "fp32" else 3
    while len(times) < runs and (time.perf_counter() - t_start) < args.cpu_seconds:
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    sample_us = sorted(times)[len(times) // 2] * 1e6
    scaled_us = sample_us * total_tokens / max(sample_tokens, 1)
    # sanity: the GPU result of the same pool agrees with the CPU one on the sample
    step(0)
    torch.cuda.synchronize()
    err = float((out[: nseq * w.q_per_seq].float().cpu() - ref).abs().max())
    return {
        "value": round(scaled_us, 1),
        "unit": "us/step",
        "cores": cores,
        "kind": "port",
        "sample": "%d of %d sequences (%d of %d kv tokens), median of %d runs after 1 warm-up, %.0f us on the "
                  "sample, scaled by kv tokens; torch-CPU fp32 gather+bmm+softmax+bmm"
                  % (nseq, w.batch, sample_tokens, total_tokens, len(times), sample_us),
        "gpu_vs_cpu_max_abs_err_on_sample": round(err, 5),
    }


if __name__ == "__main__":
    main()
