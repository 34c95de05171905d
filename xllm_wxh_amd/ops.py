"""Operator mirror of xllm::kernel for the paged-KV decode path, over the C ABI.

Names, argument meaning and error behaviour follow the reference operators:

  reshape_paged_cache(params)   xllm/core/kernels/ops_api.cpp:150-180
  quant_to_paged_cache(params)  xllm/core/kernels/ops_api.cpp:196-210
  ReshapePagedCacheParams       xllm/core/kernels/param.h:122-157
  batch_decode(...)             xllm/core/kernels/mlu/mlu_ops_api.h:126-145 (block_table form)
  batch_decode_csr(...)         xllm/core/kernels/cuda/cuda_ops_api.h:120-136 (CSR form)

Tensors are torch tensors on the GPU; this module only extracts pointers,
sizes and strides and passes them, with torch's current stream, through ctypes.
Outputs are pre-allocated by the caller and mutated in place, as in the
reference.  The reference aborts on a contract violation (glog CHECK); here the
library's non-zero status becomes an XllmHipError.

Cache tensors are given in the HND logical shape [num_blocks, num_kv_heads,
block_size, head_dim] with any strides whose last dimension is contiguous, so an
NHD buffer [num_blocks, block_size, num_kv_heads, head_dim] (the CUDA backend's
shape, xllm/core/distributed_runtime/llm_engine.cpp:574-577) is passed as
`cache.permute(0, 2, 1, 3)` or with `kv_layout="NHD"`, without a copy.
"""
import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from . import _lib

_DTYPES = {
    torch.bfloat16: _lib.BF16,
    torch.float16: _lib.FP16,
    torch.float32: _lib.FP32,
    torch.float8_e4m3fn: _lib.FP8_E4M3,
    torch.int8: _lib.INT8,
}


def _dtype_code(t):
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise _lib.XllmHipError(_lib.INVALID_ARGUMENT, "unsupported dtype %s" % t.dtype)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require(cond, msg):
    if not cond:
        raise _lib.XllmHipError(_lib.INVALID_ARGUMENT, msg)


class option:
    """Context manager: a process-wide diagnostic switch of the library (xllm_hip_set_option) set for
    the duration of a block.  Names: the keys of `_IDS`."""

    _IDS = {"force_generic": _lib.OPTION_DECODE_FORCE_GENERIC, "target_items": _lib.OPTION_DECODE_TARGET_ITEMS,
            "separate_merge": _lib.OPTION_DECODE_SEPARATE_MERGE, "stored_schedule": _lib.OPTION_DECODE_STORED_SCHEDULE,
            "item_per_head": _lib.OPTION_DECODE_ITEM_PER_HEAD,
            "four_wave_items": _lib.OPTION_DECODE_FOUR_WAVE_ITEMS, "prefill_kernel": _lib.OPTION_PREFILL_KERNEL}

    def __init__(self, name, value=1):
        self.which, self.value = self._IDS[name], int(value)

    def __enter__(self):
        lib = _lib.load()
        self.old = lib.xllm_hip_get_option(self.which)
        _lib.check(lib.xllm_hip_set_option(self.which, self.value))
        return self

    def __exit__(self, *exc):
        _lib.check(_lib.load().xllm_hip_set_option(self.which, self.old))
        return False


def _as_hnd(cache, kv_layout):
    if cache is None:
        return None
    _require(cache.dim() == 4, "cache must be 4-D, got %d-D" % cache.dim())
    if kv_layout == "NHD":
        return cache.permute(0, 2, 1, 3)
    _require(kv_layout == "HND", "kv_layout must be 'HND' or 'NHD'")
    return cache


def _cache_desc(k_cache, v_cache, k_scale, v_scale, kv_layout):
    k = _as_hnd(k_cache, kv_layout)
    v = _as_hnd(v_cache, kv_layout)
    _require(k.is_cuda, "k_cache must live on the GPU")
    _require(k.stride(3) == 1, "head_dim of k_cache must be contiguous")
    if v is not None:
        _require(v.shape == k.shape and v.dtype == k.dtype and v.stride() == k.stride(),
                 "v_cache must match k_cache in shape, dtype and strides")
    d = _lib.KvCacheDesc()
    d.k_cache = k.data_ptr()
    d.v_cache = v.data_ptr() if v is not None else None
    d.num_blocks, d.num_kv_heads, d.block_size, d.head_dim = k.shape
    d.dtype = _dtype_code(k)
    d.stride_block, d.stride_head, d.stride_slot = k.stride(0), k.stride(1), k.stride(2)
    if k_scale is not None:
        ks = k_scale.permute(0, 2, 1) if kv_layout == "NHD" else k_scale
        _require(ks.dtype == torch.float32 and tuple(ks.shape) == tuple(k.shape[:3]),
                 "k_cache_scale must be float32 [num_blocks, num_kv_heads, block_size]")
        d.k_scale = ks.data_ptr()
        d.scale_stride_block, d.scale_stride_head, d.scale_stride_slot = ks.stride()
        if v_scale is not None:
            vs = v_scale.permute(0, 2, 1) if kv_layout == "NHD" else v_scale
            _require(vs.dtype == torch.float32 and vs.shape == ks.shape and vs.stride() == ks.stride(),
                     "v_cache_scale must match k_cache_scale")
            d.v_scale = vs.data_ptr()
    return d


@dataclass
class ReshapePagedCacheParams:
    """Fields of xllm::kernel::ReshapePagedCacheParams (xllm/core/kernels/param.h:122-157)."""

    key: torch.Tensor = None                       # [num_tokens, num_kv_heads, head_dim]
    value: Optional[torch.Tensor] = None
    k_cache: torch.Tensor = None                   # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: Optional[torch.Tensor] = None
    slot_mapping: torch.Tensor = None              # [num_tokens] int32
    direction: bool = False                        # false = CONTEXT2CACHE; true is not part of this path
    k_cache_scale: Optional[torch.Tensor] = None   # [num_blocks, num_kv_heads, block_size] float32
    v_cache_scale: Optional[torch.Tensor] = None
    kv_layout: str = "HND"


def _check_write_inputs(params):
    key, value = params.key, params.value
    _require(key is not None and params.k_cache is not None and params.slot_mapping is not None,
             "key, k_cache and slot_mapping are required")
    _require(not params.direction, "direction=true (cache to context) is not part of the decode path")
    _require(key.dim() == 3, "key must be [num_tokens, num_kv_heads, head_dim]")
    # keys and values should be continuous at n_kv_heads and head_dim dims
    # (xllm/core/kernels/cuda/reshape_paged_cache.cu:68-69)
    _require(key.stride(-1) == 1 and key.stride(-2) == key.size(-1),
             "key must be contiguous in its last two dimensions")
    if value is not None:
        _require(value.shape == key.shape and value.dtype == key.dtype, "value must match key")
        _require(value.stride(-1) == 1 and value.stride(-2) == value.size(-1),
                 "value must be contiguous in its last two dimensions")
        _require(params.v_cache is not None, "value given without v_cache")
    else:
        _require(params.v_cache is None, "v_cache given without value")
    sm = params.slot_mapping
    _require(sm.dtype == torch.int32 and sm.dim() == 1 and sm.is_contiguous(),
             "slot_mapping must be a contiguous int32 vector")
    _require(sm.numel() == key.size(0), "slot_mapping has %d entries for %d tokens" % (sm.numel(), key.size(0)))


def reshape_paged_cache(params: ReshapePagedCacheParams) -> None:
    """Verbatim KV write through slot_mapping."""
    _check_write_inputs(params)
    lib = _lib.load()
    desc = _cache_desc(params.k_cache, params.v_cache, None, None, params.kv_layout)
    _require(params.key.size(1) == desc.num_kv_heads and params.key.size(2) == desc.head_dim,
             "key heads/head_dim do not match the cache")
    key, value = params.key, params.value
    _lib.check(lib.xllm_hip_reshape_paged_cache(
        ctypes.byref(desc), _ptr(key), _ptr(value), _ptr(params.slot_mapping), key.size(0),
        key.stride(0), value.stride(0) if value is not None else 0, _dtype_code(key), _stream()))


def quant_to_paged_cache(params: ReshapePagedCacheParams) -> None:
    """Per-token-per-head quantising KV write (int8 or fp8-e4m3 cache + fp32 scales)."""
    _check_write_inputs(params)
    # CHECK(params.k_cache_scale.has_value()) (xllm/core/kernels/ops_api.cpp:198-199)
    _require(params.k_cache_scale is not None, "k_cache_scale is required for quant_to_paged_cache")
    lib = _lib.load()
    desc = _cache_desc(params.k_cache, params.v_cache, params.k_cache_scale, params.v_cache_scale,
                       params.kv_layout)
    _require(params.key.size(1) == desc.num_kv_heads and params.key.size(2) == desc.head_dim,
             "key heads/head_dim do not match the cache")
    key, value = params.key, params.value
    _lib.check(lib.xllm_hip_quant_to_paged_cache(
        ctypes.byref(desc), _ptr(key), _ptr(value), _ptr(params.slot_mapping), key.size(0),
        key.stride(0), value.stride(0) if value is not None else 0, _dtype_code(key), _stream()))


# ---------------------------------------------------------------------------------------
# cache allocation
# ---------------------------------------------------------------------------------------

KV_SKEW_BYTES = 4096
_PAGE_BYTES = 2 << 20


def allocate_kv_cache(shape, dtype, device, with_scales=False, skew_bytes=KV_SKEW_BYTES):
    """K and V pools of one layer (plus fp32 scale tensors of the shape minus its last dimension when
    with_scales) — the allocation xllm/core/runtime/worker_impl.cpp:229-313 makes with one torch::zeros
    per tensor.  K and V are carved from one buffer with V starting skew_bytes past a 2 MiB boundary
    behind K: a decode work item reads block b of K and of V together, and in two separate
    allocations (addresses a multiple of 2 MiB apart) those reads meet in the same DRAM channel
    (Llama-3-8B decode, batch 64 x 4096 tokens: 162.4 us per step with separate pools, 158.8 us skewed).
    Returns (k_cache, v_cache, k_scale, v_scale); the scales are None without with_scales."""
    _require(len(shape) == 4, "cache shape must have four dimensions")
    _require(skew_bytes % 16 == 0 and skew_bytes >= 0, "skew_bytes must be a non-negative multiple of 16")

    def pair(shp, dt):
        nbytes = int(torch.Size(shp).numel()) * torch.empty(0, dtype=dt).element_size()
        v_at = (nbytes + _PAGE_BYTES - 1) // _PAGE_BYTES * _PAGE_BYTES + skew_bytes
        buf = torch.zeros(v_at + nbytes, dtype=torch.uint8, device=device)
        return buf[:nbytes].view(dt).view(shp), buf[v_at:v_at + nbytes].view(dt).view(shp)

    k, v = pair(tuple(shape), dtype)
    if not with_scales:
        return k, v, None, None
    ks, vs = pair(tuple(shape[:-1]), torch.float32)
    return k, v, ks, vs


# ---------------------------------------------------------------------------------------
# decode
# ---------------------------------------------------------------------------------------

_workspaces = {}
WORKSPACE_BYTES = 128 << 20


def decode_workspace_bytes(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim):
    return _lib.load().xllm_hip_paged_decode_workspace_bytes(batch, q_per_seq, num_q_heads, num_kv_heads, head_dim)


def get_workspace(device, nbytes):
    """Process-wide scratch per (device, stream) of WORKSPACE_BYTES bytes — the role of the reference's
    FlashinferWorkspace singleton (xllm/core/layers/cuda/flashinfer_workspace.cpp:24-38; 128 MiB is the
    default of its FLAGS_flashinfer_workspace_buffer_size).  Allocated when a stream first decodes and
    never reallocated, so that a captured graph's workspace address stays valid; a step that needs more
    raises.  Callers with other needs pass their own `workspace=` tensor instead."""
    _require(nbytes <= WORKSPACE_BYTES, "this decode step needs %d bytes of workspace, the shared buffer holds %d: "
             "pass workspace= or raise ops.WORKSPACE_BYTES before the first call on a stream" % (nbytes, WORKSPACE_BYTES))
    key = (torch.device(device), torch.cuda.current_stream(device).cuda_stream)
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def _decode_args(query, output, output_lse, block_table, seq_lens, csr, q_per_seq, scale, window_size_left,
                 max_seq_len, desc, total_kv_len=0, q_indptr=None):
    _require(query.dim() in (3, 4), "query must be [tokens, heads, dim] or [batch, q_len, heads, dim]")
    if query.dim() == 4:
        # [batch, q_len, Hq, D] (xllm/core/layers/mlu/attention.cpp:263-264)
        if q_per_seq is None:
            q_per_seq = query.size(1)
        _require(query.stride(0) == query.size(1) * query.stride(1), "4-D query must be dense over (batch, q_len)")
        q3 = query.reshape(-1, query.size(2), query.size(3))
        o3 = output.reshape(-1, output.size(-2), output.size(-1))
        _require(o3.data_ptr() == output.data_ptr(), "output must be viewable as [tokens, heads, dim]")
    else:
        q3, o3 = query, output
    q_per_seq = 1 if q_per_seq is None else int(q_per_seq)
    _require(o3.dim() == 3 and o3.shape == q3.shape and o3.dtype == q3.dtype, "output must match query")
    _require(q3.stride(2) == 1 and q3.stride(1) == q3.size(2), "query heads/head_dim must be contiguous")
    _require(o3.stride(2) == 1 and o3.stride(1) == o3.size(2), "output heads/head_dim must be contiguous")
    _require(q3.size(2) == desc.head_dim, "query head_dim %d != cache head_dim %d" % (q3.size(2), desc.head_dim))
    if q_indptr is None:
        _require(q3.size(0) % q_per_seq == 0, "query tokens not divisible by q_per_seq")
        batch = q3.size(0) // q_per_seq
    else:
        _require(q_indptr.dtype == torch.int32 and q_indptr.is_contiguous() and q_indptr.numel() >= 1,
                 "q_indptr must be contiguous int32 [batch + 1]")
        batch = q_indptr.numel() - 1

    a = _lib.DecodeArgs()
    a.q, a.out = q3.data_ptr(), o3.data_ptr()
    a.q_token_stride, a.out_token_stride = q3.stride(0), o3.stride(0)
    a.q_dtype = _dtype_code(q3)
    a.batch = batch
    a.q_indptr = q_indptr.data_ptr() if q_indptr is not None else None
    a.q_per_seq = q_per_seq
    a.num_q_heads = q3.size(1)
    a.sm_scale = float(scale)
    a.window_left = int(window_size_left) if window_size_left is not None else -1
    if output_lse is not None:
        _require(output_lse.dtype == torch.float32 and output_lse.is_contiguous()
                 and output_lse.numel() == q3.size(0) * q3.size(1), "output_lse must be float32 [tokens, heads]")
        a.lse = output_lse.data_ptr()
    if csr is None:
        _require(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
                 "block_table must be int32 [batch, max_blocks]")
        _require(seq_lens.dtype == torch.int32 and seq_lens.is_contiguous(), "seq_lens must be contiguous int32")
        _require(block_table.size(0) == a.batch and seq_lens.numel() == a.batch,
                 "block_table/seq_lens rows (%d/%d) != batch %d" % (block_table.size(0), seq_lens.numel(), a.batch))
        a.block_table = block_table.data_ptr()
        # (the row stride of a one-row table is arbitrary in torch: such a table is its one row)
        a.block_table_stride = block_table.stride(0) if block_table.size(0) > 1 else block_table.size(1)
        a.max_blocks_per_seq = block_table.size(1)
        a.seq_lens = seq_lens.data_ptr()
    else:
        indptr, indices, last_page_len = csr
        for t in (indptr, indices, last_page_len):
            _require(t.dtype == torch.int32 and t.is_contiguous(), "CSR arrays must be contiguous int32")
        _require(indptr.numel() == a.batch + 1 and last_page_len.numel() == a.batch, "CSR arrays do not match batch")
        a.kv_indptr, a.kv_indices, a.kv_last_page_len = indptr.data_ptr(), indices.data_ptr(), last_page_len.data_ptr()
    a.max_seq_len = int(max_seq_len) if max_seq_len is not None else 0
    a.total_kv_len = int(total_kv_len) if total_kv_len is not None else 0
    return a, (q3, o3)


# Pinned host buffers of the schedules made on the host, two per (device, stream) used in turn; each with the
# event recorded behind its last copy to the device, which is waited for before the buffer is written again.
_staging = {}


def _plan_host(lib, desc, args, host_kv_lens, wptr, wbytes, device):
    lens = torch.as_tensor(host_kv_lens, dtype=torch.int32, device="cpu").contiguous()
    _require(lens.numel() == args.batch, "host_kv_lens has %d entries, batch is %d" % (lens.numel(), args.batch))
    need = lib.xllm_hip_paged_decode_plan_host_bytes(args.batch, args.q_per_seq, args.num_q_heads, desc.num_kv_heads,
                                                     desc.head_dim)
    key = (device.index if device.index is not None else torch.cuda.current_device(), torch.cuda.current_stream(device).cuda_stream)
    slot = _staging.setdefault(key, {"turn": 0, "buffers": [None, None], "events": [None, None]})
    i = slot["turn"]
    slot["turn"] = 1 - i
    if slot["buffers"][i] is None or slot["buffers"][i].numel() < need:
        slot["buffers"][i] = torch.empty(max(need, 1 << 16), dtype=torch.uint8, pin_memory=True)
        slot["events"][i] = torch.cuda.Event()
    else:
        slot["events"][i].synchronize()
    buf = slot["buffers"][i]
    info = (ctypes.c_int64 * 3)()
    _lib.check(lib.xllm_hip_paged_decode_plan_host(ctypes.byref(desc), ctypes.byref(args), ctypes.c_void_p(lens.data_ptr()),
                                                   wptr, wbytes, ctypes.c_void_p(buf.data_ptr()), buf.numel(), _stream(),
                                                   info))
    slot["events"][i].record(torch.cuda.current_stream(device))
    return {"chunk_tokens": int(info[0]), "sequence_chunks": int(info[1]), "predicted_span_tokens": int(info[2])}


def _run_decode(desc, args, workspace, device, plan=True, run=True, events=None, host_kv_lens=None):
    lib = _lib.load()
    need = lib.xllm_hip_paged_decode_workspace_bytes(args.batch, args.q_per_seq, args.num_q_heads,
                                                     desc.num_kv_heads, desc.head_dim)
    ws = workspace if workspace is not None else get_workspace(device, need)
    wptr, wbytes = ctypes.c_void_p(ws.data_ptr()), ws.numel() * ws.element_size()
    if host_kv_lens is not None and plan:
        # the schedule from the host-side lengths; what follows only runs on it
        info = _plan_host(lib, desc, args, host_kv_lens, wptr, wbytes, device)
        plan = False
        if not run:
            return info
    if events is not None:
        # (ev_begin, ev_end): raw hipEvent_t handles recorded around the attention kernel
        if plan:
            _lib.check(lib.xllm_hip_paged_decode_plan(ctypes.byref(desc), ctypes.byref(args), wptr, wbytes, _stream()))
        _lib.check(lib.xllm_hip_paged_decode_run_timed(ctypes.byref(desc), ctypes.byref(args), wptr, wbytes,
                                                       _stream(), ctypes.c_void_p(events[0]),
                                                       ctypes.c_void_p(events[1])))
    elif plan and run:
        _lib.check(lib.xllm_hip_paged_decode(ctypes.byref(desc), ctypes.byref(args), wptr, wbytes, _stream()))
    elif plan:
        _lib.check(lib.xllm_hip_paged_decode_plan(ctypes.byref(desc), ctypes.byref(args), wptr, wbytes, _stream()))
    else:
        _lib.check(lib.xllm_hip_paged_decode_run(ctypes.byref(desc), ctypes.byref(args), wptr, wbytes, _stream()))


def batch_decode(query, k_cache, output, block_table, seq_lens, v_cache=None, output_lse=None,
                 q_quant_scale=None, k_cache_quant_scale=None, v_cache_quant_scale=None, out_quant_scale=None,
                 alibi_slope=None, mask=None, compute_dtype="float", max_seq_len=0, window_size_left=-1,
                 window_size_right=-1, scale=1.0, return_lse=False, kv_cache_quant_bit_size=-1, *,
                 q_per_seq=None, kv_layout="HND", workspace=None, plan=True, run=True, events=None,
                 total_kv_len=0, q_indptr=None, host_plan=False, host_kv_lens=None):
    """Paged decode in the block_table form; positional arguments as in
    xllm::kernel::mlu::batch_decode (xllm/core/kernels/mlu/mlu_ops_api.h:126-145).

    query/output: [batch, q_len, Hq, D] or [batch*q_len, Hq, D]; q_len > 1 is speculative verify
    with a causal mask among the draft tokens.  Keyword-only extras: q_per_seq (for 3-D queries),
    kv_layout, workspace (caller-owned scratch), plan/run (build the schedule once per step with
    run=False, then reuse it for every layer with plan=False), events (two raw hipEvent_t handles
    recorded just before and just after the attention kernel, for benchmarks), total_kv_len (the
    host-side sum of the kv lengths, AttentionMetadata.total_kv_len in the reference; together with
    max_seq_len it lets the library drop the merge launch when no sequence needs splitting),
    q_indptr (int32 [batch + 1]: sequences with different numbers of query tokens, the q_cu_seq_lens of
    a chunked-prefill or mixed step; q_per_seq is then the largest count, max_query_len),
    host_plan (xllm_hip_decode_args::host_plan: the kernel and its work items follow from sizes alone and the
    schedule always comes from the workspace, so that a captured run serves every step of these sizes) and
    host_kv_lens (the kv lengths as a host-side sequence of ints: the plan is then made on the host by
    xllm_hip_paged_decode_plan_host; implies host_plan).
    """
    _require(v_cache is not None, "v_cache is required (MLA-style single-cache decode is outside this path)")
    for name, t in (("q_quant_scale", q_quant_scale), ("out_quant_scale", out_quant_scale),
                    ("alibi_slope", alibi_slope), ("mask", mask)):
        if t is not None:
            raise _lib.XllmHipError(_lib.UNSUPPORTED, "%s is not supported by the HIP decode path" % name)
    _require(window_size_right is None or window_size_right < 0, "window_size_right must be -1 for decode")
    quant = k_cache_quant_scale is not None
    if kv_cache_quant_bit_size not in (-1, None):
        _require(kv_cache_quant_bit_size == 8 and quant, "kv_cache_quant_bit_size=8 needs k/v_cache_quant_scale")
    if quant:
        _require(v_cache_quant_scale is not None, "v_cache_quant_scale is required with k_cache_quant_scale")
    if return_lse:
        _require(output_lse is not None, "return_lse=True needs a pre-allocated output_lse")
    desc = _cache_desc(k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale, kv_layout)
    args, _keep = _decode_args(query, output, output_lse if return_lse or output_lse is not None else None,
                               block_table, seq_lens, None, q_per_seq, scale, window_size_left, max_seq_len, desc,
                               total_kv_len, q_indptr)
    args.host_plan = 1 if (host_plan or host_kv_lens is not None) else 0
    return _run_decode(desc, args, workspace, query.device, plan, run, events, host_kv_lens)


def batch_decode_csr(query, k_cache, v_cache, paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len,
                     window_left, sm_scale, output, output_lse=None, *, k_cache_scale=None, v_cache_scale=None,
                     q_per_seq=None, kv_layout="NHD", workspace=None, plan=True, run=True, max_seq_len=0,
                     total_kv_len=0, host_plan=False, host_kv_lens=None):
    """Paged decode in the CSR form of xllm::kernel::cuda::batch_decode
    (xllm/core/kernels/cuda/cuda_ops_api.h:120-136; the FlashInfer plan/workspace/uri
    arguments have no counterpart here).  The CUDA backend's cache layout is NHD."""
    desc = _cache_desc(k_cache, v_cache, k_cache_scale, v_cache_scale, kv_layout)
    args, _keep = _decode_args(query, output, output_lse, None, None,
                               (paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len), q_per_seq, sm_scale,
                               window_left, max_seq_len, desc, total_kv_len)
    args.host_plan = 1 if (host_plan or host_kv_lens is not None) else 0
    return _run_decode(desc, args, workspace, query.device, plan, run, None, host_kv_lens)


def decode_variant(query, k_cache, v_cache, block_table, seq_lens, k_cache_quant_scale=None,
                   v_cache_quant_scale=None, q_per_seq=None, kv_layout="HND"):
    """Name of the kernel variant batch_decode would run for these tensors."""
    desc = _cache_desc(k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale, kv_layout)
    out = torch.empty_like(query)
    args, _keep = _decode_args(query, out, None, block_table, seq_lens, None, q_per_seq, 1.0, -1, 0, desc)
    return _lib.load().xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)).decode()


DESCRIBE_FIELDS = ("workgroups", "waves_per_workgroup", "unsplit", "stored_schedule", "chunk_tokens",
                   "slots_per_cut_sequence", "kept_sequences", "kept_slots", "kept_chunk_tokens", "kv_heads_per_item",
                   "items_per_workgroup", "fused_merge", "chunk_slots_held", "chunk_slots_used")


def decode_describe(query, k_cache, v_cache, block_table, seq_lens, k_cache_quant_scale=None,
                    v_cache_quant_scale=None, q_per_seq=None, kv_layout="HND", max_seq_len=0, total_kv_len=0,
                    host_plan=False):
    """How batch_decode would run these tensors (xllm_hip_paged_decode_describe: decided on the host, nothing is
    launched): a dict of DESCRIBE_FIELDS."""
    desc = _cache_desc(k_cache, v_cache, k_cache_quant_scale, v_cache_quant_scale, kv_layout)
    out = torch.empty_like(query)
    args, _keep = _decode_args(query, out, None, block_table, seq_lens, None, q_per_seq, 1.0, -1, max_seq_len, desc,
                               total_kv_len=total_kv_len)
    args.host_plan = 1 if host_plan else 0
    vals = (ctypes.c_int64 * len(DESCRIBE_FIELDS))()
    _lib.check(_lib.load().xllm_hip_paged_decode_describe(ctypes.byref(desc), ctypes.byref(args), 0, vals,
                                                          len(DESCRIBE_FIELDS)))
    return dict(zip(DESCRIBE_FIELDS, (int(v) for v in vals)))


def csr_to_block_table(paged_kv_indptr, paged_kv_indices, paged_kv_last_page_len, block_size, max_blocks_per_seq):
    """Index-only conversion CSR -> (block_table padded with 0, seq_lens)."""
    batch = paged_kv_last_page_len.numel()
    dev = paged_kv_indptr.device
    table = torch.empty(batch, max_blocks_per_seq, dtype=torch.int32, device=dev)
    seq_lens = torch.empty(batch, dtype=torch.int32, device=dev)
    _lib.check(_lib.load().xllm_hip_csr_to_block_table(
        _ptr(paged_kv_indptr), _ptr(paged_kv_indices), _ptr(paged_kv_last_page_len), batch, block_size,
        _ptr(table), table.stride(0), max_blocks_per_seq, _ptr(seq_lens), _stream()))
    return table, seq_lens


def swap_blocks(k_cache, v_cache, src_tensor, dst_tensor, k_cache_scale=None, v_cache_scale=None, *,
                kv_layout="HND", exact=True):
    """KVCache::swap_blocks (xllm/core/framework/kv_cache/kv_cache.cpp:104-125): copy whole blocks
    src_tensor[i] -> dst_tensor[i] (int64 index tensors on the device) of K, V and the scale tensors.
    exact=True gathers every source before any destination is written, as index_select followed by
    index_copy_ does (a staging buffer is allocated for the call); exact=False copies in one pass and
    needs destinations that are not sources of the same call."""
    lib = _lib.load()
    _require(src_tensor.dtype == torch.int64 and dst_tensor.dtype == torch.int64, "block indices must be int64")
    _require(src_tensor.is_cuda and dst_tensor.is_cuda, "block indices must live on the GPU")
    _require(src_tensor.numel() == dst_tensor.numel(), "src and dst must name the same number of blocks")
    src, dst = src_tensor.contiguous(), dst_tensor.contiguous()
    desc = _cache_desc(k_cache, v_cache, k_cache_scale, v_cache_scale, kv_layout)
    n = src.numel()
    staging, nbytes = None, 0
    if exact and n > 0:
        nbytes = lib.xllm_hip_swap_blocks_staging_bytes(ctypes.byref(desc), n)
        staging = torch.empty(nbytes, dtype=torch.uint8, device=k_cache.device)
    _lib.check(lib.xllm_hip_swap_blocks(ctypes.byref(desc), _ptr(src), _ptr(dst), n,
                                        _ptr(staging) if staging is not None else None, nbytes, _stream()))


def copy_blocks(k_cache, v_cache, src_block_indices, dst_block_indices, cum_sum, k_cache_scale=None,
                v_cache_scale=None, *, kv_layout="HND"):
    """The block-copy step of a forward pass (xllm/models/llm/npu/llm_model_base.h:69-75) on the
    arrays the batch builder emits (xllm/core/framework/batch/batch_input_builder.cpp:691-720):
    source block src_block_indices[g] goes to destinations dst_block_indices[cum_sum[g-1]:cum_sum[g]]."""
    lib = _lib.load()
    for t in (src_block_indices, dst_block_indices, cum_sum):
        _require(t.dtype == torch.int32 and t.is_cuda, "block-copy index tensors must be int32 on the GPU")
    _require(src_block_indices.numel() == cum_sum.numel(), "one cum_sum entry per source block")
    desc = _cache_desc(k_cache, v_cache, k_cache_scale, v_cache_scale, kv_layout)
    _lib.check(lib.xllm_hip_copy_blocks(ctypes.byref(desc), _ptr(src_block_indices.contiguous()),
                                        _ptr(dst_block_indices.contiguous()), _ptr(cum_sum.contiguous()),
                                        src_block_indices.numel(), dst_block_indices.numel(), _stream()))


def _gather_from_cache(key, value, key_cache, value_cache, key_scale, value_scale, context_lengths, max_context_len,
                       context_seq_offset, block_tables, cache_seq_offset, quant_mode, kv_layout):
    lib = _lib.load()
    _require(key.is_cuda and key.dim() == 3 and key.stride(2) == 1 and key.stride(1) == key.size(2),
             "key must be a GPU tensor [rows, num_kv_heads, head_dim] with the last two dimensions contiguous")
    if value is not None:
        _require(value_cache is not None, "value given without value_cache")
        _require(value.dtype == key.dtype and value.shape[1:] == key.shape[1:] and value.stride(2) == 1 and
                 value.stride(1) == value.size(2), "value must match key in dtype and row shape")
    _require(block_tables is not None and block_tables.dim() == 2, "block_tables [batch, max_blocks] is required "
             "(the linear cache mode of the reference is not part of the paged path)")
    for t in (context_lengths, block_tables, context_seq_offset, cache_seq_offset):
        _require(t is None or (t.dtype == torch.int32 and t.is_cuda), "index tensors must be int32 on the GPU")
    _require(block_tables.stride(1) == 1, "block_tables rows must be contiguous")
    batch = context_lengths.numel()
    _require(block_tables.size(0) >= batch, "one block_tables row per sequence")
    per_channel = key_scale is not None and quant_mode == 0
    desc = _cache_desc(key_cache, value_cache if value is not None else None,
                       None if per_channel else key_scale, None if per_channel else value_scale, kv_layout)
    if per_channel:
        for sc in (key_scale, value_scale if value is not None else None):
            _require(sc is None or (sc.dtype == torch.float32 and sc.is_contiguous() and
                                    tuple(sc.shape) == (desc.num_kv_heads, desc.head_dim)),
                     "per-channel scales must be contiguous float32 [num_kv_heads, head_dim]")
        desc.k_scale = key_scale.data_ptr()
        desc.v_scale = value_scale.data_ptr() if value is not None and value_scale is not None else None
    _require(tuple(key.shape[1:]) == (desc.num_kv_heads, desc.head_dim), "key rows do not match the cache")
    cl = context_lengths.contiguous()
    cso = context_seq_offset.contiguous() if context_seq_offset is not None else None
    cao = cache_seq_offset.contiguous() if cache_seq_offset is not None else None
    _lib.check(lib.xllm_hip_gather_from_cache(
        ctypes.byref(desc), _ptr(key), _ptr(value) if value is not None else None, _dtype_code(key), key.stride(0),
        value.stride(0) if value is not None else 0, _ptr(cl), _ptr(cso) if cso is not None else None,
        _ptr(cao) if cao is not None else None, _ptr(block_tables), block_tables.stride(0), block_tables.size(1),
        batch, int(max_context_len), int(quant_mode), _stream()))


def reshape_from_cache(key, value, key_cache, value_cache, context_lengths, max_context_len, context_seq_offset=None,
                       block_tables=None, cache_seq_offset=None, *, kv_layout="HND"):
    """Paged mode of xllm::kernel::mlu::reshape_from_cache (xllm/core/kernels/mlu/mlu_ops_api.h:56-64;
    fields xllm/core/kernels/param.h:160-201): the cached tokens of every sequence copied verbatim
    into key/value [rows, num_kv_heads, head_dim] (same dtype as the cache), sequence b starting at
    row context_seq_offset[b] (default: packed in order)."""
    _require(key.dtype == key_cache.dtype, "reshape_from_cache copies verbatim: key and key_cache dtypes differ")
    _gather_from_cache(key, value, key_cache, value_cache, None, None, context_lengths, max_context_len,
                       context_seq_offset, block_tables, cache_seq_offset, 1, kv_layout)


def dequant_from_paged_cache(key, value, key_cache, value_cache, key_cache_quant_scale, value_cache_quant_scale,
                             context_lengths, max_context_len, context_seq_offset, block_tables, quant_mode=1,
                             quant_bit=8, *, kv_layout="HND"):
    """xllm::kernel::mlu::dequant_from_paged_cache (xllm/core/kernels/mlu/mlu_ops_api.h:79-101), the
    step before a chunked prefill over a quantised cache (xllm/core/layers/mlu/attention.cpp:196-214):
    key/value [rows, num_kv_heads, head_dim] in bf16/fp16/fp32 receive (float)q * scale.
    quant_mode 1: scales [num_blocks, num_kv_heads, block_size]; 0: [num_kv_heads, head_dim]."""
    _require(quant_bit == 8, "only 8-bit caches exist on this path")
    _require(key_cache.dtype in (torch.int8, torch.float8_e4m3fn, torch.uint8), "key_cache is not quantised")
    _require(key_cache_quant_scale is not None, "key_cache_quant_scale is required for dequant_from_paged_cache")
    _require(value is None or value_cache_quant_scale is not None, "value needs value_cache_quant_scale")
    _gather_from_cache(key, value, key_cache, value_cache, key_cache_quant_scale, value_cache_quant_scale,
                       context_lengths, max_context_len, context_seq_offset, block_tables, None, quant_mode, kv_layout)


def _rope_call(qkv, num_q, num_k, num_v, head_dim, eps, q_weight, k_weight, cos_sin_cache, interleaved, positions,
               round_each_op, cache_desc=None, slot_mapping=None):
    lib = _lib.load()
    _require(qkv.is_cuda and qkv.dim() == 2 and qkv.stride(1) == 1, "qkv must be a 2-D GPU tensor, rows contiguous")
    _require(positions.dtype in (torch.int64, torch.int32) and positions.dim() == 1 and positions.is_contiguous(),
             "position_ids must be a contiguous 1-D int64 or int32 tensor")
    _require(positions.numel() == qkv.size(0), "one position per token")
    _require(cos_sin_cache.dim() == 2 and cos_sin_cache.is_contiguous(), "cos_sin_cache must be [max_position, rotary_dim]")
    a = _lib.RopeArgs()
    a.qkv, a.token_stride, a.num_tokens = qkv.data_ptr(), qkv.stride(0), qkv.size(0)
    a.dtype = _dtype_code(qkv)
    a.num_q_heads, a.num_k_heads, a.num_v_heads, a.head_dim = num_q, num_k, num_v, head_dim
    a.rotary_dim = cos_sin_cache.size(1)
    if q_weight is not None:
        for w in (q_weight, k_weight):
            _require(w.dtype == qkv.dtype and w.dim() == 1 and w.numel() == head_dim and w.is_contiguous(),
                     "norm weights must be [head_dim] of qkv's dtype")
        a.q_weight, a.k_weight = q_weight.data_ptr(), k_weight.data_ptr()
    a.eps = eps
    a.cos_sin_dtype, a.cos_sin_cache, a.max_position = _dtype_code(cos_sin_cache), cos_sin_cache.data_ptr(), \
        cos_sin_cache.size(0)
    a.positions = positions.data_ptr()
    a.positions_int32 = int(positions.dtype == torch.int32)
    a.interleave, a.round_each_op = int(bool(interleaved)), int(bool(round_each_op))
    _lib.check(lib.xllm_hip_rope_kv_write(ctypes.byref(a), ctypes.byref(cache_desc) if cache_desc is not None else None,
                                          _ptr(slot_mapping), _stream()))


def fused_qk_norm_rope(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight, cos_sin_cache,
                       interleaved, position_ids):
    """xllm::kernel::cuda::fused_qk_norm_rope (xllm/core/kernels/cuda/cuda_ops_api.h:227-241): per-head
    RMSNorm + rotary embedding of the q and k heads of the fused buffer, in place."""
    _rope_call(qkv, num_heads_q, num_heads_k, num_heads_v, head_dim, eps, q_weight, k_weight, cos_sin_cache,
               interleaved, position_ids, False)


def rotary_embedding(positions, query, key, cos_sin_cache, is_neox):
    """xllm::kernel::cuda::rotary_embedding (xllm/core/kernels/cuda/rope.cu:152-249): rotation of query
    [tokens, heads * head_size] and, if given, key, in place, every operation rounded to the element
    type.  head_size is the last dimension of cos_sin_cache... as in the reference (rope.cu:169)."""
    head_size = cos_sin_cache.size(-1)
    for t in (query, key):
        if t is None:
            continue
        flat = t.view(t.size(0), -1) if t.dim() == 3 else t
        _require(flat.size(1) % head_size == 0, "hidden size is not a multiple of head_size")
        heads = flat.size(1) // head_size
        _rope_call(flat, heads, 0, 0, head_size, 0.0, None, None, cos_sin_cache, not is_neox, positions, True)


def rope_kv_write(qkv, num_heads_q, num_heads_kv, head_dim, cos_sin_cache, position_ids, k_cache, v_cache,
                  slot_mapping, *, q_weight=None, k_weight=None, eps=1e-6, interleaved=False, round_each_op=False,
                  k_cache_scale=None, v_cache_scale=None, kv_layout="HND"):
    """Norm (optional) + rotary embedding of q and k in place, then the KV write of the rotated k and of
    v through slot_mapping (quantising iff scales are given) — one launch for the steps 2-5 of
    Qwen2AttentionImpl::forward up to the attention call (xllm/core/layers/common/qwen2_attention.cpp:147-189)."""
    desc = _cache_desc(k_cache, v_cache, k_cache_scale, v_cache_scale, kv_layout)
    _require(slot_mapping.dtype == torch.int32 and slot_mapping.is_contiguous() and
             slot_mapping.numel() == qkv.size(0), "slot_mapping must be contiguous int32, one entry per token")
    _rope_call(qkv, num_heads_q, num_heads_kv, num_heads_kv, head_dim, eps, q_weight, k_weight, cos_sin_cache,
               interleaved, position_ids, round_each_op, desc, slot_mapping)
