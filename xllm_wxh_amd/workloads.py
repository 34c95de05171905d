"""Synthetic decode workloads: the five configurations the path is measured and checked on.

Each workload fixes shapes, dtypes, the kv-length distribution and the block-table
construction; tensors are generated from seeds (numpy for index data, torch for
values) so that the CPU checker and the GPU path see identical inputs.
"""
import math
from dataclasses import dataclass, field

import numpy as np


@dataclass(frozen=True)
class DecodeWorkload:
    name: str
    batch: int
    num_q_heads: int
    num_kv_heads: int
    head_dim: int
    block_size: int
    q_per_seq: int = 1
    q_dtype: str = "bf16"       # bf16 | fp32
    kv_dtype: str = "bf16"      # bf16 | fp32 | fp8 | int8
    seq_len_kind: str = "fixed"  # fixed | uniform | lognormal
    seq_len: int = 0             # fixed length / uniform upper bound / lognormal median
    seq_len_sigma: float = 0.0
    seq_len_min: int = 1
    seq_len_max: int = 0
    value_std: float = 1.0       # K and V values ~ N(0, 1) * value_std
    q_std: float = 1.0           # queries ~ N(0, 1) * q_std
    pool_blocks: int = 0         # 0: exactly the blocks the sequences need
    description: str = ""

    @property
    def group(self):
        return self.num_q_heads // self.num_kv_heads

    @property
    def sm_scale(self):
        return 1.0 / math.sqrt(self.head_dim)

    @property
    def kv_elem_bytes(self):
        return {"bf16": 2, "fp32": 4, "fp8": 1, "int8": 1}[self.kv_dtype]

    @property
    def q_elem_bytes(self):
        return {"bf16": 2, "fp32": 4}[self.q_dtype]


WORKLOADS = {
    "cfg1_cpu_fp32": DecodeWorkload(
        name="cfg1_cpu_fp32", batch=4, num_q_heads=14, num_kv_heads=2, head_dim=64, block_size=16,
        q_dtype="fp32", kv_dtype="fp32", seq_len_kind="uniform", seq_len=512, pool_blocks=256,
        description="fp32, 14q/2kv, D=64, bs=16, B=4, L~U{1..512}, 256-block pool, +4-token KV write"),
    "cfg2_llama3_8b_b64_ctx4k": DecodeWorkload(
        name="cfg2_llama3_8b_b64_ctx4k", batch=64, num_q_heads=32, num_kv_heads=8, head_dim=128, block_size=16,
        seq_len_kind="fixed", seq_len=4096, value_std=0.5, q_std=0.5,
        description="Llama-3-8B decode: bf16, 32q/8kv, D=128, bs=16, B=64, L=4096, q/k/v ~ N(0,1)*0.5"),
    "cfg3_ragged_b256": DecodeWorkload(
        name="cfg3_ragged_b256", batch=256, num_q_heads=32, num_kv_heads=8, head_dim=128, block_size=128,
        seq_len_kind="lognormal", seq_len=2048, seq_len_sigma=0.8, seq_len_min=16, seq_len_max=32768,
        description="ragged continuous batching: bf16, 32q/8kv, D=128, bs=128, B=256, L~lognormal(ln 2048, 0.8) in [16, 32768]"),
    "cfg4_fp8_qwen3_32b": DecodeWorkload(
        name="cfg4_fp8_qwen3_32b", batch=128, num_q_heads=64, num_kv_heads=8, head_dim=128, block_size=16,
        kv_dtype="fp8", seq_len_kind="fixed", seq_len=8192,
        description="fp8-e4m3 KV, Qwen3-32B shape: 64q/8kv, D=128, bs=16, B=128, L=8192, per-token-head fp32 scales"),
    "cfg5_int8_spec_verify": DecodeWorkload(
        name="cfg5_int8_spec_verify", batch=32, num_q_heads=64, num_kv_heads=8, head_dim=128, block_size=128,
        q_per_seq=4, kv_dtype="int8", seq_len_kind="fixed", seq_len=32768,
        description="int8 KV speculative verify: 64q/8kv, D=128, bs=128, B=32, L=32768, 4 causal draft tokens"),
    # Shapes beside the five configurations above, measured the same way (head_dim 256 as in Gemma-2 /
    # Qwen3-Next attention layers).
    "aux_d256_bf16_b64_ctx4k": DecodeWorkload(
        name="aux_d256_bf16_b64_ctx4k", batch=64, num_q_heads=16, num_kv_heads=8, head_dim=256, block_size=16,
        seq_len_kind="fixed", seq_len=4096, value_std=0.5,
        description="head_dim 256 decode: bf16, 16q/8kv, D=256, bs=16, B=64, L=4096"),
    "aux_d256_fp8_b64_ctx8k": DecodeWorkload(
        name="aux_d256_fp8_b64_ctx8k", batch=64, num_q_heads=32, num_kv_heads=8, head_dim=256, block_size=16,
        kv_dtype="fp8", seq_len_kind="fixed", seq_len=8192,
        description="head_dim 256 decode over an fp8-e4m3 cache: 32q/8kv, D=256, bs=16, B=64, L=8192"),
    "aux_d256_int8_spec_verify": DecodeWorkload(
        name="aux_d256_int8_spec_verify", batch=32, num_q_heads=64, num_kv_heads=8, head_dim=256, block_size=128,
        q_per_seq=4, kv_dtype="int8", seq_len_kind="fixed", seq_len=16384,
        description="head_dim 256 speculative verify over an int8 cache: 64q/8kv, D=256, bs=128, B=32, L=16384, 4 draft tokens"),
    # head_dim 64 (the head size of the reference's own CPU-sized test shape, Qwen2-0.5B: 14q/2kv) at a
    # size that fills the GPU.
    "aux_d64_bf16_b512_ctx4k": DecodeWorkload(
        name="aux_d64_bf16_b512_ctx4k", batch=512, num_q_heads=14, num_kv_heads=2, head_dim=64, block_size=32,
        seq_len_kind="fixed", seq_len=4096, value_std=0.5,
        description="head_dim 64 decode: bf16, 14q/2kv, D=64, bs=32, B=512, L=4096"),
    "aux_d64_int8_b512_ctx8k": DecodeWorkload(
        name="aux_d64_int8_b512_ctx8k", batch=512, num_q_heads=14, num_kv_heads=2, head_dim=64, block_size=32,
        kv_dtype="int8", seq_len_kind="fixed", seq_len=8192,
        description="head_dim 64 decode over an int8 cache: 14q/2kv, D=64, bs=32, B=512, L=8192"),
    # Small batches: the split-KV schedule (plan, attention over chunks, merge) is what is measured.
    "aux_b1_ctx32k": DecodeWorkload(
        name="aux_b1_ctx32k", batch=1, num_q_heads=32, num_kv_heads=8, head_dim=128, block_size=16,
        seq_len_kind="fixed", seq_len=32768, value_std=0.5,
        description="one sequence: bf16, 32q/8kv, D=128, bs=16, B=1, L=32768"),
    "aux_b8_ctx8k": DecodeWorkload(
        name="aux_b8_ctx8k", batch=8, num_q_heads=32, num_kv_heads=8, head_dim=128, block_size=16,
        seq_len_kind="fixed", seq_len=8192, value_std=0.5,
        description="small batch: bf16, 32q/8kv, D=128, bs=16, B=8, L=8192"),
}


def scaled(workload, batch=None, seq_len=None, seq_len_max=None, name=None):
    """A smaller instance of the same workload (same shapes and dtypes), for CPU-checkable tests."""
    import dataclasses

    kw = {}
    if batch is not None:
        kw["batch"] = batch
    if seq_len is not None:
        kw["seq_len"] = seq_len
    if seq_len_max is not None:
        kw["seq_len_max"] = seq_len_max
    kw["name"] = name or (workload.name + "_small")
    return dataclasses.replace(workload, **kw)


def make_seq_lens(w, seed=0):
    rng = np.random.default_rng(seed)
    if w.seq_len_kind == "fixed":
        lens = np.full(w.batch, w.seq_len, np.int64)
    elif w.seq_len_kind == "uniform":
        lens = rng.integers(1, w.seq_len + 1, size=w.batch)
    elif w.seq_len_kind == "lognormal":
        lens = np.rint(rng.lognormal(math.log(w.seq_len), w.seq_len_sigma, size=w.batch))
        lens = np.clip(lens, w.seq_len_min, w.seq_len_max)
    else:
        raise ValueError(w.seq_len_kind)
    return lens.astype(np.int32)


def make_block_tables(w, seq_lens, seed=0):
    """Disjoint block lists drawn from a seeded shuffle of the pool.
    Returns (block_table [B, max_blocks] int32 padded with 0, num_blocks, block_lists)."""
    rng = np.random.default_rng(seed + 1)
    need = (np.asarray(seq_lens, np.int64) + w.block_size - 1) // w.block_size
    total = int(need.sum())
    num_blocks = max(w.pool_blocks, total)
    perm = rng.permutation(num_blocks).astype(np.int32)
    table = np.zeros((w.batch, int(need.max())), np.int32)
    lists, o = [], 0
    for b in range(w.batch):
        ids = perm[o:o + need[b]]
        o += int(need[b])
        table[b, : need[b]] = ids
        lists.append(ids)
    return table, num_blocks, lists


def decode_slots(w, seq_lens, block_lists):
    """slot_mapping of the step's new tokens: the last q_per_seq positions of every sequence."""
    slots = []
    for b in range(w.batch):
        L = int(seq_lens[b])
        for pos in range(L - w.q_per_seq, L):
            slots.append(int(block_lists[b][pos // w.block_size]) * w.block_size + pos % w.block_size)
    return np.asarray(slots, np.int32)


def algorithmic_bytes(w, seq_lens):
    """Bytes one decode call must move: K and V of the valid tokens once per sequence, the scales of a
    quantised cache, q in and out once, the block table entries and the lengths."""
    total = int(np.asarray(seq_lens, np.int64).sum())
    kv = total * w.num_kv_heads * w.head_dim * 2 * w.kv_elem_bytes
    scales = total * w.num_kv_heads * 2 * 4 if w.kv_dtype in ("fp8", "int8") else 0
    qo = 2 * w.batch * w.q_per_seq * w.num_q_heads * w.head_dim * w.q_elem_bytes
    blocks = int(((np.asarray(seq_lens, np.int64) + w.block_size - 1) // w.block_size).sum())
    return kv + scales + qo + 4 * blocks + 4 * w.batch


def kv_write_bytes(w):
    """Bytes of the step's KV write: source read + cache write (+ scales)."""
    t = w.batch * w.q_per_seq
    src = 2 if w.kv_dtype != "fp32" else 4
    b = t * w.num_kv_heads * w.head_dim * (2 * src + 2 * w.kv_elem_bytes)
    if w.kv_dtype in ("fp8", "int8"):
        b += t * w.num_kv_heads * 2 * 4
    return b
