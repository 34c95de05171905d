"""The C-ABI library loads and exports every symbol include/xllm_hip_paged_kv.h declares, and its
host-side argument checks answer without launching anything (runs without a GPU)."""
import ctypes
import os
import re

import pytest

from xllm_wxh_amd import _lib
from xllm_wxh_amd import build as xbuild

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(REPO, "include", "xllm_hip_paged_kv.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        xbuild.build_library(verbose=False)
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(xllm_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    assert set(names) == set(_lib.EXPORTED_SYMBOLS)


def test_every_declared_symbol_is_exported(lib):
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_abi_version(lib):
    assert lib.xllm_hip_abi_version() == _lib.ABI_VERSION
    text = open(HEADER).read()
    assert int(re.search(r"#define XLLM_HIP_ABI_VERSION (\d+)", text).group(1)) == _lib.ABI_VERSION


def test_struct_sizes_match_the_header_layout():
    # 4 pointers + i64 + 4 i32 + 6 i64 ; natural alignment, no padding surprises
    assert ctypes.sizeof(_lib.KvCacheDesc) == 4 * 8 + 8 + 4 * 4 + 6 * 8
    assert _lib.KvCacheDesc.stride_block.offset == 56
    assert _lib.DecodeArgs.q_dtype.offset == 40
    assert _lib.DecodeArgs.block_table.offset == 64
    assert _lib.DecodeArgs.max_seq_len.offset == 120
    assert _lib.DecodeArgs.q_indptr.offset == 136
    assert _lib.DecodeArgs.host_plan.offset == 144
    assert ctypes.sizeof(_lib.DecodeArgs) == 152  # (+ 4 bytes of padding)
    # xllm_hip_rope_args: ptr, 2 i64, 6 i32, 2 ptr, f32 + i32, ptr, i64, ptr, 3 i32 (+ 4 bytes of padding)
    assert _lib.RopeArgs.q_weight.offset == 48 and _lib.RopeArgs.cos_sin_cache.offset == 72
    assert _lib.RopeArgs.positions_int32.offset == 104
    assert ctypes.sizeof(_lib.RopeArgs) == 112


def test_workspace_bytes_is_a_pure_size_function(lib):
    a = lib.xllm_hip_paged_decode_workspace_bytes(64, 1, 32, 8, 128)
    b = lib.xllm_hip_paged_decode_workspace_bytes(128, 1, 32, 8, 128)
    assert 0 < a < b
    assert a % 256 == 0
    assert lib.xllm_hip_paged_decode_workspace_bytes(64, 0, 32, 8, 128) == 0
    # partial outputs dominate: (640/Hkv + B + 1) sequence chunks x n x Hq x D fp32 (four rows per kv head:
    # the 16-row kernel's 512 work items and a quarter more)
    assert a >= (640 // 8 + 64 + 1) * 32 * 128 * 4


def test_argument_errors_are_reported_not_launched(lib):
    desc = _lib.KvCacheDesc()
    rc = lib.xllm_hip_reshape_paged_cache(ctypes.byref(desc), None, None, None, 4, 0, 0, _lib.BF16, None)
    assert rc == _lib.INVALID_ARGUMENT
    assert b"k_cache is NULL" in lib.xllm_hip_last_error()
    desc.k_cache = 0x1000
    desc.num_blocks, desc.block_size, desc.num_kv_heads, desc.head_dim = 4, 16, 2, 64
    desc.dtype = _lib.INT8
    desc.stride_block, desc.stride_head, desc.stride_slot = 2048, 1024, 64
    rc = lib.xllm_hip_reshape_paged_cache(ctypes.byref(desc), 0x2000, None, 0x3000, 4, 128, 0, _lib.BF16, None)
    assert rc == _lib.INVALID_ARGUMENT and b"copies verbatim" in lib.xllm_hip_last_error()
    rc = lib.xllm_hip_quant_to_paged_cache(ctypes.byref(desc), 0x2000, None, 0x3000, 4, 128, 0, _lib.BF16, None)
    assert rc == _lib.INVALID_ARGUMENT and b"k_cache_scale is required" in lib.xllm_hip_last_error()
    # zero tokens is a no-op, not an error
    desc.dtype = _lib.BF16
    assert lib.xllm_hip_reshape_paged_cache(ctypes.byref(desc), None, None, None, 0, 0, 0, _lib.BF16, None) == _lib.OK

    args = _lib.DecodeArgs()
    args.batch, args.q_per_seq, args.num_q_heads, args.q_dtype = 2, 1, 3, _lib.BF16
    desc.v_cache = 0x4000
    rc = lib.xllm_hip_paged_decode(ctypes.byref(desc), ctypes.byref(args), None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and b"not a multiple" in lib.xllm_hip_last_error()
    args.num_q_heads = 4
    args.q, args.out = 0x5000, 0x6000
    args.q_token_stride = args.out_token_stride = 4 * 64
    args.block_table, args.seq_lens, args.block_table_stride, args.max_blocks_per_seq = 0x7000, 0x8000, 4, 4
    rc = lib.xllm_hip_paged_decode(ctypes.byref(desc), ctypes.byref(args), None, 0, None)
    assert rc == _lib.WORKSPACE_TOO_SMALL
    with pytest.raises(_lib.XllmHipError):
        _lib.check(rc)


def test_variant_selection_is_host_only(lib):
    desc = _lib.KvCacheDesc()
    desc.k_cache, desc.v_cache = 0x10000, 0x20000
    desc.num_blocks, desc.block_size, desc.num_kv_heads, desc.head_dim = 4, 16, 8, 128
    desc.dtype = _lib.BF16
    desc.stride_block, desc.stride_head, desc.stride_slot = 8 * 16 * 128, 16 * 128, 128
    args = _lib.DecodeArgs()
    args.q = 0x30000
    args.batch, args.q_per_seq, args.num_q_heads, args.q_dtype = 2, 1, 32, _lib.BF16
    args.q_token_stride = 32 * 128
    assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b"mfma_d128"
    desc.head_dim = 64
    assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b"generic"
    # head_dim 64 with contiguous tokens and blocks of at least 32 tokens has an MFMA path of its own
    desc.block_size, desc.stride_block, desc.stride_head, desc.stride_slot = 32, 8 * 32 * 64, 32 * 64, 64
    assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b"mfma_d64"
    desc.block_size, desc.stride_block, desc.stride_head, desc.stride_slot = 16, 8 * 16 * 128, 16 * 128, 128
    desc.head_dim, desc.dtype = 128, _lib.FP32
    assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b"generic"
    desc.head_dim = 512
    assert lib.xllm_hip_paged_decode_variant(ctypes.byref(desc), ctypes.byref(args)) == b""


def _header_struct_fields(name):
    """Field names of `typedef struct <name> { ... } <name>;` in declaration order."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), text, flags=re.S).group(1)
    return [re.search(r"([A-Za-z0-9_]+)\s*$", d.strip()).group(1) for d in body.split(";") if d.strip()]


def test_header_is_plain_c_and_its_layouts_are_those_of_the_ctypes_binding(tmp_path):
    """The boundary is a C ABI: the header compiles as C99 without a HIP toolchain in sight, and
    every field of its three structs sits where the ctypes binding (what the tests, bench.py and
    any Python caller go through) puts it — offsets taken from the C compiler, not retyped."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    structs = {"xllm_hip_kv_cache": _lib.KvCacheDesc, "xllm_hip_decode_args": _lib.DecodeArgs,
               "xllm_hip_rope_args": _lib.RopeArgs}
    lines = ['#include <stddef.h>', '#include <stdio.h>', '#include "xllm_hip_paged_kv.h"', "int main(void) {"]
    for cname in structs:
        lines.append('  printf("%s . %%zu\\n", sizeof(%s));' % (cname, cname))
        for f in _header_struct_fields(cname):
            lines.append('  printf("%s %s %%zu\\n", offsetof(%s, %s));' % (cname, f, cname, f))
    lines += ["  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines) + "\n")
    exe = tmp_path / "layout"
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.dirname(HEADER),
                    str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    seen = {}
    for line in out.splitlines():
        cname, field, value = line.split()
        seen.setdefault(cname, {})[field] = int(value)
    for cname, cls in structs.items():
        assert seen[cname].pop(".") == ctypes.sizeof(cls), cname
        assert list(seen[cname]) == [f[0] for f in cls._fields_], cname  # same fields, same order
        for field, offset in seen[cname].items():
            assert getattr(cls, field).offset == offset, (cname, field)
