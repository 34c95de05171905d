"""ctypes binding of the C ABI declared in include/xllm_hip_paged_kv.h.

The library is loaded from this directory only.  There is no fallback: if the
shared object is missing or a symbol cannot be resolved, importing the ops
raises, so a GPU run can never silently take another path.
"""
import ctypes
import os

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libxllm_hip_paged_kv.so")

ABI_VERSION = 4
STATIC_WORKSPACE_BYTES = 48 << 20

# xllm_hip_dtype
BF16, FP16, FP32, FP8_E4M3, INT8 = 0, 1, 2, 3, 4
# xllm_hip_status
OK, INVALID_ARGUMENT, UNSUPPORTED, WORKSPACE_TOO_SMALL, RUNTIME_ERROR = 0, 1, 2, 3, 4

# xllm_hip_option
OPTION_DECODE_FORCE_GENERIC, OPTION_DECODE_TARGET_ITEMS, OPTION_DECODE_SEPARATE_MERGE = 0, 1, 2
OPTION_DECODE_STORED_SCHEDULE = 3
OPTION_DECODE_ITEM_PER_HEAD = 4
OPTION_DECODE_FOUR_WAVE_ITEMS = 5
OPTION_PREFILL_KERNEL = 6

STATUS_NAMES = {
    OK: "OK",
    INVALID_ARGUMENT: "INVALID_ARGUMENT",
    UNSUPPORTED: "UNSUPPORTED",
    WORKSPACE_TOO_SMALL: "WORKSPACE_TOO_SMALL",
    RUNTIME_ERROR: "RUNTIME_ERROR",
}

EXPORTED_SYMBOLS = (
    "xllm_hip_reshape_paged_cache",
    "xllm_hip_quant_to_paged_cache",
    "xllm_hip_paged_decode_workspace_bytes",
    "xllm_hip_paged_decode_plan",
    "xllm_hip_paged_decode_plan_host_bytes",
    "xllm_hip_paged_decode_plan_host",
    "xllm_hip_paged_decode_run",
    "xllm_hip_paged_decode_run_timed",
    "xllm_hip_paged_decode",
    "xllm_hip_paged_decode_static",
    "xllm_hip_csr_to_block_table",
    "xllm_hip_rope_kv_write",
    "xllm_hip_swap_blocks_staging_bytes",
    "xllm_hip_swap_blocks",
    "xllm_hip_copy_blocks",
    "xllm_hip_gather_from_cache",
    "xllm_hip_set_option",
    "xllm_hip_get_option",
    "xllm_hip_last_error",
    "xllm_hip_abi_version",
    "xllm_hip_paged_decode_variant",
    "xllm_hip_paged_decode_describe",
)


class KvCacheDesc(ctypes.Structure):
    """struct xllm_hip_kv_cache"""

    _fields_ = [
        ("k_cache", ctypes.c_void_p),
        ("v_cache", ctypes.c_void_p),
        ("k_scale", ctypes.c_void_p),
        ("v_scale", ctypes.c_void_p),
        ("num_blocks", ctypes.c_int64),
        ("block_size", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("stride_block", ctypes.c_int64),
        ("stride_head", ctypes.c_int64),
        ("stride_slot", ctypes.c_int64),
        ("scale_stride_block", ctypes.c_int64),
        ("scale_stride_head", ctypes.c_int64),
        ("scale_stride_slot", ctypes.c_int64),
    ]


class DecodeArgs(ctypes.Structure):
    """struct xllm_hip_decode_args"""

    _fields_ = [
        ("q", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("lse", ctypes.c_void_p),
        ("q_token_stride", ctypes.c_int64),
        ("out_token_stride", ctypes.c_int64),
        ("q_dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32),
        ("q_per_seq", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("sm_scale", ctypes.c_float),
        ("window_left", ctypes.c_int32),
        ("block_table", ctypes.c_void_p),
        ("block_table_stride", ctypes.c_int64),
        ("max_blocks_per_seq", ctypes.c_int32),
        ("seq_lens", ctypes.c_void_p),
        ("kv_indptr", ctypes.c_void_p),
        ("kv_indices", ctypes.c_void_p),
        ("kv_last_page_len", ctypes.c_void_p),
        ("max_seq_len", ctypes.c_int32),
        ("total_kv_len", ctypes.c_int64),
        ("q_indptr", ctypes.c_void_p),
        ("host_plan", ctypes.c_int32),
    ]


class RopeArgs(ctypes.Structure):
    """struct xllm_hip_rope_args"""

    _fields_ = [
        ("qkv", ctypes.c_void_p),
        ("token_stride", ctypes.c_int64),
        ("num_tokens", ctypes.c_int64),
        ("dtype", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_k_heads", ctypes.c_int32),
        ("num_v_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("rotary_dim", ctypes.c_int32),
        ("q_weight", ctypes.c_void_p),
        ("k_weight", ctypes.c_void_p),
        ("eps", ctypes.c_float),
        ("cos_sin_dtype", ctypes.c_int32),
        ("cos_sin_cache", ctypes.c_void_p),
        ("max_position", ctypes.c_int64),
        ("positions", ctypes.c_void_p),
        ("interleave", ctypes.c_int32),
        ("round_each_op", ctypes.c_int32),
        ("positions_int32", ctypes.c_int32),
    ]


class XllmHipError(RuntimeError):
    def __init__(self, status, message):
        self.status = status
        super().__init__("%s: %s" % (STATUS_NAMES.get(status, status), message))


_lib = None


def load():
    """Load the shared library (once) and declare every entry point's signature."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s is missing: build it with `python -m xllm_wxh_amd.build` "
            "(or __graft_entry__.build()); there is no non-HIP fallback" % LIB_PATH
        )
    lib = ctypes.CDLL(LIB_PATH)
    missing = [s for s in EXPORTED_SYMBOLS if not hasattr(lib, s)]
    if missing:
        raise ImportError("%s lacks symbols: %s" % (LIB_PATH, ", ".join(missing)))

    P = ctypes.POINTER
    i32, i64, vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
    lib.xllm_hip_reshape_paged_cache.argtypes = [P(KvCacheDesc), vp, vp, vp, i64, i64, i64, i32, vp]
    lib.xllm_hip_reshape_paged_cache.restype = ctypes.c_int
    lib.xllm_hip_quant_to_paged_cache.argtypes = [P(KvCacheDesc), vp, vp, vp, i64, i64, i64, i32, vp]
    lib.xllm_hip_quant_to_paged_cache.restype = ctypes.c_int
    lib.xllm_hip_paged_decode_workspace_bytes.argtypes = [i32, i32, i32, i32, i32]
    lib.xllm_hip_paged_decode_workspace_bytes.restype = ctypes.c_size_t
    for name in ("xllm_hip_paged_decode_plan", "xllm_hip_paged_decode_run", "xllm_hip_paged_decode"):
        fn = getattr(lib, name)
        fn.argtypes = [P(KvCacheDesc), P(DecodeArgs), vp, ctypes.c_size_t, vp]
        fn.restype = ctypes.c_int
    lib.xllm_hip_paged_decode_plan_host_bytes.argtypes = [i32, i32, i32, i32, i32]
    lib.xllm_hip_paged_decode_plan_host_bytes.restype = ctypes.c_size_t
    lib.xllm_hip_paged_decode_plan_host.argtypes = [P(KvCacheDesc), P(DecodeArgs), vp, vp, ctypes.c_size_t, vp, ctypes.c_size_t,
                                                    vp, P(ctypes.c_int64)]
    lib.xllm_hip_paged_decode_plan_host.restype = ctypes.c_int
    lib.xllm_hip_paged_decode_run_timed.argtypes = [P(KvCacheDesc), P(DecodeArgs), vp, ctypes.c_size_t, vp, vp, vp]
    lib.xllm_hip_paged_decode_run_timed.restype = ctypes.c_int
    lib.xllm_hip_paged_decode_static.argtypes = [P(KvCacheDesc), P(DecodeArgs), vp]
    lib.xllm_hip_paged_decode_static.restype = ctypes.c_int
    lib.xllm_hip_csr_to_block_table.argtypes = [vp, vp, vp, i32, i32, vp, i64, i32, vp, vp]
    lib.xllm_hip_csr_to_block_table.restype = ctypes.c_int
    lib.xllm_hip_rope_kv_write.argtypes = [P(RopeArgs), P(KvCacheDesc), vp, vp]
    lib.xllm_hip_rope_kv_write.restype = ctypes.c_int
    lib.xllm_hip_swap_blocks_staging_bytes.argtypes = [P(KvCacheDesc), i64]
    lib.xllm_hip_swap_blocks_staging_bytes.restype = ctypes.c_size_t
    lib.xllm_hip_swap_blocks.argtypes = [P(KvCacheDesc), vp, vp, i64, vp, ctypes.c_size_t, vp]
    lib.xllm_hip_swap_blocks.restype = ctypes.c_int
    lib.xllm_hip_copy_blocks.argtypes = [P(KvCacheDesc), vp, vp, vp, i32, i32, vp]
    lib.xllm_hip_copy_blocks.restype = ctypes.c_int
    lib.xllm_hip_gather_from_cache.argtypes = [P(KvCacheDesc), vp, vp, i32, i64, i64, vp, vp, vp, vp, i64, i32, i32,
                                               i32, i32, vp]
    lib.xllm_hip_gather_from_cache.restype = ctypes.c_int
    lib.xllm_hip_set_option.argtypes = [i32, i64]
    lib.xllm_hip_set_option.restype = ctypes.c_int
    lib.xllm_hip_get_option.argtypes = [i32]
    lib.xllm_hip_get_option.restype = ctypes.c_int64
    lib.xllm_hip_last_error.argtypes = []
    lib.xllm_hip_last_error.restype = ctypes.c_char_p
    lib.xllm_hip_abi_version.argtypes = []
    lib.xllm_hip_abi_version.restype = ctypes.c_int
    lib.xllm_hip_paged_decode_variant.argtypes = [P(KvCacheDesc), P(DecodeArgs)]
    lib.xllm_hip_paged_decode_variant.restype = ctypes.c_char_p
    lib.xllm_hip_paged_decode_describe.argtypes = [P(KvCacheDesc), P(DecodeArgs), ctypes.c_size_t,
                                                   P(ctypes.c_int64), ctypes.c_int32]
    lib.xllm_hip_paged_decode_describe.restype = ctypes.c_int

    if lib.xllm_hip_abi_version() != ABI_VERSION:
        raise ImportError(
            "%s has ABI version %d, this binding expects %d" % (LIB_PATH, lib.xllm_hip_abi_version(), ABI_VERSION)
        )
    _lib = lib
    return lib


def check(status):
    """Turn a non-OK status into an exception carrying the library's message."""
    if status != OK:
        raise XllmHipError(status, load().xllm_hip_last_error().decode("utf-8", "replace"))
