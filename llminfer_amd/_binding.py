"""ctypes binding of include/llmi_hip.h. Loads the in-tree libllmi_hip.so and
fails loudly when it is missing: there is no fallback path."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# LLMI_HIP_LIBRARY names another build of the same library (a tuning or diagnostic variant).
LIB_PATH = os.environ.get("LLMI_HIP_LIBRARY") or os.path.join(HERE, "libllmi_hip.so")

c_i32 = ctypes.c_int32
c_void_p = ctypes.c_void_p
c_size_t = ctypes.c_size_t

LLMI_OK = 0
KV_LAYOUT_POS_MAJOR = 0
KV_LAYOUT_HEAD_MAJOR = 1
PATH_AUTO, PATH_SINGLE_PASS, PATH_SPLIT, PATH_SPLIT_FUSED = 0, 1, 2, 3

STATUS = {
    "OK": 0, "NULL_POINTER": -1, "HEAD_DIM": -2, "KV_DIM": -3, "ALIGNMENT": -4, "POS_RANGE": -5,
    "WORKSPACE": -6, "HEAD_GROUP": -7, "LAYOUT": -8, "INVALID_ARG": -9, "LAUNCH": -10,
    "UNKNOWN_POINTER": -11, "OUT_OF_MEMORY": -12,
}


class MhaArgs(ctypes.Structure):
    _fields_ = [
        ("query", c_void_p), ("key_cache", c_void_p), ("value_cache", c_void_p),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t), ("output", c_void_p),
        ("output_f32", c_void_p),
        ("layer_id", c_i32), ("pos", c_i32), ("kv_dim", c_i32), ("kv_mul", c_i32),
        ("head_num", c_i32), ("head_dim", c_i32), ("max_seq_len", c_i32), ("kv_layout", c_i32),
        ("force_path", c_i32), ("num_splits", c_i32), ("waves_per_group", c_i32),
        ("stream", c_void_p), ("pos_device", c_void_p), ("workspace_side", c_i32),
    ]


class MhaAppendArgs(ctypes.Structure):
    _fields_ = [
        ("mha", MhaArgs), ("key_new", c_void_p), ("value_new", c_void_p), ("norm_weight", c_void_p),
        ("sin_cache", c_void_p), ("cos_cache", c_void_p), ("eps", ctypes.c_float),
    ]


class AttnOprojArgs(ctypes.Structure):
    _fields_ = [("attn", MhaAppendArgs), ("o_weight", c_void_p), ("residual", c_void_p), ("hidden", c_i32), ("one_launch", c_i32)]


class MhaStackArgs(ctypes.Structure):
    _fields_ = [("first", MhaAppendArgs), ("layer_count", c_i32), ("query_stride", ctypes.c_int64),
                ("key_new_stride", ctypes.c_int64), ("value_new_stride", ctypes.c_int64),
                ("norm_weight_stride", ctypes.c_int64), ("output_stride", ctypes.c_int64)]


class GemvArgs(ctypes.Structure):
    _fields_ = [
        ("input", c_void_p), ("weight", c_void_p), ("output", c_void_p),
        ("n", c_i32), ("k", c_i32), ("mode", c_i32), ("stream", c_void_p),
    ]


class QkvGemvArgs(ctypes.Structure):
    _fields_ = [
        ("input", c_void_p), ("weight", c_void_p), ("query", c_void_p), ("key", c_void_p), ("value", c_void_p),
        ("dim", c_i32), ("kv_dim", c_i32), ("k", c_i32), ("stream", c_void_p),
    ]


GEMV_OUT_BF16, GEMV_OUT_F32, GEMV_ADD_BF16 = 0, 1, 2


class MhaPlan(ctypes.Structure):
    _fields_ = [
        ("path", c_i32), ("num_splits", c_i32), ("rows_per_split", c_i32),
        ("waves_per_group", c_i32), ("group_pad", c_i32), ("workspace_side", c_i32), ("workspace_needed", c_size_t),
    ]


class QkNormRopeArgs(ctypes.Structure):
    _fields_ = [
        ("query", c_void_p), ("query_src", c_void_p), ("key_new", c_void_p), ("value_new", c_void_p),
        ("key_cache", c_void_p), ("value_cache", c_void_p), ("norm_weight", c_void_p),
        ("sin_cache", c_void_p), ("cos_cache", c_void_p),
        ("layer_id", c_i32), ("pos", c_i32), ("kv_dim", c_i32), ("head_num", c_i32),
        ("head_dim", c_i32), ("max_seq_len", c_i32), ("kv_layout", c_i32),
        ("eps", ctypes.c_float), ("stream", c_void_p),
    ]


DIAG_PLAIN, DIAG_SC0, DIAG_SC1, DIAG_SC0_SC1, DIAG_NT = range(5)  # llmi_hip_diag.h: cache policy of the hand-over probe


class DiagHandoverResult(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("seen", "polls", "ns", "xcc_reader", "xcc_writer")]


class PoolStats(ctypes.Structure):
    _fields_ = [(n, c_size_t) for n in (
        "backing_allocs", "reuses", "big_busy_blocks", "big_free_blocks", "small_busy_blocks",
        "small_free_blocks", "big_busy_bytes", "big_free_bytes", "small_busy_bytes",
        "small_free_bytes")]


BACKING_ALLOC_FN = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.POINTER(c_void_p), c_size_t, c_void_p)
BACKING_FREE_FN = ctypes.CFUNCTYPE(ctypes.c_int, c_void_p, c_void_p)

# name -> (restype, argtypes): every symbol include/llmi_hip.h declares.
SYMBOLS = {
    "llmi_hip_mha_plan": (ctypes.c_int, [ctypes.POINTER(MhaArgs), ctypes.POINTER(MhaPlan)]),
    "llmi_hip_mha_decode": (ctypes.c_int, [ctypes.POINTER(MhaArgs)]),
    "llmi_hip_mha_decode_static": (ctypes.c_int, [ctypes.POINTER(MhaArgs)]),
    "llmi_hip_mha_decode_append": (ctypes.c_int, [ctypes.POINTER(MhaAppendArgs)]),
    "llmi_hip_mha_decode_append_oproj": (ctypes.c_int, [ctypes.POINTER(AttnOprojArgs)]),
    "llmi_hip_mha_oproj_launches": (ctypes.c_int, [ctypes.POINTER(AttnOprojArgs)]),
    "llmi_hip_mha_decode_append_stack": (ctypes.c_int, [ctypes.POINTER(MhaStackArgs)]),
    "llmi_hip_mha_stack_launches": (ctypes.c_int, [ctypes.POINTER(MhaStackArgs)]),
    "llmi_hip_mha_workspace_bytes": (c_size_t, [c_i32, c_i32, c_i32]),
    "llmi_hip_mha_workspace_side": (ctypes.c_int, [c_void_p, c_size_t, c_void_p, ctypes.POINTER(c_i32)]),
    "llmi_hip_qk_norm_rope_append": (ctypes.c_int, [ctypes.POINTER(QkNormRopeArgs)]),
    "llmi_hip_sincos_table": (ctypes.c_int, [c_void_p, c_void_p, c_i32, c_i32, c_void_p]),
    "llmi_hip_kv_restride": (ctypes.c_int, [c_void_p, c_void_p, c_i32, c_i32, c_i32, c_i32, c_i32, c_void_p]),
    "llmi_hip_gemv": (ctypes.c_int, [ctypes.POINTER(GemvArgs)]),
    "llmi_hip_qkv_gemv": (ctypes.c_int, [ctypes.POINTER(QkvGemvArgs)]),
    "llmi_pool_create": (c_void_p, [BACKING_ALLOC_FN, BACKING_FREE_FN, c_void_p]),
    "llmi_pool_destroy": (None, [c_void_p]),
    "llmi_pool_alloc": (c_void_p, [c_void_p, c_size_t]),
    "llmi_pool_free": (ctypes.c_int, [c_void_p, c_void_p]),
    "llmi_pool_trim": (c_size_t, [c_void_p]),
    "llmi_pool_get_stats": (ctypes.c_int, [c_void_p, ctypes.POINTER(PoolStats)]),
    "llmi_hip_default_pool": (c_void_p, []),
    "llmi_hip_pool_alloc": (c_void_p, [c_size_t]),
    "llmi_hip_pool_free": (ctypes.c_int, [c_void_p]),
    "llmi_hip_memcpy": (ctypes.c_int, [c_void_p, c_void_p, c_size_t, c_i32, c_void_p, c_i32]),
    "llmi_hip_memset_zero": (ctypes.c_int, [c_void_p, c_size_t, c_void_p, c_i32]),
    "llmi_hip_abi_version": (ctypes.c_int, []),
    "llmi_hip_set_poll_limit": (c_i32, [c_i32]),
    "llmi_hip_poll_timeouts": (ctypes.c_int, [ctypes.POINTER(ctypes.c_uint64)]),
    # include/llmi_hip_probes.h
    "llmi_hip_probe_stream_read": (ctypes.c_int, [c_void_p, c_void_p, c_size_t, c_i32, c_i32, c_i32, c_void_p, c_void_p]),
    "llmi_hip_probe_stream_read_rows": (ctypes.c_int, [c_void_p, c_void_p, c_i32, c_i32, c_i32, c_i32, c_i32, c_void_p, c_void_p]),
    "llmi_hip_probe_stream_tiles": (ctypes.c_int, [c_void_p, c_void_p] + [c_i32] * 9 + [c_void_p, c_void_p]),
    "llmi_hip_probe_copy": (ctypes.c_int, [c_void_p, c_void_p, c_size_t, c_void_p]),
    "llmi_hip_probe_block_pingpong": (ctypes.c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "llmi_hip_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "llmi_hip_last_error": (ctypes.c_char_p, []),
    # include/llmi_hip_testing.h
    "llmi_hip_set_test_far_home": (c_i32, [c_i32]),
    "llmi_hip_side_from_pingpong": (c_i32, [ctypes.POINTER(ctypes.c_uint32)]),
    "llmi_hip_side_agreement": (c_i32, [ctypes.POINTER(c_i32), c_i32, ctypes.POINTER(c_i32)]),
    "llmi_hip_stagger_mask": (c_i32, [c_i32, ctypes.c_int64, c_i32]),
    "llmi_hip_workspace_side_stats": (None, [ctypes.POINTER(ctypes.c_uint64)]),
}

# include/llmi_hip_diag.h: the diagnostic probes, a library of their own (libllmi_diag.so)
DIAG_LIB_PATH = os.path.join(HERE, "libllmi_diag.so")
DIAG_SYMBOLS = {
    "llmi_diag_handover": (ctypes.c_int, [c_i32, c_i32, c_i32, c_i32, c_i32, c_void_p, c_void_p, c_void_p]),
    "llmi_diag_placement": (ctypes.c_int, [c_i32, c_i32, c_void_p, c_void_p]),
}

_lib = None
_diag = None


class LlmiError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        msg = lib().llmi_hip_strerror(status).decode()
        detail = lib().llmi_hip_last_error().decode()
        super().__init__("%s failed with status %d: %s%s" % (where, status, msg,
                                                             (" [" + detail + "]") if detail else ""))


def lib():
    """The loaded libllmi_hip.so. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libllmi_hip.so is not built (%s missing); run `python -m llminfer_amd.build`. "
                "There is no fallback implementation." % LIB_PATH)
        # PyTorch ships a HIP runtime of its own. When both are in a process, torch's has to be loaded first:
        # the library then binds to that one, and the device pointers torch hands out are its own. (Loaded the
        # other way round the process holds two runtimes, and launches fail with "no ROCm-capable device".)
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = L
    return _lib


def diag_lib():
    """The loaded libllmi_diag.so (diagnostic probes; nothing on the product path needs it)."""
    global _diag
    if _diag is None:
        lib()  # (torch's HIP runtime first, as above)
        if not os.path.exists(DIAG_LIB_PATH):
            raise RuntimeError("libllmi_diag.so is not built (%s missing); run `python -m llminfer_amd.build`." % DIAG_LIB_PATH)
        L = ctypes.CDLL(DIAG_LIB_PATH)
        for name, (restype, argtypes) in DIAG_SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _diag = L
    return _diag


def check(status, where):
    if status != LLMI_OK:
        raise LlmiError(status, where)
