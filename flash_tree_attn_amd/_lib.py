"""ctypes binding of libfta.so (declarations mirror include/fta.h)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfta.so")

ABI_VERSION = 3
FTA_F32, FTA_F16, FTA_BF16 = 0, 1, 2
FTA_I32, FTA_I64 = 0, 1
MASK_ADDITIVE_F32, MASK_PACKED_U64 = 0, 1
KERNEL_SHUFFLE, KERNEL_MFMA, KERNEL_MFMA_WIDE, KERNEL_MFMA_SPLIT_KEYS = 0, 1, 2, 3

EXPORTED_SYMBOLS = (
    "fta_abi_version", "fta_strerror", "fta_validate", "fta_plan", "fta_decode", "fta_decode_stage1",
    "fta_decode_stage2", "fta_device_cus", "fta_append_kv",
)

# status -> Python exception class
_VALUE_ERRORS = {-1, -2, -3, -4, -5, -6, -7, -8, -9}


class FtaArgs(C.Structure):
    _fields_ = [
        ("q", C.c_void_p), ("k_cache", C.c_void_p), ("v_cache", C.c_void_p),
        ("cur_k", C.c_void_p), ("cur_v", C.c_void_p), ("mask", C.c_void_p),
        ("kv_seq_len", C.c_void_p), ("out", C.c_void_p), ("mid_o", C.c_void_p), ("mid_lse", C.c_void_p),
        ("counters", C.c_void_p), ("block_table", C.c_void_p),
        ("bsz", C.c_int32), ("num_q_heads", C.c_int32), ("num_kv_heads", C.c_int32), ("cur_heads", C.c_int32),
        ("q_len", C.c_int32), ("head_dim", C.c_int32), ("cache_len", C.c_int32), ("v_cache_len", C.c_int32),
        ("block_size", C.c_int32), ("max_seq_len_hint", C.c_int32), ("mid_splits", C.c_int32),
        ("dtype", C.c_int32), ("len_dtype", C.c_int32), ("force_splits", C.c_int32), ("force_kernel", C.c_int32),
        ("counter_elems", C.c_int32), ("mask_kind", C.c_int32), ("page_size", C.c_int32), ("sm_scale", C.c_float),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
        ("ck_stride", C.c_int64 * 3), ("cv_stride", C.c_int64 * 3), ("mask_stride", C.c_int64 * 3),
        ("out_stride", C.c_int64 * 3), ("mid_o_stride", C.c_int64 * 4), ("mid_lse_stride", C.c_int64 * 3),
        ("block_table_stride", C.c_int64),
    ]


class FtaAppendArgs(C.Structure):
    _fields_ = [
        ("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("cur_k", C.c_void_p), ("cur_v", C.c_void_p),
        ("accept_idx", C.c_void_p), ("accept_len", C.c_void_p), ("kv_seq_len", C.c_void_p), ("kv_seq_len_out", C.c_void_p),
        ("block_table", C.c_void_p),
        ("bsz", C.c_int32), ("num_kv_heads", C.c_int32), ("q_len", C.c_int32), ("head_dim", C.c_int32),
        ("cache_len", C.c_int32), ("max_accept", C.c_int32), ("dtype", C.c_int32), ("len_dtype", C.c_int32),
        ("page_size", C.c_int32), ("reserved", C.c_int32),
        ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3), ("ck_stride", C.c_int64 * 3), ("cv_stride", C.c_int64 * 3),
        ("accept_idx_stride", C.c_int64), ("block_table_stride", C.c_int64),
    ]


LEN_BUCKETS = 16   # FTA_LEN_BUCKETS


class FtaPlanOut(C.Structure):
    _fields_ = [
        ("kernel", C.c_int32), ("num_splits", C.c_int32), ("chunk", C.c_int32), ("rows_per_group", C.c_int32),
        ("rows_per_wg", C.c_int32), ("row_blocks", C.c_int32), ("num_workgroups", C.c_int32), ("counter_elems", C.c_int32),
        ("single_launch", C.c_int32), ("mfma_loop", C.c_int32),
        ("mid_o_elems", C.c_int64), ("mid_lse_elems", C.c_int64),
        ("len_bound", C.c_int32 * LEN_BUCKETS), ("chunk_by_len", C.c_int32 * LEN_BUCKETS),
    ]

    def chunk_for(self, max_len: int) -> int:
        """Keys per split the kernels use for a batch whose longest sequence has max_len cached keys."""
        for bound, chunk in zip(self.len_bound, self.chunk_by_len):
            if max_len <= bound:
                return chunk
        return self.chunk_by_len[LEN_BUCKETS - 1]


class FtaError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(f"fta status {status}: {text}")
        self.status = status


_lib = None


def load() -> C.CDLL:
    """Loads libfta.so; raises (never falls back) when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m flash_tree_attn_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback implementation."
        )
    lib = C.CDLL(LIB_PATH)
    lib.fta_abi_version.restype = C.c_int
    lib.fta_strerror.restype = C.c_char_p
    lib.fta_strerror.argtypes = [C.c_int]
    lib.fta_validate.restype = C.c_int
    lib.fta_validate.argtypes = [C.POINTER(FtaArgs)]
    lib.fta_plan.restype = C.c_int
    lib.fta_plan.argtypes = [C.POINTER(FtaArgs), C.c_int, C.POINTER(FtaPlanOut)]
    lib.fta_decode.restype = C.c_int
    lib.fta_decode.argtypes = [C.POINTER(FtaArgs), C.c_void_p]
    for name in ("fta_decode_stage1", "fta_decode_stage2"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.POINTER(FtaArgs), C.c_void_p]
    lib.fta_device_cus.restype = C.c_int
    lib.fta_append_kv.restype = C.c_int
    lib.fta_append_kv.argtypes = [C.POINTER(FtaAppendArgs), C.c_void_p]
    if lib.fta_abi_version() != ABI_VERSION:
        raise ImportError(f"libfta.so has ABI {lib.fta_abi_version()}, binding expects {ABI_VERSION}; rebuild it")
    _lib = lib
    return lib


def check(status: int) -> None:
    if status == 0:
        return
    text = load().fta_strerror(status).decode()
    if status in _VALUE_ERRORS:
        err = ValueError(f"fta status {status}: {text}")
        err.status = status
        raise err
    raise FtaError(status, text)
