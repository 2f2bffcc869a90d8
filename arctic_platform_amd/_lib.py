"""ctypes binding of libzorro_fca.so (C ABI declared in include/zorro_fca.h).

There is no fallback: if the library has not been built the import of any operator
raises, and on a machine with a GPU every operator call goes through the HIP kernels.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libzorro_fca.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

FCA_BF16, FCA_FP8_E4M3, FCA_F32 = 0, 1, 2
FCA_MAX_LEVELS = 8
FCA_STATIC_SCRATCH_BYTES = 48 << 20

EXPORTS = (
    "fca_version",
    "fca_last_error",
    "fca_workspace_bytes",
    "fca_workspace_bytes_dtype",
    "fca_meta_describe",
    "fca_build_metadata",
    "fca_update_metadata",
    "fca_build_metadata_rows",
    "fca_rows_from_query_runs",
    "fca_prefix_pass",
    "fca_suffix_pass",
    "fca_forest_pass",
    "fca_merge",
    "fca_decode_step",
    "fca_decode_step_static",
    "fca_append_kv",
    "fca_gather_kv",
    "fca_calibration_copy",
    "fca_time_next_attention",
    "fca_split_layout_ints",
    "fca_split_layout_build",
    "fca_split_workspace_bytes",
    "fca_split_attention_forward",
    "fca_split_attention_backward",
    "fca_gather_rows",
    "fca_sum_rows",
)


class FcaSplitPlan(ctypes.Structure):
    _fields_ = [
        ("num_tokens", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("window", ctypes.c_int32),
        ("dropout_p", ctypes.c_float),
        ("dropout_seed", ctypes.c_uint32),
    ]


class FcaPlan(ctypes.Structure):
    _fields_ = [
        ("num_seqs", ctypes.c_int32),
        ("max_blocks", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
        ("chunk_tokens", ctypes.c_int32),
        ("rows_per_item", ctypes.c_int32),
        ("max_levels", ctypes.c_int32),
    ]


class FcaTensors(ctypes.Structure):
    _fields_ = [
        ("q_dev", ctypes.c_void_p),
        ("q_seq_stride", ctypes.c_int64),
        ("q_head_stride", ctypes.c_int64),
        ("k_cache_dev", ctypes.c_void_p),
        ("v_cache_dev", ctypes.c_void_p),
        ("kv_block_stride", ctypes.c_int64),
        ("kv_head_stride", ctypes.c_int64),
        ("kv_dtype", ctypes.c_int32),
        ("kv_reread", ctypes.c_int32),
        ("block_table_dev", ctypes.c_void_p),
        ("block_table_stride", ctypes.c_int64),
        ("k_scale_dev", ctypes.c_void_p),
        ("v_scale_dev", ctypes.c_void_p),
        ("softmax_scale", ctypes.c_float),
        ("reproducible", ctypes.c_int32),
        ("max_workgroups", ctypes.c_int32),
        ("tile_buffers", ctypes.c_int32),
    ]


class FcaMetaLayout(ctypes.Structure):
    _fields_ = [
        (name, ctypes.c_int64)
        for name in (
            "header",
            "seq_npart",
            "seq_leaf_blk",
            "node_rep",
            "node_blk",
            "node_nblk",
            "node_level",
            "node_moff",
            "node_mcnt",
            "node_ord",
            "members",
            "items",
            "max_items",
            "max_partials",
            "total_int32",
            "node_tok",
            "node_causal",
            "coop_ctr",
        )
    ]


class FcaError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"libzorro_fca error {code}: {message}")
        self.code = code


def build_library(verbose: bool = False) -> str:
    """Compile csrc/*.hip for gfx950 into libzorro_fca.so next to this file."""
    cmd = ["make", "-C", CSRC_DIR, "-B", f"OUT={LIB_PATH}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("building libzorro_fca.so failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stdout)
    return LIB_PATH


_lib = None


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
            "(or __graft_entry__.build()); there is no non-HIP fallback"
        )
    _lib = declare_signatures(ctypes.CDLL(LIB_PATH))
    return _lib


def declare_signatures(lib: ctypes.CDLL) -> ctypes.CDLL:
    """Argument and result types of every entry point of include/zorro_fca.h, set on ``lib``."""
    P, VP, I32, I64 = ctypes.POINTER, ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    SZ = P(ctypes.c_size_t)
    lib.fca_version.restype = ctypes.c_int
    lib.fca_version.argtypes = []
    lib.fca_last_error.restype = ctypes.c_char_p
    lib.fca_last_error.argtypes = []
    lib.fca_workspace_bytes.argtypes = [P(FcaPlan), SZ, SZ, SZ]
    lib.fca_workspace_bytes_dtype.argtypes = [P(FcaPlan), I32, SZ, SZ, SZ]
    lib.fca_meta_describe.argtypes = [P(FcaPlan), P(FcaMetaLayout)]
    lib.fca_build_metadata.argtypes = [P(FcaPlan), VP, I64, VP, VP, VP]
    lib.fca_update_metadata.argtypes = [P(FcaPlan), VP, I64, VP, VP, VP]
    lib.fca_build_metadata_rows.argtypes = [P(FcaPlan), VP, I64, I32, VP, VP, VP, VP, I32, VP]
    lib.fca_rows_from_query_runs.argtypes = [VP, VP, I32, I32, I32, VP, VP, VP, VP]
    attend = [P(FcaPlan), P(FcaTensors), VP, VP, VP, VP]
    lib.fca_prefix_pass.argtypes = attend
    lib.fca_suffix_pass.argtypes = attend
    lib.fca_forest_pass.argtypes = attend
    lib.fca_merge.argtypes = [P(FcaPlan), VP, VP, VP, VP, I64, I64, I32, VP, VP]
    lib.fca_decode_step.argtypes = [P(FcaPlan), P(FcaTensors), VP, VP, VP, VP, I64, I64, I32, VP, VP]
    lib.fca_decode_step_static.argtypes = [P(FcaPlan), P(FcaTensors), VP, VP, I64, I64, I32, VP, VP]
    lib.fca_append_kv.argtypes = [VP, VP, I64, I64, I32, I32, I32, VP, VP, VP, I64, I64, I32, VP, VP, VP]
    lib.fca_gather_kv.argtypes = lib.fca_append_kv.argtypes
    lib.fca_calibration_copy.argtypes = [VP, VP, ctypes.c_size_t, VP]
    lib.fca_time_next_attention.argtypes = [VP, VP]
    F32 = ctypes.c_float
    lib.fca_split_layout_ints.argtypes = [I32, P(I64)]
    lib.fca_split_layout_build.argtypes = [I32, VP, VP, VP, I32, I32, I32, VP]
    lib.fca_split_workspace_bytes.argtypes = [P(FcaSplitPlan), SZ, SZ]
    lib.fca_split_attention_forward.argtypes = [P(FcaSplitPlan), VP, I64, VP, I64, VP, I64, VP, F32, VP, VP, I64, VP, VP]
    lib.fca_split_attention_backward.argtypes = (
        [P(FcaSplitPlan)] + [VP, I64] * 5 + [VP, VP, F32, VP] + [VP, I64] * 3 + [VP]
    )
    lib.fca_gather_rows.argtypes = [VP, I64, VP, I64, I64, VP, I64, VP]
    lib.fca_sum_rows.argtypes = [VP, I64, VP, VP, I64, I64, I32, VP, I64, VP]
    for name in EXPORTS:
        if name not in ("fca_version", "fca_last_error"):
            getattr(lib, name).restype = ctypes.c_int
    return lib


def check(rc: int) -> None:
    if rc != 0:
        raise FcaError(rc, load_library().fca_last_error().decode("utf-8", "replace"))
