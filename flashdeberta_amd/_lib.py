"""ctypes binding of libfdb_hip.so (the C ABI declared in include/fdb.h).

The library is loaded after torch so that it binds to the HIP runtime torch already mapped.
There is no fallback: if the shared object is missing the import of this module raises.
"""
import ctypes
import os

import torch  # noqa: F401  (must be imported first: provides libamdhip64)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libfdb_hip.so")

FDB_F32, FDB_BF16, FDB_F16, FDB_FP8_E4M3 = 0, 1, 2, 3
FDB_NOALLOC_SCRATCH_BYTES = 32 * 1024 * 1024
FDB_BWD_MAX_WINDOW = 60  # of include/fdb.h: table rows beyond the first that one 32-row backward step may reach
FDB_VERSION = 7  # of include/fdb.h as mirrored below


class FdbAttnArgs(ctypes.Structure):
    _fields_ = (
        [(n, ctypes.c_void_p) for n in (
            "q", "k", "v", "pos_key", "pos_query", "out", "lse", "cu_seqlens", "worklist", "seq_start", "seq_len", "delta_lut",
            "q_scale", "k_scale", "pk_scale", "pq_scale", "workspace")]
        + [(n, ctypes.c_int64) for n in (
            "q_stride_b", "q_stride_t", "q_stride_h", "k_stride_b", "k_stride_t", "k_stride_h",
            "v_stride_b", "v_stride_t", "v_stride_h", "o_stride_b", "o_stride_t", "o_stride_h",
            "pk_stride_h", "pk_stride_r", "pq_stride_h", "pq_stride_r", "workspace_bytes")]
        + [(n, ctypes.c_int32) for n in (
            "batch", "heads", "head_dim", "max_seqlen", "total_tokens", "att_span", "lut_radius", "dtype", "causal", "far_splits",
            "near_splits")]
        + [("sm_scale", ctypes.c_float)]
    )


class FdbAttnBwdArgs(ctypes.Structure):
    _fields_ = (
        [(n, ctypes.c_void_p) for n in (
            "q", "k", "v", "dout", "dq", "dk", "dv", "lse", "delta", "out", "c2p_bias", "p2c_bias", "d_c2p_bias", "d_p2c_bias",
            "seq_start", "seq_len", "delta_lut")]
        + [(n + s, ctypes.c_int64) for n in ("q", "k", "v", "do", "out", "dq", "dk", "dv", "bias") for s in ("_stride_b", "_stride_t", "_stride_h")]
        + [(n, ctypes.c_int32) for n in ("batch", "heads", "head_dim", "seqlen", "att_span", "lut_radius", "lut_window", "dtype", "causal")]
        + [("sm_scale", ctypes.c_float)]
    )


EXPORTS = (
    "fdb_version", "fdb_attn_args_size", "fdb_strerror", "fdb_attn_check", "fdb_attn_fwd", "fdb_attn_fwd_part", "fdb_attn_fwd_noalloc", "fdb_attn_bwd", "fdb_attn_bwd_chain", "fdb_attn_bwd_args_size", "fdb_attn_workspace_bytes",
    "fdb_worklist_ints",
    "fdb_worklist_max_tiles", "fdb_tile_rows", "fdb_build_worklist", "fdb_delta_lut_radius", "fdb_delta_lut", "fdb_delta_lut_window",
    "fdb_quant_e4m3_per_head", "fdb_quant_e4m3_per_head_pair", "fdb_dequant_e4m3_per_head",
)


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "flashdeberta_amd: %s is missing. Build it with `python -m flashdeberta_amd.csrc.build` "
            "(needs hipcc); there is no CPU or PyTorch fallback for this path." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
    lib.fdb_version.restype = ctypes.c_int
    lib.fdb_attn_args_size.restype = ctypes.c_size_t
    if lib.fdb_attn_args_size() != ctypes.sizeof(FdbAttnArgs):
        raise ImportError("flashdeberta_amd: %s was built from a different include/fdb.h (struct size %d, binding %d); rebuild it"
                          % (LIB_PATH, lib.fdb_attn_args_size(), ctypes.sizeof(FdbAttnArgs)))
    if lib.fdb_version() != FDB_VERSION:  # the struct can change its layout and keep its size
        raise ImportError("flashdeberta_amd: %s is version %d of the C ABI, this binding is version %d; rebuild it"
                          % (LIB_PATH, lib.fdb_version(), FDB_VERSION))
    lib.fdb_strerror.restype = ctypes.c_char_p
    lib.fdb_strerror.argtypes = [ctypes.c_int]
    lib.fdb_attn_check.restype = ctypes.c_int
    lib.fdb_attn_check.argtypes = [ctypes.POINTER(FdbAttnArgs)]
    lib.fdb_attn_fwd.restype = ctypes.c_int
    lib.fdb_attn_fwd.argtypes = [ctypes.POINTER(FdbAttnArgs), vp]
    lib.fdb_attn_fwd_part.restype = ctypes.c_int
    lib.fdb_attn_fwd_part.argtypes = [ctypes.POINTER(FdbAttnArgs), i32, vp]
    lib.fdb_attn_fwd_noalloc.restype = ctypes.c_int
    lib.fdb_attn_fwd_noalloc.argtypes = [ctypes.POINTER(FdbAttnArgs), vp]
    lib.fdb_attn_bwd_args_size.restype = ctypes.c_size_t
    if lib.fdb_attn_bwd_args_size() != ctypes.sizeof(FdbAttnBwdArgs):
        raise ImportError("flashdeberta_amd: %s was built from a different include/fdb.h (backward struct size %d, binding %d); "
                          "rebuild it" % (LIB_PATH, lib.fdb_attn_bwd_args_size(), ctypes.sizeof(FdbAttnBwdArgs)))
    lib.fdb_attn_bwd.restype = ctypes.c_int
    lib.fdb_attn_bwd.argtypes = [ctypes.POINTER(FdbAttnBwdArgs), vp]
    lib.fdb_attn_bwd_chain.restype = ctypes.c_int
    lib.fdb_attn_bwd_chain.argtypes = [vp, vp, vp, vp, vp, vp, vp, i32, i32, i64, i64, i64, i64, i64, i32, i32, i32, i32, vp]
    lib.fdb_attn_workspace_bytes.restype = i64
    lib.fdb_attn_workspace_bytes.argtypes = [ctypes.POINTER(FdbAttnArgs)]
    lib.fdb_worklist_ints.restype = i64
    lib.fdb_worklist_ints.argtypes = [i32, i32]
    lib.fdb_worklist_max_tiles.restype = i32
    lib.fdb_worklist_max_tiles.argtypes = [i32, i32]
    lib.fdb_tile_rows.restype = i32
    lib.fdb_build_worklist.restype = ctypes.c_int
    lib.fdb_build_worklist.argtypes = [vp, i32, i32, vp, vp]
    lib.fdb_delta_lut_radius.restype = i32
    lib.fdb_delta_lut_radius.argtypes = [i32, i32]
    lib.fdb_delta_lut_window.restype = i32
    lib.fdb_delta_lut_window.argtypes = [i32, i32]
    lib.fdb_delta_lut.restype = ctypes.c_int
    lib.fdb_delta_lut.argtypes = [i32, i32, i32, vp]
    lib.fdb_quant_e4m3_per_head.restype = ctypes.c_int
    lib.fdb_quant_e4m3_per_head.argtypes = [vp, i64, i64, vp, i64, i64, vp, vp, i32, i32, i32, vp]
    lib.fdb_quant_e4m3_per_head_pair.restype = ctypes.c_int
    lib.fdb_quant_e4m3_per_head_pair.argtypes = [vp, vp, i64, i64, vp, vp, i64, i64, vp, vp, vp, i32, i32, i32, vp]
    lib.fdb_dequant_e4m3_per_head.restype = ctypes.c_int
    lib.fdb_dequant_e4m3_per_head.argtypes = [vp, i64, i64, vp, vp, i64, i64, i32, i32, i32, vp]
    return lib


lib = _load()


def strerror(code):
    return lib.fdb_strerror(int(code)).decode()


def check(code, what):
    """Negative codes are argument errors (ValueError), positive ones HIP errors (RuntimeError)."""
    if code == 0:
        return
    msg = "%s failed: %s (code %d)" % (what, strerror(code), code)
    if code < 0:
        raise ValueError(msg)
    raise RuntimeError(msg)
