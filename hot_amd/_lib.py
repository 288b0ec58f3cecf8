"""ctypes binding of libhot_gfx950.so (declared in include/hot_gfx950.h).

The library is the product: if it is missing this module raises, it never
falls back to a CPU or eager-PyTorch implementation.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhot_gfx950.so")

HOT_MAX_HLA_N = 64        # rows inline in the config
HOT_HQ_WORKSPACE_BYTES = 2048
HOT_MAX_HLA_BIG = 8192    # rows through hla_rows_big

# enums of include/hot_gfx950.h
F32, BF16, F16 = 0, 1, 2
ROUND_NEAREST, ROUND_STOCH = 0, 1
SCALE_TENSOR, SCALE_ROW, SCALE_SAWB = 0, 1, 2
STREAM_GX, STREAM_GW, STREAM_W, STREAM_ACT = 0, 1, 2, 3
# enum hot_gemm_variant
(GEMM_AUTO, GEMM_DMA_128_S3, GEMM_DMA_128_S4, GEMM_DMA_256_S4, GEMM_REG_128, GEMM_DMA_128_SPLITK, GEMM_SLOT_256,
 GEMM_SLOT_128, GEMM_SLOT_160X256, GEMM_SLOT_96X128, GEMM_SLOT_64X128, GEMM_SLOT_32X128) = range(12)
HOT_STATIC_MAX_CHANNELS = 16384

EXPORTS = (
    "hot_last_error", "hot_abi_version", "hot_backward_streams", "hot_kpad", "hot_hq_rowwise", "hot_hla_tokenwise",
    "hot_wq_colwise", "hot_colwise_workspace_bytes", "hot_gemm_i8", "hot_abc_workspace_bytes",
    "hot_abc_forward", "hot_backward_workspace_bytes", "hot_linear_backward", "hot_linear_backward_kernels",
    "hot_gemm_splits", "hot_hla_workspace_bytes", "hot_linear_backward_bias",
    "hot_gemm_plan", "hot_gemm_workspace_bytes", "hot_gemm_i8_variant", "hot_gemm_bf16",
    "hot_hla_tokenwise_static", "hot_measure_ceilings",
    "hot_kpad_group", "hot_abc_batched_workspace_bytes", "hot_abc_forward_batched",
    "hot_backward_batched_workspace_bytes", "hot_linear_backward_batched", "hot_backward_batched_ranges",
    "hot_gx_lowrank_workspace_bytes", "hot_gx_lowrank", "hot_gx_luq_workspace_bytes", "hot_gx_luq",
    "hot_gw_luq_workspace_bytes", "hot_gw_luq",
)


class HotConfig(C.Structure):
    """struct hot_config."""
    _fields_ = [
        ("n_o", C.c_int32), ("hla_n", C.c_int32), ("hla_r", C.c_int32),
        ("hla_rows", C.c_int32 * HOT_MAX_HLA_N),
        ("gx_bits", C.c_int32), ("w_bits", C.c_int32), ("gw_bits", C.c_int32), ("act_bits", C.c_int32),
        ("gx_round", C.c_int32), ("w_round", C.c_int32), ("gw_round", C.c_int32), ("act_round", C.c_int32),
        ("gx_scale", C.c_int32), ("w_scale", C.c_int32), ("gw_scale", C.c_int32), ("act_scale", C.c_int32),
        ("seed", C.c_uint64),
        ("hla_rows_big", C.POINTER(C.c_int32)),
        ("streams", C.c_int32), ("reserved", C.c_int32),
    ]


class HotError(RuntimeError):
    pass


_lib = None


def _declare(lib):
    vp, i32, i64, u32, u64, sz, fp = C.c_void_p, C.c_int, C.c_int64, C.c_uint32, C.c_uint64, C.c_size_t, C.c_float
    cfgp = C.POINTER(HotConfig)
    lib.hot_last_error.restype = C.c_char_p
    lib.hot_last_error.argtypes = []
    lib.hot_abi_version.restype = i32
    lib.hot_abi_version.argtypes = []
    lib.hot_backward_streams.restype = i32
    lib.hot_backward_streams.argtypes = [i64, i64, i64, cfgp]
    lib.hot_kpad.restype = i64
    lib.hot_kpad.argtypes = [i64]
    lib.hot_hq_rowwise.restype = i32
    lib.hot_hq_rowwise.argtypes = [vp, i32, i64, i64, i32, i32, i32, u64, u32, i32, vp, vp, vp, sz, vp]
    lib.hot_hla_tokenwise.restype = i32
    lib.hot_hla_tokenwise.argtypes = [vp, i32, i64, i64, i32, C.POINTER(C.c_int32), i32, i32, i32, u64, u32, i32,
                                      vp, i64, vp, vp, sz, vp]
    lib.hot_wq_colwise.restype = i32
    lib.hot_wq_colwise.argtypes = [vp, i32, i64, i64, i32, i32, i32, u64, u32, i32, vp, i64, vp, vp, sz, vp]
    lib.hot_hla_workspace_bytes.restype = sz
    lib.hot_hla_workspace_bytes.argtypes = [i64, i64, i32, i32]
    lib.hot_colwise_workspace_bytes.restype = sz
    lib.hot_colwise_workspace_bytes.argtypes = [i64]
    lib.hot_gemm_i8.restype = i32
    lib.hot_gemm_i8.argtypes = [vp, i64, vp, i64, i32, i64, i64, i64, vp, i32, vp, fp, vp, i32, i64, vp, vp]
    lib.hot_abc_workspace_bytes.restype = sz
    lib.hot_abc_workspace_bytes.argtypes = [i64, i64, cfgp]
    lib.hot_abc_forward.restype = i32
    lib.hot_abc_forward.argtypes = [vp, i32, i64, i64, cfgp, vp, vp, vp, sz, vp]
    lib.hot_backward_workspace_bytes.restype = sz
    lib.hot_backward_workspace_bytes.argtypes = [i64, i64, i64, cfgp]
    lib.hot_linear_backward.restype = i32
    lib.hot_linear_backward.argtypes = [vp, vp, i32, vp, vp, i64, i64, i64, cfgp, vp, vp, i32, vp, sz,
                                        C.POINTER(C.c_float), vp]
    lib.hot_gemm_splits.restype = i32
    lib.hot_gemm_splits.argtypes = [i64, i64, i64, i32]
    lib.hot_linear_backward_kernels.restype = i32
    lib.hot_linear_backward_kernels.argtypes = lib.hot_linear_backward.argtypes
    lib.hot_gemm_plan.restype = i32
    lib.hot_gemm_plan.argtypes = [i64, i64, i64, i32, i64, i64, sz]
    lib.hot_gemm_workspace_bytes.restype = sz
    lib.hot_gemm_workspace_bytes.argtypes = [i64, i64, i64, i32]
    lib.hot_gemm_i8_variant.restype = i32
    lib.hot_gemm_i8_variant.argtypes = [vp, i64, vp, i64, i32, i64, i64, i64, vp, i32, vp, fp, vp, i32, i64, vp,
                                        i32, vp, sz, vp]
    lib.hot_gemm_bf16.restype = i32
    lib.hot_gemm_bf16.argtypes = [vp, i64, vp, i64, i64, i64, i64, vp, vp, i32, i64, i32, vp]
    lib.hot_hla_tokenwise_static.restype = i32
    lib.hot_hla_tokenwise_static.argtypes = [vp, i32, i64, i64, i32, C.POINTER(C.c_int32), i32, i32, i32, u64, u32,
                                             i32, vp, i64, vp, vp]
    lib.hot_kpad_group.restype = i64
    lib.hot_kpad_group.argtypes = [i64, cfgp]
    lib.hot_abc_batched_workspace_bytes.restype = sz
    lib.hot_abc_batched_workspace_bytes.argtypes = [i64, i64, i64, cfgp]
    lib.hot_abc_forward_batched.restype = i32
    lib.hot_abc_forward_batched.argtypes = [vp, i32, i64, i64, i64, cfgp, vp, vp, vp, sz, vp]
    lib.hot_backward_batched_workspace_bytes.restype = sz
    lib.hot_backward_batched_workspace_bytes.argtypes = [i64, i64, i64, i64, cfgp]
    lib.hot_gx_lowrank_workspace_bytes.restype = sz
    lib.hot_gx_lowrank_workspace_bytes.argtypes = [i64, i64, i64, cfgp]
    lib.hot_gx_lowrank.restype = i32
    lib.hot_gx_lowrank.argtypes = [vp, vp, i32, i64, i64, i64, cfgp, vp, i32, vp, sz, vp]
    lib.hot_gx_luq_workspace_bytes.restype = sz
    lib.hot_gx_luq_workspace_bytes.argtypes = [i64, i64, i64, cfgp]
    lib.hot_gx_luq.restype = i32
    lib.hot_gx_luq.argtypes = [vp, vp, i32, i64, i64, i64, cfgp, vp, i32, vp, sz, vp]
    lib.hot_gw_luq_workspace_bytes.restype = sz
    lib.hot_gw_luq_workspace_bytes.argtypes = [i64, i64, i64, cfgp]
    lib.hot_gw_luq.restype = i32
    lib.hot_gw_luq.argtypes = [vp, i32, vp, vp, i64, i64, i64, cfgp, vp, i32, vp, sz, vp]
    lib.hot_backward_batched_ranges.restype = i32
    lib.hot_backward_batched_ranges.argtypes = [i64, i64, i64, i64, cfgp]
    lib.hot_linear_backward_batched.restype = i32
    lib.hot_linear_backward_batched.argtypes = [vp, vp, i32, vp, vp, i64, i64, i64, i64, cfgp, vp, vp, i32, vp, sz, vp]
    lib.hot_measure_ceilings.restype = i32
    lib.hot_measure_ceilings.argtypes = [vp, sz, C.POINTER(C.c_float), C.POINTER(C.c_float), vp]
    lib.hot_linear_backward_bias.restype = i32
    lib.hot_linear_backward_bias.argtypes = [vp, vp, i32, vp, vp, i64, i64, i64, cfgp, vp, vp, vp, i32, vp, sz, vp]


def lib():
    """The loaded library; raises HotError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HotError(
                "libhot_gfx950.so is missing (%s). Build it with `python -m hot_amd.build`; "
                "there is no fallback path." % LIB_PATH)
        handle = C.CDLL(LIB_PATH)
        for name in EXPORTS:
            if not hasattr(handle, name):
                raise HotError("libhot_gfx950.so does not export %s" % name)
        _declare(handle)
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().hot_last_error()
        raise HotError("libhot_gfx950 error %d: %s" % (rc, msg.decode("utf-8", "replace") if msg else "?"))
