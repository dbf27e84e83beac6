"""ctypes binding of liblpmm_hip.so (the C ABI declared in include/lpmm_hip.h).

There is no fallback: if the library is missing or a call fails, a RuntimeError is raised.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblpmm_hip.so")
MULTI_MAX = 48  # tensors per launch of the fused step (LPMM_MULTI_MAX in include/lpmm_hip.h)
RANK1_SMALL_SLOTS = 8192  # statistics entries of a vector lpmm_rank1_small_fold_scale_multi takes (kNdSmallSlots)
RANK1_SMALL_VALUES = 1 << 16  # longest vector worth the single workgroup that call gives it
RANK1_MULTI_MAX = 32  # tensors per launch of the two-pass rank-1 step (kR1Max in csrc/nonfused_rank1.hip)
SGD_MULTI_MAX = 64  # tensors per launch of the one-pass SGD step (kSgdMax in csrc/sgd.hip)
V4BIT_MULTI_MAX = 48  # tensors per launch of the one-pass step with an fp32 first moment (kV4Max in csrc/nonfused_m32.hip)
ABI_VERSION = 2
CODE_TABLE_BYTES = 12288  # LPMM_CODE_TABLE_BYTES

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_f = ctypes.c_float
_d = ctypes.c_double
_int = ctypes.c_int

# name -> (restype, argtypes); must list every function of include/lpmm_hip.h
PROTOTYPES = {
    "lpmm_status_string": (ctypes.c_char_p, [_int]),
    "lpmm_abi_version": (_int, []),
    "lpmm_adamw4bit_step": (_int, [_vp] * 8 + [_i64] + [_f] * 6 + [_vp]),
    "lpmm_adamw4bit_f16_step": (_int, [_vp] * 8 + [_i64] + [_f] * 6 + [_vp]),
    "lpmm_adamw4bit_step_multi": (_int, [_vp, _i64, _vp, _vp] + [_f] * 5 + [_vp]),
    "lpmm_adamw_fp32_step": (_int, [_vp] * 4 + [_i64] + [_f] * 6 + [_vp]),
    "lpmm_adamw_fp32_step_multi": (_int, [_vp, _i64] + [_f] * 5 + [_vp]),
    "lpmm_adamw_fp16_step_multi": (_int, [_vp, _i64] + [_f] * 5 + [_vp]),
    "lpmm_pack_nonlinear_4bit": (_int, [_vp, _vp, _i64, _vp, _vp]),
    "lpmm_unpack_nonlinear_4bit": (_int, [_vp, _vp, _i64, _vp, _vp]),
    "lpmm_quant_group": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp]),
    "lpmm_dequant_group": (_int, [_vp, _vp, _vp, _i64, _i64, _vp, _vp]),
    "lpmm_rank1_stats": (_int, [_vp, _i64, _i64, _vp, _vp, _vp]),
    "lpmm_quant_rank1": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "lpmm_dequant_rank1": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp, _vp]),
    "lpmm_rank1_stats_nd": (_int, [_vp, _int, _vp, _vp, _vp, _vp]),
    "lpmm_rank1_row_scale_nd": (_int, [_vp, _int, _vp, _vp, _vp]),
    "lpmm_pack_nonlinear": (_int, [_vp, _vp, _int, _i64, _vp, _vp]),
    "lpmm_pack_nonlinear_sr": (_int, [_vp, _vp, _int, _i64, ctypes.c_uint64, ctypes.c_uint64, _vp, _vp]),
    "lpmm_unpack_nonlinear": (_int, [_vp, _vp, _int, _i64, _vp, _vp]),
    "lpmm_quant_group_bits": (_int, [_vp, _i64, _i64, _vp, _int, _vp, _vp, _vp]),
    "lpmm_dequant_group_bits": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _vp, _vp]),
    "lpmm_quant_rank1_bits": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _int, _vp, _vp]),
    "lpmm_code_table_build": (_int, [_vp, _int, _vp, _vp]),
    "lpmm_quant_group_bits_table": (_int, [_vp, _i64, _i64, _vp, _int, _vp, _vp, _vp, _vp]),
    "lpmm_quant_rank1_bits_table": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _int, _vp, _vp, _vp]),
    "lpmm_dequant_rank1_bits": (_int, [_vp, _vp, _vp, _vp, _int, _i64, _i64, _vp, _vp]),
    "lpmm_nonfused_update": (_int, [_vp] * 4 + [_i64] + [_d] * 6 + [_vp]),
    "lpmm_nonfused_update_multi": (_int, [_vp, _i64] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw4bit_step_multi": (_int, [_vp, _i64, _vp, _vp] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw4bit_rank1_step_multi": (_int, [_vp, _i64, _vp, _vp] + [_d] * 5 + [_vp]),
    "lpmm_rank1_small_fold_scale_multi": (_int, [_vp, _i64, _vp]),
    "lpmm_nonfused_adamw4bit_f16_step_multi": (_int, [_vp, _i64, _vp, _vp] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw4bit_rank1_f16_step_multi": (_int, [_vp, _i64, _vp, _vp] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw4bit_rank1_pass_multi": (_int, [_vp, _i64, _vp, _vp] + [_d] * 5 + [_int, _vp]),
    "lpmm_nonfused_adamw_v4bit_step_multi": (_int, [_vp, _i64, _vp] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw_v4bit_rank1_step_multi": (_int, [_vp, _i64, _vp] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw4bit_rank1_mgroup_step_multi": (_int, [_vp, _i64, _vp, _vp, _i64] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw_bits_rank1_step_multi": (_int, [_vp, _i64, _vp, _int, _vp, _int] + [_d] * 5 + [_vp]),
    "lpmm_nonfused_adamw_bits_rank1_step_multi_table": (_int, [_vp, _i64, _vp, _int, _vp, _vp, _int, _vp] + [_d] * 5 + [_vp]),
    "lpmm_factored_workspace_bytes": (_i64, [_i64, _i64]),
    "lpmm_factored_stats": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _d, _vp, _vp]),
    "lpmm_factored_stats_static": (_int, [_vp, _i64, _i64, _vp, _vp, _vp, _d, _vp]),
    "lpmm_factored_update": (_int, [_vp] * 8 + [_i64, _i64] + [_d] * 6 + [_int, _vp]),
    "lpmm_factored_step_multi": (_int, [_vp, _i64, _vp] + [_d] * 5 + [_vp]),
    "lpmm_factored_update_fp32m": (_int, [_vp] * 6 + [_i64, _i64] + [_d] * 6 + [_vp]),
    "lpmm_sgd4bit_step_multi": (_int, [_vp, _i64, _vp] + [_d] * 4 + [_int, _int, _vp]),
    "lpmm_stream_probe": (_int, [_int] + [_vp] * 6 + [_i64, _i64, _vp]),
    "lpmm_selftest_encoders": (_int, [_vp, _vp]),
    "lpmm_selftest_bucket_encoder": (_int, [_vp, _int, _vp, _vp]),
    "lpmm_selftest_arithmetic": (_int, [_vp, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_uint32, _vp]),
}

# numpy mirrors of the multi-tensor records (lpmm_adamw4bit_tensor / lpmm_adamw_fp32_tensor)
ADAMW4BIT_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("v_codes", "<u8"),
                             ("m_scale", "<u8"), ("v_scale", "<u8"), ("n", "<i8"), ("step", "<f4"),
                             ("reserved", "<f4")])
NONFUSED_RANK1_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("m_max1", "<u8"),
                                  ("v_codes", "<u8"), ("v_rowmax", "<u8"), ("v_colmax", "<u8"),
                                  ("v_rowmax_next", "<u8"), ("v_colmax_next", "<u8"), ("rows", "<i8"),
                                  ("cols", "<i8"), ("step", "<f4"), ("reserved", "<f4")])
# float16 parameters: the one-pass record is ADAMW4BIT_TENSOR with half p, g and scales
NONFUSED_RANK1_F16_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("m_max1", "<u8"),
                                      ("v_codes", "<u8"), ("v_rowmax", "<u8"), ("v_colmax", "<u8"),
                                      ("v_rowmax_next", "<u8"), ("v_colmax_next", "<u8"), ("work", "<u8"),
                                      ("rows", "<i8"), ("cols", "<i8"), ("step", "<f4"), ("reserved", "<f4")])
RANK1_SMALL_VECTOR = np.dtype([("x", "<u8"), ("scale", "<u8"), ("stats", "<u8", (7,)), ("shape", "<i8", (7,)),
                               ("ndim", "<i4"), ("reserved", "<i4")])
ADAMW_V4BIT_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m", "<u8"), ("v_codes", "<u8"), ("v_max1", "<u8"),
                               ("n", "<i8"), ("step", "<f4"), ("reserved", "<f4")])
RANK1_V4BIT_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m", "<u8"), ("v_codes", "<u8"), ("v_rowmax", "<u8"),
                               ("v_colmax", "<u8"), ("v_rowmax_next", "<u8"), ("v_colmax_next", "<u8"),
                               ("rows", "<i8"), ("cols", "<i8"), ("step", "<f4"), ("reserved", "<f4")])
RANK1_MGROUP_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("m_max1", "<u8"),
                                ("m_max1_next", "<u8"), ("v_codes", "<u8"), ("v_rowmax", "<u8"), ("v_colmax", "<u8"),
                                ("v_rowmax_next", "<u8"), ("v_colmax_next", "<u8"), ("rows", "<i8"), ("cols", "<i8"),
                                ("step", "<f4"), ("reserved", "<f4")])
FACTORED_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("m_max1", "<u8"), ("row", "<u8"),
                            ("col", "<u8"), ("workspace", "<u8"), ("rows", "<i8"), ("cols", "<i8"), ("step", "<f4"),
                            ("first_step", "<i4")])
SGD4BIT_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m_codes", "<u8"), ("m_max1", "<u8"), ("n", "<i8"),
                           ("first_step", "<i4"), ("reserved", "<i4")])
ADAMW_FP32_TENSOR = np.dtype([("p", "<u8"), ("g", "<u8"), ("m", "<u8"), ("v", "<u8"), ("n", "<i8"),
                              ("step", "<f4"), ("reserved", "<f4")])

_lib = None


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"lpmm: {LIB_PATH} is missing. Build it with `make -C low-bit-optimizers_amd/csrc` "
                "(hipcc, gfx950). There is no CPU or PyTorch fallback for the quantised optimizer path.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        if handle.lpmm_abi_version() != ABI_VERSION:
            raise RuntimeError("lpmm: liblpmm_hip.so has ABI version "
                               f"{handle.lpmm_abi_version()}, expected {ABI_VERSION}; rebuild it")
        _lib = handle
    return _lib


def check(status, what):
    if status != 0:
        msg = lib().lpmm_status_string(status).decode()
        raise RuntimeError(f"lpmm: {what} failed: {msg} (status {status})")


def current_stream(device):
    import torch

    return torch.cuda.current_stream(device).cuda_stream
