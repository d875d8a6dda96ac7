"""ctypes binding of ``libfourier_attn_hip.so`` (the C ABI in ``include/fourier_attn_hip.h``).

There is no fallback: if the shared library is missing or a call fails, an exception is
raised.  Build it with ``python -m fourierattention_amd.build``.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libfourier_attn_hip.so")

FA_BF16, FA_FP16, FA_FP32 = 0, 1, 2
FA_NO_ROUND = FA_FP32
FA_MID_TOKEN_MAJOR, FA_MID_PAGED = 0, 1
FA_COLS_ANY, FA_COLS_HEAD_DIMS = 0, 1
DECODE_NOALLOC_SCRATCH_BYTES = 32 << 20
PAGE_TOKENS, K_DIM_PAD, V_DIM_PAD = 32, 32, 16

STATUS_NAMES = {
    0: "FA_OK", -1: "FA_ERR_NULL_POINTER", -2: "FA_ERR_BAD_SHAPE", -3: "FA_ERR_BAD_DTYPE", -4: "FA_ERR_WORKSPACE",
    -5: "FA_ERR_UNSUPPORTED", -6: "FA_ERR_LAUNCH", -7: "FA_ERR_MISALIGNED",
}


class FourierAttnError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"{STATUS_NAMES.get(code, code)}: {message}")
        self.code = code


class DecodeArgs(ctypes.Structure):
    """Mirror of ``fa_decode_args``."""
    _fields_ = [
        ("q", c_void_p),
        ("k_il", c_void_p * 2), ("v_il", c_void_p * 2),
        ("il_rows", c_int32 * 2), ("il_batch_stride", c_int64 * 2), ("il_row_stride", c_int64 * 2),
        ("k_mc", c_void_p), ("v_mc", c_void_p),
        ("k_mn", c_void_p), ("v_mn", c_void_p),
        ("k_mn_batch_stride", c_int64), ("k_mn_row_stride", c_int64),
        ("v_mn_batch_stride", c_int64), ("v_mn_row_stride", c_int64),
        ("mid_layout", c_int32), ("mid_cap_pages", c_int32),
        ("k_pad_h_list", c_void_p), ("v_pad_h_list", c_void_p),
        ("mid_max_k_pad", c_int32), ("mid_max_v_pad", c_int32),
        ("k_pad_h_host", c_void_p), ("v_pad_h_host", c_void_p),
        ("tables", c_void_p), ("force_generic", c_int32),
        ("avg_k_u", c_void_p), ("avg_k_d", c_void_p), ("scale_k", c_void_p),
        ("avg_v_u", c_void_p), ("avg_v_d", c_void_p), ("scale_v", c_void_p),
        ("kc_list", c_void_p), ("kc_h_list", c_void_p), ("kn_list", c_void_p), ("kn_h_list", c_void_p),
        ("vc_list", c_void_p), ("vc_h_list", c_void_p), ("vn_list", c_void_p), ("vn_h_list", c_void_p),
        ("Ck", c_int32), ("Cnk", c_int32), ("Cv", c_int32), ("Cnv", c_int32),
        ("out", c_void_p), ("out_cast", c_void_p),
        ("B", c_int32), ("Hq", c_int32), ("Hkv", c_int32), ("D", c_int32),
        ("q_len", c_int32), ("N", c_int32), ("L_m", c_int32), ("T", c_int32),
        ("sm_scale", c_float), ("dtype", c_int32),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("no_fuse", c_int32),
        ("upd_k_row", c_void_p), ("upd_v_row", c_void_p), ("upd_batch_stride", c_int64), ("upd_phase", c_int64),
        ("upd_T", c_int32),
    ]


class StreamArgs(ctypes.Structure):
    """Mirror of ``fa_stream_args``."""
    _fields_ = [
        ("k_new", c_void_p), ("v_new", c_void_p), ("new_batch_stride", c_int64),
        ("k_ring", c_void_p), ("v_ring", c_void_p), ("ring_batch_stride", c_int64), ("ring_row_stride", c_int64),
        ("evict_slot", c_int32), ("write_slot", c_int32),
        ("k_coef", c_void_p), ("v_coef", c_void_p), ("kc_list", c_void_p), ("vc_list", c_void_p),
        ("Ck", c_int32), ("Cv", c_int32), ("N", c_int32), ("T", c_int32), ("phase", c_int64),
        ("k_mid", c_void_p), ("v_mid", c_void_p), ("k_mid_batch_stride", c_int64), ("v_mid_batch_stride", c_int64),
        ("cap_pages", c_int32), ("mid_pos", c_int64),
        ("kn_list", c_void_p), ("kn_h_list", c_void_p), ("k_pad_h_list", c_void_p),
        ("vn_list", c_void_p), ("vn_h_list", c_void_p), ("v_pad_h_list", c_void_p),
        ("Cnk", c_int32), ("Cnv", c_int32), ("B", c_int32), ("Hkv", c_int32), ("width", c_int32), ("dtype", c_int32),
        ("skip_coef", c_int32),
    ]


_SIGNATURES = {
    "fa_last_error_string": (c_char_p, []),
    "fa_abi_version": (c_int, []),
    "fa_decode_args_size": (c_size_t, []),
    "fa_stream_args_size": (c_size_t, []),
    "fa_stream_update": (c_int, [ctypes.POINTER(StreamArgs), c_void_p]),
    "fa_mat_fourier": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                               c_int64, c_int, c_void_p, c_size_t, c_void_p]),
    "fa_mat_fourier_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "fa_mat_avg_std": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                               c_int, c_void_p, c_size_t, c_void_p]),
    "fa_mat_fourier_avg_std": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                       c_size_t, c_void_p]),
    "fa_stats_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "fa_mat_fourier_avg_std_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fa_reconstruct": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                               c_void_p]),
    "fa_coeff_update": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_void_p, c_int, c_int, c_int, c_int64, c_int,
                                c_void_p]),
    "fa_decode_attn_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "fa_decode_attn": (c_int, [POINTER(DecodeArgs), c_void_p]),
    "fa_decode_attn_noalloc": (c_int, [POINTER(DecodeArgs), c_void_p]),
    "fa_decode_attn_timed": (c_int, [POINTER(DecodeArgs), c_void_p, POINTER(c_float)]),
    "fa_decode_attn_last_fused": (c_int, []),
    "fa_linear_pack": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "fa_linear_packed_ok": (c_int, [c_int, c_int, c_int]),
    "fa_linear_packed": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "fa_decode_split_plan": (c_int, [c_int] * 7 + [c_void_p, c_void_p, c_void_p, c_void_p]),
    "fa_decode_tables_bytes": (c_size_t, [c_int]),
    "fa_decode_tables_build": (c_int, [c_void_p, c_size_t, c_int, c_int, c_void_p]),
    "fa_mid_pack": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_void_p, c_int64, c_int, c_void_p, c_void_p,
                            c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "fa_prefill_compress_ok": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "fa_prefill_compress_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "fa_prefill_compress": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_int64, c_int,
                                    c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                                    c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "fa_mid_append": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                              c_int, c_int, c_int, c_int, c_void_p]),
    "fa_mid_unpack": (c_int, [c_void_p, c_int, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                              c_int, c_int, c_void_p]),
    "fa_prefill_attn_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "fa_prefill_attn": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int,
                                c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_size_t, c_void_p]),
    "fa_add_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_float, c_int, c_void_p]),
    "fa_rope_qk": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                           c_int, c_void_p]),
    "fa_silu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int64, c_int, c_void_p]),
}

EXPORTED = tuple(_SIGNATURES)

# bumped with every change of a prototype or of an argument struct (fa_abi_version in the library)
ABI_VERSION = 3

_lib = None


def load():
    """Load the shared library once; raise if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing - the HIP extension is not built (run `python -m fourierattention_amd.build`); "
            "there is no CPU fallback")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    if lib.fa_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI version {lib.fa_abi_version()}, this binding was written for {ABI_VERSION}: "
                          "rebuild the library (`python -m fourierattention_amd.build`)")
    if lib.fa_stream_args_size() != ctypes.sizeof(StreamArgs):
        raise ImportError(f"fa_stream_args is {lib.fa_stream_args_size()} bytes in the library but "
                          f"{ctypes.sizeof(StreamArgs)} in the Python mirror")
    if lib.fa_decode_args_size() != ctypes.sizeof(DecodeArgs):
        raise ImportError(f"fa_decode_args is {lib.fa_decode_args_size()} bytes in the library but "
                          f"{ctypes.sizeof(DecodeArgs)} in the binding")
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != 0:
        raise FourierAttnError(code, load().fa_last_error_string().decode("utf-8", "replace"))
