"""ctypes binding of libw4a16_hip.so (declared in include/w4a16.h)."""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(os.path.dirname(_HERE), "lib", "libw4a16_hip.so")

OK = 0
ERR_NULL, ERR_SHAPE, ERR_GROUP, ERR_ALIGN, ERR_WORKSPACE, ERR_HIP, ERR_TUNE, ERR_TIMEOUT, ERR_TOO_LARGE, ERR_NOT_PREPARED = -1, -2, -3, -4, -5, -6, -7, -8, -9, -10

# every symbol include/w4a16.h declares: name -> (restype, argtypes)
_vp, _ci, _sz, _cf = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_float
SYMBOLS = {
    "w4a16_abi_version": (_ci, []),
    "w4a16_strerror": (ctypes.c_char_p, [_ci]),
    "w4a16_last_hip_error": (ctypes.c_char_p, []),
    "awq_dequant_bf16": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "awq_dequant_1d_tile_bytes": (_sz, [_ci, _ci, _ci]),
    "awq_dequant_1d_bf16": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_gemm_workspace_bytes": (_sz, [_ci, _ci, _ci]),
    "w4a16_ffn_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a16_workspace_init": (_ci, [_vp, _sz, _vp]),
    "w4a16_workspace_check": (_ci, [_vp, _vp]),
    "w4a16_gemv_bf16": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_gemm_bf16": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_gemv_swiglu_bf16": (_ci, [_vp] * 8 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_ffn_swiglu_bf16": (_ci, [_vp] * 12 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_gemv_add_bf16": (_ci, [_vp] * 6 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_rms_gemv_bf16": (_ci, [_vp, _vp, _cf] + [_vp] * 4 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_rms_gemv_swiglu_bf16": (_ci, [_vp, _vp, _cf] + [_vp] * 7 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_block_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a16_o_gemv_ffn_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 15 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_attention_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a16_decode_attention_bf16": (_ci, [_vp] * 5 + [_ci] * 5 + [_vp, _sz, _vp]),
    "w4a16_prefill_block_workspace_bytes": (_sz, [_ci, _ci, _ci]),
    "rms_norm_rows_bf16": (_ci, [_vp, _vp, _cf, _vp, _ci, _ci, _vp]),
    "w4a16_prefill_o_ffn_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 15 + [_ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_prefill_qkv_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a16_prefill_rms_qkv_rope_bf16": (_ci, [_vp, _vp, _cf, _vp, _vp, _vp, _vp, _ci, _ci, _vp] + [_ci] * 6 + [_vp, _sz, _vp]),
    "w4a16_prefill_rms_qkv_rope_stream_bf16": (_ci, [_vp, _vp, _cf, _vp, _vp, _ci, _ci, _vp] + [_ci] * 6 + [_vp, _sz, _vp]),
    "w4a16_prefill_o_ffn_stream_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 7 + [_ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_q4nx_prefill_rms_qkv_rope_stream_bf16": (_ci, [_vp, _vp, _cf, _vp, _vp, _ci, _ci, _vp] + [_ci] * 5 + [_vp, _sz, _vp]),
    "w4a16_q4nx_prefill_o_ffn_stream_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 7 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_prefill_attention_bf16": (_ci, [_vp, _vp, _ci, _ci, _ci, _ci, _vp]),
    "lm_head_workspace_bytes": (_sz, [_ci]),
    "w4a16_decode_attn_o_gemv_ffn_bf16": (_ci, [_vp] * 5 + [_ci] * 5 + [_vp, _sz, _vp, _vp, _cf] + [_vp] * 12 + [_vp, _vp, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_rms_gemv_sumsq_bf16": (_ci, [_vp, _vp, _ci, _vp, _cf, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp, _sz, _vp]),
    "rope_halfsplit_bf16": (_ci, [_vp, _vp, _vp, _ci, _ci, _vp]),
    "lm_head_gemv_bf16": (_ci, [_vp, _vp, _cf, _vp, _vp, _vp, _ci, _ci, _vp, _sz, _vp]),
    "q4nx_dequant_bf16": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp]),
    "q4nx_repack": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_q4nx_stream_bytes": (_sz, [_ci, _ci]),
    "w4a16_q4nx_blocks_to_stream": (_ci, [_vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_q4nx_repack_stream": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _vp]),
    "w4a16_q4nx_gemv_stream_bf16": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _vp]),
    "w4a16_q4nx_gemm_stream_bf16": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_q4nx_rms_gemv_stream_bf16": (_ci, [_vp, _vp, _ci, _vp, _cf, _vp, _vp, _ci, _ci, _vp]),
    "w4a16_q4nx_o_gemv_ffn_stream_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 8 + [_ci, _ci, _vp, _sz, _vp]),
    "w4a16_stream_bytes": (_sz, [_ci, _ci]),
    "w4a16_repack_stream": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_gemv_stream_bf16": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_probe_stream_read": (_ci, [_vp, _vp, _ci, _ci, _vp]),
    "w4a16_gemm_stream_bf16": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp]),
    "w4a16_gemm_stream_scratch_bytes": (_sz, [_ci, _ci, _ci]),
    "w4a16_gemm_stream_scratch_bf16": (_ci, [_vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_gemv_add_stream_bf16": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_gemv_swiglu_stream_bf16": (_ci, [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_rms_gemv_stream_bf16": (_ci, [_vp, _vp, _ci, _vp, _cf, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_rms_gemv_swiglu_stream_bf16": (_ci, [_vp, _vp, _cf, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_ffn_swiglu_stream_bf16": (_ci, [_vp] * 6 + [_ci, _ci, _ci, _vp]),
    "w4a16_block_stream_workspace_bytes": (_sz, [_ci, _ci]),
    "w4a16_o_gemv_ffn_stream_bf16": (_ci, [_vp, _vp, _vp, _cf] + [_vp] * 8 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_decode_attn_o_gemv_ffn_stream_bf16": (_ci, [_vp] * 5 + [_ci] * 5 + [_vp, _sz, _vp, _vp, _cf] + [_vp] * 6 + [_ci, _ci, _ci, _vp, _sz, _vp]),
    "w4a16_gemv_noalloc_bf16": (_ci, [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp]),
    "w4a16_noalloc_check": (_ci, [_vp]),
    "w4a16_tune": (_ci, [ctypes.c_char_p, _ci]),
}


class LibraryNotBuiltError(RuntimeError):
    pass


class W4A16Error(RuntimeError):
    """A C-ABI call returned a negative code."""

    def __init__(self, code, message):
        super().__init__(f"w4a16 error {code}: {message}")
        self.code = code


_lib = None


def library_path():
    return _LIB_PATH


def load_library():
    """Load the HIP library; raises LibraryNotBuiltError when it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise LibraryNotBuiltError(
            f"{_LIB_PATH} is missing: build it with `python mlir-air_amd/build.py` "
            "(there is no CPU fallback for the W4A16 kernels)"
        )
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.w4a16_abi_version() != 1:
        raise LibraryNotBuiltError(f"{_LIB_PATH}: ABI version {lib.w4a16_abi_version()} != 1, rebuild")
    _lib = lib
    return lib


def check(code):
    """Raise W4A16Error for a negative return code."""
    if code != OK:
        lib = load_library()
        msg = lib.w4a16_strerror(code).decode()
        if code == ERR_HIP:
            msg += ": " + lib.w4a16_last_hip_error().decode()
        raise W4A16Error(code, msg)
