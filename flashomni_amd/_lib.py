"""ctypes binding of the C-ABI library (include/flashomni_hip.h).

The library is the only compute path: if it is missing or does not load, every op raises.
There is no CPU or eager fallback.
"""
import ctypes
import os

from .build import LIB_PATH

_lib = None

c_i32, c_i64, c_u32, c_f32 = ctypes.c_int32, ctypes.c_int64, ctypes.c_uint32, ctypes.c_float
c_vp, c_sz, c_int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int

# name -> argument types, exactly as declared in include/flashomni_hip.h
SIGNATURES = {
    "fo_last_error": ([], ctypes.c_char_p),
    "fo_abi_version": ([], c_int),
    "fo_num_cu": ([], c_int),
    "fo_packbits": ([c_vp, c_i64, c_int, c_vp, c_vp], c_int),
    "fo_segment_packbits": ([c_vp, c_vp, c_vp, c_i32, c_int, c_vp, c_vp], c_int),
    "fo_prefill_plan": ([c_vp, c_sz, c_vp, c_vp, c_sz, c_vp, c_vp, c_u32, c_u32, c_u32, c_u32,
                         c_u32, c_u32, c_u32, c_int, c_u32, c_int, c_vp, c_vp], c_int),
    "fo_sparse_block_table": ([c_vp, c_u32, c_u32, c_vp, c_vp, c_i64, c_vp], c_int),
    "fo_decode_sizes": ([c_vp, c_vp, c_u32, c_u32, c_u32, c_u32, c_vp, c_vp, c_vp], c_int),
    "fo_decode_sparse": ([c_vp] * 7 + [c_i32, c_i32, c_i32, c_int] + [c_vp] * 9 + [c_vp, c_vp], c_int),
    "fo_decode_sparse_static_max_pairs": ([], c_i64),
    "fo_decode_sparse_static": ([c_vp] * 7 + [c_i32, c_i32, c_i32, c_int] + [c_vp] * 8 + [c_vp, c_vp], c_int),
    "fo_sparse_fa_split_workspace_bytes": ([], c_i64),
    "fo_sparse_fa_set_variant": ([c_int], c_int),
    "fo_sparse_fa_run": ([c_vp] * 5 + [c_int, c_vp, c_vp, c_vp, c_vp] + [c_i64] * 8 + [c_vp] * 4 + [c_i32, c_i32]
                         + [c_vp] * 7 + [c_i64, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_f32, c_f32, c_vp, c_vp, c_i64, c_vp],
                         c_int),
    "fo_gemm_workspace_bytes": ([c_i32, c_i32, c_i32], c_i64),
    "fo_gemm_q": ([c_vp] * 4 + [c_int] + [c_i32] * 6 + [c_vp, c_vp, c_i32, c_int, c_vp, c_i64, c_vp],
                  c_int),
    "fo_gemm_q_quant": ([c_vp] * 7 + [c_int] + [c_i32] * 6 + [c_vp, c_vp, c_i32, c_int, c_vp, c_i64, c_vp],
                        c_int),
    "fo_gemm_o": ([c_vp] * 4 + [c_int] * 4 + [c_i32] * 6 + [c_vp, c_vp, c_i32, c_int, c_vp, c_i64, c_vp],
                  c_int),
    "fo_quant_fp8_block": ([c_vp, c_int, c_i64, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_i32, c_i32, c_i32,
                            c_vp], c_int),
    "fo_symbols_from_scores": ([c_vp, c_int] + [c_i32] * 6 + [c_vp] * 7, c_int),
}

FO_BF16, FO_F16, FO_FP8_E4M3, FO_F32 = 0, 1, 2, 3
FO_BIAS_NONE, FO_BIAS_VECTOR, FO_BIAS_MATRIX = 0, 1, 2


def lib():
    """Load (once) and return the library; raises RuntimeError when it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "flashomni_amd: %s is missing; build it with `python -m flashomni_amd.build` "
                "(there is no fallback path)" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (argtypes, restype) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = handle
    return _lib


def check(rc):
    """Turn a negative return code into RuntimeError carrying the library's message
    (the reference's TORCH_CHECK failures surface as RuntimeError too)."""
    if rc != 0:
        raise RuntimeError(lib().fo_last_error().decode())


def ptr(t):
    """Device/host address of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


def dtype_code(dtype):
    import torch
    table = {torch.bfloat16: FO_BF16, torch.float16: FO_F16, torch.float8_e4m3fn: FO_FP8_E4M3,
             torch.float32: FO_F32}
    if dtype not in table:
        raise ValueError("unsupported dtype %s" % dtype)
    return table[dtype]


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def device_guard(device):
    """Context that makes ``device`` the current one for the library call inside it (the library
    launches on, and asks the properties of, the current device).  Costs nothing when it already is."""
    import torch
    if device.index is None or torch.cuda.current_device() == device.index:
        return _NO_GUARD
    return torch.cuda.device(device)


def current_stream(device):
    import torch
    return torch.cuda.current_stream(device).cuda_stream
