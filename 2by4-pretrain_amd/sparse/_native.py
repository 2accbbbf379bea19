"""ctypes binding of lib2by4_gfx950.so (C ABI declared in include/tf24.h).

There is no fallback: if the library is missing or a call fails, a RuntimeError is raised.
Every wrapper enqueues on torch's current HIP stream and passes raw device pointers.
"""
import ctypes
import os

import torch

_LIB_NAME = "lib2by4_gfx950.so"
_lib = None

# enums of tf24.h
F32, F16, BF16, E4M3, U8, E5M2, I8, I32 = 0, 1, 2, 3, 4, 5, 6, 7
ROW_MAJOR, COL_MAJOR = 0, 1
PRUNE_MAGNITUDE, PRUNE_MASK, PRUNE_MVUE, PRUNE_MVUE_PACKED, PRUNE_MVUE_SEEDED, PRUNE_MVUE_SEEDED_DEVICE = 0, 1, 2, 3, 4, 5
ACT_NONE, ACT_RELU, ACT_SILU, ACT_GELU = 0, 1, 2, 3
COMPRESSED_CANONICAL, COMPRESSED_PANEL, COMPRESSED_CUTLASS = 0, 1, 2

_DTYPES = {
    torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float8_e4m3fn: E4M3, torch.float8_e5m2: E5M2,
    torch.uint8: U8, torch.bool: U8, torch.int8: U8,
}

_i = ctypes.c_int
_i64 = ctypes.c_int64
_p = ctypes.c_void_p
_f = ctypes.c_float
_d = ctypes.c_double

_SIGNATURES = {
    "tf24_version": (ctypes.c_char_p, []),
    "tf24_last_error": (ctypes.c_char_p, []),
    "tf24_prune_compress": (_i, [_p, _i, _i, _i64, _i64, _i64, _i, _p, _i, _i64, _p, _i64, _p, _i, _p, _i, _p]),
    "tf24_prune_compress_validate": (_i, [_i, _i, _i64, _i64, _i64, _i, _i, _i, _i64, _i, _i64, _i]),
    "tf24_mvue_uniforms": (_i, [ctypes.c_uint64, ctypes.c_uint64, _i64, _i64, _i, _p, _i64, _p]),
    "tf24_prune_compress_rowsum": (_i, [_p, _i, _i, _i64, _i64, _i64, _i, _p, _i, _i64, _p, _i64, _p, _i, _p, _i, _p, _i, _p, _i64, _p]),
    "tf24_prune_compress_rowsum_workspace_bytes": (_i64, [_i64, _i64]),
    "tf24_prune_compress_rowsum_static": (_i, [_p, _i, _i, _i64, _i64, _i64, _i, _p, _i, _i64, _p, _i64, _p, _i, _p, _i, _p, _i, _p]),
    "tf24_prune_compress_rowsum_static_max_bytes": (_i64, []),
    "tf24_prune_compress_dual": (_i, [_p, _i, _i64, _i64, _i64, _p, _i, _i64, _p, _p, _p, _p, _i, _i, _p]),
    "tf24_prune_compress_dual_validate": (_i, [_i, _i64, _i64, _i64, _i, _i64, _i, _i]),
    "tf24_decompress": (_i, [_p, _i, _p, _i, _i64, _i64, _p, _p]),
    "tf24_repack": (_i, [_p, _p, _i, _i64, _i64, _i, _p, _p, _p]),
    "tf24_repack_to": (_i, [_p, _p, _i, _i64, _i64, _i, _i, _p, _p, _p]),
    "tf24_transposable_mask": (_i, [_p, _i, _i, _i64, _i64, _i64, _i, _p, _p, _p]),
    "tf24_transposable_mask_validate": (_i, [_i, _i, _i64, _i64, _i64]),
    "tf24_soft_threshold24": (_i, [_p, _i, _i, _i64, _i64, _i64, _p, _p, _p]),
    "tf24_sparse24_dense": (_i, [_p, _i, _i, _i64, _i64, _i64, _p, _p, _p]),
    "tf24_mvue24_dense": (_i, [_p, _i, _i, _i64, _i64, _i64, _p, _i64, _p, _p]),
    "tf24_masked_add": (_i, [_p, _i, _p, _i, _p, _i, _i64, _f, _p]),
    "tf24_adamw_masked_decay": (_i, [_p, _p, _i, _p, _p, _p, _i, _i64, _d, _d, _d, _d, _d, _d, _i64, _p]),
    "tf24_adamw_masked_decay_device_step": (_i, [_p, _p, _i, _p, _p, _p, _i, _i64, _d, _d, _d, _d, _d, _d, _p, _p]),
    "tf24_gelu_glu_forward": (_i, [_p, _i, _i, _i64, _i64, _i64, _p, _i64, _p]),
    "tf24_gelu_glu_backward": (_i, [_p, _i64, _p, _i, _i, _i64, _i64, _i64, _p, _i64, _p]),
    "tf24_adamw_step": (_i, [_p, _p, _i, _p, _p, _p, _p, _i64, _d, _d, _d, _d, _d, _i64, _p, _i, _p]),
    "tf24_adamw_step_partials": (_i64, [_i64]),
    "tf24_spmm": (_i, [_p, _p, _i, _i, _i64, _i64, _p, _i, _i64, _i64, _p, _i, _i, _i64, _p, _f, _i, _p, _i64, _p]),
    "tf24_spmm_workspace_bytes": (_i64, [_i, _i64, _i64, _i64]),
    "tf24_transpose": (_i, [_p, _i, _i64, _i64, _i64, _p, _i64, _p]),
    "tf24_spmm_validate": (_i, [_i, _i64, _i64, _i, _i64, _i64, _i, _i, _i64, _i]),
}


def library_path():
    return os.path.join(os.path.dirname(os.path.abspath(__file__)), _LIB_NAME)


def lib():
    """The loaded library; raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        path = library_path()
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} not found: build it with `python 2by4-pretrain_amd/build.py` "
                "(there is no fallback implementation)")
        handle = ctypes.CDLL(path)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)          # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def version():
    return lib().tf24_version().decode()


def dtype_code(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise RuntimeError(f"dtype {dtype} is not supported by the gfx950 2:4 library") from None


def operand_code(dtype):
    """dtype code of a matrix of values: like dtype_code, except that int8 / int32 are the integer
    value types (dtype_code reads int8 as a byte mask)."""
    if dtype == torch.int8:
        return I8
    if dtype == torch.int32:
        return I32
    return dtype_code(dtype)


def check(rc):
    if rc != 0:
        raise RuntimeError(lib().tf24_last_error().decode() or f"tf24 call failed with code {rc}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr():
    """The current HIP stream of the current device as an integer handle.  The raw accessor avoids
    building a torch.cuda.Stream object per call (about 12 us each, eight calls per training step)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def layout_of(t):
    """(layout, ld) of a 2-d tensor that is dense in one of its two dimensions, else None."""
    m, k = t.shape
    s0, s1 = t.stride()
    if s1 == 1 and s0 >= k:
        return ROW_MAJOR, s0
    if s0 == 1 and s1 >= m:
        return COL_MAJOR, s1
    return None


def as_matrix(t, like=None):
    """t itself when the kernels can address it (row- or column-major, 16-byte aligned, leading
    dimension a multiple of 8), otherwise a copy; with `like`, a copy laid out like that tensor."""
    if like is not None:
        lay = layout_of(like)
        mine = layout_of(t)
        if mine is None or mine[0] != lay[0] or t.data_ptr() % 16 or mine[1] % 8:
            out = torch.empty_strided(t.shape, like.stride(), dtype=t.dtype, device=t.device)
            out.copy_(t)
            return out
        return t
    lay = layout_of(t)
    if lay is None or t.data_ptr() % 16 or lay[1] % 8:
        return t.contiguous()
    return t


def ptr(t):
    return None if t is None else t.data_ptr()


def transposed_copy(t):
    """Row-major [cols, rows] copy of the 2-d row-major tensor t [rows, cols] (HIP tile transpose)."""
    rows, cols = t.shape
    out = torch.empty((cols, rows), dtype=t.dtype, device=t.device)
    check(lib().tf24_transpose(t.data_ptr(), dtype_code(t.dtype), t.stride(0), rows, cols, out.data_ptr(), rows, stream_ptr()))
    return out
