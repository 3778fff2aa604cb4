"""ctypes binding of libmoe_hip.so (C ABI: ``include/moe_hip.h``).

The library is loaded on first use, after ``torch`` so that it binds to the HIP
runtime already in the process.  There is no fallback: if the library is missing
or a call fails, the caller gets an exception.
"""
import ctypes
import os

import torch

# MOE_HIP_LIB points at another build of the same library (kernel experiments)
_LIB_PATH = os.environ.get("MOE_HIP_LIB") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "libmoe_hip.so")
_lib = None

# enums of include/moe_hip.h
DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
ACT_NONE, ACT_SILU, ACT_GELU, ACT_APPROX_GELU, ACT_SWIGLU, ACT_GEGLU = range(6)
GEMM_GATHER_A, GEMM_SCATTER_C, GEMM_SCATTER_ADD, GEMM_SAVE_PREACT = 1, 2, 4, 8
KGEMM_GATHER_A, KGEMM_GATHER_B, KGEMM_A_KMAJOR, KGEMM_B_KMAJOR = 1, 2, 4, 8
FP8_W_TILED = 4  # moe_m_grouped_gemm_fp8 only: weights stored tile-major
ROUTER_SOFTMAX_FIRST, ROUTER_NORMALIZE, ROUTER_ERNIE = 1, 2, 4

_DTYPES = {torch.float32: DTYPE_F32, torch.float16: DTYPE_F16, torch.bfloat16: DTYPE_BF16}
_ACTS = {
    None: ACT_NONE,
    "none": ACT_NONE,
    "silu": ACT_SILU,
    "gelu": ACT_GELU,
    "approx_gelu": ACT_APPROX_GELU,
    "swiglu": ACT_SWIGLU,
    "geglu": ACT_GEGLU,
}

_vp, _i64, _i32, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t

# name -> (restype, argtypes); every symbol of include/moe_hip.h
SIGNATURES = {
    "moe_version": (_i32, []),
    "moe_last_error_string": (ctypes.c_char_p, []),
    "moe_route_workspace_bytes": (_sz, [_i64, _i32]),
    "moe_route_preprocess": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _vp, _vp, _sz, _vp]),
    "moe_route_noalloc_max_bytes": (_sz, []),
    "moe_route_preprocess_noalloc": (_i32, [_vp, _i32, _i64, _i32, _vp, _vp, _vp, _vp]),
    "moe_row_gather": (_i32, [_vp, _i64, _i64, _vp, _i32, _i32, _vp, _i64, _i64, _i64, _i32, _vp]),
    "moe_row_scatter": (_i32, [_vp, _i64, _vp, _i32, _vp, _i64, _i64, _i64, _i64, _i32, _vp]),
    "moe_scale_and_reduce": (_i32, [_vp, _i64, _vp, _vp, _i64, _i64, _i32, _i64, _i32, _i32, _i64, _vp]),
    "moe_cast_from_f32": (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _i32, _vp]),
    "moe_m_grouped_gemm": (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _i64, _vp, _i64,
                                  _vp, _vp, _i32, _vp, _i32, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i64, _vp]),
    "moe_k_grouped_gemm": (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _i32, _i32, _i64,
                                  _i64, _i32, _i32, _i32, _vp]),
    "moe_kmajor_columns": (_i64, [_i64, _i32]),
    "moe_row_gather_kmajor": (_i32, [_vp, _i64, _i64, _vp, _i32, _i32, _vp, _i32, _i64, _vp, _i64, _i64,
                                     _i32, _vp]),
    "moe_act_bwd": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _vp, _vp, _i32, _vp, _i64, _vp, _i64,
                           _i64, _i32, _i32, _vp]),
    "moe_m_grouped_gemm_glu_bwd": (_i32, [_vp, _i64, _i64, _vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64,
                                          _vp, _i64, _vp, _vp, _vp, _i32, _vp, _i64, _i32, _i64, _i64,
                                          _i32, _i32, _i32, _i32, _vp]),
    "moe_quantize_rows_fp8": (_i32, [_vp, _i64, _vp, _i64, _vp, _i64, _i64, _i32, _vp]),
    "moe_m_grouped_gemm_fp8": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _vp, _vp, _i32,
                                      _vp, _i32, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i64, _vp]),
    "moe_router_workspace_bytes": (_sz, [_i64, _i32, _i32, _i32]),
    "moe_router_topk": (_i32, [_vp, _i64, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _i64, _i64, _i32, _i32,
                               _i32, _i32, _i32, _vp, _sz, _vp]),
    "moe_router_bwd": (_i32, [_vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
}


class MoeHipError(RuntimeError):
    pass


def lib_path():
    return _LIB_PATH


def load():
    """Loads libmoe_hip.so (once) and declares every entry point."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise MoeHipError(
                f"{_LIB_PATH} is missing: build it with `python moe-explore_amd/build.py` "
                "(there is no fallback path)")
        lib = ctypes.CDLL(_LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status, what):
    if status != 0:
        msg = load().moe_last_error_string().decode("utf-8", "replace")
        raise MoeHipError(f"{what} failed with status {status}: {msg}")


def dtype_code(dtype):
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}") from None


def act_code(act):
    name = None if act is None else (act.value if hasattr(act, "value") else str(act))
    try:
        return _ACTS[name]
    except KeyError:
        raise ValueError(f"unsupported activation {act!r}") from None


def ptr(t):
    return 0 if t is None else t.data_ptr()


def stream_of(t):
    """The current HIP stream of the tensor's device, as a raw handle."""
    return torch.cuda.current_stream(t.device).cuda_stream


def idx_bytes(t):
    if t.dtype == torch.int64:
        return 8
    if t.dtype == torch.int32:
        return 4
    raise ValueError(f"index tensors must be int32 or int64, got {t.dtype}")


def require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise MoeHipError("libmoe_hip runs on the GPU only; got a tensor on " + str(t.device))
