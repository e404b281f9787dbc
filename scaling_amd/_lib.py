"""ctypes binding of libmi355_layer.so (C ABI declared in include/mi355_layer.h).

The library is loaded lazily.  There is no CPU or PyTorch fallback: if the shared object has not
been built, or a kernel returns an error status, a RuntimeError is raised.
"""

import ctypes
import os
from ctypes import c_uint64, POINTER, Structure, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmi355_layer.so")

MI_BF16, MI_F16, MI_F32 = 0, 1, 2
_DTYPE_CODE = {torch.bfloat16: MI_BF16, torch.float16: MI_F16, torch.float32: MI_F32}

EXPORTS = (
    "mi_version", "mi_last_error", "mi_status_string", "mi_check_device",
    "mi_rmsnorm_fwd", "mi_add_rmsnorm_fwd", "mi_rmsnorm_bwd_workspace_bytes", "mi_rmsnorm_bwd",
    "mi_layernorm_fwd", "mi_layernorm_bwd_workspace_bytes", "mi_layernorm_bwd", "mi_gelu_fwd", "mi_gelu_bwd", "mi_cross_entropy",
    "mi_swiglu_fwd", "mi_swiglu_bwd", "mi_rotary", "mi_rotary_complex",
    "mi_attn_fwd", "mi_attn_bwd_workspace_bytes", "mi_attn_bwd_workspace_bytes_kv", "mi_attn_bwd",
    "mi_attn_decode_workspace_bytes", "mi_attn_decode", "mi_attn_decode_static_scratch_bytes", "mi_attn_decode_static",
)


class MiAttnArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k", c_void_p), ("v", c_void_p), ("o", c_void_p), ("lse", c_void_p),
        ("cu_seqlens_q", c_void_p), ("cu_seqlens_k", c_void_p),
        ("n_docs", c_int32), ("causal", c_int32),
        ("total_q", c_int64), ("total_k", c_int64),
        ("n_q_heads", c_int32), ("n_kv_heads", c_int32), ("head_dim", c_int32), ("dtype", c_int32),
        ("q_stride_token", c_int64), ("q_stride_head", c_int64),
        ("k_stride_token", c_int64), ("k_stride_head", c_int64),
        ("v_stride_token", c_int64), ("v_stride_head", c_int64),
        ("o_stride_token", c_int64), ("o_stride_head", c_int64),
        ("softmax_scale", c_float), ("flags", c_int32),
        ("rotary_cos", c_void_p), ("rotary_sin", c_void_p),
        ("position_ids_q", c_void_p), ("position_ids_k", c_void_p),
        ("rotary_table_rows", c_int64),
        ("stream", c_void_p),
        ("dropout_p", c_float), ("dropout_seed", c_uint64), ("rotary_interleaved", c_int32),
        ("q_rot_out", c_void_p),
    ]


class MiAttnBwdArgs(Structure):
    _fields_ = [
        ("fwd", MiAttnArgs),
        ("d_o", c_void_p), ("dq", c_void_p), ("dk", c_void_p), ("dv", c_void_p),
        ("dk_stride_token", c_int64), ("dk_stride_head", c_int64),
        ("dv_stride_token", c_int64), ("dv_stride_head", c_int64),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
    ]


class MiDecodeArgs(Structure):
    _fields_ = [
        ("q", c_void_p), ("k_cache", c_void_p), ("v_cache", c_void_p), ("o", c_void_p),
        ("ctx_len", c_void_p), ("k_new", c_void_p), ("v_new", c_void_p),
        ("rotary_cos", c_void_p), ("rotary_sin", c_void_p), ("position_ids", c_void_p),
        ("rotary_table_rows", c_int64),
        ("batch", c_int32), ("max_ctx", c_int32), ("n_q_heads", c_int32), ("n_kv_heads", c_int32),
        ("head_dim", c_int32), ("dtype", c_int32),
        ("cache_stride_batch", c_int64), ("cache_stride_token", c_int64), ("cache_stride_head", c_int64),
        ("softmax_scale", c_float), ("n_splits", c_int32),
        ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("stream", c_void_p),
        ("q_stride_batch", c_int64), ("k_new_stride_batch", c_int64), ("v_new_stride_batch", c_int64),
        ("rotary_interleaved", c_int32),
    ]


_lib = None
_device_checked = False


def _declare(lib):
    lib.mi_version.restype = c_int
    lib.mi_last_error.restype = c_char_p
    lib.mi_status_string.restype = c_char_p
    lib.mi_status_string.argtypes = [c_int]
    lib.mi_check_device.restype = c_int
    lib.mi_rmsnorm_fwd.restype = c_int
    lib.mi_rmsnorm_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_int, c_void_p]
    lib.mi_rmsnorm_bwd_workspace_bytes.restype = c_size_t
    lib.mi_add_rmsnorm_fwd.restype = c_int
    lib.mi_add_rmsnorm_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float, c_int, c_void_p]
    lib.mi_rmsnorm_bwd_workspace_bytes.argtypes = [c_int64, c_int64]
    lib.mi_rmsnorm_bwd.restype = c_int
    lib.mi_rmsnorm_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_int64,
                                   c_int64, c_float, c_int, c_void_p]
    lib.mi_layernorm_fwd.restype = c_int
    lib.mi_layernorm_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_float,
                                     c_int, c_void_p]
    lib.mi_layernorm_bwd_workspace_bytes.restype = c_size_t
    lib.mi_layernorm_bwd_workspace_bytes.argtypes = [c_int64, c_int64]
    lib.mi_layernorm_bwd.restype = c_int
    lib.mi_layernorm_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_size_t, c_int64, c_int64, c_float, c_int, c_void_p]
    lib.mi_gelu_fwd.restype = c_int
    lib.mi_gelu_fwd.argtypes = [c_void_p, c_void_p, c_int64, c_int, c_void_p]
    lib.mi_gelu_bwd.restype = c_int
    lib.mi_gelu_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]
    lib.mi_cross_entropy.restype = c_int
    lib.mi_cross_entropy.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
                                     c_int64, c_int64, c_int, c_void_p]
    lib.mi_swiglu_fwd.restype = c_int
    lib.mi_swiglu_fwd.argtypes = [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]
    lib.mi_swiglu_bwd.restype = c_int
    lib.mi_swiglu_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]
    lib.mi_rotary.restype = c_int
    lib.mi_rotary.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_int32,
                              c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p]
    lib.mi_rotary_complex.restype = c_int
    lib.mi_rotary_complex.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32,
                                      c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_int, c_int, c_void_p]
    lib.mi_attn_fwd.restype = c_int
    lib.mi_attn_fwd.argtypes = [POINTER(MiAttnArgs)]
    lib.mi_attn_bwd_workspace_bytes.restype = c_size_t
    lib.mi_attn_bwd_workspace_bytes.argtypes = [c_int64, c_int32, c_int32]
    lib.mi_attn_bwd_workspace_bytes_kv.restype = c_size_t
    lib.mi_attn_bwd_workspace_bytes_kv.argtypes = [c_int64, c_int64, c_int32, c_int32, c_int32]
    lib.mi_attn_bwd.restype = c_int
    lib.mi_attn_bwd.argtypes = [POINTER(MiAttnBwdArgs)]
    lib.mi_attn_decode_workspace_bytes.restype = c_size_t
    lib.mi_attn_decode_workspace_bytes.argtypes = [c_int32, c_int32, c_int32, c_int32]
    lib.mi_attn_decode.restype = c_int
    lib.mi_attn_decode.argtypes = [POINTER(MiDecodeArgs)]
    lib.mi_attn_decode_static_scratch_bytes.restype = c_size_t
    lib.mi_attn_decode_static_scratch_bytes.argtypes = []
    lib.mi_attn_decode_static.restype = c_int
    lib.mi_attn_decode_static.argtypes = [POINTER(MiDecodeArgs)]


def load(path: str = LIB_PATH):
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: the HIP extension has not been built "
                "(run `python -m scaling_amd.csrc.build`); there is no fallback path"
            )
        lib = ctypes.CDLL(path)
        _declare(lib)
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != 0:
        lib = load()
        raise RuntimeError(
            f"{what} failed: {lib.mi_status_string(status).decode()} ({status}): {lib.mi_last_error().decode()}"
        )


def require_device() -> None:
    """Raises unless the current device is a gfx950 GPU (checked once per process)."""
    global _device_checked
    if _device_checked:
        return
    if not torch.cuda.is_available():
        raise RuntimeError("scaling_amd kernels need an MI355X (gfx950) GPU; no HIP device is visible")
    check(load().mi_check_device(), "mi_check_device")
    _device_checked = True


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"dtype {dtype} is not supported by the HIP kernels") from None


def stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def ptr(t):
    return None if t is None else t.data_ptr()
