"""ctypes binding of libratchet_hip.so (declared in include/ratchet_hip.h).

The library is the product; there is no other compute path.  If it has not
been built, loading raises: nothing falls back to the host.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libratchet_hip.so")

RT_MAX_RANK = 8

# rt_status
RT_OK, RT_ERR_INVALID_ARG, RT_ERR_INVALID_SHAPE, RT_ERR_DTYPE_MISMATCH = 0, 1, 2, 3
RT_ERR_UNSUPPORTED, RT_ERR_NO_DEVICE, RT_ERR_HIP, RT_ERR_OOM = 4, 5, 6, 7
# rt_dtype
RT_F32, RT_F16, RT_Q8_0F, RT_Q8_0H, RT_Q4_K = 0, 1, 2, 3, 4
# rt_kernel_kind
RT_KERNEL_NONE, RT_KERNEL_GEMV_Q8, RT_KERNEL_GEMV_Q4K, RT_KERNEL_GEMV_FLOAT = 0, 1, 2, 3
RT_KERNEL_GEMM_F16, RT_KERNEL_GEMM_F32 = 4, 5

_Shape = ctypes.c_int64 * RT_MAX_RANK


class MatmulDesc(ctypes.Structure):
    _fields_ = [
        ("lhs_dt", ctypes.c_int32), ("rhs_dt", ctypes.c_int32),
        ("lhs_rank", ctypes.c_int32), ("rhs_rank", ctypes.c_int32),
        ("lhs_shape", _Shape), ("rhs_shape", _Shape),
        ("trans_lhs", ctypes.c_int32), ("trans_rhs", ctypes.c_int32), ("trans_out", ctypes.c_int32),
        ("has_bias", ctypes.c_int32), ("bias_dt", ctypes.c_int32), ("bias_rank", ctypes.c_int32),
        ("bias_shape", _Shape),
    ]


class GemmSpec(ctypes.Structure):
    _fields_ = [
        ("lhs_shape", ctypes.c_int64 * 2), ("rhs_shape", ctypes.c_int64 * 2), ("out_shape", ctypes.c_int64 * 2),
        ("lhs_stack", ctypes.c_int64), ("rhs_stack", ctypes.c_int64), ("out_stack", ctypes.c_int64),
        ("dim_lhs_outer", ctypes.c_int64), ("dim_rhs_outer", ctypes.c_int64), ("dim_inner", ctypes.c_int64),
        ("is_gemv", ctypes.c_int32), ("heuristic", ctypes.c_int32), ("kernel", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class GgufTensorInfo(ctypes.Structure):
    _fields_ = [
        ("name", ctypes.c_char_p), ("ggml_dtype", ctypes.c_int32), ("rank", ctypes.c_int32), ("shape", _Shape),
        ("offset", ctypes.c_uint64), ("size_in_bytes", ctypes.c_uint64),
    ]


class GgufValue(ctypes.Structure):
    _fields_ = [
        ("type", ctypes.c_int32), ("elem_type", ctypes.c_int32), ("count", ctypes.c_uint64),
        ("u64", ctypes.c_uint64), ("i64", ctypes.c_int64), ("f64", ctypes.c_double), ("str", ctypes.c_char_p),
    ]


RT_ACT_NONE, RT_ACT_GELU, RT_ACT_SILU = 0, 1, 2

class AttentionDesc(ctypes.Structure):
    """rt_attention_desc."""
    _fields_ = [
        ("dtype", ctypes.c_int32),
        ("batch", ctypes.c_int32), ("heads", ctypes.c_int32),
        ("q_len", ctypes.c_int32), ("kv_len", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("q_strides", ctypes.c_int64 * 3), ("k_strides", ctypes.c_int64 * 3),
        ("v_strides", ctypes.c_int64 * 3), ("o_strides", ctypes.c_int64 * 3),
        ("scale", ctypes.c_float),
        ("causal", ctypes.c_int32),
        ("mask_dtype", ctypes.c_int32),
        ("mask_row_stride", ctypes.c_int64),
    ]


# name -> (restype, argtypes); the single source the symbol test walks too
_vp, _u64, _i32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int32
_P = ctypes.POINTER
SIGNATURES = {
    "rt_matmul_infer": (_i32, [_P(MatmulDesc), _P(ctypes.c_int64), _P(_i32), _P(_i32)]),
    "rt_matmul_validate": (_i32, [_P(MatmulDesc)]),
    "rt_matmul_spec": (_i32, [_P(MatmulDesc), _P(GemmSpec)]),
    "rt_tensor_nbytes": (_i32, [_i32, _u64, _P(_u64)]),
    "rt_q8_0_scale_offset": (_u64, [_u64]),
    "rt_status_string": (ctypes.c_char_p, [_i32]),
    "rt_kernel_string": (ctypes.c_char_p, [_i32]),
    "rt_ctx_create": (_i32, [_i32, _P(_vp)]),
    "rt_ctx_destroy": (_i32, [_vp]),
    "rt_last_error": (ctypes.c_char_p, [_vp]),
    "rt_last_hip_error": (_i32, [_vp]),
    "rt_buf_alloc": (_i32, [_vp, _u64, _P(_vp)]),
    "rt_buf_free": (_i32, [_vp, _vp]),
    "rt_buf_upload": (_i32, [_vp, _vp, _vp, _u64, _vp]),
    "rt_buf_download": (_i32, [_vp, _vp, _vp, _u64, _vp]),
    "rt_sync": (_i32, [_vp, _vp]),
    "rt_matmul_enqueue": (_i32, [_vp, _P(MatmulDesc), _vp, _vp, _vp, _vp, _vp]),
    "rt_matmul_enqueue_fused": (_i32, [_vp, _P(MatmulDesc), _vp, _vp, _vp, _vp, _i32, _vp]),
    "rt_matmul_workspace_bytes": (_i32, [_vp, _P(MatmulDesc), _P(_u64)]),
    "rt_matmul_enqueue_ws": (_i32, [_vp, _P(MatmulDesc), _vp, _vp, _vp, _vp, _i32, _vp, _u64, _vp]),
    "rt_matmul_enqueue_static": (_i32, [_vp, _P(MatmulDesc), _vp, _vp, _vp, _vp, _i32, _vp]),
    "rt_matmul_plan_create": (_i32, [_vp, _P(MatmulDesc), _i32, _P(_vp)]),
    "rt_matmul_plan_enqueue": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp]),
    "rt_matmul_plan_destroy": (_i32, [_vp]),
    "rt_unary_enqueue": (_i32, [_vp, _i32, _i32, _vp, _vp, _u64, _vp]),
    "rt_cast_enqueue": (_i32, [_vp, _i32, _i32, _vp, _vp, _u64, _vp]),
    "rt_quantize_q8_0": (_i32, [_vp, _vp, _u64, _vp, _vp]),
    "rt_dequantize": (_i32, [_vp, _i32, _vp, _u64, _vp, _vp]),
    "rt_transcode_gguf_q8_0": (_i32, [_vp, _vp, _u64, _i32, _vp, _vp]),
    "rt_softmax_validate": (_i32, [_i32, _i32, _P(ctypes.c_int64), _i32]),
    "rt_softmax_enqueue": (_i32, [_vp, _i32, _vp, _i32, _P(ctypes.c_int64), _i32, _vp]),
    "rt_attention_validate": (_i32, [_P(AttentionDesc)]),
    "rt_attention_workspace_bytes": (_i32, [_P(AttentionDesc), _P(_u64)]),
    "rt_attention_enqueue": (_i32, [_vp, _P(AttentionDesc), _vp, _vp, _vp, _vp, _vp, _vp, _u64, _vp]),
    "rt_cache_write_enqueue": (_i32, [_vp, _i32, _vp, _vp, _P(ctypes.c_int64), _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "rt_cache_write_kv_enqueue": (_i32, [_vp, _i32, _vp, _vp, _vp, _vp, _P(ctypes.c_int64), _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "rt_gguf_parse": (_i32, [_vp, _u64, _P(_vp)]),
    "rt_gguf_free": (None, [_vp]),
    "rt_gguf_error": (ctypes.c_char_p, [_vp]),
    "rt_gguf_version": (ctypes.c_uint32, [_vp]),
    "rt_gguf_tensor_count": (_u64, [_vp]),
    "rt_gguf_metadata_count": (_u64, [_vp]),
    "rt_gguf_tensor_data_offset": (_u64, [_vp]),
    "rt_gguf_tensor_info_at": (_i32, [_vp, _u64, _P(GgufTensorInfo)]),
    "rt_gguf_find_tensor": (_i32, [_vp, ctypes.c_char_p, _P(_u64)]),
    "rt_gguf_metadata_key_at": (_i32, [_vp, _u64, _P(ctypes.c_char_p)]),
    "rt_gguf_metadata_get": (_i32, [_vp, ctypes.c_char_p, _P(GgufValue)]),
    "rt_gguf_metadata_array_get": (_i32, [_vp, ctypes.c_char_p, _u64, _P(GgufValue)]),
    "rt_ggml_type_size": (_u64, [_i32]),
    "rt_ggml_block_numel": (_u64, [_i32]),
    "rt_gguf_load_tensor": (_i32, [_vp, _vp, _vp, _u64, _u64, _i32, _vp, _vp, _vp]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Loads libratchet_hip.so; raises if it has not been built.

    A process must hold exactly one HIP runtime.  torch ships its own copy of
    libamdhip64.so.7 and supplies the device memory these bindings hand to the
    library, so torch is imported first: the library's dependency on
    libamdhip64.so.7 then resolves to the copy torch has already loaded."""
    global _lib
    if _lib is None:
        try:
            import torch  # noqa: F401  (loads the HIP runtime the library will share)
        except ImportError:
            pass
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python -m ratchet_amd.build`. "
                "ratchet_amd has no host fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def status_string(st: int) -> str:
    return lib().rt_status_string(st).decode()


def make_desc(lhs_dt, lhs_shape, rhs_dt, rhs_shape, trans_lhs=False, trans_rhs=False, trans_out=False,
              bias_dt=None, bias_shape=None) -> MatmulDesc:
    d = MatmulDesc()
    if len(lhs_shape) > RT_MAX_RANK or len(rhs_shape) > RT_MAX_RANK:
        raise ValueError("rank above RT_MAX_RANK")
    d.lhs_dt, d.rhs_dt = int(lhs_dt), int(rhs_dt)
    d.lhs_rank, d.rhs_rank = len(lhs_shape), len(rhs_shape)
    for i, v in enumerate(lhs_shape):
        d.lhs_shape[i] = int(v)
    for i, v in enumerate(rhs_shape):
        d.rhs_shape[i] = int(v)
    d.trans_lhs, d.trans_rhs, d.trans_out = int(trans_lhs), int(trans_rhs), int(trans_out)
    if bias_shape is not None:
        if len(bias_shape) > RT_MAX_RANK:
            raise ValueError("rank above RT_MAX_RANK")
        d.has_bias, d.bias_dt, d.bias_rank = 1, int(bias_dt), len(bias_shape)
        for i, v in enumerate(bias_shape):
            d.bias_shape[i] = int(v)
    return d
