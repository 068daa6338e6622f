"""ctypes binding of libmi_attention.so (the C ABI declared in include/mi_attention.h).

Loading fails loudly when the library has not been built: there is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# MI_ATTENTION_LIB points at an alternative build of the same library (kernel tuning experiments).
LIB_PATH = os.environ.get("MI_ATTENTION_LIB") or os.path.join(HERE, "lib", "libmi_attention.so")

MI_DTYPE_F16 = 1
MI_DTYPE_BF16 = 2
MI_MASK_NONE = 0
MI_MASK_CAUSAL = 1
MI_MASK_BLOCK_CAUSAL = 2
MI_MAX_SEGMENTS = 32
MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES = 16 * 1024 * 1024
MI_LINEAR_ATTN_FORM_BY_SIZE = 0
MI_LINEAR_ATTN_FORM_THREE_LAUNCHES = 1
MI_LINEAR_ATTN_FORM_ONE_LAUNCH = 2
MI_LAYOUT_TOKEN_MAJOR = 0
MI_LAYOUT_CHANNEL_MAJOR = 1

EXPORTS = [
    "mi_last_error", "mi_version", "mi_device_info", "mi_mfma_probe", "mi_set_stream", "mi_get_stream", "mi_stream_synchronize",
    "mi_malloc", "mi_free", "mi_memcpy_h2d", "mi_memcpy_d2h", "mi_memcpy_d2d_async", "mi_memset_async",
    "mi_sdpa_forward", "mi_sdpa_split_scratch_bytes", "mi_sdpa_supported", "mi_sdpa_set_kernel_choice", "mi_attention_map_avg", "mi_rope_apply", "mi_headnorm_rope", "mi_scale_rows",
    "mi_linear_attn_workspace_bytes", "mi_linear_attn_scratch_bytes", "mi_linear_attn_relu_forward", "mi_linear_attn_supported", "mi_linear_attn_relu_forward_static_scratch",
    "mi_linear_forward", "mi_linear_geglu_forward", "mi_add_inplace", "mi_add_row_bias", "mi_rms_norm_forward", "mi_flash_attention_scratch_bytes", "mi_flash_attention_qkvo_forward",
    "mi_flash_attention_q_with_kv_cached_forward", "mi_flash_attention_project_kv",
]


class MiDeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 64), ("compute_units", C.c_int32),
                ("clock_khz", C.c_int32), ("lds_bytes_per_cu", C.c_int32), ("l2_bytes", C.c_int32),
                ("hbm_bytes", C.c_int64), ("peak_mfma_16bit_flops", C.c_double)]


class MiMfmaProbeArgs(C.Structure):
    _fields_ = [("struct_size", C.c_uint32), ("dtype", C.c_int32), ("operands", C.c_void_p), ("operand_bytes", C.c_size_t),
                ("trips", C.c_int32), ("work_groups", C.c_int32), ("sink", C.c_void_p), ("sink_bytes", C.c_size_t),
                ("clocks", C.c_void_p), ("clocks_bytes", C.c_size_t), ("flops", C.c_double), ("stream", C.c_void_p)]


class MiSdpaArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("k_prefix", C.c_void_p), ("v_prefix", C.c_void_p),
        ("batch", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32), ("num_kv_heads", C.c_int32),
        ("q_len", C.c_int32), ("kv_len", C.c_int32), ("prefix_len", C.c_int32),
        ("q_row_stride", C.c_int64), ("q_batch_stride", C.c_int64),
        ("k_row_stride", C.c_int64), ("k_batch_stride", C.c_int64),
        ("v_row_stride", C.c_int64), ("v_batch_stride", C.c_int64),
        ("o_row_stride", C.c_int64), ("o_batch_stride", C.c_int64),
        ("kp_row_stride", C.c_int64), ("kp_batch_stride", C.c_int64),
        ("vp_row_stride", C.c_int64), ("vp_batch_stride", C.c_int64),
        ("scale", C.c_float), ("mask_mode", C.c_int32), ("q_offset", C.c_int32), ("window", C.c_int32),
        ("kv_valid_len", C.c_void_p), ("key_mask", C.c_void_p), ("key_mask_batch_stride", C.c_int64),
        ("n_segments", C.c_int32),
        ("seg_q_end", C.c_int32 * MI_MAX_SEGMENTS), ("seg_k_end", C.c_int32 * MI_MAX_SEGMENTS),
        ("seg_causal", C.c_int32 * MI_MAX_SEGMENTS),
        ("rope_cos_q", C.c_void_p), ("rope_sin_q", C.c_void_p), ("rope_cos_k", C.c_void_p), ("rope_sin_k", C.c_void_p),
        ("rope_split_half", C.c_int32), ("rope_k_scratch", C.c_void_p),
        ("logit_bias", C.c_void_p), ("bias_q0", C.c_int32), ("bias_cols", C.c_int32), ("bias_row_stride", C.c_int64),
        ("lse_out", C.c_void_p),
        ("cu_seqlens_q", C.c_void_p), ("cu_seqlens_k", C.c_void_p),
        ("prefix_k_scale", C.c_float), ("prefix_v_scale", C.c_float),
        ("prefix_k_row_scale", C.c_void_p), ("prefix_v_row_scale", C.c_void_p),
        ("split_scratch", C.c_void_p), ("split_scratch_bytes", C.c_size_t),
        ("stream", C.c_void_p),
    ]


class MiAttentionMapArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("lse", C.c_void_p), ("map", C.c_void_p),
        ("num_heads", C.c_int32), ("head_dim", C.c_int32), ("q_len", C.c_int32), ("kv_len", C.c_int32),
        ("q_row_stride", C.c_int64), ("k_row_stride", C.c_int64), ("map_row_stride", C.c_int64),
        ("scale", C.c_float), ("logit_bias", C.c_void_p), ("bias_q0", C.c_int32), ("bias_cols", C.c_int32),
        ("bias_row_stride", C.c_int64), ("key_mask", C.c_void_p), ("stream", C.c_void_p),
    ]


class MiRopeArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("x", C.c_void_p), ("out", C.c_void_p), ("cos", C.c_void_p), ("sin", C.c_void_p),
        ("rows", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32),
        ("x_row_stride", C.c_int64), ("out_row_stride", C.c_int64),
        ("split_half", C.c_int32), ("per_head", C.c_int32), ("stream", C.c_void_p),
    ]


class MiHeadnormRopeArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("x", C.c_void_p), ("out", C.c_void_p), ("gain", C.c_void_p), ("cos", C.c_void_p), ("sin", C.c_void_p),
        ("eps", C.c_float), ("rows", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32),
        ("x_row_stride", C.c_int64), ("out_row_stride", C.c_int64),
        ("out2", C.c_void_p), ("out2_rows", C.c_int32), ("out2_row_stride", C.c_int64), ("split_half", C.c_int32),
        ("stream", C.c_void_p),
    ]


class MiScaleRowsArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("x", C.c_void_p), ("out", C.c_void_p), ("row_scale", C.c_void_p), ("scale", C.c_float),
        ("rows", C.c_int32), ("cols", C.c_int32), ("x_row_stride", C.c_int64), ("out_row_stride", C.c_int64),
        ("stream", C.c_void_p),
    ]


class MiLinearAttnArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("o", C.c_void_p),
        ("batch", C.c_int32), ("num_heads", C.c_int32), ("head_dim", C.c_int32), ("n_tokens", C.c_int32),
        ("q_row_stride", C.c_int64), ("q_batch_stride", C.c_int64),
        ("k_row_stride", C.c_int64), ("k_batch_stride", C.c_int64),
        ("v_row_stride", C.c_int64), ("v_batch_stride", C.c_int64),
        ("o_row_stride", C.c_int64), ("o_batch_stride", C.c_int64),
        ("eps", C.c_float), ("accumulate_state", C.c_int32), ("accumulate_weight", C.c_float),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("scratch", C.c_void_p), ("scratch_bytes", C.c_size_t), ("form", C.c_int32), ("layout", C.c_int32), ("stream", C.c_void_p),
    ]


class MiLinearArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("x", C.c_void_p), ("w", C.c_void_p), ("bias", C.c_void_p), ("y", C.c_void_p),
        ("rows", C.c_int32), ("in_features", C.c_int32), ("out_features", C.c_int32),
        ("x_row_stride", C.c_int64), ("w_row_stride", C.c_int64), ("y_row_stride", C.c_int64),
        ("w_scales", C.c_void_p), ("stream", C.c_void_p),
    ]


class MiAttnBlockArgs(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32),
        ("x", C.c_void_p), ("ctx", C.c_void_p),
        ("wq", C.c_void_p), ("bq", C.c_void_p), ("wk", C.c_void_p), ("bk", C.c_void_p),
        ("wv", C.c_void_p), ("bv", C.c_void_p), ("wo", C.c_void_p), ("bo", C.c_void_p),
        ("k", C.c_void_p), ("v", C.c_void_p), ("out", C.c_void_p),
        ("batch", C.c_int32), ("q_len", C.c_int32), ("kv_len", C.c_int32),
        ("channels", C.c_int32), ("ctx_channels", C.c_int32), ("inner", C.c_int32), ("out_channels", C.c_int32),
        ("num_heads", C.c_int32), ("causal", C.c_int32),
        ("key_mask", C.c_void_p), ("key_mask_batch_stride", C.c_int64),
        ("scratch", C.c_void_p), ("scratch_bytes", C.c_size_t),
        ("wq_scales", C.c_void_p), ("wk_scales", C.c_void_p), ("wv_scales", C.c_void_p), ("wo_scales", C.c_void_p),
        ("stream", C.c_void_p),
    ]


_lib = None


def lib() -> C.CDLL:
    """The loaded C-ABI library; raises if it has not been built (python -m brodiffusion_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build the HIP extension first (python -m brodiffusion_amd.build). "
                "There is no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        L.mi_last_error.restype = C.c_char_p
        L.mi_version.restype = C.c_char_p
        L.mi_device_info.argtypes = [C.POINTER(MiDeviceInfo)]
        L.mi_mfma_probe.argtypes = [C.POINTER(MiMfmaProbeArgs)]
        L.mi_set_stream.argtypes = [C.c_void_p]
        L.mi_get_stream.restype = C.c_void_p
        L.mi_stream_synchronize.argtypes = [C.c_void_p]
        L.mi_malloc.argtypes = [C.c_size_t]
        L.mi_malloc.restype = C.c_void_p
        L.mi_free.argtypes = [C.c_void_p]
        L.mi_memcpy_h2d.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.mi_memcpy_d2h.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        L.mi_memcpy_d2d_async.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
        L.mi_memset_async.argtypes = [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p]
        L.mi_sdpa_forward.argtypes = [C.POINTER(MiSdpaArgs)]
        L.mi_sdpa_split_scratch_bytes.argtypes = [C.POINTER(MiSdpaArgs)]
        L.mi_sdpa_split_scratch_bytes.restype = C.c_size_t
        L.mi_sdpa_supported.argtypes = [C.c_int32, C.c_int32]
        L.mi_sdpa_set_kernel_choice.argtypes = [C.c_int32]
        L.mi_attention_map_avg.argtypes = [C.POINTER(MiAttentionMapArgs)]
        L.mi_rope_apply.argtypes = [C.POINTER(MiRopeArgs)]
        L.mi_headnorm_rope.argtypes = [C.POINTER(MiHeadnormRopeArgs)]
        L.mi_scale_rows.argtypes = [C.POINTER(MiScaleRowsArgs)]
        L.mi_linear_attn_workspace_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        L.mi_linear_attn_workspace_bytes.restype = C.c_size_t
        L.mi_linear_attn_scratch_bytes.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        L.mi_linear_attn_scratch_bytes.restype = C.c_size_t
        L.mi_linear_attn_relu_forward.argtypes = [C.POINTER(MiLinearAttnArgs)]
        L.mi_linear_attn_supported.argtypes = [C.c_int32, C.c_int32]
        L.mi_linear_attn_relu_forward_static_scratch.argtypes = [C.POINTER(MiLinearAttnArgs)]
        L.mi_linear_forward.argtypes = [C.POINTER(MiLinearArgs)]
        L.mi_linear_geglu_forward.argtypes = [C.POINTER(MiLinearArgs)]
        L.mi_add_inplace.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_void_p]
        L.mi_add_row_bias.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_int32, C.c_void_p]
        L.mi_rms_norm_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_int64, C.c_float,
                                          C.c_int32, C.c_void_p]
        L.mi_flash_attention_scratch_bytes.argtypes = [C.c_int32] * 5
        L.mi_flash_attention_scratch_bytes.restype = C.c_size_t
        for name in ("mi_flash_attention_qkvo_forward", "mi_flash_attention_q_with_kv_cached_forward", "mi_flash_attention_project_kv"):
            getattr(L, name).argtypes = [C.POINTER(MiAttnBlockArgs)]
        _lib = L
    return _lib


def last_error() -> str:
    return lib().mi_last_error().decode()


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: {last_error()}")
