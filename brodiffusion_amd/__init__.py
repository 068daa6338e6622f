"""MI355X-native attention path with brotensor-style operator entry points.

The compute lives in lib/libmi_attention.so (hand-written HIP for gfx950 behind the C ABI in
include/mi_attention.h). This package is the Python mirror of the host interface, used by the
tests and the benchmark; PyTorch only provides device memory and streams.
"""
from .ops import (  # noqa: F401
    SdpaMask,
    build_axial_rope_tables,
    build_qwen_rope_tables,
    device_info,
    mfma_probe,
    flash_attention_forward,
    flash_attention_project_kv,
    flash_attention_project_kv_int8w_fp16,
    flash_attention_q_with_kv_cached_int8w_fp16,
    flash_attention_qkvo_int8w_fp16,
    linear_forward_batched_int8w_fp16,
    flash_attention_q_with_kv_cached_forward,
    flash_attention_qkvo_forward,
    flash_attention_scratch_bytes,
    flash_attention_varlen_forward,
    flash_attention_windowed_forward,
    gqa_attention_masked,
    headnorm_rope,
    add_inplace_row_bias,
    add_inplace_vec,
    attention_map_avg,
    fused_linear_geglu,
    fused_linear_geglu_int8w,
    joint_attention,
    joint_attention_traced,
    cross_attention_forward_with_attn, mha_forward,
    linear_attention_relu_forward,
    linear_attention_relu_forward_static_scratch,
    linear_attention_relu_forward_channel_major,
    linear_batched,
    qwen_rope_positions,
    rms_norm_rows,
    rope_apply,
    rope_apply_perhead,
    sana_self_attention,
    rope_tables_from_positions,
    scale_rows,
    sdpa_forward,
    set_sdpa_kernel_choice,
)

__all__ = [
    "SdpaMask", "build_axial_rope_tables", "build_qwen_rope_tables", "qwen_rope_positions", "rope_tables_from_positions", "device_info", "mfma_probe", "flash_attention_forward",
    "flash_attention_windowed_forward", "gqa_attention_masked", "joint_attention",
    "linear_attention_relu_forward", "linear_attention_relu_forward_static_scratch", "linear_attention_relu_forward_channel_major", "rope_apply", "flash_attention_qkvo_forward", "flash_attention_q_with_kv_cached_forward",
    "flash_attention_project_kv", "flash_attention_scratch_bytes", "linear_batched", "headnorm_rope", "flash_attention_varlen_forward", "flash_attention_qkvo_int8w_fp16", "flash_attention_q_with_kv_cached_int8w_fp16",
    "flash_attention_project_kv_int8w_fp16", "linear_forward_batched_int8w_fp16", "fused_linear_geglu", "fused_linear_geglu_int8w", "add_inplace_vec", "add_inplace_row_bias", "joint_attention_traced", "cross_attention_forward_with_attn", "mha_forward", "attention_map_avg", "scale_rows", "rope_apply_perhead", "rms_norm_rows", "sana_self_attention", "sdpa_forward", "set_sdpa_kernel_choice",
]
