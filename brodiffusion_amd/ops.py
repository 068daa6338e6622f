"""Python mirror of the host-side operator interface for the attention path.

Names, argument order and error behaviour follow the brotensor operators the reference calls
(citations are paths in the reference repository):

    flash_attention_forward(Q, K, V, d_mask, num_heads, causal, out)        src/dit/common.cpp:194
    flash_attention_windowed_forward(Q, K, V, d_mask, num_heads, window, out) src/dit/qwenimage21_forward.cpp:662
    flash_attention_varlen_forward(q, k, v, cu_q, cu_k, n_seqs, max_q, max_k, num_heads, head_dim, causal, out)
                                                                             src/dit/krea2.cpp:574
    rope_apply(X, cos, sin, head_dim, num_heads, out)                        src/dit/common.cpp:192
    rope_apply_perhead(X, cos, sin, head_dim, num_heads, out)                src/triposplat/flow_model.cpp:374
    joint_attention(Q, K, V, cos, sin, head_dim, num_heads, out, Qr, Kr)     include/brodiffusion/dit/common.h:80-88
    joint_attention_traced(..., out, attn_avg, Qr, Kr, txt_len, image_text_bias)  include/brodiffusion/dit/common.h:117-129
    gqa_attention_masked(...)                                                include/brodiffusion/dit/common.h:144-153
    build_axial_rope_tables(txt_len, hp, wp, head_dim, axes, theta)          src/dit/common.cpp:116-184
    flash_attention_qkvo_forward(X, Ctx, Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads, causal, out)
                                                                             src/unet_blocks.cpp:264-272
    flash_attention_q_with_kv_cached_forward(X, K, V, Wq, bq, Wo, bo, d_mask, num_heads, causal, out)
                                                                             src/unet_blocks.cpp:311-317
    flash_attention_project_kv(ctx, Wk, bk, Wv, bv, K_out, V_out)            src/unet.cpp:476-480
    linear_batched(W, bias, X, Y)                                            include/brodiffusion/detail/compute.h:52
    fused_linear_geglu(X, W, b, Y), add_inplace_vec(Y, X), add_inplace_row_bias(Y, bias)
                                                                             include/brodiffusion/fused_transformer.h:20-61

Tensors are torch CUDA tensors (rows = tokens, cols = heads*head_dim), used for device memory
and the current stream only; every computation is a call through the C ABI. Shape and dtype
precondition failures raise RuntimeError("<op>: <message>") as the reference's ops throw
std::runtime_error; a CPU tensor is refused, never copied.
"""
from __future__ import annotations

import ctypes as C
import math
from dataclasses import dataclass, field
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

from . import _capi as capi


@dataclass
class SdpaMask:
    """Visibility rule of one attention call (see mi_sdpa_args in include/mi_attention.h)."""
    mode: int = capi.MI_MASK_NONE
    q_offset: int = 0
    window: int = 0
    seg_q_end: Sequence[int] = field(default_factory=list)
    seg_k_end: Sequence[int] = field(default_factory=list)
    seg_causal: Sequence[int] = field(default_factory=list)

    @staticmethod
    def causal(q_offset: int, window: int = 0) -> "SdpaMask":
        return SdpaMask(capi.MI_MASK_CAUSAL, q_offset, window)

    @staticmethod
    def block_causal(q_offset: int, seg_q_end, seg_k_end, seg_causal) -> "SdpaMask":
        return SdpaMask(capi.MI_MASK_BLOCK_CAUSAL, q_offset, 0, list(seg_q_end), list(seg_k_end), list(seg_causal))


def _fail(op: str, msg: str):
    raise RuntimeError(f"{op}: {msg}")


def _dtype_code(op: str, t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return capi.MI_DTYPE_BF16
    if t.dtype == torch.float16:
        return capi.MI_DTYPE_F16
    _fail(op, f"dtype {t.dtype} not supported (float16 / bfloat16)")


def _dev(op: str, *ts):
    """Every tensor on the GPU, and on the GPU that is current: the launch goes to the current device's stream (one process
    per GPU is the intended use; with several visible, select the tensors' device first)."""
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            _fail(op, "tensor is not on the GPU (CPU tensors are refused, not copied)")
        if t.device.index != torch.cuda.current_device():
            _fail(op, f"tensor is on cuda:{t.device.index} but the current device is cuda:{torch.cuda.current_device()}")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _as3(op: str, t: torch.Tensor, name: str):
    """(rows, cols) or (batch, rows, cols) -> (batch, rows, cols, row_stride, batch_stride)."""
    if t.dim() == 2:
        if t.stride(1) != 1:
            _fail(op, f"{name} must be contiguous along columns")
        return 1, t.shape[0], t.shape[1], t.stride(0), t.stride(0) * t.shape[0]
    if t.dim() == 3:
        if t.stride(2) != 1:
            _fail(op, f"{name} must be contiguous along columns")
        return t.shape[0], t.shape[1], t.shape[2], t.stride(1), t.stride(0)
    _fail(op, f"{name} must be (rows, cols) or (batch, rows, cols)")


def set_sdpa_kernel_choice(choice: int) -> None:
    """0 = by problem size, 1 = 128-row tiles, 2 = 256-row ping-pong kernel, 3 = the same with register-staged tiles
    (see mi_sdpa_set_kernel_choice)."""
    capi.check(capi.lib().mi_sdpa_set_kernel_choice(choice), "set_sdpa_kernel_choice")


def device_info() -> dict:
    info = capi.MiDeviceInfo()
    capi.check(capi.lib().mi_device_info(C.byref(info)), "mi_device_info")
    return {"name": info.name.decode(), "arch": info.arch.decode(), "compute_units": info.compute_units,
            "clock_khz": info.clock_khz, "lds_bytes_per_cu": info.lds_bytes_per_cu, "l2_bytes": info.l2_bytes,
            "hbm_bytes": info.hbm_bytes, "peak_mfma_16bit_flops": info.peak_mfma_16bit_flops}


def mfma_probe(operands: torch.Tensor, trips: int = 2000, reps: int = 5) -> dict:
    """Sustained rate of a bare MFMA loop on every compute unit with `operands` (a fp16 / bf16 device tensor: zeros,
    N(0,1), ...) as its inputs (mi_mfma_probe): TFLOP/s from event timing (best of `reps` launches after one warm-up
    launch) and the shader clock under that load, from the kernel's own cycle and 100 MHz counters."""
    op = "mfma_probe"
    _dev(op, operands)
    if not operands.is_contiguous():
        _fail(op, "operands must be contiguous")
    info = device_info()
    n_wg = 2 * info["compute_units"]
    sink = torch.empty(1024, dtype=torch.float32, device=operands.device)
    clocks = torch.zeros(2 * n_wg, dtype=torch.int64, device=operands.device)
    a = capi.MiMfmaProbeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, operands)
    a.operands, a.operand_bytes = operands.data_ptr(), operands.numel() * operands.element_size()
    a.trips = trips
    a.sink, a.sink_bytes = sink.data_ptr(), sink.numel() * 4
    a.clocks, a.clocks_bytes = clocks.data_ptr(), clocks.numel() * 8
    a.stream = _stream()
    best = None
    for i in range(reps + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        capi.check(capi.lib().mi_mfma_probe(C.byref(a)), "mi_mfma_probe")
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        if i > 0 and (best is None or ms < best):
            best = ms
    c = clocks.view(-1, 2).double()
    mhz = float((c[:, 0] / c[:, 1].clamp(min=1)).mean().item() * 100.0)
    return {"tflops": a.flops / (best * 1e-3) / 1e12, "ms": best, "shader_mhz": mhz, "flops": a.flops}


def sdpa_forward(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_heads: int, *, out: Optional[torch.Tensor] = None,
                 num_kv_heads: int = 0, k_prefix: Optional[torch.Tensor] = None, v_prefix: Optional[torch.Tensor] = None,
                 scale: Optional[float] = None, mask: Optional[SdpaMask] = None,
                 kv_valid_len: Optional[torch.Tensor] = None, key_mask: Optional[torch.Tensor] = None,
                 rope_q: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                 rope_k: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
                 rope_k_scratch: Optional[torch.Tensor] = None, rope_split_half: bool = False, split_scratch=None,
                 logit_bias: Optional[torch.Tensor] = None, bias_q0: int = 0, lse_out: Optional[torch.Tensor] = None,
                 prefix_k_scale: float = 1.0, prefix_v_scale: float = 1.0, prefix_k_row_scale: Optional[torch.Tensor] = None,
                 prefix_v_row_scale: Optional[torch.Tensor] = None, op: str = "sdpa_forward") -> torch.Tensor:
    """General entry: everything mi_sdpa_forward offers. Returns `out` (allocated like q if None).
    split_scratch: None = lend the module's own scratch (grown on demand, one per device, shared by all calls of the
    process: use one stream at a time) when the launch can use one, False = never split, a uint8 tensor = lend that."""
    _dev(op, q, k, v, out, k_prefix, v_prefix, kv_valid_len, key_mask, rope_k_scratch)
    dt = _dtype_code(op, q)
    if k.dtype != q.dtype or v.dtype != q.dtype:
        _fail(op, "Q, K, V must share one dtype")
    B, Lq, Dq, q_rs, q_bs = _as3(op, q, "Q")
    Bk, Lk, Dk, k_rs, k_bs = _as3(op, k, "K")
    Bv, Lv, Dv, v_rs, v_bs = _as3(op, v, "V")
    if num_heads <= 0 or Dq % num_heads != 0:
        _fail(op, "D must equal head_dim * num_heads")
    hd = Dq // num_heads
    hkv = num_kv_heads if num_kv_heads > 0 else num_heads
    if num_heads % hkv != 0:
        _fail(op, "num_kv_heads must divide num_heads")
    if (Bk, Dk) != (B, hkv * hd) or (Bv, Lv, Dv) != (B, Lk, hkv * hd):
        _fail(op, "K and V must be (Lk, kv_heads*head_dim) with Q's batch")
    if out is None:
        out = torch.empty_like(q)
    if out.shape != q.shape or out.dtype != q.dtype:
        _fail(op, "out must have Q's shape and dtype")
    _, _, _, o_rs, o_bs = _as3(op, out, "out")
    a = capi.MiSdpaArgs()
    a.struct_size = C.sizeof(capi.MiSdpaArgs)
    a.dtype = dt
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.batch, a.num_heads, a.head_dim, a.num_kv_heads = B, num_heads, hd, hkv
    a.q_len, a.kv_len = Lq, Lk
    a.q_row_stride, a.q_batch_stride = q_rs, q_bs
    a.k_row_stride, a.k_batch_stride = k_rs, k_bs
    a.v_row_stride, a.v_batch_stride = v_rs, v_bs
    a.o_row_stride, a.o_batch_stride = o_rs, o_bs
    Lp = 0
    if (k_prefix is None) != (v_prefix is None):
        _fail(op, "k_prefix and v_prefix must be given together")
    if k_prefix is not None:
        if k_prefix.dtype != q.dtype or v_prefix.dtype != q.dtype:
            _fail(op, "prefix K/V must have Q's dtype")
        Bp, Lp, Dp, kp_rs, kp_bs = _as3(op, k_prefix, "k_prefix")
        Bp2, Lp2, Dp2, vp_rs, vp_bs = _as3(op, v_prefix, "v_prefix")
        if (Bp, Dp) != (B, hkv * hd) or (Bp2, Lp2, Dp2) != (B, Lp, hkv * hd):
            _fail(op, "prefix K/V must be (prefix_len, kv_heads*head_dim) with Q's batch")
        a.k_prefix, a.v_prefix, a.prefix_len = k_prefix.data_ptr(), v_prefix.data_ptr(), Lp
        a.kp_row_stride, a.kp_batch_stride, a.vp_row_stride, a.vp_batch_stride = kp_rs, kp_bs, vp_rs, vp_bs
    a.scale = float(scale) if scale is not None else 0.0
    a.prefix_k_scale, a.prefix_v_scale = float(prefix_k_scale), float(prefix_v_scale)
    for nm, rs in (("prefix_k_row_scale", prefix_k_row_scale), ("prefix_v_row_scale", prefix_v_row_scale)):
        if rs is None:
            continue
        _dev(op, rs)
        if rs.dtype != torch.float32 or rs.numel() != Lp or not rs.is_contiguous():
            _fail(op, f"{nm} must be a contiguous float32 tensor of prefix_len ({Lp}) values")
        setattr(a, nm, rs.data_ptr())
    if mask is not None:
        a.mask_mode, a.q_offset, a.window = mask.mode, mask.q_offset, mask.window
        if mask.mode == capi.MI_MASK_BLOCK_CAUSAL:
            n = len(mask.seg_q_end)
            if n < 1 or n > capi.MI_MAX_SEGMENTS or len(mask.seg_k_end) != n or len(mask.seg_causal) != n:
                _fail(op, f"block-causal mask needs 1..{capi.MI_MAX_SEGMENTS} segments")
            a.n_segments = n
            for i in range(n):
                a.seg_q_end[i], a.seg_k_end[i], a.seg_causal[i] = int(mask.seg_q_end[i]), int(mask.seg_k_end[i]), int(mask.seg_causal[i])
    if kv_valid_len is not None:
        if kv_valid_len.dtype != torch.int32 or kv_valid_len.numel() != B or not kv_valid_len.is_contiguous():
            _fail(op, "kv_valid_len must be a contiguous int32 tensor of length batch")
        a.kv_valid_len = kv_valid_len.data_ptr()
    if key_mask is not None:
        if key_mask.dtype != torch.float32 or not key_mask.is_contiguous():
            _fail(op, "d_mask must be a contiguous float32 tensor")
        if key_mask.numel() == Lp + Lk:
            a.key_mask_batch_stride = 0
        elif key_mask.numel() == B * (Lp + Lk):
            a.key_mask_batch_stride = Lp + Lk
        else:
            _fail(op, "d_mask must hold Lk (or batch*Lk) values")
        a.key_mask = key_mask.data_ptr()
    for nm, tab, rows in (("rope_q", rope_q, Lq), ("rope_k", rope_k, Lk)):
        if tab is None:
            continue
        cs, sn = tab
        _dev(op, cs, sn)
        for t in (cs, sn):
            if t.dtype != torch.float32 or tuple(t.shape) != (rows, hd // 2) or not t.is_contiguous():
                _fail(op, f"{nm} tables must be contiguous float32 ({rows}, head_dim/2)")
        if nm == "rope_q":
            a.rope_cos_q, a.rope_sin_q = cs.data_ptr(), sn.data_ptr()
        else:
            a.rope_cos_k, a.rope_sin_k = cs.data_ptr(), sn.data_ptr()
    a.rope_split_half = int(bool(rope_split_half))
    if rope_k_scratch is not None:
        if rope_k is None:
            _fail(op, "rope_k_scratch given without rope_k tables")
        if rope_k_scratch.dtype != q.dtype or not rope_k_scratch.is_contiguous() or rope_k_scratch.numel() < k.numel():
            _fail(op, "rope_k_scratch must be contiguous, of Q's dtype and at least as large as K")
        a.rope_k_scratch = rope_k_scratch.data_ptr()
    if logit_bias is not None:
        _dev(op, logit_bias)
        if logit_bias.dtype != torch.float32 or logit_bias.dim() != 2 or logit_bias.stride(1) != 1:
            _fail(op, "logit_bias must be a 2-D float32 tensor, contiguous along columns")
        if logit_bias.shape[0] != Lq - bias_q0:
            _fail(op, f"logit_bias must have one row per query row from bias_q0 on ({Lq - bias_q0}), has {logit_bias.shape[0]}")
        a.logit_bias, a.bias_q0, a.bias_cols = logit_bias.data_ptr(), bias_q0, logit_bias.shape[1]
        a.bias_row_stride = logit_bias.stride(0)
    if lse_out is not None:
        _dev(op, lse_out)
        if lse_out.dtype != torch.float32 or lse_out.numel() != B * num_heads * Lq or not lse_out.is_contiguous():
            _fail(op, "lse_out must be a contiguous float32 tensor of batch * heads * Lq values")
        a.lse_out = lse_out.data_ptr()
    a.stream = _stream()
    if split_scratch is not False:
        need = int(capi.lib().mi_sdpa_split_scratch_bytes(C.byref(a)))
        if need > 0:
            if split_scratch is None:
                split_scratch = _own_split_scratch(q.device, need)
            _dev(op, split_scratch)
            if not split_scratch.is_contiguous():
                _fail(op, "split_scratch must be contiguous")
            a.split_scratch = split_scratch.data_ptr()
            a.split_scratch_bytes = split_scratch.numel() * split_scratch.element_size()
    capi.check(capi.lib().mi_sdpa_forward(C.byref(a)), op)
    return out


_split_scratch_cache = {}


def _own_split_scratch(device, nbytes: int) -> torch.Tensor:
    """The scratch this layer lends when the caller brings none: one per (device, current stream), grown on demand. Calls
    on one stream run in order and may share it; calls on different streams may overlap on the GPU and must not."""
    key = (device, _stream())
    t = _split_scratch_cache.get(key)
    if t is None or t.numel() < nbytes:
        t = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _split_scratch_cache[key] = t
    return t


def flash_attention_forward(Q, K, V, d_mask, num_heads: int, causal: bool, out: Optional[torch.Tensor] = None):
    """out = softmax(Q K^T / sqrt(d) [+ key mask]) V per head. causal aligns the last query with the
    last key (q_offset = Lk - Lq), as the windowed form does."""
    op = "flash_attention_forward"
    Lq, Lk = Q.shape[-2], K.shape[-2]
    mask = SdpaMask.causal(Lk - Lq) if causal else None
    return sdpa_forward(Q, K, V, num_heads, out=out, key_mask=d_mask, mask=mask, op=op)


def flash_attention_varlen_forward(q, k, v, cu_q, cu_k, n_seqs: int, max_q: int, max_k: int, num_heads: int, head_dim: int,
                                   causal: bool, out: Optional[torch.Tensor] = None):
    """Attention over n_seqs sequences of different lengths packed along the row axis: sequence i owns query rows
    [cu_q[i], cu_q[i+1]) of q / out and key rows [cu_k[i], cu_k[i+1]) of k / v (device int32 arrays of n_seqs + 1 offsets);
    max_q / max_k bound the sequence lengths. Argument order of bt::flash_attention_varlen_forward (src/dit/krea2.cpp:574)."""
    op = "flash_attention_varlen_forward"
    _dev(op, q, k, v, cu_q, cu_k, out)
    dt = _dtype_code(op, q)
    if q.dim() != 2 or k.dim() != 2 or v.dim() != 2 or q.stride(1) != 1 or k.stride(1) != 1 or v.stride(1) != 1:
        _fail(op, "q, k, v must be 2-D packed (total rows, heads*head_dim), contiguous along columns")
    if k.dtype != q.dtype or v.dtype != q.dtype or q.shape[1] != num_heads * head_dim or k.shape[1] != q.shape[1] or tuple(v.shape) != tuple(k.shape):
        _fail(op, "q, k, v must share dtype and heads*head_dim columns; k and v the same shape")
    for t, nm in ((cu_q, "cu_q"), (cu_k, "cu_k")):
        if t.dtype != torch.int32 or t.numel() != n_seqs + 1 or not t.is_contiguous():
            _fail(op, f"{nm} must be a contiguous int32 tensor of n_seqs + 1 offsets")
    if n_seqs <= 0 or max_q < 0 or max_k < 0:
        _fail(op, "n_seqs must be positive, max_q and max_k non-negative")
    if out is None:
        out = torch.empty_like(q)
    if out.shape != q.shape or out.dtype != q.dtype or out.stride(1) != 1:
        _fail(op, "out must have q's shape and dtype")
    a = capi.MiSdpaArgs()
    a.struct_size = C.sizeof(capi.MiSdpaArgs)
    a.dtype = dt
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr()
    a.batch, a.num_heads, a.head_dim = n_seqs, num_heads, head_dim
    a.q_len, a.kv_len = max_q, max_k
    a.q_row_stride, a.k_row_stride, a.v_row_stride, a.o_row_stride = q.stride(0), k.stride(0), v.stride(0), out.stride(0)
    a.q_batch_stride = a.k_batch_stride = a.v_batch_stride = a.o_batch_stride = 8      # ignored for packed sequences
    a.mask_mode = capi.MI_MASK_CAUSAL if causal else capi.MI_MASK_NONE
    a.cu_seqlens_q, a.cu_seqlens_k = cu_q.data_ptr(), cu_k.data_ptr()
    a.stream = _stream()
    capi.check(capi.lib().mi_sdpa_forward(C.byref(a)), op)
    return out


def flash_attention_windowed_forward(Q, K, V, d_mask, num_heads: int, window: int, out: Optional[torch.Tensor] = None):
    """Causal attention with q_offset = Lk - Lq: query row r sees keys [0, q_offset + r]; window > 0
    keeps the last `window` of them, window = 0 is unbounded (src/dit/qwenimage21_forward.cpp:8-13)."""
    op = "flash_attention_windowed_forward"
    if window < 0:
        _fail(op, "window must be >= 0")
    Lq, Lk = Q.shape[-2], K.shape[-2]
    return sdpa_forward(Q, K, V, num_heads, out=out, key_mask=d_mask, mask=SdpaMask.causal(Lk - Lq, window), op=op)


def _mat(op: str, t, name: str, dtype, rows=None, cols=None):
    """A dense 2-D (or, for activations, 3-D batch-major) operand of the projection ops."""
    if t is None:
        return
    _dev(op, t)
    if t.dtype != dtype:
        _fail(op, f"{name} has dtype {t.dtype}, expected {dtype}")
    if not t.is_contiguous():
        _fail(op, f"{name} must be contiguous")
    if rows is not None and t.shape[-2] != rows:
        _fail(op, f"{name} has {t.shape[-2]} rows, expected {rows}")
    if cols is not None and t.shape[-1] != cols:
        _fail(op, f"{name} has {t.shape[-1]} columns, expected {cols}")


def _weight(op: str, W, scales, name: str, dtype, rows=None, cols=None) -> int:
    """A weight operand: of the activation dtype, or INT8 with FP32 per-output-row scales. Returns the scales pointer (0: none)."""
    if scales is None:
        _mat(op, W, name, dtype, rows=rows, cols=cols)
        return 0
    _mat(op, W, name, torch.int8, rows=rows, cols=cols)
    _dev(op, scales)
    if scales.dtype != torch.float32 or scales.numel() != W.shape[0] or not scales.is_contiguous():
        _fail(op, f"{name} scales must hold {W.shape[0]} contiguous float32 values (one per output row)")
    return scales.data_ptr()


def _bias(op: str, b, name: str, dtype, n: int):
    if b is None:
        return 0
    _dev(op, b)
    if b.dtype != dtype or b.numel() != n or not b.is_contiguous():
        _fail(op, f"{name} must be a contiguous {dtype} vector of {n} values")
    return b.data_ptr()


def linear_batched(W, bias, X, Y: Optional[torch.Tensor] = None, W_scales: Optional[torch.Tensor] = None,
                   op: str = "linear_batched"):
    """Y = X W^T + bias; W (out_features, in_features), X (..., in_features). With W_scales, W is INT8 and
    Y = (X W^T) * scales + bias (see linear_forward_batched_int8w_fp16)."""
    _dev(op, W, X)
    if W.dim() != 2 or X.shape[-1] != W.shape[1]:
        _fail(op, f"X has {X.shape[-1]} columns, W is {tuple(W.shape)}")
    w_scales = _weight(op, W, W_scales, "W", X.dtype)
    _mat(op, X, "X", X.dtype)
    rows = X.numel() // X.shape[-1]
    if Y is None:
        Y = torch.empty(*X.shape[:-1], W.shape[0], dtype=X.dtype, device=X.device)
    _mat(op, Y, "Y", X.dtype, cols=W.shape[0])
    if Y.numel() != rows * W.shape[0]:
        _fail(op, "Y has the wrong number of rows")
    a = capi.MiLinearArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, X)
    a.x, a.w, a.y = X.data_ptr(), W.data_ptr(), Y.data_ptr()
    a.bias = _bias(op, bias, "bias", X.dtype, W.shape[0])
    a.rows, a.in_features, a.out_features = rows, W.shape[1], W.shape[0]
    a.w_scales = w_scales
    a.stream = _stream()
    capi.check(capi.lib().mi_linear_forward(C.byref(a)), op)
    return Y


def linear_forward_batched_int8w_fp16(W_int8, scales, bias, X, Y: Optional[torch.Tensor] = None):
    """W8A16 linear layer, argument order of bt::linear_forward_batched_int8w_fp16 (src/unet_blocks.cpp:238-240):
    W_int8 (out, in) INT8, scales (out, 1) FP32, bias of X's dtype or None."""
    return linear_batched(W_int8, bias, X, Y, W_scales=scales, op="linear_forward_batched_int8w_fp16")


def fused_linear_geglu(X, W, b, Y: Optional[torch.Tensor] = None, W_scales: Optional[torch.Tensor] = None,
                       op: str = "fused_linear_geglu"):
    """Y = a * gelu_exact(g), [a | g] = X W^T + b with W (2*D_out, D_in), b (2*D_out): the fused FF1 + GEGLU of the
    U-Net transformer block (brodiffusion::fused_linear_geglu, include/brodiffusion/fused_transformer.h:20-35). With
    W_scales, W is INT8 with one FP32 scale per row (see fused_linear_geglu_int8w)."""
    _dev(op, X, W, b, Y, W_scales)
    if W.dim() != 2 or W.shape[0] % 2 != 0 or X.shape[-1] != W.shape[1]:
        _fail(op, f"W must be (2*D_out, D_in) with D_in = {X.shape[-1]}, got {tuple(W.shape)}")
    d_out = W.shape[0] // 2
    scales_ptr = _weight(op, W, W_scales, "W", X.dtype)
    _mat(op, X, "X", X.dtype)
    rows = X.numel() // X.shape[-1]
    if Y is None:
        Y = torch.empty(*X.shape[:-1], d_out, dtype=X.dtype, device=X.device)
    _mat(op, Y, "Y", X.dtype, cols=d_out)
    if Y.numel() != rows * d_out:
        _fail(op, "Y has the wrong number of rows")
    a = capi.MiLinearArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, X)
    a.x, a.w, a.y = X.data_ptr(), W.data_ptr(), Y.data_ptr()
    a.bias = _bias(op, b, "b", X.dtype, W.shape[0])
    a.w_scales = scales_ptr
    a.rows, a.in_features, a.out_features = rows, W.shape[1], d_out
    a.stream = _stream()
    capi.check(capi.lib().mi_linear_geglu_forward(C.byref(a)), op)
    return Y


def fused_linear_geglu_int8w(X, W_int8, W_scales, b, Y: Optional[torch.Tensor] = None):
    """The W8A16 overload of brodiffusion::fused_linear_geglu (include/brodiffusion/fused_transformer.h:37-48): W_int8
    (2*D_out, D_in) INT8, W_scales (2*D_out, 1) FP32, b (2*D_out) of X's dtype. The reference runs its INT8-weight linear
    layer into a 16-bit (B, 2*D_out) buffer and a GEGLU pass over it (src/fused_transformer.cu:360-396); this is one
    GEMM that rounds the two halves where the buffer would."""
    return fused_linear_geglu(X, W_int8, b, Y, W_scales=W_scales, op="fused_linear_geglu_int8w")


def add_inplace_vec(Y, X):
    """Y += X, same shape and dtype (brodiffusion::add_inplace_vec, include/brodiffusion/fused_transformer.h:50-53)."""
    op = "add_inplace_vec"
    _dev(op, Y, X)
    if tuple(Y.shape) != tuple(X.shape) or Y.dtype != X.dtype or not Y.is_contiguous() or not X.is_contiguous():
        _fail(op, "Y and X must match in shape and dtype and be contiguous")
    capi.check(capi.lib().mi_add_inplace(Y.data_ptr(), X.data_ptr(), Y.numel(), _dtype_code(op, Y), _stream()), op)
    return Y


def add_inplace_row_bias(Y, bias):
    """Y[i, j] += bias[j]; bias holds Y's column count of values, any shape
    (brodiffusion::add_inplace_row_bias, include/brodiffusion/fused_transformer.h:55-61)."""
    op = "add_inplace_row_bias"
    _dev(op, Y, bias)
    if Y.dim() != 2 or Y.stride(1) != 1:
        _fail(op, "Y must be 2-D, contiguous along columns")
    if bias.dtype != Y.dtype or bias.numel() != Y.shape[1] or not bias.is_contiguous():
        _fail(op, f"bias must hold {Y.shape[1]} values of Y's dtype")
    capi.check(capi.lib().mi_add_row_bias(Y.data_ptr(), bias.data_ptr(), Y.shape[0], Y.shape[1], Y.stride(0), _dtype_code(op, Y), _stream()), op)
    return Y


def flash_attention_scratch_bytes(batch: int, q_len: int, kv_len: int, inner: int, with_kv: bool) -> int:
    return int(capi.lib().mi_flash_attention_scratch_bytes(batch, q_len, kv_len, inner, int(with_kv)))


def _attn_block(op: str, fn_name: str, X, Ctx, K, V, Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads, causal, out, scratch,
                scales=(None, None, None, None)):
    _dev(op, X, Ctx, K, V, Wq, Wk, Wv, Wo, d_mask, out, scratch)
    dt = X.dtype
    B, Lq, Cx, _, _ = _as3(op, X, "X")
    if not X.is_contiguous():
        _fail(op, "X must be contiguous")
    if Wq.dim() != 2 or Wo.dim() != 2:
        _fail(op, "Wq and Wo must be 2-D (out_features, in_features)")
    inner, Cout = Wq.shape[0], Wo.shape[0]
    a = capi.MiAttnBlockArgs()
    a.struct_size = C.sizeof(a)
    a.wq_scales = _weight(op, Wq, scales[0], "Wq", dt, cols=Cx)
    a.wo_scales = _weight(op, Wo, scales[3], "Wo", dt, cols=inner)
    a.dtype = _dtype_code(op, X)
    a.x, a.wq, a.wo = X.data_ptr(), Wq.data_ptr(), Wo.data_ptr()
    a.bq, a.bo = _bias(op, bq, "bq", dt, inner), _bias(op, bo, "bo", dt, Cout)
    Lk = Lq
    if K is not None:
        Bk, Lk, Ck, _, _ = _as3(op, K, "K")
        if Bk != B or Ck != inner or tuple(V.shape) != tuple(K.shape):
            _fail(op, f"K / V must be ({B} x) (Lk, {inner}) and alike")
        _mat(op, K, "K", dt)
        _mat(op, V, "V", dt)
        a.k, a.v = K.data_ptr(), V.data_ptr()
    else:
        Cc = Cx
        if Ctx is not None:
            Bc, Lk, Cc, _, _ = _as3(op, Ctx, "Ctx")
            if Bc != B:
                _fail(op, f"Ctx has batch {Bc}, X has {B}")
            _mat(op, Ctx, "Ctx", dt)
            a.ctx = Ctx.data_ptr()
        a.wk_scales = _weight(op, Wk, scales[1], "Wk", dt, rows=inner, cols=Cc)
        a.wv_scales = _weight(op, Wv, scales[2], "Wv", dt, rows=inner, cols=Cc)
        a.wk, a.wv = Wk.data_ptr(), Wv.data_ptr()
        a.bk, a.bv = _bias(op, bk, "bk", dt, inner), _bias(op, bv, "bv", dt, inner)
        a.ctx_channels = Cc
    a.batch, a.q_len, a.kv_len = B, Lq, Lk
    a.channels, a.inner, a.out_channels = Cx, inner, Cout
    a.num_heads, a.causal = num_heads, int(bool(causal))
    if d_mask is not None:
        if d_mask.dtype != torch.float32 or not d_mask.is_contiguous() or d_mask.numel() not in (Lk, B * Lk):
            _fail(op, "d_mask must be contiguous float32 with Lk (or batch*Lk) values")
        a.key_mask = d_mask.data_ptr()
        a.key_mask_batch_stride = Lk if (d_mask.numel() == B * Lk and B > 1) else 0
    if out is None:
        out = torch.empty(*X.shape[:-1], Cout, dtype=dt, device=X.device)
    _mat(op, out, "out", dt, cols=Cout)
    if out.numel() != B * Lq * Cout:
        _fail(op, "out has the wrong number of rows")
    a.out = out.data_ptr()
    need = flash_attention_scratch_bytes(B, Lq, Lk, inner, K is None)
    if scratch is None:
        scratch = torch.empty(need, dtype=torch.uint8, device=X.device)
    if not scratch.is_contiguous():
        _fail(op, "scratch must be contiguous")
    a.scratch, a.scratch_bytes = scratch.data_ptr(), scratch.numel() * scratch.element_size()
    a.stream = _stream()
    capi.check(getattr(capi.lib(), fn_name)(C.byref(a)), op)
    return out


def flash_attention_qkvo_forward(X, Ctx, Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads: int, causal: bool,
                                 out: Optional[torch.Tensor] = None, scratch: Optional[torch.Tensor] = None):
    """out = attention(X Wq^T + bq, S Wk^T + bk, S Wv^T + bv) Wo^T + bo with S = Ctx, or X when Ctx is None.
    `scratch` (flash_attention_scratch_bytes(..., with_kv=True) bytes) holds the projections; None allocates it."""
    return _attn_block("flash_attention_qkvo_forward", "mi_flash_attention_qkvo_forward", X, Ctx, None, None,
                       Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads, causal, out, scratch)


def flash_attention_q_with_kv_cached_forward(X, K, V, Wq, bq, Wo, bo, d_mask, num_heads: int, causal: bool,
                                             out: Optional[torch.Tensor] = None, scratch: Optional[torch.Tensor] = None):
    """As flash_attention_qkvo_forward with K and V already projected (the cross-attention K/V cache)."""
    return _attn_block("flash_attention_q_with_kv_cached_forward", "mi_flash_attention_q_with_kv_cached_forward", X, None, K, V,
                       Wq, bq, None, None, None, None, Wo, bo, d_mask, num_heads, causal, out, scratch)


def flash_attention_qkvo_int8w_fp16(X, Ctx, Wq_int8, Wq_scales, bq, Wk_int8, Wk_scales, bk, Wv_int8, Wv_scales, bv,
                                    Wo_int8, Wo_scales, bo, d_mask, num_heads: int, causal: bool,
                                    out: Optional[torch.Tensor] = None, scratch: Optional[torch.Tensor] = None):
    """flash_attention_qkvo_forward with INT8 weights and FP32 per-output-row scales (W8A16), argument order of
    bt::flash_attention_qkvo_int8w_fp16 (src/unet_blocks.cpp:256-262)."""
    return _attn_block("flash_attention_qkvo_int8w_fp16", "mi_flash_attention_qkvo_forward", X, Ctx, None, None,
                       Wq_int8, bq, Wk_int8, bk, Wv_int8, bv, Wo_int8, bo, d_mask, num_heads, causal, out, scratch,
                       scales=(Wq_scales, Wk_scales, Wv_scales, Wo_scales))


def flash_attention_q_with_kv_cached_int8w_fp16(X, K, V, Wq_int8, Wq_scales, bq, Wo_int8, Wo_scales, bo, d_mask, num_heads: int,
                                                causal: bool, out: Optional[torch.Tensor] = None,
                                                scratch: Optional[torch.Tensor] = None):
    """W8A16 form of flash_attention_q_with_kv_cached_forward (src/unet_blocks.cpp:305-310)."""
    return _attn_block("flash_attention_q_with_kv_cached_int8w_fp16", "mi_flash_attention_q_with_kv_cached_forward", X, None, K, V,
                       Wq_int8, bq, None, None, None, None, Wo_int8, bo, d_mask, num_heads, causal, out, scratch,
                       scales=(Wq_scales, None, None, Wo_scales))


def flash_attention_project_kv_int8w_fp16(ctx, Wk_int8, Wk_scales, bk, Wv_int8, Wv_scales, bv,
                                          K_out: Optional[torch.Tensor] = None, V_out: Optional[torch.Tensor] = None):
    """W8A16 form of flash_attention_project_kv (src/unet.cpp:470-474)."""
    return flash_attention_project_kv(ctx, Wk_int8, bk, Wv_int8, bv, K_out, V_out, scales=(Wk_scales, Wv_scales),
                                      op="flash_attention_project_kv_int8w_fp16")


def flash_attention_project_kv(ctx, Wk, bk, Wv, bv, K_out: Optional[torch.Tensor] = None, V_out: Optional[torch.Tensor] = None,
                               scales=(None, None), op: str = "flash_attention_project_kv"):
    """K_out = ctx Wk^T + bk, V_out = ctx Wv^T + bv in one launch (fills the cross-attention K/V cache)."""
    _dev(op, ctx, Wk, Wv, K_out, V_out)
    dt = ctx.dtype
    B, Lk, Cc, _, _ = _as3(op, ctx, "ctx")
    _mat(op, ctx, "ctx", dt)
    if Wk.dim() != 2 or tuple(Wv.shape) != tuple(Wk.shape):
        _fail(op, "Wk and Wv must be 2-D and alike")
    inner = Wk.shape[0]
    wk_scales = _weight(op, Wk, scales[0], "Wk", dt, cols=Cc)
    wv_scales = _weight(op, Wv, scales[1], "Wv", dt, cols=Cc)
    if K_out is None:
        K_out = torch.empty(*ctx.shape[:-1], inner, dtype=dt, device=ctx.device)
    if V_out is None:
        V_out = torch.empty(*ctx.shape[:-1], inner, dtype=dt, device=ctx.device)
    for t, nm in ((K_out, "K_out"), (V_out, "V_out")):
        _mat(op, t, nm, dt, cols=inner)
        if t.numel() != B * Lk * inner:
            _fail(op, f"{nm} has the wrong number of rows")
    a = capi.MiAttnBlockArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, ctx)
    a.ctx, a.wk, a.wv = ctx.data_ptr(), Wk.data_ptr(), Wv.data_ptr()
    a.bk, a.bv = _bias(op, bk, "bk", dt, inner), _bias(op, bv, "bv", dt, inner)
    a.k, a.v = K_out.data_ptr(), V_out.data_ptr()
    a.wk_scales, a.wv_scales = wk_scales, wv_scales
    a.batch, a.kv_len, a.ctx_channels, a.inner = B, Lk, Cc, inner
    a.stream = _stream()
    capi.check(capi.lib().mi_flash_attention_project_kv(C.byref(a)), op)
    return K_out, V_out


def _rope(op: str, X, cos, sin, head_dim, num_heads, out, per_head: bool, split_half: bool):
    _dev(op, X, cos, sin, out)
    dt = _dtype_code(op, X)
    if X.dim() != 2 or X.stride(1) != 1:
        _fail(op, "X must be (L, heads*head_dim), contiguous along columns")
    L, D = X.shape
    if head_dim <= 0 or num_heads <= 0 or D != head_dim * num_heads:
        _fail(op, "D must equal head_dim * num_heads")
    trows = L * num_heads if per_head else L
    for t in (cos, sin):
        if t.dtype != torch.float32 or tuple(t.shape) != (trows, head_dim // 2) or not t.is_contiguous():
            _fail(op, f"cos/sin must be contiguous float32 ({trows}, head_dim/2)")
    if out is None:
        out = torch.empty_like(X)
    if out.shape != X.shape or out.dtype != X.dtype or out.stride(1) != 1:
        _fail(op, "out must have X's shape and dtype")
    a = capi.MiRopeArgs()
    a.struct_size = C.sizeof(capi.MiRopeArgs)
    a.dtype = dt
    a.x, a.out, a.cos, a.sin = X.data_ptr(), out.data_ptr(), cos.data_ptr(), sin.data_ptr()
    a.rows, a.num_heads, a.head_dim = L, num_heads, head_dim
    a.x_row_stride, a.out_row_stride = X.stride(0), out.stride(0)
    a.split_half, a.per_head = int(split_half), int(per_head)
    a.stream = _stream()
    capi.check(capi.lib().mi_rope_apply(C.byref(a)), op)
    return out


def rope_apply(X, cos, sin, head_dim: int, num_heads: int, out: Optional[torch.Tensor] = None, split_half: bool = False):
    return _rope("rope_apply", X, cos, sin, head_dim, num_heads, out, False, split_half)


def rope_apply_perhead(X, cos, sin, head_dim: int, num_heads: int, out: Optional[torch.Tensor] = None,
                       split_half: bool = False):
    return _rope("rope_apply_perhead", X, cos, sin, head_dim, num_heads, out, True, split_half)


def scale_rows(X, scale: float = 1.0, row_scale: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """out = X * scale * row_scale[:, None]: the prefix-KV dial of the Qwen-Image cached step
    (src/dit/qwenimage21_forward.cpp:612-645) applied to a copy of the prefix rows, the cache itself untouched."""
    op = "scale_rows"
    _dev(op, X, row_scale, out)
    if X.dim() != 2 or X.stride(1) != 1:
        _fail(op, "X must be 2-D, contiguous along columns")
    if out is None:
        out = torch.empty_like(X)
    if out.shape != X.shape or out.dtype != X.dtype or out.stride(1) != 1:
        _fail(op, "out must have X's shape and dtype")
    a = capi.MiScaleRowsArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, X)
    a.x, a.out, a.scale = X.data_ptr(), out.data_ptr(), float(scale)
    if row_scale is not None:
        if row_scale.dtype != torch.float32 or row_scale.numel() != X.shape[0] or not row_scale.is_contiguous():
            _fail(op, f"row_scale must hold {X.shape[0]} float32 values (one per row)")
        a.row_scale = row_scale.data_ptr()
    a.rows, a.cols = X.shape
    a.x_row_stride, a.out_row_stride = X.stride(0), out.stride(0)
    a.stream = _stream()
    capi.check(capi.lib().mi_scale_rows(C.byref(a)), op)
    return out


def headnorm_rope(X, gain, eps: float, cos, sin, head_dim: int, num_heads: int, out: Optional[torch.Tensor] = None,
                  cache_out: Optional[torch.Tensor] = None, split_half: bool = False):
    """headnorm + rope_apply of the DiT blocks (src/dit/qwenimage21_forward.cpp:582-585, src/dit/flux.cpp:462-469) in
    one pass: per (row, head) RMS normalisation with `gain` (head_dim), then the rotation (cos = sin = None: the
    normalisation alone). cache_out (rows <= X's rows): its rows also receive the result — the prefix rows of K going
    into the prefix cache (qwenimage21_forward.cpp:587-597)."""
    op = "headnorm_rope"
    _dev(op, X, gain, cos, sin, out, cache_out)
    if X.dim() != 2 or X.stride(1) != 1 or X.shape[1] != head_dim * num_heads:
        _fail(op, "X must be (L, head_dim * num_heads), contiguous along columns")
    if gain.dtype != X.dtype or gain.numel() != head_dim or not gain.is_contiguous():
        _fail(op, "gain must hold head_dim values of X's dtype")
    if out is None:
        out = torch.empty_like(X)
    if out.shape != X.shape or out.dtype != X.dtype or out.stride(1) != 1:
        _fail(op, "out must have X's shape and dtype")
    a = capi.MiHeadnormRopeArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, X)
    a.x, a.out, a.gain = X.data_ptr(), out.data_ptr(), gain.data_ptr()
    if (cos is None) != (sin is None):
        _fail(op, "cos and sin must be given together")
    if cos is not None:
        for t in (cos, sin):
            if t.dtype != torch.float32 or tuple(t.shape) != (X.shape[0], head_dim // 2) or not t.is_contiguous():
                _fail(op, "cos/sin must be contiguous float32 (L, head_dim/2)")
        a.cos, a.sin = cos.data_ptr(), sin.data_ptr()
    a.eps = eps
    a.split_half = int(bool(split_half))
    a.rows, a.num_heads, a.head_dim = X.shape[0], num_heads, head_dim
    a.x_row_stride, a.out_row_stride = X.stride(0), out.stride(0)
    if cache_out is not None:
        if cache_out.dim() != 2 or cache_out.dtype != X.dtype or cache_out.shape[1] != X.shape[1] or cache_out.stride(1) != 1 \
                or cache_out.shape[0] > X.shape[0]:
            _fail(op, "cache_out must be (rows <= L, head_dim * num_heads) of X's dtype")
        a.out2, a.out2_rows, a.out2_row_stride = cache_out.data_ptr(), cache_out.shape[0], cache_out.stride(0)
    a.stream = _stream()
    capi.check(capi.lib().mi_headnorm_rope(C.byref(a)), op)
    return out


def joint_attention(Q, K, V, cos, sin, head_dim: int, num_heads: int, out: Optional[torch.Tensor] = None,
                    Qr: Optional[torch.Tensor] = None, Kr: Optional[torch.Tensor] = None, split_half: bool = False):
    """Full-bidirectional joint attention with RoPE on Q and K (include/brodiffusion/dit/common.h:74-88).
    Q is rotated while it is loaded. With a Kr scratch (K's shape and dtype) K is rotated into it by one
    pass and, as in the reference, Kr holds RoPE(K) afterwards; without one K is rotated tile by tile
    inside the attention kernel (slower; adjacent pairs only). Qr is accepted and left untouched. split_half selects the
    pair convention of the rotation as in rope_apply."""
    op = "joint_attention"
    if Q.dim() != 2 or Q.shape[1] != head_dim * num_heads:
        _fail(op, "D must equal head_dim * num_heads")
    if K.shape != Q.shape or V.shape != Q.shape:
        _fail(op, "Q/K/V must share shape (L, D)")
    if Kr is not None and (Kr.shape != K.shape or Kr.dtype != K.dtype):
        _fail(op, "Kr must have K's shape and dtype")
    return sdpa_forward(Q, K, V, num_heads, out=out, rope_q=(cos, sin), rope_k=(cos, sin), rope_k_scratch=Kr,
                        rope_split_half=split_half, op=op)


def attention_map_avg(q, k, lse, num_heads: int, *, scale: Optional[float] = None, logit_bias: Optional[torch.Tensor] = None,
                      bias_q0: int = 0, key_mask: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """(Lq, Lk) float32 map: the softmax of every head averaged over the heads. `lse` is what sdpa_forward wrote to
    lse_out for the same q, k, scale, bias and key_mask (float32 (Lk,), 1 = valid; masked columns of the map are 0)."""
    op = "attention_map_avg"
    _dev(op, q, k, lse, logit_bias, key_mask, out)
    if q.dim() != 2 or k.dim() != 2 or q.stride(1) != 1 or k.stride(1) != 1 or q.shape[1] != k.shape[1] or q.dtype != k.dtype:
        _fail(op, "q and k must be 2-D (L, heads*head_dim) of one dtype, contiguous along columns")
    Lq, Lk = q.shape[0], k.shape[0]
    if lse.dtype != torch.float32 or lse.numel() != num_heads * Lq or not lse.is_contiguous():
        _fail(op, "lse must be contiguous float32 (heads, Lq)")
    if out is None:
        out = torch.empty(Lq, Lk, dtype=torch.float32, device=q.device)
    if out.dtype != torch.float32 or tuple(out.shape) != (Lq, Lk) or out.stride(1) != 1:
        _fail(op, "out must be float32 (Lq, Lk)")
    a = capi.MiAttentionMapArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = _dtype_code(op, q)
    a.q, a.k, a.lse, a.map = q.data_ptr(), k.data_ptr(), lse.data_ptr(), out.data_ptr()
    a.num_heads, a.head_dim, a.q_len, a.kv_len = num_heads, q.shape[1] // num_heads, Lq, Lk
    a.q_row_stride, a.k_row_stride, a.map_row_stride = q.stride(0), k.stride(0), out.stride(0)
    a.scale = 0.0 if scale is None else float(scale)
    if logit_bias is not None:
        if logit_bias.dtype != torch.float32 or logit_bias.dim() != 2 or logit_bias.stride(1) != 1 or logit_bias.shape[0] != Lq - bias_q0:
            _fail(op, "logit_bias must be float32 (Lq - bias_q0, cols)")
        a.logit_bias, a.bias_q0, a.bias_cols, a.bias_row_stride = logit_bias.data_ptr(), bias_q0, logit_bias.shape[1], logit_bias.stride(0)
    if key_mask is not None:
        if key_mask.dtype != torch.float32 or key_mask.numel() != Lk or not key_mask.is_contiguous():
            _fail(op, "key_mask must be contiguous float32 (Lk,)")
        a.key_mask = key_mask.data_ptr()
    a.stream = _stream()
    capi.check(capi.lib().mi_attention_map_avg(C.byref(a)), op)
    return out


def joint_attention_traced(Q, K, V, cos, sin, head_dim: int, num_heads: int, out: Optional[torch.Tensor] = None,
                           attn_avg: Optional[torch.Tensor] = None, Qr: Optional[torch.Tensor] = None,
                           Kr: Optional[torch.Tensor] = None, txt_len: int = 0, image_text_bias: Optional[torch.Tensor] = None):
    """dit::joint_attention_traced (src/dit/common.cpp:198-329) on the device: RoPE on Q and K into Qr / Kr, attention with
    the optional image->text logit bias ((L - txt_len, txt_len) float32, added to the scaled scores of image rows against
    text keys), and the head-averaged (L, L) float32 softmax map. Returns (out, attn_avg)."""
    op = "joint_attention_traced"
    _dev(op, Q, K, V, cos, sin, image_text_bias)
    if Q.dim() != 2 or Q.shape[1] != head_dim * num_heads:
        _fail(op, "D must equal head_dim * num_heads")
    L = Q.shape[0]
    if tuple(K.shape) != tuple(Q.shape) or tuple(V.shape) != tuple(Q.shape):
        _fail(op, "Q/K/V must share shape (L, D)")
    if image_text_bias is not None:
        if txt_len < 0 or txt_len > L:
            _fail(op, "txt_len out of range for bias")
        if image_text_bias.dtype != torch.float32:
            _fail(op, "image_text_bias must be FP32")
        if tuple(image_text_bias.shape) != (L - txt_len, txt_len):
            _fail(op, "image_text_bias must be (img_len, txt_len)")
    Qr = rope_apply(Q, cos, sin, head_dim, num_heads, out=Qr)
    Kr = rope_apply(K, cos, sin, head_dim, num_heads, out=Kr)
    lse = torch.empty(num_heads, L, dtype=torch.float32, device=Q.device)
    bias = image_text_bias if (image_text_bias is not None and txt_len > 0 and txt_len < L) else None
    out = sdpa_forward(Qr, Kr, V, num_heads, out=out, logit_bias=bias, bias_q0=txt_len, lse_out=lse, op=op)
    attn_avg = attention_map_avg(Qr, Kr, lse, num_heads, logit_bias=bias, bias_q0=txt_len, out=attn_avg)
    return out, attn_avg


def cross_attention_forward_with_attn(X, Ctx, Wq, Wk, Wv, Wo, d_mask, logit_bias, num_heads: int,
                                      out: Optional[torch.Tensor] = None, attn_avg: Optional[torch.Tensor] = None):
    """bt::cross_attention_forward_with_attn as the U-Net's traced cross attention calls it (src/unet_blocks.cpp:282-290):
    Q = X Wq^T, K = Ctx Wk^T, V = Ctx Wv^T (no biases), attention with the optional additive logit bias (float32
    (Lq, Lk)) and key mask (float32 (Lk,), 1 = valid), output projection with Wo (no bias: the caller adds it), and
    the softmax averaged over the heads as a float32 (Lq, Lk) map. All on the device. Returns (out, attn_avg)."""
    op = "cross_attention_forward_with_attn"
    _dev(op, X, Ctx, Wq, Wk, Wv, Wo, d_mask, logit_bias, out, attn_avg)
    if X.dim() != 2 or Ctx.dim() != 2:
        _fail(op, "X and Ctx must be 2-D (rows, channels)")
    Lq, Lk = X.shape[0], Ctx.shape[0]
    inner = Wq.shape[0]
    if inner % num_heads != 0:
        _fail(op, "num_heads must divide the projection width")
    if logit_bias is not None and (logit_bias.dtype != torch.float32 or tuple(logit_bias.shape) != (Lq, Lk)):
        _fail(op, "logit_bias must be float32 (Lq, Lk)")
    if d_mask is not None and (d_mask.dtype != torch.float32 or d_mask.numel() != Lk):
        _fail(op, "d_mask must be float32 (Lk,)")
    q = torch.empty(Lq, inner, dtype=X.dtype, device=X.device)
    k = torch.empty(Lk, inner, dtype=X.dtype, device=X.device)
    v = torch.empty(Lk, inner, dtype=X.dtype, device=X.device)
    linear_batched(Wq, None, X, q, op=op)
    linear_batched(Wk, None, Ctx, k, op=op)
    linear_batched(Wv, None, Ctx, v, op=op)
    lse = torch.empty(num_heads, Lq, dtype=torch.float32, device=X.device)
    mask = None if d_mask is None else d_mask.reshape(Lk).contiguous()
    a = sdpa_forward(q, k, v, num_heads, logit_bias=logit_bias, key_mask=mask, lse_out=lse, op=op)
    attn_avg = attention_map_avg(q, k, lse, num_heads, logit_bias=logit_bias, key_mask=mask, out=attn_avg)
    if out is None:
        out = torch.empty(Lq, Wo.shape[0], dtype=X.dtype, device=X.device)
    linear_batched(Wo, None, a, out, op=op)
    return out, attn_avg


def mha_forward(X, Wq, Wk, Wv, Wo, bq, bk, bv, bo, d_mask, num_heads: int, qh: Optional[torch.Tensor] = None,
                kh: Optional[torch.Tensor] = None, vh: Optional[torch.Tensor] = None, attn=None,
                yc: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None):
    """bt::mha_forward as PixArt's self attention calls it on the reference's FP32 path (src/dit/pixart.cpp:325-328):
    qh = X Wq^T + bq, kh, vh likewise, yc = attention(qh, kh, vh) with the optional key mask (float32 (L,), 1 = valid),
    out = yc Wo^T + bo; biases may be None. For float16 / bfloat16 device tensors: four GEMMs and one attention launch,
    intermediates in the caller's tensors when given. The scores are never materialised, so `attn` is ignored.
    Returns (out, qh, kh, vh, yc)."""
    op = "mha_forward"
    _dev(op, X, Wq, Wk, Wv, Wo, bq, bk, bv, bo, d_mask, qh, kh, vh, yc, out)
    if X.dim() != 2:
        _fail(op, "X must be 2-D (rows, channels)")
    L, inner = X.shape[0], Wq.shape[0]
    if num_heads <= 0 or inner % num_heads != 0:
        _fail(op, "num_heads must divide the projection width")
    if Wk.shape[0] != inner or Wv.shape[0] != inner or Wo.shape[1] != inner:
        _fail(op, "Wq, Wk, Wv must project to one width, which Wo takes")
    if d_mask is not None and (d_mask.dtype != torch.float32 or d_mask.numel() != L):
        _fail(op, "d_mask must be float32 (L,)")
    qh = linear_batched(Wq, bq, X, qh, op=op)
    kh = linear_batched(Wk, bk, X, kh, op=op)
    vh = linear_batched(Wv, bv, X, vh, op=op)
    mask = None if d_mask is None else d_mask.reshape(L).contiguous()
    yc = sdpa_forward(qh, kh, vh, num_heads, out=yc, key_mask=mask, op=op)
    out = linear_batched(Wo, bo, yc, out, op=op)
    return out, qh, kh, vh, yc


def gqa_attention_masked(Q, K, V, cos, sin, head_dim: int, num_q_heads: int, num_kv_heads: int, d_mask,
                         out: Optional[torch.Tensor] = None, Kr: Optional[torch.Tensor] = None):
    """Bidirectional grouped-query attention with optional RoPE and key-padding mask
    (include/brodiffusion/dit/common.h:131-153). K/V heads are indexed in place, not widened."""
    op = "gqa_attention_masked"
    if num_kv_heads <= 0 or num_q_heads % num_kv_heads != 0:
        _fail(op, "num_kv_heads must divide num_q_heads")
    if (cos is None) != (sin is None):
        _fail(op, "cos and sin must be given together")
    rope = (cos, sin) if cos is not None else None
    return sdpa_forward(Q, K, V, num_q_heads, num_kv_heads=num_kv_heads, out=out, key_mask=d_mask,
                        rope_q=rope, rope_k=rope, rope_k_scratch=Kr if rope is not None else None, op=op)


def _linear_attn_args(op: str, Q, K, V, num_heads: int, out, eps: float, workspace, accumulate_state: bool):
    """Validated mi_linear_attn_args for token-major operands; `out` and `workspace` must be given."""
    dt = _dtype_code(op, Q)
    if K.dtype != Q.dtype or V.dtype != Q.dtype:
        _fail(op, "Q, K, V must share one dtype")
    if K.shape != Q.shape or V.shape != Q.shape:
        _fail(op, "Q/K/V must share one shape")
    B, N, D, q_rs, q_bs = _as3(op, Q, "Q")
    _, _, _, k_rs, k_bs = _as3(op, K, "K")
    _, _, _, v_rs, v_bs = _as3(op, V, "V")
    if num_heads <= 0 or D % num_heads != 0:
        _fail(op, "D must equal head_dim * num_heads")
    hd = D // num_heads
    if out.shape != Q.shape or out.dtype != Q.dtype:
        _fail(op, "out must have Q's shape and dtype")
    _, _, _, o_rs, o_bs = _as3(op, out, "out")
    need = capi.lib().mi_linear_attn_workspace_bytes(B, num_heads, hd)
    if workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.numel() * 4 < need:
        _fail(op, f"workspace must be contiguous float32 with at least {need // 4} elements")
    a = capi.MiLinearAttnArgs()
    a.struct_size = C.sizeof(capi.MiLinearAttnArgs)
    a.dtype = dt
    a.q, a.k, a.v, a.o = Q.data_ptr(), K.data_ptr(), V.data_ptr(), out.data_ptr()
    a.batch, a.num_heads, a.head_dim, a.n_tokens = B, num_heads, hd, N
    a.q_row_stride, a.q_batch_stride, a.k_row_stride, a.k_batch_stride = q_rs, q_bs, k_rs, k_bs
    a.v_row_stride, a.v_batch_stride, a.o_row_stride, a.o_batch_stride = v_rs, v_bs, o_rs, o_bs
    a.eps = eps
    a.accumulate_state = int(accumulate_state)
    a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel() * 4
    a.stream = _stream()
    return a


def linear_attention_relu_forward(Q, K, V, num_heads: int, out: Optional[torch.Tensor] = None, eps: float = 1e-15,
                                  workspace: Optional[torch.Tensor] = None, accumulate_state: bool = False,
                                  scratch: Optional[torch.Tensor] = None, form: int = 0):
    """Sana's ReLU linear attention core (src/dit/sana.cpp:470-586) on token-major (N, heads*head_dim)
    or (batch, N, heads*head_dim) operands. `workspace` (float32, batch*heads*(d*d+d)) receives the
    (S, z) state; pass it to capture the state or, with accumulate_state, to inject one. `scratch` (float32) holds
    partial states of token chunks; None allocates one, False runs without (one work group per batch item and head).
    `form`: 0 = the library picks, 1 = three launches (state per token chunk, reduction, apply), 2 = one launch with the
    state split along its value channels (mi_linear_attn_args.form)."""
    op = "linear_attention_relu_forward"
    _dev(op, Q, K, V, out, workspace, scratch if scratch is not False else None)
    if out is None:
        out = torch.empty_like(Q)
    if workspace is None:
        if accumulate_state:
            _fail(op, "accumulate_state needs a caller workspace holding a state")
        if num_heads <= 0 or Q.shape[-1] % num_heads != 0:
            _fail(op, "D must equal head_dim * num_heads")
        B = Q.shape[0] if Q.dim() == 3 else 1
        need = capi.lib().mi_linear_attn_workspace_bytes(B, num_heads, Q.shape[-1] // num_heads)
        workspace = torch.empty(need // 4, dtype=torch.float32, device=Q.device)
    a = _linear_attn_args(op, Q, K, V, num_heads, out, eps, workspace, accumulate_state)
    if scratch is False:
        scratch = torch.empty(0, dtype=torch.float32, device=Q.device)      # explicitly none: one work group per (batch, head)
    if scratch is None:
        # partial states of the token chunks (lets the state pass use the whole GPU); comes from torch's caching allocator
        scratch = torch.empty(capi.lib().mi_linear_attn_scratch_bytes(a.batch, num_heads, a.head_dim) // 4, dtype=torch.float32,
                              device=Q.device)
    if scratch.dtype != torch.float32 or not scratch.is_contiguous():
        _fail(op, "scratch must be contiguous float32")
    if scratch.numel() > 0:
        a.scratch, a.scratch_bytes = scratch.data_ptr(), scratch.numel() * 4
    a.form = int(form)
    capi.check(capi.lib().mi_linear_attn_relu_forward(C.byref(a)), op)
    return out


def linear_attention_relu_forward_channel_major(Q, K, V, num_heads: int, out: Optional[torch.Tensor] = None, eps: float = 1e-15,
                                                workspace: Optional[torch.Tensor] = None):
    """The ReLU linear-attention core on the reference's own operands: Q, K, V (and out) as (heads*head_dim, N) or
    (batch, heads*head_dim, N) channel-major tensors, the layout of q_, k_, v_ and attn_c_ around the core in
    src/dit/sana.cpp:424-444, :470-586 (mi_linear_attn_args.layout = MI_LAYOUT_CHANNEL_MAJOR). N must be a multiple of 8;
    rows may be slices of longer rows (a row stride)."""
    op = "linear_attention_relu_forward_channel_major"
    _dev(op, Q, K, V, out, workspace)
    dt = _dtype_code(op, Q)
    if K.dtype != Q.dtype or V.dtype != Q.dtype or K.shape != Q.shape or V.shape != Q.shape:
        _fail(op, "Q, K, V must share one shape and dtype")
    if out is None:
        out = torch.empty_like(Q)
    if out.shape != Q.shape or out.dtype != Q.dtype:
        _fail(op, "out must have Q's shape and dtype")
    B, D, N, q_rs, q_bs = _as3(op, Q, "Q")
    _, _, _, k_rs, k_bs = _as3(op, K, "K")
    _, _, _, v_rs, v_bs = _as3(op, V, "V")
    _, _, _, o_rs, o_bs = _as3(op, out, "out")
    if num_heads <= 0 or D % num_heads != 0:
        _fail(op, "D must equal head_dim * num_heads")
    hd = D // num_heads
    need = capi.lib().mi_linear_attn_workspace_bytes(B, num_heads, hd)
    if workspace is None:
        workspace = torch.empty(need // 4, dtype=torch.float32, device=Q.device)
    if workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.numel() * 4 < need:
        _fail(op, f"workspace must be contiguous float32 with at least {need // 4} elements")
    a = capi.MiLinearAttnArgs()
    a.struct_size = C.sizeof(capi.MiLinearAttnArgs)
    a.dtype = dt
    a.q, a.k, a.v, a.o = Q.data_ptr(), K.data_ptr(), V.data_ptr(), out.data_ptr()
    a.batch, a.num_heads, a.head_dim, a.n_tokens = B, num_heads, hd, N
    a.q_row_stride, a.q_batch_stride, a.k_row_stride, a.k_batch_stride = q_rs, q_bs, k_rs, k_bs
    a.v_row_stride, a.v_batch_stride, a.o_row_stride, a.o_batch_stride = v_rs, v_bs, o_rs, o_bs
    a.eps = eps
    a.layout = capi.MI_LAYOUT_CHANNEL_MAJOR
    a.workspace, a.workspace_bytes = workspace.data_ptr(), workspace.numel() * 4
    a.stream = _stream()
    capi.check(capi.lib().mi_linear_attn_relu_forward(C.byref(a)), op)
    return out


def linear_attention_relu_forward_static_scratch(Q, K, V, num_heads: int, out: torch.Tensor, workspace: torch.Tensor,
                                                 eps: float = 1e-15, accumulate_state: bool = False):
    """linear_attention_relu_forward for callers that must not allocate: `out` and `workspace` are the caller's, the
    partial states live in the library's static device array (mi_linear_attn_relu_forward_static_scratch). Nothing is
    allocated here or below; calls on one GPU must not overlap in time."""
    op = "linear_attention_relu_forward_static_scratch"
    _dev(op, Q, K, V, out, workspace)
    a = _linear_attn_args(op, Q, K, V, num_heads, out, eps, workspace, accumulate_state)
    capi.check(capi.lib().mi_linear_attn_relu_forward_static_scratch(C.byref(a)), op)
    return out


def rms_norm_rows(X, gain, eps: float, out: Optional[torch.Tensor] = None):
    """RMS normalisation of whole rows with a per-column gain: bt::rms_norm_forward(X, gain, eps, out) as Sana-Sprint's
    qk_norm uses it (src/dit/sana.cpp:449-461). X (rows, cols), gain (cols) of X's dtype; in place is allowed."""
    op = "rms_norm_rows"
    _dev(op, X, gain, out)
    dt = _dtype_code(op, X)
    if X.dim() != 2 or X.stride(1) != 1:
        _fail(op, "X must be (rows, cols), contiguous along columns")
    if gain.dtype != X.dtype or gain.numel() != X.shape[1] or not gain.is_contiguous():
        _fail(op, "gain must hold one value of X's dtype per column")
    if out is None:
        out = torch.empty_like(X)
    if out.shape != X.shape or out.dtype != X.dtype or out.stride(1) != 1:
        _fail(op, "out must have X's shape and dtype")
    capi.check(capi.lib().mi_rms_norm_forward(X.data_ptr(), gain.data_ptr(), out.data_ptr(), X.shape[0], X.shape[1], X.stride(0),
                                              out.stride(0), eps, dt, _stream()), op)
    return out


def sana_self_attention(x_mod, Wq, Wk, Wv, Wo, bo, num_heads: int, *, nq=None, nk=None, rms_eps: float = 1e-5,
                        attn_eps: float = 1e-15, ref_mode: str = "off", ref_state: Optional[torch.Tensor] = None,
                        ref_weight: float = 0.0, out: Optional[torch.Tensor] = None):
    """SanaDenoiser::self_attention_ (src/dit/sana.cpp:411-595) as one operator on token-major tensors: the bias-free q, k, v
    projections of x_mod (N, D), the optional qk_norm (nq, nk: per-column gains), the ReLU linear-attention core and the
    output projection (Wo, bo). The reference's channel-major (D, N) layout of the core and the two transposes around it do
    not exist here. ref_mode "capture" writes this call's (S, z) into ref_state (float32, heads x (head_dim + 1) x head_dim:
    S rows then z, the reference's FP32 cache layout, :489-497); "inject" adds ref_weight * ref_state to this call's state
    before the queries read it (:498-505) and leaves ref_state untouched."""
    op = "sana_self_attention"
    _dev(op, x_mod, Wq, Wk, Wv, Wo, bo, nq, nk, ref_state, out)
    if x_mod.dim() != 2:
        _fail(op, "x_mod must be (N, D)")
    N, D = x_mod.shape
    if num_heads <= 0 or D % num_heads != 0:
        _fail(op, "D must equal head_dim * num_heads")
    if (nq is None) != (nk is None):
        _fail(op, "the qk_norm gains come as a pair")
    if ref_mode not in ("off", "capture", "inject"):
        _fail(op, "ref_mode must be 'off', 'capture' or 'inject'")
    hd = D // num_heads
    n_state = num_heads * (hd * hd + hd)
    if ref_mode != "off":
        if ref_state is None or ref_state.dtype != torch.float32 or ref_state.numel() != n_state or not ref_state.is_contiguous():
            _fail(op, f"{ref_mode} needs a contiguous float32 ref_state of {n_state} values")
    q = linear_batched(Wq, None, x_mod)
    k = linear_batched(Wk, None, x_mod)
    v = linear_batched(Wv, None, x_mod)
    if nq is not None:
        rms_norm_rows(q, nq, rms_eps, out=q)
        rms_norm_rows(k, nk, rms_eps, out=k)
    if ref_mode == "capture":
        attn = linear_attention_relu_forward(q, k, v, num_heads, eps=attn_eps, workspace=ref_state.view(-1))
    elif ref_mode == "inject" and ref_weight != 0.0:
        attn = torch.empty_like(q)
        ws = ref_state.view(-1).clone()                   # the anchor stays as it is; the copy takes this call's state on top
        a = _linear_attn_args(op, q, k, v, num_heads, attn, attn_eps, ws, True)
        a.accumulate_weight = float(ref_weight)
        sc = torch.empty(capi.lib().mi_linear_attn_scratch_bytes(1, num_heads, hd) // 4, dtype=torch.float32, device=q.device)
        a.scratch, a.scratch_bytes = sc.data_ptr(), sc.numel() * 4
        capi.check(capi.lib().mi_linear_attn_relu_forward(C.byref(a)), op)
    else:
        attn = linear_attention_relu_forward(q, k, v, num_heads, eps=attn_eps)
    return linear_batched(Wo, bo, attn, out)


def build_axial_rope_tables(txt_len: int, hp: int, wp: int, head_dim: int, axes_dims_rope: Sequence[int],
                            theta: float = 10000.0, device="cuda"):
    """cos / sin tables (txt_len + hp*wp, head_dim/2) FP32 for the joint [text ; image] sequence
    (src/dit/common.cpp:116-184): text rows are the identity rotation, image token (i, j) has axial
    position (0, i, j), pair p of axis a turns by pos * theta^(-2p / axes[a])."""
    op = "build_axial_rope_tables"
    if head_dim % 2 != 0:
        _fail(op, "head_dim must be even")
    if sum(axes_dims_rope) != head_dim:
        _fail(op, "axes_dims_rope must sum to head_dim")
    half = head_dim // 2
    ang = np.zeros((txt_len + hp * wp, half), dtype=np.float64)
    ii, jj = np.meshgrid(np.arange(hp), np.arange(wp), indexing="ij")
    pos = [np.zeros(hp * wp), ii.reshape(-1).astype(np.float64), jj.reshape(-1).astype(np.float64)]
    off = 0
    for a, dim in enumerate(axes_dims_rope):
        cnt = dim // 2
        if a < 3 and cnt > 0:
            omega = 1.0 / np.power(float(theta), 2.0 * np.arange(cnt) / float(dim))
            ang[txt_len:, off:off + cnt] = pos[a][:, None] * omega[None, :]
        off += cnt
    cos = torch.from_numpy(np.cos(ang).astype(np.float32)).to(device)
    sin = torch.from_numpy(np.sin(ang).astype(np.float32)).to(device)
    return cos, sin


def qwen_rope_positions(prefix_segments, hp: int, wp: int) -> np.ndarray:
    """(3, L) integer positions (frame, height, width) of the Qwen-Image joint sequence [prefix segments ; target
    image hp x wp] (src/dit/qwenimage21_forward.cpp:130-161). `prefix_segments` holds ("text", n) and
    ("image", h, w) entries. A shared running position walks the sequence: a text token sits at (p, p, p) and
    advances it by one; an image block freezes the frame axis at the current position, lays its tokens on a grid
    centred on zero (first row at -(h - h//2)), then advances the position by max(h, w)."""
    cols = []
    pos = 0
    for seg in list(prefix_segments) + [("image", hp, wp)]:
        if seg[0] == "text":
            n = int(seg[1])
            run = np.arange(pos, pos + n, dtype=np.int64)
            cols.append(np.stack([run, run, run]))
            pos += n
        elif seg[0] == "image":
            h, w = int(seg[1]), int(seg[2])
            ii, jj = np.meshgrid(np.arange(h) - (h - h // 2), np.arange(w) - (w - w // 2), indexing="ij")
            cols.append(np.stack([np.full(h * w, pos, dtype=np.int64), ii.reshape(-1), jj.reshape(-1)]))
            pos += max(h, w)
        else:
            _fail("qwen_rope_positions", f"unknown segment kind {seg[0]!r}")
    return np.concatenate(cols, axis=1) if cols else np.zeros((3, 0), dtype=np.int64)


def rope_tables_from_positions(positions: np.ndarray, head_dim: int, axes_dims_rope: Sequence[int], theta: float = 10000.0):
    """FP32 (L, head_dim/2) cos / sin from per-axis integer positions (n_axes, L): pair p of axis a turns by
    position * theta^(-2p / axes[a]); the axes' pairs are concatenated in order. Angles are formed in double."""
    if head_dim % 2 != 0 or sum(axes_dims_rope) != head_dim or len(axes_dims_rope) != positions.shape[0]:
        _fail("rope_tables_from_positions", "axes_dims_rope must sum to head_dim, one entry per position axis")
    blocks = []
    for a, dim in enumerate(axes_dims_rope):
        omega = np.power(float(theta), -2.0 * np.arange(dim // 2, dtype=np.float64) / float(dim))
        blocks.append(positions[a].astype(np.float64)[:, None] * omega[None, :])
    ang = np.concatenate(blocks, axis=1)
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def build_qwen_rope_tables(prefix_segments, hp: int, wp: int, head_dim: int, axes_dims_rope: Sequence[int] = (16, 56, 56),
                           theta: float = 10000.0, device="cuda"):
    """3-axis RoPE tables of the Qwen-Image joint sequence (QwenImage21Transformer2DModel::build_rope_tables_,
    src/dit/qwenimage21_forward.cpp:124-200). A cached step slices the rows of its target tokens."""
    cos, sin = rope_tables_from_positions(qwen_rope_positions(prefix_segments, hp, wp), head_dim, axes_dims_rope, theta)
    return torch.from_numpy(cos).to(device), torch.from_numpy(sin).to(device)
