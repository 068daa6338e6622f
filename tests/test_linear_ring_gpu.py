"""The projection GEMM in its tile-walking form (in_features a multiple of 320 and at least 640, problems too small for the
128 x 128 and 256 x 256 tile kernels: the FF2 and attention projections of the U-Net's deeper levels), against the CPU
checker on the same seeded inputs: the real shapes, ragged token and feature counts, no bias, operands that are slices of
wider buffers, three problems of different sizes in one launch. Bound: FP32 accumulation and one rounding (one unit in the
last place of the result's magnitude, as in tests/test_attn_block_gpu.py); the checker follows y = x w^T + b of
bt::linear_batched (src/unet_blocks.cpp:238-240)."""
import ctypes as C

import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from brodiffusion_amd import _capi as capi
from helpers import TORCH_DT, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def _weight(oracle, seed, n_out, n_in, dtype):
    return oracle.round_to(randn(seed, (n_out, n_in), "fp32") / np.sqrt(n_in), dtype)


def _one_ulp(ref, got, dtype, what):
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.isfinite(got).all(), what
    assert np.all(np.abs(got - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6), what


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("M,N,K,bias", [
    (2048, 640, 2560, True),      # FF2 of the 32 x 32 level
    (8192, 320, 1280, True),      # FF2 of the 64 x 64 level
    (512, 1280, 1280, True),      # an attention projection of the 16 x 16 level
    (77, 1280, 640, False),       # fewer tokens than one tile, no bias
    (1000, 328, 960, True),       # 40 of 64 tokens and 8 of 64 features in the last tiles; three groups of five steps
    (3, 8, 640, False)])          # a corner of one tile
def test_ring_linear_matches_checker(oracle, dtype, M, N, K, bias):
    x = randn(51 + M, (M, K), dtype)
    w = _weight(oracle, 52 + N, N, K, dtype)
    b = randn(53 + K, (N,), dtype) if bias else None
    y = to_np(bd.linear_batched(to_dev(w, dtype), None if b is None else to_dev(b, dtype), to_dev(x, dtype)))
    assert y.shape == (M, N)
    _one_ulp(oracle.linear(x, w, b), y, dtype, f"linear {M}x{N}x{K}")


def test_ring_linear_with_strides(oracle):
    """X, W and Y as column slices of wider buffers (row strides through the C ABI); what lies beside Y stays untouched."""
    dtype, M, N, K, px, pw, py = "bf16", 900, 200, 640, 24, 8, 16
    xb = randn(61, (M, K + px), dtype)
    wb = _weight(oracle, 62, N, K + pw, dtype)
    b = randn(63, (N,), dtype)
    dxb, dwb, db = to_dev(xb, dtype), to_dev(wb, dtype), to_dev(b, dtype)
    dy = torch.full((M, N + py), 3.0, device="cuda", dtype=TORCH_DT[dtype])
    a = capi.MiLinearArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = capi.MI_DTYPE_BF16
    a.x, a.w, a.y, a.bias = dxb.data_ptr(), dwb.data_ptr(), dy.data_ptr(), db.data_ptr()
    a.rows, a.in_features, a.out_features = M, K, N
    a.x_row_stride, a.w_row_stride, a.y_row_stride = K + px, K + pw, N + py
    a.stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib().mi_linear_forward(C.byref(a)), "mi_linear_forward")
    got = to_np(dy)
    _one_ulp(oracle.linear(xb[:, :K], wb[:, :K], b), got[:, :N], dtype, "strided")
    assert (got[:, N:] == 3.0).all()


def test_three_projections_in_one_launch(oracle):
    """The Q, K and V projections of a self-attention block at C = 640 share a launch (three problems, one grid row
    each): flash_attention_qkvo_forward against the checker's block (src/unet_blocks.cpp:255-273)."""
    dtype, B, N, Cc, H = "fp16", 2, 300, 640, 8
    x = randn(71, (B, N, Cc), dtype)
    ws = [_weight(oracle, 72 + i, Cc, Cc, dtype) for i in range(4)]
    bo = oracle.round_to(randn(77, (Cc,), dtype), dtype)
    out = bd.flash_attention_qkvo_forward(to_dev(x, dtype), None, to_dev(ws[0], dtype), None, to_dev(ws[1], dtype), None,
                                          to_dev(ws[2], dtype), None, to_dev(ws[3], dtype), to_dev(bo, dtype), None, H, False)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], None, ws[0], None, ws[1], None, ws[2], None, ws[3], bo, H, dtype)
        assert_close(ref, to_np(out[b]), dtype, f"qkvo self batch {b}")
