"""The projection GEMM on problems large enough for its 256 x 256-tile kernel (about one tile per compute unit and more;
in_features a multiple of 64), through the C ABI, against the CPU checker on sampled rows of the same seeded inputs:
the benchmark shape, ragged token and feature counts (rows and columns of the last tiles are clamped on load and masked
on store), operands that are slices of larger buffers, and two problems in one launch (the K / V projections of a
cross-attention cache fill). The bound is the one of the small shapes (tests/test_attn_block_gpu.py): FP32 accumulation
and one rounding, i.e. one unit in the last place of the result's magnitude; the checker follows the definition
y = x w^T + b of bt::linear_batched (src/unet_blocks.cpp:238-240)."""
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


def _rows(M, n=192):
    """Sampled rows: the first and last rows of the problem and of tile boundaries, and a spread in between."""
    edge = [r for r in (0, 1, 255, 256, 257, 511, 512, M - 257, M - 256, M - 2, M - 1) if 0 <= r < M]
    return np.unique(np.concatenate([np.array(edge), np.linspace(0, M - 1, n).astype(np.int64)]))


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K,bias", [
    (4608, 3072, 3072, True),     # the benchmark's large linear layer
    (3600, 3336, 576, True),      # ragged last tiles along both axes (3336 = 13 * 256 + 8)
    (8192, 1536, 512, False),     # the shortest contraction the kernel takes
    (3329, 4104, 640, True)])     # one row and one 8-column piece in the last tiles
def test_large_linear_matches_checker(oracle, dtype, M, N, K, bias):
    x = randn(21 + M, (M, K), dtype)
    w = _weight(oracle, 22 + N, N, K, dtype)
    b = randn(23 + K, (N,), dtype) if bias else None
    y = to_np(bd.linear_batched(to_dev(w, dtype), None if b is None else to_dev(b, dtype), to_dev(x, dtype)))
    assert y.shape == (M, N)
    rows = _rows(M)
    _one_ulp(oracle.linear(x[rows], w, b), y[rows], dtype, f"linear {M}x{N}x{K}")


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_large_linear_with_strides(oracle, dtype):
    """X, W and Y as column slices of wider buffers (row strides through the C ABI); what lies beside Y stays untouched."""
    M, N, K, px, pw, py = 3600, 3336, 1024, 24, 8, 16
    xb = randn(31, (M, K + px), dtype)
    wb = _weight(oracle, 32, N, K + pw, dtype)
    b = randn(33, (N,), dtype)
    dxb, dwb, db = to_dev(xb, dtype), to_dev(wb, dtype), to_dev(b, dtype)
    dy = torch.full((M, N + py), 3.0, device="cuda", dtype=TORCH_DT[dtype])
    a = capi.MiLinearArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = capi.MI_DTYPE_BF16 if dtype == "bf16" else capi.MI_DTYPE_F16
    a.x, a.w, a.y, a.bias = dxb.data_ptr(), dwb.data_ptr(), dy.data_ptr(), db.data_ptr()
    a.rows, a.in_features, a.out_features = M, K, N
    a.x_row_stride, a.w_row_stride, a.y_row_stride = K + px, K + pw, N + py
    a.stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib().mi_linear_forward(C.byref(a)), "mi_linear_forward")
    got = to_np(dy)
    rows = _rows(M)
    _one_ulp(oracle.linear(xb[rows, :K], wb[:, :K], b), got[rows, :N], dtype, "strided")
    assert (got[:, N:] == 3.0).all()


def test_two_projections_in_one_launch(oracle):
    """flash_attention_project_kv (src/unet.cpp:470-474) at a size where the launch of its two problems takes the large
    kernel: each output against the checker's linear layer."""
    dtype, B, L, Cc, inner = "bf16", 2, 4096, 1536, 1536
    ctx = randn(41, (B, L, Cc), dtype)
    wk, wv = _weight(oracle, 42, inner, Cc, dtype), _weight(oracle, 43, inner, Cc, dtype)
    bk, bv = randn(44, (inner,), dtype), randn(45, (inner,), dtype)
    K_out, V_out = bd.flash_attention_project_kv(to_dev(ctx, dtype), to_dev(wk, dtype), to_dev(bk, dtype), to_dev(wv, dtype),
                                                 to_dev(bv, dtype))
    rows = _rows(B * L)
    flat = ctx.reshape(B * L, Cc)
    _one_ulp(oracle.linear(flat[rows], wk, bk), to_np(K_out).reshape(B * L, inner)[rows], dtype, "K projection")
    _one_ulp(oracle.linear(flat[rows], wv, bv), to_np(V_out).reshape(B * L, inner)[rows], dtype, "V projection")


def test_large_linear_agrees_with_small_tile_kernel():
    """A problem just below the size at which the large kernel takes over and the same rows inside a problem above it:
    both kernels accumulate the contraction in FP32 in blocks of 16 in the same order, so the shared rows agree bit for
    bit."""
    dt = torch.bfloat16
    g = torch.Generator(device="cpu").manual_seed(7)
    x = torch.randn(4608, 1024, generator=g).to(dt).cuda()
    w = (torch.randn(3072, 1024, generator=g) / 32).to(dt).cuda()
    b = torch.randn(3072, generator=g).to(dt).cuda()
    big = bd.linear_batched(w, b, x)                 # 18 x 12 tiles of 256 x 256: the large kernel
    small = bd.linear_batched(w, b, x[:2048])        # 8 x 12 tiles: the 128 x 128 kernel
    assert torch.equal(big[:2048], small)


def test_unequal_problems_in_one_launch(oracle):
    """The Q / K / V launch of a cross-attention block whose query rows far outnumber its context rows (12288 against
    512): three problems of 192, 8 and 8 tiles in one launch of the large kernel, whose grid is sized for the largest.
    Work groups beyond a small problem's own run of tiles must leave (they would repeat tiles of the neighbouring runs).
    The block equals its parts bit for bit (the K / V projections alone run on the small-tile kernel, which accumulates
    in the same order), and sampled rows of Q, K, V match the checker."""
    dtype, L, Lc, C, H = "bf16", 12288, 512, 1024, 8
    x, ctx = randn(51, (L, C), dtype), randn(52, (Lc, C), dtype)
    wq, wk, wv, wo = (_weight(oracle, 53 + i, C, C, dtype) for i in range(4))
    bq, bk, bv, bo = (oracle.round_to(randn(57 + i, (C,), dtype) * 0.25, dtype) for i in range(4))
    dx, dctx = to_dev(x, dtype), to_dev(ctx, dtype)
    dw = [to_dev(w, dtype) for w in (wq, wk, wv, wo)]
    db = [to_dev(b, dtype) for b in (bq, bk, bv, bo)]
    out = bd.flash_attention_qkvo_forward(dx, dctx, dw[0], db[0], dw[1], db[1], dw[2], db[2], dw[3], db[3], None, H, False)
    q = bd.linear_batched(dw[0], db[0], dx)
    k = bd.linear_batched(dw[1], db[1], dctx)
    v = bd.linear_batched(dw[2], db[2], dctx)
    parts = bd.linear_batched(dw[3], db[3], bd.flash_attention_forward(q, k, v, None, H, False))
    assert torch.equal(parts, out)
    rows = _rows(L, 64)
    _one_ulp(oracle.linear(x[rows], wq, bq), to_np(q)[rows], dtype, "Q projection")
    _one_ulp(oracle.linear(ctx, wk, bk), to_np(k), dtype, "K projection")
    _one_ulp(oracle.linear(ctx, wv, bv), to_np(v), dtype, "V projection")
    ref = oracle.attention_qkvo(x[rows], ctx, wq, bq, wk, bk, wv, bv, wo, bo, H, dtype)
    assert_close(ref, to_np(out)[rows], dtype, "cross-attention block with unequal projections")
