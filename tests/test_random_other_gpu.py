"""Seeded random sweeps of the bandwidth-bound operators and the projection GEMM against the CPU checker: linear
attention (random batch, tokens, heads, head_dim, strided views, with / without scratch, state injection), RoPE in
all four forms, head RMSNorm + RoPE, and the linear layer with row strides through the C ABI."""
import ctypes as C

import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from brodiffusion_amd import _capi as capi
from helpers import TOL, TORCH_DT, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_linear_attention(oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    d = int(rng.choice([32, 64, 72, 112, 128]))
    H = int(rng.integers(1, 7))
    B = int(rng.choice([1, 2, 3]))
    N = int(rng.integers(1, 1500))
    dtype = "bf16"
    wide = rng.random() < 0.5                      # operands as column slices of one (B, N, 3*D) projection
    D = H * d
    qkv = randn(70000 + seed, (B, N, 3 * D), dtype)
    dqkv = to_dev(qkv, dtype)
    if wide:
        dq, dk, dv = dqkv[..., :D], dqkv[..., D:2 * D], dqkv[..., 2 * D:]
    else:
        dq, dk, dv = (dqkv[..., i * D:(i + 1) * D].contiguous() for i in range(3))
    q, k, v = qkv[..., :D], qkv[..., D:2 * D], qkv[..., 2 * D:]
    scratch = None if rng.random() < 0.6 else False
    ws = torch.empty(B * H * (d * d + d), dtype=torch.float32, device="cuda")
    out = bd.linear_attention_relu_forward(dq, dk, dv, H, workspace=ws, scratch=scratch)
    for b in range(B):
        ref, S, z = oracle.linear_attn_relu(q[b], k[b], v[b], H, return_state=True)
        assert_close(ref, to_np(out[b]), dtype, f"seed {seed} d={d} H={H} N={N} wide={wide} scratch={scratch} batch {b}")
        got = ws.view(B, H, d * d + d)[b].cpu().numpy()
        assert np.allclose(got[:, :d * d].reshape(H, d, d), S, rtol=2e-4, atol=2e-3 * max(1.0, np.abs(S).max()) * 1e-2)
        assert np.allclose(got[:, d * d:], z, rtol=2e-4, atol=1e-3)
    if N >= 2:
        # state injection: first part captured, second part accumulated on top and applied to the second part's queries
        cut = int(rng.integers(1, N))
        ws2 = torch.empty_like(ws)
        bd.linear_attention_relu_forward(dq[:, :cut], dk[:, :cut], dv[:, :cut], H, workspace=ws2, scratch=scratch)
        out2 = bd.linear_attention_relu_forward(dq[:, cut:], dk[:, cut:], dv[:, cut:], H, workspace=ws2, accumulate_state=True, scratch=scratch)
        assert (ws2 - ws).abs().max().item() <= 1e-4 * max(1.0, ws.abs().max().item())
        unit = 2.0 ** -8
        assert (out2.float() - out[:, cut:].float()).abs().max().item() <= 2 * unit * max(1.0, out.float().abs().max().item())


@pytest.mark.parametrize("seed", list(range(10)))
def test_random_rope_and_headnorm(oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    dtype = "bf16" if rng.random() < 0.5 else "fp16"
    d = int(rng.choice([32, 64, 128] if seed % 2 else [40, 72, 96, 160]))
    H = int(rng.integers(1, 9))
    L = int(rng.integers(1, 700))
    x = randn(80000 + seed, (L, H * d), dtype)
    per_head = bool(rng.random() < 0.4)
    split_half = bool(rng.random() < 0.4)
    rows = L * H if per_head else L
    ang = rng.uniform(0, 6.28, (rows, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    dx, dcos, dsin = to_dev(x, dtype), torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    if per_head:
        got = bd.rope_apply_perhead(dx, dcos, dsin, d, H, split_half=split_half)
        ref = oracle.rope_apply(x.reshape(L * H, d), cos, sin, 1, d, split_half=split_half, round_to_dtype=dtype).reshape(L, H * d)
    else:
        got = bd.rope_apply(dx, dcos, dsin, d, H, split_half=split_half)
        ref = oracle.rope_apply(x, cos, sin, H, d, split_half=split_half, round_to_dtype=dtype)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.abs(to_np(got) - ref).max() <= unit * max(1.0, np.abs(ref).max()), f"seed {seed} d={d} per_head={per_head} split={split_half}"
    if d in (32, 64, 128) and not per_head and not split_half:
        gain = oracle.round_to(1 + 0.3 * randn(81000 + seed, (d,), "fp32"), dtype)
        eps = float(rng.choice([1e-6, 1e-5]))
        hn = bd.headnorm_rope(dx, to_dev(gain, dtype), eps, dcos, dsin, d, H)
        ref = oracle.headnorm_rope(x, gain, eps, cos, sin, H, d)
        assert np.all(np.abs(to_np(hn) - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)


@pytest.mark.parametrize("seed", list(range(10)))
def test_random_linear_with_strides(oracle, seed):
    """The C ABI's row strides (the Python op takes dense operands): X, W and Y as column / row slices of larger buffers."""
    rng = np.random.default_rng(4000 + seed)
    dtype = "bf16" if rng.random() < 0.5 else "fp16"
    M, N, K = int(rng.integers(1, 600)), 8 * int(rng.integers(1, 60)), 8 * int(rng.integers(1, 150))
    px, pw, py = (8 * int(rng.integers(0, 4)) for _ in range(3))
    xb = randn(90000 + seed, (M, K + px), dtype)
    wb = oracle.round_to(randn(91000 + seed, (N, K + pw), "fp32") / np.sqrt(K), dtype)
    b = randn(92000 + seed, (N,), dtype) if rng.random() < 0.7 else None
    dxb, dwb = to_dev(xb, dtype), to_dev(wb, dtype)
    dy = torch.full((M, N + py), 3.0, device="cuda", dtype=TORCH_DT[dtype])
    db = None if b is None else to_dev(b, dtype)
    a = capi.MiLinearArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = capi.MI_DTYPE_BF16 if dtype == "bf16" else capi.MI_DTYPE_F16
    a.x, a.w, a.y = dxb.data_ptr(), dwb.data_ptr(), dy.data_ptr()
    a.bias = 0 if db is None else db.data_ptr()
    a.rows, a.in_features, a.out_features = M, K, N
    a.x_row_stride, a.w_row_stride, a.y_row_stride = K + px, K + pw, N + py
    a.stream = torch.cuda.current_stream().cuda_stream
    capi.check(capi.lib().mi_linear_forward(C.byref(a)), "mi_linear_forward")
    ref = oracle.linear(xb[:, :K], wb[:, :K], b)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    got = to_np(dy)
    assert np.all(np.abs(got[:, :N] - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6), f"seed {seed} {M}x{N}x{K}"
    assert (got[:, N:] == 3.0).all()
