"""Tensors of more than 2^31 elements (4 GiB and up in 16-bit): row offsets no longer fit 32 bits. Sampled query rows
against the CPU checker for softmax attention; for linear attention, one call on the whole sequence against the same
sequence fed in four chunks through the state injection (every chunk's offsets are small)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, to_np

pytestmark = pytest.mark.gpu


def _big_randn(rows, cols, seed, scale=1.0):
    """(rows, cols) bf16 on the GPU, filled in slabs so that the float32 temporary stays small."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    out = torch.empty(rows, cols, dtype=torch.bfloat16, device="cuda")
    step = 1 << 16
    for r0 in range(0, rows, step):
        r1 = min(rows, r0 + step)
        out[r0:r1] = (torch.randn(r1 - r0, cols, device="cuda", generator=g) * scale).to(torch.bfloat16)
    return out


def test_cross_attention_beyond_2_31_elements(oracle):
    H, d, Lq, Lk = 16, 128, 1_200_000, 64            # Q and O: 2.46e9 elements each; row 2^20 starts at element 2^31
    q = _big_randn(Lq, H * d, 11)
    k = _big_randn(Lk, H * d, 12)
    v = _big_randn(Lk, H * d, 13)
    out = torch.full((Lq, H * d), float("nan"), dtype=torch.bfloat16, device="cuda")
    bd.flash_attention_forward(q, k, v, None, H, False, out=out)
    rows = [0, 1, 255, 256, 777_777, (1 << 20) - 1, 1 << 20, (1 << 20) + 1, 1_150_000, Lq - 257, Lq - 1]
    idx = torch.tensor(rows, device="cuda")
    ref = oracle.sdpa(to_np(q[idx]), to_np(k), to_np(v), H)
    assert_close(ref, to_np(out[idx]), "bf16", "sampled rows of a 4.9 GB query tensor")
    # nothing was left unwritten: every row sums to something finite
    assert torch.isfinite(out.float().sum(dim=1)).all()


def test_linear_attention_beyond_2_31_elements():
    H, d, N = 20, 112, 1_000_000                      # 2.24e9 elements per tensor; row 958 699 starts beyond element 2^31
    q = _big_randn(N, H * d, 21).unsqueeze(0)
    k = _big_randn(N, H * d, 22, scale=0.05).unsqueeze(0)
    v = _big_randn(N, H * d, 23).unsqueeze(0)
    ws = torch.empty(H * (d * d + d), dtype=torch.float32, device="cuda")
    whole = bd.linear_attention_relu_forward(q, k, v, H, workspace=ws)
    # the same state, built from four chunks with small offsets, applied to samples of the queries
    ws2 = torch.empty_like(ws)
    cut = N // 4
    for c in range(4):
        sl = slice(c * cut, (c + 1) * cut)
        bd.linear_attention_relu_forward(q[:, sl], k[:, sl], v[:, sl], H, workspace=ws2, accumulate_state=c > 0)
    assert (ws2 - ws).abs().max().item() <= 2e-4 * ws.abs().max().item()
    # state injection applies the accumulated state to the chunk's queries: an empty-handed chunk (k = 0 adds nothing)
    for r0 in (0, 958_600, N - 4096):
        sl = slice(r0, r0 + 4096)
        ws3 = ws.clone()
        part = bd.linear_attention_relu_forward(q[:, sl], torch.zeros_like(k[:, sl]), v[:, sl], H, workspace=ws3, accumulate_state=True)
        a, b = part.float(), whole[:, sl].float()
        assert (a - b).abs().max().item() <= 2.0 ** -7 * max(1.0, b.abs().max().item()), f"rows from {r0}"


def test_keys_beyond_2_31_elements(oracle):
    """K and V of 2.46e9 elements each under the 256-row kernel (tiles by LDS DMA). The key sequence is a 60 000-row
    block repeated 20 times, so the exact result is the attention over one block (every key and value 20 times:
    the weights renormalise) and the checker only has to walk 60 000 keys; a key tile fetched from a wrapped or
    truncated address would visit the blocks unevenly and change the result."""
    H, d, Lq, P, R = 16, 128, 4096, 60_000, 20
    q = _big_randn(Lq, H * d, 31)
    k0 = _big_randn(P, H * d, 32)
    v0 = _big_randn(P, H * d, 33)
    k, v = k0.repeat(R, 1), v0.repeat(R, 1)
    assert k.numel() > 2 ** 31
    out = bd.flash_attention_forward(q, k, v, None, H, False)
    small = bd.flash_attention_forward(q, k0, v0, None, H, False)
    assert (out.float() - small.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, small.float().abs().max().item())
    rows = [0, 1000, Lq - 1]
    ref = oracle.sdpa(to_np(q[rows]), to_np(k0), to_np(v0), H)
    assert_close(ref, to_np(out[rows]), "bf16", "sampled rows against one period of the keys")


def test_elementwise_and_rope_beyond_2_31_elements(oracle):
    """RoPE, head norm + RoPE, row scaling, the two adds and the linear layer on (1 100 000, 2048) = 2.25e9 elements;
    rows on both sides of element 2^31 against the checker (or plain arithmetic)."""
    H, d, L = 16, 128, 1_100_000
    x = _big_randn(L, H * d, 41)
    rows = [0, 5, (1 << 20) - 1, 1 << 20, (1 << 20) + 7, L - 1]
    idx = torch.tensor(rows, device="cuda")
    ang = torch.rand(L, d // 2, device="cuda", generator=torch.Generator(device="cuda").manual_seed(42)) * 6.28
    cos, sin = torch.cos(ang), torch.sin(ang)
    xs = to_np(x[idx])
    unit = 2.0 ** -8

    r = bd.rope_apply(x, cos, sin, d, H)
    ref = oracle.rope_apply(xs, cos[idx].cpu().numpy(), sin[idx].cpu().numpy(), H, d, round_to_dtype="bf16")
    assert np.abs(to_np(r[idx]) - ref).max() <= unit * max(1.0, np.abs(ref).max())
    del r

    gain = oracle.round_to(1 + 0.3 * np.arange(d, dtype=np.float32) / d, "bf16")
    hn = bd.headnorm_rope(x, torch.from_numpy(gain).cuda().to(torch.bfloat16), 1e-6, cos, sin, d, H)
    ref = oracle.headnorm_rope(xs, gain, 1e-6, cos[idx].cpu().numpy(), sin[idx].cpu().numpy(), H, d)
    assert np.all(np.abs(to_np(hn[idx]) - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)
    del hn

    rs = torch.rand(L, 1, device="cuda", generator=torch.Generator(device="cuda").manual_seed(43))
    sr = bd.scale_rows(x, 0.75, rs)
    ref = oracle.round_to(xs * (0.75 * rs[idx].cpu().numpy()), "bf16")
    assert np.abs(to_np(sr[idx]) - ref).max() <= unit * max(1.0, np.abs(ref).max())

    y = sr                                            # reuse the buffer: y += x, then y += bias per row
    before = to_np(y[idx])
    bd.add_inplace_vec(y, x)
    ref = oracle.round_to(before + xs, "bf16")
    assert np.array_equal(to_np(y[idx]), ref)
    bias = _big_randn(1, H * d, 44).reshape(H * d)
    before = to_np(y[idx])
    bd.add_inplace_row_bias(y, bias)
    assert np.array_equal(to_np(y[idx]), oracle.round_to(before + to_np(bias)[None, :], "bf16"))
    del y, sr

    w = (_big_randn(256, H * d, 45) / np.sqrt(H * d)).to(torch.bfloat16)
    out = bd.linear_batched(w, None, x)               # (1 100 000, 256): the input offsets are the large ones
    ref = oracle.linear(xs, to_np(w))
    got = to_np(out[idx])
    assert np.all(np.abs(got - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)
