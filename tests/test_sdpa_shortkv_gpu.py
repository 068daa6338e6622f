"""Cross attention to a short key sequence on large query sets: the launch where all K and V of a (batch, head) stay
in LDS and one work group walks several query tiles (picked automatically when the keys fit and there is at least one
256-row query tile per compute unit). It runs the same tile arithmetic as the 128-row kernel, so the two must agree
bit for bit; sampled rows are also checked against the CPU checker (helpers.TOL)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def rows128(*args, **kw):
    bd.set_sdpa_kernel_choice(1)
    try:
        return bd.sdpa_forward(*args, **kw)
    finally:
        bd.set_sdpa_kernel_choice(0)


@pytest.mark.parametrize("dtype,B,H,d,Lq,Lk,valid", [
    ("bf16", 2, 16, 72, 4096, 300, [77, 300]),      # PixArt cross attention, two query tiles per work group
    ("bf16", 2, 16, 72, 6500, 300, None),           # three tiles per work group, ragged last strip and last tile
    ("fp16", 2, 8, 40, 4096, 77, None),             # SD1.5 cross attention: one tile per work group
    ("bf16", 1, 24, 128, 3000, 100, [61]),          # head_dim 128: two key tiles is all that fits
    ("fp16", 1, 32, 64, 2048, 320, None),           # the longest key sequence that qualifies
    ("bf16", 1, 32, 64, 2048, 64, [1]),             # one key tile; a single visible key: output = its value row
])
def test_shortkv_matches_rows128_and_checker(oracle, dtype, B, H, d, Lq, Lk, valid):
    q = randn(9700 + Lq, (B, Lq, H * d), dtype)
    k, v = randn(9701 + Lk, (B, Lk, H * d), dtype), randn(9702 + Lk, (B, Lk, H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    vl = None if valid is None else torch.tensor(valid, dtype=torch.int32, device="cuda")
    out = bd.sdpa_forward(dq, dk, dv, H, kv_valid_len=vl)
    assert torch.equal(out, rows128(dq, dk, dv, H, kv_valid_len=vl))
    rows = np.unique(np.concatenate([np.arange(0, Lq, 211), np.arange(255, Lq, 256), np.arange(256, Lq, 256), [Lq - 1]])).astype(np.int32)
    for b in range(B):
        n = Lk if valid is None else valid[b]
        ref = oracle.sdpa(q[b], k[b, :n], v[b, :n], H, rows=rows)
        assert_close(ref[rows], to_np(out[b])[rows], dtype, f"short-kv batch {b}")
    if valid == [1]:
        assert torch.equal(out[0], dv[0, :1].expand(Lq, -1))


def test_shortkv_strided_views_and_zero_valid(oracle):
    """Q and O as column slices of wider buffers, K/V as row slices; a batch item with no valid key gives zeros."""
    dtype, B, H, d, Lq, Lk = "bf16", 2, 16, 72, 4096, 128
    D = H * d
    wide_q = to_dev(randn(9800, (B, Lq, 2 * D), dtype), dtype)
    dq = wide_q[:, :, D:]
    kv = to_dev(randn(9801, (B, Lk + 8, 2 * D), dtype), dtype)
    dk, dv = kv[:, 3:3 + Lk, :D], kv[:, 3:3 + Lk, D:]
    vl = torch.tensor([0, 90], dtype=torch.int32, device="cuda")
    wide_o = torch.full((B, Lq, 2 * D), 5.0, device="cuda", dtype=torch.bfloat16)
    out = bd.sdpa_forward(dq, dk, dv, H, kv_valid_len=vl, out=wide_o[:, :, :D])
    assert (out[0] == 0).all() and (wide_o[:, :, D:] == 5).all()
    assert torch.equal(out, rows128(dq.contiguous(), dk.contiguous(), dv.contiguous(), H, kv_valid_len=vl))


@pytest.mark.parametrize("dtype,B,H,d,Lq,Lk", [("bf16", 2, 16, 72, 4096, 200), ("fp16", 2, 8, 40, 4096, 77)])
def test_shortkv_key_mask(oracle, dtype, B, H, d, Lq, Lk):
    """A 0/1 key mask per batch item (text padding in the middle and at the end, one whole key tile hidden) on the shape
    that takes the short-key kernel, alone and together with a valid length: bit-equal to the 128-row kernel, sampled rows
    against the checker."""
    q = randn(9900 + Lq, (B, Lq, H * d), dtype)
    k, v = randn(9901 + Lk, (B, Lk, H * d), dtype), randn(9902 + Lk, (B, Lk, H * d), dtype)
    m = (np.random.default_rng(Lk).uniform(size=(B, Lk)) > 0.3).astype(np.float32)
    m[0, Lk - 9:] = 0
    if Lk > 128:
        m[1, 64:128] = 0
    dq, dk, dv, dm = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), torch.from_numpy(m).cuda()
    rows = np.unique(np.concatenate([np.arange(0, Lq, 173), [31, 32, Lq - 1]])).astype(np.int32)
    out = bd.sdpa_forward(dq, dk, dv, H, key_mask=dm)
    assert torch.equal(out, rows128(dq, dk, dv, H, key_mask=dm))
    for b in range(B):
        ref = oracle.sdpa(q[b], k[b], v[b], H, key_mask=m[b], rows=rows)
        assert_close(ref[rows], to_np(out[b])[rows], dtype, f"short-kv key mask, batch {b}")
    vl = torch.tensor([Lk - 20, 70], dtype=torch.int32, device="cuda")
    out = bd.sdpa_forward(dq, dk, dv, H, key_mask=dm, kv_valid_len=vl)
    assert torch.equal(out, rows128(dq, dk, dv, H, key_mask=dm, kv_valid_len=vl))
    for b, n in enumerate((Lk - 20, 70)):
        ref = oracle.sdpa(q[b], k[b, :n], v[b, :n], H, key_mask=m[b, :n], rows=rows)
        assert_close(ref[rows], to_np(out[b])[rows], dtype, f"short-kv key mask + valid length, batch {b}")
