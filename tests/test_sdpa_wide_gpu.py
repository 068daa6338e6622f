"""Head dimensions 256, 384 and 512 (the single wide head of the VAE mid-block attention, src/vae.cpp:259-277, reached through
flash_attention_qkvo_forward with one head) against the CPU checker: plain, ragged, causal / windowed, key padding three
ways, a scattered key mask, grouped K/V heads, batch, and the block operator itself with one head of 512 channels."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,H,d,Lq,Lk", [
    ("bf16", 1, 512, 300, 300),     # ragged: 9 full query tiles and one of 12 rows, keys end mid-tile
    ("fp16", 1, 512, 256, 256),
    ("fp16", 1, 256, 65, 64),
    ("bf16", 2, 256, 100, 333),
    ("bf16", 1, 384, 200, 131),    # the Qwen-Image VAE's width (src/vae_qwenimage.cpp:322-340)
    ("fp16", 2, 384, 33, 64),
    ("bf16", 1, 512, 1, 1),
])
def test_wide_head_matches_checker(oracle, dtype, H, d, Lq, Lk):
    q = randn(8501, (Lq, H * d), dtype); k = randn(8502, (Lk, H * d), dtype); v = randn(8503, (Lk, H * d), dtype)
    out = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, False)
    print(d, Lq, Lk, assert_close(oracle.sdpa(q, k, v, H), to_np(out), dtype, f"d={d} {Lq}x{Lk}"))


def test_wide_head_peaked_logits(oracle):
    """Queries scaled up: the softmax reference is raised along the keys; the result must not depend on it."""
    dtype, H, d, Lq, Lk = "bf16", 1, 512, 64, 320
    q = randn(8511, (Lq, H * d), dtype) * 4; k = randn(8512, (Lk, H * d), dtype); v = randn(8513, (Lk, H * d), dtype)
    q = oracle.round_to(q, dtype)
    out = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, False)
    assert_close(oracle.sdpa(q, k, v, H), to_np(out), dtype, "peaked")


@pytest.mark.parametrize("window", [0, 50])
def test_wide_head_causal_windowed(oracle, window):
    dtype, H, d, Lq, Lk = "bf16", 1, 256, 150, 290
    q = randn(8521, (Lq, H * d), dtype); k = randn(8522, (Lk, H * d), dtype); v = randn(8523, (Lk, H * d), dtype)
    out = bd.flash_attention_windowed_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, window)
    lo, hi = oracle.rows_causal(Lq, Lk, window=window)
    assert_close(oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi), to_np(out), dtype, f"window={window}")
    # rows without any visible key give zeros (src/dit/common.cpp:293)
    out0 = to_np(bd.flash_attention_windowed_forward(to_dev(q, dtype), to_dev(k[:40], dtype), to_dev(v[:40], dtype), None, H, 0))
    assert not out0[:110].any() and out0[110:].any()


def test_wide_head_key_padding_and_masks(oracle):
    dtype, B, H, d, Lq, Lk = "fp16", 2, 1, 512, 70, 200
    valid = [77, 200]
    q = randn(8531, (B, Lq, H * d), dtype); k = randn(8532, (B, Lk, H * d), dtype); v = randn(8533, (B, Lk, H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    o_len = bd.sdpa_forward(dq, dk, dv, H, kv_valid_len=torch.tensor(valid, dtype=torch.int32, device="cuda"))
    m = np.zeros((B, Lk), np.float32)
    for b in range(B):
        m[b, :valid[b]] = 1
    o_mask = bd.flash_attention_forward(dq, dk, dv, torch.from_numpy(m).cuda(), H, False)
    for b in range(B):
        ref = oracle.sdpa(q[b], k[b, :valid[b]], v[b, :valid[b]], H)
        assert_close(ref, to_np(o_len[b]), dtype, "kv_valid_len")
        assert_close(ref, to_np(o_mask[b]), dtype, "d_mask")
        o_trim = bd.flash_attention_forward(dq[b], dk[b, :valid[b]], dv[b, :valid[b]], None, H, False)
        assert torch.equal(o_trim, o_len[b]) and torch.equal(o_trim, o_mask[b])     # padding = trimming (src/pipeline.cpp:391-414)
    sm = (np.random.default_rng(8).uniform(size=Lk) > 0.5).astype(np.float32)
    sm[64:128] = 0                                                                  # a whole key tile hidden
    out = bd.flash_attention_forward(dq[0], dk[0], dv[0], torch.from_numpy(sm).cuda(), H, False)
    assert_close(oracle.sdpa(q[0], k[0], v[0], H, key_mask=sm), to_np(out), dtype, "scattered mask")
    out0 = bd.flash_attention_forward(dq[0], dk[0], dv[0], torch.zeros(Lk, device="cuda"), H, False)
    assert not to_np(out0).any()                                                    # nothing visible: zeros


def test_wide_head_grouped_kv(oracle):
    dtype, Hq, Hkv, d, Lq, Lk = "bf16", 4, 2, 256, 90, 130
    q = randn(8541, (Lq, Hq * d), dtype); k = randn(8542, (Lk, Hkv * d), dtype); v = randn(8543, (Lk, Hkv * d), dtype)
    out = bd.sdpa_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), Hq, num_kv_heads=Hkv)
    kw = np.concatenate([k[:, (h // 2) * d:(h // 2 + 1) * d] for h in range(Hq)], axis=1)
    vw = np.concatenate([v[:, (h // 2) * d:(h // 2 + 1) * d] for h in range(Hq)], axis=1)
    assert_close(oracle.sdpa(q, kw, vw, Hq), to_np(out), dtype, "gqa")


def test_vae_mid_block_attention(oracle):
    """The call of src/vae.cpp:268: flash_attention_qkvo_forward over (tokens, 512) with ONE head, biases on all four
    projections, no mask."""
    dtype, L, C = "fp16", 320, 512
    x = randn(8551, (1, L, C), dtype)
    w = {n: oracle.round_to(randn(8552 + i, (C, C), dtype) / np.sqrt(C), dtype) for i, n in enumerate(("wq", "wk", "wv", "wo"))}
    bs = {n: oracle.round_to(randn(8560 + i, (C,), dtype) * 0.1, dtype) for i, n in enumerate(("bq", "bk", "bv", "bo"))}
    d = {n: to_dev(a, dtype) for n, a in {**w, **bs}.items()}
    out = bd.flash_attention_qkvo_forward(to_dev(x, dtype), None, d["wq"], d["bq"], d["wk"], d["bk"], d["wv"], d["bv"], d["wo"], d["bo"],
                                          None, 1, False)
    ref = oracle.attention_qkvo(x[0], None, w["wq"], bs["bq"], w["wk"], bs["bk"], w["wv"], bs["bv"], w["wo"], bs["bo"], 1, dtype)
    assert_close(ref, to_np(out[0]), dtype, "vae mid block")


def test_wide_head_refuses_what_it_does_not_offer():
    H, d, L = 1, 512, 64
    q = torch.zeros(L, H * d, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="head_dim 512 does not offer a cached prefix"):
        bd.sdpa_forward(q, q, q, H, k_prefix=q[:8].clone(), v_prefix=q[:8].clone())
    with pytest.raises(RuntimeError, match="does not offer packed"):
        cu = torch.tensor([0, 32, 64], dtype=torch.int32, device="cuda")
        bd.flash_attention_varlen_forward(q, q, q, cu, cu, 2, 32, 32, H, d, False)


@pytest.mark.parametrize("split_half", [False, True], ids=["adjacent", "split_half"])
@pytest.mark.parametrize("dtype,d", [("bf16", 256), ("fp16", 384), ("bf16", 512)])
def test_wide_head_rope(oracle, dtype, d, split_half):
    """Q rotated while it is staged and K rotated into the caller's scratch at the wide head dimensions, both pair
    conventions: bit-equal to the stand-alone rotation followed by plain attention, and within the bound of the checker."""
    H, L = 1, 150
    q, k, v = (randn(8570 + d + i, (L, H * d), dtype) for i in range(3))
    ang = np.random.default_rng(d).uniform(-3, 3, (L, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    dcos, dsin = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    qr = bd.rope_apply(dq, dcos, dsin, d, H, split_half=split_half)
    kr = bd.rope_apply(dk, dcos, dsin, d, H, split_half=split_half)
    plain = bd.sdpa_forward(qr, kr, dv, H)
    fused_q = bd.sdpa_forward(dq, kr, dv, H, rope_q=(dcos, dsin), rope_split_half=split_half)
    assert torch.equal(fused_q, plain)
    Kr = torch.empty_like(dk)
    joint = bd.joint_attention(dq, dk, dv, dcos, dsin, d, H, Kr=Kr, split_half=split_half)
    assert torch.equal(Kr, kr) and torch.equal(joint, plain)
    ref = oracle.sdpa(oracle.rope_apply(q, cos, sin, H, d, split_half=split_half, round_to_dtype=dtype),
                      oracle.rope_apply(k, cos, sin, H, d, split_half=split_half, round_to_dtype=dtype), v, H)
    assert_close(ref, to_np(joint), dtype, f"wide head rope d={d} split_half={split_half}")
    # without a scratch the rotation of K would have to happen tile by tile, which these widths do not offer: refused
    # before anything is enqueued
    with pytest.raises(RuntimeError, match="does not offer K rotated tile by tile|needs rope_k_scratch"):
        bd.joint_attention(dq, dk, dv, dcos, dsin, d, H, split_half=split_half)
