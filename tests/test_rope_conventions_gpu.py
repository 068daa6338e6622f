"""Both pair conventions of RoPE on every fused path. What bt::rope_apply does inside brotensor (adjacent pairs
(x[2p], x[2p+1]) or the two halves of a head (x[p], x[p + d/2])) cannot be read from the reference, which only calls it
(src/dit/common.cpp:192-193, src/dit/qwenimage21_forward.cpp:584-585, src/triposplat/flow_model.cpp:374); so each
rotation that is fused into another kernel must offer both and agree bit for bit with the stand-alone pass of the same
convention: Q rotated on load, K rotated into the Kr scratch, and the rotation behind the head RMSNorm."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def _tables(L, d, seed):
    ang = np.random.default_rng(seed).uniform(-3, 3, (L, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    return cos, sin, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()


@pytest.mark.parametrize("choice", [1, 2, 3], ids=["rows128", "rows256", "rows256_regs"])
@pytest.mark.parametrize("split_half", [False, True], ids=["adjacent", "split_half"])
@pytest.mark.parametrize("dtype,d", [("bf16", 128), ("fp16", 40), ("bf16", 72), ("fp16", 64), ("bf16", 160)])
def test_fused_rotation_equals_standalone_pass(oracle, dtype, d, split_half, choice):
    if d == 160 and choice != 1:
        pytest.skip("head_dim 160 has the 128-row kernel only")
    H, L = 2, 333
    q, k, v = (randn(7000 + d + i, (L, H * d), dtype) for i in range(3))
    cos, sin, dcos, dsin = _tables(L, d, d)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    bd.set_sdpa_kernel_choice(choice)
    try:
        qr = bd.rope_apply(dq, dcos, dsin, d, H, split_half=split_half)
        kr = bd.rope_apply(dk, dcos, dsin, d, H, split_half=split_half)
        plain = bd.sdpa_forward(qr, kr, dv, H)
        # Q rotated while it is loaded
        fused_q = bd.sdpa_forward(dq, kr, dv, H, rope_q=(dcos, dsin), rope_split_half=split_half)
        assert torch.equal(fused_q, plain)
        # ... and K rotated into the scratch by the call itself (the form of dit::joint_attention)
        Kr = torch.empty_like(dk)
        joint = bd.joint_attention(dq, dk, dv, dcos, dsin, d, H, Kr=Kr, split_half=split_half)
        assert torch.equal(Kr, kr) and torch.equal(joint, plain)
    finally:
        bd.set_sdpa_kernel_choice(0)
    ref = oracle.sdpa(oracle.rope_apply(q, cos, sin, H, d, split_half=split_half, round_to_dtype=dtype),
                      oracle.rope_apply(k, cos, sin, H, d, split_half=split_half, round_to_dtype=dtype), v, H)
    assert_close(ref, to_np(joint), dtype, f"d={d} split_half={split_half}")
    if split_half:
        # without a scratch K would be rotated tile by tile, which exists for adjacent pairs only
        with pytest.raises(RuntimeError, match="needs rope_k_scratch"):
            bd.joint_attention(dq, dk, dv, dcos, dsin, d, H, split_half=True)


def test_the_two_conventions_differ(oracle):
    """A test that could not tell the conventions apart would pin nothing."""
    dtype, H, d, L = "bf16", 2, 128, 100
    q, k, v = (to_dev(randn(7100 + i, (L, H * d), dtype), dtype) for i in range(3))
    _, _, dcos, dsin = _tables(L, d, 5)
    a = bd.joint_attention(q, k, v, dcos, dsin, d, H, Kr=torch.empty_like(k))
    b = bd.joint_attention(q, k, v, dcos, dsin, d, H, Kr=torch.empty_like(k), split_half=True)
    assert (a.float() - b.float()).abs().max().item() > 0.05


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("L,H,d", [(300, 24, 128), (65, 5, 64), (33, 70, 32)])
def test_headnorm_rope_split_half(oracle, dtype, L, H, d):
    x = oracle.round_to(randn(7200 + L, (L, H * d), dtype) * 2.5, dtype)
    gain = oracle.round_to(1.0 + 0.2 * randn(7201, (d,), "fp32"), dtype)
    cos, sin, dcos, dsin = _tables(L, d, 7)
    dx, dg = to_dev(x, dtype), to_dev(gain, dtype)
    out = bd.headnorm_rope(dx, dg, 1e-6, dcos, dsin, d, H, split_half=True)
    normed = oracle.rms_norm(x.reshape(L * H, d), gain, 1e-6).reshape(L, H * d)       # FP32, unrounded
    exact = oracle.rope_apply(normed, cos, sin, H, d, split_half=True)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.all(np.abs(to_np(out) - exact) <= unit * np.maximum(np.abs(exact), 2.0 ** -6) * 1.02 + 1e-6)
    # the adjacent form of the same call is something else, and the cache rows follow the convention too
    adj = bd.headnorm_rope(dx, dg, 1e-6, dcos, dsin, d, H)
    assert (out.float() - adj.float()).abs().max().item() > 0.05
    cache = torch.zeros((L // 2, H * d), dtype=dx.dtype, device="cuda")
    out2 = bd.headnorm_rope(dx, dg, 1e-6, dcos, dsin, d, H, cache_out=cache, split_half=True)
    assert torch.equal(out2, out) and torch.equal(cache, out[:L // 2])
    # composed from the two library passes (two roundings): close, not equal
    composed = bd.rope_apply(bd.headnorm_rope(dx, dg, 1e-6, None, None, d, H), dcos, dsin, d, H, split_half=True)
    m = oracle.compare(to_np(composed), to_np(out))
    assert m["rel_l2"] <= TOL[dtype][0]


@pytest.mark.parametrize("dtype,H,d,L", [("bf16", 3, 128, 77), ("fp16", 2, 64, 130), ("bf16", 1, 80, 9)])
def test_split_half_vector_and_scalar_kernels_agree(oracle, dtype, H, d, L):
    """The stand-alone split-half pass has a 16-byte form (whole chunks per half head) and a per-pair form; a strided
    view whose rows are not 16-byte aligned takes the second. Same results, and per-head tables in both."""
    x = randn(7300 + d, (L, H * d), dtype)
    cos, sin, dcos, dsin = _tables(L, d, 9)
    dx = to_dev(x, dtype)
    a = bd.rope_apply(dx, dcos, dsin, d, H, split_half=True)
    wide = torch.zeros((L, H * d + 4), dtype=dx.dtype, device="cuda")
    wide[:, 4:] = dx                                     # rows start 8 bytes off a 16-byte boundary
    b = bd.rope_apply(wide[:, 4:], dcos, dsin, d, H, split_half=True)
    assert torch.equal(a, b)
    ref = oracle.rope_apply(x, cos, sin, H, d, split_half=True)
    ulp = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11      # one rounding to the storage dtype
    assert np.max(np.abs(to_np(a) - ref) / np.maximum(np.abs(ref), 1.0)) <= ulp


@pytest.mark.parametrize("dtype,H,d,L", [("bf16", 24, 128, 517), ("fp16", 8, 40, 1000), ("bf16", 16, 72, 77), ("bf16", 4, 32, 3), ("fp16", 12, 64, 130)])
def test_adjacent_pairs_with_head_count_a_multiple_of_four(oracle, dtype, H, d, L):
    """Head counts that are multiples of 4 take the stand-alone pass in which a thread rotates one chunk position of 4 heads
    with one fetch of the table entries. Same arithmetic as the general pass: bit-equal to the per-head-table entry point
    fed the same table once per head (which runs the general pass), on contiguous rows and on column slices of wider
    buffers; and within the usual bound of the checker."""
    x = randn(7300 + H + d, (L, H * d), dtype)
    cos, sin, dcos, dsin = _tables(L, d, 31 + d)
    dx = to_dev(x, dtype)
    got = bd.rope_apply(dx, dcos, dsin, d, H)
    per_head = bd.rope_apply_perhead(dx, dcos.repeat_interleave(H, dim=0).contiguous(), dsin.repeat_interleave(H, dim=0).contiguous(), d, H)
    assert torch.equal(got, per_head)
    ref = oracle.rope_apply(x, cos, sin, H, d, round_to_dtype=dtype)
    assert_close(ref, to_np(got), dtype, f"rope H={H} d={d}")
    wide_in = torch.zeros((L, 2 * H * d + 8), dtype=dx.dtype, device="cuda")
    wide_in[:, 8:8 + H * d] = dx
    wide_out = torch.full((L, 3 * H * d), 7.0, dtype=dx.dtype, device="cuda")
    bd.rope_apply(wide_in[:, 8:8 + H * d], dcos, dsin, d, H, out=wide_out[:, H * d:2 * H * d])
    assert torch.equal(wide_out[:, H * d:2 * H * d], got)
    assert (wide_out[:, :H * d] == 7).all() and (wide_out[:, 2 * H * d:] == 7).all()
