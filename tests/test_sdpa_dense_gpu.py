"""The dense instances of the 256-row kernels (no mask, no prefix, key count a multiple of 64) on query counts that are
not a multiple of the tile: the rows past the end repeat the last query row inside the kernel and must not be stored.
Sampled rows against the CPU checker, the rest against the general instance of the same kernel (reached by passing a
valid length equal to the key count)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,d,H,B,Lq,Lk", [
    ("bf16", 128, 16, 2, 3999, 4096),     # LDS-DMA kernel
    ("bf16", 72, 16, 2, 4001, 1024),      # LDS-DMA kernel, head_dim 72
    ("fp16", 40, 8, 4, 2050, 2048),       # register-staged kernel
    ("bf16", 64, 16, 2, 3841, 640),
])
def test_dense_instance_ragged_queries(oracle, dtype, d, H, B, Lq, Lk):
    q = randn(601, (B, Lq, H * d), dtype)
    k = randn(602, (B, Lk, H * d), dtype)
    v = randn(603, (B, Lk, H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    guard = torch.full((B, Lq + 300, H * d), 7.0, device="cuda", dtype=dq.dtype)   # rows behind the output stay untouched
    out = guard[:, :Lq]
    bd.sdpa_forward(dq, dk, dv, H, out=out, split_scratch=False)
    assert (guard[:, Lq:] == 7.0).all()
    full = torch.tensor([Lk] * B, dtype=torch.int32, device="cuda")
    general = bd.sdpa_forward(dq, dk, dv, H, kv_valid_len=full, split_scratch=False)
    unit = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    assert (out.float() - general.float()).abs().max().item() <= unit * max(1.0, general.float().abs().max().item())
    rows = [0, 255, 256, Lq - 257, Lq - 2, Lq - 1]
    for b in (0, B - 1):
        ref = oracle.sdpa(q[b][rows], k[b], v[b], H)
        assert_close(ref, to_np(out[b][rows]), dtype, f"batch {b}")


@pytest.mark.parametrize("dtype,d,H,Hkv,B,Lq,Lk,axes", [
    ("bf16", 128, 16, 4, 2, 2304, 2304, (16, 56, 56)),    # LDS-DMA kernel, grouped-query heads, RoPE on Q (on load) and K (scratch)
    ("fp16", 64, 16, 8, 2, 2304, 2304, (16, 24, 24)),     # register-staged kernel
])
def test_dense_instance_gqa_and_rope(oracle, dtype, d, H, Hkv, B, Lq, Lk, axes):
    """The dense instances with everything that is allowed next to them: fewer key / value heads than query heads and
    RoPE fused into the Q load, K rotated into a scratch. Sampled rows against the checker."""
    txt, hp, wp = 256, 32, 64
    assert txt + hp * wp == Lq == Lk
    q = randn(611, (B, Lq, H * d), dtype)
    k = randn(612, (B, Lk, Hkv * d), dtype)
    v = randn(613, (B, Lk, Hkv * d), dtype)
    cos, sin = oracle.build_axial_rope_tables(txt, hp, wp, d, axes)
    dcos, dsin = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    kr = torch.empty_like(dk)
    out = bd.sdpa_forward(dq, dk, dv, H, num_kv_heads=Hkv, rope_q=(dcos, dsin), rope_k=(dcos, dsin), rope_k_scratch=kr,
                          split_scratch=False)
    rows = [0, 300, Lq - 1]
    group = H // Hkv
    for b in (0, B - 1):
        qr = oracle.rope_apply(q[b][rows], cos[rows], sin[rows], H, d, round_to_dtype=dtype)
        krr = oracle.rope_apply(k[b], cos, sin, Hkv, d, round_to_dtype=dtype)
        # widen K / V to one head per query head for the checker
        kw = np.repeat(krr.reshape(Lk, Hkv, d), group, axis=1).reshape(Lk, H * d)
        vw = np.repeat(v[b].reshape(Lk, Hkv, d), group, axis=1).reshape(Lk, H * d)
        ref = oracle.sdpa(qr, kw, vw, H)
        assert_close(ref, to_np(out[b][rows]), dtype, f"batch {b}")


def test_dense_instance_with_cached_prefix(oracle):
    """The cached step of the Qwen-Image transformer (src/dit/qwenimage21_forward.cpp:599-649): unmasked, queries are
    the target rows, keys are [cached prefix ; fresh]. With whole tiles on both segments it runs on the dense instance;
    it must agree with the call on the concatenated keys and with the checker."""
    dtype, H, d, Lq, Lp = "bf16", 24, 128, 3072, 512
    q = randn(621, (Lq, H * d), dtype)
    k = randn(622, (Lq, H * d), dtype); v = randn(623, (Lq, H * d), dtype)
    kp = randn(624, (Lp, H * d), dtype); vp = randn(625, (Lp, H * d), dtype)
    dq, dk, dv, dkp, dvp = (to_dev(a, dtype) for a in (q, k, v, kp, vp))
    out = bd.sdpa_forward(dq, dk, dv, H, k_prefix=dkp, v_prefix=dvp, split_scratch=False)
    cat = bd.sdpa_forward(dq, torch.cat([dkp, dk]), torch.cat([dvp, dv]), H, split_scratch=False)
    assert (out.float() - cat.float()).abs().max().item() <= 2.0 ** -7 * max(1.0, cat.float().abs().max().item())
    rows = [0, 511, 2000, Lq - 1]
    ref = oracle.sdpa(q[rows], np.concatenate([kp, k]), np.concatenate([vp, v]), H)
    assert_close(ref, to_np(out[rows]), dtype, "cached prefix, dense instance")
    # a prefix that is not whole tiles takes the general instance and must give the same rows
    out2 = bd.sdpa_forward(dq, dk, dv, H, k_prefix=dkp[:500], v_prefix=dvp[:500], split_scratch=False)
    ref2 = oracle.sdpa(q[rows], np.concatenate([kp[:500], k]), np.concatenate([vp[:500], v]), H)
    assert_close(ref2, to_np(out2[rows]), dtype, "cached prefix of 500 rows")
