"""The prefix-KV dial of the Qwen-Image cached step inside the attention kernels: factors on the rows of the cached prefix
K and V (a scalar per side, optionally times a per-row weight), src/dit/qwenimage21_forward.cpp:606-645. The reference
scales a copy of the cached rows, rounds it to the storage type and attends over [copy ; fresh]; the kernels multiply the
FP32 scores of the prefix keys and, after the row sum, their probabilities instead. Checked against the CPU checker on
prefix rows scaled in FP32 (the mathematics), against the reference's dataflow run on the GPU (mi_scale_rows into a copy,
then the plain call), and for the properties the reference's own test of the dial holds
(tests/test_qwenimage21_slots.cpp:361-412, :580-625): the cache is never written, the same setting twice is the same
result bit for bit, a scale of 1 is no scale, an all-ones row weight is the broadcast, scalar and row weight compose."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu

KERNELS = {"auto": 0, "rows128": 1, "rows256": 2}


@pytest.fixture(autouse=True, params=list(KERNELS))
def kernel_choice(request):
    bd.set_sdpa_kernel_choice(KERNELS[request.param])
    yield request.param
    bd.set_sdpa_kernel_choice(0)


def _inputs(dtype, H, d, Lq, Lp, Lf, seed):
    q = randn(seed, (Lq, H * d), dtype)
    kp, vp = randn(seed + 1, (Lp, H * d), dtype), randn(seed + 2, (Lp, H * d), dtype)
    k, v = randn(seed + 3, (Lf, H * d), dtype), randn(seed + 4, (Lf, H * d), dtype)
    return q, kp, vp, k, v


def _reference(oracle, q, kp, vp, k, v, H, fk, fv, **kw):
    """Prefix rows times their factors in FP32 (no rounding), then plain attention over [prefix ; fresh]."""
    return oracle.sdpa(q, np.concatenate([kp * fk[:, None], k]), np.concatenate([vp * fv[:, None], v]), H, **kw)


@pytest.mark.parametrize("dtype,H,d,Lq,Lp,Lf", [("bf16", 4, 128, 300, 512, 320), ("bf16", 4, 128, 300, 333, 200),
                                                ("bf16", 3, 72, 260, 130, 190), ("fp16", 2, 64, 200, 100, 150)])
@pytest.mark.parametrize("rows", [False, True], ids=["scalar", "per_row"])
def test_dial_matches_checker_and_scaled_copy(oracle, dtype, H, d, Lq, Lp, Lf, rows):
    q, kp, vp, k, v = _inputs(dtype, H, d, Lq, Lp, Lf, 8300 + Lp)
    ks, vs = 0.75, 0.5
    rng = np.random.default_rng(Lp)
    rk = rng.uniform(0.0, 1.5, Lp).astype(np.float32) if rows else None
    rv = rng.uniform(0.0, 1.5, Lp).astype(np.float32) if rows else None
    if rows:
        rk[3] = 0.0; rv[5] = 0.0                       # a fully attenuated token on either side
    fk = ks * (rk if rows else np.ones(Lp, np.float32)); fv = vs * (rv if rows else np.ones(Lp, np.float32))
    dq, dkp, dvp, dk, dv = (to_dev(x, dtype) for x in (q, kp, vp, k, v))
    cache_before = (dkp.clone(), dvp.clone())
    drk = None if rk is None else torch.from_numpy(rk).cuda()
    drv = None if rv is None else torch.from_numpy(rv).cuda()
    kw = dict(k_prefix=dkp, v_prefix=dvp, prefix_k_scale=ks, prefix_v_scale=vs, prefix_k_row_scale=drk, prefix_v_row_scale=drv)
    out = bd.sdpa_forward(dq, dk, dv, H, **kw)
    assert torch.equal(dkp, cache_before[0]) and torch.equal(dvp, cache_before[1])       # the cache stays pristine
    assert_close(_reference(oracle, q, kp, vp, k, v, H, fk, fv), to_np(out), dtype, "dial vs checker")
    assert torch.equal(bd.sdpa_forward(dq, dk, dv, H, **kw), out)                        # the same setting again
    # the reference's dataflow on the GPU: scale a copy of the prefix rows (rounded to the storage type), then the plain call
    kc = bd.scale_rows(dkp, ks, drk); vc = bd.scale_rows(dvp, vs, drv)
    copy_route = bd.sdpa_forward(dq, dk, dv, H, k_prefix=kc, v_prefix=vc)
    m = oracle.compare(to_np(copy_route), to_np(out))
    assert m["rel_l2"] <= TOL[dtype][0] and m["max_abs"] <= TOL[dtype][1], m
    # it is a different result from the unscaled one
    plain = bd.sdpa_forward(dq, dk, dv, H, k_prefix=dkp, v_prefix=dvp)
    assert (plain.float() - out.float()).abs().max().item() > 1e-2


def test_dial_identities_and_composition(oracle):
    dtype, H, d, Lq, Lp, Lf = "bf16", 4, 128, 300, 256, 320
    q, kp, vp, k, v = (to_dev(x, dtype) for x in _inputs(dtype, H, d, Lq, Lp, Lf, 8400))
    base = dict(k_prefix=kp, v_prefix=vp)
    plain = bd.sdpa_forward(q, k, v, H, **base)
    # a scale of exactly 1 is no scale: bit for bit the unscaled call
    assert torch.equal(bd.sdpa_forward(q, k, v, H, prefix_k_scale=1.0, prefix_v_scale=1.0, **base), plain)
    ones = torch.ones(Lp, device="cuda")
    scalar = bd.sdpa_forward(q, k, v, H, prefix_k_scale=1.0, prefix_v_scale=0.5, **base)
    # an all-ones row weight is the broadcast it replaces
    assert torch.equal(bd.sdpa_forward(q, k, v, H, prefix_k_scale=1.0, prefix_v_scale=0.5, prefix_k_row_scale=ones,
                                       prefix_v_row_scale=ones, **base), scalar)
    # scalar and row weight compose: rows in {0, 1/2, 1} times 1/2 equal rows in {0, 1/4, 1/2} times 1 (all products exact)
    r = torch.tensor([0.0, 0.5, 1.0], device="cuda").repeat(Lp // 3 + 1)[:Lp].contiguous()
    a = bd.sdpa_forward(q, k, v, H, prefix_k_scale=0.5, prefix_v_scale=0.5, prefix_k_row_scale=r, prefix_v_row_scale=r, **base)
    b = bd.sdpa_forward(q, k, v, H, prefix_k_row_scale=(r * 0.5).contiguous(), prefix_v_row_scale=(r * 0.5).contiguous(), **base)
    assert torch.equal(a, b)
    assert not torch.equal(a, scalar)
    # V factors of zero on every prefix row leave the prefix in the denominator only: output = (fresh part) * its share
    zero_v = bd.sdpa_forward(q, k, v, H, prefix_v_row_scale=torch.zeros(Lp, device="cuda"), **base)
    fresh_only = bd.sdpa_forward(q, k, v, H)
    assert (zero_v.float().abs() <= fresh_only.float().abs() * 1.02 + 1e-3).all()


def test_dial_with_block_causal_mask(oracle):
    """The cached prefix in front of block-causal image blocks (the shape of the fifth benchmark configuration, smaller)."""
    dtype, H, d, Lp, blocks, bl = "bf16", 4, 128, 192, 3, 128
    Lq = blocks * bl
    q, kp, vp, k, v = _inputs(dtype, H, d, Lq, Lp, Lq, 8500)
    sq = [bl * (i + 1) for i in range(blocks)]
    sk = [Lp + e for e in sq]
    mask = bd.SdpaMask.block_causal(Lp, sq, sk, [0] * blocks)
    rk = np.linspace(0.2, 1.2, Lp).astype(np.float32); rv = np.linspace(1.2, 0.2, Lp).astype(np.float32)
    dq, dkp, dvp, dk, dv = (to_dev(x, dtype) for x in (q, kp, vp, k, v))
    out = bd.sdpa_forward(dq, dk, dv, H, k_prefix=dkp, v_prefix=dvp, mask=mask, prefix_k_scale=0.9, prefix_v_scale=1.1,
                          prefix_k_row_scale=torch.from_numpy(rk).cuda(), prefix_v_row_scale=torch.from_numpy(rv).cuda())
    lo, hi = oracle.rows_block_causal(Lq, Lp + Lq, Lp, sq, sk, [0] * blocks)
    ref = _reference(oracle, q, kp, vp, k, v, H, 0.9 * rk, 1.1 * rv, row_lo=lo, row_hi=hi)
    assert_close(ref, to_np(out), dtype, "dial under a block-causal mask")


def test_dial_errors():
    z = lambda *s: torch.zeros(*s, dtype=torch.bfloat16, device="cuda")
    q, kp, k = z(64, 256), z(32, 256), z(64, 256)
    with pytest.raises(RuntimeError, match="prefix_k_row_scale must be a contiguous float32 tensor of prefix_len"):
        bd.sdpa_forward(q, k, k, 2, k_prefix=kp, v_prefix=kp, prefix_k_row_scale=torch.zeros(31, device="cuda"))
    with pytest.raises(RuntimeError, match="must be finite"):
        bd.sdpa_forward(q, k, k, 2, k_prefix=kp, v_prefix=kp, prefix_k_scale=float("inf"))
