"""Seeded random sweep at sizes that reach the 256-row kernels under the automatic choice (at least one 256-row query
tile per compute unit): LDS-DMA, register-staged, short-key and split launches with random lengths, masks, prefixes
and valid lengths. Sampled rows against the CPU checker (helpers.TOL) and the whole output against the 128-row kernel
(<= 2 units in the last place: the two use different softmax references)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def max_ulp_diff(a, b):
    unit = 2.0 ** -8 if a.dtype == torch.bfloat16 else 2.0 ** -11
    return (a.float() - b.float()).abs().max().item() / (unit * max(1.0, b.float().abs().max().item()))


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_large_case(oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    d = int(rng.choice([40, 64, 72, 128]))
    dtype = "bf16" if rng.random() < 0.6 else "fp16"
    B = int(rng.choice([1, 2]))
    H = int(rng.choice([8, 16, 24]))
    need_tiles = -(-256 // (B * H))                      # query tiles per (batch, head) for 256 tiles in all
    Lq = 256 * need_tiles + int(rng.integers(-200, 300))
    Lq = max(Lq, 256 * (need_tiles - 1) + 1)
    mode = str(rng.choice(["none", "short", "causal", "block", "valid", "prefix"]))
    Lk = int(rng.integers(20, 320)) if mode == "short" else int(rng.integers(300, 1500))
    prefix = int(rng.integers(1, 400)) if mode in ("prefix", "block") else 0
    q = randn(60000 + seed, (B, Lq, H * d), dtype)
    k, v = randn(61000 + seed, (B, Lk, H * d), dtype), randn(62000 + seed, (B, Lk, H * d), dtype)
    kw, lo, hi, valid = {}, None, None, None
    kp = vp = None
    if prefix:
        kp, vp = randn(63000 + seed, (B, prefix, H * d), dtype), randn(64000 + seed, (B, prefix, H * d), dtype)
        kw.update(k_prefix=to_dev(kp, dtype), v_prefix=to_dev(vp, dtype))
    Ltot = prefix + Lk
    if mode == "causal":
        off = max(Ltot - Lq, 0)
        kw["mask"] = bd.SdpaMask.causal(off)
        lo, hi = oracle.rows_causal(Lq, Ltot, off, 0)
    elif mode == "block":
        cuts = sorted(set([Lq] + [int(x) for x in rng.integers(1, Lq, 3)]))
        sk = list(np.maximum.accumulate([min(Ltot, prefix + int(e * Lk / Lq) + 1) for e in cuts]))
        sc = [int(rng.random() < 0.3) for _ in cuts]
        kw["mask"] = bd.SdpaMask.block_causal(prefix, cuts, sk, sc)
        lo, hi = oracle.rows_block_causal(Lq, Ltot, prefix, cuts, sk, sc)
    elif mode in ("valid", "short") and rng.random() < 0.7:
        valid = [int(rng.integers(1, Ltot + 1)) for _ in range(B)]
        kw["kv_valid_len"] = torch.tensor(valid, dtype=torch.int32, device="cuda")
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    out = bd.sdpa_forward(dq, dk, dv, H, **kw)
    bd.set_sdpa_kernel_choice(1)
    try:
        small = bd.sdpa_forward(dq, dk, dv, H, **kw)
    finally:
        bd.set_sdpa_kernel_choice(0)
    assert max_ulp_diff(out, small) <= 2.0, f"seed {seed} {mode} d={d}"
    rows = np.unique(np.concatenate([rng.integers(0, Lq, 24), [0, Lq - 1, min(255, Lq - 1), min(256, Lq - 1)]])).astype(np.int32)
    for b in range(B):
        kk = k[b] if not prefix else np.concatenate([kp[b], k[b]])
        vv = v[b] if not prefix else np.concatenate([vp[b], v[b]])
        rl, rh = lo, hi
        if valid is not None:
            rl, rh = np.zeros(Lq, np.int32), np.full(Lq, valid[b], np.int32)
        ref = oracle.sdpa(q[b], kk, vv, H, row_lo=rl, row_hi=rh, rows=rows)
        assert_close(ref[rows], to_np(out[b])[rows], dtype, f"seed {seed} {mode} d={d} B={B} H={H} Lq={Lq} Lk={Lk} prefix={prefix} batch {b}")
