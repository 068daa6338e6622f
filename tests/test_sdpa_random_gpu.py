"""Seeded random sweep of mi_sdpa_forward against the CPU checker: shapes, head dimensions, dtypes, mask modes, prefix
lengths, grouped-query factors and valid lengths drawn at random (fixed seeds), each case run on every kernel form
that accepts it (automatic choice, 128-row, 256-row, 256-row register-staged). Tolerances: helpers.TOL."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu

HEAD_DIMS = [40, 64, 72, 80, 96, 112, 128, 160]


def draw_case(seed):
    rng = np.random.default_rng(seed)
    d = int(rng.choice(HEAD_DIMS))
    dtype = "bf16" if rng.random() < 0.6 else "fp16"
    hkv = int(rng.choice([1, 2, 3]))
    group = int(rng.choice([1, 1, 2, 4]))
    H = hkv * group
    B = int(rng.choice([1, 1, 2, 3]))
    Lq = int(rng.integers(1, 420))
    Lk = int(rng.integers(1, 420))
    prefix = int(rng.choice([0, 0, int(rng.integers(1, 200))]))
    mode = str(rng.choice(["none", "none", "causal", "window", "block", "valid"]))
    return dict(seed=seed, d=d, dtype=dtype, H=H, hkv=hkv, B=B, Lq=Lq, Lk=Lk, prefix=prefix, mode=mode, rng=rng)


@pytest.mark.parametrize("seed", list(range(40)))
def test_random_case(oracle, seed):
    c = draw_case(seed)
    d, dtype, H, hkv, B, Lq, Lk, prefix, mode, rng = (c[k] for k in ("d", "dtype", "H", "hkv", "B", "Lq", "Lk", "prefix", "mode", "rng"))
    q = randn(10000 + seed, (B, Lq, H * d), dtype)
    k, v = randn(20000 + seed, (B, Lk, hkv * d), dtype), randn(30000 + seed, (B, Lk, hkv * d), dtype)
    kp = vp = None
    if prefix:
        kp, vp = randn(40000 + seed, (B, prefix, hkv * d), dtype), randn(50000 + seed, (B, prefix, hkv * d), dtype)
    Ltot = prefix + Lk
    mask, lo, hi, valid = None, None, None, None
    if mode == "causal":
        off = Ltot - Lq if Ltot >= Lq else 0
        mask = bd.SdpaMask.causal(off)
        lo, hi = oracle.rows_causal(Lq, Ltot, off, 0)
    elif mode == "window":
        off, win = max(Ltot - Lq, 0), int(rng.integers(1, 100))
        mask = bd.SdpaMask.causal(off, win)
        lo, hi = oracle.rows_causal(Lq, Ltot, off, win)
    elif mode == "block":
        n_seg = int(rng.integers(1, 5))
        cuts = sorted(set([Lq] + [int(x) for x in rng.integers(1, Lq + 1, n_seg - 1)])) if Lq > 1 else [Lq]
        sq = cuts
        sk = [min(Ltot, prefix + e) if Lk >= Lq else min(Ltot, max(1, int(rng.integers(1, Ltot + 1)))) for e in sq]
        sk = list(np.maximum.accumulate(sk))
        sc = [int(rng.random() < 0.4) for _ in sq]
        mask = bd.SdpaMask.block_causal(prefix, sq, sk, sc)
        lo, hi = oracle.rows_block_causal(Lq, Ltot, prefix, sq, sk, sc)
    elif mode == "valid":
        valid = [int(rng.integers(0, Ltot + 1)) for _ in range(B)]
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    kw = dict(num_kv_heads=hkv if hkv != H else 0, mask=mask)
    if prefix:
        kw.update(k_prefix=to_dev(kp, dtype), v_prefix=to_dev(vp, dtype))
    if valid is not None:
        kw.update(kv_valid_len=torch.tensor(valid, dtype=torch.int32, device="cuda"))
    choices = [0, 1] + ([2, 3] if d <= 128 else [])
    outs = []
    for ch in choices:
        bd.set_sdpa_kernel_choice(ch)
        try:
            outs.append(bd.sdpa_forward(dq, dk, dv, H, **kw))
        finally:
            bd.set_sdpa_kernel_choice(0)
    group = H // hkv
    for b in range(B):
        kk = k[b] if not prefix else np.concatenate([kp[b], k[b]])
        vv = v[b] if not prefix else np.concatenate([vp[b], v[b]])
        # the checker takes one K/V head per query head: widen grouped K/V
        kk = np.repeat(kk.reshape(-1, hkv, d), group, axis=1).reshape(-1, H * d)
        vv = np.repeat(vv.reshape(-1, hkv, d), group, axis=1).reshape(-1, H * d)
        rl, rh = lo, hi
        if valid is not None:
            rl = np.zeros(Lq, np.int32)
            rh = np.full(Lq, valid[b], np.int32)
        ref = oracle.sdpa(q[b], kk, vv, H, row_lo=rl, row_hi=rh)
        for ch, o in zip(choices, outs):
            assert_close(ref, to_np(o[b]), dtype, f"seed {seed} {c['mode']} d={d} choice {ch} batch {b}")
