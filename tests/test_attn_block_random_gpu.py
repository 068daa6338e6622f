"""Seeded random sweep of the U-Net attention-block operators (flash_attention_qkvo_forward,
flash_attention_project_kv + flash_attention_q_with_kv_cached_forward; src/unet_blocks.cpp:253-330, src/unet.cpp:470-480)
against the CPU checker's composition: head dims, head counts, ragged lengths, context widths, key masks, causal, biases."""
import math
import random

import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_attention_block(oracle, seed):
    rng = random.Random(9100 + seed)
    dtype = rng.choice(["fp16", "bf16"])
    hd = rng.choice([40, 64, 72, 80, 96, 128])
    H = rng.choice([1, 2, 5, 8])
    inner = H * hd
    C = rng.choice([inner, 320, 200, 640])                   # channels of X (in-features of Wq, out-features of Wo)
    B = rng.choice([1, 2])
    L = rng.choice([1, 50, 77, 255, 256, 300, 520])
    cross = rng.random() < 0.5
    Lk = rng.choice([1, 17, 77, 128, 300]) if cross else L
    Cc = rng.choice([768, 96, C]) if cross else C
    causal = (not cross) and rng.random() < 0.3
    biases = rng.random() < 0.5
    cached = cross and rng.random() < 0.5
    x = randn(9200 + seed, (B, L, C), dtype)
    ctx = randn(9300 + seed, (B, Lk, Cc), dtype) if cross else None
    w = {"wq": randn(9400 + seed, (inner, C), dtype) / math.sqrt(C), "wk": randn(9500 + seed, (inner, Cc), dtype) / math.sqrt(Cc),
         "wv": randn(9600 + seed, (inner, Cc), dtype) / math.sqrt(Cc), "wo": randn(9700 + seed, (C, inner), dtype) / math.sqrt(inner)}
    w = {k: oracle.round_to(v, dtype) for k, v in w.items()}
    for i, (k, n) in enumerate((("bq", inner), ("bk", inner), ("bv", inner), ("bo", C))):
        w[k] = oracle.round_to(randn(9800 + 4 * seed + i, (n,), dtype), dtype) if biases else None
    d = {k: (to_dev(v, dtype) if v is not None else None) for k, v in w.items()}
    mask = None
    if rng.random() < 0.35:
        mask = (np.random.default_rng(9900 + seed).random((B, Lk)) < 0.7).astype(np.float32)
        mask[:, 0] = 1.0
    dmask = torch.from_numpy(mask).cuda() if mask is not None else None
    dx = to_dev(x, dtype)
    dctx = to_dev(ctx, dtype) if cross else None
    what = f"seed {seed}: {dtype} B={B} L={L} Lk={Lk} C={C} Cc={Cc} H={H} d={hd} cross={cross} cached={cached} causal={causal}"
    print(what, flush=True)
    if cached:
        K, V = bd.flash_attention_project_kv(dctx, d["wk"], d["bk"], d["wv"], d["bv"])
        out = bd.flash_attention_q_with_kv_cached_forward(dx, K, V, d["wq"], d["bq"], d["wo"], d["bo"], dmask, H, causal)
    else:
        out = bd.flash_attention_qkvo_forward(dx, dctx, d["wq"], d["bq"], d["wk"], d["bk"], d["wv"], d["bv"], d["wo"], d["bo"],
                                              dmask, H, causal)
    assert out.shape == (B, L, C)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], ctx[b] if cross else None, w["wq"], w["bq"], w["wk"], w["bk"], w["wv"], w["bv"], w["wo"],
                                    w["bo"], H, dtype, key_mask=mask[b] if mask is not None else None, causal=causal)
        assert_close(ref, to_np(out[b]), dtype, f"{what} batch {b}")
