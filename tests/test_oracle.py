"""Pins the CPU checker (oracle/) before anything is compared against it.

Each test fixes one function of oracle.cpp by something that does not retype its
formula: the reference's known-answer vectors, the reference header compiled as is,
a general library routine (torch float64), a numpy brute force written from the
mathematical definition, or a closed form / invariant.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


# ── seeded generator ────────────────────────────────────────────────────────
def test_randn_known_answer_vectors(oracle):
    kat = json.load(open(os.path.join(HERE, "golden", "torch_randn_kat.json")))
    assert len(kat["cases"]) == 4
    for case in kat["cases"]:
        ref = np.array(case["values"], dtype=np.float64)
        got = oracle.torch_randn_f32(case["seed"], len(ref))
        assert np.max(np.abs(got - ref)) < 1e-4  # the reference's own bound


def test_randn_refuses_short(oracle):
    with pytest.raises(ValueError):
        oracle.torch_randn_f32(0, 15)


def test_randn_matches_torch_library():
    # torch's own CPU generator is what the reference header claims to reproduce.
    import oracle
    for seed, n in [(3, 64), (2001, 1000), (99, 16)]:
        g = torch.Generator().manual_seed(seed)
        ref = torch.randn(n, generator=g, dtype=torch.float32).numpy()
        got = oracle.torch_randn_f32(seed, n)
        assert np.max(np.abs(got - ref)) < 1e-4


def test_randn_bit_equal_to_reference_header(oracle):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built (reference tree not mounted)")
    for seed, n in [(0, 16), (0, 20), (7, 32), (1001, 4099), (2 ** 33 + 5, 257), (3003, 100000)]:
        a = oracle.torch_randn_f32(seed, n)
        b = oracle.ref_torch_randn_f32(seed, n)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


# ── dtype rounding ──────────────────────────────────────────────────────────
@pytest.mark.parametrize("dtype,tdt", [("bf16", torch.bfloat16), ("fp16", torch.float16)])
def test_rounding_matches_torch_cast(oracle, dtype, tdt):
    rng = np.random.default_rng(5)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e-6).astype(np.float32),   # fp16 subnormals
        (rng.standard_normal(5000) * 3e4).astype(np.float32),    # near fp16 max
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
                  1.00390625, 1.01171875, np.inf, -np.inf], dtype=np.float32),
    ])
    ref = torch.from_numpy(x).to(tdt).to(torch.float32).numpy()
    got = oracle.round_to(x, dtype)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    bits = oracle.to_bits(x, dtype)
    ref_bits = torch.from_numpy(x).to(tdt).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(bits, ref_bits)
    assert np.array_equal(oracle.from_bits(bits, dtype).view(np.uint32), ref.view(np.uint32))


# ── RoPE tables ─────────────────────────────────────────────────────────────
def test_axial_tables_closed_form(oracle):
    txt, hp, wp, hd, axes, theta = 5, 4, 6, 32, (8, 12, 12), 10000.0
    cos, sin = oracle.build_axial_rope_tables(txt, hp, wp, hd, axes, theta)
    assert cos.shape == (txt + hp * wp, hd // 2)
    assert np.all(cos[:txt] == 1.0) and np.all(sin[:txt] == 0.0)          # text rows: identity
    # axis 0 has position 0 for every image token -> identity on its pairs
    assert np.all(cos[:, :4] == 1.0) and np.all(sin[:, :4] == 0.0)
    for (i, j) in [(0, 0), (1, 0), (3, 5), (2, 4)]:
        row = txt + i * wp + j
        for p in range(6):
            w = theta ** (-2.0 * p / 12.0)
            assert cos[row, 4 + p] == np.float32(math.cos(i * w))
            assert sin[row, 4 + p] == np.float32(math.sin(i * w))
            assert cos[row, 10 + p] == np.float32(math.cos(j * w))
            assert sin[row, 10 + p] == np.float32(math.sin(j * w))
    with pytest.raises(ValueError):
        oracle.build_axial_rope_tables(1, 2, 2, 32, (8, 8, 8))


def test_qwen_tables_positions(oracle):
    # text(3) -> positions 0,1,2 on all axes; image 2x4 -> frame 3, rows -1..0, cols -2..1, then pos = 3 + 4;
    # text(2) -> 7, 8; target 2x2 -> frame 9, rows -1..0, cols -1..0.
    segs = [("text", 3), ("image", 2, 4), ("text", 2)]
    hd, axes, theta = 16, (4, 6, 6), 10000.0
    cos, sin = oracle.build_qwen_rope_tables(segs, 2, 2, hd, axes, theta)
    assert cos.shape == (3 + 8 + 2 + 4, 8)
    f = [0, 1, 2] + [3] * 8 + [7, 8] + [9] * 4
    h = [0, 1, 2] + [-1] * 4 + [0] * 4 + [7, 8] + [-1, -1, 0, 0]
    w = [0, 1, 2] + [-2, -1, 0, 1] * 2 + [7, 8] + [-1, 0, -1, 0]
    for r in range(cos.shape[0]):
        exp_ang = ([f[r] * theta ** (-2.0 * p / 4) for p in range(2)] +
                   [h[r] * theta ** (-2.0 * p / 6) for p in range(3)] +
                   [w[r] * theta ** (-2.0 * p / 6) for p in range(3)])
        assert np.allclose(cos[r], np.cos(exp_ang), atol=1e-7)
        assert np.allclose(sin[r], np.sin(exp_ang), atol=1e-7)


# ── RoPE apply ──────────────────────────────────────────────────────────────
@pytest.mark.parametrize("split_half", [False, True])
def test_rope_apply_invariants(oracle, split_half):
    rng = np.random.default_rng(1)
    L, H, d = 7, 3, 8
    x = rng.standard_normal((L, H * d)).astype(np.float32)
    ang = rng.uniform(-3, 3, (L, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    y = oracle.rope_apply(x, cos, sin, H, d, split_half=split_half)
    xv, yv = x.reshape(L, H, d), y.reshape(L, H, d)
    pairs = [(p, p + d // 2) for p in range(d // 2)] if split_half else [(2 * p, 2 * p + 1) for p in range(d // 2)]
    for p, (i0, i1) in enumerate(pairs):
        # complex multiplication by e^{i ang}
        zin = xv[:, :, i0].astype(np.float64) + 1j * xv[:, :, i1]
        zout = zin * np.exp(1j * ang[:, p])[:, None]
        assert np.allclose(yv[:, :, i0], zout.real, atol=1e-6)
        assert np.allclose(yv[:, :, i1], zout.imag, atol=1e-6)
    # identity tables leave x untouched
    ident = oracle.rope_apply(x, np.ones_like(cos), np.zeros_like(sin), H, d, split_half=split_half)
    assert np.array_equal(ident, x)


def test_rope_relative_position_property(oracle):
    # <R(a) q, R(b) k> depends on a - b only (1-axis table built by the axial builder: hp=1).
    rng = np.random.default_rng(2)
    d = 16
    cos, sin = oracle.build_axial_rope_tables(0, 1, 12, d, (0, 0, d))
    q = np.tile(rng.standard_normal((1, d)).astype(np.float32), (12, 1))
    k = np.tile(rng.standard_normal((1, d)).astype(np.float32), (12, 1))
    qr = oracle.rope_apply(q, cos, sin, 1, d).astype(np.float64)
    kr = oracle.rope_apply(k, cos, sin, 1, d).astype(np.float64)
    G = qr @ kr.T
    for delta in range(-5, 6):
        diag = np.diagonal(G, offset=delta)
        assert np.max(np.abs(diag - diag[0])) < 1e-4


def test_rope_rounding_modes(oracle):
    rng = np.random.default_rng(3)
    x = oracle.round_to(rng.standard_normal((4, 16)), "bf16")
    ang = rng.uniform(-3, 3, (4, 4))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    y = oracle.rope_apply(x, cos, sin, 2, 8)
    yb = oracle.rope_apply(x, cos, sin, 2, 8, round_to_dtype="bf16")
    assert np.array_equal(yb, oracle.round_to(y, "bf16"))


# ── softmax attention ───────────────────────────────────────────────────────
def _brute_sdpa(q, k, v, H, scale=None, vis=None):
    """Definition, float64 numpy: out_i = sum_j softmax_j(q_i.k_j*scale) v_j over visible j."""
    Lq, D = q.shape
    Lk = k.shape[0]
    d = D // H
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    out = np.zeros((Lq, D))
    for h in range(H):
        sl = slice(h * d, (h + 1) * d)
        s = q[:, sl].astype(np.float64) @ k[:, sl].astype(np.float64).T * scale
        if vis is not None:
            s = np.where(vis, s, -np.inf)
        m = np.max(s, axis=1, keepdims=True)
        m = np.where(np.isfinite(m), m, 0.0)
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True)
        p = np.divide(e, den, out=np.zeros_like(e), where=den > 0)
        out[:, sl] = p @ v[:, sl].astype(np.float64)
    return out


@pytest.mark.parametrize("Lq,Lk,H,d", [(9, 9, 2, 8), (5, 13, 3, 40), (33, 17, 1, 72)])
def test_sdpa_vs_torch_float64(oracle, Lq, Lk, H, d):
    rng = np.random.default_rng(Lq * 100 + Lk)
    q = rng.standard_normal((Lq, H * d)).astype(np.float32)
    k = rng.standard_normal((Lk, H * d)).astype(np.float32)
    v = rng.standard_normal((Lk, H * d)).astype(np.float32)
    got = oracle.sdpa(q, k, v, H)
    tq = torch.from_numpy(q).double().view(Lq, H, d).transpose(0, 1)
    tk = torch.from_numpy(k).double().view(Lk, H, d).transpose(0, 1)
    tv = torch.from_numpy(v).double().view(Lk, H, d).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv).transpose(0, 1).reshape(Lq, H * d).numpy()
    assert np.max(np.abs(got - ref)) < 2e-6
    assert np.max(np.abs(got - _brute_sdpa(q, k, v, H))) < 2e-6


def test_sdpa_closed_forms(oracle):
    rng = np.random.default_rng(11)
    Lq, Lk, H, d = 6, 10, 2, 16
    q = rng.standard_normal((Lq, H * d)).astype(np.float32)
    v = rng.standard_normal((Lk, H * d)).astype(np.float32)
    # all keys equal -> uniform softmax -> mean of V
    k = np.tile(rng.standard_normal((1, H * d)).astype(np.float32), (Lk, 1))
    out = oracle.sdpa(q, k, v, H)
    assert np.allclose(out, np.tile(v.mean(axis=0), (Lq, 1)), atol=1e-6)
    # V constant -> output equals that constant row
    k = rng.standard_normal((Lk, H * d)).astype(np.float32)
    vc = np.tile(rng.standard_normal((1, H * d)).astype(np.float32), (Lk, 1))
    assert np.allclose(oracle.sdpa(q, k, vc, H), np.tile(vc[:1], (Lq, 1)), atol=1e-6)
    # one dominant key -> output tends to that key's value
    kd = k.copy(); qd = q.copy()
    kd[3] = 0; kd[3, :d] = 50.0; qd[:, :d] = 50.0
    outd = oracle.sdpa(qd, kd, v, H)
    assert np.allclose(outd[:, :d], np.tile(v[3, :d], (Lq, 1)), atol=1e-5)
    # permuting keys (and values with them) changes nothing beyond float summation order
    perm = rng.permutation(Lk)
    assert np.allclose(oracle.sdpa(q, k[perm], v[perm], H), oracle.sdpa(q, k, v, H), atol=1e-6)
    # explicit scale
    assert np.allclose(oracle.sdpa(q, k, v, H, scale=0.3), _brute_sdpa(q, k, v, H, scale=0.3), atol=2e-6)


def test_sdpa_key_mask_equals_trimming(oracle):
    # The reference's own equivalence: padded keys masked out == trimming to the valid rows
    # (src/pipeline.cpp:391-414) == compacting scattered valid rows (src/dit/krea2.cpp:504-529).
    rng = np.random.default_rng(12)
    Lq, Lk, H, d = 8, 20, 2, 24
    q = rng.standard_normal((Lq, H * d)).astype(np.float32)
    k = rng.standard_normal((Lk, H * d)).astype(np.float32)
    v = rng.standard_normal((Lk, H * d)).astype(np.float32)
    valid = 13
    mask = np.zeros(Lk, dtype=np.float32); mask[:valid] = 1
    assert np.array_equal(oracle.sdpa(q, k, v, H, key_mask=mask), oracle.sdpa(q, k[:valid], v[:valid], H))
    scat = (rng.uniform(size=Lk) > 0.4).astype(np.float32)
    idx = np.nonzero(scat)[0]
    assert np.array_equal(oracle.sdpa(q, k, v, H, key_mask=scat), oracle.sdpa(q, k[idx], v[idx], H))
    # nothing visible -> zeros (src/dit/common.cpp:293)
    assert np.all(oracle.sdpa(q, k, v, H, key_mask=np.zeros(Lk, np.float32)) == 0.0)


def test_sdpa_causal_rows(oracle):
    rng = np.random.default_rng(13)
    Lq, Lk, H, d = 6, 11, 2, 8
    q = rng.standard_normal((Lq, H * d)).astype(np.float32)
    k = rng.standard_normal((Lk, H * d)).astype(np.float32)
    v = rng.standard_normal((Lk, H * d)).astype(np.float32)
    lo, hi = oracle.rows_causal(Lq, Lk)          # q_offset = Lk - Lq: row r sees keys [0, 5 + r]
    assert list(hi) == [6, 7, 8, 9, 10, 11] and not lo.any()
    vis = np.arange(Lk)[None, :] <= (np.arange(Lq)[:, None] + Lk - Lq)
    got = oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi)
    assert np.max(np.abs(got - _brute_sdpa(q, k, v, H, vis=vis))) < 2e-6
    tq = torch.from_numpy(q).double().view(Lq, H, d).transpose(0, 1)
    tk = torch.from_numpy(k).double().view(Lk, H, d).transpose(0, 1)
    tv = torch.from_numpy(v).double().view(Lk, H, d).transpose(0, 1)
    ref = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, attn_mask=torch.from_numpy(vis))
    assert np.max(np.abs(got - ref.transpose(0, 1).reshape(Lq, H * d).numpy())) < 2e-6
    lo, hi = oracle.rows_causal(Lq, Lk, window=3)
    visw = vis & (np.arange(Lk)[None, :] > (np.arange(Lq)[:, None] + Lk - Lq - 3))
    got = oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi)
    assert np.max(np.abs(got - _brute_sdpa(q, k, v, H, vis=visw))) < 2e-6


def test_sdpa_block_causal_three_ways(oracle):
    """Fused block-causal call == the reference's per-segment decomposition
    (src/dit/qwenimage21_forward.cpp:650-676) == dense mask from the visibility rule
    (include/brodiffusion/dit/qwenimage21.h:31-33); cached form == prefill target rows."""
    rng = np.random.default_rng(14)
    H, d = 2, 16
    # joint sequence: text 5, image block 0 (6 tokens), text 3, target image block 1 (8 tokens)
    kinds = [("t", 5), ("i", 6), ("t", 3), ("i", 8)]
    L = sum(n for _, n in kinds)
    block_id, seg_q_end, seg_k_end, seg_causal = [], [], [], []
    pos, img = 0, 0
    for kind, n in kinds:
        pos += n
        seg_q_end.append(pos); seg_k_end.append(pos); seg_causal.append(1 if kind == "t" else 0)
        block_id += ([-1] * n) if kind == "t" else ([img] * n)
        img += kind == "i"
    q = rng.standard_normal((L, H * d)).astype(np.float32)
    k = rng.standard_normal((L, H * d)).astype(np.float32)
    v = rng.standard_normal((L, H * d)).astype(np.float32)
    lo, hi = oracle.rows_block_causal(L, L, 0, seg_q_end, seg_k_end, seg_causal)
    fused = oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi)
    dense = oracle.dense_block_causal(L, L, 0, block_id)
    assert np.array_equal(fused, oracle.sdpa(q, k, v, H, dense_mask=dense))
    assert np.max(np.abs(fused - _brute_sdpa(q, k, v, H, vis=dense.astype(bool)))) < 2e-6
    # per-segment calls
    start = 0
    for (kind, n), e in zip(kinds, seg_q_end):
        if kind == "t":
            l2, h2 = oracle.rows_causal(n, e)     # q_offset = Lk - Lq = start
            seg = oracle.sdpa(q[start:e], k[:e], v[:e], H, row_lo=l2, row_hi=h2)
        else:
            seg = oracle.sdpa(q[start:e], k[:e], v[:e], H)
        assert np.array_equal(seg, fused[start:e])
        start = e
    # cached form: target rows only, all keys, unmasked
    t0 = L - 8
    assert np.array_equal(oracle.sdpa(q[t0:], k, v, H), fused[t0:])
    # rows= sampling computes only the listed rows
    rows = np.array([0, 7, 21], dtype=np.int32)
    part = oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi, rows=rows)
    assert np.array_equal(part[rows], fused[rows])
    assert not part[np.setdiff1d(np.arange(L), rows)].any()


def test_sdpa_bias_and_attn_avg(oracle):
    rng = np.random.default_rng(15)
    L, H, d, txt = 9, 2, 8, 4
    q = rng.standard_normal((L, H * d)).astype(np.float32)
    k = rng.standard_normal((L, H * d)).astype(np.float32)
    v = rng.standard_normal((L, H * d)).astype(np.float32)
    bias = rng.standard_normal((L - txt, txt)).astype(np.float32)
    out, avg = oracle.sdpa(q, k, v, H, bias=bias, bias_q0=txt, return_attn_avg=True)
    assert np.allclose(avg.sum(axis=1), 1.0, atol=1e-6)       # rows of a softmax sum to 1
    acc = np.zeros((L, L)); ref = np.zeros((L, H * d))
    for h in range(H):
        sl = slice(h * d, (h + 1) * d)
        s = q[:, sl].astype(np.float64) @ k[:, sl].astype(np.float64).T / math.sqrt(d)
        s[txt:, :txt] += bias
        p = np.exp(s - s.max(1, keepdims=True)); p /= p.sum(1, keepdims=True)
        acc += p; ref[:, sl] = p @ v[:, sl]
    assert np.max(np.abs(avg - acc / H)) < 1e-6
    assert np.max(np.abs(out - ref)) < 2e-6


# ── linear attention ────────────────────────────────────────────────────────
@pytest.mark.parametrize("N,H,d", [(37, 2, 32), (64, 3, 112), (20, 1, 8)])
def test_linear_attention_quadratic_form(oracle, N, H, d):
    rng = np.random.default_rng(N)
    q = rng.standard_normal((N, H * d)).astype(np.float32)
    k = rng.standard_normal((N, H * d)).astype(np.float32)
    v = rng.standard_normal((N, H * d)).astype(np.float32)
    got = oracle.linear_attn_relu(q, k, v, H)
    ref = np.zeros((N, H * d))
    for h in range(H):
        sl = slice(h * d, (h + 1) * d)
        a = np.maximum(q[:, sl], 0).astype(np.float64) @ np.maximum(k[:, sl], 0).astype(np.float64).T  # (N, N)
        ref[:, sl] = (a @ v[:, sl].astype(np.float64)) / (a.sum(axis=1, keepdims=True) + 1e-15)
    scale = np.max(np.abs(ref))
    assert np.max(np.abs(got - ref)) < 2e-5 * scale


def test_linear_attention_state_additivity(oracle):
    # (S, z) of the whole sequence == sum over token chunks (the identity-seam property,
    # include/brodiffusion/dit/sana.h:102-106).
    rng = np.random.default_rng(21)
    N, H, d = 48, 2, 16
    q = rng.standard_normal((N, H * d)).astype(np.float32)
    k = rng.standard_normal((N, H * d)).astype(np.float32)
    v = rng.standard_normal((N, H * d)).astype(np.float32)
    _, S, z = oracle.linear_attn_relu(q, k, v, H, return_state=True)
    _, S1, z1 = oracle.linear_attn_relu(q[:20], k[:20], v[:20], H, return_state=True)
    _, S2, z2 = oracle.linear_attn_relu(q[20:], k[20:], v[20:], H, return_state=True)
    assert np.allclose(S, S1 + S2, atol=1e-4) and np.allclose(z, z1 + z2, atol=1e-5)
    kr = np.maximum(k[:, :d], 0)
    assert np.allclose(S[0], v[:, :d].T.astype(np.float64) @ kr, atol=1e-4)   # S = V . relu(K)^T, (d_v, d_k)
    assert np.allclose(z[0], kr.sum(axis=0), atol=1e-5)


def test_linear_attention_zero_denominator(oracle):
    # all-negative q -> relu(q) = 0 -> num = 0, den = 0 -> 0 * 1/(0 + 1e-15) = 0
    N, H, d = 16, 1, 8
    q = -np.ones((N, H * d), dtype=np.float32)
    k = np.ones((N, H * d), dtype=np.float32)
    v = np.ones((N, H * d), dtype=np.float32)
    out = oracle.linear_attn_relu(q, k, v, H)
    assert np.all(out == 0.0)


def test_compare_metrics(oracle):
    a = np.array([1.0, 2.0, 2.0]); b = np.array([1.0, 2.0, 2.5])
    m = oracle.compare(a, b)
    assert abs(m["rel_l2"] - 0.5 / 3.0) < 1e-12 and abs(m["max_abs"] - 0.5) < 1e-12


# ── linear layer and the projection composition ─────────────────────────────
@pytest.mark.parametrize("M,N,K", [(7, 5, 3), (33, 320, 768), (1, 8, 1000)])
def test_linear_vs_numpy_float64(oracle, M, N, K):
    rng = np.random.default_rng(M * 1000 + N)
    x = rng.standard_normal((M, K)).astype(np.float32)
    w = rng.standard_normal((N, K)).astype(np.float32)
    b = rng.standard_normal(N).astype(np.float32)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.allclose(oracle.linear(x, w), ref, rtol=1e-6, atol=1e-6)
    assert np.allclose(oracle.linear(x, w, b), ref + b, rtol=1e-6, atol=1e-6)


def test_linear_weight_layout_is_out_by_in(oracle):
    """Row n of W produces output feature n: a one-hot weight row copies one input column, a transposed
    reading would copy a different one (the matrix is not square and not symmetric)."""
    M, N, K = 4, 3, 5
    x = np.arange(M * K, dtype=np.float32).reshape(M, K)
    w = np.zeros((N, K), np.float32)
    w[0, 4] = 1; w[1, 0] = 2; w[2, 2] = -1
    y = oracle.linear(x, w, np.array([10, 20, 30], np.float32))
    assert np.array_equal(y, np.stack([x[:, 4] + 10, 2 * x[:, 0] + 20, -x[:, 2] + 30], axis=1))


def test_attention_qkvo_composition(oracle):
    """Identity projections reduce the block to plain attention; the kv_cached form with K, V taken from
    the projections equals the full form; fp32 vs rounded intermediates differ only by rounding."""
    rng = np.random.default_rng(5)
    L, Lc, C, H = 19, 7, 16, 2
    x = rng.standard_normal((L, C)).astype(np.float32)
    ctx = rng.standard_normal((Lc, 24)).astype(np.float32)
    eye = np.eye(C, dtype=np.float32)
    got = oracle.attention_qkvo(x, None, eye, None, eye, None, eye, None, eye, None, H, "fp32")
    assert np.allclose(got, oracle.sdpa(x, x, x, H), atol=1e-6)
    wq, wo = (rng.standard_normal((C, C)).astype(np.float32) / 4 for _ in range(2))
    wk, wv = (rng.standard_normal((C, 24)).astype(np.float32) / 5 for _ in range(2))
    bq, bk, bv, bo = (rng.standard_normal(C).astype(np.float32) for _ in range(4))
    full = oracle.attention_qkvo(x, ctx, wq, bq, wk, bk, wv, bv, wo, bo, H, "fp32")
    k, v = oracle.linear(ctx, wk, bk), oracle.linear(ctx, wv, bv)
    cached = oracle.attention_qkvo(x, None, wq, bq, None, None, None, None, wo, bo, H, "fp32", k=k, v=v)
    assert np.array_equal(full, cached)
    by_hand = oracle.linear(oracle.sdpa(oracle.linear(x, wq, bq), k, v, H), wo, bo)
    assert np.array_equal(full, by_hand)
    rounded = oracle.attention_qkvo(x, ctx, wq, bq, wk, bk, wv, bv, wo, bo, H, "bf16")
    assert 0 < np.abs(rounded - full).max() < 0.05


# ── per-head RMS normalisation ───────────────────────────────────────────────
def test_rms_norm_vs_torch_float64_and_invariants(oracle):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((37, 128)).astype(np.float32) * 3
    g = rng.standard_normal(128).astype(np.float32)
    eps = 1e-6
    ref = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (128,), torch.from_numpy(g).double(), eps).numpy()
    got = oracle.rms_norm(x, g, eps)
    assert np.allclose(got, ref, rtol=1e-6, atol=1e-7)
    # unit gain: every row leaves with RMS 1 (eps is negligible against these rows)
    unit = oracle.rms_norm(x, np.ones(128, np.float32), eps)
    assert np.allclose(np.sqrt((unit.astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=1e-5)
    # scale invariance: normalising 5x gives what normalising x gives
    assert np.allclose(oracle.rms_norm(5 * x, g, 0.0), oracle.rms_norm(x, g, 0.0), rtol=1e-6, atol=1e-7)
    # eps sits inside the square root: a zero row stays zero, a tiny row is damped by sqrt(eps)
    tiny = np.full((1, 128), 1e-4, np.float32)
    assert np.allclose(oracle.rms_norm(tiny, np.ones(128, np.float32), 1e-6), 1e-4 / np.sqrt(1e-8 + 1e-6), rtol=1e-5)
    assert np.array_equal(oracle.rms_norm(np.zeros((2, 128), np.float32), g, eps), np.zeros((2, 128), np.float32))


def test_headnorm_rope_is_norm_then_rotation(oracle):
    rng = np.random.default_rng(12)
    L, H, d = 9, 3, 32
    x = rng.standard_normal((L, H * d)).astype(np.float32)
    g = rng.standard_normal(d).astype(np.float32)
    ang = rng.uniform(0, 6.28, (L, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    got = oracle.headnorm_rope(x, g, 1e-6, cos, sin, H, d)
    by_hand = np.empty_like(x)
    for l in range(L):
        for h in range(H):
            row = x[l, h * d:(h + 1) * d].astype(np.float64)
            y = row / np.sqrt((row ** 2).mean() + 1e-6) * g
            by_hand[l, h * d:(h + 1) * d:2] = y[0::2] * cos[l] - y[1::2] * sin[l]
            by_hand[l, h * d + 1:(h + 1) * d:2] = y[0::2] * sin[l] + y[1::2] * cos[l]
    assert np.allclose(got, by_hand, rtol=1e-5, atol=1e-6)
    assert np.allclose(oracle.headnorm_rope(x, g, 1e-6, None, None, H, d), oracle.rms_norm(x.reshape(L * H, d), g, 1e-6).reshape(L, H * d))


def test_geglu_exact_vs_torch_float64(oracle):
    rng = np.random.default_rng(21)
    t = (rng.standard_normal((13, 2 * 24)) * 2).astype(np.float32)
    td = torch.from_numpy(t).double()
    ref = (td[:, :24] * torch.nn.functional.gelu(td[:, 24:], approximate="none")).numpy()
    assert np.allclose(oracle.geglu_exact(t), ref, rtol=1e-6, atol=1e-7)
    # gelu(0) = 0 and gelu(x) - gelu(-x) = x, seen through unit values
    g = np.array([[1.0, 1.0, 1.0, 0.0, 1.7, -1.7]], np.float32)
    out = oracle.geglu_exact(g)
    assert out[0, 0] == 0.0 and abs((out[0, 1] - out[0, 2]) - 1.7) < 1e-6
    # the value half is the first half: swapping the halves changes the result
    assert not np.allclose(oracle.geglu_exact(t), oracle.geglu_exact(np.concatenate([t[:, 24:], t[:, :24]], axis=1)))


def test_window_is_counted_in_positions(oracle):
    """A windowed query at position p sees keys (p - window, p] that exist: hand-worked for queries that run past the
    last key (outside what the reference calls: there q_offset = Lk - Lq and both readings coincide)."""
    lo, hi = oracle.rows_causal(5, 3, 0, 2)
    assert list(zip(lo, hi)) == [(0, 1), (0, 2), (1, 3), (2, 3), (3, 3)]
    lo, hi = oracle.rows_causal(3, 10, 7, 4)          # q_offset = Lk - Lq: the last 4 keys up to the diagonal
    assert list(zip(lo, hi)) == [(4, 8), (5, 9), (6, 10)]
