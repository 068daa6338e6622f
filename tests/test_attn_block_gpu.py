"""The projection GEMM and the attention-with-projections operators of the U-Net spatial transformer
(src/unet_blocks.cpp:255-327, src/unet.cpp:470-480) through the C ABI, against the CPU checker on the same
seeded inputs. Shapes are the SD1.5 levels: C = 320 / 640 / 1280 with 8 heads (head_dim 40 / 80 / 160),
4096 / 1024 / 256 tokens, text context 77 x 768. Tolerances as everywhere (helpers.TOL): bf16 rel-L2 <= 5e-3,
max-abs <= 2e-2; fp16 rel-L2 <= 1e-3, max-abs <= 5e-3 — relative to outputs of unit scale, which the weight
scaling below arranges."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, TORCH_DT, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def weight(seed, n_out, n_in, dtype):
    """N(0, 1/n_in): a projection of unit-variance rows has unit variance."""
    import oracle
    return oracle.round_to(randn(seed, (n_out, n_in), "fp32") / np.sqrt(n_in), dtype)


# ── linear layer ─────────────────────────────────────────────────────────────
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("M,N,K,bias", [
    (1, 8, 8, False), (77, 320, 768, True), (300, 72, 1000, True), (4096, 320, 320, False),
    (257, 1280, 1280, True), (64, 64, 64, True), (129, 136, 200, False), (8192, 640, 320, True)])
def test_linear_matches_checker(oracle, dtype, M, N, K, bias):
    x = randn(11 + M, (M, K), dtype)
    w = weight(12 + N, N, K, dtype)
    b = randn(13 + K, (N,), dtype) if bias else None
    y = bd.linear_batched(to_dev(w, dtype), None if b is None else to_dev(b, dtype), to_dev(x, dtype))
    assert y.shape == (M, N)
    m = assert_close(oracle.linear(x, w, b), to_np(y), dtype, f"linear {M}x{N}x{K}")
    # FP32 accumulation and one rounding: within one unit in the last place of the result's magnitude
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    ref = oracle.linear(x, w, b)
    assert np.all(np.abs(to_np(y) - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.01 + 1e-6), m


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_linear_exact_on_small_integers(oracle, dtype):
    """Inputs in {-1, 0, 1} and K = 128: every partial sum is an integer below 2^8, exact in FP32 and in both
    storage types, so the result must equal the checker bit for bit — any misplaced row, column or
    contraction chunk shows."""
    rng = np.random.default_rng(1)
    M, N, K = 203, 152, 128
    x = rng.integers(-1, 2, (M, K)).astype(np.float32)
    w = rng.integers(-1, 2, (N, K)).astype(np.float32)
    b = rng.integers(-3, 4, N).astype(np.float32)
    y = bd.linear_batched(to_dev(w, dtype), to_dev(b, dtype), to_dev(x, dtype))
    assert np.array_equal(to_np(y), oracle.linear(x, w, b))
    assert np.array_equal(to_np(y), x @ w.T + b)


def test_linear_against_torch_fp32():
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(1000, 768, device="cuda", generator=g).bfloat16()
    w = (torch.randn(320, 768, device="cuda", generator=g) / 768 ** 0.5).bfloat16()
    b = torch.randn(320, device="cuda", generator=g).bfloat16()
    ref = torch.nn.functional.linear(x.float(), w.float(), b.float())
    y = bd.linear_batched(w, b, x)
    assert (y.float() - ref).abs().max().item() <= 2.0 ** -8 * max(1.0, ref.abs().max().item())
    # 3-D activations are rows of one matrix
    y3 = bd.linear_batched(w, b, x.view(4, 250, 768))
    assert y3.shape == (4, 250, 320) and torch.equal(y3.view(1000, 320), y)
    # writes only its own rows and columns
    big = torch.full((1002, 320), 7.0, device="cuda", dtype=torch.bfloat16)
    bd.linear_batched(w, b, x, big[1:1001])
    assert torch.equal(big[1:1001], y) and (big[0] == 7).all() and (big[1001] == 7).all()


def test_linear_argument_errors():
    x = torch.zeros(4, 20, device="cuda", dtype=torch.bfloat16)
    w = torch.zeros(8, 20, device="cuda", dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="multiples of 8"):
        bd.linear_batched(w, None, x)
    with pytest.raises(RuntimeError, match="columns"):
        bd.linear_batched(torch.zeros(8, 24, device="cuda", dtype=torch.bfloat16), None, x)
    with pytest.raises(RuntimeError, match="not on the GPU"):
        bd.linear_batched(w.cpu(), None, x)
    assert bd.linear_batched(torch.zeros(8, 24, device="cuda", dtype=torch.bfloat16), None,
                             torch.zeros(0, 24, device="cuda", dtype=torch.bfloat16)).shape == (0, 8)


# ── attention with projections ───────────────────────────────────────────────
def block_weights(seed, C, Cctx, inner, dtype, biases):
    ws = {"wq": weight(seed + 1, inner, C, dtype), "wk": weight(seed + 2, inner, Cctx, dtype),
          "wv": weight(seed + 3, inner, Cctx, dtype), "wo": weight(seed + 4, C, inner, dtype)}
    for i, (nm, n) in enumerate((("bq", inner), ("bk", inner), ("bv", inner), ("bo", C))):
        ws[nm] = randn(seed + 10 + i, (n,), dtype) * 0.25 if (biases or nm == "bo") else None
        if ws[nm] is not None:
            import oracle
            ws[nm] = oracle.round_to(ws[nm], dtype)
    return ws


def dev(ws, dtype):
    return {k: (None if v is None else to_dev(v, dtype)) for k, v in ws.items()}


@pytest.mark.parametrize("dtype,B,L,C,H,biases", [
    ("fp16", 2, 4096, 320, 8, False),   # SD1.5 level 0 (the reference passes no Q/K/V bias, src/unet_blocks.cpp:264-272)
    ("fp16", 1, 1024, 640, 8, False),
    ("bf16", 1, 256, 1280, 8, True),
    ("bf16", 1, 100, 144, 2, True),     # head_dim 72, ragged length
])
def test_qkvo_self_attention(oracle, dtype, B, L, C, H, biases):
    x = randn(7000 + L, (B, L, C), dtype)
    ws = block_weights(7100 + C, C, C, C, dtype, biases)
    d = dev(ws, dtype)
    out = bd.flash_attention_qkvo_forward(to_dev(x, dtype), None, d["wq"], d["bq"], d["wk"], d["bk"], d["wv"], d["bv"],
                                          d["wo"], d["bo"], None, H, False)
    assert out.shape == (B, L, C)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], None, ws["wq"], ws["bq"], ws["wk"], ws["bk"], ws["wv"], ws["bv"],
                                    ws["wo"], ws["bo"], H, dtype)
        print("qkvo self", dtype, L, C, assert_close(ref, to_np(out[b]), dtype, f"qkvo self batch {b}"))
    # the same block from its parts: three linear calls, attention, one linear call — identical kernels, identical bits
    dx = to_dev(x, dtype)
    q = bd.linear_batched(d["wq"], d["bq"], dx)
    k = bd.linear_batched(d["wk"], d["bk"], dx)
    v = bd.linear_batched(d["wv"], d["bv"], dx)
    parts = bd.linear_batched(d["wo"], d["bo"], bd.flash_attention_forward(q, k, v, None, H, False))
    assert torch.equal(parts, out)


@pytest.mark.parametrize("dtype,L,C,H,with_mask", [("fp16", 1024, 1152, 16, False), ("bf16", 300, 144, 2, True)])
def test_mha_forward(oracle, dtype, L, C, H, with_mask):
    """bt::mha_forward as PixArt's self attention calls it (src/dit/pixart.cpp:325-328: 16 heads of 72, biases on all
    four projections): every intermediate against the checker, and the whole against flash_attention_qkvo_forward."""
    x = randn(7300 + L, (L, C), dtype)
    ws = block_weights(7400 + C, C, C, C, dtype, True)
    d = dev(ws, dtype)
    mask = None
    if with_mask:
        mask = np.ones(L, np.float32)
        mask[L - 11:] = 0
        mask[2] = 0
    dmask = None if mask is None else torch.from_numpy(mask).cuda()
    out, qh, kh, vh, yc = bd.mha_forward(to_dev(x, dtype), d["wq"], d["wk"], d["wv"], d["wo"], d["bq"], d["bk"], d["bv"], d["bo"],
                                         dmask, H)
    q = oracle.round_to(oracle.linear(x, ws["wq"], ws["bq"]), dtype)
    k = oracle.round_to(oracle.linear(x, ws["wk"], ws["bk"]), dtype)
    v = oracle.round_to(oracle.linear(x, ws["wv"], ws["bv"]), dtype)
    assert_close(q, to_np(qh), dtype, "mha qh")
    assert_close(k, to_np(kh), dtype, "mha kh")
    assert_close(v, to_np(vh), dtype, "mha vh")
    a = oracle.round_to(oracle.sdpa(q, k, v, H, key_mask=mask), dtype)
    assert_close(a, to_np(yc), dtype, "mha yc")
    print("mha_forward", dtype, L, C, assert_close(oracle.linear(a, ws["wo"], ws["bo"]), to_np(out), dtype, "mha out"))
    fused = bd.flash_attention_qkvo_forward(to_dev(x, dtype), None, d["wq"], d["bq"], d["wk"], d["bk"], d["wv"], d["bv"],
                                            d["wo"], d["bo"], dmask, H, False)
    assert torch.equal(fused, out)
    # caller-owned intermediates are written in place
    own = [torch.empty(L, C, dtype=TORCH_DT[dtype], device="cuda") for _ in range(5)]
    res = bd.mha_forward(to_dev(x, dtype), d["wq"], d["wk"], d["wv"], d["wo"], d["bq"], d["bk"], d["bv"], d["bo"], dmask, H,
                         qh=own[0], kh=own[1], vh=own[2], yc=own[3], out=own[4])
    assert res[0].data_ptr() == own[4].data_ptr() and torch.equal(own[4], out) and torch.equal(own[3], yc)
    with pytest.raises(RuntimeError, match="num_heads must divide"):
        bd.mha_forward(to_dev(x, dtype), d["wq"], d["wk"], d["wv"], d["wo"], None, None, None, None, None, 7)


@pytest.mark.parametrize("dtype,B,L,C,H", [("fp16", 2, 4096, 320, 8), ("bf16", 1, 1024, 640, 8), ("fp16", 1, 64, 1280, 8)])
def test_qkvo_cross_attention_and_kv_cache(oracle, dtype, B, L, C, H):
    Lc, Cc = 77, 768
    x = randn(7200 + L, (B, L, C), dtype)
    ctx = randn(7300 + L, (B, Lc, Cc), dtype)
    ws = block_weights(7400 + C, C, Cc, C, dtype, False)
    d = dev(ws, dtype)
    dx, dctx = to_dev(x, dtype), to_dev(ctx, dtype)
    out = bd.flash_attention_qkvo_forward(dx, dctx, d["wq"], None, d["wk"], None, d["wv"], None, d["wo"], d["bo"], None, H, False)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], ctx[b], ws["wq"], None, ws["wk"], None, ws["wv"], None, ws["wo"], ws["bo"], H, dtype)
        print("qkvo cross", dtype, L, C, assert_close(ref, to_np(out[b]), dtype, f"qkvo cross batch {b}"))
    # K/V projected once (src/unet.cpp:476-480), then the cached form every step (src/unet_blocks.cpp:311-317)
    K, V = bd.flash_attention_project_kv(dctx, d["wk"], None, d["wv"], None)
    assert K.shape == (B, Lc, C)
    for b in range(B):
        assert_close(oracle.round_to(oracle.linear(ctx[b], ws["wk"]), dtype), to_np(K[b]), dtype, "project_kv K")
        assert_close(oracle.round_to(oracle.linear(ctx[b], ws["wv"]), dtype), to_np(V[b]), dtype, "project_kv V")
    cached = bd.flash_attention_q_with_kv_cached_forward(dx, K, V, d["wq"], None, d["wo"], d["bo"], None, H, False)
    assert torch.equal(cached, out)
    # a lent scratch gives the same result and is enough at exactly the advertised size
    n = bd.flash_attention_scratch_bytes(B, L, Lc, C, True)
    scratch = torch.empty(n, dtype=torch.uint8, device="cuda")
    again = bd.flash_attention_qkvo_forward(dx, dctx, d["wq"], None, d["wk"], None, d["wv"], None, d["wo"], d["bo"], None, H, False,
                                            scratch=scratch)
    assert torch.equal(again, out)
    with pytest.raises(RuntimeError, match="scratch of"):
        bd.flash_attention_qkvo_forward(dx, dctx, d["wq"], None, d["wk"], None, d["wv"], None, d["wo"], d["bo"], None, H, False,
                                        scratch=scratch[:n - 256])


@pytest.mark.parametrize("causal", [False, True])
def test_qkvo_key_mask_and_causal(oracle, causal):
    dtype, B, L, Lc, C, Cc, H = "bf16", 2, 200, 48, 320, 96, 8
    x, ctx = randn(7501, (B, L, C), dtype), randn(7502, (B, Lc, Cc), dtype)
    ws = block_weights(7510, C, Cc, C, dtype, True)
    d = dev(ws, dtype)
    mask = np.ones((B, Lc), np.float32)
    mask[0, 30:] = 0
    mask[1, ::3] = 0
    dmask = torch.from_numpy(mask).cuda()
    out = bd.flash_attention_qkvo_forward(to_dev(x, dtype), to_dev(ctx, dtype), d["wq"], d["bq"], d["wk"], d["bk"], d["wv"], d["bv"],
                                          d["wo"], d["bo"], dmask, H, causal)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], ctx[b], ws["wq"], ws["bq"], ws["wk"], ws["bk"], ws["wv"], ws["bv"], ws["wo"], ws["bo"],
                                    H, dtype, key_mask=mask[b], causal=causal)
        assert_close(ref, to_np(out[b]), dtype, f"qkvo masked causal={causal} batch {b}")
    if causal:
        # with kv_len < q_len the first q_len - kv_len rows see no key: attention output 0, so out = bo
        rows = to_np(out[0, : L - Lc])
        assert np.array_equal(rows, np.broadcast_to(to_np(d["bo"]), rows.shape))


def test_attn_block_argument_errors():
    dt = torch.bfloat16
    z = lambda *s: torch.zeros(*s, device="cuda", dtype=dt)
    x, w = z(16, 64), z(64, 64)
    with pytest.raises(RuntimeError, match="no attention kernel"):
        bd.flash_attention_qkvo_forward(x, None, w, None, w, None, w, None, w, None, None, 8, False)   # head_dim 8
    with pytest.raises(RuntimeError, match="does not divide"):
        bd.flash_attention_qkvo_forward(x, None, w, None, w, None, w, None, w, None, None, 3, False)
    with pytest.raises(RuntimeError, match="Wk has"):
        bd.flash_attention_qkvo_forward(x, z(5, 32), w, None, w, None, w, None, w, None, None, 1, False)
    with pytest.raises(RuntimeError, match="K / V"):
        bd.flash_attention_q_with_kv_cached_forward(x, z(5, 32), z(5, 32), w, None, w, None, None, 1, False)
    # empty query set is a no-op with an empty result
    assert bd.flash_attention_qkvo_forward(z(0, 64), None, w, None, w, None, w, None, w, None, None, 1, False).shape == (0, 64)


# ── INT8 weights with per-output-row scales (W8A16) ──────────────────────────
def quantised(seed, n_out, n_in, pow2=False):
    rng = np.random.default_rng(seed)
    q = rng.integers(-127, 128, (n_out, n_in)).astype(np.int8)
    if pow2:
        scales = np.full(n_out, 2.0 ** -8, np.float32) * (2.0 ** rng.integers(-1, 2, n_out)).astype(np.float32)
    else:
        scales = (rng.uniform(0.5, 1.5, n_out) / (73.0 * np.sqrt(n_in))).astype(np.float32)     # rows of unit-variance weights
    return q, scales, q.astype(np.float32) * scales[:, None]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("M,N,K", [(77, 320, 768), (8192, 320, 320), (300, 72, 1000), (257, 1280, 1280)])
def test_linear_int8w_matches_checker(oracle, dtype, M, N, K):
    x = randn(31 + M, (M, K), dtype)
    q, scales, w = quantised(32 + N, N, K)
    b = randn(33 + K, (N,), dtype)
    dq, ds = torch.from_numpy(q).cuda(), torch.from_numpy(scales).cuda()
    y = bd.linear_forward_batched_int8w_fp16(dq, ds, to_dev(b, dtype), to_dev(x, dtype))
    ref = oracle.linear(x, w, b)                                             # the dequantised weight in FP32
    assert_close(ref, to_np(y), dtype, f"int8w linear {M}x{N}x{K}")
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.all(np.abs(to_np(y) - ref) <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)
    with pytest.raises(RuntimeError, match="scales must hold"):
        bd.linear_forward_batched_int8w_fp16(dq, ds[:-1], None, to_dev(x, dtype))
    with pytest.raises(RuntimeError, match="dtype"):
        bd.linear_forward_batched_int8w_fp16(dq.to(torch.int16), ds, None, to_dev(x, dtype))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_int8w_equals_16bit_weights_when_exactly_representable(dtype):
    """Power-of-two scales: the dequantised weight is exact in fp16 / bf16 and scaling the accumulator by a power of
    two is exact, so the W8A16 path and the 16-bit path must give the same bits."""
    M, N, K = 1000, 320, 768
    q, scales, w = quantised(41, N, K, pow2=True)
    x = to_dev(randn(42, (M, K), dtype), dtype)
    b = to_dev(randn(43, (N,), dtype), dtype)
    dq, ds = torch.from_numpy(q).cuda(), torch.from_numpy(scales).cuda()
    assert torch.equal(bd.linear_forward_batched_int8w_fp16(dq, ds, None, x), bd.linear_batched(to_dev(w, dtype), None, x))
    # with a bias the two epilogues (fused multiply-add, then conversion / add and conversion in one mixed-precision
    # instruction) may round a value that sits on a tie differently: at most one unit in the last place, rarely
    y8, y16 = bd.linear_forward_batched_int8w_fp16(dq, ds, b, x), bd.linear_batched(to_dev(w, dtype), b, x)
    unit = 2.0 ** -7 if dtype == "bf16" else 2.0 ** -10
    diff = (y8.float() - y16.float()).abs()
    assert (diff <= unit * y16.float().abs().clamp(min=1.0)).all() and (diff > 0).float().mean().item() < 1e-3


def test_qkvo_int8w_block_and_kv_cache(oracle):
    dtype, B, L, C, H, Lc, Cc = "fp16", 2, 1024, 320, 8, 77, 768
    x, ctx = randn(7601, (B, L, C), dtype), randn(7602, (B, Lc, Cc), dtype)
    (qq, sq, wq), (qk, sk, wk), (qv, sv, wv), (qo, so, wo) = (quantised(7610 + i, C, cin) for i, cin in enumerate((C, Cc, Cc, C)))
    bo = randn(7620, (C,), dtype) * 0.25
    bo = oracle.round_to(bo, dtype)
    g = lambda a: torch.from_numpy(a).cuda()
    dx, dctx, dbo = to_dev(x, dtype), to_dev(ctx, dtype), to_dev(bo, dtype)
    out = bd.flash_attention_qkvo_int8w_fp16(dx, dctx, g(qq), g(sq), None, g(qk), g(sk), None, g(qv), g(sv), None, g(qo), g(so), dbo,
                                             None, H, False)
    for b in range(B):
        ref = oracle.attention_qkvo(x[b], ctx[b], wq, None, wk, None, wv, None, wo, bo, H, dtype)
        print("int8w qkvo", assert_close(ref, to_np(out[b]), dtype, f"int8w qkvo batch {b}"))
    K, V = bd.flash_attention_project_kv_int8w_fp16(dctx, g(qk), g(sk), None, g(qv), g(sv), None)
    cached = bd.flash_attention_q_with_kv_cached_int8w_fp16(dx, K, V, g(qq), g(sq), None, g(qo), g(so), dbo, None, H, False)
    assert torch.equal(cached, out)
    # self-attention form: Q, K, V all from X in one INT8 launch
    (_, _, wk1), (_, _, wv1) = quantised(7630, C, C), quantised(7631, C, C)
    qk1, sk1, _ = quantised(7630, C, C)
    qv1, sv1, _ = quantised(7631, C, C)
    out_self = bd.flash_attention_qkvo_int8w_fp16(dx, None, g(qq), g(sq), None, g(qk1), g(sk1), None, g(qv1), g(sv1), None,
                                                  g(qo), g(so), dbo, None, H, False)
    ref = oracle.attention_qkvo(x[0], None, wq, None, wk1, None, wv1, None, wo, bo, H, dtype)
    assert_close(ref, to_np(out_self[0]), dtype, "int8w qkvo self")
    # mixing an INT8 Q weight with 16-bit K / V weights in the one projection launch is refused
    with pytest.raises(RuntimeError, match="cannot share a launch"):
        bd.ops._attn_block("flash_attention_qkvo_int8w_fp16", "mi_flash_attention_qkvo_forward", dx, None, None, None,
                           g(qq), None, to_dev(wk1, dtype), None, to_dev(wv1, dtype), None, g(qo), dbo, None, H, False, None, None,
                           scales=(g(sq), None, None, g(so)))
