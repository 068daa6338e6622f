"""GPU parity of the softmax-attention path against the CPU checker, through the C ABI."""
import math

import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def assert_same(a: torch.Tensor, b: torch.Tensor, exact: bool, what: str = ""):
    """Two routes to the same result: bit-identical where both run the same arithmetic in the same order,
    else equal to rounding: each is within one unit in the last place of the exact value, so they differ by
    at most two (2^-7 of the magnitude in bf16, 2^-10 in fp16)."""
    if exact:
        assert torch.equal(a, b), what
    else:
        ulp2 = 2.0 ** -7 if a.dtype == torch.bfloat16 else 2.0 ** -10
        err = (a.float() - b.float()).abs().max().item()
        assert err <= ulp2 * max(1.0, b.float().abs().max().item()), f"{what}: max abs diff {err}"


@pytest.fixture(autouse=True, params=["rows128", "rows256_pingpong", "rows256_pingpong_regs"])
def kernel_choice(request):
    """Every case runs on all kernels: 4 wavefronts x 128 rows; 8 wavefronts x 256 rows (ping-pong) with
    LDS-DMA tiles where available (head_dim 128) and with register-staged tiles."""
    bd.set_sdpa_kernel_choice({"rows128": 1, "rows256_pingpong": 2, "rows256_pingpong_regs": 3}[request.param])
    yield request.param
    bd.set_sdpa_kernel_choice(0)


def _oracle_batched(oracle, q, k, v, H, **kw):
    return np.stack([oracle.sdpa(q[b], k[b], v[b], H, **kw) for b in range(q.shape[0])])


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("d", [40, 64, 72, 80, 96, 112, 128, 160])
def test_noncausal_all_head_dims(oracle, d, dtype):
    B, H, Lq, Lk = 2, 2, 200, 333          # ragged: neither a multiple of the 128 / 64 tiles
    q = randn(10 + d, (B, Lq, H * d), dtype); k = randn(20 + d, (B, Lk, H * d), dtype); v = randn(30 + d, (B, Lk, H * d), dtype)
    out = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, False)
    assert_close(_oracle_batched(oracle, q, k, v, H), to_np(out), dtype, f"d={d}")


@pytest.mark.parametrize("Lq,Lk", [(1, 1), (1, 64), (64, 1), (128, 64), (129, 65), (127, 63), (300, 17), (5, 700)])
def test_edge_lengths(oracle, Lq, Lk):
    dtype, H, d = "bf16", 3, 128
    q = randn(1, (Lq, H * d), dtype); k = randn(2, (Lk, H * d), dtype); v = randn(3, (Lk, H * d), dtype)
    out = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, False)
    assert_close(oracle.sdpa(q, k, v, H), to_np(out), dtype, f"{Lq}x{Lk}")


def test_empty_query_is_noop():
    dtype, H, d = "bf16", 2, 64
    q = torch.empty((0, H * d), dtype=torch.bfloat16, device="cuda")
    k = to_dev(randn(2, (8, H * d), dtype), dtype)
    out = bd.flash_attention_forward(q, k, k, None, H, False)
    assert out.shape == (0, H * d)


@pytest.mark.parametrize("dtype,d", [("bf16", 128), ("fp16", 40), ("bf16", 72)])
@pytest.mark.parametrize("window", [0, 50])
def test_causal_windowed(oracle, dtype, d, window):
    H, Lq, Lk = 2, 150, 290                  # q_offset = 140: the diagonal cuts tiles mid-way
    q = randn(41, (Lq, H * d), dtype); k = randn(42, (Lk, H * d), dtype); v = randn(43, (Lk, H * d), dtype)
    out = bd.flash_attention_windowed_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, window)
    lo, hi = oracle.rows_causal(Lq, Lk, window=window)
    assert_close(oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi), to_np(out), dtype, f"window={window}")
    if window == 0:
        out2 = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, True)
        assert torch.equal(out, out2)


def test_causal_rows_without_keys_are_zero(oracle):
    # q_offset = Lk - Lq < 0: the first rows see no key at all -> zeros (src/dit/common.cpp:293)
    dtype, H, d, Lq, Lk = "bf16", 2, 64, 100, 40
    q = randn(51, (Lq, H * d), dtype); k = randn(52, (Lk, H * d), dtype); v = randn(53, (Lk, H * d), dtype)
    out = to_np(bd.flash_attention_windowed_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, H, 0))
    lo, hi = oracle.rows_causal(Lq, Lk)
    assert (hi[:59] == 0).all() and hi[60] == 1
    assert not out[:60].any()
    assert_close(oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi), out, dtype)


@pytest.mark.parametrize("dtype,d", [("bf16", 72), ("fp16", 40), ("bf16", 128)])
def test_key_mask_equals_trimmed(oracle, kernel_choice, dtype, d):
    """Key padding three ways (kv_valid_len, 0/1 d_mask, trimmed K/V) must agree: the reference handles
    padding by trimming to the valid rows (src/pipeline.cpp:391-414)."""
    B, H, Lq, Lk = 2, 2, 130, 300
    valid = [77, 300]
    q = randn(61, (B, Lq, H * d), dtype); k = randn(62, (B, Lk, H * d), dtype); v = randn(63, (B, Lk, H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    vl = torch.tensor(valid, dtype=torch.int32, device="cuda")
    o_len = bd.sdpa_forward(dq, dk, dv, H, kv_valid_len=vl)
    m = np.zeros((B, Lk), dtype=np.float32)
    for b in range(B):
        m[b, :valid[b]] = 1
    o_mask = bd.flash_attention_forward(dq, dk, dv, torch.from_numpy(m).cuda(), H, False)
    for b in range(B):
        ref = oracle.sdpa(q[b], k[b, :valid[b]], v[b, :valid[b]], H)
        assert_close(ref, to_np(o_len[b]), dtype, "kv_valid_len")
        assert_close(ref, to_np(o_mask[b]), dtype, "d_mask")
        o_trim = bd.flash_attention_forward(dq[b], dk[b, :valid[b]], dv[b, :valid[b]], None, H, False)
        # (the 256-row kernels take a 0/1 mask in an instance of their own, whose softmax blanks keys bit by bit)
        assert_same(o_trim, o_len[b], True, "trimmed vs kv_valid_len")
        assert_same(o_trim, o_mask[b], kernel_choice == "rows128", "trimmed vs d_mask")


def test_scattered_key_mask_and_empty_mask(oracle):
    dtype, H, d, Lq, Lk = "bf16", 2, 128, 70, 200
    q = randn(71, (Lq, H * d), dtype); k = randn(72, (Lk, H * d), dtype); v = randn(73, (Lk, H * d), dtype)
    rng = np.random.default_rng(7)
    m = (rng.uniform(size=Lk) > 0.5).astype(np.float32)
    m[64:128] = 0                                   # one whole key tile masked out
    out = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), torch.from_numpy(m).cuda(), H, False)
    assert_close(oracle.sdpa(q, k, v, H, key_mask=m), to_np(out), dtype)
    out0 = bd.flash_attention_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), torch.zeros(Lk, device="cuda"), H, False)
    assert not to_np(out0).any()


@pytest.mark.parametrize("dtype,d", [("bf16", 128), ("fp16", 40), ("bf16", 72), ("fp16", 96), ("bf16", 64)])
def test_key_mask_with_other_masks(oracle, dtype, d):
    """A scattered 0/1 key mask (per batch item) together with a causal window, with a valid length, and over a cached
    prefix (the mask is indexed over [prefix ; fresh]): every kernel form against the checker. Tiles that the mask hides
    entirely, rows whose visible keys are all masked (zeros), and a mask of -0.0 entries (hidden like +0.0)."""
    B, H, Lq, Lk = 2, 2, 200, 330
    q = randn(81, (B, Lq, H * d), dtype); k = randn(82, (B, Lk, H * d), dtype); v = randn(83, (B, Lk, H * d), dtype)
    rng = np.random.default_rng(d)
    m = (rng.uniform(size=(B, Lk)) > 0.4).astype(np.float32)
    m[0, 128:192] = 0                                # a whole key tile hidden in batch item 0
    m[1, :70] = 0                                    # the first tile and a bit more hidden in batch item 1
    m[1, 100] = -0.0
    m[1, 101] = 1.0
    dq, dk, dv, dm = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), torch.from_numpy(m).cuda()
    window = 90
    lo, hi = oracle.rows_causal(Lq, Lk, window=window)
    out = bd.sdpa_forward(dq, dk, dv, H, key_mask=dm, mask=bd.SdpaMask.causal(Lk - Lq, window))
    for b in range(B):
        assert_close(oracle.sdpa(q[b], k[b], v[b], H, key_mask=m[b], row_lo=lo, row_hi=hi), to_np(out[b]), dtype, f"mask + window, batch {b}")
    vl = torch.tensor([300, 150], dtype=torch.int32, device="cuda")
    out = bd.sdpa_forward(dq, dk, dv, H, key_mask=dm, kv_valid_len=vl)
    for b, n in enumerate((300, 150)):
        assert_close(oracle.sdpa(q[b], k[b, :n], v[b, :n], H, key_mask=m[b, :n]), to_np(out[b]), dtype, f"mask + valid_len, batch {b}")
    # cached prefix of 100 rows (a partly filled prefix tile), the other 230 keys fresh; one mask row shared by the batch
    out = bd.sdpa_forward(dq, dk[:, 100:].contiguous(), dv[:, 100:].contiguous(), H, k_prefix=dk[:, :100].contiguous(),
                          v_prefix=dv[:, :100].contiguous(), key_mask=dm[0])
    for b in range(B):
        assert_close(oracle.sdpa(q[b], k[b], v[b], H, key_mask=m[0]), to_np(out[b]), dtype, f"mask over prefix + fresh, batch {b}")
    # early rows of batch item 1 see only masked keys under a causal mask without offset: zeros
    out = to_np(bd.sdpa_forward(dq[1, :60], dk[1], dv[1], H, key_mask=dm[1], mask=bd.SdpaMask.causal(0)))
    lo, hi = oracle.rows_causal(60, Lk, q_offset=0)
    assert_close(oracle.sdpa(q[1, :60], k[1], v[1], H, key_mask=m[1], row_lo=lo, row_hi=hi), out, dtype, "rows without visible keys")
    assert not out.any()


def _block_causal_case(prefix, blocks):
    """cfg4-shaped: cached prefix of `prefix` text keys; query blocks of sizes `blocks`; block b sees
    the prefix plus blocks 0..b."""
    seg_q_end = list(np.cumsum(blocks))
    seg_k_end = [prefix + e for e in seg_q_end]
    return seg_q_end, seg_k_end, [0] * len(blocks)


@pytest.mark.parametrize("prefix,blocks", [(96, [80, 80, 80, 80]), (64, [128, 128]), (70, [33, 190, 60])])
def test_block_causal_prefix_kv(oracle, kernel_choice, prefix, blocks):
    dtype, H, d = "bf16", 2, 128
    Lq = sum(blocks)
    q = randn(81, (Lq, H * d), dtype); kf = randn(82, (Lq, H * d), dtype); vf = randn(83, (Lq, H * d), dtype)
    kp = randn(84, (prefix, H * d), dtype); vp = randn(85, (prefix, H * d), dtype)
    sq, sk, sc = _block_causal_case(prefix, blocks)
    mask = bd.SdpaMask.block_causal(prefix, sq, sk, sc)
    out = bd.sdpa_forward(to_dev(q, dtype), to_dev(kf, dtype), to_dev(vf, dtype), H, k_prefix=to_dev(kp, dtype),
                          v_prefix=to_dev(vp, dtype), mask=mask)
    k = np.concatenate([kp, kf]); v = np.concatenate([vp, vf])
    lo, hi = oracle.rows_block_causal(Lq, prefix + Lq, prefix, sq, sk, sc)
    assert_close(oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi), to_np(out), dtype)
    # the reference reaches the same result as one unmasked call per image segment over keys [0, e)
    # (src/dit/qwenimage21_forward.cpp:664-669). Key tiles restart at the prefix boundary, so the two
    # forms sum in the same order - and agree bit for bit - when prefix_len is a multiple of the 64-key
    # tile; otherwise they agree to rounding (the reference's own cached-vs-prefill bound is 2e-3).
    dk, dv = to_dev(k, dtype), to_dev(v, dtype)
    s = 0
    for e, ke in zip(sq, sk):
        seg = bd.flash_attention_forward(to_dev(q[s:e], dtype), dk[:ke], dv[:ke], None, H, False)
        if prefix % 64 == 0 and kernel_choice == "rows128":
            assert torch.equal(seg, out[s:e])
        else:
            assert (seg.float() - out[s:e].float()).abs().max().item() <= 2e-3 * max(1.0, out.float().abs().max().item())
        s = e


def test_block_causal_with_text_segments(oracle, kernel_choice):
    """Prefill form with causal text runs and bidirectional image blocks in one launch
    (src/dit/qwenimage21_forward.cpp:650-676)."""
    dtype, H, d = "bf16", 2, 128
    kinds = [("t", 70), ("i", 100), ("t", 30), ("i", 150)]
    L = sum(n for _, n in kinds)
    sq = list(np.cumsum([n for _, n in kinds])); sk = sq; sc = [1 if kd == "t" else 0 for kd, _ in kinds]
    q = randn(91, (L, H * d), dtype); k = randn(92, (L, H * d), dtype); v = randn(93, (L, H * d), dtype)
    out = bd.sdpa_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), H, mask=bd.SdpaMask.block_causal(0, sq, sk, sc))
    block_id, img = [], 0
    for kd, n in kinds:
        block_id += [-1] * n if kd == "t" else [img] * n
        img += kd == "i"
    dense = oracle.dense_block_causal(L, L, 0, block_id)
    assert_close(oracle.sdpa(q, k, v, H, dense_mask=dense), to_np(out), dtype)
    # per-segment calls through the reference's own entry points
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    s = 0
    for (kd, n), e in zip(kinds, sq):
        if kd == "t":
            seg = bd.flash_attention_windowed_forward(dq[s:e], dk[:e], dv[:e], None, H, 0)
        else:
            seg = bd.flash_attention_forward(dq[s:e], dk[:e], dv[:e], None, H, False)
        # rows of several segments share a wavefront in the one-launch form, and a wavefront re-references
        # its softmax as a whole: same values to rounding, bit-identical on the kernel that keeps exact row maxima
        assert_same(seg, out[s:e], kernel_choice == "rows128", "per-segment call vs one launch")
        s = e


@pytest.mark.parametrize("dtype,d,axes", [("bf16", 128, (16, 56, 56)), ("fp16", 64, (16, 24, 24)), ("bf16", 40, (8, 16, 16))])
def test_joint_attention_fused_rope(oracle, kernel_choice, dtype, d, axes):
    H, txt, hp, wp = 2, 37, 9, 11
    L = txt + hp * wp
    q = randn(101, (L, H * d), dtype); k = randn(102, (L, H * d), dtype); v = randn(103, (L, H * d), dtype)
    cos, sin = bd.build_axial_rope_tables(txt, hp, wp, d, axes)
    ocos, osin = oracle.build_axial_rope_tables(txt, hp, wp, d, axes)
    assert np.max(np.abs(to_np(cos) - ocos)) < 1e-6 and np.max(np.abs(to_np(sin) - osin)) < 1e-6
    out = bd.joint_attention(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), cos, sin, d, H)
    # the reference rotates into tensors of Q's dtype before attention (src/dit/common.cpp:192-193)
    qr = oracle.rope_apply(q, ocos, osin, H, d, round_to_dtype=dtype)
    kr = oracle.rope_apply(k, ocos, osin, H, d, round_to_dtype=dtype)
    assert_close(oracle.sdpa(qr, kr, v, H), to_np(out), dtype)
    # fused == stand-alone rope_apply followed by plain attention
    dqr = bd.rope_apply(to_dev(q, dtype), cos, sin, d, H)
    dkr = bd.rope_apply(to_dev(k, dtype), cos, sin, d, H)
    out2 = bd.flash_attention_forward(dqr, dkr, to_dev(v, dtype), None, H, False)
    # the 256-row kernels fold the softmax scale into Q before its rounding: one rounding when fused, two when not
    assert_same(out, out2, kernel_choice == "rows128", "fused vs stand-alone RoPE")
    # with the Kr scratch of the reference signature: K rotated by one pass, Kr holds RoPE(K) afterwards
    Kr = torch.zeros_like(dkr)
    out3 = bd.joint_attention(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), cos, sin, d, H, Kr=Kr)
    assert torch.equal(Kr, dkr)
    assert_same(out3, out2, kernel_choice == "rows128", "Kr scratch form vs stand-alone RoPE")


def test_rope_k_scratch_batched_strided(oracle):
    """The scratch form with batch > 1 and a strided K (K cut out of a fused QKV projection)."""
    dtype, B, H, d, L = "bf16", 2, 2, 128, 200
    qkv = randn(105, (B, L, 3 * H * d), dtype)
    dqkv = to_dev(qkv, dtype)
    dq, dk, dv = dqkv[..., :H * d], dqkv[..., H * d:2 * H * d], dqkv[..., 2 * H * d:]
    ocos, osin = oracle.build_axial_rope_tables(8, 12, 16, d, (16, 56, 56))
    cos, sin = torch.from_numpy(ocos).cuda(), torch.from_numpy(osin).cuda()
    Kr = torch.empty((B, L, H * d), dtype=dq.dtype, device="cuda")
    out = bd.sdpa_forward(dq, dk, dv, H, rope_q=(cos, sin), rope_k=(cos, sin), rope_k_scratch=Kr)
    fused = bd.sdpa_forward(dq, dk, dv, H, rope_q=(cos, sin), rope_k=(cos, sin))
    assert torch.equal(out, fused)
    for b in range(B):
        q, k, v = qkv[b, :, :H * d], qkv[b, :, H * d:2 * H * d], qkv[b, :, 2 * H * d:]
        qr = oracle.rope_apply(q, ocos, osin, H, d, round_to_dtype=dtype)
        kr = oracle.rope_apply(k, ocos, osin, H, d, round_to_dtype=dtype)
        assert_close(oracle.sdpa(qr, kr, v, H), to_np(out[b]), dtype)
        assert_close(kr, to_np(Kr[b]), dtype)


def test_rope_on_fresh_keys_only_with_prefix(oracle):
    """Cached step: prefix K is stored post-RoPE, fresh K and Q are rotated with the table rows of
    their positions (src/dit/qwenimage21_forward.cpp:301-307, :587-649)."""
    dtype, H, d, prefix, hp, wp = "bf16", 2, 128, 50, 8, 8
    img = hp * wp
    cos, sin = oracle.build_qwen_rope_tables([("text", prefix)], hp, wp, d)
    pcos, psin = bd.build_qwen_rope_tables([("text", prefix)], hp, wp, d)      # the product's host builder
    assert np.max(np.abs(to_np(pcos) - cos)) < 1e-6 and np.max(np.abs(to_np(psin) - sin)) < 1e-6
    k_all = randn(111, (prefix + img, H * d), dtype); v_all = randn(112, (prefix + img, H * d), dtype)
    q = randn(113, (img, H * d), dtype)
    kr_all = oracle.rope_apply(k_all, cos, sin, H, d, round_to_dtype=dtype)
    qr = oracle.rope_apply(q, cos[prefix:], sin[prefix:], H, d, round_to_dtype=dtype)
    ref = oracle.sdpa(qr, kr_all, v_all, H)
    tc = torch.from_numpy(cos[prefix:].copy()).cuda(); ts = torch.from_numpy(sin[prefix:].copy()).cuda()
    out = bd.sdpa_forward(to_dev(q, dtype), to_dev(k_all[prefix:], dtype), to_dev(v_all[prefix:], dtype), H,
                          k_prefix=to_dev(kr_all[:prefix], dtype), v_prefix=to_dev(v_all[:prefix], dtype),
                          rope_q=(tc, ts), rope_k=(tc, ts))
    assert_close(ref, to_np(out), dtype)


def test_gqa_masked(oracle):
    dtype, d, Hq, Hkv, L = "bf16", 128, 4, 2, 150
    q = randn(121, (L, Hq * d), dtype); k = randn(122, (L, Hkv * d), dtype); v = randn(123, (L, Hkv * d), dtype)
    m = np.ones(L, dtype=np.float32); m[120:] = 0
    out = bd.gqa_attention_masked(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), None, None, d, Hq, Hkv,
                                  torch.from_numpy(m).cuda())
    # widen K/V as the reference does (src/dit/common.cpp:359-375): kv head g serves q heads [g*r, (g+1)*r)
    kw = k.reshape(L, Hkv, 1, d).repeat(2, axis=2).reshape(L, Hq * d)
    vw = v.reshape(L, Hkv, 1, d).repeat(2, axis=2).reshape(L, Hq * d)
    assert_close(oracle.sdpa(q, kw, vw, Hq, key_mask=m), to_np(out), dtype)


def test_scale_strides_and_views(oracle):
    dtype, H, d, Lq, Lk = "fp16", 2, 64, 90, 140
    q = randn(131, (Lq, H * d), dtype); k = randn(132, (Lk, H * d), dtype); v = randn(133, (Lk, H * d), dtype)
    # K and V as column slices of one packed (Lk, 2*H*d) tensor: row stride != H*d
    kv = torch.cat([to_dev(k, dtype), to_dev(v, dtype)], dim=1)
    out = torch.zeros((Lq, 2 * H * d), dtype=torch.float16, device="cuda")
    bd.sdpa_forward(to_dev(q, dtype), kv[:, :H * d], kv[:, H * d:], H, scale=0.2, out=out[:, H * d:])
    assert_close(oracle.sdpa(q, k, v, H, scale=0.2), to_np(out[:, H * d:]), dtype)
    assert not out[:, :H * d].any()


def test_deterministic(oracle):
    dtype, H, d, L = "bf16", 4, 128, 500
    dq, dk, dv = (to_dev(randn(s, (L, H * d), dtype), dtype) for s in (141, 142, 143))
    a = bd.flash_attention_forward(dq, dk, dv, None, H, False)
    b = bd.flash_attention_forward(dq, dk, dv, None, H, False)
    assert torch.equal(a, b)          # bit-exact across runs, as the reference's smoke tests demand


def test_closed_forms_on_device():
    dtype, H, d, Lq, Lk = "bf16", 2, 128, 100, 260
    q = to_dev(randn(151, (Lq, H * d), dtype), dtype)
    v = randn(152, (Lk, H * d), dtype)
    k_same = to_dev(np.tile(randn(153, (1, H * d), dtype), (Lk, 1)), dtype)
    out = to_np(bd.flash_attention_forward(q, k_same, to_dev(v, dtype), None, H, False))
    assert np.max(np.abs(out - v.mean(axis=0)[None, :])) < 2e-2     # equal keys -> mean of V
    v_const = np.tile(randn(154, (1, H * d), dtype), (Lk, 1))
    k = to_dev(randn(155, (Lk, H * d), dtype), dtype)
    out = to_np(bd.flash_attention_forward(q, k, to_dev(v_const, dtype), None, H, False))
    assert np.max(np.abs(out - v_const[:1])) < 2e-2                 # constant V -> that constant


def test_errors():
    q = torch.zeros((8, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="flash_attention_forward: D must equal"):
        bd.flash_attention_forward(q, q, q, None, 3, False)
    with pytest.raises(RuntimeError, match="no kernel"):
        bd.flash_attention_forward(q, q, q, None, 8, False)          # head_dim 32
    with pytest.raises(RuntimeError, match="not on the GPU"):
        bd.flash_attention_forward(q.cpu(), q, q, None, 2, False)
    with pytest.raises(RuntimeError, match="dtype"):
        bd.flash_attention_forward(q.float(), q.float(), q.float(), None, 2, False)
    with pytest.raises(RuntimeError, match="K and V must be"):
        bd.flash_attention_forward(q, q[:, :128], q, None, 2, False)


def test_block_causal_maximum_segment_count(oracle, kernel_choice):
    """The segment table holds 32 entries: 32 alternating text / image segments of ragged lengths behind a cached
    prefix, in one launch; one more segment is refused."""
    dtype, H, d, prefix = "bf16", 2, 64, 37
    lens = [5 + (7 * i) % 23 + (29 if i % 2 else 0) for i in range(32)]
    kinds = [("t" if i % 2 == 0 else "i", n) for i, n in enumerate(lens)]
    L = sum(lens)
    sq = [int(x) for x in np.cumsum(lens)]
    sk = [prefix + e for e in sq]
    sc = [1 if kd == "t" else 0 for kd, _ in kinds]
    q = randn(301, (L, H * d), dtype); k = randn(302, (L, H * d), dtype); v = randn(303, (L, H * d), dtype)
    kp = randn(304, (prefix, H * d), dtype); vp = randn(305, (prefix, H * d), dtype)
    mask = bd.SdpaMask.block_causal(prefix, sq, sk, sc)
    out = bd.sdpa_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), H, mask=mask,
                          k_prefix=to_dev(kp, dtype), v_prefix=to_dev(vp, dtype))
    lo, hi = oracle.rows_block_causal(L, prefix + L, prefix, sq, sk, sc)
    ref = oracle.sdpa(q, np.concatenate([kp, k]), np.concatenate([vp, v]), H, row_lo=lo, row_hi=hi)
    assert_close(ref, to_np(out), dtype, "32 segments")
    with pytest.raises(RuntimeError, match="segments"):
        bd.sdpa_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), H,
                        mask=bd.SdpaMask.block_causal(0, sq + [L + 1], sq + [L + 1], sc + [0]))
