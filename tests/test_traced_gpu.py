"""Traced / steered joint attention on the device (dit::joint_attention_traced, src/dit/common.cpp:198-329): RoPE on
Q and K, attention with the optional image->text logit bias, and the head-averaged softmax map. The reference does
this in a host loop over downloaded tensors; the CPU checker restates that loop (orc_sdpa with bias and attn_avg).
Output tolerance as for every attention call (helpers.TOL); the map is FP32 on both sides: probabilities are compared
absolutely (<= 2e-5 on values <= 1; scores come from the same bf16 inputs with FP32 accumulation on both sides, the
exponential on the GPU is the hardware exp2) and its rows must sum to 1."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["by_size", "rows128", "rows256", "rows256_regs"])
def kernel_choice(request):
    """The bias and the softmax denominators exist in the 128-row kernel and in an instance of each 256-row kernel."""
    bd.set_sdpa_kernel_choice({"by_size": 0, "rows128": 1, "rows256": 2, "rows256_regs": 3}[request.param])
    yield request.param
    bd.set_sdpa_kernel_choice(0)


def tables(oracle, txt, hp, wp, d, axes):
    cos, sin = oracle.build_axial_rope_tables(txt, hp, wp, d, axes)
    return cos, sin, torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()


@pytest.mark.parametrize("dtype,H,d,txt,hp,wp,axes,with_bias", [
    ("bf16", 4, 128, 37, 9, 11, (16, 56, 56), True),
    ("bf16", 4, 128, 37, 9, 11, (16, 56, 56), False),
    ("fp16", 3, 64, 64, 8, 8, (16, 24, 24), True),
    ("bf16", 2, 72, 5, 20, 13, (8, 32, 32), True),        # 265 rows: ragged tiles on both axes
])
def test_traced_matches_checker(oracle, kernel_choice, dtype, H, d, txt, hp, wp, axes, with_bias):
    L = txt + hp * wp
    q, k, v = (randn(9400 + i, (L, H * d), dtype) for i in range(3))
    cos, sin, dcos, dsin = tables(oracle, txt, hp, wp, d, axes)
    bias = (randn(9410, (L - txt, txt), "fp32") * 1.5).astype(np.float32) if with_bias else None
    dbias = None if bias is None else torch.from_numpy(bias).cuda()
    out, avg = bd.joint_attention_traced(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), dcos, dsin, d, H,
                                         txt_len=txt, image_text_bias=dbias)
    qr = oracle.rope_apply(q, cos, sin, H, d, round_to_dtype=dtype)
    kr = oracle.rope_apply(k, cos, sin, H, d, round_to_dtype=dtype)
    ref_o, ref_avg = oracle.sdpa(qr, kr, v, H, bias=bias, bias_q0=txt, return_attn_avg=True)
    print(assert_close(ref_o, to_np(out), dtype, "traced output"))
    got = to_np(avg)
    assert got.shape == (L, L) and avg.dtype == torch.float32
    assert np.abs(got - ref_avg).max() <= 2e-5, np.abs(got - ref_avg).max()
    assert np.abs(got.sum(axis=1) - 1.0).max() <= 1e-4
    if with_bias:
        # the bias steers: without it the image rows put different mass on the text keys
        _, avg0 = bd.joint_attention_traced(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), dcos, dsin, d, H)
        assert np.abs(to_np(avg0)[txt:, :txt] - got[txt:, :txt]).max() > 1e-3
        assert np.abs(to_np(avg0)[:txt] - got[:txt]).max() <= 1e-6          # text rows carry no bias


@pytest.mark.parametrize("with_bias", [True, False])
def test_traced_at_a_shape_whose_plain_call_splits_its_last_round(oracle, with_bias):
    """Flux at 768 px (512 text + 48 x 48 image rows, 24 heads of 128): a plain attention call of this shape cuts its last
    round of work groups along the key axis when a scratch is lent. The traced call asks for the softmax denominators
    (and a bias), which the split launch does not provide, so it must not take that route (it runs on the 256-row
    kernel's instance with bias and denominators): sampled rows of the output and of the map against the checker, and no
    split scratch is asked for."""
    import ctypes as C
    from brodiffusion_amd import _capi as capi
    dtype, H, d, txt, hp, wp = "bf16", 24, 128, 512, 48, 48
    L = txt + hp * wp
    q, k, v = (randn(9700 + i, (L, H * d), dtype) for i in range(3))
    cos, sin, dcos, dsin = tables(oracle, txt, hp, wp, d, (16, 56, 56))
    bias = (randn(9710, (L - txt, txt), "fp32") * 1.5).astype(np.float32) if with_bias else None
    dbias = None if bias is None else torch.from_numpy(bias).cuda()
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    out, avg = bd.joint_attention_traced(dq, dk, dv, dcos, dsin, d, H, txt_len=txt, image_text_bias=dbias)
    rows = np.concatenate([np.arange(0, txt, 37), np.arange(txt + 5, L, 53)]).astype(np.int32)
    qr = oracle.rope_apply(q, cos, sin, H, d, round_to_dtype=dtype)
    kr = oracle.rope_apply(k, cos, sin, H, d, round_to_dtype=dtype)
    ref_o, ref_avg = oracle.sdpa(qr, kr, v, H, bias=bias, bias_q0=txt, rows=rows, return_attn_avg=True)
    assert_close(ref_o[rows], to_np(out)[rows], dtype, "traced output")
    got = to_np(avg)
    assert np.abs(got[rows] - ref_avg[rows]).max() <= 2e-5
    assert np.abs(got.sum(axis=1) - 1.0).max() <= 1e-4
    # the plain call of this shape does split; with a request for the denominators it must not
    a = capi.MiSdpaArgs()
    a.struct_size = C.sizeof(capi.MiSdpaArgs)
    a.dtype, a.batch, a.num_heads, a.head_dim, a.q_len, a.kv_len = capi.MI_DTYPE_BF16, 1, H, d, L, L
    a.q, a.k, a.v, a.o = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), out.data_ptr()
    assert capi.lib().mi_sdpa_split_scratch_bytes(C.byref(a)) > 0
    lse = torch.empty(H * L, dtype=torch.float32, device="cuda")
    a.lse_out = lse.data_ptr()
    assert capi.lib().mi_sdpa_split_scratch_bytes(C.byref(a)) == 0


def test_traced_equals_fused_path_without_bias(oracle):
    """With no bias the traced output is the ordinary joint attention (same kernels up to the 128-row form)."""
    dtype, H, d, txt, hp, wp = "bf16", 8, 128, 32, 16, 16
    L = txt + hp * wp
    q, k, v = (to_dev(randn(9500 + i, (L, H * d), dtype), dtype) for i in range(3))
    _, _, dcos, dsin = tables(oracle, txt, hp, wp, d, (16, 56, 56))
    out, avg = bd.joint_attention_traced(q, k, v, dcos, dsin, d, H)
    bd.set_sdpa_kernel_choice(1)
    try:
        fused = bd.joint_attention(q, k, v, dcos, dsin, d, H, Kr=torch.empty_like(k))
    finally:
        bd.set_sdpa_kernel_choice(0)
    assert (out.float() - fused.float()).abs().max().item() <= 2.0 ** -7
    # a constant bias over all text keys of a row changes nothing only if it covers every key: here it covers the text
    # keys alone, so it must move mass between text and image keys, by the closed form p_txt' = p_txt e^c / (p_txt e^c + 1 - p_txt)
    c = 0.7
    bias = torch.full((L - txt, txt), c, dtype=torch.float32, device="cuda")
    _, avg_b = bd.joint_attention_traced(q, k, v, dcos, dsin, d, 1 * H, txt_len=txt, image_text_bias=bias)
    # per head the closed form holds exactly; averaged over heads only the direction is fixed: text mass grows
    assert (avg_b[txt:, :txt].sum(dim=1) > avg[txt:, :txt].sum(dim=1)).all()


def test_single_head_bias_closed_form(oracle):
    dtype, H, d, txt, hp, wp = "bf16", 1, 128, 40, 8, 8
    L = txt + hp * wp
    q, k, v = (to_dev(randn(9600 + i, (L, H * d), dtype), dtype) for i in range(3))
    _, _, dcos, dsin = tables(oracle, txt, hp, wp, d, (16, 56, 56))
    _, a0 = bd.joint_attention_traced(q, k, v, dcos, dsin, d, H)
    c = -1.3
    bias = torch.full((L - txt, txt), c, dtype=torch.float32, device="cuda")
    _, a1 = bd.joint_attention_traced(q, k, v, dcos, dsin, d, H, txt_len=txt, image_text_bias=bias)
    p = a0[txt:, :txt].sum(dim=1).double()
    expect = p * np.exp(c) / (p * np.exp(c) + 1 - p)
    assert (a1[txt:, :txt].sum(dim=1).double() - expect).abs().max().item() <= 1e-5


def test_traced_errors():
    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, device="cuda", dtype=dt)
    q = z(16, 128)
    cs = z(16, 64, dt=torch.float32)
    with pytest.raises(RuntimeError, match=r"image_text_bias must be \(img_len, txt_len\)"):
        bd.joint_attention_traced(q, q, q, cs, cs, 128, 1, txt_len=4, image_text_bias=z(12, 5, dt=torch.float32))
    with pytest.raises(RuntimeError, match="image_text_bias must be FP32"):
        bd.joint_attention_traced(q, q, q, cs, cs, 128, 1, txt_len=4, image_text_bias=z(12, 4))
    with pytest.raises(RuntimeError, match="txt_len out of range"):
        bd.joint_attention_traced(q, q, q, cs, cs, 128, 1, txt_len=40, image_text_bias=z(12, 4, dt=torch.float32))
    with pytest.raises(RuntimeError, match="share shape"):
        bd.joint_attention_traced(q, z(8, 128), q, cs, cs, 128, 1)


@pytest.mark.parametrize("dtype,Lq,Lk,C,Cctx,H,with_bias,with_mask", [
    ("fp16", 1024, 77, 320, 768, 8, True, False),      # SD1.5 level 0 cross attention, traced and steered
    ("fp16", 256, 77, 640, 768, 8, False, False),      # level 1 (head_dim 80), plain trace
    ("bf16", 300, 50, 128, 96, 2, True, True),         # ragged sizes, bias and key mask together
])
def test_cross_attention_with_attn(oracle, kernel_choice, dtype, Lq, Lk, C, Cctx, H, with_bias, with_mask):
    """bt::cross_attention_forward_with_attn as src/unet_blocks.cpp:282-290 calls it: projections, attention with logit
    bias / key mask, output projection, head-averaged map."""
    x, ctx = randn(9501, (Lq, C), dtype), randn(9502, (Lk, Cctx), dtype)
    wq = oracle.round_to(randn(9503, (C, C), "fp32") / np.sqrt(C), dtype)
    wk = oracle.round_to(randn(9504, (C, Cctx), "fp32") / np.sqrt(Cctx), dtype)
    wv = oracle.round_to(randn(9505, (C, Cctx), "fp32") / np.sqrt(Cctx), dtype)
    wo = oracle.round_to(randn(9506, (C, C), "fp32") / np.sqrt(C), dtype)
    bias = (randn(9507, (Lq, Lk), "fp32") * 1.5).astype(np.float32) if with_bias else None
    mask = None
    if with_mask:
        mask = np.ones(Lk, np.float32)
        mask[Lk - 7:] = 0
        mask[3] = 0
    d = lambda a: to_dev(a, dtype)
    out, avg = bd.cross_attention_forward_with_attn(
        d(x), d(ctx), d(wq), d(wk), d(wv), d(wo), None if mask is None else torch.from_numpy(mask).cuda(),
        None if bias is None else torch.from_numpy(bias).cuda(), H)
    q = oracle.round_to(oracle.linear(x, wq), dtype)
    k = oracle.round_to(oracle.linear(ctx, wk), dtype)
    v = oracle.round_to(oracle.linear(ctx, wv), dtype)
    ref_a, ref_avg = oracle.sdpa(q, k, v, H, key_mask=mask, bias=bias, return_attn_avg=True)
    ref = oracle.linear(oracle.round_to(ref_a, dtype), wo)
    assert_close(ref, to_np(out), dtype, "cross attention with map: output")
    got = to_np(avg)
    # The projected Q and K are rounded to the tensor dtype on both sides, and a sum that lands near a rounding
    # boundary goes either way: single elements differ by one unit in the last place, which moves a score, and with
    # it a probability, by about that fraction. (Attention and map alone, on identical Q and K, agree to 1e-6:
    # test_traced_matches_checker.)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.all(np.abs(got - ref_avg) <= 5e-5 + 2 * unit * ref_avg)
    assert np.abs(got.sum(axis=1) - 1.0).max() <= 1e-4
    if with_mask:
        assert (got[:, mask == 0] == 0).all()
