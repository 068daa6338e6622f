"""SanaDenoiser::self_attention_ (src/dit/sana.cpp:411-595) as one operator, against the CPU checker's pieces composed the
way the reference composes them: bias-free q / k / v projections, optional qk_norm across the full inner dimension
(:449-461), ReLU linear attention per head (:470-520), biased output projection (:587-594), with the identity seam's
capture and inject (:489-506). The reference keeps q, k, v and the attention output channel-major, (D, N); the operator
stays token-major from x_mod to out, so the comparison is on (N, D) tensors throughout. Intermediates are tensors of the
compute dtype on both sides. Also the row RMSNorm on its own (bt::rms_norm_forward)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def _weights(oracle, D, seed, dtype):
    w = lambda s: oracle.round_to(randn(seed + s, (D, D), "fp32") / np.sqrt(D), dtype)
    return w(0), w(1), w(2), w(3), oracle.round_to(0.1 * randn(seed + 4, (D,), "fp32"), dtype)


def _reference(oracle, x, wq, wk, wv, wo, bo, H, dtype, nq=None, nk=None, anchor=None, weight=0.0):
    N, D = x.shape
    d = D // H
    q = oracle.round_to(oracle.linear(x, wq), dtype)
    k = oracle.round_to(oracle.linear(x, wk), dtype)
    v = oracle.round_to(oracle.linear(x, wv), dtype)
    if nq is not None:
        q = oracle.round_to(oracle.rms_norm(q, nq, 1e-5), dtype)
        k = oracle.round_to(oracle.rms_norm(k, nk, 1e-5), dtype)
    attn, S, z = oracle.linear_attn_relu(q, k, v, H, return_state=True)
    state = np.concatenate([S.reshape(H, d * d), z.reshape(H, d)], axis=1)        # per head: d rows of S, then z
    if anchor is not None:
        tot = state.astype(np.float64) + weight * anchor.astype(np.float64)
        St, zt = tot[:, :d * d].reshape(H, d, d), tot[:, d * d:]
        qr = np.maximum(q, 0).reshape(N, H, d).astype(np.float64)
        num = np.einsum("hij,nhj->nhi", St, qr); den = np.einsum("hj,nhj->nh", zt, qr)
        attn = (num / (den[..., None] + 1e-15)).reshape(N, D).astype(np.float32)
    out = oracle.linear(oracle.round_to(attn, dtype), wo, bo)
    return out, state


@pytest.mark.parametrize("N,H,d,qk_norm", [(256, 10, 32, False), (300, 6, 32, True), (1024, 70, 32, False), (128, 4, 112, True)])
def test_sana_self_attention_matches_checker(oracle, N, H, d, qk_norm):
    dtype, D = "bf16", H * d
    x = randn(9900 + N, (N, D), dtype)
    wq, wk, wv, wo, bo = _weights(oracle, D, 9910 + N, dtype)
    nq = oracle.round_to(1.0 + 0.2 * randn(9920, (D,), "fp32"), dtype) if qk_norm else None
    nk = oracle.round_to(1.0 + 0.2 * randn(9921, (D,), "fp32"), dtype) if qk_norm else None
    dev = lambda a: None if a is None else to_dev(a, dtype)
    state = torch.zeros(H * (d * d + d), dtype=torch.float32, device="cuda")
    out = bd.sana_self_attention(dev(x), dev(wq), dev(wk), dev(wv), dev(wo), dev(bo), H, nq=dev(nq), nk=dev(nk),
                                 ref_mode="capture", ref_state=state)
    ref, ref_state = _reference(oracle, x, wq, wk, wv, wo, bo, H, dtype, nq, nk)
    assert_close(ref, to_np(out), dtype, "sana self attention")
    got_state = state.cpu().numpy().reshape(H, d * d + d)
    # the projections round q, k, v to the compute dtype on both sides and a sum near a rounding boundary goes either way,
    # so the states agree to the relative size of one such flip, not to FP32 rounding
    assert np.abs(got_state - ref_state).max() <= 2e-3 * np.abs(ref_state).max()
    plain = bd.sana_self_attention(dev(x), dev(wq), dev(wk), dev(wv), dev(wo), dev(bo), H, nq=dev(nq), nk=dev(nk))
    assert torch.equal(plain, out)                                        # capturing changes nothing


def test_sana_identity_seam_inject(oracle):
    dtype, N, H, d = "bf16", 256, 8, 32
    D = H * d
    x, xa = randn(9930, (N, D), dtype), randn(9931, (N, D), dtype)
    wq, wk, wv, wo, bo = _weights(oracle, D, 9940, dtype)
    dev = lambda a: to_dev(a, dtype)
    W = (dev(wq), dev(wk), dev(wv), dev(wo), dev(bo))
    anchor = torch.zeros(H * (d * d + d), dtype=torch.float32, device="cuda")
    bd.sana_self_attention(dev(xa), *W, H, ref_mode="capture", ref_state=anchor)
    before = anchor.clone()
    weight = 0.6
    out = bd.sana_self_attention(dev(x), *W, H, ref_mode="inject", ref_state=anchor, ref_weight=weight)
    assert torch.equal(anchor, before)                                    # the anchor is read, never written
    _, anchor_ref = _reference(oracle, xa, wq, wk, wv, wo, bo, H, dtype)
    ref, _ = _reference(oracle, x, wq, wk, wv, wo, bo, H, dtype, anchor=anchor_ref, weight=weight)
    assert_close(ref, to_np(out), dtype, "inject")
    # weight 0 is no injection at all
    off = bd.sana_self_attention(dev(x), *W, H)
    zero = bd.sana_self_attention(dev(x), *W, H, ref_mode="inject", ref_state=anchor, ref_weight=0.0)
    assert torch.equal(zero, off) and not torch.equal(out, off)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("rows,cols", [(300, 2240), (7, 8), (64, 4096), (3, 16384)])
def test_rms_norm_rows(oracle, dtype, rows, cols):
    x = oracle.round_to(randn(9950 + cols, (rows, cols), dtype) * 3.0, dtype)
    g = oracle.round_to(1.0 + 0.3 * randn(9951, (cols,), "fp32"), dtype)
    dx = to_dev(x, dtype)
    out = bd.rms_norm_rows(dx, to_dev(g, dtype), 1e-5)
    exact = oracle.rms_norm(x, g, 1e-5)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11                    # one rounding to the storage dtype
    assert np.all(np.abs(to_np(out) - exact) <= unit * np.maximum(np.abs(exact), 2.0 ** -6) * 1.02 + 1e-6)
    bd.rms_norm_rows(dx, to_dev(g, dtype), 1e-5, out=dx)                   # in place
    assert torch.equal(dx, out)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        bd.rms_norm_rows(torch.zeros(4, 12, dtype=dx.dtype, device="cuda"), torch.zeros(12, dtype=dx.dtype, device="cuda"), 1e-5)
