"""Per-head RMSNorm + RoPE in one pass (mi_headnorm_rope) against the CPU checker; the reference runs the two as
separate passes with a rounding in between (src/dit/qwenimage21_forward.cpp:582-585), so both forms of the checker
are compared: FP32 in between (what the kernel computes: one rounding, error within one unit in the last place) and
rounded in between (the reference's dataflow: agreement to the usual tolerance)."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
@pytest.mark.parametrize("L,H,d,axes", [(577, 24, 128, (16, 56, 56)), (64, 5, 64, (16, 24, 24)), (33, 70, 32, (8, 12, 12)), (1, 1, 128, (16, 56, 56)),
                                      (100, 8, 64, (16, 24, 24)), (50, 12, 32, (8, 12, 12))])   # head counts that are multiples of 4: one thread per 4 heads
def test_headnorm_rope_matches_checker(oracle, dtype, L, H, d, axes):
    x = randn(9000 + L, (L, H * d), dtype) * 2.5
    x = oracle.round_to(x, dtype)
    gain = oracle.round_to(1.0 + 0.2 * randn(9001, (d,), "fp32"), dtype)
    hp = max(1, int(np.sqrt(L)) - 1)
    wp = hp
    txt = L - hp * wp
    cos, sin = oracle.build_axial_rope_tables(txt, hp, wp, d, axes)
    dx, dg = to_dev(x, dtype), to_dev(gain, dtype)
    dcos, dsin = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    out = bd.headnorm_rope(dx, dg, 1e-6, dcos, dsin, d, H)
    exact = oracle.headnorm_rope(x, gain, 1e-6, cos, sin, H, d)                       # FP32 in between, unrounded
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.all(np.abs(to_np(out) - exact) <= unit * np.maximum(np.abs(exact), 2.0 ** -6) * 1.02 + 1e-6)
    # Outputs reach magnitude ~8 here, where one unit in the last place of bf16 is 0.03: the absolute bound of the
    # attention tolerances does not apply to this elementwise result; rel-L2 does, plus a bound in units of the last
    # place of the largest value (the extra rounding of the two-pass form moves both members of a rotated pair by
    # half a unit of the LARGER member, whatever the size of the result).
    def close(ref, got, what):
        m = oracle.compare(ref, got)
        assert m["rel_l2"] <= TOL[dtype][0], f"{what}: {m}"
        assert m["max_abs"] <= 3 * unit * max(1.0, float(np.abs(ref).max())), f"{what}: {m}"
    two_pass = oracle.headnorm_rope(x, gain, 1e-6, cos, sin, H, d, round_to_dtype=dtype, round_between=dtype)
    close(two_pass, to_np(out), "headnorm_rope vs the two-pass dataflow")
    # the normalisation alone, and the two library passes composed
    normed = bd.headnorm_rope(dx, dg, 1e-6, None, None, d, H)
    close(oracle.headnorm_rope(x, gain, 1e-6, None, None, H, d), to_np(normed), "headnorm alone")
    composed = bd.rope_apply(normed, dcos, dsin, d, H)
    close(to_np(composed), to_np(out), "fused vs norm then rope_apply")


def test_headnorm_rope_cache_rows_in_place_and_strides(oracle):
    dtype, L, H, d, prefix = "bf16", 300, 24, 128, 77
    x = randn(9100, (L, H * d), dtype)
    gain = oracle.round_to(randn(9101, (d,), "fp32"), dtype)
    cos, sin = oracle.build_axial_rope_tables(L - 256, 16, 16, d, (16, 56, 56))
    dx, dg = to_dev(x, dtype), to_dev(gain, dtype)
    dcos, dsin = torch.from_numpy(cos).cuda(), torch.from_numpy(sin).cuda()
    cache = torch.full((prefix + 2, H * d), 9.0, device="cuda", dtype=torch.bfloat16)
    out = bd.headnorm_rope(dx, dg, 1e-6, dcos, dsin, d, H, cache_out=cache[:prefix])
    assert torch.equal(cache[:prefix], out[:prefix]) and (cache[prefix:] == 9).all()
    # a column slice of a wider (L, 3*D) projection as input, in place
    wide = torch.zeros(L, 3 * H * d, device="cuda", dtype=torch.bfloat16)
    wide[:, H * d:2 * H * d] = dx
    view = wide[:, H * d:2 * H * d]
    bd.headnorm_rope(view, dg, 1e-6, dcos, dsin, d, H, out=view)
    assert torch.equal(view, out)
    assert (wide[:, :H * d] == 0).all() and (wide[:, 2 * H * d:] == 0).all()


def test_headnorm_rope_errors():
    z = lambda *s, dt=torch.bfloat16: torch.zeros(*s, device="cuda", dtype=dt)
    with pytest.raises(RuntimeError, match="head_dim 40 not supported"):
        bd.headnorm_rope(z(4, 80), z(40), 1e-6, None, None, 40, 2)
    with pytest.raises(RuntimeError, match="gain must hold"):
        bd.headnorm_rope(z(4, 256), z(64), 1e-6, None, None, 128, 2)
    with pytest.raises(RuntimeError, match="cos/sin"):
        bd.headnorm_rope(z(4, 256), z(128), 1e-6, z(4, 32, dt=torch.float32), z(4, 32, dt=torch.float32), 128, 2)
    with pytest.raises(RuntimeError, match="not on the GPU"):
        bd.headnorm_rope(z(4, 256).cpu(), z(128), 1e-6, None, None, 128, 2)
    assert bd.headnorm_rope(z(0, 256), z(128), 1e-6, None, None, 128, 2).shape == (0, 256)


# ── row scaling: the prefix-KV dial ──────────────────────────────────────────
@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_scale_rows(oracle, dtype):
    rows, cols = 77, 3072
    x = randn(9200, (rows, cols), dtype)
    w = (0.25 + np.arange(rows, dtype=np.float32) / 64).astype(np.float32)
    dx = to_dev(x, dtype)
    dw = torch.from_numpy(w).cuda()
    got = bd.scale_rows(dx, 0.75, dw)
    ref = oracle.round_to(x * (np.float32(0.75) * w)[:, None], dtype)          # one FP32 product, one rounding
    assert np.array_equal(to_np(got), ref)
    assert torch.equal(bd.scale_rows(dx, 1.0), dx)
    assert torch.equal(bd.scale_rows(bd.scale_rows(dx, 0.5), 0.5), bd.scale_rows(dx, 0.25))
    # in place on a row slice of a larger buffer
    buf = torch.zeros(rows + 3, cols, device="cuda", dtype=dx.dtype)
    buf[1:rows + 1] = dx
    bd.scale_rows(buf[1:rows + 1], 0.75, dw, out=buf[1:rows + 1])
    assert torch.equal(buf[1:rows + 1], got) and (buf[0] == 0).all() and (buf[rows + 1:] == 0).all()
    with pytest.raises(RuntimeError, match="row_scale must hold 77"):
        bd.scale_rows(dx, 1.0, dw[:5])


def test_prefix_dial_equals_scaled_keys_and_values(oracle):
    """Attention over [scaled prefix ; fresh] against the checker fed the same scaled rows."""
    dtype, H, d, prefix, Lq = "bf16", 4, 128, 96, 200
    q, kf, vf = (randn(9300 + i, (Lq, H * d), dtype) for i in range(3))
    kp, vp = randn(9304, (prefix, H * d), dtype), randn(9305, (prefix, H * d), dtype)
    dq, dkf, dvf, dkp, dvp = (to_dev(t, dtype) for t in (q, kf, vf, kp, vp))
    ks, vs = bd.scale_rows(dkp, 0.5), bd.scale_rows(dvp, 1.25)
    out = bd.sdpa_forward(dq, dkf, dvf, H, k_prefix=ks, v_prefix=vs)
    k = np.concatenate([oracle.round_to(kp * np.float32(0.5), dtype), kf])
    v = np.concatenate([oracle.round_to(vp * np.float32(1.25), dtype), vf])
    assert_close(oracle.sdpa(q, k, v, H), to_np(out), dtype, "prefix dial")
    assert not torch.equal(out, bd.sdpa_forward(dq, dkf, dvf, H, k_prefix=dkp, v_prefix=dvp))
