"""The SD1.5 transformer block's fused helpers (include/brodiffusion/fused_transformer.h:20-61): FF1 + exact GEGLU in
one GEMM, Y += X, Y += row bias. Shapes and tolerances of the reference's own parity test come first
(tests/test_fused_parity.cpp:172-200, :268-276: inputs uniform in [-1, 1] x scale rounded to fp16, fused against
linear followed by geglu, relative 0.01 / absolute 0.008), then the real FF sizes against the CPU checker."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def uniform(seed, shape, scale, dtype, oracle, offset=0.0):
    rng = np.random.default_rng(seed)
    return oracle.round_to((rng.uniform(-1.0, 1.0, shape) * scale + offset).astype(np.float32), dtype)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("B,d_in,d_out", [(40, 64, 48), (128, 128, 96), (8192, 320, 1280), (2048, 640, 2560), (77, 1280, 5120), (1, 8, 8),
                                          # ragged last tiles of the 256-token-tile form (in_features a multiple of 320, at least one
                                          # tile per compute unit): 160 of 256 tokens, 8 of 64 features
                                          (4000, 320, 1032), (3000, 640, 1480)])
def test_fused_linear_geglu(oracle, dtype, B, d_in, d_out):
    x = uniform(21, (B, d_in), 1.0, dtype, oracle)
    w = uniform(22, (2 * d_out, d_in), 0.1, dtype, oracle)
    b = uniform(23, (2 * d_out,), 0.2, dtype, oracle)
    dx, dw, db = to_dev(x, dtype), to_dev(w, dtype), to_dev(b, dtype)
    y = bd.fused_linear_geglu(dx, dw, db)
    assert y.shape == (B, d_out)
    ref = oracle.geglu_exact(oracle.linear(x, w, b))                      # exact: no intermediate rounding
    err = np.abs(to_np(y) - ref)
    assert err.max() <= 0.008 + 0.01 * np.abs(ref).max()                  # the reference's bound
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    assert np.all(err <= unit * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)   # FP32 throughout, one rounding
    # unfused composition on the device (what the reference compares against): linear, round, then geglu
    t = bd.linear_batched(dw, db, dx)
    unfused = oracle.geglu_exact(to_np(t))
    assert np.abs(to_np(y) - unfused).max() <= 0.008 + 0.01 * np.abs(unfused).max()


@pytest.mark.parametrize("B,d_in,d_out", [(200, 64, 72), (4000, 320, 1032)])
def test_fused_linear_geglu_without_bias(oracle, B, d_in, d_out):
    """No bias (the C ABI takes a null pointer): both kernel forms, the small one and the one that walks 256-token tiles."""
    dtype = "bf16"
    x = uniform(25, (B, d_in), 1.0, dtype, oracle)
    w = uniform(26, (2 * d_out, d_in), 0.1, dtype, oracle)
    y = to_np(bd.fused_linear_geglu(to_dev(x, dtype), to_dev(w, dtype), None))
    ref = oracle.geglu_exact(oracle.linear(x, w, None))
    err = np.abs(y - ref)
    assert np.all(err <= 2.0 ** -8 * np.maximum(np.abs(ref), 2.0 ** -6) * 1.05 + 2e-6)


def _quantised(seed, n_out, n_in):
    rng = np.random.default_rng(seed)
    q = rng.integers(-127, 128, (n_out, n_in)).astype(np.int8)
    scales = (rng.uniform(0.5, 1.5, n_out) / (73.0 * np.sqrt(n_in))).astype(np.float32)     # rows of unit-variance weights
    return q, scales, q.astype(np.float32) * scales[:, None]


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("B,d_in,d_out", [(40, 64, 48), (8192, 320, 1280), (300, 1280, 5120), (1000, 328, 72)])
def test_fused_linear_geglu_int8w(oracle, dtype, B, d_in, d_out):
    """The W8A16 overload (include/brodiffusion/fused_transformer.h:37-48). The reference composes it from its INT8-weight
    linear layer into a 16-bit (B, 2*D_out) buffer and a GEGLU pass over that buffer (src/fused_transformer.cu:360-396);
    the single GEMM here rounds the two halves where the buffer would, so it must agree with that composition run on the
    device (the linear layer's output, then the checker's GEGLU) to the final rounding, and with the checker end to end."""
    x = uniform(41, (B, d_in), 1.0, dtype, oracle)
    q, scales, w = _quantised(42 + d_out, 2 * d_out, d_in)
    b = uniform(43, (2 * d_out,), 0.2, dtype, oracle)
    dx, db = to_dev(x, dtype), to_dev(b, dtype)
    dq, ds = torch.from_numpy(q).cuda(), torch.from_numpy(scales).cuda()
    y = to_np(bd.fused_linear_geglu_int8w(dx, dq, ds, db))
    assert y.shape == (B, d_out)
    unit = 2.0 ** -8 if dtype == "bf16" else 2.0 ** -11
    composed = oracle.geglu_exact(to_np(bd.linear_forward_batched_int8w_fp16(dq, ds, db, dx)))
    assert np.all(np.abs(y - composed) <= unit * np.maximum(np.abs(composed), 2.0 ** -6) * 1.05 + 2e-6)
    ref = oracle.geglu_exact(oracle.round_to(oracle.linear(x, w, b), dtype))
    assert np.abs(y - ref).max() <= 0.008 + 0.01 * np.abs(ref).max()        # the reference's bound for the 16-bit form
    with pytest.raises(RuntimeError, match="scales must hold"):
        bd.fused_linear_geglu_int8w(dx, dq, ds[:-1], db)
    with pytest.raises(RuntimeError, match="int8"):
        bd.fused_linear_geglu_int8w(dx, dq.to(torch.int16), ds, db)


def test_geglu_gate_tails(oracle):
    """gelu_exact over the whole range of the gate, one gate value per output column: a zero weight and the gate's value as
    its bias, value half = 1. The left tail keeps its relative accuracy (x Phi(x) down to the smallest normal numbers of
    the output type), the right tail is the identity."""
    dtype, B, d_in = "bf16", 64, 64
    gates = np.concatenate([np.linspace(-12.0, 12.0, 193), [-0.0, 1e-3, -1e-3, 30.0, -30.0, 5.5, -5.5]]).astype(np.float32)
    gates = oracle.round_to(gates, dtype)
    d_out = len(gates)                                   # 200 columns: a multiple of 8
    w = np.zeros((2 * d_out, d_in), np.float32)
    b = np.concatenate([np.ones(d_out, np.float32), gates])
    x = uniform(27, (B, d_in), 1.0, dtype, oracle)
    y = to_np(bd.fused_linear_geglu(to_dev(x, dtype), to_dev(w, dtype), to_dev(b, dtype)))
    # x Phi(x) with Phi from the complementary error function in double (scipy): 1 + erf loses the left tail to cancellation,
    # in the checker's double arithmetic beyond x = -7 and in the reference's FP32 beyond x = -5.5, where it returns 0
    from scipy.special import erfc
    g64 = gates.astype(np.float64)
    ref = np.tile((0.5 * g64 * erfc(-g64 / np.sqrt(2.0)))[None, :], (B, 1))
    assert np.isfinite(y).all()
    assert np.all(np.abs(y - ref) <= 2.0 ** -8 * np.abs(ref) * 1.05 + 1e-37)   # one bf16 rounding, relative, at every magnitude
    near = np.abs(gates) <= 5.0                                               # where the checker's own formula is accurate
    chk = oracle.geglu_exact(np.tile(b[None, :], (B, 1)))
    assert np.all(np.abs(y[:, near] - chk[:, near]) <= 2.0 ** -8 * np.abs(chk[:, near]) * 1.05 + 1e-12)


def test_geglu_halves_and_errors(oracle):
    """Value half first, gate half second: a weight whose gate rows are zero and gate bias is large gives a * g."""
    dtype, B, d_in, d_out = "fp16", 64, 64, 64
    x = uniform(31, (B, d_in), 1.0, dtype, oracle)
    w = np.zeros((2 * d_out, d_in), np.float32)
    w[:d_out] = uniform(32, (d_out, d_in), 0.1, dtype, oracle)
    b = np.zeros(2 * d_out, np.float32)
    b[d_out:] = 8.0                                                        # gelu(8) = 8 to fp16 precision
    y = bd.fused_linear_geglu(to_dev(x, dtype), to_dev(w, dtype), to_dev(b, dtype))
    ref = oracle.round_to(oracle.linear(x, w[:d_out]) * np.float32(8.0), dtype)
    assert np.abs(to_np(y) - ref).max() <= 2.0 ** -10 * np.abs(ref).max()
    z = lambda *s: torch.zeros(*s, device="cuda", dtype=torch.float16)
    with pytest.raises(RuntimeError, match=r"W must be \(2\*D_out, D_in\)"):
        bd.fused_linear_geglu(z(4, 64), z(63, 64), z(63))
    with pytest.raises(RuntimeError, match="b must be"):
        bd.fused_linear_geglu(z(4, 64), z(64, 64), z(32))


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("rows,cols", [(10, 37), (64, 64), (8192, 320), (3, 1)])
def test_add_inplace_vec(oracle, dtype, rows, cols):
    y0 = uniform(31, (rows, cols), 1.0, dtype, oracle)
    x = uniform(32, (rows, cols), 1.0, dtype, oracle)
    y = to_dev(y0, dtype)
    bd.add_inplace_vec(y, to_dev(x, dtype))
    assert np.array_equal(to_np(y), oracle.round_to(y0 + x, dtype))        # one FP32 add, one rounding
    # an unaligned view (offset by one element) takes the scalar path and gives the same values
    buf = torch.zeros(rows * cols + 1, device="cuda", dtype=y.dtype)
    buf[1:] = to_dev(y0, dtype).reshape(-1)
    bd.add_inplace_vec(buf[1:], to_dev(x, dtype).reshape(-1))
    assert torch.equal(buf[1:].reshape(rows, cols), y) and buf[0] == 0


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
@pytest.mark.parametrize("rows,cols", [(13, 29), (48, 80), (8192, 320)])
def test_add_inplace_row_bias(oracle, dtype, rows, cols):
    y0 = uniform(41, (rows, cols), 1.0, dtype, oracle)
    b = uniform(42, (cols,), 0.5, dtype, oracle)
    y = to_dev(y0, dtype)
    bd.add_inplace_row_bias(y, to_dev(b, dtype).reshape(cols, 1))          # (cols, 1) and (1, cols) both accepted
    assert np.array_equal(to_np(y), oracle.round_to(y0 + b[None, :], dtype))
    with pytest.raises(RuntimeError, match="bias must hold"):
        bd.add_inplace_row_bias(y, to_dev(b, dtype)[:-1])
