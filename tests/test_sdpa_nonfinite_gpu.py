"""Non-finite inputs to softmax attention, on every kernel form, against the CPU checker, through the C ABI.

The reference's host loop (src/dit/common.cpp:269-293) does not guard against them: a NaN score makes the row's
denominator NaN (`denom > 0` is then false, inv = 0, and 0 * NaN = NaN), a +Inf score gives exp(Inf - Inf) = NaN the
same way, a -Inf score is an ordinary vanishing term; a NaN in V poisons its output column through `o += p * v`. The
reference's NaN probes (BRODIFFUSION_FLUX_NANCHECK, src/dit/flux.cpp:127, :787-797) rely on such values staying visible
downstream, so the kernels must not launder them: exactly the outputs the checker makes NaN must be NaN, and every other
output must meet the usual bound. (The library is compiled with -fno-honor-nans; these tests hold the softmax code to
the behaviour its comparisons assume.)
"""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import TOL, randn, to_dev, to_np

pytestmark = pytest.mark.gpu

KERNELS = {"auto": 0, "rows128": 1, "rows256": 2, "rows256_regs": 3}


@pytest.fixture(autouse=True, params=list(KERNELS))
def kernel_choice(request):
    bd.set_sdpa_kernel_choice(KERNELS[request.param])
    yield request.param
    bd.set_sdpa_kernel_choice(0)


def _check(ref, got, dtype, what, expect_nan_rows=None):
    """Same NaN pattern; finite entries within the parity bound."""
    nan_ref, nan_got = np.isnan(ref), np.isnan(got)
    assert np.array_equal(nan_ref, nan_got), (f"{what}: NaN pattern differs: checker {nan_ref.sum()} NaN outputs, GPU {nan_got.sum()}; "
                                              f"first differing index {np.argwhere(nan_ref != nan_got)[:1]}")
    if expect_nan_rows is not None:
        assert nan_ref.any(axis=1).sum() == expect_nan_rows, f"{what}: the case was meant to poison {expect_nan_rows} rows, the checker has {nan_ref.any(axis=1).sum()}"
    ok = ~nan_ref
    assert np.isfinite(got[ok]).all(), f"{what}: infinite output where the checker is finite"
    rel, mx = TOL[dtype]
    r, g = ref[ok].astype(np.float64), got[ok].astype(np.float64)
    rel_l2 = np.linalg.norm(r - g) / (np.linalg.norm(r) + 1e-300)
    assert rel_l2 <= rel and np.max(np.abs(r - g), initial=0.0) <= mx, f"{what}: rel_l2 {rel_l2:.3e}, max_abs {np.max(np.abs(r - g)):.3e}"


def _run(q, k, v, H, dtype, **kw):
    return to_np(bd.sdpa_forward(to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype), H, **kw))


CASES = [("bf16", 128), ("bf16", 72), ("fp16", 40), ("fp16", 64)]


@pytest.mark.parametrize("dtype,d", CASES)
@pytest.mark.parametrize("value", [np.nan, np.inf, -np.inf])
def test_nonfinite_query_element(oracle, dtype, d, value):
    """One element of one query row: only that row of that head is affected (NaN: every score of the row; +-Inf: scores of
    +-Inf by the sign of the key's element, and one +Inf is enough for a NaN row)."""
    H, Lq, Lk = 2, 300, 640
    q, k, v = randn(400 + d, (Lq, H * d), dtype), randn(401 + d, (Lk, H * d), dtype), randn(402 + d, (Lk, H * d), dtype)
    q[37, d + 3] = value      # head 1
    q[299, 5] = value         # head 0, last row of a partly filled tile
    ref = oracle.sdpa(q, k, v, H)
    assert np.isnan(ref[37, d:]).all() and np.isnan(ref[299, :d]).all() and not np.isnan(ref[37, :d]).any()
    _check(ref, _run(q, k, v, H, dtype), dtype, f"d={d} query element {value}", expect_nan_rows=2)
    # the masked instances of the same kernels
    vl = torch.tensor([600], dtype=torch.int32, device="cuda")
    _check(oracle.sdpa(q, k[:600], v[:600], H), _run(q, k, v, H, dtype, kv_valid_len=vl), dtype, f"d={d} query element {value}, valid_len")


@pytest.mark.parametrize("dtype,d", CASES)
def test_nan_key_element(oracle, dtype, d):
    """A NaN in one key row makes that key's score NaN for every query of the head: the whole head is NaN, the other is not."""
    H, Lq, Lk = 2, 300, 640
    q, k, v = randn(410 + d, (Lq, H * d), dtype), randn(411 + d, (Lk, H * d), dtype), randn(412 + d, (Lk, H * d), dtype)
    k[130, d + 7] = np.nan
    ref = oracle.sdpa(q, k, v, H)
    assert np.isnan(ref[:, d:]).all() and not np.isnan(ref[:, :d]).any()
    _check(ref, _run(q, k, v, H, dtype), dtype, f"d={d} NaN key")
    # a causal mask hides key 130 from the rows before it: they stay finite
    lo, hi = oracle.rows_causal(Lq, Lk, q_offset=0)
    got = _run(q, k, v, H, dtype, mask=bd.SdpaMask.causal(0))
    ref = oracle.sdpa(q, k, v, H, row_lo=lo, row_hi=hi)
    assert not np.isnan(ref[:130]).any() and np.isnan(ref[130:, d:]).all()
    _check(ref, got, dtype, f"d={d} NaN key, causal")


@pytest.mark.parametrize("dtype,d", CASES)
@pytest.mark.parametrize("value", [np.inf, -np.inf])
def test_infinite_key_element(oracle, dtype, d, value):
    """+-Inf in one key element: the key's score is +Inf for the queries whose matching element has the same sign (NaN
    rows) and -Inf for the others, which simply do not see the key."""
    H, Lq, Lk = 2, 300, 640
    q, k, v = randn(420 + d, (Lq, H * d), dtype), randn(421 + d, (Lk, H * d), dtype), randn(422 + d, (Lk, H * d), dtype)
    k[77, 9] = value          # head 0
    ref = oracle.sdpa(q, k, v, H)
    n_nan = int(np.isnan(ref[:, 0]).sum())
    assert 0 < n_nan < Lq and not np.isnan(ref[:, d:]).any()
    _check(ref, _run(q, k, v, H, dtype), dtype, f"d={d} key element {value}")


@pytest.mark.parametrize("dtype,d", CASES)
def test_nan_value_element(oracle, dtype, d):
    """A NaN in V reaches one output column of one head, in every row that sees the key."""
    H, Lq, Lk = 2, 300, 640
    q, k, v = randn(430 + d, (Lq, H * d), dtype), randn(431 + d, (Lk, H * d), dtype), randn(432 + d, (Lk, H * d), dtype)
    v[500, d + 11] = np.nan
    ref = oracle.sdpa(q, k, v, H)
    assert np.isnan(ref[:, d + 11]).all() and np.isnan(ref).sum() == Lq
    _check(ref, _run(q, k, v, H, dtype), dtype, f"d={d} NaN value")


def test_short_key_kernel_nonfinite(oracle, kernel_choice):
    """The cross-attention shape that takes the short-key kernel when the kernel is chosen by size."""
    dtype, B, H, d, Lq, Lk = "bf16", 2, 16, 72, 2048, 300
    q, k, v = randn(440, (B, Lq, H * d), dtype), randn(441, (B, Lk, H * d), dtype), randn(442, (B, Lk, H * d), dtype)
    q[0, 100, 3 * d + 1] = np.nan
    q[1, 2047, 5] = np.inf
    k[1, 40, 2 * d + 2] = np.nan
    k[0, 290, 7 * d] = np.nan       # beyond the valid length of batch item 0: never seen
    valid = [77, 221]
    vl = torch.tensor(valid, dtype=torch.int32, device="cuda")
    out = _run(q, k, v, H, dtype, kv_valid_len=vl)
    rows = np.unique(np.concatenate([np.arange(0, Lq, 9), [100, 2047]])).astype(np.int32)
    for b in range(B):
        ref = oracle.sdpa(q[b], k[b, :valid[b]], v[b, :valid[b]], H, rows=rows)
        _check(ref[rows], out[b][rows], dtype, f"short keys, batch {b}")
    assert np.isnan(out[0, 100, 3 * d:4 * d]).all() and not np.isnan(out[0, :, 7 * d:8 * d]).any()
    assert np.isnan(out[1, :, 2 * d:3 * d]).all()


def test_split_launch_nonfinite(oracle, kernel_choice):
    """The launch whose last round is cut along the key axis: a NaN row must survive the merge of its parts, and a part
    that is all NaN must not leak into the rows of other tiles."""
    if kernel_choice not in ("auto", "rows256"):
        pytest.skip("the split belongs to the DMA kernel")
    dtype, H, d, L = "bf16", 24, 128, 2816
    q, k, v = randn(450, (L, H * d), dtype), randn(451, (L, H * d), dtype), randn(452, (L, H * d), dtype)
    q[2700, 23 * d + 4] = np.nan          # a row of the last round (the highest logical tiles)
    q[5, 0] = np.inf
    out = _run(q, k, v, H, dtype)
    rows = np.unique(np.concatenate([np.arange(3, L, 41), [5, 2700]])).astype(np.int32)
    ref = oracle.sdpa(q, k, v, H, rows=rows)
    _check(ref[rows], out[rows], dtype, "split launch")
    assert np.isnan(out[2700, 23 * d:]).all() and np.isnan(out[5, :d]).all()
    assert np.isnan(out).any(axis=1).sum() == 2
