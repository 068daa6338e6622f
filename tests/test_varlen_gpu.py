"""Packed variable-length attention (bt::flash_attention_varlen_forward, src/dit/krea2.cpp:574): every sequence must
equal an ordinary call on its own rows (same kernel, same bits), and the checker on those rows."""
import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def own_rows(*args, **kw):
    bd.set_sdpa_kernel_choice(1)      # the packed form runs on the 128-row kernel
    try:
        return bd.flash_attention_forward(*args, **kw)
    finally:
        bd.set_sdpa_kernel_choice(0)


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("dtype,H,d,q_lens,k_lens", [
    ("bf16", 4, 128, [5, 300, 1, 129, 64], [5, 300, 1, 129, 64]),       # self attention, ragged
    ("fp16", 8, 40, [200, 17, 128], [77, 300, 1]),                      # different query and key lengths
    ("bf16", 2, 72, [32] * 40, [32] * 40),                              # the reference's use: equal short sequences (krea2.cpp:561-576)
])
def test_varlen_equals_per_sequence_calls(oracle, dtype, H, d, q_lens, k_lens, causal):
    if causal and any(qn > kn for qn, kn in zip(q_lens, k_lens)):
        q_lens = [min(a, b) for a, b in zip(q_lens, k_lens)]
    cq, ck = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32), np.concatenate([[0], np.cumsum(k_lens)]).astype(np.int32)
    q = randn(9900, (int(cq[-1]), H * d), dtype)
    k, v = randn(9901, (int(ck[-1]), H * d), dtype), randn(9902, (int(ck[-1]), H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    out = bd.flash_attention_varlen_forward(dq, dk, dv, torch.from_numpy(cq).cuda(), torch.from_numpy(ck).cuda(), len(q_lens),
                                            max(q_lens), max(k_lens), H, d, causal)
    for i in range(len(q_lens)):
        qs, qe, ks, ke = cq[i], cq[i + 1], ck[i], ck[i + 1]
        alone = own_rows(dq[qs:qe], dk[ks:ke], dv[ks:ke], None, H, causal)
        assert torch.equal(out[qs:qe], alone), f"sequence {i}"
        if i < 3:
            lo = hi = None
            if causal:
                lo, hi = oracle.rows_causal(int(qe - qs), int(ke - ks))
            assert_close(oracle.sdpa(q[qs:qe], k[ks:ke], v[ks:ke], H, row_lo=lo, row_hi=hi), to_np(out[qs:qe]), dtype, f"sequence {i}")


def test_varlen_empty_sequence_and_errors():
    H, d = 2, 64
    q = torch.randn(20, H * d, device="cuda").bfloat16()
    cu = torch.tensor([0, 7, 7, 20], dtype=torch.int32, device="cuda")       # the middle sequence is empty
    out = bd.flash_attention_varlen_forward(q, q, q, cu, cu, 3, 13, 13, H, d, False)
    assert torch.equal(out[:7], own_rows(q[:7], q[:7], q[:7], None, H, False))
    assert torch.equal(out[7:], own_rows(q[7:], q[7:], q[7:], None, H, False))
    with pytest.raises(RuntimeError, match="n_seqs \\+ 1 offsets"):
        bd.flash_attention_varlen_forward(q, q, q, cu[:3], cu, 3, 13, 13, H, d, False)
    with pytest.raises(RuntimeError, match="int32"):
        bd.flash_attention_varlen_forward(q, q, q, cu.long(), cu, 3, 13, 13, H, d, False)
