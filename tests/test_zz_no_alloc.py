"""mi_linear_attn_relu_forward_static_scratch: the linear-attention entry point that allocates nothing and keeps its partial
states in a static device array of the library. Through the C ABI, against mi_linear_attn_relu_forward with a caller scratch
(same kernels, same split of the tokens: bit-identical output and state) and against the CPU checker; two calls in a row, the
second smaller, so that what the first call left in the array must not leak into the second."""
import ctypes as C

import numpy as np
import pytest
import torch

from brodiffusion_amd import _capi as capi
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def _args(q, k, v, o, ws, H, d, accumulate=False):
    B, N, _ = q.shape
    a = capi.MiLinearAttnArgs()
    a.struct_size = C.sizeof(capi.MiLinearAttnArgs)
    a.dtype = capi.MI_DTYPE_BF16
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr()
    a.batch, a.num_heads, a.head_dim, a.n_tokens = B, H, d, N
    a.eps = 1e-15
    a.accumulate_state = int(accumulate)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * 4
    a.form = capi.MI_LINEAR_ATTN_FORM_THREE_LAUNCHES      # the form whose partial states need the scratch this file is about
    a.stream = torch.cuda.current_stream().cuda_stream
    return a


def _both(oracle, B, H, d, N, seed, accumulate=False):
    lib = capi.lib()
    dtype = "bf16"
    q, k, v = (randn(seed + i, (B, N, H * d), dtype) for i in range(3))
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    need = lib.mi_linear_attn_workspace_bytes(B, H, d)
    assert 8 * need <= capi.MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES          # both routes may split 8 ways
    state0 = torch.from_numpy(randn(seed + 7, (need // 4,), "fp32")).cuda() if accumulate else torch.zeros(need // 4, device="cuda")
    # reference route: caller scratch of full size
    o_ref, ws_ref = torch.empty_like(dq), state0.clone()
    scratch = torch.empty(lib.mi_linear_attn_scratch_bytes(B, H, d) // 4, dtype=torch.float32, device="cuda")
    a = _args(dq, dk, dv, o_ref, ws_ref, H, d, accumulate)
    a.scratch, a.scratch_bytes = scratch.data_ptr(), scratch.numel() * 4
    assert lib.mi_linear_attn_relu_forward(C.byref(a)) == 0, capi.last_error()
    # static route: outputs prefilled so that an entry point that writes nothing cannot pass
    o_st, ws_st = torch.full_like(dq, 7.0), state0.clone()
    a = _args(dq, dk, dv, o_st, ws_st, H, d, accumulate)
    # the property the entry point exists for: no device memory is taken or returned during the call, neither through
    # torch's allocator nor behind its back (free device memory as the driver reports it)
    torch.cuda.synchronize()
    free0, held0 = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    assert lib.mi_linear_attn_relu_forward_static_scratch(C.byref(a)) == 0, capi.last_error()
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free0 and torch.cuda.memory_allocated() <= held0
    assert torch.equal(o_st, o_ref) and torch.equal(ws_st, ws_ref)
    if not accumulate:
        for b in range(B):
            assert_close(oracle.linear_attn_relu(q[b], k[b], v[b], H), to_np(o_st[b]), dtype, f"batch {b}")


def test_static_scratch_entry_point_two_calls_in_a_row(oracle):
    _both(oracle, 2, 20, 112, 1024, 9800)          # fills 8 partial slots per (batch, head)
    _both(oracle, 1, 6, 112, 300, 9810)            # smaller: fewer heads, fewer and shorter chunks, same array
    _both(oracle, 2, 70, 32, 512, 9820)            # another head_dim: the slots are laid out differently
    _both(oracle, 1, 6, 112, 300, 9830, accumulate=True)


def test_static_scratch_reduced_split(oracle):
    """A state of 5.3 MB: the 16 MiB array holds three partial states per (batch, head) instead of eight, so the tokens are
    split less far than with a caller scratch of full size and the two routes no longer add in the same order; the result
    is held to the checker instead."""
    lib = capi.lib()
    dtype, B, H, d, N = "bf16", 2, 40, 128, 1536
    need = lib.mi_linear_attn_workspace_bytes(B, H, d)
    assert 1 <= capi.MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES // need < 8
    q, k, v = (randn(9840 + i, (B, N, H * d), dtype) for i in range(3))
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    o, ws = torch.full_like(dq, 7.0), torch.zeros(need // 4, device="cuda")
    assert lib.mi_linear_attn_relu_forward_static_scratch(C.byref(_args(dq, dk, dv, o, ws, H, d))) == 0, capi.last_error()
    torch.cuda.synchronize()
    for b in range(B):
        assert_close(oracle.linear_attn_relu(q[b], k[b], v[b], H), to_np(o[b]), dtype, f"reduced split, batch {b}")


def test_static_scratch_entry_point_limits():
    lib = capi.lib()
    B, H, d, N = 8, 40, 128, 8                      # state 8 * 40 * (128 * 128 + 128) * 4 = 21 MB > 16 MiB
    x = torch.zeros((B, N, H * d), dtype=torch.bfloat16, device="cuda")
    o = torch.empty_like(x)
    ws = torch.zeros(lib.mi_linear_attn_workspace_bytes(B, H, d) // 4, device="cuda")
    a = _args(x, x, x, o, ws, H, d)
    assert lib.mi_linear_attn_relu_forward_static_scratch(C.byref(a)) == -1
    assert "static scratch holds 16777216" in capi.last_error()
    # the same problem is served by the entry point with a caller scratch (here: none lent, one work group per head)
    assert lib.mi_linear_attn_relu_forward(C.byref(a)) == 0, capi.last_error()
    torch.cuda.synchronize()
    assert not o.float().abs().max().item() > 0     # all-zero inputs: 0 / eps
    sc = torch.empty(16, device="cuda")
    a = _args(x[:1], x[:1], x[:1], o[:1], ws, H, d)
    a.scratch, a.scratch_bytes = sc.data_ptr(), 64
    assert lib.mi_linear_attn_relu_forward_static_scratch(C.byref(a)) == -1 and "takes no scratch" in capi.last_error()
