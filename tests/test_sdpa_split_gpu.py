"""Key-axis split of the last round of work groups (mi_sdpa_args.split_scratch): a launch whose query tiles do not
fill the GPU a whole number of times cuts the tiles of the last round into pieces for all compute units and merges
the partial results. The split result must agree with the unsplit launch to rounding (each part's normalised output
is rounded to the storage type once more before the merge: at most 2 units in the last place) and with the CPU
checker to the usual tolerance (helpers.TOL)."""
import ctypes as C

import numpy as np
import pytest
import torch

import brodiffusion_amd as bd
from brodiffusion_amd import _capi as capi
from helpers import assert_close, randn, to_dev, to_np

pytestmark = pytest.mark.gpu


def max_ulp_diff(a, b):
    unit = 2.0 ** -8 if a.dtype == torch.bfloat16 else 2.0 ** -11
    return (a.float() - b.float()).abs().max().item() / (unit * max(1.0, b.float().abs().max().item()))


def split_bytes(q, k, v, H, **kw):
    """What the library says it needs for this call (0 = it would not split)."""
    a = capi.MiSdpaArgs()
    a.struct_size = C.sizeof(a)
    a.dtype = capi.MI_DTYPE_BF16 if q.dtype == torch.bfloat16 else capi.MI_DTYPE_F16
    a.q, a.k, a.v, a.o = q.data_ptr(), k.data_ptr(), v.data_ptr(), q.data_ptr()
    B = q.shape[0] if q.dim() == 3 else 1
    a.batch, a.num_heads, a.head_dim = B, H, q.shape[-1] // H
    a.q_len, a.kv_len = q.shape[-2], k.shape[-2]
    for key, val in kw.items():
        setattr(a, key, val)
    return int(capi.lib().mi_sdpa_split_scratch_bytes(C.byref(a)))


@pytest.mark.parametrize("dtype,B,H,d,Lq,Lk", [
    ("bf16", 1, 24, 128, 4096, 4096),    # 384 tiles on 256 compute units: the last round is half full, tiles cut in two
    ("bf16", 1, 24, 128, 3328, 3328),    # 312 tiles: a nearly empty last round, many parts per tile
    ("bf16", 2, 16, 72, 4352, 4352),     # head_dim 72, batch 2
    ("fp16", 1, 20, 128, 4500, 2500),    # ragged: last query tile partial, key count not a multiple of 64
])
def test_split_matches_unsplit_and_checker(oracle, dtype, B, H, d, Lq, Lk):
    q = randn(8101, (B, Lq, H * d), dtype)
    k, v = randn(8102, (B, Lk, H * d), dtype), randn(8103, (B, Lk, H * d), dtype)
    dq, dk, dv = to_dev(q, dtype), to_dev(k, dtype), to_dev(v, dtype)
    need = split_bytes(dq, dk, dv, H)
    assert need > 0, "this shape is expected to qualify for the split"
    plain = bd.sdpa_forward(dq, dk, dv, H, split_scratch=False)
    scratch = torch.full((need,), 0xFF, dtype=torch.uint8, device="cuda")      # stale NaN patterns must not matter
    split = bd.sdpa_forward(dq, dk, dv, H, split_scratch=scratch)
    assert max_ulp_diff(split, plain) <= 2.0
    # sampled rows against the checker (all heads, rows spread over every query tile and its edges)
    rows = np.unique(np.concatenate([np.arange(0, Lq, 97), np.arange(255, Lq, 256), np.arange(256, Lq, 256), [Lq - 1]])).astype(np.int32)
    for b in range(B):
        ref = oracle.sdpa(q[b], k[b], v[b], H, rows=rows)
        assert_close(ref[rows], to_np(split[b])[rows], dtype, f"split batch {b}")
    # the module's own scratch (default) gives the same bits as a lent one, call after call
    again = bd.sdpa_forward(dq, dk, dv, H)
    assert torch.equal(again, split)
    # one byte short: the library falls back to the unsplit launch
    short = bd.sdpa_forward(dq, dk, dv, H, split_scratch=scratch[: need - 16])
    assert torch.equal(short, plain)


def test_split_then_smaller_call_reuses_scratch(oracle):
    dtype, H, d = "bf16", 24, 128
    big = [to_dev(randn(8200 + i, (4096, H * d), dtype), dtype) for i in range(3)]
    small = [to_dev(randn(8210 + i, (3328, H * d), dtype), dtype) for i in range(3)]
    scratch = torch.empty(max(split_bytes(*big, H), split_bytes(*small, H)), dtype=torch.uint8, device="cuda")
    o_big = bd.sdpa_forward(*big, H, split_scratch=scratch)
    o_small = bd.sdpa_forward(*small, H, split_scratch=scratch)
    assert max_ulp_diff(o_small, bd.sdpa_forward(*small, H, split_scratch=False)) <= 2.0
    assert torch.equal(o_big, bd.sdpa_forward(*big, H, split_scratch=scratch))


def test_split_with_fused_q_rope_and_rotated_k_scratch(oracle):
    """The headline call: RoPE on Q while loading, K rotated into the caller's scratch, then the split launch."""
    dtype, H, d, txt, hp, wp = "bf16", 24, 128, 512, 56, 64
    L = txt + hp * wp
    assert L == 4096
    q, k, v = (to_dev(randn(8300 + i, (L, H * d), dtype), dtype) for i in range(3))
    cos, sin = bd.build_axial_rope_tables(txt, hp, wp, d, (16, 56, 56))
    kr = torch.empty_like(k)
    with_split = bd.sdpa_forward(q, k, v, H, rope_q=(cos, sin), rope_k=(cos, sin), rope_k_scratch=kr)
    without = bd.sdpa_forward(q, k, v, H, rope_q=(cos, sin), rope_k=(cos, sin), rope_k_scratch=kr, split_scratch=False)
    assert max_ulp_diff(with_split, without) <= 2.0


def test_calls_that_do_not_split():
    H, d = 24, 128
    q = torch.zeros(4608, H * d, device="cuda", dtype=torch.bfloat16)
    h = q[:4096]
    assert split_bytes(h, h, h, H) > 0
    assert split_bytes(q, q, q, H) == 0                                               # last round 22/32 full: runs faster unsplit
    assert split_bytes(h, h, h, H, mask_mode=capi.MI_MASK_CAUSAL) == 0                # masked: tiles differ in length
    assert split_bytes(q[:2304], q, q, H) == 0                                        # fewer tiles than compute units
    assert split_bytes(h, h, h, 32) == 0                                              # 512 tiles: two full rounds
    assert split_bytes(h, q[:512], q[:512], H) == 0                                   # 8 key tiles: nothing to gain
    q40 = torch.zeros(2, 4096, 320, device="cuda", dtype=torch.float16)
    assert split_bytes(q40, q40, q40, 8) == 0                                         # head_dim 40 runs on the kernel without split


def test_own_split_scratch_is_per_stream():
    """Two streams run split launches of different problems at the same time with the scratch the Python layer lends by
    itself: each stream has its own (a shared one would be written by both launches at once), and every result equals the
    one computed alone, bit for bit."""
    H, d = 24, 128
    probs = []
    for i, L in enumerate((3328, 4096)):
        q, k, v = (to_dev(randn(8300 + 3 * i + j, (1, L, H * d), "bf16"), "bf16") for j in range(3))
        assert split_bytes(q, k, v, H) > 0
        probs.append((q, k, v, bd.sdpa_forward(q, k, v, H)))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for _ in range(4):                      # alternate the submissions so that the launches overlap on the GPU
        for s, (q, k, v, _), o in zip(streams, probs, outs):
            with torch.cuda.stream(s):
                o.append(bd.sdpa_forward(q, k, v, H))
    torch.cuda.synchronize()
    from brodiffusion_amd import ops
    keys = [key for key in ops._split_scratch_cache if key[1] in {s.cuda_stream for s in streams}]
    assert len(keys) == 2 and ops._split_scratch_cache[keys[0]].data_ptr() != ops._split_scratch_cache[keys[1]].data_ptr()
    for (_, _, _, ref), o in zip(probs, outs):
        for got in o:
            assert torch.equal(got, ref)
