"""The operators make no allocation, host synchronisation or memset of their own, so a step built from them can be
captured in a HIP graph (the reference states this property for its fused step, include/brodiffusion/denoiser.h:155-163).
One graph holds a call of every family with caller-owned outputs and scratch; it is replayed several times on new input
values, with eager work and synchronisations in between, and every replay must reproduce the eager results bit for bit."""
import pytest
import torch

import brodiffusion_amd as bd

pytestmark = pytest.mark.gpu


def test_graph_replays_equal_eager():
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(77)
    rnd = lambda *s, dt=torch.bfloat16: torch.randn(*s, device=dev, generator=g).to(dt)
    H, d, txt, hp, wp = 4, 128, 64, 16, 32
    L = txt + hp * wp
    q, k, v = (rnd(L, H * d) for _ in range(3))
    cos, sin = bd.build_axial_rope_tables(txt, hp, wp, d, (16, 56, 56))
    o_joint, kr = torch.empty_like(q), torch.empty_like(k)
    # block-causal with a cached prefix
    kp, vp = rnd(96, H * d), rnd(96, H * d)
    mask = bd.SdpaMask.block_causal(96, [192, 384, L], [96 + 192, 96 + 384, 96 + L], [0, 0, 0])
    o_block = torch.empty_like(q)
    # linear attention with a lent scratch
    lq, lk, lv = (rnd(2, 512, 4 * 112) for _ in range(3))
    ws = torch.empty(2 * 4 * (112 * 112 + 112), dtype=torch.float32, device=dev)
    lsc = torch.empty(8 * ws.numel(), dtype=torch.float32, device=dev)
    o_lin = torch.empty_like(lq)
    # attention block with projections, GEGLU, adds
    C = 320
    x = rnd(2, 256, C, dt=torch.float16)
    wq, wk, wv, wo = (rnd(C, C, dt=torch.float16) / C ** 0.5 for _ in range(4))
    bo = rnd(C, dt=torch.float16)
    o_blk = torch.empty_like(x)
    scratch = torch.empty(bd.flash_attention_scratch_bytes(2, 256, 256, C, True), dtype=torch.uint8, device=dev)
    wg, bg = rnd(2 * 640, C, dt=torch.float16) / C ** 0.5, rnd(2 * 640, dt=torch.float16)
    o_ff = torch.empty(2 * 256, 640, dtype=torch.float16, device=dev)
    gain = (1 + 0.1 * rnd(d)).to(torch.bfloat16)
    o_hn = torch.empty_like(k)
    # a linear layer large enough for the 256 x 256-tile kernel
    xl, wl, bl = rnd(4608, 1024), rnd(3072, 1024) / 32, rnd(3072)
    o_big = torch.empty(4608, 3072, dtype=torch.bfloat16, device=dev)
    # the tile-walking GEMM forms: FF1 + GEGLU with 128-token tiles (at least two per compute unit) and a long contraction
    # over few tiles (FF2)
    xr = rnd(4096, C, dt=torch.float16)
    wr, br = rnd(2 * 1280, C, dt=torch.float16) / C ** 0.5, rnd(2 * 1280, dt=torch.float16)
    o_ring = torch.empty(4096, 1280, dtype=torch.float16, device=dev)
    x2, w2, b2 = rnd(512, 1280, dt=torch.float16), rnd(640, 1280, dt=torch.float16) / 36, rnd(640, dt=torch.float16)
    o_ff2 = torch.empty(512, 640, dtype=torch.float16, device=dev)

    def step():
        bd.joint_attention(q, k, v, cos, sin, d, H, out=o_joint, Kr=kr)
        bd.sdpa_forward(q, k, v, H, out=o_block, mask=mask, k_prefix=kp, v_prefix=vp, split_scratch=False)
        bd.linear_attention_relu_forward(lq, lk, lv, 4, out=o_lin, workspace=ws, scratch=lsc)
        bd.flash_attention_qkvo_forward(x, None, wq, None, wk, None, wv, None, wo, bo, None, 8, False, out=o_blk, scratch=scratch)
        bd.fused_linear_geglu(x.view(512, C), wg, bg, o_ff)
        bd.add_inplace_vec(o_blk, x)
        bd.headnorm_rope(k, gain, 1e-6, cos, sin, d, H, out=o_hn)
        bd.linear_batched(wl, bl, xl, o_big)
        bd.fused_linear_geglu(xr, wr, br, o_ring)
        bd.linear_batched(w2, b2, x2, o_ff2)

    outs = (o_joint, o_block, o_lin, o_blk, o_ff, o_hn, o_big, o_ring, o_ff2, ws)
    step()                                            # warm-up outside the capture (first-use set-up of the library)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for it in range(4):
        for t in (q, k, v, lq, lk, lv, x, xl, xr, x2):
            t.copy_(rnd(*t.shape, dt=t.dtype))        # eager work between the replays: new input values
        step()
        torch.cuda.synchronize()
        eager = [t.clone() for t in outs]
        for t in outs:
            t.fill_(float("nan")) if t.dtype != torch.float32 else t.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("joint", "block-causal", "linear attention", "attention block", "geglu", "headnorm", "large linear", "geglu, walked tiles", "ff2, walked tiles", "state"), eager, outs):
            assert torch.equal(a, b), f"replay {it}: {name} differs from the eager call"
