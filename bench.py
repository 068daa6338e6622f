#!/usr/bin/env python3
"""Attention hot-path benchmark on one MI355X.

A step is one call of the hot path on the headline workload: Flux.1 double-stream joint attention,
B=1, H=24, head_dim=128, 512 text + 4096 image tokens, bf16, RoPE (axes 16/56/56, theta 1e4) applied
to Q and K inside the attention launch. Inputs are synthetic N(0,1) from the seeded generator the reference's
harnesses use (torch_randn_f32 of include/brodiffusion/detail/torch_rng.h = torch's CPU generator; configuration c
takes seeds 1000 c + 1, + 2, + 3 for Q, K, V), rounded once to the GPU dtype and resident in HBM before the timed
region. Prints ONE JSON line.

  metric      attention TFLOP/s, algorithmic FLOPs = 4 * B * H * Lq * Lk * d (QK^T and PV, nothing else)
  roofline    the flash kernel against MI355X dense bf16 MFMA peak (2.5 PFLOP/s), kernel time from HIP
              events on the launch stream over the timed region
  cpu_baseline the CPU checker (a port of the reference's FP32/FP64 host attention loop) timed on this
              host's cores on a bounded sample of the same workload (all threads, and one thread), the GPU
              result of the timed step compared with it on the sampled rows, and the same for every configuration
  configs     ms per call and TFLOP/s (GB/s for linear attention) of every benchmark configuration, measured
              outside the timed region
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_MFMA_BF16_TFLOPS = 2500.0   # MI355X dense bf16 / fp16 MFMA, published
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E, published
# HBM bytes per launch of the headline kernel. Not measured in this run: a constant taken from rocprofv3 --pmc FETCH_SIZE /
# WRITE_SIZE runs of `bench.py --traffic-probe` (counter values and calibration in the file named below):
# (FETCH_SIZE KiB x 2.00 calibration) fetched + WRITE_SIZE KiB written.
TRAFFIC_BYTES_PER_LAUNCH = (69300 * 2 + 27648) * 1024
TRAFFIC_SOURCE = "profiles/sdpa_fwd_pp_dma_bf16_flux_joint_4608_hbm_traffic.txt"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true")
    ap.add_argument("--traffic-probe", action="store_true",
                    help="few launches of the headline step and of cfg5 plus one 256 MiB tensor copy; run under rocprofv3 --pmc "
                         "FETCH_SIZE (or WRITE_SIZE): the copy calibrates the counter, the step gives HBM bytes per launch")
    return ap.parse_args()


PREHEAT_S = 0.15   # the GPU clock needs ~50 ms of sustained load to settle (kernel time falls ~20% over it)


def preheat(torch, fn, seconds=PREHEAT_S):
    """Untimed launches of `fn` for `seconds` of wall time so that measurements start at settled clocks."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def event_ms(torch, fn, iters, warm=0.05):
    """Per-call milliseconds (min, mean) from HIP events on the current stream."""
    preheat(torch, fn, warm)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(iters)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    ts = [a.elapsed_time(b) for a, b in evs]
    return min(ts), sum(ts) / len(ts)


def graph_ms(torch, fn, calls=20, reps=5):
    """Per-call milliseconds of `fn` as the GPU sees it: `calls` calls captured into one HIP graph, the replay timed with
    events (min over `reps` replays). For calls of a few microseconds the event timing above measures how fast Python
    submits them, not how long the GPU takes. None if the call cannot be captured."""
    try:
        fn()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(calls):
                fn()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        best = None
        for _ in range(reps):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            g.replay()
            b.record()
            torch.cuda.synchronize()
            t = a.elapsed_time(b) / calls
            best = t if best is None else min(best, t)
        return round(best, 4)
    except Exception as e:   # a failed capture must not take the benchmark line with it
        sys.stderr.write("graph timing skipped: %s\n" % e)
        return None


def calibration(torch, bd):
    """What the matrix pipes of this box sustain right now: a bare v_mfma_f32_32x32x16_bf16 loop on every compute unit
    (mi_mfma_probe) with all-zero and with N(0,1) operands, after the same preheat as the timed step. The clock is
    power-managed, so the two differ, and boxes differ; MFMA-bound rows can be divided by the N(0,1) figure."""
    g = torch.Generator(device="cuda").manual_seed(77)
    rnd = torch.randn(1 << 20, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
    res = {"what": "bare v_mfma_f32_32x32x16_bf16 loop on all compute units (mi_mfma_probe), 8 wavefronts per work group, 2 work groups per CU"}
    for name, ops in (("zeros", torch.zeros_like(rnd)), ("randn", rnd)):
        preheat(torch, lambda: bd.mfma_probe(ops, trips=500, reps=1), 0.1)
        r = bd.mfma_probe(ops, trips=4000, reps=5)
        res[f"mfma_loop_{name}_tflops"] = round(r["tflops"], 1)
        res[f"mfma_loop_{name}_shader_mhz"] = round(r["shader_mhz"], 0)
    return res


def seeded(torch, seed, shape, dtype):
    """N(0,1) values of torch's CPU generator for `seed` (what torch_randn_f32(seed, n) of the reference's torch_rng.h
    reproduces), rounded once to `dtype`, on the GPU."""
    n = 1
    for e in shape:
        n *= e
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, generator=g, dtype=torch.float32).reshape(shape).to(dtype).cuda()


def config_inputs(torch):
    """Q, K, V (and what else a call takes) of the benchmark configurations other than the headline one."""
    f16, b16 = torch.float16, torch.bfloat16
    c = {}
    c["cfg1"] = tuple(seeded(torch, 1000 + i, (2, 4096, 320), f16) for i in (1, 2, 3))
    c["cfg2a"] = tuple(seeded(torch, 2000 + i, (2, 4096, 1152), b16) for i in (1, 2, 3))
    # text keys / values from seeds 2011 / 2012, valid length of batch item b = 20 + (first output of std::mt19937(2099 + b)) % 281:
    # the tensors tests/test_baseline_configs_gpu.py checks (numpy's legacy seeding is the same init_genrand)
    import numpy as np
    valid = [20 + int(np.random.RandomState(2099 + b).randint(0, 2 ** 32, dtype=np.uint64)) % 281 for b in range(2)]
    c["cfg2b"] = (c["cfg2a"][0], seeded(torch, 2011, (2, 300, 1152), b16), seeded(torch, 2012, (2, 300, 1152), b16), valid)
    c["cfg4"] = (seeded(torch, 4001, (4096, 3072), b16), seeded(torch, 4002, (4608, 3072), b16), seeded(torch, 4003, (4608, 3072), b16))
    c["cfg5a"] = tuple(seeded(torch, 5000 + i, (2, 1024, 2240), b16) for i in (1, 2, 3))
    c["cfg5b"] = tuple(seeded(torch, 5010 + i, (2, 4096, 2240), b16) for i in (1, 2, 3))
    return c


def all_configs(torch, bd, cin, keep):
    """Every benchmark configuration: ms per call (min and mean over 20 calls), TFLOP/s or GB/s, fraction of peak."""
    g = torch.Generator(device="cuda").manual_seed(1234)

    def rnd(*shape, dt=torch.bfloat16):
        return torch.randn(*shape, device="cuda", dtype=torch.float32, generator=g).to(dt)

    out = {}

    def sdpa_entry(name, flops, fn, dtype, hbm_bytes=None):
        """hbm_bytes: algorithmic bytes of a call that sits below the ridge (~312 FLOP/B) and is therefore bound by HBM,
        not by the matrix pipes; such a row also carries GB/s and its fraction of the HBM peak (from the graph time: a
        call this short is submitted more slowly than it runs)."""
        mn, av = event_ms(torch, fn, 20)
        out[name] = {"ms_min": round(mn, 4), "ms_mean": round(av, 4), "tflops": round(flops / (mn * 1e-3) / 1e12, 1),
                     "frac_mfma_peak": round(flops / (mn * 1e-3) / 1e12 / PEAK_MFMA_BF16_TFLOPS, 4), "dtype": dtype,
                     "gflop": round(flops / 1e9, 2), "ms_graph": graph_ms(torch, fn)}
        if hbm_bytes is not None:
            t = out[name]["ms_graph"] or mn
            out[name].update({"bound": "hbm", "mbytes": round(hbm_bytes / 1e6, 2), "flop_per_byte": round(flops / hbm_bytes, 1),
                              "gbs": round(hbm_bytes / (t * 1e-3) / 1e9, 1), "frac_hbm_peak": round(hbm_bytes / (t * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)})

    q, k, v = cin["cfg1"]
    o1 = torch.empty_like(q)
    sdpa_entry("cfg1_sd15_selfattn_d40_fp16", 4 * 2 * 8 * 4096 * 4096 * 40, lambda: bd.flash_attention_forward(q, k, v, None, 8, False, out=o1), "fp16")
    keep["cfg1"] = o1
    # the same attention inside the U-Net block: Q/K/V projections (one launch), attention, output projection
    x, ctx = rnd(2, 4096, 320, dt=torch.float16), rnd(2, 77, 768, dt=torch.float16)
    wq, wk, wv, wo = (rnd(320, 320, dt=torch.float16) / 320 ** 0.5 for _ in range(4))
    wk2, wv2 = (rnd(320, 768, dt=torch.float16) / 768 ** 0.5 for _ in range(2))
    bo = rnd(320, dt=torch.float16)
    blk_out = torch.empty_like(x)
    blk_scratch = torch.empty(bd.flash_attention_scratch_bytes(2, 4096, 4096, 320, True), dtype=torch.uint8, device="cuda")
    sdpa_entry("sd15_unet_block_selfattn_qkvo_c320_fp16", 4 * 2 * 8 * 4096 * 4096 * 40 + 4 * 2 * 8192 * 320 * 320,
               lambda: bd.flash_attention_qkvo_forward(x, None, wq, None, wk, None, wv, None, wo, bo, None, 8, False, out=blk_out, scratch=blk_scratch), "fp16")
    kc1, vc1 = bd.flash_attention_project_kv(ctx, wk2, None, wv2, None)
    sdpa_entry("sd15_unet_block_crossattn_kvcached_c320_fp16", 4 * 2 * 8 * 4096 * 77 * 40 + 2 * 2 * 8192 * 320 * 320,
               lambda: bd.flash_attention_q_with_kv_cached_forward(x, kc1, vc1, wq, None, wo, bo, None, 8, False, out=blk_out, scratch=blk_scratch), "fp16",
               # x in, Q out and in, attention out and in, block out (6 passes over 8192 x 320) + K / V + the two weights
               hbm_bytes=2 * (6 * 8192 * 320 + 2 * 2 * 77 * 320 + 2 * 320 * 320))
    x2 = x.view(8192, 320)
    y2 = torch.empty(8192, 320, dtype=torch.float16, device="cuda")
    sdpa_entry("linear_8192x320x320_fp16", 2 * 8192 * 320 * 320, lambda: bd.linear_batched(wo, bo, x2, y2), "fp16")
    xl, wl = rnd(4608, 3072), rnd(3072, 3072) / 3072 ** 0.5
    yl = torch.empty(4608, 3072, dtype=torch.bfloat16, device="cuda")
    sdpa_entry("linear_4608x3072x3072_bf16", 2 * 4608 * 3072 * 3072, lambda: bd.linear_batched(wl, None, xl, yl), "bf16")
    del xl, wl, yl
    # FF1 + exact GEGLU of the same block: 8192 tokens, 320 -> 2 x 1280
    wg_, bg_ = rnd(2560, 320, dt=torch.float16) / 320 ** 0.5, rnd(2560, dt=torch.float16)
    yg_ = torch.empty(8192, 1280, dtype=torch.float16, device="cuda")
    sdpa_entry("sd15_unet_block_ff1_geglu_8192x320x2560_fp16", 2 * 8192 * 2560 * 320, lambda: bd.fused_linear_geglu(x2, wg_, bg_, yg_), "fp16")
    q, k, v = cin["cfg2a"]
    o2a = torch.empty_like(q)
    sdpa_entry("cfg2a_pixart_selfattn_d72_bf16", 4 * 2 * 16 * 4096 * 4096 * 72, lambda: bd.flash_attention_forward(q, k, v, None, 16, False, out=o2a), "bf16")
    keep["cfg2a"] = o2a
    _, kc, vc, valid = cin["cfg2b"]
    vl = torch.tensor(valid, dtype=torch.int32, device="cuda")
    o2b = torch.empty_like(q)
    sdpa_entry("cfg2b_pixart_crossattn_d72_bf16", 4 * 16 * 4096 * sum(valid) * 72, lambda: bd.sdpa_forward(q, kc, vc, 16, kv_valid_len=vl, out=o2b), "bf16",
               hbm_bytes=2 * (2 * q.numel() + 2 * sum(valid) * 1152))    # Q in, O out, the valid K and V rows
    out["cfg2b_pixart_crossattn_d72_bf16"]["valid_len"] = valid
    keep["cfg2b"] = o2b
    q, k, v = (rnd(4608, 3072) for _ in range(3))
    cos, sin = bd.build_axial_rope_tables(512, 64, 64, 128, (16, 56, 56))
    kr3 = torch.empty_like(k)
    sdpa_entry("cfg3_flux_joint_d128_bf16_rope", 4 * 24 * 4608 * 4608 * 128, lambda: bd.joint_attention(q, k, v, cos, sin, 128, 24, Kr=kr3), "bf16")
    out["cfg3_flux_joint_d128_bf16_rope_fused_k"] = None
    sdpa_entry("cfg3_flux_joint_d128_bf16_rope_fused_k", 4 * 24 * 4608 * 4608 * 128, lambda: bd.joint_attention(q, k, v, cos, sin, 128, 24), "bf16")
    qb, kall, vall = cin["cfg4"]                       # keys: 512 cached prefix rows (their own buffers), then 4096 fresh rows
    kp, vp, kb, vb = kall[:512].clone(), vall[:512].clone(), kall[512:].clone(), vall[512:].clone()
    sq = [1024, 2048, 3072, 4096]
    sk = [512 + e for e in sq]
    mask = bd.SdpaMask.block_causal(512, sq, sk, [0] * 4)
    o4 = torch.empty_like(qb)
    sdpa_entry("cfg4_qwen_blockcausal_prefixkv_d128_bf16", 4 * 24 * sum(1024 * e for e in sk) * 128,
               lambda: bd.sdpa_forward(qb, kb, vb, 24, k_prefix=kp, v_prefix=vp, mask=mask, out=o4), "bf16")
    keep["cfg4"] = o4
    out["cfg4_qwen_blockcausal_prefixkv_d128_bf16"]["dense_equivalent_gflop"] = round(4 * 24 * 4096 * 4608 * 128 / 1e9, 2)
    # dit::joint_attention_traced at Flux size (src/dit/common.cpp:198-329): RoPE of Q and K, attention with the image->text
    # logit bias and the softmax denominators, the head-averaged (L, L) map; and the attention launch of that call alone
    tb = rnd(4096, 512, dt=torch.float32) * 0.5
    o3x = torch.empty_like(q)
    qr3, tmap, lse3 = torch.empty_like(q), torch.empty(4608, 4608, dtype=torch.float32, device="cuda"), torch.empty(24, 4608, dtype=torch.float32, device="cuda")
    sdpa_entry("flux_joint_attention_traced_bias_map_d128_bf16", 2 * 4 * 24 * 4608 * 4608 * 128 - 2 * 24 * 4608 * 4608 * 128,
               lambda: bd.joint_attention_traced(q, k, v, cos, sin, 128, 24, out=o3x, attn_avg=tmap, Qr=qr3, Kr=kr3, txt_len=512, image_text_bias=tb), "bf16")
    out["flux_joint_attention_traced_bias_map_d128_bf16"]["note"] = "FLOPs: attention (QK^T, PV) + the map's second QK^T"
    sdpa_entry("flux_traced_attention_half_bias_lse_d128_bf16", 4 * 24 * 4608 * 4608 * 128,
               lambda: bd.sdpa_forward(qr3, kr3, v, 24, out=o3x, logit_bias=tb, bias_q0=512, lse_out=lse3), "bf16")
    del tmap, tb
    # dit::gqa_attention_masked at the shape the reference's kernel benchmark uses for it (tools/bench_krea2_kernels.cpp:78-79,
    # :179-192: 48 query heads, 12 K/V heads, head_dim 128, 512 text + 4096 image rows), key padding mask hiding text keys
    # 77..511; and the same call without a mask
    qg, kg, vg = rnd(4608, 48 * 128), rnd(4608, 12 * 128), rnd(4608, 12 * 128)
    og = torch.empty_like(qg)
    dm = torch.ones(4608, dtype=torch.float32, device="cuda")
    dm[77:512] = 0
    sdpa_entry("gqa_attention_masked_48q12kv_d128_L4608_bf16", 4 * 48 * 4608 * (4608 - 435) * 128,
               lambda: bd.gqa_attention_masked(qg, kg, vg, None, None, 128, 48, 12, dm, out=og), "bf16")
    sdpa_entry("gqa_attention_unmasked_48q12kv_d128_L4608_bf16", 4 * 48 * 4608 * 4608 * 128,
               lambda: bd.gqa_attention_masked(qg, kg, vg, None, None, 128, 48, 12, None, out=og), "bf16")
    del qg, kg, vg, og
    # bt::flash_attention_windowed_forward (src/dit/qwenimage21_forward.cpp:662): window 0 = causal, and a 1024-key window
    pairs_causal = 4608 * 4609 // 2
    pairs_win = sum(min(r + 1, 1024) for r in range(4608))
    sdpa_entry("windowed_causal_w0_d128_L4608_bf16", 4 * 24 * pairs_causal * 128, lambda: bd.flash_attention_windowed_forward(q, k, v, None, 24, 0, out=o3x), "bf16")
    sdpa_entry("windowed_w1024_d128_L4608_bf16", 4 * 24 * pairs_win * 128, lambda: bd.flash_attention_windowed_forward(q, k, v, None, 24, 1024, out=o3x), "bf16")
    xh, gh = rnd(4608, 3072), rnd(128)
    oh = torch.empty_like(xh)
    hn = lambda: bd.headnorm_rope(xh, gh, 1e-6, cos, sin, 128, 24, out=oh)   # noqa: E731
    mn, av = event_ms(torch, hn, 20)
    nbytes = 2 * xh.numel() * 2
    out["headnorm_rope_4608x24x128_bf16"] = {"ms_min": round(mn, 4), "ms_mean": round(av, 4), "gbs": round(nbytes / (mn * 1e-3) / 1e9, 1),
                                             "frac_hbm_peak": round(nbytes / (mn * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "dtype": "bf16",
                                             "mbytes": round(nbytes / 1e6, 2), "ms_graph": graph_ms(torch, hn)}
    # measured ceiling for the HBM-bound rows: a device-to-device copy of the size of cfg5b's four streams
    # (73.4 MB read + 73.4 MB written), by the same timing method
    csrc = torch.empty(73_400_320, dtype=torch.uint8, device="cuda").fill_(1)
    cdst = torch.empty_like(csrc)
    mn, av = event_ms(torch, lambda: cdst.copy_(csrc), 20)
    copy_gbs = 2 * csrc.numel() / (mn * 1e-3) / 1e9
    out["hbm_copy_ceiling_147mb"] = {"ms_min": round(mn, 4), "ms_mean": round(av, 4), "gbs": round(copy_gbs, 1),
                                     "frac_hbm_peak": round(copy_gbs / PEAK_HBM_GBS, 4)}
    del csrc, cdst
    for name, n, key in (("cfg5a_sana_linear_n1024_d112_bf16", 1024, "cfg5a"), ("cfg5b_sana_linear_n4096_d112_bf16", 4096, "cfg5b")):
        ql, kl, vl_ = cin[key]
        ws = torch.empty(40 * (112 * 112 + 112), dtype=torch.float32, device="cuda")
        sc = torch.empty(8 * ws.numel(), dtype=torch.float32, device="cuda")     # partial states (mi_linear_attn_scratch_bytes)
        o = torch.empty_like(ql)
        la = lambda: bd.linear_attention_relu_forward(ql, kl, vl_, 20, out=o, workspace=ws, scratch=sc)   # noqa: E731
        mn, av = event_ms(torch, la, 20)
        nbytes = 4 * 2 * n * 2240 * 2
        out[name] = {"ms_min": round(mn, 4), "ms_mean": round(av, 4), "gbs": round(nbytes / (mn * 1e-3) / 1e9, 1),
                     "frac_hbm_peak": round(nbytes / (mn * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     "frac_copy_ceiling": round(nbytes / (mn * 1e-3) / 1e9 / copy_gbs, 4), "dtype": "bf16 in, f32 accumulate",
                     "mbytes": round(nbytes / 1e6, 2), "ms_graph": graph_ms(torch, la)}
        keep[key] = o
        # the two kernel forms side by side (the row above is the library's own choice by size), and the same values as
        # (heads*head_dim, N) channel-major tensors, the layout of the reference's core (src/dit/sana.cpp:424-444)
        for form, tag in ((1, "three_launches"), (2, "one_launch")):
            out[name]["us_graph_" + tag] = round(1e3 * (graph_ms(torch, lambda: bd.linear_attention_relu_forward(
                ql, kl, vl_, 20, out=o, workspace=ws, scratch=sc, form=form)) or 0.0), 1)
        qc, kc_, vc_ = (t.transpose(1, 2).contiguous() for t in (ql, kl, vl_))
        oc = torch.empty_like(qc)
        out[name]["us_graph_channel_major"] = round(1e3 * (graph_ms(torch, lambda: bd.linear_attention_relu_forward_channel_major(
            qc, kc_, vc_, 20, out=oc, workspace=ws)) or 0.0), 1)
        bd.linear_attention_relu_forward(ql, kl, vl_, 20, out=o, workspace=ws, scratch=sc)     # `o` holds the by-size result again
        del qc, kc_, vc_, oc
    return out


def cpu_baseline(torch, headline, cin, keep):
    """The CPU checker (a port of the reference's host attention loop, src/dit/common.cpp:246-305, and of Sana's FP32 core,
    src/dit/sana.cpp:470-520) timed on this host on bounded samples of the same workloads, and the GPU results of this run
    compared with it on the sampled rows. Headline: RoPE on all of Q and K, then the exact attention loop for a subset of
    query rows (all heads, all 4608 keys; all rows where the host finishes them within ~12 s), once on all threads and
    once on one thread (~3 s). Every other configuration: one batch item on all threads (a few seconds each)."""
    import numpy as np
    import oracle as orc

    def host(t):
        return t.detach().float().cpu().numpy()

    def parity(ref, got, dtype):
        m = orc.compare(ref, got)
        rel, mx = (5e-3, 2e-2) if dtype == "bf16" else (1e-3, 5e-3)
        return {"rel_l2": float(f"{m['rel_l2']:.3e}"), "max_abs": float(f"{m['max_abs']:.3e}"), "within_tolerance": bool(m["rel_l2"] <= rel and m["max_abs"] <= mx)}

    threads = orc.max_threads()
    H, d, L = 24, 128, 4608
    q, k, v, cos, sin, out = headline
    q, k, v, cos, sin = host(q), host(k), host(v), host(cos), host(sin)
    probe = np.arange(0, L, L // 32, dtype=np.int32)[:32]
    t0 = time.perf_counter()
    orc.sdpa(q, k, v, H, rows=probe)
    per_row = (time.perf_counter() - t0) / len(probe)
    n_rows = int(max(64, min(L, 12.0 / max(per_row, 1e-6))))
    rows = np.unique(np.linspace(0, L - 1, n_rows).astype(np.int32))
    t0 = time.perf_counter()
    qr = orc.rope_apply(q, cos, sin, H, d, round_to_dtype="bf16")
    kr = orc.rope_apply(k, cos, sin, H, d, round_to_dtype="bf16")
    ref = orc.sdpa(qr, kr, v, H, rows=rows)
    dt = time.perf_counter() - t0
    flops = 4.0 * H * len(rows) * L * d
    res = {"value": round(flops / dt / 1e12, 5), "unit": "TFLOP/s", "cores": threads, "kind": "port",
           "sample": f"{len(rows)} of {L} query rows x 24 heads x all 4608 keys, RoPE on all of Q and K included, "
                     f"{dt:.1f} s on {threads} OpenMP threads; full call extrapolates to {dt * L / len(rows):.0f} s",
           "parity_of_timed_step": parity(ref[rows], host(out)[rows], "bf16")}
    # the faithful single-thread form of the same loop, on fewer rows
    per_row_1 = dt * threads / len(rows)                    # one thread's time per query row, about
    rows1 = rows[np.unique(np.linspace(0, len(rows) - 1, max(8, min(len(rows), int(3.0 / max(per_row_1, 1e-6))))).astype(np.int32))]
    t0 = time.perf_counter()
    orc.sdpa(qr, kr, v, H, rows=rows1, n_threads=1)
    dt1 = time.perf_counter() - t0
    res["single_thread"] = {"value": round(4.0 * H * len(rows1) * L * d / dt1 / 1e12, 5), "unit": "TFLOP/s", "cores": 1,
                            "sample": f"{len(rows1)} query rows x 24 heads x all keys (RoPE passes not included), {dt1:.1f} s on one thread; "
                                      f"full call extrapolates to {dt1 * L / len(rows1):.0f} s"}
    orc.sdpa(q[:8], k[:8], v[:8], H, n_threads=threads)      # back to all threads for what follows
    if cin is None:
        return res

    def sdpa_cfg(name, qh, kh, vh, Hc, dtype, gpu_rows, n_rows, **kw):
        Lq, Lk = qh.shape[0], kh.shape[0]
        rws = np.unique(np.linspace(0, Lq - 1, n_rows).astype(np.int32))
        t0 = time.perf_counter()
        r = orc.sdpa(qh, kh, vh, Hc, rows=rws, **kw)
        dtc = time.perf_counter() - t0
        hi = kw.get("row_hi")
        pairs = float(sum(int(hi[i]) for i in rws)) if hi is not None else float(len(rws)) * Lk
        all_pairs = float(np.sum(hi)) if hi is not None else float(Lq) * Lk
        dd = qh.shape[1] // Hc
        return {"value": round(4.0 * Hc * pairs * dd / dtc / 1e12, 5), "unit": "TFLOP/s", "cores": threads,
                "sample": f"{len(rws)} of {Lq} query rows of one batch item x {Hc} heads, {dtc:.2f} s; one batch item extrapolates to "
                          f"{dtc * all_pairs / pairs:.2f} s",
                "parity": parity(r[rws], gpu_rows[rws], dtype)}

    cfgs = {}
    q1, k1, v1 = (host(t[0]) for t in cin["cfg1"])
    cfgs["cfg1_sd15_selfattn_d40_fp16"] = sdpa_cfg("cfg1", q1, k1, v1, 8, "fp16", host(keep["cfg1"][0]), 4096)
    q2, k2, v2 = (host(t[0]) for t in cin["cfg2a"])
    cfgs["cfg2a_pixart_selfattn_d72_bf16"] = sdpa_cfg("cfg2a", q2, k2, v2, 16, "bf16", host(keep["cfg2a"][0]), 4096)
    valid = cin["cfg2b"][3]
    kc, vc = host(cin["cfg2b"][1][0])[:valid[0]], host(cin["cfg2b"][2][0])[:valid[0]]
    cfgs["cfg2b_pixart_crossattn_d72_bf16"] = sdpa_cfg("cfg2b", q2, kc, vc, 16, "bf16", host(keep["cfg2b"][0]), 4096)
    q4, k4, v4 = (host(t) for t in cin["cfg4"])
    sq = [1024, 2048, 3072, 4096]
    lo, hi = orc.rows_block_causal(4096, 4608, 512, sq, [512 + e for e in sq], [0] * 4)
    cfgs["cfg4_qwen_blockcausal_prefixkv_d128_bf16"] = sdpa_cfg("cfg4", q4, k4, v4, 24, "bf16", host(keep["cfg4"]), 4096, row_lo=lo, row_hi=hi)
    for name, key in (("cfg5a_sana_linear_n1024_d112_bf16", "cfg5a"), ("cfg5b_sana_linear_n4096_d112_bf16", "cfg5b")):
        ql, kl, vl = (host(t[0]) for t in cin[key])
        t0 = time.perf_counter()
        r = orc.linear_attn_relu(ql, kl, vl, 20)
        dtc = time.perf_counter() - t0
        nbytes = 4 * ql.size * 2
        cfgs[name] = {"value": round(nbytes / dtc / 1e9, 3), "unit": "GB/s", "cores": threads,
                      "sample": f"one of the 2 batch items, whole, {dtc:.2f} s (algorithmic bytes of the bf16 streams, as for the GPU figure)",
                      "parity": parity(r, host(keep[key][0]), "bf16")}
    res["configs"] = cfgs
    return res


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (got --gpus {args.gpus}): this attention path has no multi-GPU leg; "
              "heads shard across GPUs without exchange.", file=sys.stderr)
        sys.exit(2)
    import torch
    import brodiffusion_amd as bd
    from brodiffusion_amd import _capi
    _capi.lib()                              # fails loudly if the HIP extension is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)

    B, H, d, txt, hp, wp = 1, 24, 128, 512, 64, 64
    L = txt + hp * wp
    g = torch.Generator(device="cuda").manual_seed(3000)     # (probe tensors only)
    q, k, v = (seeded(torch, 3000 + i, (L, H * d), torch.bfloat16) for i in (1, 2, 3))
    cos, sin = bd.build_axial_rope_tables(txt, hp, wp, d, (16, 56, 56))
    out = torch.empty_like(q)
    kr = torch.empty_like(k)                 # the Kr scratch of the reference's joint_attention signature
    flops = 4.0 * B * H * L * L * d

    def step():
        bd.joint_attention(q, k, v, cos, sin, d, H, out=out, Kr=kr)

    if args.traffic_probe:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        # cfg5 (Sana ReLU linear attention, B=2 H=20 d=112 N=4096) rides along: its kernels are the HBM-bound ones
        lq, lk, lv = (torch.randn(2, 4096, 2240, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16) for _ in range(3))
        lo = torch.empty_like(lq)
        lws = torch.empty(2 * 20 * (112 * 112 + 112), dtype=torch.float32, device="cuda")
        lsc = torch.empty(8 * lws.numel(), dtype=torch.float32, device="cuda")
        # cfg5a (N=1024, the one-launch form) and cfg2b (PixArt cross attention, the short-key kernel) ride along as well
        sq, sk, sv = (torch.randn(2, 1024, 2240, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16) for _ in range(3))
        so = torch.empty_like(sq)
        cq = torch.randn(2, 4096, 1152, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
        ck, cv = (torch.randn(2, 300, 1152, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16) for _ in range(2))
        co = torch.empty_like(cq)
        cvl = torch.tensor([77, 105], dtype=torch.int32, device="cuda")
        zeros = torch.zeros(1 << 20, dtype=torch.bfloat16, device="cuda")
        noise = torch.randn(1 << 20, device="cuda", dtype=torch.float32, generator=g).to(torch.bfloat16)
        for _ in range(3):
            dst.copy_(src)
            step()
            bd.linear_attention_relu_forward(lq, lk, lv, 20, out=lo, workspace=lws, scratch=lsc)
            bd.linear_attention_relu_forward(sq, sk, sv, 20, out=so, workspace=lws, scratch=lsc)
            bd.sdpa_forward(cq, ck, cv, 16, kv_valid_len=cvl, out=co)
            bd.mfma_probe(zeros, trips=2000, reps=1)
            bd.mfma_probe(noise, trips=2000, reps=1)
        torch.cuda.synchronize()
        print(json.dumps({"traffic_probe": "3 x (256 MiB copy, headline step, Sana linear attention N=4096 and N=1024, PixArt cross attention, "
                                           "MFMA loop on zeros and on N(0,1))"}))
        return
    preheat(torch, step)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    step_ms_events = e0.elapsed_time(e1) / args.steps
    # the dominant kernel alone (attention with Q rotated on load, keys read from the rotated copy): the same
    # launch the step makes after its K rotation pass, back to back on this stream between two events
    e0.record()
    for _ in range(args.steps):
        bd.sdpa_forward(q, kr, v, H, out=out, rope_q=(cos, sin))
    e1.record()
    torch.cuda.synchronize()
    kernel_ms = e0.elapsed_time(e1) / args.steps

    ms_per_step = wall * 1e3 / args.steps
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    res = {
        "metric": "attention TFLOP/s + % of MI355X bf16 MFMA peak (Flux 4608-token SDPA)",
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "Flux.1 joint attention B=1 H=24 d=128 L=512+4096, RoPE axes 16/56/56 (Q rotated on load, K by one pass into the Kr scratch), non-causal",
                   "gflop_per_step": round(flops / 1e9, 2)},
        "pct_of_mfma_peak": round(100.0 * (flops / (ms_per_step * 1e-3) / 1e12) / PEAK_MFMA_BF16_TFLOPS, 2),
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_MFMA_BF16_TFLOPS, 4), "traffic": TRAFFIC_BYTES_PER_LAUNCH,
                     "traffic_source": "constant from counter runs, not measured in this run: " + TRAFFIC_SOURCE,
                     "kernel": "sdpa_fwd_pp_dma_kernel<__bf16, 128, dense>", "kernel_ms": round(kernel_ms, 4),
                     "step_ms_events": round(step_ms_events, 4)},
        "device": bd.device_info(),
    }
    cal = calibration(torch, bd)
    cal["headline_kernel_frac_of_randn_loop"] = round(achieved / cal["mfma_loop_randn_tflops"], 4)
    cal["headline_kernel_frac_of_zeros_loop"] = round(achieved / cal["mfma_loop_zeros_tflops"], 4)
    res["calibration"] = cal
    step()                                    # `out` holds the result of a step: compared with the checker below
    torch.cuda.synchronize()
    cin, keep = None, {}
    if not args.no_configs:
        cin = config_inputs(torch)
        res["configs"] = all_configs(torch, bd, cin, keep)
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(torch, (q, k, v, cos, sin, out), cin, keep)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
