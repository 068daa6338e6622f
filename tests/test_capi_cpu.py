"""No-GPU checks of the boundary: the C-ABI library loads, exports every symbol the header declares,
the ctypes mirrors have the C struct sizes, and precondition failures are reported without a launch."""
import ctypes as C
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "mi_attention.h")


@pytest.fixture(scope="module")
def capi():
    from brodiffusion_amd import _capi
    if not os.path.exists(_capi.LIB_PATH):
        from brodiffusion_amd import build
        build.build()
    return _capi


def _declared():
    txt = open(HEADER).read()
    return re.findall(r"MI_API\s+[\w\s\*]+?\b(mi_\w+)\s*\(", txt)


def test_header_symbols_exported(capi):
    names = _declared()
    assert len(names) >= 15 and set(names) == set(capi.EXPORTS)
    lib = capi.lib()
    for n in names:
        assert getattr(lib, n) is not None
    assert b"gfx950" in lib.mi_version()


def test_struct_sizes_match_c(capi, tmp_path):
    src = tmp_path / "sz.c"
    src.write_text('#include "mi_attention.h"\n#include <stdio.h>\nint main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu\\n",'
                   'sizeof(mi_sdpa_args),sizeof(mi_rope_args),sizeof(mi_linear_attn_args),sizeof(mi_device_info_t),'
                   'sizeof(mi_headnorm_rope_args),sizeof(mi_scale_rows_args),sizeof(mi_attention_map_args),sizeof(mi_linear_args),'
                   'sizeof(mi_attn_block_args));return 0;}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", "-std=c99", "-I" + os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    sizes = [int(x) for x in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split()]
    assert sizes == [C.sizeof(capi.MiSdpaArgs), C.sizeof(capi.MiRopeArgs), C.sizeof(capi.MiLinearAttnArgs),
                     C.sizeof(capi.MiDeviceInfo), C.sizeof(capi.MiHeadnormRopeArgs), C.sizeof(capi.MiScaleRowsArgs),
                     C.sizeof(capi.MiAttentionMapArgs), C.sizeof(capi.MiLinearArgs), C.sizeof(capi.MiAttnBlockArgs)]


def test_argument_validation_without_launch(capi):
    lib = capi.lib()
    a = capi.MiSdpaArgs()
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "struct_size" in capi.last_error()
    a.struct_size = C.sizeof(capi.MiSdpaArgs)
    a.dtype, a.head_dim, a.num_heads, a.batch = capi.MI_DTYPE_BF16, 32, 2, 1
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "no kernel" in capi.last_error()
    a.head_dim = 128
    a.q_len = 0                                     # empty query: success, nothing launched
    assert lib.mi_sdpa_forward(C.byref(a)) == 0 and capi.last_error() == ""
    a.q_len, a.kv_len = 4, 4
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "must not be null" in capi.last_error()
    a.q = a.k = a.v = a.o = 0x1008                  # never dereferenced: alignment is checked first
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "16-byte aligned" in capi.last_error()
    a.q = a.k = a.v = a.o = 0x1000
    a.q_row_stride = 100
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "multiples of 8" in capi.last_error()
    a.q_row_stride = 0
    a.mask_mode = capi.MI_MASK_BLOCK_CAUSAL
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "n_segments" in capi.last_error()
    a.n_segments = 2
    a.seg_q_end[0], a.seg_q_end[1] = 3, 2
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "non-decreasing" in capi.last_error()
    a.seg_q_end[1] = 3
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "segments cover" in capi.last_error()
    a.mask_mode = 7
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "unknown mask_mode" in capi.last_error()
    a.mask_mode = 0
    a.num_kv_heads = 3
    assert lib.mi_sdpa_forward(C.byref(a)) == -1 and "does not divide" in capi.last_error()
    for hd in (40, 64, 72, 80, 96, 112, 128, 160):
        assert lib.mi_sdpa_supported(capi.MI_DTYPE_F16, hd) == 1 and lib.mi_sdpa_supported(capi.MI_DTYPE_BF16, hd) == 1
    assert lib.mi_sdpa_supported(capi.MI_DTYPE_BF16, 48) == 0 and lib.mi_sdpa_supported(3, 128) == 0

    r = capi.MiRopeArgs()
    r.struct_size = C.sizeof(capi.MiRopeArgs)
    r.rows, r.num_heads, r.head_dim, r.dtype = 4, 2, 7, capi.MI_DTYPE_BF16
    r.x = r.out = r.cos = r.sin = 0x1000
    assert lib.mi_rope_apply(C.byref(r)) == -1 and "even" in capi.last_error()

    l = capi.MiLinearAttnArgs()
    l.struct_size = C.sizeof(capi.MiLinearAttnArgs)
    l.dtype, l.head_dim, l.num_heads, l.batch, l.n_tokens = capi.MI_DTYPE_F16, 112, 2, 1, 8
    assert lib.mi_linear_attn_relu_forward(C.byref(l)) == -1 and "no kernel" in capi.last_error()
    l.dtype = capi.MI_DTYPE_BF16
    l.q = l.k = l.v = l.o = 0x1000
    assert lib.mi_linear_attn_relu_forward(C.byref(l)) == -1 and "workspace needs" in capi.last_error()
    assert lib.mi_linear_attn_workspace_bytes(2, 20, 112) == 2 * 20 * (112 * 112 + 112) * 4
    assert lib.mi_linear_attn_scratch_bytes(2, 20, 112) % lib.mi_linear_attn_workspace_bytes(2, 20, 112) == 0


def test_split_scratch_is_not_offered_to_calls_the_split_kernel_cannot_serve(capi):
    """The key-axis split of the last round exists in one kernel form only, which neither adds a logit bias nor writes
    the softmax denominators: a call that asks for either must be told 0 bytes, so that no host layer lends a scratch
    and sends it down that route. (No GPU: the planner assumes 256 compute units.)"""
    lib = capi.lib()
    a = capi.MiSdpaArgs()
    a.struct_size = C.sizeof(capi.MiSdpaArgs)
    a.dtype, a.batch, a.num_heads, a.head_dim, a.q_len, a.kv_len = capi.MI_DTYPE_BF16, 1, 24, 128, 2816, 2816
    a.q = a.k = a.v = a.o = 0x1000                  # never dereferenced: only the launch geometry is planned
    plain = lib.mi_sdpa_split_scratch_bytes(C.byref(a))
    assert plain > 0
    a.lse_out = 0x2000
    assert lib.mi_sdpa_split_scratch_bytes(C.byref(a)) == 0
    a.lse_out = None
    a.logit_bias, a.bias_q0, a.bias_cols = 0x3000, 512, 512
    assert lib.mi_sdpa_split_scratch_bytes(C.byref(a)) == 0
    a.logit_bias = None
    assert lib.mi_sdpa_split_scratch_bytes(C.byref(a)) == plain


def test_python_mirror_refuses_cpu_tensors():
    import torch
    import brodiffusion_amd as bd
    x = torch.zeros((8, 256), dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="flash_attention_forward: tensor is not on the GPU"):
        bd.flash_attention_forward(x, x, x, None, 2, False)
    with pytest.raises(RuntimeError, match="rope_apply: tensor is not on the GPU"):
        bd.rope_apply(x, torch.zeros(8, 64), torch.zeros(8, 64), 128, 2)
    with pytest.raises(RuntimeError, match="axes_dims_rope must sum"):
        bd.build_axial_rope_tables(4, 2, 2, 32, (8, 8, 8), device="cpu")
    cos, sin = bd.build_axial_rope_tables(3, 2, 2, 16, (4, 6, 6), device="cpu")
    import oracle
    oc, os_ = oracle.build_axial_rope_tables(3, 2, 2, 16, (4, 6, 6))
    assert abs(cos.numpy() - oc).max() < 1e-7 and abs(sin.numpy() - os_).max() < 1e-7


def test_qwen_rope_tables_host_builder():
    """The host-side 3-axis table builder (src/dit/qwenimage21_forward.cpp:124-200) against the checker's
    restatement and against positions worked out by hand."""
    import numpy as np
    import brodiffusion_amd as bd
    import oracle
    segs = [("text", 5), ("image", 3, 4), ("text", 2)]
    pos = bd.qwen_rope_positions(segs, 2, 3)
    # text 0..4 at (p,p,p); image 3x4 at frame 5, rows -2..0 (h0 = -(3 - 1)), cols -2..1; position then 5 + max(3,4) = 9;
    # text at 9, 10; target 2x3 at frame 11, rows -1..0, cols -2..0
    assert pos.shape == (3, 5 + 12 + 2 + 6)
    assert pos[:, 4].tolist() == [4, 4, 4] and pos[:, 5].tolist() == [5, -2, -2] and pos[:, 16].tolist() == [5, 0, 1]
    assert pos[:, 17].tolist() == [9, 9, 9] and pos[:, 19].tolist() == [11, -1, -2] and pos[:, 24].tolist() == [11, 0, 0]
    cos, sin = bd.build_qwen_rope_tables(segs, 2, 3, 16, (4, 6, 6), device="cpu")
    oc, os_ = oracle.build_qwen_rope_tables(segs, 2, 3, 16, axes=(4, 6, 6))
    assert cos.shape == oc.shape and abs(cos.numpy() - oc).max() < 1e-7 and abs(sin.numpy() - os_).max() < 1e-7
    # pair 1 of the height axis (dim 6) at height position -2: angle -2 * theta^(-2/6)
    ang = -2.0 * 10000.0 ** (-2.0 / 6.0)
    assert abs(cos[5, 2 + 1].item() - np.cos(ang)) < 1e-6 and abs(sin[5, 2 + 1].item() - np.sin(ang)) < 1e-6
    with pytest.raises(RuntimeError, match="axes_dims_rope"):
        bd.build_qwen_rope_tables(segs, 2, 3, 16, (4, 4, 4), device="cpu")


def test_host_cpp_layer_error_paths():
    from brodiffusion_amd import build
    if not os.path.exists(build.HOST_TEST):
        build.build_host()
    r = subprocess.run([build.HOST_TEST, "--cpu"], capture_output=True, text=True)
    assert r.returncode == 0 and "test_host_ops: OK" in r.stdout, r.stdout + r.stderr


def test_split_planning_arithmetic_brute_force():
    """tests/cpp/test_split_geo.cpp: the formulas that cut the last round of an attention launch into pieces (shared by
    the host planner and the kernels) against their definition, over 180 (tiles, key steps, slots) configurations."""
    from brodiffusion_amd import build
    if not os.path.exists(build.SPLIT_TEST):
        build.build_host()
    r = subprocess.run([build.SPLIT_TEST], capture_output=True, text=True)
    assert r.returncode == 0 and "test_split_geo: OK" in r.stdout, r.stdout + r.stderr
