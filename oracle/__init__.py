"""TEST INFRASTRUCTURE ONLY: ctypes/numpy front end of the CPU checker (oracle.cpp).

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
package; the product (brodiffusion_amd) never does. All arrays are float32 numpy,
row-major (L, H*d) with head h in columns [h*d, (h+1)*d).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libref_rng.so")


def build(with_ref: bool | None = None) -> None:
    """Compile liboracle.so (and _ref/ when the reference tree is mounted)."""
    targets = ["all"]
    if with_ref is None:
        with_ref = os.path.isdir("/root/reference/include/brodiffusion")
    if with_ref:
        targets.append("ref")
    subprocess.run(["make", "-C", _HERE, "-B", *targets], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return C.CDLL(_LIB_PATH)


_lib = _load()
_f32p = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_u16p = np.ctypeslib.ndpointer(dtype=np.uint16, flags="C_CONTIGUOUS")

_lib.orc_torch_randn_f32.argtypes = [C.c_uint64, C.c_size_t, _f32p]
_lib.orc_torch_randn_f32.restype = C.c_int
for _n in ("orc_round_bf16", "orc_round_f16"):
    getattr(_lib, _n).argtypes = [_f32p, C.c_size_t]
    getattr(_lib, _n).restype = None
for _n in ("orc_f32_to_bf16_bits", "orc_f32_to_f16_bits"):
    getattr(_lib, _n).argtypes = [_f32p, C.c_size_t, _u16p]
    getattr(_lib, _n).restype = None
for _n in ("orc_bf16_bits_to_f32", "orc_f16_bits_to_f32"):
    getattr(_lib, _n).argtypes = [_u16p, C.c_size_t, _f32p]
    getattr(_lib, _n).restype = None
_lib.orc_build_axial_rope_tables.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, _i32p, C.c_int, C.c_float,
                                             _f32p, _f32p]
_lib.orc_build_axial_rope_tables.restype = C.c_int
_lib.orc_build_qwen_rope_tables.argtypes = [_i32p, _i32p, _i32p, C.c_int, C.c_int, C.c_int, C.c_int, _i32p,
                                            C.c_double, C.c_void_p, C.c_void_p]
_lib.orc_build_qwen_rope_tables.restype = C.c_int
_lib.orc_rope_apply.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f32p]
_lib.orc_rope_apply.restype = None
_lib.orc_sdpa.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_double,
                          C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                          C.c_void_p, C.c_int, _f32p, C.c_void_p, C.c_int]
_lib.orc_sdpa.restype = None
_lib.orc_rows_causal.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, _i32p, _i32p]
_lib.orc_rows_causal.restype = None
_lib.orc_rows_block_causal.argtypes = [C.c_int, C.c_int, C.c_int, _i32p, _i32p, _i32p, C.c_int, _i32p, _i32p]
_lib.orc_rows_block_causal.restype = None
_lib.orc_dense_block_causal.argtypes = [C.c_int, C.c_int, C.c_int, _i32p,
                                        np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")]
_lib.orc_dense_block_causal.restype = None
_lib.orc_linear_attn_relu.argtypes = [_f32p, _f32p, _f32p, C.c_int, C.c_int, C.c_int, C.c_float, _f32p,
                                      C.c_void_p, C.c_void_p, C.c_int]
_lib.orc_linear_attn_relu.restype = None
_lib.orc_rms_norm.argtypes = [_f32p, _f32p, C.c_double, C.c_int, C.c_int, _f32p]
_lib.orc_rms_norm.restype = None
_lib.orc_geglu_exact.argtypes = [_f32p, C.c_int, C.c_int, _f32p]
_lib.orc_geglu_exact.restype = None
_lib.orc_linear.argtypes = [_f32p, _f32p, C.c_void_p, C.c_int, C.c_int, C.c_int, _f32p, C.c_int]
_lib.orc_linear.restype = None
_lib.orc_max_threads.restype = C.c_int


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def max_threads() -> int:
    return int(_lib.orc_max_threads())


def torch_randn_f32(seed: int, n: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    if _lib.orc_torch_randn_f32(seed, n, out) != 0:
        raise ValueError("torch_randn_f32: n must be >= 16")
    return out


def ref_torch_randn_f32(seed: int, n: int) -> np.ndarray:
    """The reference's own header, compiled as is (oracle/_ref); raises if not built."""
    if not os.path.exists(_REF_PATH):
        raise FileNotFoundError(_REF_PATH)
    ref = C.CDLL(_REF_PATH)
    ref.ref_torch_randn_f32.argtypes = [C.c_uint64, C.c_size_t, _f32p]
    ref.ref_torch_randn_f32.restype = C.c_int
    out = np.empty(n, dtype=np.float32)
    if ref.ref_torch_randn_f32(seed, n, out) != 0:
        raise ValueError("reference torch_randn_f32 refused n")
    return out


def have_ref() -> bool:
    return os.path.exists(_REF_PATH)


def round_to(x: np.ndarray, dtype: str) -> np.ndarray:
    """Round float32 values to the nearest bf16 / fp16 value (ties to even), keep float32 storage."""
    y = _f32(x).copy()
    flat = y.reshape(-1)
    if dtype == "bf16":
        _lib.orc_round_bf16(flat, flat.size)
    elif dtype == "fp16":
        _lib.orc_round_f16(flat, flat.size)
    elif dtype != "fp32":
        raise ValueError(dtype)
    return y


def to_bits(x: np.ndarray, dtype: str) -> np.ndarray:
    xf = _f32(x)
    out = np.empty(xf.shape, dtype=np.uint16)
    fn = _lib.orc_f32_to_bf16_bits if dtype == "bf16" else _lib.orc_f32_to_f16_bits
    fn(xf.reshape(-1), xf.size, out.reshape(-1))
    return out


def from_bits(b: np.ndarray, dtype: str) -> np.ndarray:
    bb = np.ascontiguousarray(b, dtype=np.uint16)
    out = np.empty(bb.shape, dtype=np.float32)
    fn = _lib.orc_bf16_bits_to_f32 if dtype == "bf16" else _lib.orc_f16_bits_to_f32
    fn(bb.reshape(-1), bb.size, out.reshape(-1))
    return out


def build_axial_rope_tables(txt_len, hp, wp, head_dim, axes, theta=10000.0):
    L = txt_len + hp * wp
    cos = np.empty((L, head_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    ax = np.asarray(axes, dtype=np.int32)
    if _lib.orc_build_axial_rope_tables(txt_len, hp, wp, head_dim, ax, len(ax), theta, cos, sin) != 0:
        raise ValueError("build_axial_rope_tables: axes must sum to an even head_dim")
    return cos, sin


def build_qwen_rope_tables(segments, hp, wp, head_dim, axes=(16, 56, 56), theta=10000.0):
    """segments: list of ("text", n) or ("image", h, w) making up the prefix."""
    kind = np.array([0 if s[0] == "text" else 1 for s in segments], dtype=np.int32).reshape(-1)
    a = np.array([s[1] for s in segments], dtype=np.int32).reshape(-1)
    b = np.array([s[2] if s[0] != "text" else 0 for s in segments], dtype=np.int32).reshape(-1)
    if len(segments) == 0:
        kind = np.zeros(1, np.int32); a = np.zeros(1, np.int32); b = np.zeros(1, np.int32)
    ax = np.asarray(axes, dtype=np.int32)
    L = _lib.orc_build_qwen_rope_tables(kind, a, b, len(segments), hp, wp, head_dim, ax, theta, None, None)
    if L < 0:
        raise ValueError("build_qwen_rope_tables: bad head_dim / axes")
    cos = np.empty((L, head_dim // 2), dtype=np.float32)
    sin = np.empty_like(cos)
    _lib.orc_build_qwen_rope_tables(kind, a, b, len(segments), hp, wp, head_dim, ax, theta, _ptr(cos), _ptr(sin))
    return cos, sin


def rope_apply(x, cos, sin, num_heads, head_dim, split_half=False, round_to_dtype="fp32"):
    x = _f32(x)
    L = x.shape[0]
    assert x.shape[1] == num_heads * head_dim and cos.shape == (L, head_dim // 2) == sin.shape
    out = np.empty_like(x)
    mode = {"fp32": 0, "bf16": 1, "fp16": 2}[round_to_dtype]
    _lib.orc_rope_apply(x, _f32(cos), _f32(sin), L, num_heads, head_dim, int(split_half), mode, out)
    return out


def rows_causal(Lq, Lk, q_offset=None, window=0):
    if q_offset is None:
        q_offset = Lk - Lq
    lo = np.empty(Lq, dtype=np.int32)
    hi = np.empty(Lq, dtype=np.int32)
    _lib.orc_rows_causal(Lq, Lk, q_offset, window, lo, hi)
    return lo, hi


def rows_block_causal(Lq, Lk, q_offset, seg_q_end, seg_k_end, seg_causal):
    lo = np.empty(Lq, dtype=np.int32)
    hi = np.empty(Lq, dtype=np.int32)
    _lib.orc_rows_block_causal(Lq, Lk, q_offset, np.asarray(seg_q_end, np.int32), np.asarray(seg_k_end, np.int32),
                               np.asarray(seg_causal, np.int32), len(seg_q_end), lo, hi)
    return lo, hi


def dense_block_causal(Lq, Lk, q_offset, block_id):
    mask = np.empty((Lq, Lk), dtype=np.uint8)
    _lib.orc_dense_block_causal(Lq, Lk, q_offset, np.asarray(block_id, np.int32), mask)
    return mask


def sdpa(q, k, v, num_heads, scale=None, key_mask=None, row_lo=None, row_hi=None, dense_mask=None,
         bias=None, bias_q0=0, rows=None, return_attn_avg=False, n_threads=0):
    """softmax(q k^T * scale [masks]) v per head; see orc_sdpa in oracle.cpp."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    Lq, D = q.shape
    Lk = k.shape[0]
    d = D // num_heads
    assert D == num_heads * d and k.shape == (Lk, D) == v.shape
    out = np.zeros((Lq, D), dtype=np.float32)
    km = None if key_mask is None else _f32(key_mask)
    lo = None if row_lo is None else np.ascontiguousarray(row_lo, np.int32)
    hi = None if row_hi is None else np.ascontiguousarray(row_hi, np.int32)
    dm = None if dense_mask is None else np.ascontiguousarray(dense_mask, np.uint8)
    bs = None if bias is None else _f32(bias)
    rw = None if rows is None else np.ascontiguousarray(rows, np.int32)
    avg = np.zeros((Lq, Lk), dtype=np.float32) if return_attn_avg else None
    _lib.orc_sdpa(q, k, v, Lq, Lk, num_heads, d, -1.0 if scale is None else float(scale), _ptr(km), _ptr(lo),
                  _ptr(hi), _ptr(dm), _ptr(bs), int(bias_q0), 0 if bs is None else bs.shape[1], _ptr(rw),
                  0 if rw is None else rw.size, out, _ptr(avg), n_threads)
    return (out, avg) if return_attn_avg else out


def linear_attn_relu(q, k, v, num_heads, eps=1e-15, return_state=False, n_threads=0):
    q, k, v = _f32(q), _f32(k), _f32(v)
    N, D = q.shape
    d = D // num_heads
    out = np.empty((N, D), dtype=np.float32)
    S = np.empty((num_heads, d, d), dtype=np.float32) if return_state else None
    z = np.empty((num_heads, d), dtype=np.float32) if return_state else None
    _lib.orc_linear_attn_relu(q, k, v, N, num_heads, d, eps, out, _ptr(S), _ptr(z), n_threads)
    return (out, S, z) if return_state else out


def rms_norm(x, gain, eps):
    """Row-wise RMS normalisation of a (rows, cols) array with a (cols) gain."""
    x = _f32(x)
    rows, cols = x.shape
    out = np.empty_like(x)
    _lib.orc_rms_norm(x, _f32(gain).reshape(cols), float(eps), rows, cols, out)
    return out


def headnorm_rope(x, gain, eps, cos, sin, num_heads, head_dim, round_to_dtype="fp32", round_between=None):
    """headnorm then rope_apply (src/dit/qwenimage21_forward.cpp:582-585) on x (L, heads*head_dim). round_between
    names the dtype the normalised tensor is rounded to before the rotation, as the reference's two passes do;
    None keeps FP32 in between (what the fused kernel computes)."""
    x = _f32(x)
    L = x.shape[0]
    y = rms_norm(x.reshape(L * num_heads, head_dim), gain, eps).reshape(L, num_heads * head_dim)
    if round_between is not None:
        y = round_to(y, round_between)
    if cos is None:
        return round_to(y, round_to_dtype)
    return rope_apply(y, cos, sin, num_heads, head_dim, round_to_dtype=round_to_dtype)


def geglu_exact(t):
    """(rows, 2*d_out) -> (rows, d_out): value half times exact GELU of the gate half."""
    t = _f32(t)
    rows, two_d = t.shape
    out = np.empty((rows, two_d // 2), dtype=np.float32)
    _lib.orc_geglu_exact(t, rows, two_d // 2, out)
    return out


def linear(x, w, bias=None, n_threads=0):
    """y = x w^T + bias; x (M, K), w (N, K), bias (N) or None."""
    x, w = _f32(x), _f32(w)
    M, K = x.shape
    N = w.shape[0]
    assert w.shape == (N, K)
    b = None if bias is None else _f32(bias).reshape(N)
    y = np.empty((M, N), dtype=np.float32)
    _lib.orc_linear(x, w, _ptr(b), M, N, K, y, n_threads)
    return y


def attention_qkvo(x, ctx, wq, bq, wk, bk, wv, bv, wo, bo, num_heads, dtype, key_mask=None, causal=False,
                   k=None, v=None, n_threads=0):
    """bt::flash_attention_qkvo_forward (src/unet_blocks.cpp:264-272) as linear -> attention -> linear for one
    batch item; with k / v given, the kv_cached form (src/unet_blocks.cpp:311-317). Q, K, V and the attention
    output are rounded to `dtype` between the stages ("fp32" keeps them exact)."""
    q = round_to(linear(x, wq, bq, n_threads), dtype)
    if k is None:
        src = x if ctx is None else ctx
        k = round_to(linear(src, wk, bk, n_threads), dtype)
        v = round_to(linear(src, wv, bv, n_threads), dtype)
    Lq, Lk = q.shape[0], k.shape[0]
    lo = hi = None
    if causal:
        lo, hi = rows_causal(Lq, Lk)
    a = round_to(sdpa(q, k, v, num_heads, key_mask=key_mask, row_lo=lo, row_hi=hi, n_threads=n_threads), dtype)
    return linear(a, wo, bo, n_threads)


def compare(ref: np.ndarray, x: np.ndarray) -> dict:
    """cosine, rel-L2 and max-abs as printed by the reference's parity scripts
    (scripts/qwenimage21_dit_parity.sh:27-33)."""
    r = np.asarray(ref, dtype=np.float64).reshape(-1)
    y = np.asarray(x, dtype=np.float64).reshape(-1)
    nr = np.linalg.norm(r)
    return {
        "cos": float(r @ y / (nr * np.linalg.norm(y) + 1e-300)),
        "rel_l2": float(np.linalg.norm(r - y) / (nr + 1e-300)),
        "max_abs": float(np.max(np.abs(r - y))) if r.size else 0.0,
    }
