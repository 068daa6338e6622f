// Stand-alone rotary position embedding for gfx950: out = RoPE(x) with FP32 tables.
// Bandwidth-bound elementwise pass (one read and one write of x); used where the rotated
// tensor itself must exist in HBM (the prefix cache keeps post-RoPE K). Attention calls
// apply the rotation while loading Q and K instead.
#include "internal.h"

namespace mi {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// Adjacent pairs (x[2p], x[2p+1]): one thread rotates one 16-byte chunk = 4 pairs.
template <typename T>
__global__ void __launch_bounds__(256) rope_adjacent_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                            const float* __restrict__ cs, const float* __restrict__ sn,
                                                            int rows, int H, int d, long x_rs, long o_rs, int per_head) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    const int cpr = H * d / 8;  // chunks per row
    const long total = static_cast<long>(rows) * cpr;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const int r = static_cast<int>(idx / cpr);
        const int c = static_cast<int>(idx - static_cast<long>(r) * cpr);
        const int col = c * 8;
        const int h = col / d;
        const int dc = col - h * d;  // multiple of 8 inside the head
        const long trow = per_head ? static_cast<long>(r) * H + h : r;
        const f32x4 cv = *reinterpret_cast<const f32x4*>(cs + trow * (d / 2) + dc / 2);
        const f32x4 sv = *reinterpret_cast<const f32x4*>(sn + trow * (d / 2) + dc / 2);
        t8 v = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + r * x_rs + col));
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float a = static_cast<float>(v[2 * p]);
            const float b = static_cast<float>(v[2 * p + 1]);
            v[2 * p] = static_cast<T>(rope_re(a, b, cv[p], sv[p]));
            v[2 * p + 1] = static_cast<T>(rope_im(a, b, cv[p], sv[p]));
        }
        *reinterpret_cast<u32x4*>(out + r * o_rs + col) = __builtin_bit_cast(u32x4, v);
    }
}

// Adjacent pairs with one table for all heads: a thread rotates the same 16-byte chunk position of 4 heads of a row, so the
// chunk's table entries are fetched once for the four and 4 data loads are in flight per thread. The heads of a thread
// are n_hg apart (h = j * n_hg + hg), so that for each j the lanes of a wavefront touch consecutive heads, i.e. one
// contiguous piece of the row. Same arithmetic per element as the kernel above.
template <typename T>
__global__ void __launch_bounds__(256) rope_adjacent_heads_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                                  const float* __restrict__ cs, const float* __restrict__ sn,
                                                                  int rows, int H, int d, long x_rs, long o_rs) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    constexpr int HB = 4;
    const int cpd = d / 8, n_hg = H / HB;
    const long total = static_cast<long>(rows) * n_hg * cpd;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const long t = idx / cpd;
        const int dcq = static_cast<int>(idx - t * cpd);
        const long r = t / n_hg;
        const int hg = static_cast<int>(t - r * n_hg);
        const f32x4 cv = *reinterpret_cast<const f32x4*>(cs + r * (d / 2) + dcq * 4);
        const f32x4 sv = *reinterpret_cast<const f32x4*>(sn + r * (d / 2) + dcq * 4);
        u32x4 raw[HB];
#pragma unroll
        for (int j = 0; j < HB; ++j) raw[j] = *reinterpret_cast<const u32x4*>(x + r * x_rs + (j * n_hg + hg) * d + dcq * 8);
#pragma unroll
        for (int j = 0; j < HB; ++j) {
            t8 v = __builtin_bit_cast(t8, raw[j]);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const float a = static_cast<float>(v[2 * p]);
                const float b = static_cast<float>(v[2 * p + 1]);
                v[2 * p] = static_cast<T>(rope_re(a, b, cv[p], sv[p]));
                v[2 * p + 1] = static_cast<T>(rope_im(a, b, cv[p], sv[p]));
            }
            *reinterpret_cast<u32x4*>(out + r * o_rs + (j * n_hg + hg) * d + dcq * 8) = __builtin_bit_cast(u32x4, v);
        }
    }
}

// Split-half pairs (x[p], x[p + d/2]): one thread per pair (d/2 need not be a multiple of 8).
template <typename T>
__global__ void __launch_bounds__(256) rope_split_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                         const float* __restrict__ cs, const float* __restrict__ sn,
                                                         int rows, int H, int d, long x_rs, long o_rs, int per_head) {
    const int half = d / 2;
    const int ppr = H * half;  // pairs per row
    const long total = static_cast<long>(rows) * ppr;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const int r = static_cast<int>(idx / ppr);
        const int q = static_cast<int>(idx - static_cast<long>(r) * ppr);
        const int h = q / half;
        const int pp = q - h * half;
        const long trow = per_head ? static_cast<long>(r) * H + h : r;
        const float c = cs[trow * half + pp], s = sn[trow * half + pp];
        const float a = static_cast<float>(x[r * x_rs + h * d + pp]);
        const float b = static_cast<float>(x[r * x_rs + h * d + pp + half]);
        out[r * o_rs + h * d + pp] = static_cast<T>(rope_re(a, b, c, s));
        out[r * o_rs + h * d + pp + half] = static_cast<T>(rope_im(a, b, c, s));
    }
}

// Split-half pairs where half a head is whole 16-byte chunks (d % 16 == 0): one thread rotates the 8 pairs formed by
// chunk c of the lower half and chunk c of the upper half. Same arithmetic as rope_split_kernel.
template <typename T>
__global__ void __launch_bounds__(256) rope_split_vec_kernel(const T* x, T* out, const float* __restrict__ cs,
                                                             const float* __restrict__ sn, int rows, int H, int d, long x_rs,
                                                             long o_rs, int per_head) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    const int half = d / 2;
    const int upr = H * half / 8;  // units (8 pairs) per row
    const long total = static_cast<long>(rows) * upr;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const int r = static_cast<int>(idx / upr);
        const int u = static_cast<int>(idx - static_cast<long>(r) * upr);
        const int h = u / (half / 8);
        const int pp = (u - h * (half / 8)) * 8;   // first pair of the unit
        const long trow = per_head ? static_cast<long>(r) * H + h : r;
        const f32x4 c0 = *reinterpret_cast<const f32x4*>(cs + trow * half + pp), c1 = *reinterpret_cast<const f32x4*>(cs + trow * half + pp + 4);
        const f32x4 s0 = *reinterpret_cast<const f32x4*>(sn + trow * half + pp), s1 = *reinterpret_cast<const f32x4*>(sn + trow * half + pp + 4);
        t8 lo = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + r * x_rs + h * d + pp));
        t8 hi = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + r * x_rs + h * d + pp + half));
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float a = static_cast<float>(lo[e]), b = static_cast<float>(hi[e]);
            const float c = e < 4 ? c0[e & 3] : c1[e & 3], sv = e < 4 ? s0[e & 3] : s1[e & 3];
            lo[e] = static_cast<T>(rope_re(a, b, c, sv));
            hi[e] = static_cast<T>(rope_im(a, b, c, sv));
        }
        *reinterpret_cast<u32x4*>(out + r * o_rs + h * d + pp) = __builtin_bit_cast(u32x4, lo);
        *reinterpret_cast<u32x4*>(out + r * o_rs + h * d + pp + half) = __builtin_bit_cast(u32x4, hi);
    }
}

// Per-head RMS normalisation fused with the rotation (adjacent or split-half pairs) and an optional second destination for the
// leading rows: y = RoPE(x * rsqrt(mean_d(x^2) + eps) * gain), one read of x, one rounding. One thread per 16-byte
// chunk; the CPR = d/8 threads of a head row are neighbouring lanes of one wavefront (CPR is a power of two <= 16),
// so the sum of squares is CPR-lane butterfly. Everything is FP32 between the load and the single rounding.
template <typename T, int CPR>
__global__ void __launch_bounds__(256) headnorm_rope_kernel(const T* x, T* out, T* out2,
                                                            const T* __restrict__ gain, const float* __restrict__ cs,
                                                            const float* __restrict__ sn, int rows, int H, float eps,
                                                            long x_rs, long o_rs, long o2_rs, int out2_rows, int split_half) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    constexpr int d = CPR * 8;
    const int cpr = H * CPR;
    const long total = static_cast<long>(rows) * cpr;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const int r = static_cast<int>(idx / cpr);
        const int c = static_cast<int>(idx - static_cast<long>(r) * cpr);
        const int col = c * 8;
        const int dc = (c % CPR) * 8;
        const t8 v = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + r * x_rs + col));
        const t8 g = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(gain + dc));
        float f[8];
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) { f[e] = static_cast<float>(v[e]); ss = __builtin_fmaf(f[e], f[e], ss); }
#pragma unroll
        for (int off = 1; off < CPR; off <<= 1) ss += __shfl_xor(ss, off);
        const float inv = __builtin_amdgcn_rsqf(ss * (1.0f / d) + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) f[e] = f[e] * inv * static_cast<float>(g[e]);
        t8 o;
        if (cs != nullptr && split_half) {
            // the partner of chunk c is chunk c ^ (CPR / 2) of the same head row, held by the lane CPR / 2 away; the lower
            // half yields the real parts, the upper half the imaginary parts of the 8 pairs the two chunks form
            const bool upper = dc >= d / 2;
            const int pp = upper ? dc - d / 2 : dc;
            const f32x4 c0 = *reinterpret_cast<const f32x4*>(cs + static_cast<long>(r) * (d / 2) + pp);
            const f32x4 c1 = *reinterpret_cast<const f32x4*>(cs + static_cast<long>(r) * (d / 2) + pp + 4);
            const f32x4 s0 = *reinterpret_cast<const f32x4*>(sn + static_cast<long>(r) * (d / 2) + pp);
            const f32x4 s1 = *reinterpret_cast<const f32x4*>(sn + static_cast<long>(r) * (d / 2) + pp + 4);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float other = __shfl_xor(f[e], CPR / 2);
                const float a = upper ? other : f[e], b = upper ? f[e] : other;
                const float c = e < 4 ? c0[e & 3] : c1[e & 3], sv = e < 4 ? s0[e & 3] : s1[e & 3];
                o[e] = static_cast<T>(upper ? rope_im(a, b, c, sv) : rope_re(a, b, c, sv));
            }
        } else if (cs != nullptr) {
            const f32x4 cv = *reinterpret_cast<const f32x4*>(cs + static_cast<long>(r) * (d / 2) + dc / 2);
            const f32x4 sv = *reinterpret_cast<const f32x4*>(sn + static_cast<long>(r) * (d / 2) + dc / 2);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                o[2 * p] = static_cast<T>(rope_re(f[2 * p], f[2 * p + 1], cv[p], sv[p]));
                o[2 * p + 1] = static_cast<T>(rope_im(f[2 * p], f[2 * p + 1], cv[p], sv[p]));
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(f[e]);
        }
        const u32x4 bits = __builtin_bit_cast(u32x4, o);
        *reinterpret_cast<u32x4*>(out + r * o_rs + col) = bits;
        if (r < out2_rows) *reinterpret_cast<u32x4*>(out2 + r * o2_rs + col) = bits;
    }
}

// The same for head counts that are multiples of 4: a thread takes one chunk position of 4 heads of a row (heads n_hg
// apart, so that for each of the four the lanes of a wavefront touch one contiguous piece of the row), with one fetch of
// the gain and table entries and one index computation for the four, and 4 loads in flight. Same arithmetic per element.
template <typename T, int CPR>
__global__ void __launch_bounds__(256) headnorm_rope_heads_kernel(const T* x, T* out, T* out2,
                                                                  const T* __restrict__ gain, const float* __restrict__ cs,
                                                                  const float* __restrict__ sn, int rows, int H, float eps,
                                                                  long x_rs, long o_rs, long o2_rs, int out2_rows, int split_half) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    constexpr int d = CPR * 8, HB = 4;
    const int n_hg = H / HB;
    const long total = static_cast<long>(rows) * n_hg * CPR;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const long t = idx / CPR;
        const int cq = static_cast<int>(idx - t * CPR);
        const long r = t / n_hg;
        const int hg = static_cast<int>(t - r * n_hg);
        const int dc = cq * 8;
        u32x4 raw[HB];
#pragma unroll
        for (int j = 0; j < HB; ++j) raw[j] = *reinterpret_cast<const u32x4*>(x + r * x_rs + (j * n_hg + hg) * d + dc);
        const t8 g = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(gain + dc));
        f32x4 c0 = {0.f, 0.f, 0.f, 0.f}, c1 = c0, s0 = c0, s1 = c0;
        const bool upper = dc >= d / 2;
        if (cs != nullptr && split_half) {
            const int pp = upper ? dc - d / 2 : dc;
            c0 = *reinterpret_cast<const f32x4*>(cs + r * (d / 2) + pp);
            c1 = *reinterpret_cast<const f32x4*>(cs + r * (d / 2) + pp + 4);
            s0 = *reinterpret_cast<const f32x4*>(sn + r * (d / 2) + pp);
            s1 = *reinterpret_cast<const f32x4*>(sn + r * (d / 2) + pp + 4);
        } else if (cs != nullptr) {
            c0 = *reinterpret_cast<const f32x4*>(cs + r * (d / 2) + dc / 2);
            s0 = *reinterpret_cast<const f32x4*>(sn + r * (d / 2) + dc / 2);
        }
#pragma unroll
        for (int j = 0; j < HB; ++j) {
            const t8 v = __builtin_bit_cast(t8, raw[j]);
            float f[8];
            float ss = 0.f;
#pragma unroll
            for (int e = 0; e < 8; ++e) { f[e] = static_cast<float>(v[e]); ss = __builtin_fmaf(f[e], f[e], ss); }
#pragma unroll
            for (int off = 1; off < CPR; off <<= 1) ss += __shfl_xor(ss, off);
            const float inv = __builtin_amdgcn_rsqf(ss * (1.0f / d) + eps);
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] = f[e] * inv * static_cast<float>(g[e]);
            t8 o;
            if (cs != nullptr && split_half) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float other = __shfl_xor(f[e], CPR / 2);
                    const float a = upper ? other : f[e], b = upper ? f[e] : other;
                    const float c = e < 4 ? c0[e & 3] : c1[e & 3], sv = e < 4 ? s0[e & 3] : s1[e & 3];
                    o[e] = static_cast<T>(upper ? rope_im(a, b, c, sv) : rope_re(a, b, c, sv));
                }
            } else if (cs != nullptr) {
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    o[2 * p] = static_cast<T>(rope_re(f[2 * p], f[2 * p + 1], c0[p], s0[p]));
                    o[2 * p + 1] = static_cast<T>(rope_im(f[2 * p], f[2 * p + 1], c0[p], s0[p]));
                }
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(f[e]);
            }
            const u32x4 bits = __builtin_bit_cast(u32x4, o);
            const long col = static_cast<long>(j * n_hg + hg) * d + dc;
            *reinterpret_cast<u32x4*>(out + r * o_rs + col) = bits;
            if (r < out2_rows) *reinterpret_cast<u32x4*>(out2 + r * o2_rs + col) = bits;
        }
    }
}

// out[r][c] = x[r][c] * scale * (row_scale ? row_scale[r] : 1): one thread per 16-byte chunk.
template <typename T>
__global__ void __launch_bounds__(256) scale_rows_kernel(const T* x, T* out, const float* __restrict__ row_scale, float scale,
                                                         int rows, int cols, long x_rs, long o_rs) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    const int cpr = cols / 8;
    const long total = static_cast<long>(rows) * cpr;
    for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += gridDim.x * 256L) {
        const int r = static_cast<int>(idx / cpr);
        const int col = static_cast<int>(idx - static_cast<long>(r) * cpr) * 8;
        const float f = row_scale ? scale * row_scale[r] : scale;
        t8 v = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + r * x_rs + col));
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = static_cast<T>(static_cast<float>(v[e]) * f);
        *reinterpret_cast<u32x4*>(out + r * o_rs + col) = __builtin_bit_cast(u32x4, v);
    }
}

template <typename T>
int launch_headnorm(const mi_headnorm_rope_args* a, long x_rs, long o_rs, long o2_rs, hipStream_t st) {
    const long work = static_cast<long>(a->rows) * a->num_heads * a->head_dim / 8;
    long blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    const T* x = static_cast<const T*>(a->x);
    T* o = static_cast<T*>(a->out);
    T* o2 = static_cast<T*>(a->out2);
    const T* g = static_cast<const T*>(a->gain);
    const int r2 = a->out2 ? a->out2_rows : 0;
    const bool four = a->num_heads % 4 == 0;
    const long blocks4 = (blocks + 3) / 4;
#define MI_HEADNORM_CASE(CPR)                                                                                          \
    case CPR * 8:                                                                                                      \
        if (four)                                                                                                      \
            hipLaunchKernelGGL((headnorm_rope_heads_kernel<T, CPR>), dim3(blocks4), dim3(256), 0, st, x, o, o2, g, a->cos, \
                               a->sin, a->rows, a->num_heads, a->eps, x_rs, o_rs, o2_rs, r2, a->split_half);           \
        else                                                                                                           \
            hipLaunchKernelGGL((headnorm_rope_kernel<T, CPR>), dim3(blocks), dim3(256), 0, st, x, o, o2, g, a->cos,    \
                               a->sin, a->rows, a->num_heads, a->eps, x_rs, o_rs, o2_rs, r2, a->split_half);           \
        break;
    switch (a->head_dim) {
        MI_HEADNORM_CASE(4)
        MI_HEADNORM_CASE(8)
        MI_HEADNORM_CASE(16)
        default: return fail("mi_headnorm_rope: head_dim %d not supported (32, 64, 128)", a->head_dim);
    }
#undef MI_HEADNORM_CASE
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_headnorm_rope launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch(const mi_rope_args* a, long x_rs, long o_rs, hipStream_t st) {
    const long work = a->split_half ? static_cast<long>(a->rows) * a->num_heads * (a->head_dim / 2)
                                    : static_cast<long>(a->rows) * a->num_heads * a->head_dim / 8;
    long blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks < 1) blocks = 1;
    const T* x = static_cast<const T*>(a->x);
    T* o = static_cast<T*>(a->out);
    const uintptr_t al = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->out) | reinterpret_cast<uintptr_t>(a->cos) |
                         reinterpret_cast<uintptr_t>(a->sin);
    if (a->split_half && a->head_dim % 16 == 0 && x_rs % 8 == 0 && o_rs % 8 == 0 && (al & 15u) == 0) {
        long vb = (static_cast<long>(a->rows) * a->num_heads * (a->head_dim / 16) + 255) / 256;
        if (vb > 256 * 32) vb = 256 * 32;
        hipLaunchKernelGGL(rope_split_vec_kernel<T>, dim3(vb), dim3(256), 0, st, x, o, a->cos, a->sin, a->rows, a->num_heads,
                           a->head_dim, x_rs, o_rs, a->per_head);
    } else if (a->split_half) {
        hipLaunchKernelGGL(rope_split_kernel<T>, dim3(blocks), dim3(256), 0, st, x, o, a->cos, a->sin, a->rows,
                           a->num_heads, a->head_dim, x_rs, o_rs, a->per_head);
    } else if (!a->per_head && a->num_heads % 4 == 0) {
        long hb = (work / 4 + 255) / 256;
        if (hb > 256 * 32) hb = 256 * 32;
        hipLaunchKernelGGL(rope_adjacent_heads_kernel<T>, dim3(hb), dim3(256), 0, st, x, o, a->cos, a->sin, a->rows,
                           a->num_heads, a->head_dim, x_rs, o_rs);
    } else {
        hipLaunchKernelGGL(rope_adjacent_kernel<T>, dim3(blocks), dim3(256), 0, st, x, o, a->cos, a->sin, a->rows,
                           a->num_heads, a->head_dim, x_rs, o_rs, a->per_head);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_rope_apply launch: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace
}  // namespace mi

extern "C" int mi_rope_apply(const mi_rope_args* a) {
    using mi::fail;
    mi::clear_error();
    if (!a) return fail("mi_rope_apply: null args");
    if (a->struct_size != sizeof(mi_rope_args)) return fail("mi_rope_apply: struct_size mismatch");
    if (a->rows < 0 || a->num_heads <= 0 || a->head_dim <= 0) return fail("mi_rope_apply: bad shape");
    if (a->rows == 0) return 0;
    if (!a->x || !a->out || !a->cos || !a->sin) return fail("mi_rope_apply: null tensor");
    if (a->head_dim % 2 != 0) return fail("mi_rope_apply: head_dim must be even");
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    const long x_rs = a->x_row_stride ? a->x_row_stride : D;
    const long o_rs = a->out_row_stride ? a->out_row_stride : D;
    if (x_rs < D || o_rs < D) return fail("mi_rope_apply: row stride smaller than heads*head_dim");
    if (!a->split_half) {
        if (a->head_dim % 8 != 0) return fail("mi_rope_apply: adjacent-pair kernel needs head_dim %% 8 == 0");
        if (x_rs % 8 != 0 || o_rs % 8 != 0) return fail("mi_rope_apply: row strides must be multiples of 8 elements");
        const uintptr_t al = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->out) |
                             reinterpret_cast<uintptr_t>(a->cos) | reinterpret_cast<uintptr_t>(a->sin);
        if (al & 15u) return fail("mi_rope_apply: pointers must be 16-byte aligned");
    }
    hipStream_t st = mi::resolve_stream(a->stream);
    if (a->dtype == MI_DTYPE_BF16) return mi::launch<__bf16>(a, x_rs, o_rs, st);
    if (a->dtype == MI_DTYPE_F16) return mi::launch<_Float16>(a, x_rs, o_rs, st);
    return fail("mi_rope_apply: dtype %d not supported", a->dtype);
}

extern "C" int mi_headnorm_rope(const mi_headnorm_rope_args* a) {
    using mi::fail;
    mi::clear_error();
    if (!a) return fail("mi_headnorm_rope: null args");
    if (a->struct_size != sizeof(mi_headnorm_rope_args)) return fail("mi_headnorm_rope: struct_size mismatch");
    if (a->rows < 0 || a->num_heads <= 0) return fail("mi_headnorm_rope: bad shape");
    if (a->head_dim != 32 && a->head_dim != 64 && a->head_dim != 128)
        return fail("mi_headnorm_rope: head_dim %d not supported (32, 64, 128)", a->head_dim);
    if (a->rows == 0) return 0;
    if (!a->x || !a->out || !a->gain) return fail("mi_headnorm_rope: x, out and gain must not be null");
    if ((a->cos == nullptr) != (a->sin == nullptr)) return fail("mi_headnorm_rope: cos and sin must be given together");
    if (!(a->eps >= 0.f)) return fail("mi_headnorm_rope: eps must be >= 0");
    if (a->out2_rows < 0 || a->out2_rows > a->rows) return fail("mi_headnorm_rope: out2_rows %d outside 0..rows", a->out2_rows);
    if (a->split_half != 0 && a->split_half != 1) return fail("mi_headnorm_rope: split_half must be 0 or 1");
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    const long x_rs = a->x_row_stride ? a->x_row_stride : D;
    const long o_rs = a->out_row_stride ? a->out_row_stride : D;
    const long o2_rs = a->out2_row_stride ? a->out2_row_stride : D;
    if (x_rs < D || o_rs < D || o2_rs < D) return fail("mi_headnorm_rope: row stride smaller than heads*head_dim");
    if (x_rs % 8 != 0 || o_rs % 8 != 0 || o2_rs % 8 != 0) return fail("mi_headnorm_rope: row strides must be multiples of 8 elements");
    const uintptr_t al = reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->out) | reinterpret_cast<uintptr_t>(a->out2) |
                         reinterpret_cast<uintptr_t>(a->gain) | reinterpret_cast<uintptr_t>(a->cos) | reinterpret_cast<uintptr_t>(a->sin);
    if (al & 15u) return fail("mi_headnorm_rope: pointers must be 16-byte aligned");
    hipStream_t st = mi::resolve_stream(a->stream);
    if (a->dtype == MI_DTYPE_BF16) return mi::launch_headnorm<__bf16>(a, x_rs, o_rs, o2_rs, st);
    if (a->dtype == MI_DTYPE_F16) return mi::launch_headnorm<_Float16>(a, x_rs, o_rs, o2_rs, st);
    return fail("mi_headnorm_rope: dtype %d not supported", a->dtype);
}

extern "C" int mi_scale_rows(const mi_scale_rows_args* a) {
    using mi::fail;
    mi::clear_error();
    if (!a) return fail("mi_scale_rows: null args");
    if (a->struct_size != sizeof(mi_scale_rows_args)) return fail("mi_scale_rows: struct_size mismatch");
    if (a->rows < 0 || a->cols <= 0 || a->cols % 8 != 0) return fail("mi_scale_rows: cols must be a positive multiple of 8, rows >= 0");
    if (a->rows == 0) return 0;
    if (!a->x || !a->out) return fail("mi_scale_rows: x and out must not be null");
    const long x_rs = a->x_row_stride ? a->x_row_stride : a->cols;
    const long o_rs = a->out_row_stride ? a->out_row_stride : a->cols;
    if (x_rs < a->cols || o_rs < a->cols || x_rs % 8 != 0 || o_rs % 8 != 0)
        return fail("mi_scale_rows: row strides must be multiples of 8 elements and at least cols");
    if ((reinterpret_cast<uintptr_t>(a->x) | reinterpret_cast<uintptr_t>(a->out)) & 15u) return fail("mi_scale_rows: pointers must be 16-byte aligned");
    if (reinterpret_cast<uintptr_t>(a->row_scale) & 3u) return fail("mi_scale_rows: row_scale must be 4-byte aligned");
    const long work = static_cast<long>(a->rows) * (a->cols / 8);
    long blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    hipStream_t st = mi::resolve_stream(a->stream);
    if (a->dtype == MI_DTYPE_BF16)
        hipLaunchKernelGGL(mi::scale_rows_kernel<__bf16>, dim3(blocks), dim3(256), 0, st, static_cast<const __bf16*>(a->x),
                           static_cast<__bf16*>(a->out), a->row_scale, a->scale, a->rows, a->cols, x_rs, o_rs);
    else if (a->dtype == MI_DTYPE_F16)
        hipLaunchKernelGGL(mi::scale_rows_kernel<_Float16>, dim3(blocks), dim3(256), 0, st, static_cast<const _Float16*>(a->x),
                           static_cast<_Float16*>(a->out), a->row_scale, a->scale, a->rows, a->cols, x_rs, o_rs);
    else
        return fail("mi_scale_rows: dtype %d not supported", a->dtype);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_scale_rows launch: %s", hipGetErrorString(e));
    return 0;
}
