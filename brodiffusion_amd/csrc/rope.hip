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

template <typename T>
int launch(const mi_rope_args* a, long x_rs, long o_rs, hipStream_t st) {
    const long work = a->split_half ? static_cast<long>(a->rows) * a->num_heads * (a->head_dim / 2)
                                    : static_cast<long>(a->rows) * a->num_heads * a->head_dim / 8;
    long blocks = (work + 255) / 256;
    if (blocks > 256 * 32) blocks = 256 * 32;
    if (blocks < 1) blocks = 1;
    const T* x = static_cast<const T*>(a->x);
    T* o = static_cast<T*>(a->out);
    if (a->split_half) {
        hipLaunchKernelGGL(rope_split_kernel<T>, dim3(blocks), dim3(256), 0, st, x, o, a->cos, a->sin, a->rows,
                           a->num_heads, a->head_dim, x_rs, o_rs, a->per_head);
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
