// The two elementwise helpers of the U-Net transformer block: Y += X over flat storage and Y[r][c] += bias[c].
// Bandwidth-bound passes; 16-byte accesses where base addresses and the element count allow, a scalar loop otherwise
// (the reference's own tests use 10 x 37 and 13 x 29 tensors). FP32 add, one rounding.
#include "internal.h"

namespace mi {
namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <typename T>
__global__ void __launch_bounds__(256) add_inplace_kernel(T* y, const T* x, long n, int vec_ok) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    const long stride = gridDim.x * 256L;
    const long n8 = vec_ok ? n / 8 : 0;
    for (long i = blockIdx.x * 256L + threadIdx.x; i < n8; i += stride) {
        t8 a = __builtin_bit_cast(t8, reinterpret_cast<const u32x4*>(y)[i]);
        const t8 b = __builtin_bit_cast(t8, reinterpret_cast<const u32x4*>(x)[i]);
#pragma unroll
        for (int e = 0; e < 8; ++e) a[e] = static_cast<T>(static_cast<float>(a[e]) + static_cast<float>(b[e]));
        reinterpret_cast<u32x4*>(y)[i] = __builtin_bit_cast(u32x4, a);
    }
    for (long i = n8 * 8 + blockIdx.x * 256L + threadIdx.x; i < n; i += stride)
        y[i] = static_cast<T>(static_cast<float>(y[i]) + static_cast<float>(x[i]));
}

template <typename T>
__global__ void __launch_bounds__(256) add_row_bias_kernel(T* y, const T* bias, int rows, int cols, long y_rs, int vec_ok) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    const long stride = gridDim.x * 256L;
    if (vec_ok) {
        const int cpr = cols / 8;
        const long total = static_cast<long>(rows) * cpr;
        for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += stride) {
            const long r = idx / cpr;
            const int c = static_cast<int>(idx - r * cpr) * 8;
            t8 a = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(y + r * y_rs + c));
            const t8 b = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(bias + c));
#pragma unroll
            for (int e = 0; e < 8; ++e) a[e] = static_cast<T>(static_cast<float>(a[e]) + static_cast<float>(b[e]));
            *reinterpret_cast<u32x4*>(y + r * y_rs + c) = __builtin_bit_cast(u32x4, a);
        }
    } else {
        const long total = static_cast<long>(rows) * cols;
        for (long idx = blockIdx.x * 256L + threadIdx.x; idx < total; idx += stride) {
            const long r = idx / cols;
            const int c = static_cast<int>(idx - r * cols);
            y[r * y_rs + c] = static_cast<T>(static_cast<float>(y[r * y_rs + c]) + static_cast<float>(bias[c]));
        }
    }
}

// RMS normalisation of whole rows: one work group per row (grid-stride over rows), the row held in registers between
// the sum of squares and the scaling (up to kRmsChunks 16-byte chunks per thread), FP32 arithmetic, one rounding.
constexpr int kRmsChunks = 8;   // 256 threads x 8 chunks x 8 elements = rows of up to 16384 columns
template <typename T>
__global__ void __launch_bounds__(256) rms_norm_rows_kernel(const T* x, const T* __restrict__ gain, T* out, int rows, int cols,
                                                            long x_rs, long o_rs, float eps) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    __shared__ float red[4];
    const int cpr = cols / 8;
    const int tid = threadIdx.x;
    for (int r = blockIdx.x; r < rows; r += gridDim.x) {
        t8 v[kRmsChunks];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < kRmsChunks; ++i) {
            const int c = tid + 256 * i;
            if (c < cpr) {
                v[i] = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(x + static_cast<long>(r) * x_rs + c * 8));
#pragma unroll
                for (int e = 0; e < 8; ++e) { const float f = static_cast<float>(v[i][e]); ss = __builtin_fmaf(f, f, ss); }
            }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) ss += __shfl_xor(ss, off);
        __syncthreads();                      // the previous row's readers are done with `red`
        if ((tid & 63) == 0) red[tid >> 6] = ss;
        __syncthreads();
        const float inv = __builtin_amdgcn_rsqf((red[0] + red[1] + red[2] + red[3]) / static_cast<float>(cols) + eps);
#pragma unroll
        for (int i = 0; i < kRmsChunks; ++i) {
            const int c = tid + 256 * i;
            if (c < cpr) {
                const t8 g = __builtin_bit_cast(t8, *reinterpret_cast<const u32x4*>(gain + c * 8));
                t8 o;
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = static_cast<T>(static_cast<float>(v[i][e]) * inv * static_cast<float>(g[e]));
                *reinterpret_cast<u32x4*>(out + static_cast<long>(r) * o_rs + c * 8) = __builtin_bit_cast(u32x4, o);
            }
        }
    }
}

long grid_for(long work) {
    long blocks = (work + 255) / 256;
    return blocks < 1 ? 1 : (blocks > 256 * 32 ? 256 * 32 : blocks);
}

}  // namespace
}  // namespace mi

using mi::fail;

extern "C" {

int mi_add_inplace(void* y, const void* x, int64_t n_elements, int32_t dtype, void* stream) {
    mi::clear_error();
    if (n_elements < 0) return fail("mi_add_inplace: negative element count");
    if (n_elements == 0) return 0;
    if (!y || !x) return fail("mi_add_inplace: null tensor");
    if ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(x)) & 1u) return fail("mi_add_inplace: pointers must be 2-byte aligned");
    const int vec_ok = ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0;
    hipStream_t st = mi::resolve_stream(stream);
    const dim3 grid(static_cast<unsigned>(mi::grid_for(vec_ok ? (n_elements + 7) / 8 : n_elements)));
    if (dtype == MI_DTYPE_BF16)
        hipLaunchKernelGGL(mi::add_inplace_kernel<__bf16>, grid, dim3(256), 0, st, static_cast<__bf16*>(y), static_cast<const __bf16*>(x), n_elements, vec_ok);
    else if (dtype == MI_DTYPE_F16)
        hipLaunchKernelGGL(mi::add_inplace_kernel<_Float16>, grid, dim3(256), 0, st, static_cast<_Float16*>(y), static_cast<const _Float16*>(x), n_elements, vec_ok);
    else
        return fail("mi_add_inplace: dtype %d not supported", dtype);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_add_inplace launch: %s", hipGetErrorString(e));
    return 0;
}

int mi_add_row_bias(void* y, const void* bias, int32_t rows, int32_t cols, int64_t y_row_stride, int32_t dtype, void* stream) {
    mi::clear_error();
    if (rows < 0 || cols <= 0) return fail("mi_add_row_bias: bad shape");
    if (rows == 0) return 0;
    if (!y || !bias) return fail("mi_add_row_bias: null tensor");
    const long y_rs = y_row_stride ? y_row_stride : cols;
    if (y_rs < cols) return fail("mi_add_row_bias: row stride smaller than cols");
    const int vec_ok = cols % 8 == 0 && y_rs % 8 == 0 && ((reinterpret_cast<uintptr_t>(y) | reinterpret_cast<uintptr_t>(bias)) & 15u) == 0;
    hipStream_t st = mi::resolve_stream(stream);
    const dim3 grid(static_cast<unsigned>(mi::grid_for(static_cast<long>(rows) * (vec_ok ? cols / 8 : cols))));
    if (dtype == MI_DTYPE_BF16)
        hipLaunchKernelGGL(mi::add_row_bias_kernel<__bf16>, grid, dim3(256), 0, st, static_cast<__bf16*>(y), static_cast<const __bf16*>(bias), rows, cols, y_rs, vec_ok);
    else if (dtype == MI_DTYPE_F16)
        hipLaunchKernelGGL(mi::add_row_bias_kernel<_Float16>, grid, dim3(256), 0, st, static_cast<_Float16*>(y), static_cast<const _Float16*>(bias), rows, cols, y_rs, vec_ok);
    else
        return fail("mi_add_row_bias: dtype %d not supported", dtype);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_add_row_bias launch: %s", hipGetErrorString(e));
    return 0;
}

int mi_rms_norm_forward(const void* x, const void* gain, void* out, int32_t rows, int32_t cols, int64_t x_row_stride,
                        int64_t out_row_stride, float eps, int32_t dtype, void* stream) {
    mi::clear_error();
    if (rows < 0 || cols <= 0 || cols % 8 != 0) return fail("mi_rms_norm_forward: cols must be a positive multiple of 8, rows >= 0");
    if (cols > 256 * 8 * mi::kRmsChunks) return fail("mi_rms_norm_forward: rows of more than %d columns are not supported", 256 * 8 * mi::kRmsChunks);
    if (rows == 0) return 0;
    if (!x || !gain || !out) return fail("mi_rms_norm_forward: null tensor");
    if (!(eps >= 0.f)) return fail("mi_rms_norm_forward: eps must be >= 0");
    const long x_rs = x_row_stride ? x_row_stride : cols, o_rs = out_row_stride ? out_row_stride : cols;
    if (x_rs < cols || o_rs < cols || x_rs % 8 != 0 || o_rs % 8 != 0)
        return fail("mi_rms_norm_forward: row strides must be multiples of 8 elements and at least cols");
    if ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(gain) | reinterpret_cast<uintptr_t>(out)) & 15u)
        return fail("mi_rms_norm_forward: pointers must be 16-byte aligned");
    hipStream_t st = mi::resolve_stream(stream);
    const dim3 grid(static_cast<unsigned>(rows < 256 * 16 ? rows : 256 * 16));
    if (dtype == MI_DTYPE_BF16)
        hipLaunchKernelGGL(mi::rms_norm_rows_kernel<__bf16>, grid, dim3(256), 0, st, static_cast<const __bf16*>(x), static_cast<const __bf16*>(gain),
                           static_cast<__bf16*>(out), rows, cols, x_rs, o_rs, eps);
    else if (dtype == MI_DTYPE_F16)
        hipLaunchKernelGGL(mi::rms_norm_rows_kernel<_Float16>, grid, dim3(256), 0, st, static_cast<const _Float16*>(x), static_cast<const _Float16*>(gain),
                           static_cast<_Float16*>(out), rows, cols, x_rs, o_rs, eps);
    else
        return fail("mi_rms_norm_forward: dtype %d not supported", dtype);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_rms_norm_forward launch: %s", hipGetErrorString(e));
    return 0;
}

}  // extern "C"
