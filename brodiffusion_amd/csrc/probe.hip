// Calibration probe of the benchmark: what the matrix pipes of THIS GPU sustain right now, with nothing else in the way.
//
// Every wavefront loads 16 MFMA operands from a caller buffer once and then issues nothing but independent
// v_mfma_f32_32x32x16 instructions (four accumulator chains, operands rotating so that the pipe's inputs toggle the way
// the data does). The sustained rate depends on the operand values because the clock is power-managed: all-zero operands
// run near the nominal clock, N(0,1) operands well below it. A benchmark that reports an MFMA-bound kernel against the
// nominal peak prints these two rates next to it, so that a reader can divide the state of the box out of the figure.
// Besides the launch (timed by the caller with events) one wavefront per work group reports the shader cycles and the
// constant-rate 100 MHz ticks its loop took: cycles / ticks * 100 is the clock in MHz under this load.
#include <algorithm>

#include "internal.h"

namespace mi {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kProbeThreads = 512;            // 8 wavefronts = 2 per SIMD, four independent accumulator chains each
constexpr int kProbeMfmaPerTrip = 8;
constexpr double kFlopPerMfma = 2.0 * 32 * 32 * 16;

template <typename V8> __device__ __forceinline__ f32x16 mfma(V8 a, V8 b, f32x16 c);
template <> __device__ __forceinline__ f32x16 mfma<bf16x8>(bf16x8 a, bf16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
template <> __device__ __forceinline__ f32x16 mfma<f16x8>(f16x8 a, f16x8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }

template <typename V8>
__global__ void __launch_bounds__(kProbeThreads, 2) mfma_probe_kernel(int trips, const u32x4* data, unsigned n_chunks, float* sink,
                                                                      unsigned long long* clocks) {
    V8 a[8], b[8];
    const unsigned t = blockIdx.x * kProbeThreads + threadIdx.x;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a[i] = __builtin_bit_cast(V8, data[(t * 16u + i) % n_chunks]);
        b[i] = __builtin_bit_cast(V8, data[(t * 16u + 8u + i) % n_chunks]);
    }
    f32x16 c0, c1, c2, c3;
#pragma unroll
    for (int e = 0; e < 16; ++e) c0[e] = c1[e] = c2[e] = c3[e] = 0.f;
    const unsigned long long r0 = wall_clock64();
    const unsigned long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < trips; ++it) {
#pragma unroll
        for (int j = 0; j < kProbeMfmaPerTrip; j += 4) {
            c0 = mfma<V8>(a[j], b[j], c0);
            c1 = mfma<V8>(a[j + 1], b[j + 1], c1);
            c2 = mfma<V8>(a[j + 2], b[j + 2], c2);
            c3 = mfma<V8>(a[j + 3], b[j + 3], c3);
        }
    }
    const unsigned long long t1 = __builtin_readcyclecounter();
    const unsigned long long r1 = wall_clock64();
    sink[t & 1023u] = c0[0] + c1[1] + c2[2] + c3[3];
    if (threadIdx.x == 0 && clocks) {
        clocks[2 * blockIdx.x] = t1 - t0;
        clocks[2 * blockIdx.x + 1] = r1 - r0;
    }
}

}  // namespace
}  // namespace mi

extern "C" int mi_mfma_probe(mi_mfma_probe_args* a) {
    using mi::fail;
    mi::clear_error();
    if (!a) return fail("mi_mfma_probe: null args");
    if (a->struct_size != sizeof(mi_mfma_probe_args)) return fail("mi_mfma_probe: struct_size mismatch");
    if (a->dtype != MI_DTYPE_BF16 && a->dtype != MI_DTYPE_F16) return fail("mi_mfma_probe: dtype %d is neither fp16 nor bf16", a->dtype);
    if (!a->operands || a->operand_bytes < 4096 || (reinterpret_cast<uintptr_t>(a->operands) & 15u))
        return fail("mi_mfma_probe: operands must be a 16-byte aligned device buffer of at least 4096 bytes");
    if (!a->sink || a->sink_bytes < 4096) return fail("mi_mfma_probe: sink must hold 4096 bytes");
    if (a->trips <= 0 || a->trips > (1 << 24)) return fail("mi_mfma_probe: trips must be in 1..2^24");
    const int n_cu = mi::device_cu_count();
    const int blocks = 2 * n_cu;
    if (a->clocks && a->clocks_bytes < static_cast<size_t>(blocks) * 16)
        return fail("mi_mfma_probe: clocks must hold %d bytes (two 64-bit counts per work group, %d work groups)", blocks * 16, blocks);
    const unsigned n_chunks = static_cast<unsigned>(std::min<size_t>(a->operand_bytes / 16, 1u << 30));
    hipStream_t st = mi::resolve_stream(a->stream);
    auto* data = static_cast<const mi::u32x4*>(a->operands);
    auto* clocks = reinterpret_cast<unsigned long long*>(a->clocks);
    if (a->dtype == MI_DTYPE_BF16)
        hipLaunchKernelGGL((mi::mfma_probe_kernel<mi::bf16x8>), dim3(blocks), dim3(mi::kProbeThreads), 0, st, a->trips, data, n_chunks, a->sink, clocks);
    else
        hipLaunchKernelGGL((mi::mfma_probe_kernel<mi::f16x8>), dim3(blocks), dim3(mi::kProbeThreads), 0, st, a->trips, data, n_chunks, a->sink, clocks);
    MI_HIP_CHECK(hipGetLastError());
    a->work_groups = blocks;
    a->flops = static_cast<double>(blocks) * (mi::kProbeThreads / 64) * a->trips * mi::kProbeMfmaPerTrip * mi::kFlopPerMfma;
    return 0;
}
