// ReLU linear attention for gfx950 (MI355X): O[n] = (S relu(Q[n])) / (z . relu(Q[n]) + eps) with
// S = V^T relu(K) (d x d) and z = sum_n relu(K[n]) per (batch, head).
//
// The op is HBM-bound: Q, K, V are read once and O written once (4 streams of (N, H*d) 16-bit
// values); the d x d contractions are small and run on MFMA so they hide under the memory time.
//   state kernel: one work group reduces a chunk of tokens. K (ReLU applied on the way in) and V
//                 tiles of 64 tokens sit row-major in LDS; both MFMA operands need the token axis
//                 contiguous per lane, which ds_read_b64_tr_b16 (LDS transpose read) delivers.
//                 z comes from the same K fragments against an all-ones A operand. Partial (S, z)
//                 are added to the FP32 workspace with atomics.
//   apply kernel: S is staged in LDS as 16-bit A operand, relu(Q) rows are B operands straight from
//                 global memory; the denominator is an exact FP32 dot of z with the lane's own Q
//                 values plus one exchange between lanes l and l^32.
#include <algorithm>

#include "internal.h"

namespace mi {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef int i32x2 __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int kTN = 64;  // tokens per LDS tile in the state kernel

template <typename T> struct Mma;
template <> struct Mma<__bf16> {
    using v8 = bf16x8;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<_Float16> {
    using v8 = f16x8;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

struct LinDev {
    const void* q; const void* k; const void* v; void* o;
    int B, H, N;
    long q_rs, q_bs, k_rs, k_bs, v_rs, v_bs, o_rs, o_bs;
    float eps;
    float* ws;      // per (b,h): D*D floats of S (row = value channel), then D floats of z
    int tokens_per_group;
};

template <int D> struct LGeo {
    static constexpr int DP = (D + 31) / 32 * 32;
    static constexpr int NB = DP / 32;
    static constexpr int KC = DP / 16;
    static constexpr int T_STRIDE = ((DP * 2 + 63) / 128) * 128 + 64;  // tiles read by transpose reads
    static constexpr int S_STRIDE = DP * 2 + 16;                       // S rows read by ds_read_b128
    static constexpr int CPR = D / 8;
    static constexpr int NCH = kTN * CPR;
    static constexpr int NLD = (NCH + kThreads - 1) / kThreads;
    static constexpr int WS_FLOATS = D * D + D;
};

template <typename T>
__device__ __forceinline__ u32x4 relu8(u32x4 raw) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    t8 x = __builtin_bit_cast(t8, raw);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = x[i] > static_cast<T>(0.f) ? x[i] : static_cast<T>(0.f);
    return __builtin_bit_cast(u32x4, x);
}

__global__ void __launch_bounds__(256) fill_zero_kernel(float* p, long n) {
    for (long i = blockIdx.x * 256L + threadIdx.x; i < n; i += gridDim.x * 256L) p[i] = 0.f;
}

// ── state: (S, z) += over this group's token chunk ──
template <typename T, int D>
__global__ void __launch_bounds__(kThreads) linattn_state_kernel(const LinDev p) {
    using G = LGeo<D>;
    using V8 = typename Mma<T>::v8;
    __shared__ __attribute__((aligned(16))) unsigned char Ks[kTN * G::T_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned char Vs[kTN * G::T_STRIDE];

    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int n_begin = blockIdx.x * p.tokens_per_group;
    const int n_end = min(p.N, n_begin + p.tokens_per_group);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    const T* const k_base = static_cast<const T*>(p.k) + b * p.k_bs + h * D;
    const T* const v_base = static_cast<const T*>(p.v) + b * p.v_bs + h * D;

    // wave -> (row block of S, share of the 4 k-steps of a tile)
    constexpr int NTS = G::NB >= 3 ? 1 : 4 / G::NB;  // token splits
    constexpr int KSTEPS = 4 / NTS;
    const int rb = wave % G::NB;
    const int ts = wave / G::NB;
    const bool active = wave < G::NB * NTS;
    const bool does_z = active && rb == 0;

    if constexpr (G::DP > D) {  // pad columns stay zero for the whole kernel
        constexpr int PC = (G::DP - D) / 8;
        for (int i = tid; i < kTN * PC; i += kThreads) {
            const int off = (i / PC) * G::T_STRIDE + D * 2 + (i % PC) * 16;
            *reinterpret_cast<u32x4*>(Ks + off) = u32x4{0, 0, 0, 0};
            *reinterpret_cast<u32x4*>(Vs + off) = u32x4{0, 0, 0, 0};
        }
    }

    f32x16 acc[G::NB], zacc[G::NB];
#pragma unroll
    for (int cb = 0; cb < G::NB; ++cb)
#pragma unroll
        for (int e = 0; e < 16; ++e) { acc[cb][e] = 0.f; zacc[cb][e] = 0.f; }
    V8 ones;
#pragma unroll
    for (int t = 0; t < 8; ++t) ones[t] = static_cast<T>(1.f);

    u32x4 kreg[G::NLD], vreg[G::NLD];
    auto issue_loads = [&](int n0) {
#pragma unroll
        for (int i = 0; i < G::NLD; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR, cc = idx - (idx / G::CPR) * G::CPR;
            const int n = n0 + row;
            kreg[i] = u32x4{0, 0, 0, 0};
            vreg[i] = u32x4{0, 0, 0, 0};
            if (idx < G::NCH && n < n_end) {
                kreg[i] = *reinterpret_cast<const u32x4*>(k_base + static_cast<long>(n) * p.k_rs + cc * 8);
                vreg[i] = *reinterpret_cast<const u32x4*>(v_base + static_cast<long>(n) * p.v_rs + cc * 8);
            }
        }
    };
    auto store_tile = [&]() {
#pragma unroll
        for (int i = 0; i < G::NLD; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR, cc = idx - (idx / G::CPR) * G::CPR;
            if (idx < G::NCH) {
                *reinterpret_cast<u32x4*>(Ks + row * G::T_STRIDE + cc * 16) = relu8<T>(kreg[i]);
                *reinterpret_cast<u32x4*>(Vs + row * G::T_STRIDE + cc * 16) = vreg[i];
            }
        }
    };

    const int trow = (lane & 15) >> 2;
    const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    if (n_begin < n_end) issue_loads(n_begin);
    for (int n0 = n_begin; n0 < n_end; n0 += kTN) {
        store_tile();
        __syncthreads();
        if (n0 + kTN < n_end) issue_loads(n0 + kTN);
        if (active) {
#pragma unroll
            for (int s = 0; s < KSTEPS; ++s) {
                const int ks = ts * KSTEPS + s;
                const int trow0 = 16 * ks + 4 * lh + trow;
                const unsigned char* vptr = Vs + trow0 * G::T_STRIDE + (32 * rb + tcol) * 2;
                const s16x4 a_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vptr));
                const s16x4 a_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                    (__attribute__((address_space(3))) s16x4*)(vptr + 8 * G::T_STRIDE));
                const V8 a = __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
                for (int cb = 0; cb < G::NB; ++cb) {
                    const unsigned char* kptr = Ks + trow0 * G::T_STRIDE + (32 * cb + tcol) * 2;
                    const s16x4 b_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(kptr));
                    const s16x4 b_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(kptr + 8 * G::T_STRIDE));
                    const V8 bk = __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7));
                    acc[cb] = Mma<T>::run(a, bk, acc[cb]);
                    if (does_z) zacc[cb] = Mma<T>::run(ones, bk, zacc[cb]);
                }
            }
        }
        __syncthreads();
    }

    if (active) {
        float* const S = p.ws + static_cast<long>(bh) * G::WS_FLOATS;
        float* const z = S + D * D;
#pragma unroll
        for (int cb = 0; cb < G::NB; ++cb) {
            const int j = 32 * cb + lq;
            if (j < D) {
#pragma unroll
                for (int bb = 0; bb < 4; ++bb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int i = 32 * rb + 8 * bb + 4 * lh + e;
                        if (i < D) atomicAdd(S + i * D + j, acc[cb][4 * bb + e]);
                    }
                if (does_z && lh == 0) atomicAdd(z + j, zacc[cb][0]);
            }
        }
    }
}

// ── apply: O = (S relu(Q)) / (z . relu(Q) + eps) ──
template <typename T, int D>
__global__ void __launch_bounds__(kThreads) linattn_apply_kernel(const LinDev p) {
    using G = LGeo<D>;
    using V8 = typename Mma<T>::v8;
    __shared__ __attribute__((aligned(16))) unsigned char Ss[G::DP * G::S_STRIDE];
    __shared__ __attribute__((aligned(16))) float Zs[G::DP];

    const int bh = blockIdx.y;
    const int b = bh / p.H, h = bh % p.H;
    const int n_begin = blockIdx.x * p.tokens_per_group;
    const int n_end = min(p.N, n_begin + p.tokens_per_group);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const float* const S = p.ws + static_cast<long>(bh) * G::WS_FLOATS;
    const float* const z = S + D * D;

    // stage S (FP32 -> T) and z (FP32) in LDS; pad rows/columns are zero
    for (int idx = tid; idx < G::DP * (G::DP / 4); idx += kThreads) {
        const int i = idx / (G::DP / 4);
        const int j = (idx - i * (G::DP / 4)) * 4;
        f32x4 sv = {0.f, 0.f, 0.f, 0.f};
        if (i < D && j < D) sv = *reinterpret_cast<const f32x4*>(S + i * D + j);
        typedef T t4 __attribute__((ext_vector_type(4)));
        t4 tv;
#pragma unroll
        for (int e = 0; e < 4; ++e) tv[e] = static_cast<T>(sv[e]);
        *reinterpret_cast<t4*>(Ss + i * G::S_STRIDE + j * 2) = tv;
    }
    for (int j = tid; j < G::DP; j += kThreads) Zs[j] = j < D ? z[j] : 0.f;
    __syncthreads();

    for (int n0 = n_begin + wave * 32; n0 < n_end; n0 += 4 * 32) {
        const int n = n0 + lq;
        const bool valid = n < n_end;
        V8 qf[G::KC];
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) {
            const int d0 = 16 * c + 8 * lh;
            u32x4 raw = {0, 0, 0, 0};
            if (valid && d0 < D) raw = relu8<T>(*reinterpret_cast<const u32x4*>(q_base + static_cast<long>(n) * p.q_rs + d0));
            qf[c] = __builtin_bit_cast(V8, raw);
            const f32x4 z0 = *reinterpret_cast<const f32x4*>(Zs + d0);
            const f32x4 z1 = *reinterpret_cast<const f32x4*>(Zs + d0 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                den = __builtin_fmaf(z0[e], static_cast<float>(qf[c][e]), den);
                den = __builtin_fmaf(z1[e], static_cast<float>(qf[c][4 + e]), den);
            }
        }
        {
            // results copied to scalars before the bit cast (a bit cast of a vector element
            // expression reads element 0 for every index with this compiler)
            const int di = __builtin_bit_cast(int, den);
            const i32x2 r = __builtin_amdgcn_permlane32_swap(di, di, false, false);
            const int r0 = r[0], r1 = r[1];
            den = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
        }
        // the reference forms the reciprocal as rsqrt(den + eps)^2 in FP32
        const float rs = __builtin_amdgcn_rsqf(den + p.eps);
        const float recip = rs * rs;
#pragma unroll
        for (int rb = 0; rb < G::NB; ++rb) {
            f32x16 acc;
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[e] = 0.f;
#pragma unroll
            for (int c = 0; c < G::KC; ++c) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(Ss + (32 * rb + lq) * G::S_STRIDE + (16 * c + 8 * lh) * 2);
                acc = Mma<T>::run(__builtin_bit_cast(V8, a), qf[c], acc);
            }
            if (valid) {
#pragma unroll
                for (int bb = 0; bb < 4; ++bb) {
                    const int i0 = 32 * rb + 8 * bb + 4 * lh;
                    if (i0 < D) {
                        typedef T t4 __attribute__((ext_vector_type(4)));
                        t4 ov;
#pragma unroll
                        for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(acc[4 * bb + e] * recip);
                        *reinterpret_cast<t4*>(o_base + static_cast<long>(n) * p.o_rs + i0) = ov;
                    }
                }
            }
        }
    }
}

template <typename T, int D>
int launch_d(LinDev p, bool accumulate, int n_cu, hipStream_t st) {
    using G = LGeo<D>;
    const int BH = p.B * p.H;
    if (!accumulate) {
        const long n = static_cast<long>(BH) * G::WS_FLOATS;
        const int blocks = static_cast<int>(std::min<long>((n + 255) / 256, 2048));
        hipLaunchKernelGGL(fill_zero_kernel, dim3(blocks), dim3(256), 0, st, p.ws, n);
    }
    // enough groups to fill the chip about twice over, chunks a multiple of the 64-token tile
    auto pick = [&](int min_tokens) {
        int t = min_tokens;
        while (static_cast<long>(BH) * ((p.N + t - 1) / t) > 4L * n_cu && t < p.N) t *= 2;
        return t;
    };
    p.tokens_per_group = pick(128);
    hipLaunchKernelGGL((linattn_state_kernel<T, D>), dim3((p.N + p.tokens_per_group - 1) / p.tokens_per_group, BH),
                       dim3(kThreads), 0, st, p);
    p.tokens_per_group = pick(128);
    hipLaunchKernelGGL((linattn_apply_kernel<T, D>), dim3((p.N + p.tokens_per_group - 1) / p.tokens_per_group, BH),
                       dim3(kThreads), 0, st, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_linear_attn_relu_forward launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_t(const LinDev& p, int d, bool acc, int n_cu, hipStream_t st) {
    switch (d) {
        case 32: return launch_d<T, 32>(p, acc, n_cu, st);
        case 64: return launch_d<T, 64>(p, acc, n_cu, st);
        case 72: return launch_d<T, 72>(p, acc, n_cu, st);
        case 112: return launch_d<T, 112>(p, acc, n_cu, st);
        case 128: return launch_d<T, 128>(p, acc, n_cu, st);
        default: return fail("mi_linear_attn_relu_forward: head_dim %d has no kernel (32, 64, 72, 112, 128)", d);
    }
}

// S sums N products per entry and overflows FP16's range at image sizes (the reason the reference
// runs this core in BF16, src/dit/sana.cpp:526-530), so only BF16 operands are accepted.
bool lin_supported(int dtype, int d) {
    if (dtype != MI_DTYPE_BF16) return false;
    return d == 32 || d == 64 || d == 72 || d == 112 || d == 128;
}

}  // namespace
}  // namespace mi

extern "C" {

int mi_linear_attn_supported(int32_t dtype, int32_t head_dim) { return mi::lin_supported(dtype, head_dim) ? 1 : 0; }

size_t mi_linear_attn_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim) {
    if (batch <= 0 || num_heads <= 0 || head_dim <= 0) return 0;
    return static_cast<size_t>(batch) * num_heads * (static_cast<size_t>(head_dim) * head_dim + head_dim) * sizeof(float);
}

int mi_linear_attn_relu_forward(const mi_linear_attn_args* a) {
    using mi::fail;
    mi::clear_error();
    if (!a) return fail("mi_linear_attn_relu_forward: null args");
    if (a->struct_size != sizeof(mi_linear_attn_args)) return fail("mi_linear_attn_relu_forward: struct_size mismatch");
    if (!mi::lin_supported(a->dtype, a->head_dim))
        return fail("mi_linear_attn_relu_forward: no kernel for dtype %d head_dim %d", a->dtype, a->head_dim);
    if (a->batch <= 0 || a->num_heads <= 0 || a->n_tokens < 0) return fail("mi_linear_attn_relu_forward: bad shape");
    if (a->n_tokens == 0) return 0;
    if (!a->q || !a->k || !a->v || !a->o) return fail("mi_linear_attn_relu_forward: null tensor");
    const size_t need = mi_linear_attn_workspace_bytes(a->batch, a->num_heads, a->head_dim);
    if (!a->workspace || a->workspace_bytes < need)
        return fail("mi_linear_attn_relu_forward: workspace needs %zu bytes (got %zu)", need, a->workspace ? a->workspace_bytes : 0);
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    mi::LinDev p;
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o;
    p.B = a->batch; p.H = a->num_heads; p.N = a->n_tokens;
    auto rs = [D](int64_t s) { return s ? static_cast<long>(s) : D; };
    p.q_rs = rs(a->q_row_stride); p.k_rs = rs(a->k_row_stride); p.v_rs = rs(a->v_row_stride); p.o_rs = rs(a->o_row_stride);
    p.q_bs = a->q_batch_stride ? a->q_batch_stride : p.q_rs * a->n_tokens;
    p.k_bs = a->k_batch_stride ? a->k_batch_stride : p.k_rs * a->n_tokens;
    p.v_bs = a->v_batch_stride ? a->v_batch_stride : p.v_rs * a->n_tokens;
    p.o_bs = a->o_batch_stride ? a->o_batch_stride : p.o_rs * a->n_tokens;
    const long strides[] = {p.q_rs, p.k_rs, p.v_rs, p.o_rs, p.q_bs, p.k_bs, p.v_bs, p.o_bs};
    for (long s : strides)
        if (s % 8 != 0) return fail("mi_linear_attn_relu_forward: strides must be multiples of 8 elements");
    if (p.q_rs < D || p.k_rs < D || p.v_rs < D || p.o_rs < D)
        return fail("mi_linear_attn_relu_forward: row stride smaller than heads*head_dim");
    const uintptr_t al = reinterpret_cast<uintptr_t>(a->q) | reinterpret_cast<uintptr_t>(a->k) | reinterpret_cast<uintptr_t>(a->v) |
                         reinterpret_cast<uintptr_t>(a->o) | reinterpret_cast<uintptr_t>(a->workspace);
    if (al & 15u) return fail("mi_linear_attn_relu_forward: pointers must be 16-byte aligned");
    p.eps = a->eps;
    p.ws = static_cast<float*>(a->workspace);
    p.tokens_per_group = 0;
    hipStream_t st = mi::resolve_stream(a->stream);
    const int n_cu = mi::device_cu_count();
    return mi::launch_t<__bf16>(p, a->head_dim, a->accumulate_state != 0, n_cu, st);
}

}  // extern "C"
