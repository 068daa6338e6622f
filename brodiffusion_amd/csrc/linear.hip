// Y = X W^T + b for fp16 / bf16 on gfx950: the projection GEMM around the attention core.
//
// X is (M, K) and W is (N, K), both with the contraction index contiguous, which is exactly the operand layout of
// v_mfma_f32_32x32x16: a lane reads 8 consecutive contraction elements of ONE row of either operand. The product is
// computed transposed (MFMA rows = output features, MFMA columns = tokens), so a lane ends up with 4 consecutive
// output features of one token per accumulator group and writes them as one 8-byte store, bias added in FP32 before
// the single rounding.
//
// Work group: 256 threads = 4 wavefronts in a 2 x 2 arrangement over a BM x BN output tile, contraction step 64.
// Operand tiles go global -> registers -> LDS with 16-byte accesses, double buffered so that the loads of step t+1 are
// in flight while step t multiplies; one barrier per step. LDS rows are 144 bytes (128 + 16): 16 consecutive rows start
// on distinct 16-byte bank groups, so the ds_read_b128 fragment reads are conflict free.
// Up to three problems share one launch (blockIdx.y): the Q, K and V projections of an attention block.
// Large problems with 16-bit weights go to the 256 x 256-tile kernel of linear_dma.hip instead (launch_linear decides).
#include "internal.h"

namespace mi {
namespace gemm {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct Mma;
template <> struct Mma<__bf16> {
    using v8 = bf16x8;
    using v4 = bf16x4;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
};
template <> struct Mma<_Float16> {
    using v8 = f16x8;
    using v4 = f16x4;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
};

constexpr int kBK = 64;                // contraction elements per step
constexpr int kRowBytes = kBK * 2 + 16;  // LDS row stride
constexpr int kThreads = 256;

// One 16-byte chunk column (tid % 8) and 32 rows per pass: ROWS / 32 loads per thread and tile.
// GATED (the W tile of the GEGLU form): the tile's 32-row groups alternate between the value half and the gate half
// of W — group 2j holds value features row0 + 32 j .., group 2j+1 the gate rows of the same features (n_rows further
// down) — so that one wavefront's two 32-feature blocks are the value and the gate of the same outputs.
template <int ROWS, bool GATED = false>
__device__ __forceinline__ void load_tile(u32x4 (&r)[ROWS / 32], const char* base, long ld, int row0, int n_rows,
                                          int k0, int K, int tid) {
    const int kc = k0 + (tid & 7) * 8;
    const long col = kc < K ? kc : 0;   // chunks past the end of the contraction are blanked when they are stored
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        int row;
        if constexpr (GATED) row = min(row0 + (tid >> 3) + 32 * (i >> 1), n_rows - 1) + (i & 1) * n_rows;
        else row = min(row0 + (tid >> 3) + 32 * i, n_rows - 1);  // rows past the end repeat the last one; never stored
        r[i] = *reinterpret_cast<const u32x4*>(base + (static_cast<long>(row) * ld + col) * 2);
    }
}
// INT8 weight tile: the same 8 contraction elements per thread and row are 8 bytes in memory; they are widened to T
// (exactly: |w| <= 128) on their way to LDS, the per-row scale is applied to the accumulator in the epilogue.
template <int ROWS>
__device__ __forceinline__ void load_tile_int8(u32x2 (&raw)[ROWS / 32], const char* base, long ld, int row0, int n_rows,
                                               int k0, int K, int tid) {
    const int kc = k0 + (tid & 7) * 8;
    const long col = kc < K ? kc : 0;
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        const int row = min(row0 + (tid >> 3) + 32 * i, n_rows - 1);
        raw[i] = *reinterpret_cast<const u32x2*>(base + static_cast<long>(row) * ld + col);
    }
}

// Registers -> LDS. Nothing touches the loaded registers before this point, so the wait for the loads sits here,
// behind the MFMAs of the tile that is in LDS, and not where the loads are issued (blanking the chunks past the end
// of the contraction, or widening the weight bytes, right after the load made every step wait out the full memory
// latency before its first MFMA). k_ok: the thread's 8 contraction elements lie inside K.
template <int ROWS>
__device__ __forceinline__ void store_tile(const u32x4 (&r)[ROWS / 32], char* lds, int tid, bool k_ok) {
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i)
        *reinterpret_cast<u32x4*>(lds + ((tid >> 3) + 32 * i) * kRowBytes + (tid & 7) * 16) = k_ok ? r[i] : u32x4{0u, 0u, 0u, 0u};
}
template <typename T, int ROWS>
__device__ __forceinline__ void store_tile_int8(const u32x2 (&raw)[ROWS / 32], char* lds, int tid, bool k_ok) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    typedef signed char c8 __attribute__((ext_vector_type(8)));
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        const c8 q = __builtin_bit_cast(c8, raw[i]);
        t8 w;
#pragma unroll
        for (int e = 0; e < 8; ++e) w[e] = static_cast<T>(static_cast<float>(q[e]));
        *reinterpret_cast<u32x4*>(lds + ((tid >> 3) + 32 * i) * kRowBytes + (tid & 7) * 16) =
            k_ok ? __builtin_bit_cast(u32x4, w) : u32x4{0u, 0u, 0u, 0u};
    }
}

// GEGLU: W is (2 N, K) and bias (2 N): value half on top, gate half below; the output (M, N) is
// value * gelu_exact(gate) (diffusers' GEGLU with the erf form of GELU). A work group's 128 W-tile rows are 64 output
// features times {value, gate}; each wavefront holds both accumulators of its 32 features, so the product of the two
// halves never leaves registers and the (M, 2 N) intermediate does not exist.
// W8: W is INT8 (N, K) with one FP32 scale per row (LinearProblem::w_scale): Y = (X Wq^T) * scale + bias.
template <typename T, int BM, int BN, bool GEGLU = false, bool W8 = false>
__global__ __launch_bounds__(kThreads) void linear_kernel(const LinearBatch batch) {
    using M = Mma<T>;
    constexpr int TM = BM / 64, TN = BN / 64;  // 32 x 32 blocks per wavefront along tokens / features
    static_assert(!GEGLU || TN == 2, "the GEGLU form pairs the two feature blocks of a wavefront");
    static_assert(!(GEGLU && W8), "no INT8-weight GEGLU form");
    constexpr int BN_OUT = GEGLU ? BN / 2 : BN;   // output features per tile
    constexpr int X_BYTES = BM * kRowBytes, W_BYTES = BN * kRowBytes;
    extern __shared__ __attribute__((aligned(16))) char lds[];  // [2][X tile ; W tile]

    const LinearProblem& p = batch.p[blockIdx.y];
    const int tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int tiles_m = (p.M + BM - 1) / BM;
    if (static_cast<int>(blockIdx.x) >= tiles_m * tiles_n) return;  // uniform: this problem has fewer tiles than the grid
    const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN_OUT;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int lq = lane & 31, lh = lane >> 5;
    const int wm = wave & 1, wn = wave >> 1;
    const char* xg = static_cast<const char*>(p.x);
    const char* wg = static_cast<const char*>(p.w);

    f32x16 acc[TN][TM];
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

    // While tile t is multiplied out of LDS, tile t + 1 is on its way into registers; it goes to the other LDS buffer at
    // the end of the step. (The loads stay under `if (more)`: issued unconditionally, the compiler sinks them behind
    // the MFMAs, next to the store, and the step waits out the memory latency again. A second register set, two tiles
    // ahead, and 256 x 256 tiles with 8 wavefronts measured no faster.)
    u32x4 xr[BM / 32];
    u32x4 wr[W8 ? 1 : BN / 32];
    u32x2 wr8[W8 ? BN / 32 : 1];
    auto load_tiles = [&](int k0) {
        load_tile<BM>(xr, xg, p.ldx, m0, p.M, k0, p.K, tid);
        if constexpr (W8) load_tile_int8<BN>(wr8, wg, p.ldw, n0, p.N, k0, p.K, tid);
        else load_tile<BN, GEGLU>(wr, wg, p.ldw, n0, p.N, k0, p.K, tid);
    };
    auto store_tiles = [&](char* dst, int k0) {
        const bool k_ok = k0 + (tid & 7) * 8 < p.K;
        store_tile<BM>(xr, dst, tid, k_ok);
        if constexpr (W8) store_tile_int8<T, BN>(wr8, dst + X_BYTES, tid, k_ok);
        else store_tile<BN>(wr, dst + X_BYTES, tid, k_ok);
    };
    load_tiles(0);
    store_tiles(lds, 0);
    __syncthreads();

    const int n_steps = (p.K + kBK - 1) / kBK;
    for (int t = 0; t < n_steps; ++t) {
        const char* cur = lds + (t & 1) * (X_BYTES + W_BYTES);
        char* nxt = lds + ((t + 1) & 1) * (X_BYTES + W_BYTES);
        const bool more = t + 1 < n_steps;
        if (more) load_tiles((t + 1) * kBK);
        const char* xs = cur + (wm * TM * 32 + lq) * kRowBytes + lh * 16;
        const char* ws = cur + X_BYTES + (wn * TN * 32 + lq) * kRowBytes + lh * 16;
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
            typename M::v8 xf[TM], wf[TN];
#pragma unroll
            for (int b = 0; b < TM; ++b) xf[b] = *reinterpret_cast<const typename M::v8*>(xs + b * 32 * kRowBytes + kk * 32);
#pragma unroll
            for (int a = 0; a < TN; ++a) wf[a] = *reinterpret_cast<const typename M::v8*>(ws + a * 32 * kRowBytes + kk * 32);
#pragma unroll
            for (int a = 0; a < TN; ++a)
#pragma unroll
                for (int b = 0; b < TM; ++b) acc[a][b] = M::run(wf[a], xf[b], acc[a][b]);
        }
        if (more) store_tiles(nxt, (t + 1) * kBK);
        __syncthreads();
    }

    // acc[a][b][4g + i]: feature n0 + (wn*TN + a)*32 + 8g + 4*lh + i of token m0 + (wm*TM + b)*32 + lq
    char* yg = static_cast<char*>(p.y);
    const T* bias = static_cast<const T*>(p.bias);
    if constexpr (GEGLU) {
        // acc[0] = value, acc[1] = gate of features n0 + wn*32 + 8g + 4*lh + i
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = n0 + wn * 32 + 8 * g + 4 * lh;
            if (n >= p.N) continue;
            float bv[4] = {0.f, 0.f, 0.f, 0.f}, bg[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
                const typename M::v4 b4 = *reinterpret_cast<const typename M::v4*>(bias + n);
                const typename M::v4 g4 = *reinterpret_cast<const typename M::v4*>(bias + p.N + n);
#pragma unroll
                for (int i = 0; i < 4; ++i) { bv[i] = static_cast<float>(b4[i]); bg[i] = static_cast<float>(g4[i]); }
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int m = m0 + (wm * TM + b) * 32 + lq;
                if (m >= p.M) continue;
                typename M::v4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float val = acc[0][b][4 * g + i] + bv[i];
                    const float gate = acc[1][b][4 * g + i] + bg[i];
                    o[i] = static_cast<T>(val * (0.5f * gate * (1.0f + erff(gate * 0.70710678118654752f))));
                }
                *reinterpret_cast<typename M::v4*>(yg + (static_cast<long>(m) * p.ldy + n) * 2) = o;
            }
        }
        return;
    }
#pragma unroll
    for (int a = 0; a < TN; ++a) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = n0 + (wn * TN + a) * 32 + 8 * g + 4 * lh;
            if (n >= p.N) continue;  // N is a multiple of 8, so the 4 features are in or out together
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias) {
                const typename M::v4 b4 = *reinterpret_cast<const typename M::v4*>(bias + n);
#pragma unroll
                for (int i = 0; i < 4; ++i) bv[i] = static_cast<float>(b4[i]);
            }
            float sc[4] = {1.f, 1.f, 1.f, 1.f};
            if constexpr (W8) {
#pragma unroll
                for (int i = 0; i < 4; ++i) sc[i] = p.w_scale[n + i];
            }
#pragma unroll
            for (int b = 0; b < TM; ++b) {
                const int m = m0 + (wm * TM + b) * 32 + lq;
                if (m >= p.M) continue;
                typename M::v4 o;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if constexpr (W8) o[i] = static_cast<T>(__builtin_fmaf(acc[a][b][4 * g + i], sc[i], bv[i]));
                    else o[i] = static_cast<T>(acc[a][b][4 * g + i] + bv[i]);
                }
                *reinterpret_cast<typename M::v4*>(yg + (static_cast<long>(m) * p.ldy + n) * 2) = o;
            }
        }
    }
}

template <typename T, int BM, int BN, bool GEGLU = false, bool W8 = false>
int launch_tiles(const LinearBatch& batch, int n_problems, hipStream_t st) {
    constexpr int BN_OUT = GEGLU ? BN / 2 : BN;
    int max_tiles = 0;
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        max_tiles = max(max_tiles, ((p.M + BM - 1) / BM) * ((p.N + BN_OUT - 1) / BN_OUT));
    }
    constexpr size_t lds = 2 * static_cast<size_t>(BM + BN) * kRowBytes;
    static_assert(lds <= 160 * 1024, "operand ring exceeds the LDS of a compute unit");
    auto kern = linear_kernel<T, BM, BN, GEGLU, W8>;
    if (lds > 64 * 1024) {
        static thread_local bool raised = false;
        if (!raised) {
            MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            raised = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(max_tiles, n_problems), dim3(kThreads), lds, st, batch);
    MI_HIP_CHECK(hipGetLastError());
    return 0;
}

template <typename T>
int launch_t(const LinearBatch& batch, int n_problems, hipStream_t st, bool geglu) {
    if (geglu) {
        // 64-token tiles unless 128-token tiles alone fill the GPU twice over
        const long big = static_cast<long>((batch.p[0].M + 127) / 128) * ((batch.p[0].N + 63) / 64);
        if (big >= 2L * device_cu_count() && batch.p[0].K >= 1024) return launch_tiles<T, 128, 128, true>(batch, 1, st);
        return launch_tiles<T, 64, 128, true>(batch, 1, st);
    }
    // 128 x 128 tiles when they alone fill the GPU twice over and the contraction is long enough to pay for their
    // longer prologue, else 64 x 64 (more, smaller work groups: the projections of one attention block are small
    // problems; Q, K, V of 8192 x 320 x 320 in one launch: 15 us with 64 x 64 tiles, 22 us with 128 x 128)
    long big = 0;
    int min_k = 0x7fffffff;
    for (int i = 0; i < n_problems; ++i) {
        big += static_cast<long>((batch.p[i].M + 127) / 128) * ((batch.p[i].N + 127) / 128);
        min_k = min(min_k, batch.p[i].K);
    }
    const bool w8 = batch.p[0].w_scale != nullptr;
    if (big >= 2L * device_cu_count() && min_k >= 1024)
        return w8 ? launch_tiles<T, 128, 128, false, true>(batch, n_problems, st) : launch_tiles<T, 128, 128>(batch, n_problems, st);
    return w8 ? launch_tiles<T, 64, 64, false, true>(batch, n_problems, st) : launch_tiles<T, 64, 64>(batch, n_problems, st);
}

}  // namespace gemm

int launch_linear(const LinearBatch& batch, int n_problems, int dtype, hipStream_t st, bool geglu) {
    if (geglu && n_problems != 1) return fail("linear: the GEGLU form takes one problem per launch");
    if (n_problems < 1 || n_problems > kMaxLinearProblems) return fail("linear: %d problems in one launch (1..%d)", n_problems, kMaxLinearProblems);
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        if (p.M <= 0 || p.N <= 0 || p.K <= 0) return fail("linear: empty problem %d (%d x %d x %d)", i, p.M, p.N, p.K);
        if (p.N % 8 || p.K % 8) return fail("linear: in_features %d and out_features %d must be multiples of 8", p.K, p.N);
        if ((p.w_scale != nullptr) != (batch.p[0].w_scale != nullptr)) return fail("linear: INT8 and 16-bit weights cannot share a launch");
        if (p.w_scale && geglu) return fail("linear: there is no INT8-weight GEGLU form");
        if (reinterpret_cast<uintptr_t>(p.w_scale) & 3u) return fail("linear: weight scales must be 4-byte aligned");
        if (p.ldx % 8 || p.ldw % 8 || p.ldy % 8) return fail("linear: row strides must be multiples of 8 elements");
        if (p.ldx < p.K || p.ldw < p.K || p.ldy < p.N) return fail("linear: a row stride is smaller than the row");
        const uintptr_t al = reinterpret_cast<uintptr_t>(p.x) | reinterpret_cast<uintptr_t>(p.w) |
                             reinterpret_cast<uintptr_t>(p.y) | reinterpret_cast<uintptr_t>(p.bias);
        if (!p.x || !p.w || !p.y) return fail("linear: null operand in problem %d", i);
        if (al & 15u) return fail("linear: operands must be 16-byte aligned");
        if (static_cast<long>((p.M + 63) / 64) * ((p.N + 63) / 64) > 0x7fffffffL) return fail("linear: problem too large for one launch");
    }
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_F16) return fail("linear: dtype %d is neither MI_DTYPE_F16 nor MI_DTYPE_BF16", dtype);
    if (!geglu && linear_dma_takes(batch, n_problems, device_cu_count())) return launch_linear_dma(batch, n_problems, dtype, st);
    if (dtype == MI_DTYPE_BF16) return gemm::launch_t<__bf16>(batch, n_problems, st, geglu);
    if (dtype == MI_DTYPE_F16) return gemm::launch_t<_Float16>(batch, n_problems, st, geglu);
    return fail("linear: dtype %d is neither MI_DTYPE_F16 nor MI_DTYPE_BF16", dtype);
}

}  // namespace mi
