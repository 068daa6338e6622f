// Y = X W^T + b for fp16 / bf16 on gfx950: the projection GEMM around the attention core.
//
// X is (M, K) and W is (N, K), both with the contraction index contiguous, which is exactly the operand layout of
// v_mfma_f32_32x32x16: a lane reads 8 consecutive contraction elements of ONE row of either operand. The product is
// computed transposed (MFMA rows = output features, MFMA columns = tokens), so a lane ends up with 4 consecutive
// output features of one token per accumulator group; bias is added in FP32 before the single rounding and the tile
// leaves through LDS as whole 16-byte pieces of rows of Y.
//
// Streaming form (linear_kernel): 256 threads = 4 wavefronts in a 2 x 2 arrangement over a BM x BN output tile,
// contraction step 64. Operand tiles go global -> registers -> LDS with 16-byte accesses, double buffered so that the
// loads of step t+1 are in flight while step t multiplies; one barrier per step. LDS rows are 144 bytes (128 + 16): 16
// consecutive rows start on distinct 16-byte bank groups, so the ds_read_b128 fragment reads are conflict free.
// Up to three problems share one launch (blockIdx.y): the Q, K and V projections of an attention block.
// Ring form (linear_ring_kernel): work groups that stay and walk tiles with five contraction steps in flight, for the
// GEGLU FF1 of the U-Net (launch_t decides).
// Large problems with 16-bit weights go to the 256 x 256-tile kernel of linear_dma.hip instead (launch_linear decides).
#include <type_traits>
#include <utility>

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
constexpr int kRing = 5;               // contraction steps in flight in the ring form (K a multiple of 320)

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
template <int ROWS, bool GATED = false>
__device__ __forceinline__ void load_tile_int8(u32x2 (&raw)[ROWS / 32], const char* base, long ld, int row0, int n_rows,
                                               int k0, int K, int tid) {
    const int kc = k0 + (tid & 7) * 8;
    const long col = kc < K ? kc : 0;
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        int row;
        if constexpr (GATED) row = min(row0 + (tid >> 3) + 32 * (i >> 1), n_rows - 1) + (i & 1) * n_rows;   // as in load_tile
        else row = min(row0 + (tid >> 3) + 32 * i, n_rows - 1);
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

// x * Phi(x), the erf form of GELU (gelu_exact_scalar, src/fused_transformer.cu:89-92), branch free. With z = |x| / sqrt 2,
// erfc(z) = t exp(-z^2 + P(t)), t = 1 / (1 + z / 2) (the Chebyshev fit of Numerical Recipes' erfcc, fractional error below
// 1.2e-7 for all z >= 0), and Phi(x) = erfc(z) / 2 for x < 0, 1 - erfc(z) / 2 otherwise - so the left tail keeps its
// relative accuracy, which the sum 1 + erf loses to cancellation. Here in base 2 with the constants folded: the
// coefficients of P are multiplied by log2 e, its constant term also takes the factor 1/2 (-1 in the exponent), and
// z^2 log2 e = (|x| sqrt(log2 e / 2))^2. 19 FP32 instructions and 2 transcendentals; against x Phi(x) in double the
// relative error stays below 4e-6 for |x| < 6 and 1.5e-5 down to x = -12.
__device__ __forceinline__ float gelu_erf(float x) {
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(ax, 0.35355339059327373f, 1.f));
    const float zs = ax * 0.849321800288f;
    float q = 0.246517298f;
    q = __builtin_fmaf(q, t, -1.18611495f);
    q = __builtin_fmaf(q, t, 2.14747446f);
    q = __builtin_fmaf(q, t, -1.63775315f);
    q = __builtin_fmaf(q, t, 0.402321582f);
    q = __builtin_fmaf(q, t, -0.26875686f);
    q = __builtin_fmaf(q, t, 0.139630057f);
    q = __builtin_fmaf(q, t, 0.539700616f);
    q = __builtin_fmaf(q, t, 1.4427292f);
    q = __builtin_fmaf(q, t, -2.82574822f);
    const float half_erfc = t * __builtin_amdgcn_exp2f(__builtin_fmaf(-zs, zs, q));
    return x * (x < 0.f ? half_erfc : 1.f - half_erfc);
}

// acc * scale + bias of the INT8-weight forms as an FP32 value of its own. Left to itself the compiler merges the
// multiply-add with the rounding to T that follows (v_fma_mixlo_f16: one rounding of the exact result) in some places and
// not in others, and the plain and the GEGLU form of the same layer then disagree by a unit in the last place in about 3
// outputs of 100 000; as a separate FP32 operation it is the FP32 multiply-add and conversion of the reference's kernel
// everywhere.
__device__ __forceinline__ float scaled_acc(float acc, float scale, float bias) {
    float r = __builtin_fmaf(acc, scale, bias);
    asm volatile("" : "+v"(r));
    return r;
}

// What the two kernels below share: the MFMA step and the epilogue of a BM x BN tile held by WM x WN wavefronts. GEGLU: W is (2 N, K) and bias (2 N): value half on top, gate half below; the output (M, N) is
// value * gelu_exact(gate) (diffusers' GEGLU with the erf form of GELU). A work group's 128 W-tile rows are 64 output
// features times {value, gate}; each wavefront holds both accumulators of its 32 features, so the product of the two
// halves never leaves registers and the (M, 2 N) intermediate does not exist.
// W8: W is INT8 (N, K) with one FP32 scale per row (LinearProblem::w_scale): Y = (X Wq^T) * scale + bias.
// GEGLU with W8 (2 N scales): the reference composes this one from its INT8-weight linear layer and a GEGLU pass over a
// 16-bit (M, 2 N) buffer (src/fused_transformer.cu:360-396); here the two halves are rounded to T at the same point,
// in registers, so the result is the composition's without the buffer.
template <typename T, int BM, int BN, bool GEGLU, bool W8, int WM = 2, int WN = 2>
struct TileMath {
    using M = Mma<T>;
    using V4 = typename M::v4;
    static constexpr int NT = 64 * WM * WN;                       // threads: WM x WN wavefronts over tokens x features
    static constexpr int TM = BM / (32 * WM), TN = BN / (32 * WN);  // 32 x 32 blocks per wavefront along tokens / features
    static_assert(!GEGLU || TN == 2, "the GEGLU form pairs the two feature blocks of a wavefront");
    static constexpr int BN_OUT = GEGLU ? BN / 2 : BN;   // output features per tile
    static constexpr int X_BYTES = BM * kRowBytes, W_BYTES = BN * kRowBytes;
    static constexpr int kOutRow = BN_OUT * 2 + 16;      // staged output row (bytes)
    static constexpr int kOutBytes = BM * kOutRow;

    int tid, lq, lh, wm, wn;
    __device__ __forceinline__ explicit TileMath(int tid_) : tid(tid_) {
        const int lane = tid & 63, wave = tid >> 6;
        lq = lane & 31; lh = lane >> 5; wm = wave % WM; wn = wave / WM;
    }
    static __device__ __forceinline__ void clear(f32x16 (&acc)[TN][TM]) {
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int b = 0; b < TM; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;
    }
    // The bias of this lane's features of the tile at feature n0, requested long before the epilogue (there each of these
    // loads would be a memory latency of its own). Straight-line code: lanes without a bias read the first bytes of W and
    // blank what they got, so that no wait for these loads is placed before the operand loads that follow.
    // GEGLU: [0] = value half, [1] = gate half.
    __device__ __forceinline__ void request_bias(V4 (&braw)[TN][4], const LinearProblem& p, int n0) const {
        const T* bias = static_cast<const T*>(p.bias);
#pragma unroll
        for (int a = 0; a < TN; ++a)
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int feat = GEGLU ? n0 + wn * 32 + 8 * g + 4 * lh : n0 + (wn * TN + a) * 32 + 8 * g + 4 * lh;
                const bool there = bias != nullptr && feat < p.N;
                const T* src = there ? bias + feat + (GEGLU ? a * p.N : 0) : static_cast<const T*>(p.w);
                const V4 raw = *reinterpret_cast<const V4*>(src);
                const V4 zero = {static_cast<T>(0.f), static_cast<T>(0.f), static_cast<T>(0.f), static_cast<T>(0.f)};
                braw[a][g] = there ? raw : zero;
            }
    }
    // the four k-substeps of 16 of one step for every 32 x 32 block of this wavefront, operands from the LDS tile pair at `cur`
    __device__ __forceinline__ void multiply(f32x16 (&acc)[TN][TM], const char* cur) const {
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
    }
    // acc[a][b][4g + i]: feature n0 + (wn*TN + a)*32 + 8g + 4*lh + i of token m0 + (wm*TM + b)*32 + lq.
    // The results leave through LDS (`stage`, kOutBytes, not in use by anything else): a lane holds 4 features of one token
    // per group, and written from there a wavefront's store instruction would touch 32 rows of Y with 16 bytes each.
    // Staged, consecutive threads write consecutive 16-byte pieces of a row.
    __device__ __forceinline__ void write_tile(const f32x16 (&acc)[TN][TM], const V4 (&braw)[TN][4], const LinearProblem& p, char* stage,
                                               int m0, int n0) const {
        if constexpr (GEGLU) {
            // acc[0] = value, acc[1] = gate of features n0 + wn*32 + 8g + 4*lh + i
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const int feat = wn * 32 + 8 * g + 4 * lh;
                float bv[4], bg[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) { bv[i] = static_cast<float>(braw[0][g][i]); bg[i] = static_cast<float>(braw[1][g][i]); }
                float sv[4] = {1.f, 1.f, 1.f, 1.f}, sg[4] = {1.f, 1.f, 1.f, 1.f};
                if constexpr (W8) {
                    if (n0 + feat < p.N) {   // N is a multiple of 8, so the 4 features are in or out together
#pragma unroll
                        for (int i = 0; i < 4; ++i) { sv[i] = p.w_scale[n0 + feat + i]; sg[i] = p.w_scale[p.N + n0 + feat + i]; }
                    }
                }
#pragma unroll
                for (int b = 0; b < TM; ++b) {
                    V4 o;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float val, gate;
                        if constexpr (W8) {
                            val = static_cast<float>(static_cast<T>(scaled_acc(acc[0][b][4 * g + i], sv[i], bv[i])));
                            gate = static_cast<float>(static_cast<T>(scaled_acc(acc[1][b][4 * g + i], sg[i], bg[i])));
                        } else {
                            val = acc[0][b][4 * g + i] + bv[i];
                            gate = acc[1][b][4 * g + i] + bg[i];
                        }
                        o[i] = static_cast<T>(val * gelu_erf(gate));
                    }
                    *reinterpret_cast<V4*>(stage + ((wm * TM + b) * 32 + lq) * kOutRow + feat * 2) = o;
                }
            }
        } else {
#pragma unroll
            for (int a = 0; a < TN; ++a) {
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    const int feat = (wn * TN + a) * 32 + 8 * g + 4 * lh;
                    float bv[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) bv[i] = static_cast<float>(braw[a][g][i]);
                    float sc[4] = {1.f, 1.f, 1.f, 1.f};
                    if constexpr (W8) {
                        if (n0 + feat < p.N) {   // N is a multiple of 8, so the 4 features are in or out together
#pragma unroll
                            for (int i = 0; i < 4; ++i) sc[i] = p.w_scale[n0 + feat + i];
                        }
                    }
#pragma unroll
                    for (int b = 0; b < TM; ++b) {
                        V4 o;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            if constexpr (W8) o[i] = static_cast<T>(scaled_acc(acc[a][b][4 * g + i], sc[i], bv[i]));
                            else o[i] = static_cast<T>(acc[a][b][4 * g + i] + bv[i]);
                        }
                        *reinterpret_cast<V4*>(stage + ((wm * TM + b) * 32 + lq) * kOutRow + feat * 2) = o;
                    }
                }
            }
        }
        __syncthreads();
        char* yg = static_cast<char*>(p.y);
        constexpr int PPR = BN_OUT / 8;   // 16-byte pieces per staged row
#pragma unroll
        for (int idx = tid; idx < BM * PPR; idx += NT) {
            const int row = idx / PPR, piece = idx % PPR;
            if (m0 + row < p.M && n0 + piece * 8 < p.N)
                *reinterpret_cast<u32x4*>(yg + (static_cast<long>(m0 + row) * p.ldy + n0 + piece * 8) * 2) =
                    *reinterpret_cast<const u32x4*>(stage + row * kOutRow + piece * 16);
        }
    }
};

// The streaming form: one work group per output tile, one contraction step prefetched while the previous one is multiplied.
template <typename T, int BM, int BN, bool GEGLU = false, bool W8 = false>
__global__ __launch_bounds__(kThreads) void linear_kernel(const LinearBatch batch) {
    using TM_ = TileMath<T, BM, BN, GEGLU, W8>;
    constexpr int TM = TM_::TM, TN = TM_::TN, BN_OUT = TM_::BN_OUT, X_BYTES = TM_::X_BYTES, W_BYTES = TM_::W_BYTES;
    static_assert(TM_::kOutBytes <= 2 * (X_BYTES + W_BYTES), "the staged output fits the operand buffers");
    extern __shared__ __attribute__((aligned(16))) char lds[];  // [2][X tile ; W tile]

    const LinearProblem& p = batch.p[blockIdx.y];
    const int tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int tiles_m = (p.M + BM - 1) / BM;
    if (static_cast<int>(blockIdx.x) >= tiles_m * tiles_n) return;  // uniform: this problem has fewer tiles than the grid
    const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN_OUT;

    const int tid = threadIdx.x;
    const TM_ tm(tid);
    const char* xg = static_cast<const char*>(p.x);
    const char* wg = static_cast<const char*>(p.w);

    f32x16 acc[TN][TM];
    TM_::clear(acc);
    typename TM_::V4 braw[TN][4];
    tm.request_bias(braw, p, n0);

    // While tile t is multiplied out of LDS, tile t + 1 is on its way into registers; it goes to the other LDS buffer at
    // the end of the step. (The loads stay under `if (more)`: issued unconditionally, the compiler sinks them behind
    // the MFMAs, next to the store, and the step waits out the memory latency again. A second register set, two tiles
    // ahead, and 256 x 256 tiles with 8 wavefronts measured no faster.)
    u32x4 xr[BM / 32];
    u32x4 wr[W8 ? 1 : BN / 32];
    u32x2 wr8[W8 ? BN / 32 : 1];
    auto load_tiles = [&](int k0) {
        load_tile<BM>(xr, xg, p.ldx, m0, p.M, k0, p.K, tid);
        if constexpr (W8) load_tile_int8<BN, GEGLU>(wr8, wg, p.ldw, n0, p.N, k0, p.K, tid);
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
        tm.multiply(acc, cur);
        if (more) store_tiles(nxt, (t + 1) * kBK);
        __syncthreads();
    }
    tm.write_tile(acc, braw, p, lds, m0, n0);
}

// The ring form, for contractions that are a multiple of kRing steps (the channel counts of the U-Net: 320, 640, 1280 and
// their FF multiples). A work group of the streaming form lives a few microseconds, most of them waiting: every step for
// the one tile it prefetched, at the start for its first, and the tile's few hundred cycles of MFMAs hide none of it.
// Here a work group stays and walks output tiles (a contiguous run per XCD, so that the tiles sharing X rows meet in one
// L2), and the operand tiles of kRing consecutive steps are in flight at any time, across tile boundaries: the registers
// of step t + 1 go to LDS during step t and are at once requested again for step t + 1 + kRing (of this output tile or of
// the next). All loads are unconditional, straight-line code (past the last tile they re-read the first rows of the
// operands), so the waits the compiler places count exactly, and nothing ever waits for a store.
template <typename T, int BM, int BN, bool GEGLU = false, int WM = 2, int WN = 2>
__global__ __launch_bounds__(64 * WM * WN) void linear_ring_kernel(const LinearBatch batch) {
    using TM_ = TileMath<T, BM, BN, GEGLU, false, WM, WN>;
    constexpr int RP = TM_::NT / 8;             // tile rows per pass of the work group (8 threads per 128-byte row piece)
    constexpr int XL = BM / RP, WL = BN / RP;   // loads per thread, operand and step
    static_assert(BM % RP == 0 && BN % RP == 0 && RP % 32 == 0, "whole passes; a pass covers whole 32-row groups");
    constexpr int TM = TM_::TM, TN = TM_::TN, BN_OUT = TM_::BN_OUT, X_BYTES = TM_::X_BYTES, W_BYTES = TM_::W_BYTES;
    constexpr int R = kRing;
    extern __shared__ __attribute__((aligned(16))) char lds[];  // [2][X tile ; W tile], then the staged output
    char* const stage = lds + 2 * (X_BYTES + W_BYTES);

    const LinearProblem& p = batch.p[blockIdx.y];
    const int tiles_n = (p.N + BN_OUT - 1) / BN_OUT;
    const int tiles_m = (p.M + BM - 1) / BM;
    const int n_tiles = tiles_m * tiles_n;
    // consecutive work-group ids go to the 8 XCDs in turn: every XCD takes a contiguous run of tiles
    const int run = (n_tiles + 7) >> 3;
    const int stride = static_cast<int>(gridDim.x) >> 3;
    const int run_end = min(((static_cast<int>(blockIdx.x) & 7) + 1) * run, n_tiles);
    int tile = (static_cast<int>(blockIdx.x) & 7) * run + (static_cast<int>(blockIdx.x) >> 3);
    if (tile >= run_end) return;   // uniform

    const int tid = threadIdx.x;
    const TM_ tm(tid);
    const char* xg = static_cast<const char*>(p.x);
    const char* wg = static_cast<const char*>(p.w);
    const unsigned x_pitch = static_cast<unsigned>(p.ldx) * 2u, w_pitch = static_cast<unsigned>(p.ldw) * 2u;
    const unsigned k_bytes = static_cast<unsigned>(p.K) * 2u;

    // ── the load cursor: kRing steps ahead of the multiplication; 32-bit byte offsets from the operand bases ──
    int c_tile = tile;
    unsigned c_k = 0;                       // byte offset of the cursor's step in a row (uniform)
    const unsigned kcol = (tid & 7) * 16u;  // this thread's 16 bytes of a step
    unsigned xrow[XL], wrow[WL];
    auto cursor_rows = [&]() {
        if (c_tile < run_end) {
            const int m0 = (c_tile / tiles_n) * BM, n0 = (c_tile % tiles_n) * BN_OUT;
#pragma unroll
            for (int i = 0; i < XL; ++i) xrow[i] = static_cast<unsigned>(min(m0 + (tid >> 3) + RP * i, p.M - 1)) * x_pitch + kcol;
#pragma unroll
            for (int i = 0; i < WL; ++i) {
                // (GEGLU: the tile's 32-row groups alternate between the value and the gate half of W, see load_tile)
                const int r = (tid >> 3) + RP * i, grp = r >> 5;
                const int row = GEGLU ? min(n0 + 32 * (grp >> 1) + (r & 31), p.N - 1) + (grp & 1) * p.N : min(n0 + r, p.N - 1);
                wrow[i] = static_cast<unsigned>(row) * w_pitch + kcol;
            }
        } else {   // past the last tile: the first row of either operand
#pragma unroll
            for (int i = 0; i < XL; ++i) xrow[i] = kcol;
#pragma unroll
            for (int i = 0; i < WL; ++i) wrow[i] = kcol;
        }
    };
    u32x4 xs_[R][XL], ws_[R][WL];
    auto request = [&](auto s_tag) {
        constexpr int s = decltype(s_tag)::value;
#pragma unroll
        for (int i = 0; i < XL; ++i) xs_[s][i] = *reinterpret_cast<const u32x4*>(xg + (xrow[i] + c_k));
#pragma unroll
        for (int i = 0; i < WL; ++i) ws_[s][i] = *reinterpret_cast<const u32x4*>(wg + (wrow[i] + c_k));
        c_k += kBK * 2;
        if (c_k == k_bytes) {   // uniform: on to the next output tile of this work group
            c_k = 0;
            c_tile += stride;
            cursor_rows();
        }
    };
    auto to_lds = [&](auto s_tag, char* dst) {
        constexpr int s = decltype(s_tag)::value;
#pragma unroll
        for (int i = 0; i < XL; ++i) *reinterpret_cast<u32x4*>(dst + ((tid >> 3) + RP * i) * kRowBytes + (tid & 7) * 16) = xs_[s][i];
#pragma unroll
        for (int i = 0; i < WL; ++i) *reinterpret_cast<u32x4*>(dst + X_BYTES + ((tid >> 3) + RP * i) * kRowBytes + (tid & 7) * 16) = ws_[s][i];
    };
    cursor_rows();
    [&]<int... S>(std::integer_sequence<int, S...>) { (request(std::integral_constant<int, S>{}), ...); }(std::make_integer_sequence<int, R>{});
    to_lds(std::integral_constant<int, 0>{}, lds);
    request(std::integral_constant<int, 0>{});
    __syncthreads();

    const int groups = p.K / (R * kBK);
    int par = 0;   // LDS buffer of the step about to be multiplied
    f32x16 acc[TN][TM];
    for (; tile < run_end; tile += stride) {
        const int m0 = (tile / tiles_n) * BM, n0 = (tile % tiles_n) * BN_OUT;
        typename TM_::V4 braw[TN][4];
        tm.request_bias(braw, p, n0);
        TM_::clear(acc);
        int g = 0;
        do {   // (at least one group: a loop that may not run would make the wait for the bias a wait for every load)
            [&]<int... S>(std::integer_sequence<int, S...>) {
                ([&] {
                    // step S of the group: the registers of the following step go to the other buffer and are requested anew
                    constexpr int nxt = (S + 1) % R;
                    to_lds(std::integral_constant<int, nxt>{}, lds + (par ^ 1) * (X_BYTES + W_BYTES));
                    request(std::integral_constant<int, nxt>{});
                    tm.multiply(acc, lds + par * (X_BYTES + W_BYTES));
                    __syncthreads();
                    par ^= 1;
                }(), ...);
            }(std::make_integer_sequence<int, R>{});
        } while (++g < groups);
        tm.write_tile(acc, braw, p, stage, m0, n0);
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
    // (launched by name: a launch through a pointer variable is dropped by this compiler when the host code is built with
    // -fsanitize=undefined)
    const void* const kern = reinterpret_cast<const void*>(&linear_kernel<T, BM, BN, GEGLU, W8>);
    if (lds > 64 * 1024) {
        static thread_local bool raised = false;
        if (!raised) {
            MI_HIP_CHECK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
            raised = true;
        }
    }
    hipLaunchKernelGGL((linear_kernel<T, BM, BN, GEGLU, W8>), dim3(max_tiles, n_problems), dim3(kThreads), lds, st, batch);
    MI_HIP_CHECK(hipGetLastError());
    return 0;
}

// The ring form: 16-bit weights, contractions that are a multiple of kRing steps, operands addressable with 32-bit byte
// offsets from their bases.
inline bool ring_form_takes(const LinearBatch& batch, int n_problems, bool geglu) {
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        if (p.w_scale != nullptr || p.K % (kRing * kBK) != 0) return false;
        if (static_cast<long>(p.M) * p.ldx * 2 >= (1L << 32) || static_cast<long>(p.N) * (geglu ? 2 : 1) * p.ldw * 2 >= (1L << 32)) return false;
    }
    return true;
}

template <typename T, int BM, int BN, bool GEGLU = false, int WM = 2, int WN = 2>
int launch_ring(const LinearBatch& batch, int n_problems, hipStream_t st) {
    using TM_ = TileMath<T, BM, BN, GEGLU, false, WM, WN>;
    int max_tiles = 0;
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        max_tiles = max(max_tiles, ((p.M + BM - 1) / BM) * ((p.N + TM_::BN_OUT - 1) / TM_::BN_OUT));
    }
    constexpr size_t lds = 2 * static_cast<size_t>(BM + BN) * kRowBytes + TM_::kOutBytes;
    static_assert(lds <= 160 * 1024, "operand buffers and staged output exceed the LDS of a compute unit");
    const void* const kern = reinterpret_cast<const void*>(&linear_ring_kernel<T, BM, BN, GEGLU, WM, WN>);
    static thread_local int per_cu = 0;   // work groups a compute unit holds at once
    if (per_cu == 0) {
        if (lds > 64 * 1024)
            MI_HIP_CHECK(hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds)));
        int n = 0;
        MI_HIP_CHECK(hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kern, TM_::NT, lds));
        per_cu = max(n, 1);
    }
    // as many work groups as the GPU holds at once, split over the problems; a multiple of 8 (one run of tiles per XCD)
    const int grid_x = min((max_tiles + 7) / 8 * 8, max(8, per_cu * device_cu_count() / n_problems / 8 * 8));
    hipLaunchKernelGGL((linear_ring_kernel<T, BM, BN, GEGLU, WM, WN>), dim3(grid_x, n_problems), dim3(TM_::NT), lds, st, batch);
    MI_HIP_CHECK(hipGetLastError());
    return 0;
}

template <typename T>
int launch_t(const LinearBatch& batch, int n_problems, hipStream_t st, bool geglu) {
    if (geglu) {
        // the ring form when its 128-token tiles give every compute unit two: FF1 of the U-Net's widest levels
        // (8192 x 320 -> 2 x 1280: 31 us against 40 for the streaming form, 33 with 256-token tiles, whose 640 tiles are
        // 2.5 per compute unit; 2048 x 640 -> 2 x 2560: 28 against 33)
        if (ring_form_takes(batch, 1, true) && static_cast<long>((batch.p[0].M + 127) / 128) * ((batch.p[0].N + 63) / 64) >= 2L * device_cu_count())
            return launch_ring<T, 128, 128, true, 4, 2>(batch, 1, st);
        // 64-token tiles unless 128-token tiles alone fill the GPU twice over
        const long big = static_cast<long>((batch.p[0].M + 127) / 128) * ((batch.p[0].N + 63) / 64);
        const bool w8g = batch.p[0].w_scale != nullptr;
        if (big >= 2L * device_cu_count() && batch.p[0].K >= 1024)
            return w8g ? launch_tiles<T, 128, 128, true, true>(batch, 1, st) : launch_tiles<T, 128, 128, true>(batch, 1, st);
        return w8g ? launch_tiles<T, 64, 128, true, true>(batch, 1, st) : launch_tiles<T, 64, 128, true>(batch, 1, st);
    }
    // 128 x 128 tiles when they alone fill the GPU twice over and the contraction is long enough to pay for their
    // longer prologue, else 64 x 64 (more, smaller work groups: the projections of one attention block are small
    // problems)
    long big = 0;
    int min_k = 0x7fffffff;
    for (int i = 0; i < n_problems; ++i) {
        big += static_cast<long>((batch.p[i].M + 127) / 128) * ((batch.p[i].N + 127) / 128);
        min_k = min(min_k, batch.p[i].K);
    }
    const bool w8 = batch.p[0].w_scale != nullptr;
    if (big >= 2L * device_cu_count() && min_k >= 1024)
        return w8 ? launch_tiles<T, 128, 128, false, true>(batch, n_problems, st) : launch_tiles<T, 128, 128>(batch, n_problems, st);
    // long contractions over few tiles (FF2 of the U-Net: 2048 x 2560 -> 640, 30 -> 21 us; 8192 x 1280 -> 320, 22 -> 17 us): the
    // ring form, whose five steps in flight shorten the per-step chain of memory latencies; at 320 it measures the same
    // (with many tiles per compute unit the streaming form's work groups cover for each other: 2048 x 640 -> 5120, 2560
    // tiles, 28 us against 34)
    long tiles64 = 0;
    for (int i = 0; i < n_problems; ++i) tiles64 += static_cast<long>((batch.p[i].M + 63) / 64) * ((batch.p[i].N + 63) / 64);
    if (min_k >= 2 * kRing * kBK && tiles64 <= 4L * device_cu_count() && ring_form_takes(batch, n_problems, false))
        return launch_ring<T, 64, 64>(batch, n_problems, st);
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
