// Y = X W^T + b for large problems on gfx950: 256 x 256 output tiles, 8 wavefronts, operand blocks moved global -> LDS
// by DMA into rings.
//
// The work group's 512 threads are 8 wavefronts in a 2 (feature halves) x 4 (token quarters) arrangement; a wavefront owns
// 128 features x 64 tokens = 4 x 2 accumulator blocks of v_mfma_f32_32x32x16 (128 registers). As in linear.hip the product
// is computed transposed (MFMA rows = features), so both operands are read along their contiguous contraction index.
//
// Operands arrive in blocks of 64 contraction elements: per operand a 256-row x 128-byte tile (32 KB) = 32 LDS-DMA
// instructions of 1 KB (8 rows each: whole 128-byte lines; with 64-byte row pieces the DMA path measured half the
// throughput, 33 instead of 60 bytes per clock and CU, which is no more than this kernel consumes), dealt out four per
// wavefront. An instruction deposits the 16-byte pieces of its 64 lanes back to back, so a tile row is 128 bytes in LDS
// with no padding; bank conflicts of the fragment reads (one row per lane, 16-byte pieces, 16 consecutive rows per phase)
// are avoided by an XOR swizzle applied for free on the global side: the piece that lands in position c of row r is piece
// c ^ ((r >> 1) & 7). X blocks live in a ring of two stages, W blocks in a ring of three (160 KB in all).
//
// A block is multiplied in two half-steps of 32 contraction elements (16 MFMAs per wavefront each). Half-step t of block b:
//   1. read the 12 fragments of half-step t + 1 into the other register set
//   2. issue this wavefront's 4 DMA instructions: first half of a block: W of block b + 2 (into the stage of W block b - 1);
//      second half: X of block b + 2 (into the stage of X block b, whose fragments are all in registers by now)
//   3. 16 MFMAs
//   4. first half: wait until all but this wavefront's 4 youngest DMA instructions have landed (X and W of block b + 1);
//      barrier
// The order of 1 and 2 matters: an LDS read issued behind an LDS-DMA load of the same wavefront does not return before
// that load has landed; issuing the DMA in two small bursts, a whole half-step before the next reads, keeps that wait short
// (one burst of 8 per block measured 25 % slower).
// The accumulators leave through LDS (bias added in FP32, one rounding) so that global stores are full 16-byte pieces of
// consecutive threads along a row.
#include <type_traits>
#include <utility>

#include "internal.h"

namespace mi {
namespace gemm_dma {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mma;
template <> struct Mma<__bf16> {
    using v8 = bf16x8;
    using v4 = bf16x4;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};
template <> struct Mma<_Float16> {
    using v8 = f16x8;
    using v4 = f16x4;
    static __device__ __forceinline__ f32x16 run(v8 a, v8 b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};

constexpr int kTile = 256;                       // tokens and features per work group
constexpr int kBK = 64;                          // contraction elements per block (one stage)
constexpr int kThreads = 512;
constexpr int kOpBytes = kTile * kBK * 2;        // one operand block in LDS
constexpr int kXStages = 2, kWStages = 3;
constexpr int kWRing = kXStages * kOpBytes;      // the W ring starts behind the X ring
constexpr int kOutStride = kTile * 2 + 16;       // staged output row (bytes)
constexpr int kLdsBytes = (kXStages + kWStages) * kOpBytes;
static_assert(kTile * kOutStride <= kLdsBytes, "the staged output fits the rings");
static_assert(kLdsBytes <= 160 * 1024, "LDS of a compute unit");

template <typename T>
__global__ void __launch_bounds__(kThreads, 2) linear_dma_kernel(const LinearBatch batch) {
    using M = Mma<T>;
    using V8 = typename M::v8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const LinearProblem& p = batch.p[blockIdx.y];
    const int tiles_n = (p.N + kTile - 1) / kTile;
    const int tiles_m = (p.M + kTile - 1) / kTile;
    const int n_tiles = tiles_m * tiles_n;
    // consecutive work-group ids go to the 8 XCDs in turn: give every XCD (one L2) a contiguous run of tiles, which
    // share their X rows and walk W together
    const int chunk = (n_tiles + 7) >> 3;
    // (the grid is sized for the problem of the launch with the most tiles: a smaller problem's run is shorter than the
    //  grid's, and a group past the end of its XCD's run would repeat a tile of the next XCD's)
    const int in_run = static_cast<int>(blockIdx.x) >> 3;
    const int logical = (static_cast<int>(blockIdx.x) & 7) * chunk + in_run;
    if (in_run >= chunk || logical >= n_tiles) return;
    const int m0 = (logical / tiles_n) * kTile, n0 = (logical % tiles_n) * kTile;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
    const int wn = wave & 1, wm = wave >> 1;

    // ── DMA duty: instructions 4 wave .. 4 wave + 3 of either operand; instruction j fills rows 8 j .. 8 j + 7 ──
    const unsigned char* xg = static_cast<const unsigned char*>(p.x) + static_cast<long>(m0) * p.ldx * 2;
    const unsigned char* wg = static_cast<const unsigned char*>(p.w) + static_cast<long>(n0) * p.ldw * 2;
    unsigned xoff[4], woff[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int j = 4 * wave + u;
        const int r = 8 * j + (lane >> 3);
        const int piece = (lane & 7) ^ ((r >> 1) & 7);
        xoff[u] = static_cast<unsigned>(min(r, p.M - 1 - m0)) * (static_cast<unsigned>(p.ldx) * 2u) + piece * 16u;
        woff[u] = static_cast<unsigned>(min(r, p.N - 1 - n0)) * (static_cast<unsigned>(p.ldw) * 2u) + piece * 16u;
    }
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)lds));
    auto dma = [&](unsigned voff, const unsigned char* base, unsigned dst) {
        // (the LDS destination travels in m0; the s_nop is the wait state an LDS-DMA instruction needs behind a write of m0)
        asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(base), "{m0}"(dst) : "memory");
    };
    auto dma_x = [&](int stage) {
        const unsigned dst = lds_base + stage * kOpBytes + 4 * wave * 1024;
#pragma unroll
        for (int u = 0; u < 4; ++u) dma(xoff[u], xg, dst + u * 1024);
        xg += kBK * 2;
    };
    auto dma_w = [&](int stage) {
        const unsigned dst = lds_base + kWRing + stage * kOpBytes + 4 * wave * 1024;
#pragma unroll
        for (int u = 0; u < 4; ++u) dma(woff[u], wg, dst + u * 1024);
        wg += kBK * 2;
    };

    // ── fragment reads: row lq of a 32-row block, 16-byte piece 4 h + 2 kc + lh of the row (swizzled position) ──
    const int f = (lq >> 1) & 7;
    unsigned frag[2][2];   // [half][kc]
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) frag[h][kc] = lq * 128 + (((4 * h + 2 * kc + lh) ^ f) << 4);
    const unsigned x_blk = wm * 64 * 128;                         // this wavefront's first token row, in bytes
    const unsigned w_blk = kWRing + wn * 128 * 128;
    V8 wf[2][4][2], xf[2][2][2];   // [register set][block][kc]
    // fragments of half-step t (block t / 2, half t % 2) into register set t % 2
    auto read_frags = [&](auto set_tag, int t) {
        constexpr int S = decltype(set_tag)::value;
        const int b = t >> 1;
        const unsigned char* xs = lds + (b & 1) * kOpBytes + x_blk;
        const unsigned char* ws = lds + (b % 3) * kOpBytes + w_blk;
#pragma unroll
        for (int kc = 0; kc < 2; ++kc) {
            const unsigned fr = frag[S][kc];
#pragma unroll
            for (int i = 0; i < 4; ++i) wf[S][i][kc] = *reinterpret_cast<const V8*>(ws + i * 4096 + fr);
#pragma unroll
            for (int j = 0; j < 2; ++j) xf[S][j][kc] = *reinterpret_cast<const V8*>(xs + j * 4096 + fr);
        }
    };

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    const int nb = p.K / kBK;      // blocks
    const int nt = 2 * nb;         // half-steps
    // prologue: blocks 0 and 1 in LDS
    dma_x(0);
    dma_w(0);
    if (nb > 1) { dma_x(1); dma_w(1); }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;
    using Kc0 = std::integral_constant<int, 0>;
    using Kc1 = std::integral_constant<int, 1>;
    read_frags(Set0{}, 0);

    auto mfma_half = [&](auto set_tag, auto kc_tag) {
        constexpr int S = decltype(set_tag)::value, kc = decltype(kc_tag)::value;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = M::run(wf[S][i][kc], xf[S][j][kc], acc[i][j]);
    };
    // half-step t (set S = t % 2): fragment reads of half-step t + 1, then the DMA of half of the block after next
    auto feed = [&](auto set_tag, int t) -> bool {
        constexpr int S = decltype(set_tag)::value;
        read_frags(std::integral_constant<int, 1 - S>{}, t + 1);   // (behind the last half-step: a stage of no block, never used)
        const int nxt = (t >> 1) + 2;
        const bool more = nxt < nb;
        if (more) {
            if constexpr (S == 0) dma_w(nxt % 3);
            else dma_x(nxt & 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        return more;
    };
    auto close_half = [&](auto set_tag, bool more) {
        constexpr int S = decltype(set_tag)::value;
        __builtin_amdgcn_sched_barrier(0);
        // first half of a block: X and W of the next block have landed (everything but the 4 instructions just issued), and
        // this wavefront's fragment reads of the X stage that the next half-step's DMA overwrites have returned
        if constexpr (S == 0) {
            if (more) asm volatile("s_waitcnt vmcnt(4) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        }
        __builtin_amdgcn_s_barrier();
    };
    for (int t = 0; t < nt; t += 2) {
        const bool m0_ = feed(Set0{}, t);
        mfma_half(Set0{}, Kc0{});
        mfma_half(Set0{}, Kc1{});
        close_half(Set0{}, m0_);
        const bool m1_ = feed(Set1{}, t + 1);
        mfma_half(Set1{}, Kc0{});
        mfma_half(Set1{}, Kc1{});
        close_half(Set1{}, m1_);
    }

    // ── epilogue: acc[i][j][4 g + e] is feature wn*128 + 32 i + 8 g + 4 lh + e of token wm*64 + 32 j + lq ──
    const T* bias = static_cast<const T*>(p.bias);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int feat = wn * 128 + 32 * i + 8 * g + 4 * lh;
            float bv[4] = {0.f, 0.f, 0.f, 0.f};
            if (bias && n0 + feat < p.N) {
                const typename M::v4 b4 = *reinterpret_cast<const typename M::v4*>(bias + n0 + feat);
#pragma unroll
                for (int e = 0; e < 4; ++e) bv[e] = static_cast<float>(b4[e]);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                typename M::v4 o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = static_cast<T>(acc[i][j][4 * g + e] + bv[e]);
                *reinterpret_cast<typename M::v4*>(lds + (wm * 64 + 32 * j + lq) * kOutStride + feat * 2) = o;
            }
        }
    __syncthreads();
    unsigned char* yg = static_cast<unsigned char*>(p.y);
    const int cc = tid & 31;   // 16-byte piece of a row
#pragma unroll 4
    for (int r = tid >> 5; r < kTile; r += kThreads / 32) {
        if (m0 + r < p.M && n0 + cc * 8 < p.N)
            *reinterpret_cast<u32x4*>(yg + (static_cast<long>(m0 + r) * p.ldy + n0 + cc * 8) * 2) =
                *reinterpret_cast<const u32x4*>(lds + r * kOutStride + cc * 16);
    }
}

template <typename T>
int launch_t(const LinearBatch& batch, int n_problems, hipStream_t st) {
    int max_tiles = 0;
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        max_tiles = max(max_tiles, ((p.M + kTile - 1) / kTile) * ((p.N + kTile - 1) / kTile));
    }
    static thread_local bool raised = false;
    if (!raised) {
        MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&linear_dma_kernel<T>), hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));
        raised = true;
    }
    hipLaunchKernelGGL((linear_dma_kernel<T>), dim3(((max_tiles + 7) / 8) * 8, n_problems), dim3(kThreads), kLdsBytes, st, batch);
    MI_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace gemm_dma

// Large plain problems (16-bit weights, no GEGLU) whose 256 x 256 tiles give most compute units one work group.
bool linear_dma_takes(const LinearBatch& batch, int n_problems, int n_cu) {
    long tiles = 0;
    for (int i = 0; i < n_problems; ++i) {
        const LinearProblem& p = batch.p[i];
        if (p.w_scale != nullptr || p.K % gemm_dma::kBK != 0 || p.K < 512) return false;
        if (static_cast<long>(p.ldx) * 2 * gemm_dma::kTile >= (1L << 31) || static_cast<long>(p.ldw) * 2 * gemm_dma::kTile >= (1L << 31)) return false;
        tiles += static_cast<long>((p.M + gemm_dma::kTile - 1) / gemm_dma::kTile) * ((p.N + gemm_dma::kTile - 1) / gemm_dma::kTile);
    }
    return 4 * tiles >= 3L * n_cu;
}

int launch_linear_dma(const LinearBatch& batch, int n_problems, int dtype, hipStream_t st) {
    if (dtype == MI_DTYPE_BF16) return gemm_dma::launch_t<__bf16>(batch, n_problems, st);
    if (dtype == MI_DTYPE_F16) return gemm_dma::launch_t<_Float16>(batch, n_problems, st);
    return fail("linear: dtype %d is neither MI_DTYPE_F16 nor MI_DTYPE_BF16", dtype);
}

}  // namespace mi
