// ReLU linear attention for gfx950 (MI355X): O[n] = (S relu(Q[n])) / (z . relu(Q[n]) + eps) with
// S = V^T relu(K) (d x d) and z = sum_n relu(K[n]) per (batch, head).
//
// The op is HBM-bound: Q, K, V are read once and O written once (4 streams of (N, H*d) 16-bit
// values); the d x d contractions are small and run on MFMA so they hide under the memory time.
//   state kernel: one work group reduces a chunk of tokens. K (ReLU applied on the way in) and V
//                 tiles of 128 tokens sit row-major in LDS; both MFMA operands need the token axis
//                 contiguous per lane, which ds_read_b64_tr_b16 (LDS transpose read) delivers. A
//                 wavefront owns a 64 x 64 piece of S, so every fragment it reads feeds two MFMAs.
//                 z falls out of the same product as an extra row of S (a column of ones in V's
//                 zero pad), or comes from the K fragments against an all-ones operand where the
//                 head dimension leaves no pad. No atomics anywhere: results are bit-reproducible.
//   reduce kernel: adds the partial states of the token chunks into the state, in a fixed order.
//   apply kernel: S is staged in LDS as 16-bit A operand, relu(Q) rows are B operands; the denominator
//                 is an exact FP32 dot of z with the lane's own Q values plus one exchange between
//                 lanes l and l^32.
#include <algorithm>
#include <type_traits>

#include <atomic>

#include "internal.h"

// Partial states of mi_linear_attn_relu_forward_static_scratch: device memory that belongs to the library, one copy per
// GPU, present from the moment the code object is loaded until the process ends. Host code never uses this name as an
// address (on the host it is only a handle for hipGetSymbolAddress): kernels and copies get static_scratch_ptr().
static __device__ __align__(256) unsigned char scratch[MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES];

namespace mi {
namespace {

// Device address of `scratch` on the current GPU, looked up once per device (each GPU holds its own copy at its own
// address). Two threads that meet here for the first time both look up the same address.
constexpr int kMaxDevices = 64;
std::atomic<unsigned char*> g_static_scratch[kMaxDevices];
int static_scratch_ptr(unsigned char** out) {
    int dev = -1;
    MI_HIP_CHECK(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return fail("mi_linear_attn_relu_forward_static_scratch: device %d outside 0..%d", dev, kMaxDevices - 1);
    unsigned char* ptr = g_static_scratch[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        MI_HIP_CHECK(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return fail("mi_linear_attn_relu_forward_static_scratch: hipGetSymbolAddress returned null");
        g_static_scratch[dev].store(ptr, std::memory_order_release);
    }
    *out = ptr;
    return 0;
}

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
    float* part;    // partial states of the token chunks: [(b,h)][chunk][D*D + D], or null
    int n_part;     // chunks per (b,h) in `part`
    int add_to_state;   // no partials: this group's (S, z) is added to the state instead of replacing it
    float old_weight;   // weight of the state that was there before, where the call accumulates
    int tokens_per_group;
    int n_chunks;   // token chunks per (batch, head)
    int n_blocks;   // work groups with work = B * H * n_chunks
    int form;       // MI_LINEAR_ATTN_FORM_*
    int channel_major;   // operands are (heads * head_dim, tokens) per batch item; row strides are between channel rows
};
constexpr int kFusedMaxTokens = 1024;   // up to here the one-launch form is taken for sliced heads when the kernel is picked by size

template <int D> struct LGeo {
    static constexpr int DP = (D + 31) / 32 * 32;
    static constexpr int NB = DP / 32;
    static constexpr int KC = DP / 16;
    static constexpr int T_STRIDE = ((DP * 2 + 63) / 128) * 128 + 64;  // tiles read by transpose reads
    static constexpr int S_STRIDE = DP * 2 + 16;                       // rows read one per lane by ds_read_b128
    static constexpr int CPR = D / 8;
    static constexpr int CPRP = DP / 8;
    static constexpr int NCH = kTN * CPR;
    static constexpr int NLD = (NCH + kThreads - 1) / kThreads;
    static constexpr int WS_FLOATS = D * D + D;
};

// ReLU of 8 packed 16-bit floats. Both formats keep the sign in the top bit, so as signed 16-bit integers every negative
// value (and -0) is below zero and every positive one keeps its bits: a packed integer max with 0 is the ReLU.
typedef short s16x2 __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ u32x4 relu8(u32x4 raw) {
    u32x4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const unsigned w = raw[i];
        const s16x2 x = __builtin_bit_cast(s16x2, w);
        const s16x2 r = __builtin_elementwise_max(x, s16x2{0, 0});
        out[i] = __builtin_bit_cast(unsigned, r);
    }
    return out;
}


// Work group -> (batch*head, token chunk). Hardware work-group ids go round the 8 XCDs, each with its own L2: the
// logical index is arranged so that one XCD gets a contiguous range of heads with all their chunks. Then the heads
// whose 2*D-byte row segments share cache lines (a token row holds all heads side by side) meet in the same L2,
// and so do the work groups that read the same (S, z).
__device__ __forceinline__ bool lin_block(const LinDev& p, int& bh, int& chunk) {
    const int per_xcd = (p.n_blocks + 7) >> 3;
    const int logical = (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
    if (logical >= p.n_blocks) return false;
    bh = logical / p.n_chunks;
    chunk = logical - bh * p.n_chunks;
    return true;
}

// ── state: (S, z) of this group's token chunk ──
// The pass streams K and V rows with little arithmetic; what limits it besides HBM is the LDS read path, because both
// MFMA operands come out of LDS through transpose reads. So a wavefront owns a rectangle of 32x32 blocks of S (2 x 2 where
// S has 16 blocks: 4 MFMAs per 4 fragments read instead of 1 per 2), and the wavefronts that are left over split the 16-token
// steps of every tile among themselves. Loads are branch-free (rows past the end of the chunk are fetched from its last
// row and K is blanked at the LDS store, which removes their contribution to S and z) and all issued before the first is
// used; the next tile's rows are in flight in registers while the current one is multiplied.
// z = sum of relu(K) rows: where the padded head dimension leaves room (d = 72, 112) column d of the V tile in LDS holds
// ones, so row d of S is z and costs nothing; otherwise the wavefronts of the first block row multiply the K fragments
// with an all-ones operand as well.
// At the end the wavefronts put their blocks into FP32 images of (S, z) in LDS (one image per token share, added in a
// fixed order), which then go out in full rows with plain stores: to the state itself when the group covers the whole
// (batch, head), else to the group's slot among the partial states that a small reduction kernel adds up (atomic adds from several
// groups to one address are executed at the memory side on this multi-die GPU and were measured to cost far more than
// the whole pass).
constexpr int kStateThreads = 512;
constexpr int kStateWaves = kStateThreads / 64;
constexpr int kMaxStateSplit = 8;   // most token chunks per (batch, head) whose partial states the workspace can hold
constexpr int kStateTile = 128;

template <int D> struct StateGeo {
    using G = LGeo<D>;
    static constexpr int RBW = G::NB == 3 ? 3 : (G::NB >= 2 ? 2 : 1);            // block rows of a wavefront's rectangle
    static constexpr int CBW = G::NB == 3 ? 1 : (G::NB >= 2 ? 2 : 1);            // block columns
    static constexpr int NOWN = (G::NB / RBW) * (G::NB / CBW);                   // rectangles that tile S
    static constexpr int NTS = kStateWaves / NOWN;                               // wavefronts sharing a rectangle (token split)
    static constexpr int KSTEPS = (kStateTile / 16) / NTS;                       // 16-token steps per wavefront and tile
    static constexpr bool Z_IN_PAD = G::DP > D;                                  // z as row D of S
    static constexpr int Z_ROW = Z_IN_PAD ? D : G::DP;                           // row of the FP32 image that holds z
    static constexpr int NCH = kStateTile * G::CPR;
    static constexpr int NLD = (NCH + kStateThreads - 1) / kStateThreads;
    static constexpr int TILE_BYTES = kStateTile * G::T_STRIDE;
    static constexpr int S_FLOATS = G::DP * G::DP + G::DP;
    static constexpr int LDS_BYTES = 2 * TILE_BYTES > NTS * S_FLOATS * 4 ? 2 * TILE_BYTES : NTS * S_FLOATS * 4;
    static_assert((kStateTile / 16) % NTS == 0 && NTS >= 1, "token steps must divide among the sharing wavefronts");
};

template <typename T, int D>
__global__ void __launch_bounds__(kStateThreads) linattn_state_kernel(const LinDev p) {
    using G = LGeo<D>;
    using SG = StateGeo<D>;
    using V8 = typename Mma<T>::v8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    unsigned char* const Ks = lds;
    unsigned char* const Vs = lds + SG::TILE_BYTES;

    int bh, chunk;
    if (!lin_block(p, bh, chunk)) return;
    const int b = bh / p.H, h = bh % p.H;
    const int n_begin = chunk * p.tokens_per_group;
    const int n_end = min(p.N, n_begin + p.tokens_per_group);
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    const T* const k_base = static_cast<const T*>(p.k) + b * p.k_bs + h * D;
    const T* const v_base = static_cast<const T*>(p.v) + b * p.v_bs + h * D;

    // wave -> (rectangle of S, share of the k-steps of a tile)
    const int own = wave % SG::NOWN;
    const int ts = wave / SG::NOWN;
    const int rb0 = (own / (G::NB / SG::CBW)) * SG::RBW, cb0 = (own % (G::NB / SG::CBW)) * SG::CBW;
    const bool active = ts < SG::NTS;
    const bool does_z = !SG::Z_IN_PAD && active && rb0 == 0;

    if constexpr (G::DP > D) {  // pad columns stay as written here for the whole kernel: zero, and ones in column D of V
        constexpr int PC = (G::DP - D) / 8;
        typedef T t8 __attribute__((ext_vector_type(8)));
        t8 one_first;
#pragma unroll
        for (int e = 0; e < 8; ++e) one_first[e] = static_cast<T>(e == 0 ? 1.f : 0.f);
        for (int i = tid; i < kStateTile * PC; i += kStateThreads) {
            const int off = (i / PC) * G::T_STRIDE + D * 2 + (i % PC) * 16;
            *reinterpret_cast<u32x4*>(Ks + off) = u32x4{0, 0, 0, 0};
            *reinterpret_cast<u32x4*>(Vs + off) = (i % PC) == 0 ? __builtin_bit_cast(u32x4, one_first) : u32x4{0, 0, 0, 0};
        }
    }

    f32x16 acc[SG::RBW][SG::CBW], zacc[SG::CBW];
#pragma unroll
    for (int e = 0; e < 16; ++e) {
#pragma unroll
        for (int j = 0; j < SG::CBW; ++j) {
            zacc[j][e] = 0.f;
#pragma unroll
            for (int i = 0; i < SG::RBW; ++i) acc[i][j][e] = 0.f;
        }
    }
    V8 ones;
#pragma unroll
    for (int t = 0; t < 8; ++t) ones[t] = static_cast<T>(1.f);

    // Two register sets, so that the loads of two tiles are in flight while a third is multiplied: with one set a group
    // waits out most of the memory latency once per tile. All loads are unconditional (rows past the end of the chunk
    // repeat its last row), which keeps the order "older set, newer set" the same on every path and lets the wait in
    // front of an LDS store cover the older set only.
    u32x4 kregA[SG::NLD], vregA[SG::NLD], kregB[SG::NLD], vregB[SG::NLD];
    const int last = n_end - 1;
    auto issue_loads = [&](u32x4 (&kreg)[SG::NLD], u32x4 (&vreg)[SG::NLD], int n0) {
#pragma unroll
        for (int i = 0; i < SG::NLD; ++i) {
            const int idx = min(tid + kStateThreads * i, SG::NCH - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            const long n = min(n0 + row, last);
            kreg[i] = *reinterpret_cast<const u32x4*>(k_base + n * p.k_rs + cc * 8);
            vreg[i] = *reinterpret_cast<const u32x4*>(v_base + n * p.v_rs + cc * 8);
        }
    };
    auto store_tile = [&](const u32x4 (&kreg)[SG::NLD], const u32x4 (&vreg)[SG::NLD], int n0) {
#pragma unroll
        for (int i = 0; i < SG::NLD; ++i) {
            const int idx = tid + kStateThreads * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < SG::NCH) {
                u32x4 kv = relu8<T>(kreg[i]);
                if (n0 + row > last) kv = u32x4{0, 0, 0, 0};
                *reinterpret_cast<u32x4*>(Ks + row * G::T_STRIDE + cc * 16) = kv;
                *reinterpret_cast<u32x4*>(Vs + row * G::T_STRIDE + cc * 16) = vreg[i];
            }
        }
    };
    auto frag = [&](const unsigned char* ptr) -> V8 {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr + 8 * G::T_STRIDE));
        return __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };

    const int trow = (lane & 15) >> 2;
    const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    auto multiply_tile = [&]() {
        if (active) {
#pragma unroll
            for (int s = 0; s < SG::KSTEPS; ++s) {
                const int trow0 = 16 * (ts * SG::KSTEPS + s) + 4 * lh + trow;
                V8 a[SG::RBW], bk[SG::CBW];
#pragma unroll
                for (int i = 0; i < SG::RBW; ++i) a[i] = frag(Vs + trow0 * G::T_STRIDE + (32 * (rb0 + i) + tcol) * 2);
#pragma unroll
                for (int j = 0; j < SG::CBW; ++j) bk[j] = frag(Ks + trow0 * G::T_STRIDE + (32 * (cb0 + j) + tcol) * 2);
#pragma unroll
                for (int j = 0; j < SG::CBW; ++j) {
#pragma unroll
                    for (int i = 0; i < SG::RBW; ++i) acc[i][j] = Mma<T>::run(a[i], bk[j], acc[i][j]);
                    if (does_z) zacc[j] = Mma<T>::run(ones, bk[j], zacc[j]);
                }
            }
        }
    };
    // The loop takes two tiles per turn and has one way out, at the bottom: a second exit between the halves would give
    // the compiler a path on which set A is the newer one, and its waits at the top would drain both sets.
    const int n_tiles = (n_end - n_begin + kStateTile - 1) / kStateTile;
    int n0 = n_begin;
    issue_loads(kregA, vregA, n0);
    issue_loads(kregB, vregB, n0 + kStateTile);
    for (int pairs = n_tiles >> 1; pairs > 0; --pairs) {
        store_tile(kregA, vregA, n0);
        __syncthreads();
        issue_loads(kregA, vregA, n0 + 2 * kStateTile);
        multiply_tile();
        __syncthreads();
        store_tile(kregB, vregB, n0 + kStateTile);
        __syncthreads();
        issue_loads(kregB, vregB, n0 + 3 * kStateTile);
        multiply_tile();
        __syncthreads();
        n0 += 2 * kStateTile;
    }
    if (n_tiles & 1) {
        store_tile(kregA, vregA, n0);
        __syncthreads();
        multiply_tile();
        __syncthreads();
    }

    // blocks -> FP32 images of (S, z) in LDS (rows of DP floats, then one more row for z where it is not a row of S),
    // reusing the tile space. Wavefronts that share a rectangle (each took a share of every tile's tokens) write one
    // image each; the images are added in a fixed order on the way out, so the result does not depend on which wavefront
    // finishes first. Every element that is read back is written: the rectangles tile S, those of the first block row
    // cover the separate z row.
    float* const Sl = reinterpret_cast<float*>(lds);
    if (active) {
        float* const img = Sl + ts * SG::S_FLOATS;
#pragma unroll
        for (int jb = 0; jb < SG::CBW; ++jb) {
            const int j = 32 * (cb0 + jb) + lq;
#pragma unroll
            for (int ib = 0; ib < SG::RBW; ++ib)
#pragma unroll
                for (int bb = 0; bb < 4; ++bb)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int i = 32 * (rb0 + ib) + 8 * bb + 4 * lh + e;
                        img[i * G::DP + j] = acc[ib][jb][4 * bb + e];
                    }
            if (does_z && lh == 0) img[G::DP * G::DP + j] = zacc[jb][0];
        }
    }
    __syncthreads();
    // this group's (S, z): straight into the state when it covers the whole (batch, head), else into its partial slot
    float* const S = p.part ? p.part + (static_cast<long>(bh) * p.n_part + chunk) * G::WS_FLOATS
                            : p.ws + static_cast<long>(bh) * G::WS_FLOATS;
    const float* const old_state = p.add_to_state ? S : nullptr;      // the only group of this (batch, head)
    for (int idx = tid; idx < (D + 1) * (D / 4); idx += kStateThreads) {
        const int i = idx / (D / 4), j = (idx - i * (D / 4)) * 4;     // i == D: the z row
        const float* const src = Sl + (i < D ? i : SG::Z_ROW) * G::DP + j;
        f32x4 v = *reinterpret_cast<const f32x4*>(src);
#pragma unroll
        for (int t = 1; t < SG::NTS; ++t) v += *reinterpret_cast<const f32x4*>(src + t * SG::S_FLOATS);
        if (old_state) v += *reinterpret_cast<const f32x4*>(old_state + i * D + j) * p.old_weight;
        *reinterpret_cast<f32x4*>(S + i * D + j) = v;
    }
}

// state (+)= sum of the partial states of the token chunks, one element per thread and step.
__global__ void __launch_bounds__(256) linattn_reduce_kernel(float* ws, const float* part, int n_part, long ws_floats4, long total4,
                                                             int accumulate, float old_weight) {
    for (long i = blockIdx.x * 256L + threadIdx.x; i < total4; i += gridDim.x * 256L) {
        const long bh = i / ws_floats4, off = i - bh * ws_floats4;
        f32x4 v = accumulate ? reinterpret_cast<const f32x4*>(ws)[i] * old_weight : f32x4{0.f, 0.f, 0.f, 0.f};
        for (int c = 0; c < n_part; ++c) v += reinterpret_cast<const f32x4*>(part)[(bh * n_part + c) * ws_floats4 + off];
        reinterpret_cast<f32x4*>(ws)[i] = v;
    }
}

// ── apply: O = (S relu(Q)) / (z . relu(Q) + eps) ──
// S sits in LDS as 16-bit A operand for the whole group. Tokens go through in tiles of 128 (32 per wavefront, one per
// lane pair): the Q rows are fetched with full-row coalescing (the next tile is in flight in registers), ReLU'd and
// staged in LDS, where each lane picks the B-operand fragments of its own token; the denominator is an exact FP32
// dot of z with those values plus one exchange between lanes l and l^32. Results leave through the same LDS tile so
// that the stores are full 16-byte chunks of contiguous row segments.
template <typename T, int D>
__global__ void __launch_bounds__(kThreads) linattn_apply_kernel(const LinDev p) {
    using G = LGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int TM = 128;                       // tokens per tile
    constexpr int NQ = (TM * G::CPR + kThreads - 1) / kThreads;
    __shared__ __attribute__((aligned(16))) unsigned char Ss[G::DP * G::S_STRIDE];
    __shared__ __attribute__((aligned(16))) unsigned char Qs[TM * G::S_STRIDE];
    __shared__ __attribute__((aligned(16))) float Zs[G::DP];

    int bh, chunk;
    if (!lin_block(p, bh, chunk)) return;
    const int b = bh / p.H, h = bh % p.H;
    const int n_begin = chunk * p.tokens_per_group;
    const int n_end = min(p.N, n_begin + p.tokens_per_group);
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const float* const S = p.ws + static_cast<long>(bh) * G::WS_FLOATS;
    const float* const z = S + D * D;
    const int last = n_end - 1;

    u32x4 qreg[NQ];
    auto issue_q = [&](int n0) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = min(tid + kThreads * i, TM * G::CPR - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            qreg[i] = *reinterpret_cast<const u32x4*>(q_base + static_cast<long>(min(n0 + row, last)) * p.q_rs + cc * 8);
        }
    };
    issue_q(n_begin);

    // stage S (FP32 -> T) and z (FP32) in LDS; pad rows/columns are zero. All loads are issued before the first
    // conversion (pad positions read a clamped address and are blanked).
    {
        constexpr int NS = (G::DP * (G::DP / 4) + kThreads - 1) / kThreads;
        f32x4 sv[NS];
#pragma unroll
        for (int t = 0; t < NS; ++t) {
            const int idx = min(tid + kThreads * t, G::DP * (G::DP / 4) - 1);
            const int i = idx / (G::DP / 4), j = (idx - i * (G::DP / 4)) * 4;
            sv[t] = *reinterpret_cast<const f32x4*>(S + min(i, D - 1) * D + min(j, D - 4));
        }
#pragma unroll
        for (int t = 0; t < NS; ++t) {
            const int idx = tid + kThreads * t;
            const int i = idx / (G::DP / 4), j = (idx - i * (G::DP / 4)) * 4;
            typedef T t4 __attribute__((ext_vector_type(4)));
            t4 tv;
#pragma unroll
            for (int e = 0; e < 4; ++e) tv[e] = (i < D && j < D) ? static_cast<T>(sv[t][e]) : static_cast<T>(0.f);
            if (idx < G::DP * (G::DP / 4)) *reinterpret_cast<t4*>(Ss + i * G::S_STRIDE + j * 2) = tv;
        }
    }
    for (int j = tid; j < G::DP; j += kThreads) Zs[j] = j < D ? z[j] : 0.f;
    if constexpr (G::DP > D) {  // pad chunks of the Q tile stay zero
        constexpr int PC = (G::DP - D) / 8;
        for (int i = tid; i < TM * PC; i += kThreads)
            *reinterpret_cast<u32x4*>(Qs + (i / PC) * G::S_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
    }

    for (int n0 = n_begin; n0 < n_end; n0 += TM) {
        // Q tile: registers -> LDS (ReLU on the way), then the next tile's loads
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < TM * G::CPR) *reinterpret_cast<u32x4*>(Qs + row * G::S_STRIDE + cc * 16) = relu8<T>(qreg[i]);
        }
        __syncthreads();
        if (n0 + TM < n_end) issue_q(n0 + TM);

        const int trow = wave * 32 + lq;          // this lane's token within the tile
        V8 qf[G::KC];
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) {
            const int d0 = 16 * c + 8 * lh;
            qf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Qs + trow * G::S_STRIDE + d0 * 2));
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
        __syncthreads();                          // every lane holds its fragments: the tile can take the results
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
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                const int i0 = 32 * rb + 8 * bb + 4 * lh;
                typedef T t4 __attribute__((ext_vector_type(4)));
                t4 ov;
#pragma unroll
                for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(acc[4 * bb + e] * recip);
                *reinterpret_cast<t4*>(Qs + trow * G::S_STRIDE + i0 * 2) = ov;
            }
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < TM * G::CPR && n0 + row <= last)
                *reinterpret_cast<u32x4*>(o_base + static_cast<long>(n0 + row) * p.o_rs + cc * 8) =
                    *reinterpret_cast<const u32x4*>(Qs + row * G::S_STRIDE + cc * 16);
        }
        if constexpr (G::DP > D) {
            // the results overwrote the zero pad chunks of the tile (value channels D..DP-1 are zero anyway: the pad
            // rows of S are zero), nothing to restore
        }
        __syncthreads();
    }
}


// ── one launch, no hand-over: the state is split along its VALUE-channel axis ──
// Work group (batch, head, r) owns rows [32 r, 32 r + 32) of S (value channels) and every column. Pass 1 streams all of K
// and the 64-byte slice of V that holds its channels, giving S[32 r .. 32 r + 32, :] and the whole z (it reads all of K
// anyway); pass 2, the same work group, streams all of Q and writes its 64-byte slice of O. Nothing is exchanged between
// work groups: no partial states in memory, no reduction kernel, no fence, no atomics, one launch. The price is that the
// DP / 32 work groups of a head each read K and Q; they are numbered next to each other so that they share an XCD and the
// repeats come out of its L2.
// Inside a work group the 8 wavefronts are independent in both passes: each walks 32-token units of its own (unit u of
// wavefront w is tokens [32 (w + 8 u), + 32)), fetched with full-row coalescing two units ahead into two register sets
// and staged through a private LDS slice, so no work-group barrier stands in either streaming loop and about 150 KB of
// loads are in flight per compute unit. All vector-memory instructions in the loops are unconditional (past the end a
// wavefront re-fetches its last unit, and a lane without an output chunk of its own repeats another lane's store), so
// that the compiler's wait counts stay exact and a wait for the older register set does not drain the younger one.
// Between the passes the 8 partial states meet in LDS as FP32 images and are added in a fixed order: bit-reproducible.
// z costs one accumulator: the A operand "ones in row j" sends the token sum of K's column block j to row j of it.
constexpr int kFusedThreads = 512;
constexpr int kFusedWaves = kFusedThreads / 64;
constexpr int kFU = 32;                     // tokens per unit

template <int D> struct FusedGeo {
    using G = LGeo<D>;
    static constexpr int NS = G::NB;                                   // work groups (value-channel slices) per (batch, head)
    static constexpr int VT_STRIDE = 64;                               // V slice tile: 32 channels, rows back to back (64 mod 128)
    static constexpr int P1_SLICE = kFU * (G::T_STRIDE + VT_STRIDE);   // pass 1: K rows then V rows of a unit
    static constexpr int IMG_FLOATS = 32 * G::DP + G::DP;              // 32 rows of S and z
    static constexpr int O_STRIDE = 64 + 16;                           // pass 2: staged output rows (32 channels)
    static constexpr int P2_SLICE = kFU * G::S_STRIDE;                 // pass 2: Q rows of a unit (the output rows reuse it)
    static constexpr int SB_BYTES = 32 * G::S_STRIDE;                  // the slice of S as 16-bit A operand
    static constexpr int cmax(int a, int b) { return a > b ? a : b; }
    static constexpr int WORK_BYTES = cmax(cmax(kFusedWaves * P1_SLICE, kFusedWaves * IMG_FLOATS * 4), kFusedWaves * P2_SLICE);
    static constexpr int LDS_BYTES = WORK_BYTES + SB_BYTES + G::DP * 4;
    static_assert(kFU * O_STRIDE <= P2_SLICE, "the staged output fits the unit's Q slice");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of a compute unit");
};

template <typename T, int D>
__global__ void __launch_bounds__(kFusedThreads, 2) linattn_fused_kernel(const LinDev p) {
    using G = LGeo<D>;
    using FG = FusedGeo<D>;
    using V8 = typename Mma<T>::v8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    int bh, slice;
    {
        LinDev q = p;
        q.n_chunks = FG::NS;
        if (!lin_block(q, bh, slice)) return;
    }
    const int b = bh / p.H, h = bh % p.H;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    const T* const k_base = static_cast<const T*>(p.k) + b * p.k_bs + h * D;
    const T* const v_base = static_cast<const T*>(p.v) + b * p.v_bs + h * D + 32 * slice;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D + 32 * slice;
    constexpr int VCH = 4;                                   // 16-byte chunks of a slice row
    const int v_chunks = min(VCH, (D - 32 * slice) / 8);     // ... that exist (the last slice of a padded head is narrower)
    const int n_units = (p.N + kFU - 1) / kFU;
    const int last_unit = n_units - 1;
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // ───────────── pass 1: S[slice rows, :] and z over this wavefront's units ─────────────
    unsigned char* const Kp = lds + wave * FG::P1_SLICE;
    unsigned char* const Vp = Kp + kFU * G::T_STRIDE;
    constexpr int NK = (kFU * G::CPR + 63) / 64;             // K loads per lane and unit
    constexpr int NV = kFU * VCH / 64;                       // V loads per lane and unit (2)
    if constexpr (G::DP > D) {                               // pad columns of the K rows stay zero
        constexpr int PC = (G::DP - D) / 8;
        for (int i = lane; i < kFU * PC; i += 64)
            *reinterpret_cast<u32x4*>(Kp + (i / PC) * G::T_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
    }
    auto issue_kv = [&](u32x4 (&kreg)[NK], u32x4 (&vreg)[NV], int unit) {
        const long n0 = static_cast<long>(min(unit, last_unit)) * kFU;
        const long last = p.N - 1;
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int idx = min(lane + 64 * i, kFU * G::CPR - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            kreg[i] = *reinterpret_cast<const u32x4*>(k_base + min(n0 + row, last) * p.k_rs + cc * 8);
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / VCH, cc = min(idx - row * VCH, v_chunks - 1);
            vreg[i] = *reinterpret_cast<const u32x4*>(v_base + min(n0 + row, last) * p.v_rs + cc * 8);
        }
    };
    auto store_kv = [&](const u32x4 (&kreg)[NK], const u32x4 (&vreg)[NV], int unit) {
        const int n0 = unit * kFU;
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < kFU * G::CPR) {
                u32x4 kv = relu8<T>(kreg[i]);
                if (n0 + row >= p.N) kv = u32x4{0, 0, 0, 0};     // a token that does not exist adds nothing to S and z
                *reinterpret_cast<u32x4*>(Kp + row * G::T_STRIDE + cc * 16) = kv;
            }
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / VCH, cc = idx - row * VCH;
            *reinterpret_cast<u32x4*>(Vp + row * FG::VT_STRIDE + cc * 16) = cc < v_chunks ? vreg[i] : u32x4{0, 0, 0, 0};
        }
    };
    auto frag = [&](const unsigned char* ptr, int stride) -> V8 {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr + 8 * stride));
        return __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    f32x16 acc[G::NB], zacc;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        zacc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < G::NB; ++j) acc[j][e] = 0.f;
    }
    // A operand "ones in row j, zeros elsewhere": lane (row lq) holds 8 ones if lq == j. One register pair of ones per
    // lane and a mask per block (built where it is used) instead of four operands held through the loop.
    const unsigned one2 = (std::is_same_v<T, __bf16> ? 0x3f803f80u : 0x3c003c00u);
    auto sel = [&](int j) -> V8 {
        const unsigned w = lq == j ? one2 : 0u;
        return __builtin_bit_cast(V8, u32x4{w, w, w, w});
    };
    const int trow = (lane & 15) >> 2;
    const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    auto multiply_unit = [&]() {
#pragma unroll
        for (int s2 = 0; s2 < kFU / 16; ++s2) {
            const int r0 = 16 * s2 + 4 * lh + trow;
            const V8 a = frag(Vp + r0 * FG::VT_STRIDE + tcol * 2, FG::VT_STRIDE);
            V8 bk[G::NB];
#pragma unroll
            for (int j = 0; j < G::NB; ++j) bk[j] = frag(Kp + r0 * G::T_STRIDE + (32 * j + tcol) * 2, G::T_STRIDE);
#pragma unroll
            for (int j = 0; j < G::NB; ++j) {
                acc[j] = Mma<T>::run(a, bk[j], acc[j]);
                zacc = Mma<T>::run(sel(j), bk[j], zacc);
            }
        }
    };
    {
        u32x4 kA[NK], vA[NV], kB[NK], vB[NV];
        int u = wave;
        issue_kv(kA, vA, u);
        issue_kv(kB, vB, u + kFusedWaves);
        // two units per turn, one way out (at the bottom): on every path set A is the older one
        for (; u < n_units; u += 2 * kFusedWaves) {
            store_kv(kA, vA, u);
            wave_sync();
            issue_kv(kA, vA, u + 2 * kFusedWaves);
            multiply_unit();
            wave_sync();
            if (u + kFusedWaves < n_units) {
                store_kv(kB, vB, u + kFusedWaves);
                wave_sync();
            }
            issue_kv(kB, vB, u + 3 * kFusedWaves);
            if (u + kFusedWaves < n_units) {
                multiply_unit();
                wave_sync();
            }
        }
    }
    __syncthreads();     // every wavefront is done with its K / V slice: the space takes the FP32 images

    // ───────────── the 8 partial states -> one; the state to memory, the slice as A operand to LDS ─────────────
    // (the lane id is made opaque from here on: otherwise every per-lane address of pass 2 is computed in front of pass 1
    //  and spilled around it)
    int lane2 = lane;
    asm volatile("" : "+v"(lane2));
    const int lq2 = lane2 & 31, lh2 = lane2 >> 5;
    float* const img = reinterpret_cast<float*>(lds) + wave * FG::IMG_FLOATS;
#pragma unroll
    for (int j = 0; j < G::NB; ++j) {
#pragma unroll
        for (int bb = 0; bb < 4; ++bb)
#pragma unroll
            for (int e = 0; e < 4; ++e) img[(8 * bb + 4 * lh2 + e) * G::DP + 32 * j + lq2] = acc[j][4 * bb + e];
    }
    if (lh2 == 0) {
#pragma unroll
        for (int j = 0; j < G::NB; ++j) img[32 * G::DP + 32 * j + lq2] = zacc[j];     // row j of the z accumulator: column block j
    }
    // the first two units of pass 2 are requested now: their latency passes while the state is put together
    constexpr int NQ = (kFU * G::CPR + 63) / 64;
    auto issue_q = [&](u32x4 (&qreg)[NQ], int unit) {
        const long n0 = static_cast<long>(min(unit, last_unit)) * kFU;
        const long last = p.N - 1;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = min(lane2 + 64 * i, kFU * G::CPR - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            qreg[i] = *reinterpret_cast<const u32x4*>(q_base + min(n0 + row, last) * p.q_rs + cc * 8);
        }
    };
    u32x4 qA[NQ], qB[NQ];
    issue_q(qA, wave);
    issue_q(qB, wave + kFusedWaves);
    __syncthreads();
    unsigned char* const Sb = lds + FG::WORK_BYTES;
    float* const Zs = reinterpret_cast<float*>(Sb + FG::SB_BYTES);
    float* const ws = p.ws + static_cast<long>(bh) * G::WS_FLOATS;
    const float* const img0 = reinterpret_cast<const float*>(lds);
    for (int idx = tid; idx < FG::IMG_FLOATS / 4; idx += kFusedThreads) {
        const int i = idx / (G::DP / 4), j = (idx - i * (G::DP / 4)) * 4;        // i == 32: the z row
        f32x4 v = *reinterpret_cast<const f32x4*>(img0 + i * G::DP + j);
#pragma unroll
        for (int w = 1; w < kFusedWaves; ++w) v += *reinterpret_cast<const f32x4*>(img0 + w * FG::IMG_FLOATS + i * G::DP + j);
        const int row = 32 * slice + i;
        if (i < 32) {
            typedef T t4 __attribute__((ext_vector_type(4)));
            t4 tv;
#pragma unroll
            for (int e = 0; e < 4; ++e) tv[e] = (row < D && j < D) ? static_cast<T>(v[e]) : static_cast<T>(0.f);
            *reinterpret_cast<t4*>(Sb + i * G::S_STRIDE + j * 2) = tv;
            if (row < D && j < D) *reinterpret_cast<f32x4*>(ws + row * D + j) = v;
        } else {
            *reinterpret_cast<f32x4*>(Zs + j) = j < D ? v : f32x4{0.f, 0.f, 0.f, 0.f};
            if (slice == 0 && j < D) *reinterpret_cast<f32x4*>(ws + D * D + j) = v;
        }
    }
    __syncthreads();     // S slice and z are in place; the image space becomes the Q slices

    // ───────────── pass 2: O[:, slice] = (S[slice rows, :] relu(Q)) / (z . relu(Q) + eps) ─────────────
    V8 sf[G::KC];        // this lane's row of the slice, all contraction steps
#pragma unroll
    for (int c = 0; c < G::KC; ++c) sf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Sb + lq2 * G::S_STRIDE + (16 * c + 8 * lh2) * 2));
    unsigned char* const Qp = lds + wave * FG::P2_SLICE;
    if constexpr (G::DP > D) {
        constexpr int PC = (G::DP - D) / 8;
        for (int i = lane2; i < kFU * PC; i += 64)
            *reinterpret_cast<u32x4*>(Qp + (i / PC) * G::S_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
    }
    auto apply_unit = [&](const u32x4 (&qreg)[NQ], int unit) {
        const int n0 = unit * kFU;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = lane2 + 64 * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < kFU * G::CPR) *reinterpret_cast<u32x4*>(Qp + row * G::S_STRIDE + cc * 16) = relu8<T>(qreg[i]);
        }
        wave_sync();
        V8 qf[G::KC];
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) {
            const int d0 = 16 * c + 8 * lh2;
            qf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Qp + lq2 * G::S_STRIDE + d0 * 2));
            const f32x4 z0 = *reinterpret_cast<const f32x4*>(Zs + d0);
            const f32x4 z1 = *reinterpret_cast<const f32x4*>(Zs + d0 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                den = __builtin_fmaf(z0[e], static_cast<float>(qf[c][e]), den);
                den = __builtin_fmaf(z1[e], static_cast<float>(qf[c][4 + e]), den);
            }
        }
        {
            const int di = __builtin_bit_cast(int, den);
            const i32x2 r = __builtin_amdgcn_permlane32_swap(di, di, false, false);
            const int r0 = r[0], r1 = r[1];
            den = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
        }
        const float rs = __builtin_amdgcn_rsqf(den + p.eps);       // the reference's reciprocal: rsqrt(den + eps)^2 in FP32
        const float recip = rs * rs;
        f32x16 o;
#pragma unroll
        for (int e = 0; e < 16; ++e) o[e] = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) o = Mma<T>::run(sf[c], qf[c], o);
        wave_sync();          // every lane2 holds its Q fragments: the slice takes the results
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
            typedef T t4 __attribute__((ext_vector_type(4)));
            t4 ov;
#pragma unroll
            for (int e = 0; e < 4; ++e) ov[e] = static_cast<T>(o[4 * bb + e] * recip);
            *reinterpret_cast<t4*>(Qp + lq2 * FG::O_STRIDE + (8 * bb + 4 * lh2) * 2) = ov;
        }
        wave_sync();
        const int last_row = min(kFU, p.N - n0) - 1;
#pragma unroll
        for (int i = 0; i < kFU * VCH / 64; ++i) {
            const int idx = lane2 + 64 * i;
            const int row = min(idx / VCH, last_row), cc = min(idx % VCH, v_chunks - 1);
            *reinterpret_cast<u32x4*>(o_base + static_cast<long>(n0 + row) * p.o_rs + cc * 8) =
                *reinterpret_cast<const u32x4*>(Qp + row * FG::O_STRIDE + cc * 16);
        }
        wave_sync();          // the staged rows are read before the next unit's Q rows overwrite them
        if constexpr (G::DP > D) {
            // the output rows (80-byte stride) ran over pad chunks of the Q rows: zero again
            constexpr int PC = (G::DP - D) / 8;
            for (int i = lane2; i < kFU * PC; i += 64)
                *reinterpret_cast<u32x4*>(Qp + (i / PC) * G::S_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
        }
    };
    {
        for (int u = wave; u < n_units; u += 2 * kFusedWaves) {
            apply_unit(qA, u);
            issue_q(qA, u + 2 * kFusedWaves);
            // (unconditional: past its last unit a wavefront applies the last unit of the call once more and stores the same
            //  bytes again, so that the number of stores between two waits is fixed)
            apply_unit(qB, min(u + kFusedWaves, last_unit));
            issue_q(qB, u + 3 * kFusedWaves);
        }
    }
}


// ── the same one-launch form on CHANNEL-MAJOR operands ──
// Q, K, V, O as (heads * head_dim, tokens) per batch item, a row per channel: the layout in which the reference keeps
// these tensors around its core (src/dit/sana.cpp:424-444, :470-586). The contraction of pass 1 runs over tokens, which
// are contiguous here, so K and V rows go to LDS as they are (64-byte pieces of a row per 32-token unit, rows padded to
// 80 bytes) and every MFMA operand is one 16-byte read; pass 2 contracts over channels, so its B operand (a token's
// channels) comes out of the channel-by-token tile through transpose reads, and the result tile is turned back into
// channel rows in LDS before it is stored. Everything else — one work group per (batch, head, 32 value channels),
// independent wavefronts, two register sets, unconditional vector-memory instructions, the merge of the eight partial
// states in a fixed order — is the token-major kernel's. Consecutive units go to the same wavefront in pairs: the two
// halves of a 128-byte line of a channel row are then fetched by one wavefront back to back.
template <int D> struct FusedCmGeo {
    using G = LGeo<D>;
    static constexpr int NS = G::NB;
    static constexpr int KV_STRIDE = kFU * 2 + 16;                      // pass 1: a unit's 32 tokens of one channel, padded
    static constexpr int P1_SLICE = (G::DP + 32) * KV_STRIDE;           // K channels, then the slice's V channels
    static constexpr int IMG_FLOATS = 32 * G::DP + G::DP;
    static constexpr int Q_STRIDE = kFU * 2;                            // pass 2: channel rows back to back (64 mod 128: transpose reads)
    static constexpr int O_STRIDE = kFU * 2 + 16;
    static constexpr int cmax(int a, int b) { return a > b ? a : b; }
    static constexpr int P2_SLICE = cmax(G::DP * Q_STRIDE, 32 * O_STRIDE);   // the staged output rows reuse the unit's Q slice
    static constexpr int SB_BYTES = 32 * G::S_STRIDE;
    static constexpr int WORK_BYTES = cmax(cmax(kFusedWaves * P1_SLICE, kFusedWaves * IMG_FLOATS * 4), kFusedWaves * P2_SLICE);
    static constexpr int LDS_BYTES = WORK_BYTES + SB_BYTES + G::DP * 4;
    static_assert(32 * O_STRIDE <= P2_SLICE, "the staged output fits the unit's Q slice");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS of a compute unit");
};

template <typename T, int D>
__global__ void __launch_bounds__(kFusedThreads, 2) linattn_fused_cm_kernel(const LinDev p) {
    using G = LGeo<D>;
    using FG = FusedCmGeo<D>;
    using V8 = typename Mma<T>::v8;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    int bh, slice;
    {
        LinDev q = p;
        q.n_chunks = FG::NS;
        if (!lin_block(q, bh, slice)) return;
    }
    const int b = bh / p.H, h = bh % p.H;
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63;
    const int lq = lane & 31, lh = lane >> 5;
    // channel rows of this head; strides are in elements between channel rows
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + static_cast<long>(h) * D * p.q_rs;
    const T* const k_base = static_cast<const T*>(p.k) + b * p.k_bs + static_cast<long>(h) * D * p.k_rs;
    const T* const v_base = static_cast<const T*>(p.v) + b * p.v_bs + (static_cast<long>(h) * D + 32 * slice) * p.v_rs;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + (static_cast<long>(h) * D + 32 * slice) * p.o_rs;
    const int v_rows = min(32, D - 32 * slice);              // value channels of this slice that exist
    constexpr int UCH = kFU / 8;                             // 16-byte chunks of a unit's tokens in one channel row (4)
    const int n_units = (p.N + kFU - 1) / kFU;               // N is a multiple of 8: a chunk is whole or absent
    const int last_unit = n_units - 1;
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // units go to wavefronts in pairs: turn t of wavefront w is units 16 t + 2 w and 16 t + 2 w + 1
    constexpr int kTurn = 2 * kFusedWaves;

    // ───────────── pass 1 ─────────────
    unsigned char* const Kp = lds + wave * FG::P1_SLICE;
    unsigned char* const Vp = Kp + G::DP * FG::KV_STRIDE;
    constexpr int NK = (D * UCH + 63) / 64;
    constexpr int NV = 32 * UCH / 64;                        // 2
    if constexpr (G::DP > D) {                               // channel rows past the head dimension stay zero
        for (int i = lane; i < (G::DP - D) * UCH; i += 64)
            *reinterpret_cast<u32x4*>(Kp + (D + i / UCH) * FG::KV_STRIDE + (i % UCH) * 16) = u32x4{0, 0, 0, 0};
    }
    auto chunk_col = [&](int unit, int cc) { return static_cast<long>(min(unit, last_unit)) * kFU + 8 * cc; };
    auto issue_kv = [&](u32x4 (&kreg)[NK], u32x4 (&vreg)[NV], int unit) {
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int idx = min(lane + 64 * i, D * UCH - 1);
            const int row = idx / UCH, cc = idx - row * UCH;
            kreg[i] = *reinterpret_cast<const u32x4*>(k_base + row * p.k_rs + min(chunk_col(unit, cc), static_cast<long>(p.N) - 8));
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = lane + 64 * i;
            const int row = min(idx / UCH, v_rows - 1), cc = idx % UCH;
            vreg[i] = *reinterpret_cast<const u32x4*>(v_base + row * p.v_rs + min(chunk_col(unit, cc), static_cast<long>(p.N) - 8));
        }
    };
    auto store_kv = [&](const u32x4 (&kreg)[NK], const u32x4 (&vreg)[NV], int unit) {
        const int n0 = unit * kFU;
#pragma unroll
        for (int i = 0; i < NK; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / UCH, cc = idx - row * UCH;
            if (idx < D * UCH) {
                u32x4 kv = relu8<T>(kreg[i]);
                if (n0 + 8 * cc >= p.N) kv = u32x4{0, 0, 0, 0};          // tokens that do not exist add nothing
                *reinterpret_cast<u32x4*>(Kp + row * FG::KV_STRIDE + cc * 16) = kv;
            }
        }
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / UCH, cc = idx - row * UCH;
            *reinterpret_cast<u32x4*>(Vp + row * FG::KV_STRIDE + cc * 16) = row < v_rows ? vreg[i] : u32x4{0, 0, 0, 0};
        }
    };
    f32x16 acc[G::NB], zacc;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        zacc[e] = 0.f;
#pragma unroll
        for (int j = 0; j < G::NB; ++j) acc[j][e] = 0.f;
    }
    const unsigned one2 = (std::is_same_v<T, __bf16> ? 0x3f803f80u : 0x3c003c00u);
    auto sel = [&](int j) -> V8 {
        const unsigned w = lq == j ? one2 : 0u;
        return __builtin_bit_cast(V8, u32x4{w, w, w, w});
    };
    auto multiply_unit = [&]() {
#pragma unroll
        for (int s2 = 0; s2 < kFU / 16; ++s2) {
            const int off = (16 * s2 + 8 * lh) * 2;              // this lane's 8 tokens of the step
            const V8 a = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Vp + lq * FG::KV_STRIDE + off));
            V8 bk[G::NB];
#pragma unroll
            for (int j = 0; j < G::NB; ++j) bk[j] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Kp + (32 * j + lq) * FG::KV_STRIDE + off));
#pragma unroll
            for (int j = 0; j < G::NB; ++j) {
                acc[j] = Mma<T>::run(a, bk[j], acc[j]);
                zacc = Mma<T>::run(sel(j), bk[j], zacc);
            }
        }
    };
    {
        u32x4 kA[NK], vA[NV], kB[NK], vB[NV];
        int u = 2 * wave;
        issue_kv(kA, vA, u);
        issue_kv(kB, vB, u + 1);
        for (; u < n_units; u += kTurn) {
            store_kv(kA, vA, u);
            wave_sync();
            issue_kv(kA, vA, u + kTurn);
            multiply_unit();
            wave_sync();
            if (u + 1 < n_units) {
                store_kv(kB, vB, u + 1);
                wave_sync();
            }
            issue_kv(kB, vB, u + kTurn + 1);
            if (u + 1 < n_units) {
                multiply_unit();
                wave_sync();
            }
        }
    }
    __syncthreads();

    // ───────────── the 8 partial states -> one ─────────────
    int lane2 = lane;
    asm volatile("" : "+v"(lane2));
    const int lq2 = lane2 & 31, lh2 = lane2 >> 5;
    float* const img = reinterpret_cast<float*>(lds) + wave * FG::IMG_FLOATS;
#pragma unroll
    for (int j = 0; j < G::NB; ++j) {
#pragma unroll
        for (int bb = 0; bb < 4; ++bb)
#pragma unroll
            for (int e = 0; e < 4; ++e) img[(8 * bb + 4 * lh2 + e) * G::DP + 32 * j + lq2] = acc[j][4 * bb + e];
    }
    if (lh2 == 0) {
#pragma unroll
        for (int j = 0; j < G::NB; ++j) img[32 * G::DP + 32 * j + lq2] = zacc[j];
    }
    constexpr int NQ = (D * UCH + 63) / 64;
    auto issue_q = [&](u32x4 (&qreg)[NQ], int unit) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = min(lane2 + 64 * i, D * UCH - 1);
            const int row = idx / UCH, cc = idx - row * UCH;
            qreg[i] = *reinterpret_cast<const u32x4*>(q_base + row * p.q_rs + min(chunk_col(unit, cc), static_cast<long>(p.N) - 8));
        }
    };
    u32x4 qA[NQ], qB[NQ];
    issue_q(qA, 2 * wave);
    issue_q(qB, 2 * wave + 1);
    __syncthreads();
    unsigned char* const Sb = lds + FG::WORK_BYTES;
    float* const Zs = reinterpret_cast<float*>(Sb + FG::SB_BYTES);
    float* const ws = p.ws + static_cast<long>(bh) * G::WS_FLOATS;
    const float* const img0 = reinterpret_cast<const float*>(lds);
    for (int idx = tid; idx < FG::IMG_FLOATS / 4; idx += kFusedThreads) {
        const int i = idx / (G::DP / 4), j = (idx - i * (G::DP / 4)) * 4;
        f32x4 v = *reinterpret_cast<const f32x4*>(img0 + i * G::DP + j);
#pragma unroll
        for (int w = 1; w < kFusedWaves; ++w) v += *reinterpret_cast<const f32x4*>(img0 + w * FG::IMG_FLOATS + i * G::DP + j);
        const int row = 32 * slice + i;
        if (i < 32) {
            typedef T t4 __attribute__((ext_vector_type(4)));
            t4 tv;
#pragma unroll
            for (int e = 0; e < 4; ++e) tv[e] = (row < D && j < D) ? static_cast<T>(v[e]) : static_cast<T>(0.f);
            *reinterpret_cast<t4*>(Sb + i * G::S_STRIDE + j * 2) = tv;
            if (row < D && j < D) *reinterpret_cast<f32x4*>(ws + row * D + j) = v;
        } else {
            *reinterpret_cast<f32x4*>(Zs + j) = j < D ? v : f32x4{0.f, 0.f, 0.f, 0.f};
            if (slice == 0 && j < D) *reinterpret_cast<f32x4*>(ws + D * D + j) = v;
        }
    }
    __syncthreads();

    // ───────────── pass 2 ─────────────
    // The transpose reads below hand a lane the channels 16 c + 4 lh + {0..3} and 16 c + 8 + 4 lh + {0..3} of its token (two
    // 4 x 4 blocks), not 8 consecutive ones; the A operand and z take their contraction elements in the same order.
    V8 sf[G::KC];
#pragma unroll
    for (int c = 0; c < G::KC; ++c) {
        typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
        const u32x2 a0 = *reinterpret_cast<const u32x2*>(Sb + lq2 * G::S_STRIDE + (16 * c + 4 * lh2) * 2);
        const u32x2 a1 = *reinterpret_cast<const u32x2*>(Sb + lq2 * G::S_STRIDE + (16 * c + 8 + 4 * lh2) * 2);
        sf[c] = __builtin_bit_cast(V8, u32x4{a0[0], a0[1], a1[0], a1[1]});
    }
    unsigned char* const Qp = lds + wave * FG::P2_SLICE;
    if constexpr (G::DP > D) {
        for (int i = lane2; i < (G::DP - D) * UCH; i += 64)
            *reinterpret_cast<u32x4*>(Qp + (D + i / UCH) * FG::Q_STRIDE + (i % UCH) * 16) = u32x4{0, 0, 0, 0};
    }
    auto frag = [&](const unsigned char* ptr) -> V8 {
        const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr));
        const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(ptr + 8 * FG::Q_STRIDE));
        return __builtin_bit_cast(V8, (s16x8)__builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    const int trow = (lane2 & 15) >> 2;
    const int tcol = 16 * ((lane2 >> 4) & 1) + 4 * (lane2 & 3);
    auto apply_unit = [&](const u32x4 (&qreg)[NQ], int unit) {
        const int n0 = unit * kFU;
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = lane2 + 64 * i;
            const int row = idx / UCH, cc = idx - row * UCH;
            if (idx < D * UCH) *reinterpret_cast<u32x4*>(Qp + row * FG::Q_STRIDE + cc * 16) = relu8<T>(qreg[i]);
        }
        wave_sync();
        V8 qf[G::KC];
        float den = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) {
            // token lq2 (a column of the tile), channels 16 c + 4 lh2 + {0..3} and 16 c + 8 + 4 lh2 + {0..3} (rows): the B
            // operand of S relu(Q)
            qf[c] = frag(Qp + (16 * c + 4 * lh2 + trow) * FG::Q_STRIDE + tcol * 2);
            const int d0 = 16 * c + 4 * lh2;
            const f32x4 z0 = *reinterpret_cast<const f32x4*>(Zs + d0);
            const f32x4 z1 = *reinterpret_cast<const f32x4*>(Zs + d0 + 8);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                den = __builtin_fmaf(z0[e], static_cast<float>(qf[c][e]), den);
                den = __builtin_fmaf(z1[e], static_cast<float>(qf[c][4 + e]), den);
            }
        }
        {
            const int di = __builtin_bit_cast(int, den);
            const i32x2 r = __builtin_amdgcn_permlane32_swap(di, di, false, false);
            const int r0 = r[0], r1 = r[1];
            den = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
        }
        const float rs = __builtin_amdgcn_rsqf(den + p.eps);
        const float recip = rs * rs;
        f32x16 o;
#pragma unroll
        for (int e = 0; e < 16; ++e) o[e] = 0.f;
#pragma unroll
        for (int c = 0; c < G::KC; ++c) o = Mma<T>::run(sf[c], qf[c], o);
        wave_sync();
        // the result tile back into channel rows: element (channel 8 bb + 4 lh2 + e, token lq2)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb)
#pragma unroll
            for (int e = 0; e < 4; ++e)
                *reinterpret_cast<T*>(Qp + (8 * bb + 4 * lh2 + e) * FG::O_STRIDE + lq2 * 2) = static_cast<T>(o[4 * bb + e] * recip);
        wave_sync();
        const int last_cc = min(UCH, (p.N - n0) / 8) - 1;
#pragma unroll
        for (int i = 0; i < 32 * UCH / 64; ++i) {
            const int idx = lane2 + 64 * i;
            const int row = min(idx / UCH, v_rows - 1), cc = min(idx % UCH, last_cc);
            *reinterpret_cast<u32x4*>(o_base + row * p.o_rs + n0 + 8 * cc) =
                *reinterpret_cast<const u32x4*>(Qp + row * FG::O_STRIDE + cc * 16);
        }
        wave_sync();
    };
    for (int u = 2 * wave; u < n_units; u += kTurn) {
        apply_unit(qA, u);
        issue_q(qA, u + kTurn);
        apply_unit(qB, min(u + 1, last_unit));
        issue_q(qB, u + kTurn + 1);
    }
}

template <typename T, int D>
int launch_d(LinDev p, bool accumulate, int max_split, int n_cu, hipStream_t st) {
    using G = LGeo<D>;
    const int BH = p.B * p.H;
    // One launch with the state split along its value channels, when the call does not add to a state that is already
    // there (every work group of a head would read the old z while one of them replaces it) and its work groups fill
    // enough of the GPU; otherwise three launches (state per token chunk, reduction, apply).
    if (p.channel_major) {
        using FG = FusedCmGeo<D>;
        const long groups = static_cast<long>(BH) * FG::NS;
        if (groups >= (1L << 24)) return fail("mi_linear_attn_relu_forward: too many (batch, head) pairs for one launch");
        static thread_local bool raised_cm = false;
        if (!raised_cm) {
            MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&linattn_fused_cm_kernel<T, D>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                             FG::LDS_BYTES));
            raised_cm = true;
        }
        p.n_blocks = static_cast<int>(groups);
        hipLaunchKernelGGL((linattn_fused_cm_kernel<T, D>), dim3(((p.n_blocks + 7) / 8) * 8), dim3(kFusedThreads), FG::LDS_BYTES, st, p);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail("mi_linear_attn_relu_forward launch: %s", hipGetErrorString(e));
        return 0;
    }
    {
        using FG = FusedGeo<D>;
        const int groups = BH * FG::NS;
        const bool fits = !accumulate && static_cast<long>(BH) * FG::NS < (1L << 24);
        // Picked by size (measured, 256 compute units): with one slice per head (head_dim 32) nothing is read twice and the
        // single launch wins at every length once its work groups cover a quarter of the GPU; with several slices every
        // work group pulls all of K and Q through its own compute unit's L2 port (about 50 GB/s each), which costs more
        // than the two extra launches from about 2000 tokens on (head_dim 112, 40 heads: 13.6 against 18.5 us at 512
        // tokens, 20.5 against 23.4 at 1024, 32 against 31 at 2048, 55 against 42 at 4096).
        const bool by_size = fits && (FG::NS == 1 ? 4 * groups >= n_cu : (2 * groups >= n_cu && p.N <= kFusedMaxTokens));
        if (fits && (p.form == MI_LINEAR_ATTN_FORM_ONE_LAUNCH || (p.form == MI_LINEAR_ATTN_FORM_BY_SIZE && by_size))) {
            static thread_local bool raised = false;
            if (!raised) {
                MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&linattn_fused_kernel<T, D>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 FG::LDS_BYTES));
                raised = true;
            }
            p.n_blocks = groups;
            hipLaunchKernelGGL((linattn_fused_kernel<T, D>), dim3(((groups + 7) / 8) * 8), dim3(kFusedThreads), FG::LDS_BYTES, st, p);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail("mi_linear_attn_relu_forward launch: %s", hipGetErrorString(e));
            return 0;
        }
    }
    // State pass. The tokens of a head are split over enough groups to keep most CUs streaming, if the caller lent a
    // scratch for the partial states; each group needs a few tiles to amortise its prologue and epilogue.
    {
        LinDev ps = p;
        const int tiles = (ps.N + kStateTile - 1) / kStateTile;
        // the largest split that still gives every group a CU of its own and at least two tiles (40 heads on 256 CUs: 6;
        // two groups per CU measured slower, a power of two leaves a third of the CUs idle)
        int split = 1;
        for (int s2 = 2; s2 <= max_split; ++s2)
            if (BH * s2 <= n_cu && tiles / s2 >= 2) split = s2;
        ps.tokens_per_group = ((tiles + split - 1) / split) * kStateTile;
        ps.n_chunks = (ps.N + ps.tokens_per_group - 1) / ps.tokens_per_group;
        ps.n_blocks = BH * ps.n_chunks;
        const bool partials = max_split > 0 && (accumulate || ps.n_chunks > 1);
        ps.part = partials ? p.part : nullptr;
        ps.n_part = ps.n_chunks;
        ps.add_to_state = (!partials && accumulate) ? 1 : 0;
        hipLaunchKernelGGL((linattn_state_kernel<T, D>), dim3(((ps.n_blocks + 7) / 8) * 8), dim3(kStateThreads),
                           StateGeo<D>::LDS_BYTES, st, ps);
        if (partials) {
            const long ws4 = G::WS_FLOATS / 4, total4 = static_cast<long>(BH) * ws4;   // D is a multiple of 8: whole 16-byte pieces
            const int blocks = static_cast<int>(std::min<long>((total4 + 255) / 256, 2048));
            hipLaunchKernelGGL(linattn_reduce_kernel, dim3(blocks), dim3(256), 0, st, p.ws, p.part, ps.n_part, ws4, total4,
                               accumulate ? 1 : 0, p.old_weight);
        }
    }
    // Apply pass: chunks are whole tiles, and as few of them per group as keep every group resident at once (two work
    // groups per CU hide each other's latencies): the staging of S is paid once per group, and a second, partly filled round of
    // groups would pay it again (N = 4096, 40 heads: 440 groups of 3 tiles instead of 640 of 2, 45.6 -> 43.4 us for the call).
    auto grid_of = [&](LinDev& q) {
        q.n_chunks = (q.N + q.tokens_per_group - 1) / q.tokens_per_group;
        q.n_blocks = BH * q.n_chunks;
        return dim3(((q.n_blocks + 7) / 8) * 8);
    };
    {
        const int tiles = (p.N + 127) / 128;
        const int per_bh = std::max(1, 2 * n_cu / BH);
        p.tokens_per_group = 128 * ((tiles + per_bh - 1) / per_bh);
    }
    hipLaunchKernelGGL((linattn_apply_kernel<T, D>), grid_of(p), dim3(kThreads), 0, st, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_linear_attn_relu_forward launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_t(const LinDev& p, int d, bool acc, int max_split, int n_cu, hipStream_t st) {
    switch (d) {
        case 32: return launch_d<T, 32>(p, acc, max_split, n_cu, st);
        case 64: return launch_d<T, 64>(p, acc, max_split, n_cu, st);
        case 72: return launch_d<T, 72>(p, acc, max_split, n_cu, st);
        case 112: return launch_d<T, 112>(p, acc, max_split, n_cu, st);
        case 128: return launch_d<T, 128>(p, acc, max_split, n_cu, st);
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

namespace mi {
namespace {
// Shared body of the two entry points: `part` / `part_bytes` is the memory for the partial states of the token chunks
// (the caller's scratch, the library's static scratch, or none).
int linear_attn_forward(const mi_linear_attn_args* a, const char* op, void* part, size_t part_bytes) {
    if (a->batch <= 0 || a->num_heads <= 0 || a->n_tokens < 0) return fail("%s: bad shape", op);
    if (a->n_tokens == 0) return 0;
    if (!a->q || !a->k || !a->v || !a->o) return fail("%s: null tensor", op);
    const size_t need = mi_linear_attn_workspace_bytes(a->batch, a->num_heads, a->head_dim);
    if (!a->workspace || a->workspace_bytes < need)
        return fail("%s: workspace needs %zu bytes (got %zu)", op, need, a->workspace ? a->workspace_bytes : 0);
    // the scratch decides how far the tokens of a head may be split over work groups (one partial state per chunk)
    int max_split = 0;
    if (part) {
        if (reinterpret_cast<uintptr_t>(part) & 15u) return fail("%s: scratch must be 16-byte aligned", op);
        max_split = static_cast<int>(std::min<size_t>(part_bytes / need, kMaxStateSplit));
    }
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    if (a->layout != MI_LAYOUT_TOKEN_MAJOR && a->layout != MI_LAYOUT_CHANNEL_MAJOR) return fail("%s: layout must be 0 (token-major) or 1 (channel-major)", op);
    const bool cm = a->layout == MI_LAYOUT_CHANNEL_MAJOR;
    LinDev p;
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o;
    p.B = a->batch; p.H = a->num_heads; p.N = a->n_tokens;
    p.channel_major = cm ? 1 : 0;
    // token-major: a row is a token (heads*head_dim values); channel-major: a row is a channel (n_tokens values)
    const long row_len = cm ? a->n_tokens : D, n_rows = cm ? D : a->n_tokens;
    auto rs = [row_len](int64_t s) { return s ? static_cast<long>(s) : row_len; };
    p.q_rs = rs(a->q_row_stride); p.k_rs = rs(a->k_row_stride); p.v_rs = rs(a->v_row_stride); p.o_rs = rs(a->o_row_stride);
    p.q_bs = a->q_batch_stride ? a->q_batch_stride : p.q_rs * n_rows;
    p.k_bs = a->k_batch_stride ? a->k_batch_stride : p.k_rs * n_rows;
    p.v_bs = a->v_batch_stride ? a->v_batch_stride : p.v_rs * n_rows;
    p.o_bs = a->o_batch_stride ? a->o_batch_stride : p.o_rs * n_rows;
    if (cm) {
        // 16-byte pieces of a channel row hold 8 tokens each; the state cannot be added onto in place in the only form
        // these operands have (every work group of a head reads the old z while one of them replaces it)
        if (a->n_tokens % 8 != 0) return fail("%s: channel-major operands need n_tokens to be a multiple of 8 (got %d)", op, a->n_tokens);
        if (a->accumulate_state) return fail("%s: accumulate_state is not offered for channel-major operands (run into a second workspace and add the states)", op);
    }
    const long strides[] = {p.q_rs, p.k_rs, p.v_rs, p.o_rs, p.q_bs, p.k_bs, p.v_bs, p.o_bs};
    for (long s : strides)
        if (s % 8 != 0) return fail("%s: strides must be multiples of 8 elements", op);
    if (p.q_rs < row_len || p.k_rs < row_len || p.v_rs < row_len || p.o_rs < row_len)
        return fail("%s: row stride smaller than a row (%ld elements)", op, row_len);
    const uintptr_t al = reinterpret_cast<uintptr_t>(a->q) | reinterpret_cast<uintptr_t>(a->k) | reinterpret_cast<uintptr_t>(a->v) |
                         reinterpret_cast<uintptr_t>(a->o) | reinterpret_cast<uintptr_t>(a->workspace);
    if (al & 15u) return fail("%s: pointers must be 16-byte aligned", op);
    p.eps = a->eps;
    p.ws = static_cast<float*>(a->workspace);
    p.part = max_split > 0 ? static_cast<float*>(part) : nullptr; p.n_part = 0; p.add_to_state = 0;
    p.old_weight = a->accumulate_weight != 0.f ? a->accumulate_weight : 1.f;
    p.tokens_per_group = 0;
    if (a->form < MI_LINEAR_ATTN_FORM_BY_SIZE || a->form > MI_LINEAR_ATTN_FORM_ONE_LAUNCH) return fail("%s: form must be 0 (by size), 1 (three launches) or 2 (one launch)", op);
    p.form = a->form;
    hipStream_t st = resolve_stream(a->stream);
    const int n_cu = device_cu_count();
    return launch_t<__bf16>(p, a->head_dim, a->accumulate_state != 0, max_split, n_cu, st);
}
}  // namespace
}  // namespace mi

extern "C" {

int mi_linear_attn_supported(int32_t dtype, int32_t head_dim) { return mi::lin_supported(dtype, head_dim) ? 1 : 0; }

size_t mi_linear_attn_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim) {
    if (batch <= 0 || num_heads <= 0 || head_dim <= 0) return 0;
    return static_cast<size_t>(batch) * num_heads * (static_cast<size_t>(head_dim) * head_dim + head_dim) * sizeof(float);
}

size_t mi_linear_attn_scratch_bytes(int32_t batch, int32_t num_heads, int32_t head_dim) {
    return mi_linear_attn_workspace_bytes(batch, num_heads, head_dim) * mi::kMaxStateSplit;
}

int mi_linear_attn_relu_forward(const mi_linear_attn_args* a) {
    using mi::fail;
    const char* op = "mi_linear_attn_relu_forward";
    mi::clear_error();
    if (!a) return fail("%s: null args", op);
    if (a->struct_size != sizeof(mi_linear_attn_args)) return fail("%s: struct_size mismatch", op);
    if (!mi::lin_supported(a->dtype, a->head_dim)) return fail("%s: no kernel for dtype %d head_dim %d", op, a->dtype, a->head_dim);
    return mi::linear_attn_forward(a, op, a->scratch, a->scratch ? a->scratch_bytes : 0);
}

int mi_linear_attn_relu_forward_static_scratch(const mi_linear_attn_args* a) {
    using mi::fail;
    const char* op = "mi_linear_attn_relu_forward_static_scratch";
    mi::clear_error();
    if (!a) return fail("%s: null args", op);
    if (a->struct_size != sizeof(mi_linear_attn_args)) return fail("%s: struct_size mismatch", op);
    if (!mi::lin_supported(a->dtype, a->head_dim)) return fail("%s: no kernel for dtype %d head_dim %d", op, a->dtype, a->head_dim);
    if (a->scratch || a->scratch_bytes) return fail("%s: takes no scratch (the partial states live in the library's own static device array)", op);
    // one partial state per (batch, head) must fit; larger problems belong to the entry point that takes a caller scratch
    const size_t need = mi_linear_attn_workspace_bytes(a->batch, a->num_heads, a->head_dim);
    if (a->batch > 0 && a->num_heads > 0 && need > static_cast<size_t>(MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES))
        return fail("%s: the state of batch %d x heads %d x head_dim %d takes %zu bytes, the static scratch holds %zu: use "
                    "mi_linear_attn_relu_forward with a caller scratch", op, a->batch, a->num_heads, a->head_dim, need,
                    static_cast<size_t>(MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES));
    unsigned char* ptr = nullptr;
    if (mi::static_scratch_ptr(&ptr) != 0) return -1;
    return mi::linear_attn_forward(a, op, ptr, static_cast<size_t>(MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES));
}

}  // extern "C"
