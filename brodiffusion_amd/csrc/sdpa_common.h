// Building blocks shared by the softmax-attention kernels for gfx950: MFMA wrappers, the LDS tile
// geometry for a head dimension, the per-row visibility interval, Q fragment loading with RoPE, and
// the three per-tile stages (S^T = K Q^T, online softmax, O^T += V^T P^T).
//
// Register layouts (v_mfma_f32_32x32x16, wave64; lq = lane % 32, lh = lane / 32):
//   A operand: lane holds row lq, 8 consecutive contraction elements starting at 8*lh
//   B operand: lane holds column lq, the same 8 contraction elements
//   C/D:       lane holds column lq; acc[4b + i] is row 8b + 4*lh + i
// The score tile is computed transposed (rows = keys, columns = queries), so a lane holds scores of
// ONE query and the accumulator layout of P^T is directly the B operand of O^T += V^T P^T.
#pragma once
#include <type_traits>
#include <utility>

#include "internal.h"

namespace mi {
namespace sdpa {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBN = 64;  // key rows per LDS tile
constexpr float kNegInf = -__builtin_huge_valf();
constexpr float kLazyLog2 = 8.0f;  // raise the softmax reference only when a tile exceeds it by 2^8

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

// LDS geometry of one K/V tile for head dimension D.
template <int D> struct HeadGeo {
    static constexpr int DK = (D + 15) / 16 * 16;  // contraction extent of K Q^T (zero padded)
    static constexpr int DV = (D + 31) / 32 * 32;  // output rows of V^T P^T
    static constexpr int KC = DK / 16;
    static constexpr int VB = DV / 32;
    // K rows are read one row per lane with ds_read_b128: a stride of 16 * odd bytes puts 16
    // consecutive rows on distinct banks.
    static constexpr int K_STRIDE = DK * 2 + 16;
    // V is read by ds_read_b64_tr_b16: 4 consecutive rows x 64 contiguous bytes per 32 lanes; a
    // stride that is 64 mod 128 bytes puts those 4 rows on distinct bank groups.
    static constexpr int V_STRIDE = ((DV * 2 + 63) / 128) * 128 + 64;
    static constexpr int K_BYTES = kBN * K_STRIDE;
    static constexpr int V_BYTES = kBN * V_STRIDE;
    static constexpr int O_STRIDE = DK * 2 + 16;
    static constexpr int CPR = D / 8;  // 16-byte chunks per row that hold data
    static constexpr int NCH = kBN * CPR;
};

// v_permlane32_swap exchanges the upper 32 lanes of its first operand with the lower 32 lanes of
// its second; fed the same value twice it leaves (own, partner) in the lower half and
// (partner, own) in the upper half, so max / sum of the two results is the reduction over lanes
// l and l^32. (The results are copied to scalars before the bit cast: a bit cast applied to a
// vector element expression reads element 0 for every index with this compiler.)
__device__ __forceinline__ float exchange_max(float x) {
    const int xi = __builtin_bit_cast(int, x);
    const i32x2 r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const int r0 = r[0], r1 = r[1];
    return fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
}
__device__ __forceinline__ float exchange_sum(float x) {
    const int xi = __builtin_bit_cast(int, x);
    const i32x2 r = __builtin_amdgcn_permlane32_swap(xi, xi, false, false);
    const int r0 = r[0], r1 = r[1];
    return __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
}

// Rotate the 4 adjacent pairs held in one 16-byte chunk, FP32 arithmetic, one rounding back to T.
// (post_scale multiplies the rotated value before the rounding; 1 leaves it bit-identical to the stand-alone pass.)
template <typename T>
__device__ __forceinline__ u32x4 rope_chunk(u32x4 raw, f32x4 c, f32x4 s, float post_scale = 1.f) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    t8 x = __builtin_bit_cast(t8, raw);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const float a = static_cast<float>(x[2 * p]);
        const float b = static_cast<float>(x[2 * p + 1]);
        x[2 * p] = static_cast<T>(rope_re(a, b, c[p], s[p]) * post_scale);
        x[2 * p + 1] = static_cast<T>(rope_im(a, b, c[p], s[p]) * post_scale);
    }
    return __builtin_bit_cast(u32x4, x);
}
template <typename T>
__device__ __forceinline__ u32x4 scale_chunk(u32x4 raw, float f) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    t8 x = __builtin_bit_cast(t8, raw);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = static_cast<T>(static_cast<float>(x[e]) * f);
    return __builtin_bit_cast(u32x4, x);
}

// Visible key interval [lo, hi) of query row `qrow` (empty -> lo = hi = 0).
__device__ __forceinline__ void row_interval(const SdpaDev& p, int b, int qrow, bool qvalid, int& lo, int& hi) {
    lo = 0;
    hi = p.Lk;
    if (p.kv_valid_len) hi = min(hi, p.kv_valid_len[b]);
    if (p.mask_mode == MI_MASK_CAUSAL) {
        const int pos1 = p.q_offset + qrow + 1;
        hi = min(hi, pos1);
        if (p.window > 0) lo = max(0, pos1 - p.window);
    } else if (p.mask_mode == MI_MASK_BLOCK_CAUSAL) {
        // a scalar loop over the segment table (uniform index: scalar loads from the kernel arguments)
        int sk = p.seg_k_end[0], sc = p.seg_causal[0];
#pragma unroll 1
        for (int s = 1; s < p.n_seg; ++s)
            if (qrow >= p.seg_q_end[s - 1]) { sk = p.seg_k_end[s]; sc = p.seg_causal[s]; }
        hi = min(hi, sk);
        if (sc) hi = min(hi, p.q_offset + qrow + 1);
    }
    if (!qvalid || hi <= lo) { lo = 0; hi = 0; }
}

// Extents of the 64 rows of a wavefront (each row is held by lanes l and l^32).
struct WaveExtent { int lo_min, lo_max, hi_min, hi_max; };
__device__ __forceinline__ WaveExtent wave_extent(int lo, int hi) {
    WaveExtent w{hi > lo ? lo : 0x7fffffff, lo, hi, hi};
#pragma unroll
    for (int off = 16; off >= 1; off >>= 1) {
        w.lo_min = min(w.lo_min, __shfl_xor(w.lo_min, off));
        w.lo_max = max(w.lo_max, __shfl_xor(w.lo_max, off));
        w.hi_min = min(w.hi_min, __shfl_xor(w.hi_min, off));
        w.hi_max = max(w.hi_max, __shfl_xor(w.hi_max, off));
    }
    // identical in every lane now: move to scalar registers so tile decisions are scalar branches
    w.lo_min = __builtin_amdgcn_readfirstlane(w.lo_min);
    w.lo_max = __builtin_amdgcn_readfirstlane(w.lo_max);
    w.hi_min = __builtin_amdgcn_readfirstlane(w.hi_min);
    w.hi_max = __builtin_amdgcn_readfirstlane(w.hi_max);
    return w;
}

// The Q tile of a work group goes through LDS once. A lane needs the 16-byte pieces of ONE query row (B operand of
// K Q^T), so direct loads would touch one cache line per lane and instruction, and the RoPE tables twice as many;
// instead the rows are fetched with full-row coalescing (consecutive threads take consecutive 16-byte chunks of a row,
// of Q and of the cos / sin tables), rotated in registers and stored row-major at stride O_STRIDE (the layout the
// output staging uses later). All loads are issued before the first is used: out-of-range rows and the zero-pad
// chunk are fetched from a clamped address and blanked at the store.
// q_scale != 1 folds a factor (softmax scale times log2 e) into Q before its single rounding to T.
// The loads and the stores of the staging are separate steps, so that a kernel can put other work (the first key tiles'
// DMA) between them; `store<I0, I1>` stores the chunks of load rounds [I0, I1) with tile row `row_base` at the start of
// `Qs` (a tile may be staged in pieces through a smaller buffer when its rounds fall on whole rows).
template <typename T, int D, int NT, int ROWS>
struct QTileLoad {
    using G = HeadGeo<D>;
    static constexpr int CPRK = G::DK / 8;     // chunks per staged row (data chunks, then the zero pad)
    static constexpr int NCH = ROWS * CPRK;
    static constexpr int NI = (NCH + NT - 1) / NT;
    u32x4 raw[NI];
    f32x4 cs[NI], sn[NI];
    __device__ __forceinline__ void issue(const SdpaDev& p, const T* q_base, int q0, int tid, int last_row) {
        const bool rope = p.cos_q != nullptr && !p.rope_split;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int idx = min(tid + NT * i, NCH - 1);
            const int row = idx / CPRK, cc = min(idx - row * CPRK, G::CPR - 1);
            const int qrow = min(q0 + row, last_row);
            raw[i] = *reinterpret_cast<const u32x4*>(q_base + static_cast<long>(qrow) * p.q_rs + cc * 8);
            if (rope) {
                cs[i] = *reinterpret_cast<const f32x4*>(p.cos_q + static_cast<long>(qrow) * (D / 2) + cc * 4);
                sn[i] = *reinterpret_cast<const f32x4*>(p.sin_q + static_cast<long>(qrow) * (D / 2) + cc * 4);
            }
        }
    }
    template <int I0 = 0, int I1 = NI>
    __device__ __forceinline__ void store(unsigned char* Qs, const SdpaDev& p, int q0, int tid, int last_row, float q_scale = 1.f, int row_base = 0) const {
        const bool rope = p.cos_q != nullptr && !p.rope_split;
#pragma unroll
        for (int i = I0; i < I1; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / CPRK, cc = idx - row * CPRK;
            u32x4 v = raw[i];
            if (rope) v = rope_chunk<T>(v, cs[i], sn[i], q_scale);
            else if (q_scale != 1.f) v = scale_chunk<T>(v, q_scale);
            if (q0 + row > last_row || cc >= G::CPR) v = u32x4{0, 0, 0, 0};
            if (idx < NCH) *reinterpret_cast<u32x4*>(Qs + (row - row_base) * G::O_STRIDE + cc * 16) = v;
        }
    }
};

// Split-half pairs (x[p], x[p + D/2]) sit in different 16-byte chunks, so that rotation is a second pass over staged
// rows (tile rows [row_base, row_base + rows) at the start of `Qs`, stored and made visible by a barrier before): one
// thread takes 4 pairs, i.e. 8 bytes from each half of a row (and the 4 table entries they share), and writes them back.
// Same arithmetic and single rounding as the stand-alone pass; rows past the end are zero.
template <typename T, int D, int NT>
__device__ __forceinline__ void rope_split_staged(unsigned char* Qs, const SdpaDev& p, int q0, int tid, int last_row, float q_scale, int row_base, int rows) {
    using G = HeadGeo<D>;
    typedef T t4 __attribute__((ext_vector_type(4)));
    constexpr int UPR = D / 8;             // units of 4 pairs per row
    for (int u = tid; u < rows * UPR; u += NT) {
        const int row = u / UPR, g = u - row * UPR;
        const int qrow = min(q0 + row_base + row, last_row);
        const f32x4 c4 = *reinterpret_cast<const f32x4*>(p.cos_q + static_cast<long>(qrow) * (D / 2) + g * 4);
        const f32x4 s4 = *reinterpret_cast<const f32x4*>(p.sin_q + static_cast<long>(qrow) * (D / 2) + g * 4);
        t4* const lo_p = reinterpret_cast<t4*>(Qs + row * G::O_STRIDE + g * 8);
        t4* const hi_p = reinterpret_cast<t4*>(Qs + row * G::O_STRIDE + D + g * 8);
        t4 lo = *lo_p, hi = *hi_p;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const float a = static_cast<float>(lo[e]), b = static_cast<float>(hi[e]);
            lo[e] = static_cast<T>(rope_re(a, b, c4[e], s4[e]) * q_scale);
            hi[e] = static_cast<T>(rope_im(a, b, c4[e], s4[e]) * q_scale);
        }
        *lo_p = lo;
        *hi_p = hi;
    }
}

template <typename T, int D, int NT, int ROWS>
__device__ __forceinline__ void stage_q_tile(unsigned char* Qs, const SdpaDev& p, const T* q_base, int q0, int tid, float q_scale = 1.f,
                                             int last_row_override = -1) {
    const int last_row = last_row_override >= 0 ? last_row_override : p.Lq - 1;   // (a packed sequence has its own length)
    QTileLoad<T, D, NT, ROWS> ql;
    ql.issue(p, q_base, q0, tid, last_row);
    ql.store(Qs, p, q0, tid, last_row, q_scale);
    if (p.cos_q != nullptr && p.rope_split) {
        __syncthreads();
        rope_split_staged<T, D, NT>(Qs, p, q0, tid, last_row, q_scale, 0, ROWS);
    }
}

// Q fragments of this lane's query row (tile row `trow`) from the staged tile.
template <typename T, int D>
__device__ __forceinline__ void read_q_frags(typename Mma<T>::v8 (&qf)[HeadGeo<D>::KC], const unsigned char* Qs, int trow, int lh) {
    using V8 = typename Mma<T>::v8;
#pragma unroll
    for (int c = 0; c < HeadGeo<D>::KC; ++c)
        qf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Qs + trow * HeadGeo<D>::O_STRIDE + (16 * c + 8 * lh) * 2));
}

// The MFMA work of one step as a single software-pipelined stream: first O^T += V^T P^T for one
// 64-key tile (if DO_PV), then S^T = K Q^T for one 64-key tile (if DO_QK). Every MFMA takes its A
// operand from LDS; the LDS reads run kAhead operands ahead of the MFMA that consumes them so that
// LDS latency hides behind the matrix pipe, and the order is pinned with scheduling barriers.
//   PV operand (c4, vb): V^T fragment = head-dim block vb x 16-key chunk c4, through two LDS transpose
//     reads (within 16 lanes, lane j supplies the address of 4 consecutive head-dim elements of key
//     row j/4, and lane i receives 4 consecutive keys of head-dim column i).
//   QK operand (kb, c):  K fragment = key block kb x 16 head-dim elements, one 16-byte read per lane.
constexpr int kAhead = 4;
#define MI_SCHED_BARRIER __builtin_amdgcn_sched_barrier(0);

// `mid` is called once, a few MFMAs into the stream: work placed there (tile movement) issues in
// the shadow of the matrix pipe.
struct NoMid { __device__ __forceinline__ void operator()() const {} };

// TO_EXPONENT (needs both products): the stream scores first and then, in the shadow of the PV MFMAs (which do not
// touch the scores), turns every raw score s into the softmax exponent x = s * cl2 + neg_ref with one FP32 fused
// multiply-add, a few per MFMA slot, first block first (its MFMAs retired long ago). The scale therefore never touches a
// 16-bit operand, and the VALU work costs no time of its own while the matrix pipe is the busier unit.
template <int NPV, int J>
__device__ __forceinline__ void scores_to_exponents(f32x16 (&sacc)[2], float cl2, float neg_ref) {
    constexpr int E0 = 32 * J / NPV, E1 = 32 * (J + 1) / NPV;
#pragma unroll
    for (int e = E0; e < E1; ++e) sacc[e >> 4][e & 15] = __builtin_fmaf(sacc[e >> 4][e & 15], cl2, neg_ref);
}

template <typename T, int D, bool DO_PV, bool DO_QK, typename Mid = NoMid, bool TO_EXPONENT = false>
__device__ __forceinline__ void mfma_stream(const unsigned char* Vs, const unsigned char* Ks, const typename Mma<T>::v8 (&pf)[4],
                                            const typename Mma<T>::v8 (&qf)[HeadGeo<D>::KC], f32x16 (&oacc)[HeadGeo<D>::VB],
                                            f32x16 (&sacc)[2], int lane, Mid mid = Mid(), float cl2 = 1.f, float neg_ref = 0.f) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    static_assert(!TO_EXPONENT || (DO_PV && DO_QK), "the exponent pass rides under the PV product of a stream that also scores");
    constexpr int NPV = DO_PV ? 4 * G::VB : 0;
    constexpr int NQK = DO_QK ? 2 * G::KC : 0;
    constexpr int N = NPV + NQK;
    if constexpr (N == 0) return;
    // position i of the stream: PV first by default, QK first when the exponents are formed under the PV part
    constexpr int PV0 = TO_EXPONENT ? NQK : 0;     // first PV position
    constexpr int QK0 = TO_EXPONENT ? 0 : NPV;     // first QK position
    const int lq = lane & 31;
    const int lh = lane >> 5;
    const int trow = (lane & 15) >> 2;
    const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
    const unsigned char* const vlane = Vs + (4 * lh + trow) * G::V_STRIDE + tcol * 2;
    const unsigned char* const klane = Ks + lq * G::K_STRIDE + 8 * lh * 2;
    auto is_pv = [](int i) { return i >= PV0 && i < PV0 + NPV; };
    auto fetch = [&](int i) -> V8 {
        if (is_pv(i)) {
            const int j = i - PV0;
            const int c4 = j / G::VB, vb = j % G::VB;
            const unsigned char* vptr = vlane + 16 * c4 * G::V_STRIDE + 32 * vb * 2;
            const s16x4 v_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vptr));
            const s16x4 v_hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vptr + 8 * G::V_STRIDE));
            const s16x8 a = __builtin_shufflevector(v_lo, v_hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(V8, a);
        } else {
            const int k = i - QK0;
            const int kb = k / G::KC, c = k % G::KC;
            const u32x4 a = *reinterpret_cast<const u32x4*>(klane + 32 * kb * G::K_STRIDE + 16 * c * 2);
            return __builtin_bit_cast(V8, a);
        }
    };
    V8 ring[kAhead];
#pragma unroll
    for (int i = 0; i < kAhead && i < N; ++i) ring[i] = fetch(i);
    [&]<int... I>(std::integer_sequence<int, I...>) {
        ([&] {
            constexpr int i = I;
            const V8 a = ring[i % kAhead];
            if constexpr (i >= PV0 && i < PV0 + NPV) {
                constexpr int j = i - PV0;
                constexpr int c4 = j / G::VB, vb = j % G::VB;
                oacc[vb] = Mma<T>::run(a, pf[c4], oacc[vb]);
            } else {
                constexpr int k = i - QK0;
                constexpr int kb = k / G::KC, c = k % G::KC;
                if constexpr (c == 0) {
                    const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    sacc[kb] = Mma<T>::run(a, qf[c], zero);
                } else {
                    sacc[kb] = Mma<T>::run(a, qf[c], sacc[kb]);
                }
            }
            if constexpr (i + kAhead < N) ring[i % kAhead] = fetch(i + kAhead);
            if constexpr (TO_EXPONENT && i >= PV0 && i < PV0 + NPV) scores_to_exponents<NPV, i - PV0>(sacc, cl2, neg_ref);
            MI_SCHED_BARRIER
            if constexpr (i == (N > 8 ? 5 : 0)) {
                mid();
                MI_SCHED_BARRIER
            }
        }(), ...);
    }(std::make_integer_sequence<int, N>{});
}

// score, or -inf when `x` is outside [0, top] (x = key - lo, top = hi - 1 - lo) or `extra` is negative: the sign of
// x | (top - x) | extra selects the bits of -inf. Integer arithmetic on the lane's own values on purpose: 32 compares
// would put 32 lane masks into scalar registers at once, and the scalars that live through the key loop would be
// spilled around them. (The score is taken by value: a bit cast of a vector element expression reads element 0 for
// every index with this compiler.)
__device__ __forceinline__ float blank_outside(float score, int x, int top, int extra = 0) {
    const unsigned out = static_cast<unsigned>((x | (top - x) | extra) >> 31);   // all ones when blanked
    const unsigned bits = __builtin_bit_cast(unsigned, score);
    return __builtin_bit_cast(float, (bits & ~out) | (0xff800000u & out));
}

// Factors carried by the rows of the cached prefix (the dial's scalar times the optional per-row weight), handed to the
// softmax of a prefix tile by value; on == false: the tile has none. Rows of a partly filled last prefix tile that lie
// past the prefix read its last entry; their scores are blanked anyway.
struct PrefixScale {
    bool on = false;
    const float* k_row = nullptr; const float* v_row = nullptr;
    float ks = 1.f, vs = 1.f;
    int Lp = 0;
    __device__ __forceinline__ float k(int key) const { return k_row ? ks * k_row[min(key, Lp - 1)] : ks; }
    __device__ __forceinline__ float v(int key) const { return v_row ? vs * v_row[min(key, Lp - 1)] : vs; }
};
__device__ __forceinline__ PrefixScale prefix_scale_of(const SdpaDev& p, bool tile_in_prefix) {
    PrefixScale s;
    s.on = p.prefix_scaled && tile_in_prefix;
    s.k_row = p.pk_row; s.v_row = p.pv_row; s.ks = p.pk_scale; s.vs = p.pv_scale; s.Lp = p.Lp;
    return s;
}
// key index of accumulator element e of key block kb for this lane half
__device__ __forceinline__ int key_of(int j0, int kb, int e, int lh) { return j0 + 32 * kb + 8 * (e >> 2) + 4 * lh + (e & 3); }

// Online-softmax state of one lane (one query row, shared with lane l^32).
// m is the reference the exponentials are taken against; it is raised only when a tile's maximum
// exceeds it by more than 2^kLazyLog2, so most tiles skip the rescale of l and O. The result does
// not depend on which reference is used.
struct SoftmaxState {
    float m = kNegInf;  // raw-score units
    float mc = 0.f;     // m * scale_log2 (0 while m is -inf)
    float l = 0.f;      // this lane's share of the denominator
};

// Masks (if `masked`, a wave-uniform flag), exponentiates and packs one score tile into the B operands
// of the PV product. The mask step only touches the scores, so the two cases share every other
// instruction and the accumulators are updated at one place only (separate masked / unmasked copies of
// this function cost the register allocator ~70 registers in copies of O).
template <typename T, int D, bool PSCALE = false>
__device__ __forceinline__ void softmax_tile(f32x16 (&sacc)[2], typename Mma<T>::v8 (&pf)[4], f32x16 (&oacc)[HeadGeo<D>::VB],
                                             SoftmaxState& st, float cl2, float lazy_raw, bool masked, int j0, int lo, int hi,
                                             int lh, const float* mask_tile, const float* bias_row = nullptr, int bias_cols = 0,
                                             float bias_k = 0.f, PrefixScale prefix = PrefixScale()) {
    // tile of the cached prefix whose rows carry factors (PSCALE instances only): K's factor multiplies the raw scores
    if (PSCALE && prefix.on) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[kb][e] *= prefix.k(key_of(j0, kb, e, lh));
    }
    if (masked) {
        // additive logit bias of this lane's query row (null: none) for keys below bias_cols, in raw-score units
        if (bias_row) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const int key = j0 + 32 * kb + 8 * (e >> 2) + 4 * lh + (e & 3);
                    if (key < bias_cols) sacc[kb][e] = __builtin_fmaf(bias_row[key], bias_k, sacc[kb][e]);
                }
        }
        // mask_tile: the 64 key-mask values of this tile staged in LDS (null when the call has no key mask)
        if (mask_tile) {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int bb = 0; bb < 4; ++bb) {
                    const int kbase = 32 * kb + 8 * bb + 4 * lh;
                    const f32x4 mk = *reinterpret_cast<const f32x4*>(mask_tile + kbase);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const float score = sacc[kb][4 * bb + i], mv = mk[i];
                        // a key-mask value of +-0 hides the key: (bits of |m|) - 1 is negative exactly then
                        const int hidden = static_cast<int>(__builtin_bit_cast(unsigned, mv) & 0x7fffffffu) - 1;
                        sacc[kb][4 * bb + i] = blank_outside(score, j0 + kbase + i - lo, hi - 1 - lo, hidden);
                    }
                }
        } else {
            const int d0 = j0 + 4 * lh - lo, top = hi - 1 - lo;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float score = sacc[kb][e];
                    sacc[kb][e] = blank_outside(score, d0 + 32 * kb + 8 * (e >> 2) + (e & 3), top);
                }
        }
    }
    float mloc = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
    for (int e = 1; e < 16; ++e) mloc = fmaxf(mloc, fmaxf(sacc[0][e], sacc[1][e]));
    mloc = exchange_max(mloc);
    if (__any(mloc > st.m + lazy_raw)) {
        const float m_new = fmaxf(st.m, mloc);
        const float mc_new = (m_new == kNegInf) ? 0.f : m_new * cl2;
        const float alpha = __builtin_amdgcn_exp2f(st.m * cl2 - mc_new);  // 1 where unchanged, 0 from -inf
        st.m = m_new;
        st.mc = mc_new;
        st.l *= alpha;
#pragma unroll
        for (int vb = 0; vb < HeadGeo<D>::VB; ++vb)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[vb][e] *= alpha;
    }
    float lsum0 = 0.f, lsum1 = 0.f;
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[0][e], cl2, -st.mc));
        const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[1][e], cl2, -st.mc));
        sacc[0][e] = p0;
        sacc[1][e] = p1;
        lsum0 += p0;
        lsum1 += p1;
    }
    st.l += lsum0 + lsum1;
    // ... and V's factor multiplies the probabilities, after the row sum has been taken
    if (PSCALE && prefix.on) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[kb][e] *= prefix.v(key_of(j0, kb, e, lh));
    }
    // P^T as B operand: 16-key chunk c4 is acc[8*(c4%2) .. +7] of block c4/2
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4)
#pragma unroll
        for (int t = 0; t < 8; ++t) pf[c4][t] = static_cast<T>(sacc[c4 >> 1][8 * (c4 & 1) + t]);
}

// Softmax step of the 256-row kernels. The scores arrive as exponents relative to the row's reference,
// x = s * (scale * log2 e) - ref (one FP32 fused multiply-add per raw score, done by the MFMA stream in the shadow of the
// PV product: Q, K and the raw scores never see the scale), so P = exp2(x) needs no further arithmetic and the usual tile
// maximum is not computed at all: per 64-key tile and lane 32 v_exp, 32 adds and 16 packs.
//   * The reference of a row is the maximum of its first tile with a visible key (then its largest term is 1, so the
//     denominator stays >= 1), and is raised to a later tile's maximum only when that tile's terms get large (lane sum
//     above 2^10, or overflow). Any reference gives the same softmax; these two rules keep every term within FP32 / T range.
//   * Both cases, and rows that have not seen a key yet, take the slow path below (wave-uniform branch): row maximum,
//     shift of l, O, the exponents and the reference, new exponentials. Lanes l and l^32 share a row and decide from
//     row-wide values only.
// acc + v[2i] + v[2i+1], products with 1 exact, FP32 accumulation (v_dot2c_f32_bf16 / v_dot2c_f32_f16).
template <typename T>
__device__ __forceinline__ float pair_sum(const typename Mma<T>::v8& v, int i, float acc) {
    typedef T t2 __attribute__((ext_vector_type(2)));
    const t2 pr = {v[2 * i], v[2 * i + 1]};
    const t2 one = {static_cast<T>(1.f), static_cast<T>(1.f)};
    if constexpr (std::is_same_v<T, __bf16>) return __builtin_amdgcn_fdot2_f32_bf16(pr, one, acc, false);
    else return __builtin_amdgcn_fdot2(pr, one, acc, false);
}

// What the XTRA instances of the 256-row kernels bring to a tile's softmax: the visibility bits of the tile's 64 keys (bit i
// of kw0: key i of the tile passes the key mask, kw1: key 32 + i; all ones without a mask) and this lane's row of the additive
// logit bias (null: the tile or the row has none), which is given in natural-log units and added to the exponents times log2 e.
struct TileExtra {
    unsigned kw0 = ~0u, kw1 = ~0u;
    const float* bias_row = nullptr;
    int bias_cols = 0;
    bool bias_vec = false;   // the whole tile lies below bias_cols and its 4-key pieces are 16-byte aligned in every row
};

struct RelSoftmaxState {
    float l = 0.f;          // this lane's share of the denominator
    float neg_ref = 0.f;    // minus the row's reference, in exponent (base-2) units
    bool started = false;   // the row has a reference (it has seen a visible key)
};
constexpr float kRelSumMax = 1024.f;

template <typename T, int D, bool PSCALE = false, bool XTRA = false>
__device__ __forceinline__ void softmax_tile_rel(f32x16 (&sacc)[2], typename Mma<T>::v8 (&pf)[4], f32x16 (&oacc)[HeadGeo<D>::VB],
                                                 RelSoftmaxState& st, bool masked, bool dead_row, int j0, int lo, int hi, int lh,
                                                 PrefixScale prefix = PrefixScale(), TileExtra xt = TileExtra()) {
    // Tile of the cached prefix whose rows carry factors (wave-uniform flag; PSCALE instances only, so that the other
    // instances keep their register budget). The scores arrive as exponents x = s * cl2 - ref; K's factor f belongs on s:
    // x' = f * (x + ref) - ref.
    if (PSCALE && prefix.on) {
        const float nr = st.neg_ref;
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[kb][e] = __builtin_fmaf(prefix.k(key_of(j0, kb, e, lh)), sacc[kb][e] - nr, nr);
    }
    if (masked) {
        const int d0 = j0 + 4 * lh - lo, top = hi - 1 - lo;   // keys outside [lo, hi) become -inf
        if constexpr (XTRA) {
            if (xt.bias_row) {
                constexpr float kLog2e = 1.4426950408889634f;
                if (xt.bias_vec) {
                    // a lane's 32 keys are 8 pieces of 4 consecutive ones: all loads go out before the first is used
                    f32x4 bv[2][4];
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int bb = 0; bb < 4; ++bb) bv[kb][bb] = *reinterpret_cast<const f32x4*>(xt.bias_row + j0 + 32 * kb + 8 * bb + 4 * lh);
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int e = 0; e < 16; ++e) sacc[kb][e] = __builtin_fmaf(bv[kb][e >> 2][e & 3], kLog2e, sacc[kb][e]);
                } else {
#pragma unroll
                    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                        for (int e = 0; e < 16; ++e) {
                            const int key = key_of(j0, kb, e, lh);
                            if (key < xt.bias_cols) sacc[kb][e] = __builtin_fmaf(xt.bias_row[key], kLog2e, sacc[kb][e]);
                        }
                }
            }
            // hidden keys as set bits, this lane half's keys first: accumulator element e of block kb is key
            // 32 kb + 4 lh + c with c = 8 (e / 4) + e % 4, and bit c moved to the sign position blanks the score
            const unsigned h0 = ~(xt.kw0 >> (4 * lh)), h1 = ~(xt.kw1 >> (4 * lh));
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float score = sacc[kb][e];
                    const int c = 8 * (e >> 2) + (e & 3);
                    sacc[kb][e] = blank_outside(score, d0 + 32 * kb + c, top, static_cast<int>((kb ? h1 : h0) << (31 - c)));
                }
        } else {
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float score = sacc[kb][e];
                    sacc[kb][e] = blank_outside(score, d0 + 32 * kb + 8 * (e >> 2) + (e & 3), top);
                }
        }
    }
    // Row sum of the tile. Up to head_dim 96 the key step is bound by its VALU instructions, and the sum is taken from the
    // packed 16-bit P (one v_dot2c per pair against (1, 1), FP32 accumulation: half the instructions, and the denominator
    // sums exactly the values the PV product uses; measured 4 % faster at head_dim 40 and 72). From 112 on the matrix
    // pipe is the busier unit and the same change measured 6 % slower, so there the FP32 exponentials are added.
    // (not in the XTRA instances: their denominators are an output, from which the attention map is rebuilt in FP32, so they
    // sum the exponentials before the rounding to 16 bits.)
    constexpr bool PAIR_SUM = HeadGeo<D>::VB < 4 && !XTRA;
    auto exponentiate = [&]() -> float {
        float s0 = 0.f, s1 = 0.f;
        if (PSCALE && prefix.on) {
            // V's factor multiplies the probabilities that go into the PV product; the row sum takes them as they are
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4)
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const int kb = c4 >> 1, e = 8 * (c4 & 1) + t;
                    const float pr = __builtin_amdgcn_exp2f(sacc[kb][e]);
                    pf[c4][t] = static_cast<T>(pr * prefix.v(key_of(j0, kb, e, lh)));
                    if (t & 1) s1 += pr; else s0 += pr;
                }
            return s0 + s1;
        }
        // P^T as B operand: 16-key chunk c4 is acc[8*(c4%2) .. +7] of block c4/2
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4) {
            if constexpr (PAIR_SUM) {
#pragma unroll
                for (int t = 0; t < 8; ++t) pf[c4][t] = static_cast<T>(__builtin_amdgcn_exp2f(sacc[c4 >> 1][8 * (c4 & 1) + t]));
                s0 = pair_sum<T>(pf[c4], 0, s0);
                s1 = pair_sum<T>(pf[c4], 1, s1);
                s0 = pair_sum<T>(pf[c4], 2, s0);
                s1 = pair_sum<T>(pf[c4], 3, s1);
            } else {
#pragma unroll
                for (int t = 0; t < 8; t += 2) {
                    const float p0 = __builtin_amdgcn_exp2f(sacc[c4 >> 1][8 * (c4 & 1) + t]);
                    const float p1 = __builtin_amdgcn_exp2f(sacc[c4 >> 1][8 * (c4 & 1) + t + 1]);
                    pf[c4][t] = static_cast<T>(p0);
                    pf[c4][t + 1] = static_cast<T>(p1);
                    s0 += p0;
                    s1 += p1;
                }
            }
        }
        return s0 + s1;
    };
    float ls = exponentiate();
    const bool fine = (st.started || dead_row) && ls < kRelSumMax;   // false also for inf / nan sums
    if (__any(!fine)) {
        float mloc = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
        for (int e = 1; e < 16; ++e) mloc = fmaxf(mloc, fmaxf(sacc[0][e], sacc[1][e]));
        mloc = exchange_max(mloc);
        const bool visible = mloc > kNegInf;
        // a started row only ever moves its reference up (its terms then stay <= 1)
        const float shift = !visible ? 0.f : (st.started ? fmaxf(mloc, 0.f) : mloc);
        const float alpha = st.started ? __builtin_amdgcn_exp2f(-shift) : 1.f;   // nothing accumulated before the first key
        st.started = st.started || visible;
        st.l *= alpha;
#pragma unroll
        for (int vb = 0; vb < HeadGeo<D>::VB; ++vb)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[vb][e] *= alpha;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            sacc[0][e] -= shift;
            sacc[1][e] -= shift;
        }
        st.neg_ref -= shift;
        ls = exponentiate();
    }
    st.l += ls;
}

// 1 / l for a row with visible keys, 0 for a row without any (its output is zero, src/dit/common.cpp:293). The value is made
// opaque to the optimiser on purpose: the library is compiled with -fno-honor-nans, under which O * select(l > 0, 1 / l, 0)
// may be folded on the assumption that O is never NaN. A row whose scores were not finite has O = NaN and l = NaN and must
// come out NaN (src/dit/common.cpp:269-305 makes it so); the hardware multiply delivers that (NaN * 0 = NaN) as long as it
// is executed, whichever way the comparison on a NaN falls.
__device__ __forceinline__ float row_inverse(float l_tot) {
    float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    asm volatile("" : "+v"(inv));
    return inv;
}

// Normalised output rows of one wavefront into the LDS staging area (row-major, O_STRIDE).
template <typename T, int D>
__device__ __forceinline__ void stage_output(unsigned char* Os, int row, int lh, const f32x16 (&oacc)[HeadGeo<D>::VB], float inv) {
    using G = HeadGeo<D>;
    typedef T t4 __attribute__((ext_vector_type(4)));
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
            const int d0 = 32 * vb + 8 * bb + 4 * lh;
            if (d0 < D) {
                t4 ov;
#pragma unroll
                for (int i = 0; i < 4; ++i) ov[i] = static_cast<T>(oacc[vb][4 * bb + i] * inv);
                *reinterpret_cast<t4*>(Os + row * G::O_STRIDE + d0 * 2) = ov;
            }
        }
}

}  // namespace sdpa
}  // namespace mi
