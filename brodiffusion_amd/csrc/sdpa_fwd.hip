// Flash-style softmax attention forward for gfx950 (MI355X), hand-written.
//
// One work group = 4 wavefronts = 128 query rows of one (batch, head); each wavefront
// owns 32 query rows for the whole key loop. Key/value tiles of 64 rows are staged in
// LDS and shared by the 4 wavefronts.
//
// The score tile is computed TRANSPOSED, S^T = K Q^T, with v_mfma_f32_32x32x16:
//   A = K tile from LDS   (lane l: key row l%32, 8 contiguous head-dim elements at 8*(l/32))
//   B = Q^T in registers  (lane l: query l%32,   same 8 head-dim elements)
//   C = S^T               (lane l: query l%32;   acc[4b+i] is key 8b + 4*(l/32) + i)
// so every lane holds scores of ONE query: the online-softmax row statistics need one
// exchange between lanes l and l^32 (v_permlane32_swap) and no LDS. The accumulator layout
// of P^T is already the B-operand layout of the second product O^T = V^T P^T (keys of a
// 16-key chunk in the order acc[8c'..8c'+7]), so P never leaves registers. V^T comes from
// the row-major V tile through ds_read_b64_tr_b16 (LDS transpose read), which hands each
// lane 4 consecutive keys of one head-dim column.
//
// Not in HBM: scores, probabilities, rotated Q/K (RoPE is applied as Q and K are loaded),
// the [prefix ; fresh] K/V concatenation (two source pointers), any mask tensor (per-row
// visible-key intervals; key tiles outside every row's interval are skipped).
#include "internal.h"

namespace mi {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128;      // query rows per work group
constexpr int kBN = 64;       // key rows per LDS tile
constexpr int kThreads = 256;
constexpr float kNegInf = -__builtin_huge_valf();

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

template <int D> struct Geo {
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
    static constexpr int M_BYTES = kBN * 4;
    static constexpr int O_STRIDE = DK * 2 + 16;
    static constexpr int O_BYTES = kBM * O_STRIDE;
    static constexpr int KV_BYTES = K_BYTES + V_BYTES + M_BYTES;
    static constexpr int LDS_BYTES = (KV_BYTES > O_BYTES ? KV_BYTES : O_BYTES);
    static constexpr int CPR = D / 8;  // 16-byte chunks per row that hold data
    static constexpr int NCH = kBN * CPR;
    static constexpr int NLD = (NCH + kThreads - 1) / kThreads;
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

// Rotate the 4 adjacent pairs held in one 16-byte chunk: (x0, x1) -> (x0 c - x1 s, x0 s + x1 c),
// FP32 arithmetic, one rounding back to T.
template <typename T>
__device__ __forceinline__ u32x4 rope_chunk(u32x4 raw, f32x4 c, f32x4 s) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    t8 x = __builtin_bit_cast(t8, raw);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const float a = static_cast<float>(x[2 * p]);
        const float b = static_cast<float>(x[2 * p + 1]);
        x[2 * p] = static_cast<T>(rope_re(a, b, c[p], s[p]));
        x[2 * p + 1] = static_cast<T>(rope_im(a, b, c[p], s[p]));
    }
    return __builtin_bit_cast(u32x4, x);
}

template <typename T, int D, bool ROPE_K>
__global__ void __launch_bounds__(kThreads, (D > 128 ? 1 : 2)) sdpa_fwd_kernel(const SdpaDev p) {
    using G = Geo<D>;
    using V8 = typename Mma<T>::v8;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* const Ks = smem;
    unsigned char* const Vs = smem + G::K_BYTES;
    float* const Ms = reinterpret_cast<float*>(smem + G::K_BYTES + G::V_BYTES);
    __shared__ int red[8];

    // Work-group id -> (batch, head, query tile). Hardware deals consecutive work-group ids
    // round-robin over the 8 XCDs; undo that so each XCD (one L2) gets a contiguous run of
    // logical tiles, i.e. query tiles that share the same K/V.
    const int chunk = (p.n_blocks + 7) >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    if (logical >= p.n_blocks) return;
    int qt = logical % p.n_q_tiles;
    const int bh = logical / p.n_q_tiles;
    const int h = bh % p.H;
    const int b = bh / p.H;
    if (p.mask_mode != MI_MASK_NONE) qt = p.n_q_tiles - 1 - qt;  // longest key ranges first

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int lq = lane & 31;
    const int lh = lane >> 5;
    const int q0 = qt * kBM;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < p.Lq;

    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    const int hk = h / p.kv_group;
    const T* const k_base = static_cast<const T*>(p.k) + b * p.k_bs + hk * D;
    const T* const v_base = static_cast<const T*>(p.v) + b * p.v_bs + hk * D;
    const T* const kp_base = p.kp ? static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D : nullptr;
    const T* const vp_base = p.vp ? static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D : nullptr;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;

    // ── visible key interval [lo, hi) of this lane's query row ──
    int lo = 0, hi = p.Lk;
    if (p.kv_valid_len) hi = min(hi, p.kv_valid_len[b]);
    if (p.mask_mode == MI_MASK_CAUSAL) {
        const int pos1 = p.q_offset + qrow + 1;
        hi = min(hi, pos1);
        if (p.window > 0) lo = max(0, pos1 - p.window);
    } else if (p.mask_mode == MI_MASK_BLOCK_CAUSAL) {
        // static indices only: the segment table stays in scalar registers
        int sk = p.seg_k_end[0], sc = p.seg_causal[0];
#pragma unroll
        for (int s = 1; s < MI_MAX_SEGMENTS; ++s)
            if (s < p.n_seg && qrow >= p.seg_q_end[s - 1]) { sk = p.seg_k_end[s]; sc = p.seg_causal[s]; }
        hi = min(hi, sk);
        if (sc) hi = min(hi, p.q_offset + qrow + 1);
    }
    if (!qvalid || hi <= lo) { lo = 0; hi = 0; }
    // wave-wide and group-wide extents
    int w_lo_min = hi > lo ? lo : 0x7fffffff, w_hi_max = hi, w_hi_min = hi, w_lo_max = lo;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        w_lo_min = min(w_lo_min, __shfl_xor(w_lo_min, off));
        w_hi_max = max(w_hi_max, __shfl_xor(w_hi_max, off));
        w_hi_min = min(w_hi_min, __shfl_xor(w_hi_min, off));
        w_lo_max = max(w_lo_max, __shfl_xor(w_lo_max, off));
    }
    if (lane == 0) { red[wave] = w_lo_min; red[4 + wave] = w_hi_max; }

    // ── zero the LDS pad columns once (tile loads never touch them) ──
    if constexpr (G::DK > D) {
        for (int r = tid; r < kBN; r += kThreads)
            *reinterpret_cast<u32x4*>(Ks + r * G::K_STRIDE + D * 2) = u32x4{0, 0, 0, 0};
    }
    if constexpr (G::DV > D) {
        constexpr int PC = (G::DV - D) / 8;
        for (int i = tid; i < kBN * PC; i += kThreads)
            *reinterpret_cast<u32x4*>(Vs + (i / PC) * G::V_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
    }
    __syncthreads();
    const int g_lo = min(min(red[0], red[1]), min(red[2], red[3]));
    const int kv_stop = max(max(red[4], red[5]), max(red[6], red[7]));
    const int kv_start = g_lo == 0x7fffffff ? 0 : (g_lo / kBN) * kBN;

    // ── Q fragments (B operand of K Q^T), RoPE applied on the way in ──
    V8 qf[G::KC];
#pragma unroll
    for (int c = 0; c < G::KC; ++c) {
        const int d0 = 16 * c + 8 * lh;
        u32x4 raw = u32x4{0, 0, 0, 0};
        if (qvalid && d0 < D) {
            raw = *reinterpret_cast<const u32x4*>(q_base + static_cast<long>(qrow) * p.q_rs + d0);
            if (p.cos_q) {
                const f32x4 cs = *reinterpret_cast<const f32x4*>(p.cos_q + static_cast<long>(qrow) * (D / 2) + d0 / 2);
                const f32x4 sn = *reinterpret_cast<const f32x4*>(p.sin_q + static_cast<long>(qrow) * (D / 2) + d0 / 2);
                raw = rope_chunk<T>(raw, cs, sn);
            }
        }
        qf[c] = __builtin_bit_cast(V8, raw);
    }

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    float m_run = kNegInf;  // running max of raw scores
    float l_run = 0.f;      // this lane's share of the running denominator
    const float cl2 = p.scale_log2;

    // ── tile prefetch registers ──
    u32x4 kreg[G::NLD], vreg[G::NLD];
    float mreg = 1.f;

    auto issue_loads = [&](int j0) {
#pragma unroll
        for (int i = 0; i < G::NLD; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            const int j = j0 + row;
            kreg[i] = u32x4{0, 0, 0, 0};
            vreg[i] = u32x4{0, 0, 0, 0};
            if (idx < G::NCH && j < kv_stop) {
                if (j < p.Lp) {
                    kreg[i] = *reinterpret_cast<const u32x4*>(kp_base + static_cast<long>(j) * p.kp_rs + cc * 8);
                    vreg[i] = *reinterpret_cast<const u32x4*>(vp_base + static_cast<long>(j) * p.vp_rs + cc * 8);
                } else {
                    const long jr = j - p.Lp;
                    kreg[i] = *reinterpret_cast<const u32x4*>(k_base + jr * p.k_rs + cc * 8);
                    vreg[i] = *reinterpret_cast<const u32x4*>(v_base + jr * p.v_rs + cc * 8);
                }
            }
        }
        if (p.key_mask && tid < kBN) {
            const int j = j0 + tid;
            mreg = j < p.Lk ? p.key_mask[b * p.key_mask_bs + j] : 0.f;
        }
    };
    auto store_tile = [&](int j0) {
        // The rotation tables are fetched here rather than with the tile: they are L2 hits
        // shared by every head, and holding them across the MFMA section would cost
        // 8 registers per chunk exactly where pressure peaks. Prefix rows are stored rotated.
        f32x4 creg[ROPE_K ? G::NLD : 1], sreg[ROPE_K ? G::NLD : 1];
        if constexpr (ROPE_K) {
#pragma unroll
            for (int i = 0; i < G::NLD; ++i) {
                const int idx = tid + kThreads * i;
                const int row = idx / G::CPR;
                const int cc = idx - row * G::CPR;
                const int j = j0 + row;
                creg[i] = f32x4{1.f, 1.f, 1.f, 1.f};
                sreg[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                if (idx < G::NCH && j < kv_stop && j >= p.Lp) {
                    const long jr = j - p.Lp;
                    creg[i] = *reinterpret_cast<const f32x4*>(p.cos_k + jr * (D / 2) + cc * 4);
                    sreg[i] = *reinterpret_cast<const f32x4*>(p.sin_k + jr * (D / 2) + cc * 4);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < G::NLD; ++i) {
            const int idx = tid + kThreads * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (idx < G::NCH) {
                u32x4 kk = kreg[i];
                if constexpr (ROPE_K) kk = rope_chunk<T>(kk, creg[i], sreg[i]);
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = kk;
                *reinterpret_cast<u32x4*>(Vs + row * G::V_STRIDE + cc * 16) = vreg[i];
            }
        }
        if (p.key_mask && tid < kBN) Ms[tid] = mreg;
    };

    if (kv_start < kv_stop) issue_loads(kv_start);

    for (int j0 = kv_start; j0 < kv_stop; j0 += kBN) {
        store_tile(j0);
        __syncthreads();
        if (j0 + kBN < kv_stop) issue_loads(j0 + kBN);

        // wavefronts none of whose rows can see this tile only help with the loads
        if (j0 < w_hi_max && j0 + kBN > w_lo_min) {
            // ── S^T = K Q^T : 2 blocks of 32 keys ──
            f32x16 sacc[2];
#pragma unroll
            for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
                for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
#pragma unroll
                for (int c = 0; c < G::KC; ++c) {
                    const u32x4 a = *reinterpret_cast<const u32x4*>(Ks + (32 * kb + lq) * G::K_STRIDE + (16 * c + 8 * lh) * 2);
                    sacc[kb] = Mma<T>::run(__builtin_bit_cast(V8, a), qf[c], sacc[kb]);
                }
            }
            // ── visibility ──
            const bool need_mask = (j0 + kBN > w_hi_min) || (j0 < w_lo_max) || (p.key_mask != nullptr);
            if (need_mask) {
#pragma unroll
                for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                    for (int bb = 0; bb < 4; ++bb) {
                        const int kbase = 32 * kb + 8 * bb + 4 * lh;
                        f32x4 mv = {1.f, 1.f, 1.f, 1.f};
                        if (p.key_mask) mv = *reinterpret_cast<const f32x4*>(Ms + kbase);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = j0 + kbase + i;
                            const bool vis = key >= lo && key < hi && mv[i] != 0.f;
                            if (!vis) sacc[kb][4 * bb + i] = kNegInf;
                        }
                    }
            }
            // ── online softmax (base 2) ──
            float mloc = kNegInf;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mloc = fmaxf(mloc, sacc[kb][e]);
            mloc = exchange_max(mloc);
            const float m_new = fmaxf(m_run, mloc);
            const float mc = (m_new == kNegInf) ? 0.f : m_new * cl2;
            const float alpha = (m_run == kNegInf) ? 0.f : __builtin_amdgcn_exp2f(m_run * cl2 - mc);
            m_run = m_new;
            float lsum = 0.f;
#pragma unroll
            for (int kb = 0; kb < 2; ++kb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    const float pe = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][e], cl2, -mc));
                    sacc[kb][e] = pe;
                    lsum += pe;
                }
            l_run = l_run * alpha + lsum;
#pragma unroll
            for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
                for (int e = 0; e < 16; ++e) oacc[vb][e] *= alpha;
            // ── P^T as B operand: 16-key chunk c4 = acc[8*(c4%2) .. +7] of block c4/2 ──
            V8 pf[4];
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4)
#pragma unroll
                for (int t = 0; t < 8; ++t) pf[c4][t] = static_cast<T>(sacc[c4 >> 1][8 * (c4 & 1) + t]);
            // ── O^T += V^T P^T ──
            const int trow = (lane & 15) >> 2;                     // key row inside a 4-key group
            const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);  // head-dim column inside a 32 block
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
#pragma unroll
                for (int vb = 0; vb < G::VB; ++vb) {
                    const unsigned char* vptr = Vs + (16 * c4 + 4 * lh + trow) * G::V_STRIDE + (32 * vb + tcol) * 2;
                    const s16x4 v_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(vptr));
                    const s16x4 v_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(vptr + 8 * G::V_STRIDE));
                    const s16x8 a = __builtin_shufflevector(v_lo, v_hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    oacc[vb] = Mma<T>::run(__builtin_bit_cast(V8, a), pf[c4], oacc[vb]);
                }
            }
        }
        __syncthreads();
    }

    // ── epilogue: normalise, transpose through LDS, write full rows ──
    const float l_tot = exchange_sum(l_run);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    unsigned char* const Os = smem;
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
                *reinterpret_cast<t4*>(Os + (wave * 32 + lq) * G::O_STRIDE + d0 * 2) = ov;
            }
        }
    __syncthreads();
    for (int idx = tid; idx < kBM * G::CPR; idx += kThreads) {
        const int row = idx / G::CPR;
        const int cc = idx - row * G::CPR;
        if (q0 + row < p.Lq)
            *reinterpret_cast<u32x4*>(o_base + static_cast<long>(q0 + row) * p.o_rs + cc * 8) =
                *reinterpret_cast<const u32x4*>(Os + row * G::O_STRIDE + cc * 16);
    }
}

template <typename T, int D>
int launch_d(const SdpaDev& p, hipStream_t stream) {
    const bool rope_k = p.cos_k != nullptr;
    const dim3 grid(((p.n_blocks + 7) / 8) * 8), block(kThreads);
    const size_t lds = Geo<D>::LDS_BYTES;
    if (rope_k) {
        hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, true>), grid, block, lds, stream, p);
    } else {
        hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, false>), grid, block, lds, stream, p);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_fwd launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_t(const SdpaDev& p, int head_dim, hipStream_t stream) {
    switch (head_dim) {
        case 40: return launch_d<T, 40>(p, stream);
        case 64: return launch_d<T, 64>(p, stream);
        case 72: return launch_d<T, 72>(p, stream);
        case 80: return launch_d<T, 80>(p, stream);
        case 96: return launch_d<T, 96>(p, stream);
        case 112: return launch_d<T, 112>(p, stream);
        case 128: return launch_d<T, 128>(p, stream);
        case 160: return launch_d<T, 160>(p, stream);
        default: return fail("mi_sdpa_forward: head_dim %d has no kernel (40, 64, 72, 80, 96, 112, 128, 160)", head_dim);
    }
}

}  // namespace

bool sdpa_supported(int dtype, int head_dim) {
    if (dtype != MI_DTYPE_F16 && dtype != MI_DTYPE_BF16) return false;
    switch (head_dim) {
        case 40: case 64: case 72: case 80: case 96: case 112: case 128: case 160: return true;
        default: return false;
    }
}

int launch_sdpa(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream) {
    if (dtype == MI_DTYPE_BF16) return launch_t<__bf16>(p, head_dim, stream);
    if (dtype == MI_DTYPE_F16) return launch_t<_Float16>(p, head_dim, stream);
    return fail("mi_sdpa_forward: dtype %d not supported (fp16 = 1, bf16 = 2)", dtype);
}

}  // namespace mi
