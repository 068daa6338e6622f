// Flash-style softmax attention forward for gfx950 (MI355X), hand-written. Two kernels share the
// building blocks of sdpa_common.h:
//
//   sdpa_fwd_pp_kernel   8 wavefronts = 256 query rows per work group, 2 wavefronts per SIMD. The two
//                        wavefronts of a SIMD run half a tile apart: while one issues the MFMAs of
//                        O += V^T P (tile t) and S = K Q^T (tile t+1), the other does the softmax of
//                        its own tile on the VALU, so the matrix and vector pipes of the SIMD are busy
//                        at the same time. The phase shift is set up once by one extra barrier for the
//                        second group and kept by the two work-group barriers of every iteration.
//   sdpa_fwd_kernel      4 wavefronts = 128 query rows per work group, 2 work groups per CU; used when
//                        the problem has too few 256-row tiles to fill the chip.
//
// Key/value tiles of 64 rows are staged in LDS (double buffered, loaded one tile ahead through
// registers). Not in HBM: scores, probabilities, rotated Q/K (RoPE is applied as Q and K are loaded),
// the [prefix ; fresh] K/V concatenation (two source pointers), any mask tensor (per-row visible-key
// intervals; key tiles outside every row's interval are skipped).
#include "sdpa_common.h"

namespace mi {
namespace {

using namespace sdpa;

// Work-group id -> logical tile. Hardware deals consecutive work-group ids round-robin over the 8
// XCDs; undo that so each XCD (one L2) gets a contiguous run of logical tiles, i.e. query tiles that
// share the same K/V. Returns -1 for the padding groups of the last round.
__device__ __forceinline__ int logical_block(int n_blocks) {
    const int chunk = (n_blocks + 7) >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    return logical < n_blocks ? logical : -1;
}

// Cooperative K/V tile movement for a work group of NT threads: global -> registers -> LDS.
// kreg / vreg hold this thread's 16-byte chunks of one K tile and one V tile (possibly different tiles).
template <typename T, int D, int NT, bool ROPE_K>
struct TileMover {
    using G = HeadGeo<D>;
    static constexpr int NLD = (G::NCH + NT - 1) / NT;
    static constexpr bool EXACT = (G::NCH % NT) == 0;
    const SdpaDev& p;
    const T* k_base; const T* v_base; const T* kp_base; const T* vp_base;
    int tid, kv_stop;
    u32x4 kreg[NLD], vreg[NLD];

    // which: 0 = K tile into kreg, 1 = V tile into vreg
    template <int WHICH>
    __device__ __forceinline__ void issue(int j0) {
        u32x4 (&reg)[NLD] = WHICH == 0 ? kreg : vreg;
        const T* fresh = WHICH == 0 ? k_base : v_base;
        const T* pre = WHICH == 0 ? kp_base : vp_base;
        const long f_rs = WHICH == 0 ? p.k_rs : p.v_rs;
        const long p_rs = WHICH == 0 ? p.kp_rs : p.vp_rs;
        const bool in_prefix = j0 + kBN <= p.Lp;
        const bool in_fresh = j0 >= p.Lp;
        if ((in_prefix || in_fresh) && j0 + kBN <= kv_stop) {
            // whole tile from one buffer: uniform base pointer plus a fixed per-thread byte offset
            const unsigned char* base = in_fresh ? reinterpret_cast<const unsigned char*>(fresh + static_cast<long>(j0 - p.Lp) * f_rs)
                                                 : reinterpret_cast<const unsigned char*>(pre + static_cast<long>(j0) * p_rs);
            const unsigned rsb = static_cast<unsigned>(in_fresh ? f_rs : p_rs) * 2u;
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int idx = tid + NT * i;
                const int row = idx / G::CPR;
                const int cc = idx - row * G::CPR;
                if (EXACT || idx < G::NCH) reg[i] = *reinterpret_cast<const u32x4*>(base + (static_cast<unsigned>(row) * rsb + cc * 16u));
            }
        } else {
            // tile straddles the prefix / fresh boundary or the end of the visible keys
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int idx = tid + NT * i;
                const int row = idx / G::CPR;
                const int cc = idx - row * G::CPR;
                const int j = j0 + row;
                reg[i] = u32x4{0, 0, 0, 0};
                if ((EXACT || idx < G::NCH) && j < kv_stop) {
                    const T* r = j < p.Lp ? pre + static_cast<long>(j) * p_rs : fresh + static_cast<long>(j - p.Lp) * f_rs;
                    reg[i] = *reinterpret_cast<const u32x4*>(r + cc * 8);
                }
            }
        }
    }
    __device__ __forceinline__ void store_k(int j0, unsigned char* Ks) {
        // The rotation tables are fetched here rather than with the tile: they are L2 hits shared by
        // every head, and holding them across the MFMA section would cost 8 registers per chunk
        // exactly where pressure peaks. Prefix rows are stored already rotated.
        f32x4 creg[ROPE_K ? NLD : 1], sreg[ROPE_K ? NLD : 1];
        if constexpr (ROPE_K) {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int idx = tid + NT * i;
                const int row = idx / G::CPR;
                const int cc = idx - row * G::CPR;
                const int j = j0 + row;
                creg[i] = f32x4{1.f, 1.f, 1.f, 1.f};
                sreg[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                if ((EXACT || idx < G::NCH) && j < kv_stop && j >= p.Lp) {
                    const long jr = j - p.Lp;
                    creg[i] = *reinterpret_cast<const f32x4*>(p.cos_k + jr * (D / 2) + cc * 4);
                    sreg[i] = *reinterpret_cast<const f32x4*>(p.sin_k + jr * (D / 2) + cc * 4);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (EXACT || idx < G::NCH) {
                u32x4 kk = kreg[i];
                if constexpr (ROPE_K) kk = rope_chunk<T>(kk, creg[i], sreg[i]);
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = kk;
            }
        }
    }
    __device__ __forceinline__ void store_v(unsigned char* Vs) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (EXACT || idx < G::NCH) *reinterpret_cast<u32x4*>(Vs + row * G::V_STRIDE + cc * 16) = vreg[i];
        }
    }
};

// Zero the LDS pad columns of `stages` K and V buffers once (tile stores never touch them).
template <int D, int NT>
__device__ __forceinline__ void zero_pads(unsigned char* kbuf0, unsigned char* vbuf0, int k_stage_bytes, int v_stage_bytes, int stages, int tid) {
    using G = HeadGeo<D>;
    for (int st = 0; st < stages; ++st) {
        if constexpr (G::DK > D) {
            for (int r = tid; r < kBN; r += NT)
                *reinterpret_cast<u32x4*>(kbuf0 + st * k_stage_bytes + r * G::K_STRIDE + D * 2) = u32x4{0, 0, 0, 0};
        }
        if constexpr (G::DV > D) {
            constexpr int PC = (G::DV - D) / 8;
            for (int i = tid; i < kBN * PC; i += NT)
                *reinterpret_cast<u32x4*>(vbuf0 + st * v_stage_bytes + (i / PC) * G::V_STRIDE + D * 2 + (i % PC) * 16) = u32x4{0, 0, 0, 0};
        }
    }
}

// Coalesced write-out of BM staged rows.
template <typename T, int D, int NT>
__device__ __forceinline__ void write_output(const unsigned char* Os, T* o_base, long o_rs, int q0, int Lq, int BM, int tid) {
    using G = HeadGeo<D>;
    for (int idx = tid; idx < BM * G::CPR; idx += NT) {
        const int row = idx / G::CPR;
        const int cc = idx - row * G::CPR;
        if (q0 + row < Lq)
            *reinterpret_cast<u32x4*>(o_base + static_cast<long>(q0 + row) * o_rs + cc * 8) =
                *reinterpret_cast<const u32x4*>(Os + row * G::O_STRIDE + cc * 16);
    }
}

// ───────────────────────────── 4-wavefront kernel ─────────────────────────────
constexpr int kThreads4 = 256;
template <int D> constexpr int lds_bytes_4() {
    using G = HeadGeo<D>;
    const int kv = 2 * (G::K_BYTES + G::V_BYTES);
    const int o = 128 * G::O_STRIDE;
    return kv > o ? kv : o;
}

template <typename T, int D, bool ROPE_K>
__global__ void __launch_bounds__(kThreads4, (D > 128 ? 1 : 2)) sdpa_fwd_kernel(const SdpaDev p) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int BM = 128;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int red[8];
    constexpr int STAGE = G::K_BYTES + G::V_BYTES;

    const int logical = logical_block(p.n_blocks);
    if (logical < 0) return;
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
    const int q0 = qt * BM;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < p.Lq;
    const int hk = h / p.kv_group;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const float* const key_mask = p.key_mask ? p.key_mask + b * p.key_mask_bs : nullptr;

    int lo, hi;
    row_interval(p, b, qrow, qvalid, lo, hi);
    const WaveExtent we = wave_extent(lo, hi);
    if (lane == 0) { red[wave] = we.lo_min; red[4 + wave] = we.hi_max; }
    zero_pads<D, kThreads4>(smem, smem + G::K_BYTES, STAGE, STAGE, 2, tid);
    __syncthreads();
    const int g_lo = min(min(red[0], red[1]), min(red[2], red[3]));
    const int kv_stop = max(max(red[4], red[5]), max(red[6], red[7]));
    const int kv_start = g_lo == 0x7fffffff ? 0 : (g_lo / kBN) * kBN;

    V8 qf[G::KC];
    load_q_frags<T, D>(qf, p, q_base, qrow, qvalid, lh);

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    SoftmaxState st;
    const float cl2 = p.scale_log2;
    const float lazy_raw = kLazyLog2 / cl2;

    TileMover<T, D, kThreads4, ROPE_K> mv{p,
                                          static_cast<const T*>(p.k) + b * p.k_bs + hk * D,
                                          static_cast<const T*>(p.v) + b * p.v_bs + hk * D,
                                          p.kp ? static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D : nullptr,
                                          p.vp ? static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D : nullptr,
                                          tid, kv_stop, {}, {}};

    // key loop, LDS double buffered: one barrier per tile
    if (kv_start < kv_stop) {
        mv.template issue<0>(kv_start);
        mv.template issue<1>(kv_start);
        mv.store_k(kv_start, smem);
        mv.store_v(smem + G::K_BYTES);
        if (kv_start + kBN < kv_stop) { mv.template issue<0>(kv_start + kBN); mv.template issue<1>(kv_start + kBN); }
    }
    __syncthreads();
    int stage = 0;
    for (int j0 = kv_start; j0 < kv_stop; j0 += kBN) {
        const unsigned char* Ks = smem + stage * STAGE;
        const unsigned char* Vs = Ks + G::K_BYTES;
        // wavefronts none of whose rows can see this tile only help with the loads
        if (j0 < we.hi_max && j0 + kBN > we.lo_min) {
            f32x16 sacc[2];
            V8 pf[4];
            qk_tile<T, D>(Ks, qf, lq, lh, sacc);
            const bool interior = (j0 >= we.lo_max) && (j0 + kBN <= we.hi_min) && (key_mask == nullptr);
            if (interior) softmax_tile<T, D, false>(sacc, pf, oacc, st, cl2, lazy_raw, j0, lo, hi, lh, key_mask, p.Lk);
            else softmax_tile<T, D, true>(sacc, pf, oacc, st, cl2, lazy_raw, j0, lo, hi, lh, key_mask, p.Lk);
            pv_tile<T, D>(Vs, pf, lane, oacc);
        }
        if (j0 + kBN < kv_stop) {
            unsigned char* Kn = smem + (stage ^ 1) * STAGE;
            mv.store_k(j0 + kBN, Kn);
            mv.store_v(Kn + G::K_BYTES);
        }
        if (j0 + 2 * kBN < kv_stop) { mv.template issue<0>(j0 + 2 * kBN); mv.template issue<1>(j0 + 2 * kBN); }
        __syncthreads();
        stage ^= 1;
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    stage_output<T, D>(smem, wave * 32 + lq, lh, oacc, inv);
    __syncthreads();
    write_output<T, D, kThreads4>(smem, o_base, p.o_rs, q0, p.Lq, BM, tid);
}

// ───────────────────────── 8-wavefront ping-pong kernel ─────────────────────────
constexpr int kThreads8 = 512;
template <int D> constexpr int lds_bytes_8() {
    using G = HeadGeo<D>;
    const int kv = 2 * (G::K_BYTES + G::V_BYTES);
    const int o = 256 * G::O_STRIDE;
    return kv > o ? kv : o;
}

// Time is counted in slots separated by work-group barriers. Group 0 (wavefronts 0-3) runs its MFMA
// phase in even slots and its VALU phase in odd slots; group 1 (wavefronts 4-7, sharing the SIMDs of
// 0-3) the other way round. With t = slot / 2:
//   MFMA phase:  O += V_t^T P_t ;  S_{t+1} = K_{t+1} Q^T           (reads LDS tiles K_{t+1}, V_t)
//   VALU phase:  P = softmax(S) of the tile just scored; store this thread's share of tiles
//                K_{t+2}, V_{t+1} into the LDS buffers of K_t, V_{t-1}; issue the next global loads
// Tiles K_{t+1}, V_t are complete in LDS before slot 2t and last read in slot 2t+1, and the buffers
// they replace were last read in slot 2t-1, so two buffers per operand suffice.
template <typename T, int D, bool ROPE_K>
__global__ void __launch_bounds__(kThreads8, 2) sdpa_fwd_pp_kernel(const SdpaDev p) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int BM = 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int red[16];
    unsigned char* const Kbuf = smem;                    // 2 x K tile
    unsigned char* const Vbuf = smem + 2 * G::K_BYTES;   // 2 x V tile

    const int logical = logical_block(p.n_blocks);
    if (logical < 0) return;
    int qt = logical % p.n_q_tiles;
    const int bh = logical / p.n_q_tiles;
    const int h = bh % p.H;
    const int b = bh / p.H;
    if (p.mask_mode != MI_MASK_NONE) qt = p.n_q_tiles - 1 - qt;  // longest key ranges first

    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int grp = wave >> 2;      // phase group
    const int lane = tid & 63;
    const int lq = lane & 31;
    const int lh = lane >> 5;
    const int q0 = qt * BM;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < p.Lq;
    const int hk = h / p.kv_group;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const float* const key_mask = p.key_mask ? p.key_mask + b * p.key_mask_bs : nullptr;

    int lo, hi;
    row_interval(p, b, qrow, qvalid, lo, hi);
    const WaveExtent we = wave_extent(lo, hi);
    if (lane == 0) { red[wave] = we.lo_min; red[8 + wave] = we.hi_max; }
    zero_pads<D, kThreads8>(Kbuf, Vbuf, G::K_BYTES, G::V_BYTES, 2, tid);
    __syncthreads();
    int g_lo = red[0], kv_stop = red[8];
#pragma unroll
    for (int w = 1; w < 8; ++w) { g_lo = min(g_lo, red[w]); kv_stop = max(kv_stop, red[8 + w]); }
    const int kv_start = g_lo == 0x7fffffff ? 0 : (g_lo / kBN) * kBN;
    const int n_tiles = kv_stop > kv_start ? (kv_stop - kv_start + kBN - 1) / kBN : 0;

    V8 qf[G::KC];
    load_q_frags<T, D>(qf, p, q_base, qrow, qvalid, lh);

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    SoftmaxState st;
    const float cl2 = p.scale_log2;
    const float lazy_raw = kLazyLog2 / cl2;

    TileMover<T, D, kThreads8, ROPE_K> mv{p,
                                          static_cast<const T*>(p.k) + b * p.k_bs + hk * D,
                                          static_cast<const T*>(p.v) + b * p.v_bs + hk * D,
                                          p.kp ? static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D : nullptr,
                                          p.vp ? static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D : nullptr,
                                          tid, kv_stop, {}, {}};
    auto tile_j0 = [&](int t) { return kv_start + t * kBN; };
    auto tile_active = [&](int t) { return t < n_tiles && tile_j0(t) < we.hi_max && tile_j0(t) + kBN > we.lo_min; };
    // this thread's share of tiles K_kt, V_vt: registers -> LDS, then prefetch K_{kt+1}, V_{vt+1}
    auto advance_tiles = [&](int kt, int vt) {
        if (kt < n_tiles) mv.store_k(tile_j0(kt), Kbuf + (kt & 1) * G::K_BYTES);
        if (vt < n_tiles) mv.store_v(Vbuf + (vt & 1) * G::V_BYTES);
        if (kt + 1 < n_tiles) mv.template issue<0>(tile_j0(kt + 1));
        if (vt + 1 < n_tiles) mv.template issue<1>(tile_j0(vt + 1));
    };
    f32x16 sacc[2];
    V8 pf[4];
    auto softmax_of = [&](int t) {
        const int j0 = tile_j0(t);
        const bool interior = (j0 >= we.lo_max) && (j0 + kBN <= we.hi_min) && (key_mask == nullptr);
        if (interior) softmax_tile<T, D, false>(sacc, pf, oacc, st, cl2, lazy_raw, j0, lo, hi, lh, key_mask, p.Lk);
        else softmax_tile<T, D, true>(sacc, pf, oacc, st, cl2, lazy_raw, j0, lo, hi, lh, key_mask, p.Lk);
    };

    if (n_tiles > 0) {
        // ── prologue, both groups in step: K_0 to LDS, score and exponentiate tile 0 ──
        mv.template issue<0>(tile_j0(0));
        mv.store_k(tile_j0(0), Kbuf);
        if (n_tiles > 1) mv.template issue<0>(tile_j0(1));
        mv.template issue<1>(tile_j0(0));
        __syncthreads();
        if (tile_active(0)) {
            qk_tile<T, D>(Kbuf, qf, lq, lh, sacc);
            softmax_of(0);
        }
        advance_tiles(1, 0);   // K_1, V_0 to LDS; registers now hold K_2, V_1
        __syncthreads();
        // ── group 1 falls one slot behind: its first slot only moves tiles ──
        if (grp == 1) {
            advance_tiles(2, 1);
            __syncthreads();
        }
        for (int t = 0; t < n_tiles; ++t) {
            // MFMA phase
            __builtin_amdgcn_s_setprio(2);
            if (tile_active(t)) pv_tile<T, D>(Vbuf + (t & 1) * G::V_BYTES, pf, lane, oacc);
            if (tile_active(t + 1)) qk_tile<T, D>(Kbuf + ((t + 1) & 1) * G::K_BYTES, qf, lq, lh, sacc);
            __builtin_amdgcn_s_setprio(0);
            __syncthreads();
            // VALU phase
            if (tile_active(t + 1)) softmax_of(t + 1);
            advance_tiles(t + 2 + grp, t + 1 + grp);
            __syncthreads();
        }
        if (grp == 0) __syncthreads();
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    stage_output<T, D>(smem, wave * 32 + lq, lh, oacc, inv);
    __syncthreads();
    write_output<T, D, kThreads8>(smem, o_base, p.o_rs, q0, p.Lq, BM, tid);
}

template <typename T, int D>
int launch_d(SdpaDev p, int n_cu, hipStream_t stream) {
    const bool rope_k = p.cos_k != nullptr;
    // 256-row tiles when they give every CU at least one work group; head_dim above 128 does not fit
    // two wavefronts per SIMD and stays on the 128-row kernel.
    const long tiles256 = static_cast<long>(p.B) * p.H * ((p.Lq + 255) / 256);
    const int choice = sdpa_kernel_choice();
    const bool pingpong = D <= 128 && (choice == 2 || (choice == 0 && tiles256 >= n_cu));
    if (pingpong) {
        p.n_q_tiles = (p.Lq + 255) / 256;
        p.n_blocks = static_cast<int>(tiles256);
        const dim3 grid(((p.n_blocks + 7) / 8) * 8), block(kThreads8);
        if constexpr (D <= 128) {
            if (rope_k) hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, true>), grid, block, lds_bytes_8<D>(), stream, p);
            else hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, false>), grid, block, lds_bytes_8<D>(), stream, p);
        }
    } else {
        p.n_q_tiles = (p.Lq + 127) / 128;
        p.n_blocks = p.B * p.H * p.n_q_tiles;
        const dim3 grid(((p.n_blocks + 7) / 8) * 8), block(kThreads4);
        if (rope_k) hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, true>), grid, block, lds_bytes_4<D>(), stream, p);
        else hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, false>), grid, block, lds_bytes_4<D>(), stream, p);
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_fwd launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_t(const SdpaDev& p, int head_dim, int n_cu, hipStream_t stream) {
    switch (head_dim) {
        case 40: return launch_d<T, 40>(p, n_cu, stream);
        case 64: return launch_d<T, 64>(p, n_cu, stream);
        case 72: return launch_d<T, 72>(p, n_cu, stream);
        case 80: return launch_d<T, 80>(p, n_cu, stream);
        case 96: return launch_d<T, 96>(p, n_cu, stream);
        case 112: return launch_d<T, 112>(p, n_cu, stream);
        case 128: return launch_d<T, 128>(p, n_cu, stream);
        case 160: return launch_d<T, 160>(p, n_cu, stream);
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
    const int n_cu = device_cu_count();
    if (dtype == MI_DTYPE_BF16) return launch_t<__bf16>(p, head_dim, n_cu, stream);
    if (dtype == MI_DTYPE_F16) return launch_t<_Float16>(p, head_dim, n_cu, stream);
    return fail("mi_sdpa_forward: dtype %d not supported (fp16 = 1, bf16 = 2)", dtype);
}

}  // namespace mi
