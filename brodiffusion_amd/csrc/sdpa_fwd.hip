// Flash-style softmax attention forward for gfx950 (MI355X), hand-written. Four kernels share the building blocks of
// sdpa_common.h; launch_d picks one per call:
//
//   sdpa_fwd_kernel         4 wavefronts = 128 query rows per work group, K/V tiles through registers into padded LDS,
//                           double buffered. Small problems, head_dim 160, calls with a key mask, a logit bias, a
//                           request for the softmax denominators, or packed variable-length sequences.
//   sdpa_fwd_pp_kernel      8 wavefronts = 256 query rows, 2 wavefronts per SIMD, one work-group barrier per key tile:
//                           between two barriers every wavefront runs the MFMA stream (O += V^T P of tile t, then
//                           S = K Q^T of tile t+1) and one softmax, in opposite order in the two groups of four, so the
//                           matrix pipe and the VALU of a SIMD are busy at the same time.
//   sdpa_fwd_pp_dma_kernel  the same schedule with K/V tiles moved global -> LDS by DMA (head_dim 72 and 128), optionally
//                           with the last, partly filled round of work groups cut along the key axis (SPLIT) and merged
//                           by sdpa_combine_kernel.
//   sdpa_shortkv_kernel     short key sequences (cross attention): K and V of a head stay in LDS, a work group walks
//                           several query tiles, no barrier in the key loop.
//
// Not in HBM: scores, probabilities, rotated Q (RoPE is applied as Q is loaded; K either the same way or by one pass into
// a caller scratch), the [prefix ; fresh] K/V concatenation (two source pointers), any mask tensor (per-row visible-key
// intervals; key tiles outside every row's interval are skipped).
#include <type_traits>

#include "sdpa_tiles.h"

namespace mi {
namespace {

using namespace sdpa;


// ───────────────────────────── 4-wavefront kernel ─────────────────────────────
constexpr int kThreads4 = 256;
template <int D> constexpr int lds_bytes_4() {
    using G = HeadGeo<D>;
    const int kv = 2 * (G::K_BYTES + G::V_BYTES + kBN * 4);
    const int o = 128 * G::O_STRIDE;
    return kv > o ? kv : o;
}

// VARLEN: the batch items are sequences of different lengths packed back to back along the row axis
// (cu_q / cu_k: device arrays of batch + 1 row offsets, the cu_seqlens convention); Lq and Lk of the launch are the
// longest sequence and only size the grid. Each work group rebuilds the launch view for its own sequence.
// PSCALE: the rows of the cached prefix carry factors (the prefix-KV dial); a separate instance so that the code for it
// costs the other instances no registers.
template <typename T, int D, bool ROPE_K, bool VARLEN = false, bool PSCALE = false>
__global__ void __launch_bounds__(kThreads4, (D > 128 ? 1 : 2)) sdpa_fwd_kernel(const SdpaDev p_in) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int BM = 128;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int red[8];
    constexpr int STAGE = G::K_BYTES + G::V_BYTES + kBN * 4;   // K tile, V tile, 64 key-mask floats

    int qt, bh;
    if (!block_to_tile(p_in, qt, bh)) return;
    const int h = bh % p_in.H;
    const SdpaDev& p = p_in;
    // this work group's sequence: row offsets into the packed tensors, its own lengths and causal offset
    int b = bh / p.H, Lq = p.Lq, Lk = p.Lk, q_offset = p.q_offset;
    long q_row0 = 0, k_row0 = 0;
    if constexpr (VARLEN) {
        const int qs = p.cu_q[b], ks = p.cu_k[b];
        Lq = p.cu_q[b + 1] - qs;
        Lk = p.cu_k[b + 1] - ks;
        if (qt * BM >= Lq) return;
        q_row0 = qs; k_row0 = ks;
        q_offset = Lk - Lq;   // causal: the last query meets the last key, per sequence
        b = 0;                // batch strides do not apply to packed rows
    }

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in a scalar register
    const int lane = tid & 63;
    const int lq = lane & 31;
    const int lh = lane >> 5;
    const int q0 = qt * BM;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < Lq;
    const int hk = h / p.kv_group;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + q_row0 * p.q_rs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + q_row0 * p.o_rs + h * D;
    const float* const key_mask = p.key_mask ? p.key_mask + b * p.key_mask_bs : nullptr;
    const float* const bias_row = (p.bias && qvalid && qrow >= p.bias_q0) ? p.bias + static_cast<long>(qrow - p.bias_q0) * p.bias_rs : nullptr;

    int lo, hi;
    if constexpr (VARLEN) {
        lo = 0;
        hi = p.mask_mode == MI_MASK_CAUSAL ? min(Lk, q_offset + qrow + 1) : Lk;
        if (!qvalid || hi <= lo) { lo = 0; hi = 0; }
    } else {
        row_interval(p, b, qrow, qvalid, lo, hi);
    }
    const WaveExtent we = wave_extent(lo, hi);
    if (lane == 0) { red[wave] = we.lo_min; red[4 + wave] = we.hi_max; }
    V8 qf[G::KC];
    stage_q_tile<T, D, kThreads4, BM>(smem, p, q_base, q0, tid, 1.f, Lq - 1);
    __syncthreads();
    read_q_frags<T, D>(qf, smem, wave * 32 + lq, lh);
    __syncthreads();
    zero_pads<D, kThreads4>(smem, smem + G::K_BYTES, STAGE, STAGE, 2, tid);
    __syncthreads();
    const int g_lo = __builtin_amdgcn_readfirstlane(min(min(red[0], red[1]), min(red[2], red[3])));
    const int kv_stop = __builtin_amdgcn_readfirstlane(max(max(red[4], red[5]), max(red[6], red[7])));
    const TilePlan plan(g_lo == 0x7fffffff ? 0 : g_lo, kv_stop, p.Lp);

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    SoftmaxState st;
    const float cl2 = p.scale_log2;
    const float lazy_raw = kLazyLog2 / cl2;

    TileMover<T, D, kThreads4, ROPE_K> mv{p, plan,
                                          reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.k) + b * p.k_bs + k_row0 * p.k_rs + hk * D),
                                          reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.v) + b * p.v_bs + k_row0 * p.v_rs + hk * D),
                                          reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D),
                                          reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D),
                                          tid, {}, {}, 1.f};

    // key loop, LDS double buffered: one barrier per tile
    const int n_tiles = plan.n_tiles;
    if (n_tiles > 0) {
        mv.template issue<0>(0);
        mv.template issue<1>(0);
        if (key_mask) mv.issue_mask(0, key_mask);
        mv.store_k(0, smem);
        mv.store_v(0, smem + G::K_BYTES);
        if (key_mask) mv.store_mask(reinterpret_cast<float*>(smem + G::K_BYTES + G::V_BYTES));
        if (n_tiles > 1) {
            mv.template issue<0>(1);
            mv.template issue<1>(1);
            if (key_mask) mv.issue_mask(1, key_mask);
        }
    }
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
        const unsigned char* Ks = smem + (t & 1) * STAGE;
        const unsigned char* Vs = Ks + G::K_BYTES;
        const float* Ms = key_mask ? reinterpret_cast<const float*>(Vs + G::V_BYTES) : nullptr;
        const int j0 = plan.j0(t);
        const int lim = plan.limit(t);
        // wavefronts none of whose rows can see this tile only help with the loads
        if (j0 < we.hi_max && j0 + kBN > we.lo_min) {
            f32x16 sacc[2];
            V8 pf[4];
            mfma_stream<T, D, false, true>(Vs, Ks, pf, qf, oacc, sacc, lane);
            const bool biased = p.bias != nullptr && j0 < p.bias_cols;
            const bool interior = (j0 >= we.lo_max) && (j0 + kBN <= min(we.hi_min, lim)) && (key_mask == nullptr) && !biased;
            softmax_tile<T, D, PSCALE>(sacc, pf, oacc, st, cl2, lazy_raw, !interior, j0, lo, min(hi, lim), lh, Ms,
                                       biased ? bias_row : nullptr, p.bias_cols, p.inv_scale,
                                       PSCALE ? prefix_scale_of(p, plan.in_prefix(t)) : PrefixScale());
            mfma_stream<T, D, true, false>(Vs, Ks, pf, qf, oacc, sacc, lane);
        }
        if (t + 1 < n_tiles) {
            unsigned char* Kn = smem + ((t + 1) & 1) * STAGE;
            mv.store_k(t + 1, Kn);
            mv.store_v(t + 1, Kn + G::K_BYTES);
            if (key_mask) mv.store_mask(reinterpret_cast<float*>(Kn + G::K_BYTES + G::V_BYTES));
        }
        if (t + 2 < n_tiles) {
            mv.template issue<0>(t + 2);
            mv.template issue<1>(t + 2);
            if (key_mask) mv.issue_mask(t + 2, key_mask);
        }
        __syncthreads();
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = row_inverse(l_tot);
    // base-2 log of the row's denominator in exponent units: p(key) = exp2(score * scale_log2 [+ bias * log2 e] - lse);
    // +inf for a row without visible keys, so that every p is 0
    if (p.lse && qvalid && lh == 0)
        p.lse[(static_cast<long>(b) * p.H + h) * Lq + qrow] = l_tot > 0.f ? st.mc + __builtin_amdgcn_logf(l_tot) : __builtin_huge_valf();
    stage_output<T, D>(smem, wave * 32 + lq, lh, oacc, inv);
    __syncthreads();
    write_output<T, D, kThreads4>(smem, o_base, p.o_rs, q0, Lq, BM, tid);
}

// ───────────────────────── short key sequences (cross attention) ─────────────────────────
// When all keys of a (batch, head) fit in LDS (cross attention to a text prompt: 77 to ~300 keys) the call moves far more
// bytes than it multiplies (Q in, O out: ~120 FLOP per byte at 77-105 keys of head_dim 72, below the ridge of ~312), so
// it is bound by HBM and by fixed costs, and the kernels above, whose work groups all stage, wait and drain at the same
// moments, are all prologue and epilogue. Here a work group of 8 wavefronts loads the K and V of its (batch, head) ONCE
// (only the tiles below the batch item's valid length, all loads in flight together), meets at one barrier, and from
// then on every wavefront is on its own: it walks 32-row query units, staging each through a private LDS slice (the
// unit's rows are fetched with full-row coalescing one unit ahead, the output leaves the same way), so no barrier stands
// in the key loop or between units and the eight wavefronts drift apart: while some wait for their rows, others
// multiply, and the memory pipe sees a steady stream instead of bursts. Unmasked calls (kv_valid_len and a 0/1 key mask
// allowed), no RoPE, no prefix. Same tile arithmetic as the 128-row kernel: bit-identical results.
constexpr int kShortMaxTiles = 5;   // 320 keys
template <int D> constexpr int shortkv_lds_bytes(int n_kt, bool with_mask) {
    using G = HeadGeo<D>;
    return 256 * G::O_STRIDE + n_kt * (G::K_BYTES + G::V_BYTES + (with_mask ? kBN * 4 : 0));
}
// most key tiles that fit in LDS next to the staging slices at head dimension D (the prologue holds that many in registers)
template <int D> constexpr int shortkv_max_tiles() {
    int n = kShortMaxTiles;
    while (n > 1 && shortkv_lds_bytes<D>(n, false) > 160 * 1024) --n;
    return n;
}

template <typename T, int D>
__global__ void __launch_bounds__(kThreads8, 2) sdpa_shortkv_kernel(const SdpaDev p, int n_kt, int units_per_group, int groups_per_head) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int UM = 32;                         // query rows of a unit (one wavefront)
    constexpr int SLICE = UM * G::O_STRIDE;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];

    const int logical = logical_block(p.n_blocks);
    if (logical < 0) return;
    const int bh = logical / groups_per_head;
    const int grp = logical - bh * groups_per_head;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.kv_group;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
    unsigned char* const Qs = smem + wave * SLICE;            // this wavefront's staging slice
    unsigned char* const Kall = smem + 8 * SLICE;
    unsigned char* const Vall = Kall + n_kt * G::K_BYTES;
    float* const Mall = reinterpret_cast<float*>(Vall + n_kt * G::V_BYTES);
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;

    // keys of this batch item (uniform): only the tiles that hold one are loaded and multiplied
    int kv_len = p.Lk;
    if (p.kv_valid_len) kv_len = min(kv_len, max(p.kv_valid_len[b], 0));
    kv_len = __builtin_amdgcn_readfirstlane(kv_len);
    const int n_kt_b = (kv_len + kBN - 1) / kBN;

    // ── a unit's Q rows: fetched with full-row coalescing into registers, stored to the slice when the unit's turn comes ──
    constexpr int CPRK = G::DK / 8;
    constexpr int NQ = UM * CPRK / 64;
    static_assert(UM * CPRK % 64 == 0, "a unit's chunks divide among the lanes");
    u32x4 qraw[NQ];
    auto q_issue = [&](int q0) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / CPRK, cc = min(idx - row * CPRK, G::CPR - 1);
            qraw[i] = *reinterpret_cast<const u32x4*>(q_base + static_cast<long>(min(q0 + row, p.Lq - 1)) * p.q_rs + cc * 8);
        }
    };
    auto q_store = [&](int q0) {
#pragma unroll
        for (int i = 0; i < NQ; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / CPRK, cc = idx - row * CPRK;
            u32x4 v = qraw[i];
            if (q0 + row >= p.Lq || cc >= G::CPR) v = u32x4{0, 0, 0, 0};
            *reinterpret_cast<u32x4*>(Qs + row * G::O_STRIDE + cc * 16) = v;
        }
    };
    // LDS traffic of one wavefront is executed in order; the fences keep the compiler from reordering around them
    auto wave_sync = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    const int n_units = (p.Lq + UM - 1) / UM;
    const int u_end = min((grp + 1) * units_per_group, n_units);
    int u = grp * units_per_group + wave;
    if (u < u_end) q_issue(u * UM);

    // ── the K and V tiles of this (batch, head) and the key-mask values: every load is issued before the first is stored ──
    {
        constexpr int NLD = (G::NCH + kThreads8 - 1) / kThreads8;
        const unsigned char* const k_base = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.k) + b * p.k_bs + hk * D);
        const unsigned char* const v_base = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.v) + b * p.v_bs + hk * D);
        const unsigned k_rsb = static_cast<unsigned>(p.k_rs) * 2u, v_rsb = static_cast<unsigned>(p.v_rs) * 2u;
        constexpr int MAXT = shortkv_max_tiles<D>();
        u32x4 kreg[MAXT][NLD], vreg[MAXT][NLD];
        float mval = 0.f;
        if (p.key_mask && tid < n_kt_b * kBN && tid < kv_len) mval = p.key_mask[b * p.key_mask_bs + tid];
#pragma unroll
        for (int t = 0; t < MAXT; ++t) {
            if (t < n_kt_b) {
                const int last = min(kv_len - t * kBN, kBN) - 1;   // rows past the last key repeat it and are stored as zeros
#pragma unroll
                for (int i = 0; i < NLD; ++i) {
                    const int idx = min(tid + kThreads8 * i, G::NCH - 1);
                    const unsigned row = static_cast<unsigned>(t * kBN + min(idx / G::CPR, last));
                    const unsigned cc = static_cast<unsigned>(idx % G::CPR);
                    kreg[t][i] = *reinterpret_cast<const u32x4*>(k_base + (static_cast<unsigned long>(row) * k_rsb + cc * 16u));
                    vreg[t][i] = *reinterpret_cast<const u32x4*>(v_base + (static_cast<unsigned long>(row) * v_rsb + cc * 16u));
                }
            }
        }
        zero_pads<D, kThreads8>(Kall, Vall, G::K_BYTES, G::V_BYTES, n_kt_b, tid);
        if (p.key_mask && tid < n_kt * kBN) Mall[tid] = mval;
#pragma unroll
        for (int t = 0; t < MAXT; ++t) {
            if (t < n_kt_b) {
                const int nvalid = kv_len - t * kBN;
#pragma unroll
                for (int i = 0; i < NLD; ++i) {
                    const int idx = tid + kThreads8 * i;
                    const int row = idx / G::CPR, cc = idx - row * G::CPR;
                    if (idx < G::NCH) {
                        const bool live = row < nvalid;
                        *reinterpret_cast<u32x4*>(Kall + t * G::K_BYTES + row * G::K_STRIDE + cc * 16) = live ? kreg[t][i] : u32x4{0, 0, 0, 0};
                        *reinterpret_cast<u32x4*>(Vall + t * G::V_BYTES + row * G::V_STRIDE + cc * 16) = live ? vreg[t][i] : u32x4{0, 0, 0, 0};
                    }
                }
            }
        }
    }
    __syncthreads();   // K, V and the mask values are in place: the only barrier of the kernel

    const float cl2 = p.scale_log2;
    const float lazy_raw = kLazyLog2 / cl2;
    for (; u < u_end; u += 8) {
        const int q0 = u * UM;
        q_store(q0);
        wave_sync();
        V8 qf[G::KC];
        read_q_frags<T, D>(qf, Qs, lq, lh);
        wave_sync();       // the slice is free again (it takes the output next)
        // The next unit's rows, unconditionally (past its last unit a wavefront fetches the current one again, from cache):
        // vector-memory loads and stores complete in one order here, so the wait in front of the next q_store can pass over
        // this unit's output stores only if the compiler can count them, i.e. if neither the loads nor the stores sit
        // under a condition. With a conditional load the next unit waited for this unit's stores to land.
        q_issue(u + 8 < u_end ? q0 + 8 * UM : q0);

        f32x16 oacc[G::VB];
#pragma unroll
        for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
        SoftmaxState st;
        for (int t = 0; t < n_kt_b; ++t) {
            const int j0 = t * kBN;
            const unsigned char* Ks = Kall + t * G::K_BYTES;
            const unsigned char* Vs = Vall + t * G::V_BYTES;
            f32x16 sacc[2];
            V8 pf[4];
            mfma_stream<T, D, false, true>(Vs, Ks, pf, qf, oacc, sacc, lane);
            const bool interior = j0 + kBN <= kv_len && p.key_mask == nullptr;
            softmax_tile<T, D>(sacc, pf, oacc, st, cl2, lazy_raw, !interior, j0, 0, kv_len, lh, p.key_mask ? Mall + j0 : nullptr);
            mfma_stream<T, D, true, false>(Vs, Ks, pf, qf, oacc, sacc, lane);
        }
        const float l_tot = exchange_sum(st.l);
        const float inv = row_inverse(l_tot);
        stage_output<T, D>(Qs, lq, lh, oacc, inv);
        wave_sync();
        // (a fixed number of unconditional stores, see above: a lane without a chunk of its own, or whose row lies past the
        //  end of Q, stores a chunk that another lane stores too, same bytes to the same address)
        const int last_row = min(UM, p.Lq - q0) - 1;
#pragma unroll
        for (int i = 0; i < (UM * G::CPR + 63) / 64; ++i) {
            const int idx = min(lane + 64 * i, UM * G::CPR - 1);
            const int row = min(idx / G::CPR, last_row), cc = idx % G::CPR;
            *reinterpret_cast<u32x4*>(o_base + static_cast<long>(q0 + row) * p.o_rs + cc * 8) =
                *reinterpret_cast<const u32x4*>(Qs + row * G::O_STRIDE + cc * 16);
        }
        wave_sync();       // the staged rows are read before the next unit's Q overwrites them
    }
}

// ───────────────────────── 8-wavefront ping-pong kernel ─────────────────────────

// Eight wavefronts, 32 query rows each; wavefronts w and w + 4 share a SIMD. One work-group barrier per
// key tile. Between two barriers (step t; step -1 has no P yet and only scores tile 0) every wavefront runs
//   the MFMA stream:  O += V_t^T P_t ;  S_{t+1} = K_{t+1} Q^T   (reads LDS tiles V_t, K_{t+1}), and
//   one softmax:      P = softmax(S) of the scores it holds,
// in opposite order in the two groups: group 0 (wavefronts 0-3) streams first and then turns S_{t+1} into
// P_{t+1}; group 1 first turns S_t (scored in the previous step) into P_t and then streams. So on every SIMD
// one wavefront feeds the matrix pipe while the other is in its VALU part, and neither waits for the other
// before the end of the step: a barrier between the two halves (strict ping-pong) makes each stream run
// alone with its LDS and dependency latencies exposed and was measured ~1.6x slower.
// In the shadow of the stream the wavefront stores its share of tiles K_{t+2}, V_{t+1} into the LDS buffers
// of K_t, V_{t-1} (last read in step t-1) and issues the global loads of K_{t+3}, V_{t+2}; two buffers per
// operand suffice.
// DENSE: as in the DMA form below (no mask, no prefix, whole key tiles only); instantiated for head_dim up to 64, where
// it measures 2-3 % faster (at 80 the compiler's allocation of that instance goes wrong: twice as slow).
// XTRA: key mask, logit bias and softmax denominators (see sdpa_fwd_pp_dma_kernel).
template <typename T, int D, bool ROPE_K, bool DENSE = false, bool XTRA = false>
__global__ void __launch_bounds__(kThreads8, 2) sdpa_fwd_pp_kernel(const SdpaDev p) {
    static_assert(!XTRA || (!DENSE && !ROPE_K), "key mask, bias and denominators belong to the general form");
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int BM = 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int red[16];
    unsigned char* const Kbuf = smem;                    // 2 x K tile
    unsigned char* const Vbuf = smem + 2 * G::K_BYTES;   // 2 x V tile

    int qt, bh;
    if (!block_to_tile(p, qt, bh)) return;
    const int h = bh % p.H;
    const int b = bh / p.H;

    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform, kept in a scalar register
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

    int lo = 0, hi = p.Lk;   // DENSE: rows past the end of Q repeat its last row and are never stored
    if constexpr (!DENSE) row_interval(p, b, qrow, qvalid, lo, hi);
    WaveExtent we{0, 0, p.Lk, p.Lk};
    if constexpr (!DENSE) {
        we = wave_extent(lo, hi);
        if (lane == 0) { red[wave] = we.lo_min; red[8 + wave] = we.hi_max; }
    }
    V8 qf[G::KC];
    stage_q_tile<T, D, kThreads8, BM>(smem, p, q_base, q0, tid);
    __syncthreads();
    read_q_frags<T, D>(qf, smem, wave * 32 + lq, lh);
    __syncthreads();
    // K pad columns must be zero; the V buffers are zeroed whole because the first pass through the
    // MFMA stream multiplies a zero P with whatever the second V buffer holds
    zero_pads<D, kThreads8>(Kbuf, Vbuf, G::K_BYTES, G::V_BYTES, 2, tid);
    for (int i = tid; i < 2 * G::V_BYTES / 16; i += kThreads8) *reinterpret_cast<u32x4*>(Vbuf + i * 16) = u32x4{0, 0, 0, 0};
    __syncthreads();
    int g_lo = 0, kv_stop = p.Lk;
    if constexpr (!DENSE) {
        g_lo = red[0]; kv_stop = red[8];
#pragma unroll
        for (int w = 1; w < 8; ++w) { g_lo = min(g_lo, red[w]); kv_stop = max(kv_stop, red[8 + w]); }
        g_lo = __builtin_amdgcn_readfirstlane(g_lo);
        kv_stop = __builtin_amdgcn_readfirstlane(kv_stop);
    }
    const TilePlan plan(g_lo == 0x7fffffff ? 0 : g_lo, kv_stop, p.Lp);
    const int n_tiles = plan.n_tiles;
    // XTRA: visibility words of the plan's tiles behind the tile buffers (visible after the barrier that ends the prologue)
    const unsigned long long* const kbits = (XTRA && p.key_mask) ? reinterpret_cast<const unsigned long long*>(smem + p.kbits_off) : nullptr;
    if constexpr (XTRA) build_key_bits(p, plan, b, smem + p.kbits_off, wave, lane);
    const float* const bias_row = (XTRA && p.bias && qvalid && qrow >= p.bias_q0) ? p.bias + static_cast<long>(qrow - p.bias_q0) * p.bias_rs : nullptr;
    TileExtra xt;

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    RelSoftmaxState st;
    const bool dead_row = hi <= lo;
    const float cl2 = p.scale_log2;

    const unsigned char* const k_head = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.k) + b * p.k_bs + hk * D);
    const unsigned char* const v_head = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.v) + b * p.v_bs + hk * D);
    // (the dense launch is whole tiles of one segment: its mover does no arithmetic per tile)
    auto make_mover = [&]() {
        if constexpr (DENSE) return DenseMover<T, D, kThreads8>(k_head, p.k_rs, v_head, p.v_rs, tid, wave);
        else return TileMover<T, D, kThreads8, ROPE_K>{p, plan, k_head, v_head,
                                                       reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D),
                                                       reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D),
                                                       tid, {}, {}, 1.f};
    };
    auto mv = make_mover();
    auto tile_active = [&](int t) {
        if (t < 0 || t >= n_tiles) return false;
        const int j0 = plan.j0(t);
        return j0 < we.hi_max && j0 + kBN > we.lo_min;
    };
    // this thread's share of tiles K_kt, V_vt: registers -> LDS, then prefetch K_{kt+1}, V_{vt+1}
    // (the walk measured 18 % faster at head_dim 40, 9 % at 64, and no faster from 80 on, where a thread moves two chunks)
    constexpr bool WALK = !ROPE_K && D <= 64;
    static_assert(!DENSE || WALK, "the dense mover is a walk");
    auto advance_tiles = [&](int kt, int vt) {
        if constexpr (!WALK) {
            if (kt < n_tiles) mv.store_k(kt, Kbuf + (kt & 1) * G::K_BYTES);
            if (vt < n_tiles) mv.store_v(vt, Vbuf + (vt & 1) * G::V_BYTES);
            if (kt + 1 < n_tiles) mv.template issue<0>(kt + 1);
            if (vt + 1 < n_tiles) mv.template issue<1>(vt + 1);
        } else {
            // tiles are fetched strictly in order, so the mover walks them with its cursors
            if (kt < n_tiles) mv.store_held_k(Kbuf + (kt & 1) * G::K_BYTES);
            if (vt < n_tiles) mv.store_held_v(Vbuf + (vt & 1) * G::V_BYTES);
            if (kt + 1 < n_tiles) mv.template issue_next<0>();
            if (vt + 1 < n_tiles) mv.template issue_next<1>();
        }
    };
    f32x16 sacc[2];
    V8 pf[4];
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) pf[c4] = __builtin_bit_cast(V8, u32x4{0, 0, 0, 0});

    if (n_tiles > 0) {
        // ── prologue: K_0 into LDS; registers then hold K_1, V_0 ──
        if constexpr (!WALK) {
            mv.template issue<0>(0);
            mv.store_k(0, Kbuf);
            if (n_tiles > 1) mv.template issue<0>(1);
            mv.template issue<1>(0);
        } else {
            mv.start_walk();
            mv.template issue_next<0>();
            mv.store_held_k(Kbuf);
            if (n_tiles > 1) mv.template issue_next<0>();
            mv.template issue_next<1>();
        }
        __syncthreads();
        auto softmax_of = [&](int tt) {
            if constexpr (DENSE) {
                if (tt >= 0 && tt < n_tiles) {
                    softmax_tile_rel<T, D>(sacc, pf, oacc, st, false, false, 0, 0, p.Lk, lh);
                    return;
                }
            }
            if constexpr (XTRA) {
                xt = TileExtra();
                if (kbits) {
                    const unsigned long long w = kbits[min(max(tt, 0), max(n_tiles - 1, 0))];
                    xt.kw0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(w));
                    xt.kw1 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(w >> 32));
                }
                xt.bias_cols = p.bias_cols;
            }
            if (!DENSE && tile_active(tt) && (!XTRA || (xt.kw0 | xt.kw1) != 0u)) {
                const int j0 = plan.j0(tt);
                const int lim = plan.limit(tt);
                bool interior = (j0 >= we.lo_max) && (j0 + kBN <= min(we.hi_min, lim));
                if constexpr (XTRA) {
                    const bool biased = p.bias != nullptr && j0 < p.bias_cols;
                    interior = interior && (xt.kw0 & xt.kw1) == ~0u && !biased;
                    xt.bias_row = biased ? bias_row : nullptr;
                    xt.bias_vec = p.bias_vec_ok && (j0 & 3) == 0 && j0 + kBN <= p.bias_cols;
                }
                softmax_tile_rel<T, D, false, XTRA>(sacc, pf, oacc, st, !interior, dead_row, j0, lo, min(hi, lim), lh, PrefixScale(), xt);
            } else {
                // nothing visible to this wavefront in that tile: the next PV pass must add zero
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) pf[c4] = __builtin_bit_cast(V8, u32x4{0, 0, 0, 0});
            }
        };
        // step -1 only scores tile 0 (there is no P yet)
        for (int t = -1; t < n_tiles; ++t) {
            if (grp == 1) {
                softmax_of(t);
                MI_SCHED_BARRIER
            }
            // Always the full stream: at t = -1 P is zero and the (zero-filled) V buffer adds nothing;
            // after the last tile the extra scores are never read. This wavefront's share of the tile
            // movement rides along in the stream (measured faster than in front of the softmax: the stores
            // and loads issue in the shadow of the matrix pipe).
            auto mover = [&]() { advance_tiles(t + 2, t + 1); };
            mfma_stream<T, D, true, true, decltype(mover), true>(Vbuf + (t & 1) * G::V_BYTES, Kbuf + ((t + 1) & 1) * G::K_BYTES, pf, qf,
                                                                 oacc, sacc, lane, mover, cl2, st.neg_ref);
            if (grp == 0) {
                MI_SCHED_BARRIER
                softmax_of(t + 1);
            }
            __syncthreads();
        }
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = row_inverse(l_tot);
    if constexpr (XTRA) {
        if (p.lse && qvalid && lh == 0)
            p.lse[(static_cast<long>(b) * p.H + h) * p.Lq + qrow] = l_tot > 0.f ? __builtin_amdgcn_logf(l_tot) - st.neg_ref : __builtin_huge_valf();
    }
    stage_output<T, D>(smem, wave * 32 + lq, lh, oacc, inv);
    __syncthreads();
    write_output<T, D, kThreads8>(smem, o_base, p.o_rs, q0, p.Lq, BM, tid);
}

// ─────────────── 8-wavefront kernel with tiles by LDS DMA ───────────────
// Same schedule as sdpa_fwd_pp_kernel, but K/V tiles go from global memory straight into LDS
// (global_load_lds_dwordx4: lane i of a wavefront deposits its 16 bytes at base + 16*i), so tile
// movement costs no registers and no LDS store instructions. A DMA instruction writes 1024 contiguous
// bytes, so rows sit in LDS back to back without padding; a 64-key tile is D/8 such instructions per
// operand, dealt out to the 8 wavefronts in turn. Bank conflicts of the unpadded rows:
//   head_dim 128 (256-byte rows): avoided by an XOR swizzle, 16-byte chunk c of row r lives at chunk position
//     c ^ f(r), f(r) = 4*(r%4) + (r/4)%4, applied for free on the global side (each lane fetches the chunk that
//     belongs in its LDS slot) and undone in the LDS read addresses: K reads (one row per lane, 16 consecutive
//     rows) hit 16 distinct slots, V transpose reads (4 rows x 64 bytes per 32 lanes) 4 distinct 64-byte windows;
//   head_dim 72 (144-byte rows): 16 consecutive rows start on 16 distinct multiples of 4 banks, so the K reads are
//     conflict-free as they are; the V transpose reads overlap a little.
// Without padding, the fragment reads of the zero-padded part of the head dimension (columns D..DK-1 of K,
// D..DV-1 of V) run into the first bytes of the next row: real key rows (rows past the end of a segment are fetched
// from its last row), multiplied by the zero pad of Q, or producing output columns that are never stored. A little
// zero-filled slack behind each ring keeps the reads of the last row inside the allocation.
// Tiles are ring-buffered three deep: the loads of K_{t+3}, V_{t+2} are issued in step t, awaited at
// the end of step t+1 and read in step t+2. The key loop is unrolled by three so that every LDS offset
// is an instruction immediate; tile pointers advance incrementally in scalar registers.
constexpr int kDmaStages = 3;
template <int D> struct DmaGeo {
    using G = HeadGeo<D>;
    static constexpr int ROWB = D * 2;                       // bytes per row in LDS (no padding)
    static constexpr int TILE = kBN * ROWB;                  // = (D / 8) KB
    static constexpr int NDMA = TILE / 1024;                 // DMA instructions per operand tile
    static constexpr int SLACK = 256;                        // zero bytes behind each ring
    static constexpr int RING = kDmaStages * TILE + SLACK;
    static constexpr int VOFF = RING;
    static constexpr int MAXI = (2 * NDMA + 7) / 8;          // most DMA instructions of one wavefront per step
    static constexpr bool SWZ = D == 128;
    // The Q tile is staged behind the rings, so that the first key tiles can be in flight while it is loaded, rotated and
    // picked apart; where rings + a whole staged tile exceed the LDS of a compute unit it goes through in two halves
    // (rows 0..127 for wavefronts 0..3, then rows 128..255 for wavefronts 4..7). The output is staged over the rings,
    // which are dead by then.
    static constexpr int QOFF = 2 * RING;
    static constexpr bool Q_HALVES = QOFF + 256 * G::O_STRIDE > 160 * 1024;
    static constexpr int Q_BYTES = (Q_HALVES ? 128 : 256) * G::O_STRIDE;
    static constexpr int lds_bytes() {
        const int kvq = QOFF + Q_BYTES;
        const int o = 256 * G::O_STRIDE;
        return kvq > o ? kvq : o;
    }
    static_assert(QOFF + Q_BYTES <= 160 * 1024, "rings and Q staging exceed the LDS of a compute unit");
};
// (head_dim 40 works the same way but measured no faster than the register-staged kernel: not instantiated)
template <int D> constexpr bool dma_kernel_available() { return D == 72 || D == 128; }

__device__ __forceinline__ int swz(int row) { return 4 * (row & 3) + ((row >> 2) & 3); }

// SPLIT: the launch follows p.split — a work group either processes one whole query tile or one piece of the last
// round, i.e. one or more (tile, key range) parts in sequence, each leaving a partial result in its scratch slot
// (merged by sdpa_combine_kernel). Only for unmasked calls without prefix.
// DENSE: no mask of any kind and key counts (cached prefix, if any, and fresh) that are multiples of 64: every tile is whole and visible to
// every row, so the masked form of the softmax and the per-step bookkeeping (which tile, its limit, whether this
// wavefront sees it whole) drop out of the kernel, and with them their registers: measured 6 % faster at head_dim 128
// and 8 % at 72 than the general form on the same dense call.
// PSCALE: the general form with the prefix-KV dial (factors on the rows of the cached prefix) in its softmax.
// XTRA: the general form with a key mask (one visibility bit per key, 64-bit words per key tile built once per work group
// in LDS behind the rings), an additive logit bias and the softmax denominators as an output (traced attention).
template <typename T, int D, bool SPLIT, bool DENSE = false, bool PSCALE = false, bool XTRA = false>
__global__ void __launch_bounds__(kThreads8, 2) sdpa_fwd_pp_dma_kernel(const SdpaDev p) {
    static_assert(!(SPLIT && DENSE), "the split launch clips key ranges per part");
    static_assert(!PSCALE || (!SPLIT && !DENSE), "the dial belongs to the general form");
    static_assert(!XTRA || (!SPLIT && !DENSE && !PSCALE), "key mask, bias and denominators belong to the general form");
    using G = HeadGeo<D>;
    using DG = DmaGeo<D>;
    using V8 = typename Mma<T>::v8;
    constexpr int BM = 256;
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ int red[16];

    // ── what this work group does ──
    int qt, bh;
    int kv_begin = 0, kv_end = 0x7fffffff;   // key range of the current part
    unsigned char* part = nullptr;            // scratch slot of the current part; null: the output itself
    // SPLIT bookkeeping (all wave-uniform): tail steps [seg_s, seg_end) of group xg still to do
    int xg = 0, n_full = 0, seg_s = 0, seg_end = 0, piece = 0, tail_steps = 0, n_pieces = 0;
    bool whole = true;
    if constexpr (!SPLIT) {
        if (!block_to_tile(p, qt, bh)) return;
    } else {
        xg = static_cast<int>(blockIdx.x) & 7;
        const int i = static_cast<int>(blockIdx.x) >> 3;
        n_full = p.split.full_of(xg);
        whole = i < n_full;
        if (whole) {
            const int logical = xg * p.split.chunk + i;
            qt = logical % p.n_q_tiles;
            bh = logical / p.n_q_tiles;
        } else {
            tail_steps = p.split.tail_of(xg) * p.split.T;
            n_pieces = p.split.pieces_for(tail_steps);
            piece = i - n_full;
            if (piece >= n_pieces) return;
            seg_s = SplitGeo::piece_begin(piece, tail_steps, n_pieces);
            seg_end = SplitGeo::piece_begin(piece + 1, tail_steps, n_pieces);
            qt = bh = 0;
        }
    }
  for (;;) {   // one pass per part (a single pass unless SPLIT)
    // The thread id is made opaque per pass: otherwise every address computation of the prologue and the epilogue,
    // being the same for all parts, is hoisted out of this loop and stays in registers through the key loop.
    int tid = threadIdx.x;
    if constexpr (SPLIT) asm volatile("" : "+v"(tid));
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;
    const int lane = tid & 63;
    const int lq = lane & 31;
    const int lh = lane >> 5;
    if constexpr (SPLIT) {
        if (!whole) {
            const int tt = seg_s / p.split.T;                  // tail tile of this group
            const int s0 = seg_s - tt * p.split.T;
            const int s1 = min(seg_end - tt * p.split.T, p.split.T);
            const int logical = xg * p.split.chunk + n_full + tt;
            qt = logical % p.n_q_tiles;
            bh = logical / p.n_q_tiles;
            kv_begin = s0 * kBN;
            kv_end = s1 * kBN;
            part = nullptr;
            if (s0 != 0 || s1 != p.split.T) {
                const int k = piece - SplitGeo::piece_of(tt * p.split.T, tail_steps, n_pieces);
                part = p.split_scratch + (static_cast<long>(xg * p.split.max_tail + tt) * p.split.max_parts + k) * SplitGeo::slot_bytes(D);
            }
            seg_s = tt * p.split.T + s1;
        }
    }
    const int h = bh % p.H;
    const int b = bh / p.H;
    const int q0 = qt * BM;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < p.Lq;
    const int hk = h / p.kv_group;
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;

    const int n_keys = p.Lk;   // counts the cached prefix rows, which come first
    int lo = 0, hi = n_keys;   // DENSE: rows past the end of Q repeat its last row and are never stored
    if constexpr (!DENSE) row_interval(p, b, qrow, qvalid, lo, hi);
    if constexpr (SPLIT) {
        lo = max(lo, kv_begin);
        hi = min(hi, kv_end);
        if (hi <= lo) { lo = 0; hi = 0; }
    }
    WaveExtent we{0, 0, n_keys, n_keys};
    if constexpr (!DENSE) {
        we = wave_extent(lo, hi);
        if (lane == 0) { red[wave] = we.lo_min; red[8 + wave] = we.hi_max; }
    }
    V8 qf[G::KC];
    // the Q rows (and their RoPE tables) are requested first; they are rotated and staged further down, behind the issue of
    // the first key tiles' DMA, so that both latencies run together
    using QL = QTileLoad<T, D, kThreads8, BM>;
    static_assert(!DG::Q_HALVES || (QL::NI % 2 == 0 && kThreads8 * (QL::NI / 2) == 128 * QL::CPRK), "half of the load rounds must be half of the rows");
    QL ql;
    ql.issue(p, q_base, q0, tid, p.Lq - 1);
    // the first pass through the MFMA stream multiplies a zero P with the last V buffer; the slack behind both rings is zero
    for (int i = tid; i < (DG::TILE + DG::SLACK) / 16; i += kThreads8)
        *reinterpret_cast<u32x4*>(smem + DG::VOFF + (kDmaStages - 1) * DG::TILE + i * 16) = u32x4{0, 0, 0, 0};
    for (int i = tid; i < DG::SLACK / 16; i += kThreads8)
        *reinterpret_cast<u32x4*>(smem + kDmaStages * DG::TILE + i * 16) = u32x4{0, 0, 0, 0};
    __syncthreads();
    int g_lo = 0, kv_stop = n_keys;
    if constexpr (!DENSE) {
        g_lo = red[0]; kv_stop = red[8];
#pragma unroll
        for (int w = 1; w < 8; ++w) { g_lo = min(g_lo, red[w]); kv_stop = max(kv_stop, red[8 + w]); }
        g_lo = __builtin_amdgcn_readfirstlane(g_lo);
        kv_stop = __builtin_amdgcn_readfirstlane(kv_stop);
    }
    const TilePlan plan(g_lo == 0x7fffffff ? 0 : g_lo, kv_stop, p.Lp);
    const int n_tiles = plan.n_tiles;
    // XTRA: visibility words of the plan's tiles (made visible to all wavefronts by the barrier that ends the prologue)
    const unsigned long long* const kbits = (XTRA && p.key_mask) ? reinterpret_cast<const unsigned long long*>(smem + p.kbits_off) : nullptr;
    if constexpr (XTRA) build_key_bits(p, plan, b, smem + p.kbits_off, wave, lane);
    const float* const bias_row = (XTRA && p.bias && qvalid && qrow >= p.bias_q0) ? p.bias + static_cast<long>(qrow - p.bias_q0) * p.bias_rs : nullptr;

    f32x16 oacc[G::VB];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    RelSoftmaxState st;
    const bool dead_row = hi <= lo;
    const float cl2 = p.scale_log2;

    // ── DMA duty of this wavefront: instructions i = wave, wave + 8, ... of the list [K 0..NDMA-1, V 0..NDMA-1];
    //    instruction j of an operand fills LDS bytes [1024 j, 1024 j + 1024) of the tile = chunks 64 j + lane ──
    TileCursor kc, vc;
    kc.init(plan, reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.kp) + b * p.kp_bs + hk * D), static_cast<unsigned>(p.kp_rs) * 2u,
            reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.k) + b * p.k_bs + hk * D), static_cast<unsigned>(p.k_rs) * 2u, p.Lp);
    vc.init(plan, reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.vp) + b * p.vp_bs + hk * D), static_cast<unsigned>(p.vp_rs) * 2u,
            reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.v) + b * p.v_bs + hk * D), static_cast<unsigned>(p.v_rs) * 2u, p.Lp);
    int drow[DG::MAXI];        // tile row this lane fetches in its m-th instruction
    unsigned dcol[DG::MAXI];   // byte offset inside that row
#pragma unroll
    for (int m = 0; m < DG::MAXI; ++m) {
        const int i = wave + 8 * m;
        const int j = i < DG::NDMA ? i : i - DG::NDMA;
        const int g = 64 * j + lane;
        const int row = g / G::CPR;
        int cc = g - row * G::CPR;
        if constexpr (DG::SWZ) cc ^= swz(row);     // the chunk this slot must receive
        drow[m] = row;
        dcol[m] = static_cast<unsigned>(cc) * 16u;
        if constexpr (DENSE) {
            // whole tiles of one segment only: the lane's byte offset inside a tile never changes
            const bool is_k = DG::NDMA % 8 == 0 ? m < DG::MAXI / 2 : i < DG::NDMA;
            dcol[m] += static_cast<unsigned>(row) * (static_cast<unsigned>(is_k ? p.k_rs : p.v_rs) * 2u);
        }
    }
    // One DMA instruction. Written as inline assembly on purpose: for the compiler's builtin every later LDS read may
    // alias the DMA's LDS write, so it waits for the load to land (vmcnt(0)) before the next ds_read. The tiles
    // written here are never read before the explicit wait + barrier at the end of the following step.
    const unsigned lds_base = static_cast<unsigned>(reinterpret_cast<size_t>((__attribute__((address_space(3))) unsigned char*)smem));
    auto dma = [&](const TileCursor& c, int m, int j, int lds_off) {
        unsigned voff = dcol[m];
        if constexpr (!DENSE) voff += static_cast<unsigned>(min(drow[m], min(c.rows_left, kBN) - 1)) * c.rsb;
        const unsigned dst = lds_base + lds_off + j * 1024;
        // (the LDS base travels in m0 as a declared input: the compiler writes the register itself and knows it is taken;
        //  the s_nop is the wait state an LDS-DMA instruction needs behind a write of m0)
        asm volatile("s_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(c.ptr), "{m0}"(dst) : "memory");
    };
    // this wavefront's share of the loads of one K tile (if do_k) and one V tile (if do_v); returns how many it issued
    auto dma_tiles = [&](bool do_k, int k_off, bool do_v, int v_off) -> int {
        int n = 0;
#pragma unroll
        for (int m = 0; m < DG::MAXI; ++m) {
            const int i = wave + 8 * m;
            if constexpr (DG::NDMA % 8 == 0) {
                // every wavefront has the same duty: its first MAXI / 2 instructions are K, the others V
                if (m < DG::MAXI / 2) { if (do_k) { dma(kc, m, i, k_off); ++n; } }
                else { if (do_v) { dma(vc, m, i - DG::NDMA, v_off); ++n; } }
            } else {
                if (i < DG::NDMA) { if (do_k) { dma(kc, m, i, k_off); ++n; } }
                else if (i < 2 * DG::NDMA) { if (do_v) { dma(vc, m, i - DG::NDMA, v_off); ++n; } }
            }
        }
        return n;
    };
    auto wait_all_but = [&](int n) {     // loads complete in order: everything older than the last n has landed
        if (n >= 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (n == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
        else if (n == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else if (n == 1) asm volatile("s_waitcnt vmcnt(1)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    static_assert(DG::MAXI <= 4, "wait_all_but covers at most 4 loads per step");

    // ── LDS read addresses (stage and block offsets are immediates) ──
    // K fragment (kb, c): row 32kb + lq, chunk 2c + lh (at position (2c + lh) ^ f(lq) in the swizzled layout)
    const int fk = swz(lq);
    unsigned kaddr[G::KC];
#pragma unroll
    for (int c = 0; c < G::KC; ++c) kaddr[c] = lq * DG::ROWB + ((DG::SWZ ? ((2 * c + lh) ^ fk) : (2 * c + lh)) << 4);
    // V fragment (c4, vb), halves hh = 0, 1: key row 16c4 + 4lh + 8hh + trow, 8 bytes at head-dim 32vb + tcol
    const int trow = (lane & 15) >> 2;
    const int j4 = lane & 3;
    const int g1 = (lane >> 4) & 1;
    unsigned vaddr[G::VB][2];
#pragma unroll
    for (int vb = 0; vb < G::VB; ++vb)
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int row = 4 * lh + 8 * hh + trow;
            const int chunk = 4 * vb + 2 * g1 + (j4 >> 1);
            vaddr[vb][hh] = DG::VOFF + row * DG::ROWB + ((DG::SWZ ? (chunk ^ swz(row)) : chunk) << 4) + 8 * (j4 & 1);
        }

    static_assert(G::DK == D || G::DK - D == 8, "the pad of a K row is the upper lane half of its last fragment");
    const unsigned pad_keep = lh ? 0u : ~0u;

    f32x16 sacc[2];
    V8 pf[4];
#pragma unroll
    for (int c4 = 0; c4 < 4; ++c4) pf[c4] = __builtin_bit_cast(V8, u32x4{0, 0, 0, 0});

    auto tile_active = [&](int t) {
        if (t < 0 || t >= n_tiles) return false;
        const int j0 = plan.j0(t);
        return j0 < we.hi_max && j0 + kBN > we.lo_min;
    };

    // One step t of the loop with S = (t + 1) % 3 known at compile time:
    //   reads K_{t+1} from K stage S and V_t from V stage (S + 2) % 3,
    //   loads K_{t+3} into K stage (S + 2) % 3 and V_{t+2} into V stage (S + 1) % 3.
    auto step = [&](auto stage_tag, int t) {
        constexpr int S = decltype(stage_tag)::value;
        constexpr int KS = S * DG::TILE, VS = ((S + 2) % 3) * DG::TILE;
        constexpr int KD = ((S + 2) % 3) * DG::TILE, VD = DG::VOFF + ((S + 1) % 3) * DG::TILE;
        const bool load_k = t + 3 < n_tiles, load_v = t + 2 < n_tiles;
        int issued = 0;
        // XTRA: the visibility word of the tile whose softmax this wavefront runs in this step, fetched here, ahead of this
        // step's DMA instructions (an LDS read behind them would wait for them to land)
        TileExtra xt;
        if constexpr (XTRA) {
            if (kbits) {
                const unsigned long long w = kbits[min(max(grp == 1 ? t : t + 1, 0), max(n_tiles - 1, 0))];
                xt.kw0 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(w));
                xt.kw1 = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(w >> 32));
            }
            xt.bias_cols = p.bias_cols;
        }
        auto softmax_of = [&](int tt) {
            if constexpr (DENSE) {
                if (tt >= 0 && tt < n_tiles) {
                    softmax_tile_rel<T, D>(sacc, pf, oacc, st, false, false, 0, 0, n_keys, lh);
                    return;
                }
            }
            if (!DENSE && tile_active(tt) && (!XTRA || (xt.kw0 | xt.kw1) != 0u)) {
                const int j0 = plan.j0(tt);
                const int lim = plan.limit(tt);
                bool interior = (j0 >= we.lo_max) && (j0 + kBN <= min(we.hi_min, lim));
                if constexpr (XTRA) {
                    const bool biased = p.bias != nullptr && j0 < p.bias_cols;
                    interior = interior && (xt.kw0 & xt.kw1) == ~0u && !biased;
                    xt.bias_row = biased ? bias_row : nullptr;
                    xt.bias_vec = p.bias_vec_ok && (j0 & 3) == 0 && j0 + kBN <= p.bias_cols;
                }
                softmax_tile_rel<T, D, PSCALE, XTRA>(sacc, pf, oacc, st, !interior, dead_row, j0, lo, min(hi, lim), lh,
                                                     PSCALE ? prefix_scale_of(p, plan.in_prefix(tt)) : PrefixScale(), xt);
            } else {
                // nothing visible to this wavefront in that tile: the next PV pass must add zero
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) pf[c4] = __builtin_bit_cast(V8, u32x4{0, 0, 0, 0});
            }
        };
        // An LDS read issued behind an LDS-DMA load does not return before that load has landed (measured: the
        // read takes the full memory latency), so the DMA instructions of a step go where the wavefront has no
        // LDS access ahead of it for a long time: right before its softmax.
        auto issue_dma = [&]() {
            issued = dma_tiles(load_k, KD, load_v, VD);
            if (DENSE && p.Lp == 0) {
                if (load_k) kc.ptr += kBN * kc.rsb;
                if (load_v) vc.ptr += kBN * vc.rsb;
            } else {
                if (load_k) kc.next();
                if (load_v) vc.next();
            }
        };
        // group 1 turns the scores of its previous step into P first, so that its MFMA stream meets group 0's softmax
        if (grp == 1) {
            issue_dma();
            MI_SCHED_BARRIER
            softmax_of(t);
            MI_SCHED_BARRIER
        }
        {
            // the stream scores first (S_{t+1} = K_{t+1} Q^T), then O += V_t^T P_t; under the PV MFMAs, which do not touch
            // the scores, each raw score becomes the softmax exponent x = s * cl2 - ref (see mfma_stream)
            constexpr int NQK = 2 * G::KC, NPV = 4 * G::VB, N = NQK + NPV;
            auto fetch = [&](int i) -> V8 {
                if (i >= NQK) {
                    const int j = i - NQK;
                    const int c4 = j / G::VB, vb = j % G::VB;
                    const s16x4 v_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(smem + VS + 16 * c4 * DG::ROWB + vaddr[vb][0]));
                    const s16x4 v_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                        (__attribute__((address_space(3))) s16x4*)(smem + VS + 16 * c4 * DG::ROWB + vaddr[vb][1]));
                    const s16x8 a = __builtin_shufflevector(v_lo, v_hi, 0, 1, 2, 3, 4, 5, 6, 7);
                    return __builtin_bit_cast(V8, a);
                } else {
                    const int kb = i / G::KC, c = i % G::KC;
                    u32x4 a = *reinterpret_cast<const u32x4*>(smem + KS + 32 * kb * DG::ROWB + kaddr[c]);
                    // the upper lane half of the last fragment holds the first elements of the NEXT key row where the head
                    // dimension is padded (unpadded rows): blanked, because Q's zero pad does not silence a NaN or an
                    // infinity there, and the next row may be one that this query must not see
                    if (G::DK > D && c == G::KC - 1) a &= pad_keep;
                    return __builtin_bit_cast(V8, a);
                }
            };
            V8 ring[kAhead];
#pragma unroll
            for (int i = 0; i < kAhead; ++i) ring[i] = fetch(i);
            const float neg_ref = st.neg_ref;
            [&]<int... I>(std::integer_sequence<int, I...>) {
                ([&] {
                    constexpr int i = I;
                    const V8 a = ring[i % kAhead];
                    if constexpr (i >= NQK) {
                        constexpr int j = i - NQK;
                        constexpr int c4 = j / G::VB, vb = j % G::VB;
                        oacc[vb] = Mma<T>::run(a, pf[c4], oacc[vb]);
                    } else {
                        constexpr int kb = i / G::KC, c = i % G::KC;
                        if constexpr (c == 0) {
                            const f32x16 zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                            sacc[kb] = Mma<T>::run(a, qf[c], zero);
                        } else {
                            sacc[kb] = Mma<T>::run(a, qf[c], sacc[kb]);
                        }
                    }
                    if constexpr (i + kAhead < N) ring[i % kAhead] = fetch(i + kAhead);
                    if constexpr (i >= NQK) scores_to_exponents<NPV, i - NQK>(sacc, cl2, neg_ref);
                    MI_SCHED_BARRIER
                }(), ...);
            }(std::make_integer_sequence<int, N>{});
        }
        if (grp == 0) {
            MI_SCHED_BARRIER
            issue_dma();
            MI_SCHED_BARRIER
            softmax_of(t + 1);
        }
        // The tiles loaded in the PREVIOUS step are read in the next one: wait for those only (this step's
        // loads stay in flight), then meet the other wavefronts.
        if constexpr (DG::NDMA % 8 == 0) {
            // every wavefront issues NDMA / 8 loads per operand tile: the count follows from the flags alone
            if (load_k) wait_all_but(DG::NDMA / 4);
            else if (load_v) wait_all_but(DG::NDMA / 8);
            else wait_all_but(0);
        } else {
            wait_all_but(issued);
        }
        __syncthreads();
    };

    if (n_tiles > 0) {
        // prologue: K_0, K_1, V_0 (the loop loads K_{t+3}, V_{t+2} from t = -1 on); cursors end at K_2, V_1
        dma_tiles(true, 0, false, 0);
        if (n_tiles > 1) { kc.next(); dma_tiles(true, DG::TILE, false, 0); }
        if (n_tiles > 2) kc.next();
        dma_tiles(false, 0, true, DG::VOFF);
        if (n_tiles > 1) vc.next();
    }
    {
        // the Q tile, rotated on its way into the staging buffer behind the rings; every lane then picks the fragments of
        // its own row
        unsigned char* const Qs = smem + DG::QOFF;
        const bool split_pairs = p.cos_q != nullptr && p.rope_split;
        if constexpr (!DG::Q_HALVES) {
            ql.store(Qs, p, q0, tid, p.Lq - 1);
            if (split_pairs) {
                __syncthreads();
                rope_split_staged<T, D, kThreads8>(Qs, p, q0, tid, p.Lq - 1, 1.f, 0, BM);
            }
            __syncthreads();
            read_q_frags<T, D>(qf, Qs, wave * 32 + lq, lh);
        } else {
            ql.template store<0, QL::NI / 2>(Qs, p, q0, tid, p.Lq - 1, 1.f, 0);
            if (split_pairs) {
                __syncthreads();
                rope_split_staged<T, D, kThreads8>(Qs, p, q0, tid, p.Lq - 1, 1.f, 0, BM / 2);
            }
            __syncthreads();
            if (grp == 0) read_q_frags<T, D>(qf, Qs, wave * 32 + lq, lh);
            __syncthreads();
            ql.template store<QL::NI / 2, QL::NI>(Qs, p, q0, tid, p.Lq - 1, 1.f, BM / 2);
            if (split_pairs) {
                __syncthreads();
                rope_split_staged<T, D, kThreads8>(Qs, p, q0, tid, p.Lq - 1, 1.f, BM / 2, BM / 2);
            }
            __syncthreads();
            if (grp == 1) read_q_frags<T, D>(qf, Qs, (wave - 4) * 32 + lq, lh);
        }
    }
    if (n_tiles > 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        for (int t = -1; t < n_tiles; t += 3) {
            step(std::integral_constant<int, 0>{}, t);
            if (t + 1 >= n_tiles) break;
            step(std::integral_constant<int, 1>{}, t + 1);
            if (t + 2 >= n_tiles) break;
            step(std::integral_constant<int, 2>{}, t + 2);
        }
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = row_inverse(l_tot);
    if constexpr (XTRA) {
        // base-2 log of the row's denominator in exponent units: p(key) = exp2(score * scale_log2 [+ bias * log2 e] - lse);
        // +inf for a row without visible keys, so that every p is 0
        if (p.lse && qvalid && lh == 0)
            p.lse[(static_cast<long>(b) * p.H + h) * p.Lq + qrow] = l_tot > 0.f ? __builtin_amdgcn_logf(l_tot) - st.neg_ref : __builtin_huge_valf();
    }
    stage_output<T, D>(smem, wave * 32 + lq, lh, oacc, inv);
    __syncthreads();
    if constexpr (!SPLIT) {
        write_output<T, D, kThreads8>(smem, o_base, p.o_rs, q0, p.Lq, BM, tid);
        break;
    } else {
        if (part == nullptr) {
            write_output<T, D, kThreads8>(smem, o_base, p.o_rs, q0, p.Lq, BM, tid);
        } else {
            // normalised partial output of the part, then per row the softmax reference (log2 domain) and the
            // denominator relative to it: the part's weight in the merge is l * 2^ref
            write_output<T, D, kThreads8>(smem, reinterpret_cast<T*>(part), D, 0, min(BM, p.Lq - q0), BM, tid);
            if (lh == 0) {
                float* stat = reinterpret_cast<float*>(part + static_cast<long>(BM) * D * 2);
                stat[wave * 32 + lq] = -st.neg_ref;
                stat[BM + wave * 32 + lq] = l_tot;
            }
        }
        if (whole || seg_s >= seg_end) break;
        __syncthreads();   // the staged output is read by all threads before the next part stages its Q tile
    }
  }
}

// Merge of the parts of one split query tile: out = sum_k w_k O_k / sum_k w_k with w_k = l_k 2^(ref_k - max ref).
// blockIdx.x = (XCD group, tail tile); tiles that were written whole are skipped.
template <typename T, int D>
__global__ void __launch_bounds__(256) sdpa_combine_kernel(const SdpaDev p) {
    typedef T t8 __attribute__((ext_vector_type(8)));
    constexpr int BM = 256, CPR = D / 8;
    const SplitGeo& sg = p.split;
    const int xg = static_cast<int>(blockIdx.x) & 7, tt = static_cast<int>(blockIdx.x) >> 3;
    if (tt >= sg.tail_of(xg)) return;
    const int S = sg.tail_of(xg) * sg.T, np = sg.pieces_for(S);
    const int first = SplitGeo::piece_of(tt * sg.T, S, np);
    const int n_parts = SplitGeo::piece_of((tt + 1) * sg.T - 1, S, np) - first + 1;
    if (n_parts == 1) return;
    const int logical = xg * sg.chunk + sg.full_of(xg) + tt;
    const int qt = logical % p.n_q_tiles, bh = logical / p.n_q_tiles;
    const int h = bh % p.H, b = bh / p.H;
    const int q0 = qt * BM;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const unsigned char* slots = p.split_scratch + static_cast<long>(xg * sg.max_tail + tt) * sg.max_parts * SplitGeo::slot_bytes(D);
    // one 16-byte piece of one row per thread; blockIdx.y walks the tile (many short work groups: the merge is a
    // chain of two dependent loads per part, hidden by occupancy rather than by unrolling)
    {
        const int idx = static_cast<int>(blockIdx.y) * 256 + static_cast<int>(threadIdx.x);
        if (idx >= BM * CPR) return;
        const int row = idx / CPR, cc = idx - row * CPR;
        if (q0 + row >= p.Lq) return;
        // a part without visible keys has denominator 0 and is skipped; one whose denominator is NaN (a non-finite score)
        // must not be: it makes the row NaN, as it would in an unsplit launch. Hence the test on the bits.
        // (the bits pass through an empty asm statement: left visible, the optimiser turns the integer test back into a
        //  floating-point comparison that is false for a NaN, which -fno-honor-nans entitles it to)
        auto empty = [](float l) {
            unsigned bits = __builtin_bit_cast(unsigned, l);
            asm volatile("" : "+v"(bits));
            return (bits & 0x7fffffffu) == 0u;
        };
        float ref = kNegInf;
        for (int k = 0; k < n_parts; ++k) {
            const float* stat = reinterpret_cast<const float*>(slots + k * SplitGeo::slot_bytes(D) + static_cast<long>(BM) * D * 2);
            if (!empty(stat[BM + row])) ref = fmaxf(ref, stat[row]);
        }
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        float wsum = 0.f;
        for (int k = 0; k < n_parts; ++k) {
            const unsigned char* slot = slots + k * SplitGeo::slot_bytes(D);
            const float* stat = reinterpret_cast<const float*>(slot + static_cast<long>(BM) * D * 2);
            const float l = stat[BM + row];
            if (empty(l)) continue;
            const float w = l * __builtin_amdgcn_exp2f(stat[row] - ref);
            wsum += w;
            const t8 o = *reinterpret_cast<const t8*>(slot + (static_cast<long>(row) * D + cc * 8) * 2);
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[e] = __builtin_fmaf(w, static_cast<float>(o[e]), acc[e]);
        }
        const float inv = row_inverse(wsum);
        t8 out;
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = static_cast<T>(acc[e] * inv);
        *reinterpret_cast<t8*>(o_base + static_cast<long>(q0 + row) * p.o_rs + cc * 8) = out;
    }
}

// Decides whether the launch splits its last round (see SplitGeo) and fills p.split. The split costs every tail work
// group a second prologue and the launch a merge pass (together about ten key steps), so it is taken only when it
// shortens the last round by more than that — and only when the last round would fill at most half of the GPU:
// under sustained MFMA load the GPU runs at its power limit, a partly idle last round runs at a higher clock, and
// measured time follows the total work rather than the number of rounds (432 tiles on 256 compute units take 1.70
// times one full round, not 2). Measured on head_dim 128, 24 heads: last round 7/32 full: 12 % faster with the
// split, 10/32: 10 %, 16/32: 6 %, 22/32: 5 % slower.
template <int D>
bool plan_split(SdpaDev& p, int n_cu) {
    p.split = SplitGeo{};
    if constexpr (!dma_kernel_available<D>()) return false;
    if (p.mask_mode != MI_MASK_NONE || p.kv_valid_len || p.key_mask || p.Lp > 0 || p.cos_k || p.cu_q) return false;
    // the logit bias and the softmax denominators exist in the 128-row kernel only
    if (p.bias != nullptr || p.lse != nullptr) return false;
    if (n_cu < 8 || n_cu % 8 != 0 || sdpa_kernel_choice() == 1 || sdpa_kernel_choice() == 3) return false;
    const long tiles = static_cast<long>(p.B) * p.H * ((p.Lq + 255) / 256);
    const int T = (p.Lk + kBN - 1) / kBN;
    if (tiles < n_cu || tiles > (1 << 24) || T < 16 || T > (1 << 20)) return false;
    SplitGeo g{};
    g.T = T; g.n_blocks = static_cast<int>(tiles); g.chunk = static_cast<int>((tiles + 7) / 8); g.cu_g = n_cu / 8;
    const int tail0 = g.tail_of(0);
    if (tail0 == 0 || 2 * tail0 > g.cu_g) return false;
    const int np0 = g.pieces_for(tail0 * T);
    const int piece_len = (tail0 * T + np0 - 1) / np0;
    if (T - piece_len < 12) return false;
    for (int xg = 0; xg < 8; ++xg) {
        const int tail = g.tail_of(xg), S = tail * T, np = g.pieces_for(S);
        g.max_tail = max(g.max_tail, tail);
        for (int tt = 0; tt < tail; ++tt)
            g.max_parts = max(g.max_parts, SplitGeo::piece_of((tt + 1) * T - 1, S, np) - SplitGeo::piece_of(tt * T, S, np) + 1);
    }
    g.enabled = 1;
    p.split = g;
    return true;
}
template <int D>
size_t split_scratch_bytes_d(SdpaDev p, int n_cu) {
    if (!plan_split<D>(p, n_cu)) return 0;
    return static_cast<size_t>(8) * p.split.max_tail * p.split.max_parts * SplitGeo::slot_bytes(D);
}

template <typename T, int D>
int launch_d(SdpaDev p, int n_cu, hipStream_t stream) {
    const bool rope_k = p.cos_k != nullptr;
    if (p.cu_q != nullptr) {
        p.n_q_tiles = (p.Lq + 127) / 128;
        p.n_blocks = p.B * p.H * p.n_q_tiles;
        hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, false, true>), dim3(grid_blocks(p)), dim3(kThreads4), lds_bytes_4<D>(), stream, p);
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) return fail("sdpa_fwd launch: %s", hipGetErrorString(e));
        return 0;
    }
    if constexpr (dma_kernel_available<D>()) {
        if (p.split_scratch != nullptr && plan_split<D>(p, n_cu) &&
            p.split_scratch_bytes >= static_cast<size_t>(8) * p.split.max_tail * p.split.max_parts * SplitGeo::slot_bytes(D)) {
            p.n_q_tiles = (p.Lq + 255) / 256;
            p.n_blocks = p.split.n_blocks;
            int per_group = 0;
            for (int xg = 0; xg < 8; ++xg)
                per_group = max(per_group, p.split.full_of(xg) + p.split.pieces_for(p.split.tail_of(xg) * p.split.T));
            hipLaunchKernelGGL((sdpa_fwd_pp_dma_kernel<T, D, true>), dim3(8 * per_group), dim3(kThreads8), DmaGeo<D>::lds_bytes(), stream, p);
            hipLaunchKernelGGL((sdpa_combine_kernel<T, D>), dim3(8 * p.split.max_tail, (256 * (D / 8) + 255) / 256), dim3(256), 0, stream, p);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail("sdpa_fwd launch: %s", hipGetErrorString(e));
            return 0;
        }
        p.split = SplitGeo{};
    }
    // 256-row tiles when they give every CU at least one work group; head_dim above 128 does not fit
    // two wavefronts per SIMD and stays on the 128-row kernel.
    const long tiles256 = static_cast<long>(p.B) * p.H * ((p.Lq + 255) / 256);
    const int choice = sdpa_kernel_choice();
    // calls with a key mask, a logit bias or a request for the softmax denominators take the XTRA instances of the 256-row
    // kernels (visibility words of all key tiles in LDS behind the tile buffers), unless K is rotated tile by tile, the
    // prefix-KV dial is on as well, or the key sequence is too long for the words to fit: then the 128-row kernel
    const bool xtra = p.key_mask != nullptr || p.bias != nullptr || p.lse != nullptr;
    const long kbits_bytes = p.key_mask ? 8L * ((p.Lk + kBN - 1) / kBN + 2) : 0;
    const bool xtra_ok = !xtra || (!rope_k && !p.prefix_scaled && kbits_bytes <= 24 * 1024);   // (the words share the LDS with rings and Q staging)
    // calls with the prefix-KV dial stay on the 128-row kernel unless the DMA kernel (which has an instance for it) takes them
    const bool dial_ok = !p.prefix_scaled || (dma_kernel_available<D>() && !rope_k && choice != 3);
    const bool pingpong = D <= 128 && xtra_ok && dial_ok && (choice >= 2 || (choice == 0 && tiles256 >= n_cu));
    // short key sequences whose K and V fit in LDS next to a query tile: one work group walks several query tiles
    const int n_kt = (p.Lk + kBN - 1) / kBN;
    if (D <= 128 && choice == 0 && p.mask_mode == MI_MASK_NONE && p.bias == nullptr && p.lse == nullptr &&
        p.Lp == 0 && !rope_k && p.cos_q == nullptr && n_kt >= 1 && n_kt <= shortkv_max_tiles<(D <= 128 ? D : 128)>() && tiles256 >= n_cu &&
        shortkv_lds_bytes<D>(n_kt, p.key_mask != nullptr) <= 160 * 1024) {
        if constexpr (D <= 128) {
            p.n_q_tiles = (p.Lq + 255) / 256;
            const int n_strip = static_cast<int>(tiles256 / n_cu);   // 256 query rows per work group and round: about one work group per CU
            const int strips_per_head = (p.n_q_tiles + n_strip - 1) / n_strip;
            p.n_blocks = p.B * p.H * strips_per_head;
            hipLaunchKernelGGL((sdpa_shortkv_kernel<T, D>), dim3(grid_blocks(p)), dim3(kThreads8), shortkv_lds_bytes<D>(n_kt, p.key_mask != nullptr), stream, p,
                               n_kt, 8 * n_strip, strips_per_head);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return fail("sdpa_fwd launch: %s", hipGetErrorString(e));
            return 0;
        }
    }
    if (pingpong) {
        p.n_q_tiles = (p.Lq + 255) / 256;
        p.n_blocks = static_cast<int>(tiles256);
        const dim3 grid(grid_blocks(p)), block(kThreads8);
        if constexpr (D <= 128) {
            if (xtra) {
                const bool dma = dma_kernel_available<D>() && sdpa_kernel_choice() != 3;
                if constexpr (dma_kernel_available<D>()) {
                    if (dma) {
                        p.kbits_off = DmaGeo<D>::lds_bytes();
                        hipLaunchKernelGGL((sdpa_fwd_pp_dma_kernel<T, D, false, false, false, true>), grid, block,
                                           DmaGeo<D>::lds_bytes() + kbits_bytes, stream, p);
                    }
                }
                if (!dma) {
                    p.kbits_off = lds_bytes_8<D>();
                    hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, false, false, true>), grid, block, lds_bytes_8<D>() + kbits_bytes, stream, p);
                }
            }
            else if (rope_k) hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, true>), grid, block, lds_bytes_8<D>(), stream, p);
            else if (dma_kernel_available<D>() && sdpa_kernel_choice() != 3) {
                if constexpr (dma_kernel_available<D>()) {
                    // whole key tiles only; a cached prefix may come first if it is whole tiles too and laid out like K / V
                    const bool dense = p.mask_mode == MI_MASK_NONE && p.kv_valid_len == nullptr && p.Lk % kBN == 0 && !p.prefix_scaled &&
                                       (p.Lp == 0 || (p.Lp % kBN == 0 && p.kp_rs == p.k_rs && p.vp_rs == p.v_rs));
                    if (dense) hipLaunchKernelGGL((sdpa_fwd_pp_dma_kernel<T, D, false, true>), grid, block, DmaGeo<D>::lds_bytes(), stream, p);
                    else if (p.prefix_scaled) hipLaunchKernelGGL((sdpa_fwd_pp_dma_kernel<T, D, false, false, true>), grid, block, DmaGeo<D>::lds_bytes(), stream, p);
                    else hipLaunchKernelGGL((sdpa_fwd_pp_dma_kernel<T, D, false>), grid, block, DmaGeo<D>::lds_bytes(), stream, p);
                }
            }
            else if (D <= 64 && p.mask_mode == MI_MASK_NONE && p.kv_valid_len == nullptr && p.Lp == 0 && p.Lk % kBN == 0) {
                if constexpr (D <= 64) hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, false, true>), grid, block, lds_bytes_8<D>(), stream, p);
            }
            else hipLaunchKernelGGL((sdpa_fwd_pp_kernel<T, D, false>), grid, block, lds_bytes_8<D>(), stream, p);
        }
    } else {
        p.n_q_tiles = (p.Lq + 127) / 128;
        p.n_blocks = p.B * p.H * p.n_q_tiles;
        const dim3 grid(grid_blocks(p)), block(kThreads4);
        if (p.prefix_scaled) {
            if (rope_k) return fail("mi_sdpa_forward: the prefix-KV dial with K rotated tile by tile is not supported (lend rope_k_scratch)");
            hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, false, false, true>), grid, block, lds_bytes_4<D>(), stream, p);
        }
        else if (rope_k) hipLaunchKernelGGL((sdpa_fwd_kernel<T, D, true>), grid, block, lds_bytes_4<D>(), stream, p);
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
        default: return fail("mi_sdpa_forward: head_dim %d has no kernel (40, 64, 72, 80, 96, 112, 128, 160, 256, 384, 512)", head_dim);
    }
}

}  // namespace

bool sdpa_supported(int dtype, int head_dim) {
    if (dtype != MI_DTYPE_F16 && dtype != MI_DTYPE_BF16) return false;
    switch (head_dim) {
        case 40: case 64: case 72: case 80: case 96: case 112: case 128: case 160: return true;
        default: return sdpa_wide_head(head_dim);
    }
}

size_t sdpa_split_scratch_bytes(const SdpaDev& p, int dtype, int head_dim) {
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_F16) return 0;
    const int n_cu = device_cu_count();
    if (head_dim == 72) return split_scratch_bytes_d<72>(p, n_cu);
    if (head_dim == 128) return split_scratch_bytes_d<128>(p, n_cu);
    return 0;
}

int launch_sdpa(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream) {
    if (sdpa_wide_head(head_dim)) return launch_sdpa_wide(p, dtype, head_dim, stream);
    const int n_cu = device_cu_count();
    if (dtype == MI_DTYPE_BF16) return launch_t<__bf16>(p, head_dim, n_cu, stream);
    if (dtype == MI_DTYPE_F16) return launch_t<_Float16>(p, head_dim, n_cu, stream);
    return fail("mi_sdpa_forward: dtype %d not supported (fp16 = 1, bf16 = 2)", dtype);
}

}  // namespace mi
