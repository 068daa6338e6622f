// Work distribution and K/V tile movement shared by the softmax-attention kernels: work-group id -> (query tile, head),
// the cut of the key axis into 64-row tiles, the walk over those tiles, and the cooperative global -> registers -> LDS
// tile mover with its LDS pad handling and the coalesced write-out of a staged output tile.
#pragma once
#include "sdpa_common.h"

namespace mi {
namespace sdpa {

// Work-group id -> logical tile. Hardware deals consecutive work-group ids round-robin over the 8
// XCDs; undo that so each XCD (one L2) gets a contiguous run of logical tiles, i.e. query tiles that
// share the same K/V. Returns -1 for the padding groups of the last round.
__device__ __forceinline__ int logical_block(int n_blocks) {
    const int chunk = (n_blocks + 7) >> 3;
    const int logical = (blockIdx.x & 7) * chunk + (blockIdx.x >> 3);
    return logical < n_blocks ? logical : -1;
}

// Work-group id -> (query tile, batch*head). False for the padding groups of the grid.
// Unmasked calls: every tile costs the same, so the order only serves locality (logical_block).
// Masked calls (causal, windowed, block-causal): later query tiles see more keys, and work groups start in id
// order, so ids run over the query tiles from the last to the first with the heads innermost — the longest tiles
// start first and the short ones fill the gaps at the end (longest-processing-time order). The head count is
// padded to a multiple of 8 in id space so that id % 8, the XCD, still depends on the head alone and an XCD
// keeps meeting the same K/V.
__device__ __forceinline__ bool block_to_tile(const SdpaDev& p, int& qt, int& bh) {
    if (p.mask_mode == MI_MASK_NONE) {
        const int logical = logical_block(p.n_blocks);
        if (logical < 0) return false;
        qt = logical % p.n_q_tiles;
        bh = logical / p.n_q_tiles;
        return true;
    }
    const int bh8 = (p.B * p.H + 7) & ~7;
    qt = p.n_q_tiles - 1 - static_cast<int>(blockIdx.x) / bh8;
    bh = static_cast<int>(blockIdx.x) % bh8;
    return qt >= 0 && bh < p.B * p.H;
}
// Grid size that block_to_tile expects for n_q_tiles query tiles.
inline unsigned grid_blocks(const SdpaDev& p) {
    if (p.mask_mode == MI_MASK_NONE) return static_cast<unsigned>(((p.n_blocks + 7) / 8) * 8);
    return static_cast<unsigned>(((p.B * p.H + 7) & ~7) * p.n_q_tiles);
}

// The key axis is cut into 64-row tiles that never straddle the prefix / fresh boundary: prefix
// tiles start at a multiple of 64 below prefix_len (the last one may be partial), fresh tiles start at
// prefix_len + a multiple of 64. Rows of a tile at or beyond its segment's limit are zero in LDS and
// masked in the scores.
struct TilePlan {
    int pre_lo, pre_hi, n_pre;  // prefix rows [pre_lo, pre_hi)
    int fr_lo, fr_hi, n_tiles;  // all keys are numbered over [prefix ; fresh]
    __device__ __forceinline__ TilePlan(int first_key, int stop_key, int Lp) {
        pre_lo = first_key < Lp ? (first_key / kBN) * kBN : Lp;
        pre_hi = min(stop_key, Lp);
        n_pre = pre_hi > pre_lo ? (pre_hi - pre_lo + kBN - 1) / kBN : 0;
        fr_lo = first_key > Lp ? Lp + ((first_key - Lp) / kBN) * kBN : Lp;
        fr_hi = stop_key;
        const int n_fr = fr_hi > fr_lo ? (fr_hi - fr_lo + kBN - 1) / kBN : 0;
        n_tiles = n_pre + n_fr;
    }
    __device__ __forceinline__ bool in_prefix(int t) const { return t < n_pre; }
    __device__ __forceinline__ int j0(int t) const { return t < n_pre ? pre_lo + t * kBN : fr_lo + (t - n_pre) * kBN; }
    __device__ __forceinline__ int limit(int t) const { return t < n_pre ? pre_hi : fr_hi; }
};

// Visibility words of a plan's key tiles from a key mask (a key is hidden where the mask holds +0 or -0): bit i of word t
// says whether key i of tile t is visible; keys at or past the tile's segment limit count as hidden. Built by the
// wavefronts of a work group in turn (one ballot per tile) into LDS at `dst`; the caller's next barrier publishes them.
__device__ __forceinline__ void build_key_bits(const SdpaDev& p, const TilePlan& plan, int b, unsigned char* dst, int wave, int lane,
                                               int n_waves = 8) {
    if (!p.key_mask) return;
    const float* const km = p.key_mask + b * p.key_mask_bs;
    unsigned long long* const out = reinterpret_cast<unsigned long long*>(dst);
    for (int t = wave; t < plan.n_tiles; t += n_waves) {
        const int j = plan.j0(t) + lane;
        unsigned bits = 0;
        if (j < plan.limit(t)) bits = __builtin_bit_cast(unsigned, km[j]) & 0x7fffffffu;
        const unsigned long long w = __ballot(bits != 0u);
        if (lane == 0) out[t] = w;
    }
}

// Walks the tiles of one operand (K or V) in order, keeping the tile's base pointer, row stride and
// the number of rows left in the current segment (prefix, then fresh) in scalar registers.
struct TileCursor {
    const unsigned char* ptr;     // first row of the current tile
    unsigned rsb;                 // row stride in bytes
    int rows_left;                // rows of the segment from the current tile on
    int t;                        // index of the current tile
    // fresh segment, entered when t reaches n_pre
    const unsigned char* fresh_ptr;
    unsigned fresh_rsb;
    int fresh_rows, n_pre;
    __device__ __forceinline__ void init(const TilePlan& plan, const unsigned char* pre_base, unsigned pre_rsb,
                                         const unsigned char* fr_base, unsigned fr_rsb, int Lp) {
        fresh_ptr = fr_base + static_cast<unsigned long>(plan.fr_lo - Lp) * fr_rsb;
        fresh_rsb = fr_rsb;
        fresh_rows = plan.fr_hi - plan.fr_lo;
        n_pre = plan.n_pre;
        t = 0;
        if (n_pre > 0) { ptr = pre_base + static_cast<unsigned long>(plan.pre_lo) * pre_rsb; rsb = pre_rsb; rows_left = plan.pre_hi - plan.pre_lo; }
        else { ptr = fresh_ptr; rsb = fresh_rsb; rows_left = fresh_rows; }
    }
    __device__ __forceinline__ void next() {
        ++t;
        if (t == n_pre) { ptr = fresh_ptr; rsb = fresh_rsb; rows_left = fresh_rows; }
        else { ptr += kBN * rsb; rows_left -= kBN; }
    }
};

// Cooperative K/V tile movement for a work group of NT threads: global -> registers -> LDS.
// kreg / vreg hold this thread's 16-byte chunks of one K tile and one V tile (possibly different tiles).
template <typename T, int D, int NT, bool ROPE_K>
struct TileMover {
    using G = HeadGeo<D>;
    static constexpr int NLD = (G::NCH + NT - 1) / NT;
    static constexpr bool EXACT = (G::NCH % NT) == 0;
    const SdpaDev& p;
    const TilePlan& plan;
    const unsigned char* k_base; const unsigned char* v_base; const unsigned char* kp_base; const unsigned char* vp_base;
    int tid;
    u32x4 kreg[NLD], vreg[NLD];
    float mreg;   // key-mask value of key row `tid` of the K tile in kreg (threads 0..63, 4-wavefront kernel)

    // key-mask values travel with the K tile: one float per key row, staged next to the tile in LDS
    __device__ __forceinline__ void issue_mask(int t, const float* key_mask) {
        if (tid < kBN) {
            const int j = plan.j0(t) + tid;
            mreg = j < plan.limit(t) ? key_mask[j] : 0.f;
        }
    }
    __device__ __forceinline__ void store_mask(float* Ms) {
        if (tid < kBN) Ms[tid] = mreg;
    }

    // Sequential walk (8-wavefront kernel): kc / vc stand on the next tile to fetch, k_rows / v_rows are the rows that
    // exist in the tile held in kreg / vreg. Tile pointers advance by scalar additions; nothing is recomputed from t.
    TileCursor kc, vc;
    int k_rows, v_rows;
    __device__ __forceinline__ void start_walk() {
        kc.init(plan, kp_base, static_cast<unsigned>(p.kp_rs) * 2u, k_base, static_cast<unsigned>(p.k_rs) * 2u, p.Lp);
        vc.init(plan, vp_base, static_cast<unsigned>(p.vp_rs) * 2u, v_base, static_cast<unsigned>(p.v_rs) * 2u, p.Lp);
        k_rows = v_rows = 0;
    }
    template <int WHICH>
    __device__ __forceinline__ void issue_next() {
        u32x4 (&reg)[NLD] = WHICH == 0 ? kreg : vreg;
        TileCursor& c = WHICH == 0 ? kc : vc;
        const int rows = min(c.rows_left, kBN);
        (WHICH == 0 ? k_rows : v_rows) = rows;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = min(idx / G::CPR, rows - 1);   // rows past the end repeat the last one (zeroed by the store)
            const int cc = idx % G::CPR;
            if (EXACT || idx < G::NCH) reg[i] = *reinterpret_cast<const u32x4*>(c.ptr + (static_cast<unsigned>(row) * c.rsb + cc * 16u));
        }
        c.next();
    }
    // the tiles held in kreg / vreg (fetched by issue_next) into LDS
    __device__ __forceinline__ void store_held_k(unsigned char* Ks) {
        static_assert(!ROPE_K, "the walk stores K as fetched");
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (EXACT || idx < G::NCH)
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = row < k_rows ? kreg[i] : u32x4{0, 0, 0, 0};
        }
    }
    __device__ __forceinline__ void store_held_v(unsigned char* Vs) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (EXACT || idx < G::NCH)
                *reinterpret_cast<u32x4*>(Vs + row * G::V_STRIDE + cc * 16) = row < v_rows ? vreg[i] : u32x4{0, 0, 0, 0};
        }
    }

    // WHICH: 0 = K tile t into kreg, 1 = V tile t into vreg
    template <int WHICH>
    __device__ __forceinline__ void issue(int t) {
        u32x4 (&reg)[NLD] = WHICH == 0 ? kreg : vreg;
        const bool pre = plan.in_prefix(t);
        const int j0 = plan.j0(t);
        const int nvalid = plan.limit(t) - j0;   // rows of this tile that exist
        // uniform base pointer of the tile plus a fixed per-thread byte offset
        const unsigned rsb = static_cast<unsigned>(pre ? (WHICH == 0 ? p.kp_rs : p.vp_rs) : (WHICH == 0 ? p.k_rs : p.v_rs)) * 2u;
        const unsigned char* base = pre ? (WHICH == 0 ? kp_base : vp_base) + static_cast<unsigned long>(j0) * rsb
                                        : (WHICH == 0 ? k_base : v_base) + static_cast<unsigned long>(j0 - p.Lp) * rsb;
        // Rows past the end of the segment are read from its last row (always valid memory) and
        // replaced by zeros when the tile is written to LDS: no branch and no register
        // initialisation stands between the loads, so they all go out back to back.
        const int last = min(nvalid, kBN) - 1;
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = min(idx / G::CPR, last);
            const int cc = idx % G::CPR;
            if (EXACT || idx < G::NCH) reg[i] = *reinterpret_cast<const u32x4*>(base + (static_cast<unsigned>(row) * rsb + cc * 16u));
        }
    }
    __device__ __forceinline__ void store_k(int t, unsigned char* Ks) {
        // The rotation tables are fetched here rather than with the tile: they are L2 hits shared by
        // every head, and holding them across the MFMA section would cost 8 registers per chunk
        // exactly where pressure peaks. Prefix rows are stored already rotated.
        f32x4 creg[ROPE_K ? NLD : 1], sreg[ROPE_K ? NLD : 1];
        const int nvalid_k = plan.limit(t) - plan.j0(t);
        bool rot = false;
        if constexpr (ROPE_K) {
            rot = !plan.in_prefix(t);
            if (rot) {
                const int jr0 = plan.j0(t) - p.Lp;
                const int nvalid = plan.limit(t) - plan.j0(t);
#pragma unroll
                for (int i = 0; i < NLD; ++i) {
                    const int idx = tid + NT * i;
                    const int row = idx / G::CPR;
                    const int cc = idx - row * G::CPR;
                    creg[i] = f32x4{1.f, 1.f, 1.f, 1.f};
                    sreg[i] = f32x4{0.f, 0.f, 0.f, 0.f};
                    if ((EXACT || idx < G::NCH) && row < nvalid) {
                        creg[i] = *reinterpret_cast<const f32x4*>(p.cos_k + static_cast<long>(jr0 + row) * (D / 2) + cc * 4);
                        sreg[i] = *reinterpret_cast<const f32x4*>(p.sin_k + static_cast<long>(jr0 + row) * (D / 2) + cc * 4);
                    }
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
                if constexpr (ROPE_K) { if (rot) kk = rope_chunk<T>(kk, creg[i], sreg[i]); }
                if (row >= nvalid_k) kk = u32x4{0, 0, 0, 0};
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = kk;
            }
        }
    }
    __device__ __forceinline__ void store_v(int t, unsigned char* Vs) {
        const int nvalid = plan.limit(t) - plan.j0(t);
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = tid + NT * i;
            const int row = idx / G::CPR;
            const int cc = idx - row * G::CPR;
            if (EXACT || idx < G::NCH)
                *reinterpret_cast<u32x4*>(Vs + row * G::V_STRIDE + cc * 16) = row < nvalid ? vreg[i] : u32x4{0, 0, 0, 0};
        }
    }
};

// The same walk for launches that consist of whole 64-row tiles of one segment (no cached prefix, no ragged end): the
// base address of the next tile advances in scalar registers and this thread's byte offsets inside a tile (global and
// LDS) are computed once, so a load is one instruction with a scalar base and a fixed vector offset, a store has no
// select, and whether a thread takes part in round i is the same for its whole wavefront (a scalar branch).
template <typename T, int D, int NT>
struct DenseMover {
    using G = HeadGeo<D>;
    static constexpr int NLD = (G::NCH + NT - 1) / NT;
    static_assert(G::NCH % 64 == 0, "rounds end on wavefront boundaries");
    const unsigned char* kptr; const unsigned char* vptr;   // next tile to fetch
    unsigned k_tile_bytes, v_tile_bytes;
    int wave;
    unsigned kgo[NLD], vgo[NLD];    // byte offsets of this thread's chunks inside a tile in memory
    unsigned klo[NLD], vlo[NLD];    // ... and inside the LDS tile
    u32x4 kreg[NLD], vreg[NLD];
    __device__ __forceinline__ DenseMover(const unsigned char* k_base, long k_rs, const unsigned char* v_base, long v_rs, int tid, int wave_)
        : kptr(k_base), vptr(v_base), k_tile_bytes(static_cast<unsigned>(k_rs) * 2u * kBN), v_tile_bytes(static_cast<unsigned>(v_rs) * 2u * kBN), wave(wave_) {
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int idx = min(tid + NT * i, G::NCH - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            kgo[i] = static_cast<unsigned>(row) * (static_cast<unsigned>(k_rs) * 2u) + cc * 16u;
            vgo[i] = static_cast<unsigned>(row) * (static_cast<unsigned>(v_rs) * 2u) + cc * 16u;
            klo[i] = row * G::K_STRIDE + cc * 16;
            vlo[i] = row * G::V_STRIDE + cc * 16;
        }
    }
    __device__ __forceinline__ bool mine(int i) const { return wave * 64 + NT * i < G::NCH; }
    __device__ __forceinline__ void start_walk() {}
    template <int WHICH>
    __device__ __forceinline__ void issue_next() {
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            if (mine(i)) {
                if constexpr (WHICH == 0) kreg[i] = *reinterpret_cast<const u32x4*>(kptr + kgo[i]);
                else vreg[i] = *reinterpret_cast<const u32x4*>(vptr + vgo[i]);
            }
        if constexpr (WHICH == 0) kptr += k_tile_bytes; else vptr += v_tile_bytes;
    }
    __device__ __forceinline__ void store_held_k(unsigned char* Ks) {
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            if (mine(i)) *reinterpret_cast<u32x4*>(Ks + klo[i]) = kreg[i];
    }
    __device__ __forceinline__ void store_held_v(unsigned char* Vs) {
#pragma unroll
        for (int i = 0; i < NLD; ++i)
            if (mine(i)) *reinterpret_cast<u32x4*>(Vs + vlo[i]) = vreg[i];
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

constexpr int kThreads8 = 512;
template <int D> constexpr int lds_bytes_8() {
    using G = HeadGeo<D>;
    const int kv = 2 * (G::K_BYTES + G::V_BYTES);
    const int o = 256 * G::O_STRIDE;
    return kv > o ? kv : o;
}

}  // namespace sdpa
}  // namespace mi
