// Internal declarations shared by the translation units of libmi_attention.so.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>

#include "mi_attention.h"

namespace mi {

// Records the message mi_last_error() returns for this thread; always returns -1.
int fail(const char* fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();
hipStream_t resolve_stream(void* s);
// Compute units of the current device (cached per thread; 256 if the query fails).
int device_cu_count();

#define MI_HIP_CHECK(expr)                                                          \
    do {                                                                            \
        hipError_t _e = (expr);                                                     \
        if (_e != hipSuccess) return ::mi::fail("%s: %s", #expr, hipGetErrorString(_e)); \
    } while (0)

// Split of the last, partly filled round of an unmasked attention launch.
//
// A launch of n_blocks equal query tiles on a GPU that runs n_cu work groups at a time takes ceil(n_blocks / n_cu)
// rounds even when the last round fills only part of the GPU (432 tiles on 256 compute units: 2 rounds for 1.69
// rounds of work). With the split, the tiles of the full rounds are processed whole and the tiles of the last round
// are cut along the KEY axis into as many equal pieces as there are work-group slots; a piece covers the end of one
// tile and the start of the next, each part leaves a normalised partial output plus its softmax statistics in a
// scratch slot, and a small second kernel merges the parts of every tile. Everything is done per XCD group (work
// groups whose id is g mod 8 share an L2): group g owns the logical tiles [g*chunk, (g+1)*chunk) and cu_g work-group
// slots. All quantities are counted in key tiles of 64 keys ("steps"); T is the number of steps of one query tile.
struct SplitGeo {
    int enabled;
    int T, chunk, n_blocks, cu_g;
    int max_tail;   // most tail tiles of any group
    int max_parts;  // partial slots per tail tile
    static constexpr int kMinPiece = 8;   // shortest piece worth a work group of its own, in steps
    __host__ __device__ int tiles_of(int g) const { const int n = n_blocks - g * chunk; return n < 0 ? 0 : (n > chunk ? chunk : n); }
    __host__ __device__ int full_of(int g) const { return tiles_of(g) / cu_g * cu_g; }
    __host__ __device__ int tail_of(int g) const { return tiles_of(g) - full_of(g); }
    // pieces the tail steps S of a group are cut into
    __host__ __device__ int pieces_for(int S) const {
        if (S <= 0) return 0;
        const int np = S / kMinPiece;
        return np < 1 ? 1 : (np > cu_g ? cu_g : np);
    }
    // piece c of np covers tail steps [piece_begin(c), piece_begin(c + 1))
    __host__ __device__ static int piece_begin(int c, int S, int np) { return static_cast<int>(static_cast<long>(c) * S / np); }
    // the piece that holds tail step x
    __host__ __device__ static int piece_of(int x, int S, int np) { return static_cast<int>((static_cast<long>(x + 1) * np + S - 1) / S) - 1; }
    // bytes of one partial slot: 256 rows of head_dim 16-bit values, then 256 references and 256 denominators (FP32)
    __host__ __device__ static long slot_bytes(int head_dim) { return 256L * head_dim * 2 + 256L * 8; }
};

// Device-side view of one softmax-attention launch. Strides in elements.
struct SdpaDev {
    const void* q; const void* k; const void* v; void* o;
    const void* kp; const void* vp;
    int B, H, Lq, Lk, Lp;  // Lk = Lp + fresh rows
    int kv_group;          // query heads per K/V head
    long q_rs, q_bs, k_rs, k_bs, v_rs, v_bs, o_rs, o_bs, kp_rs, kp_bs, vp_rs, vp_bs;
    float scale_log2;      // scale * log2(e)
    int mask_mode, q_offset, window;
    const int* kv_valid_len;
    const float* key_mask; long key_mask_bs;
    int n_seg;
    int seg_q_end[MI_MAX_SEGMENTS];
    int seg_k_end[MI_MAX_SEGMENTS];
    int seg_causal[MI_MAX_SEGMENTS];
    const float* cos_q; const float* sin_q;
    const float* cos_k; const float* sin_k;
    int rope_split;               // 0: adjacent pairs, 1: the two halves of a head (Q only: K then arrives rotated)
    int n_q_tiles; int n_blocks;  // logical work items = B*H*n_q_tiles
    // additive logit bias (natural-log units, added to the scaled score) for query rows >= bias_q0 and keys < bias_cols
    const float* bias; int bias_q0, bias_cols; long bias_rs;
    int bias_vec_ok;              // bias base 16-byte aligned and bias_rs a multiple of 4: rows can be read 4 floats at a time
    float inv_scale;              // 1 / scale: the bias in units of the raw dot product
    const int* cu_q; const int* cu_k;   // packed variable-length sequences: [B + 1] row offsets, or null
    float* lse;                   // [B][H][Lq] base-2 log of the softmax denominator in exponent units, or null
    int prefix_scaled;            // the rows of the cached prefix carry factors: K rows pk_scale * pk_row[j], V rows pv_scale * pv_row[j]
    float pk_scale, pv_scale;
    const float* pk_row; const float* pv_row;   // [Lp] or null
    int kbits_off;                // byte offset in dynamic LDS of the key-visibility words (256-row kernels with a key mask)
    SplitGeo split;               // enabled != 0: split the last round along the key axis
    unsigned char* split_scratch; // partial slots, [8 groups][max_tail][max_parts] of SplitGeo::slot_bytes
    size_t split_scratch_bytes;   // what the caller lent
};

// One rotation, written with explicit fused multiply-adds so that every kernel that rotates
// (stand-alone pass, Q load, K tile load) rounds identically: (a + ib)(c + is).
__device__ __forceinline__ float rope_re(float a, float b, float c, float s) { return __builtin_fmaf(a, c, -(b * s)); }
__device__ __forceinline__ float rope_im(float a, float b, float c, float s) { return __builtin_fmaf(a, s, b * c); }

// 0 = pick by problem size, 1 = 128-row kernel, 2 = 256-row ping-pong kernel (mi_sdpa_set_kernel_choice).
int sdpa_kernel_choice();

int launch_sdpa(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream);
// Scratch bytes with which launch_sdpa would split the last round of this launch (0: it would not split).
size_t sdpa_split_scratch_bytes(const SdpaDev& p, int dtype, int head_dim);
bool sdpa_supported(int dtype, int head_dim);
// Head dimensions 256, 384 and 512 (sdpa_wide.hip): one 32-row query tile per work group, the head dimension dealt out to its wavefronts.
bool sdpa_wide_head(int head_dim);
int launch_sdpa_wide(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream);

// Device-side view of the head-averaged attention map launch (batch 1).
struct MapDev {
    const void* q; const void* k;
    const float* lse;             // [H][Lq], as written by the attention launch
    float* map;                   // (Lq, Lk) FP32
    int H, Lq, Lk;
    long q_rs, k_rs, map_rs;
    float scale_log2;
    const float* bias; int bias_q0, bias_cols; long bias_rs;
    const float* key_mask;        // [Lk] or null
};
int launch_attention_map(const MapDev& p, int dtype, int head_dim, hipStream_t stream);

// One Y = X W^T + bias problem: X (M, K), W (N, K), Y (M, N), bias (N) or null; strides in elements.
struct LinearProblem {
    const void* x; const void* w; const void* bias; void* y;
    const float* w_scale;   // non-null: w is INT8 (N, K) with one FP32 scale per row, Y = (X Wq^T) * scale + bias
    int M, N, K;
    long ldx, ldw, ldy;
};
constexpr int kMaxLinearProblems = 3;
struct LinearBatch { LinearProblem p[kMaxLinearProblems]; };
// Validates and launches up to kMaxLinearProblems problems as one grid.
// geglu: problem 0 has W (2 N, K) and bias (2 N), value half first; Y (M, N) = value * gelu_exact(gate).
int launch_linear(const LinearBatch& batch, int n_problems, int dtype, hipStream_t stream, bool geglu = false);
// The 256 x 256-tile form with LDS-DMA operand rings (linear_dma.hip): whether it takes a validated launch, and the launch.
bool linear_dma_takes(const LinearBatch& batch, int n_problems, int n_cu);
int launch_linear_dma(const LinearBatch& batch, int n_problems, int dtype, hipStream_t stream);

}  // namespace mi
