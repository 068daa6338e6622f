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
    int n_q_tiles; int n_blocks;  // logical work items = B*H*n_q_tiles
};

// One rotation, written with explicit fused multiply-adds so that every kernel that rotates
// (stand-alone pass, Q load, K tile load) rounds identically: (a + ib)(c + is).
__device__ __forceinline__ float rope_re(float a, float b, float c, float s) { return __builtin_fmaf(a, c, -(b * s)); }
__device__ __forceinline__ float rope_im(float a, float b, float c, float s) { return __builtin_fmaf(a, s, b * c); }

// 0 = pick by problem size, 1 = 128-row kernel, 2 = 256-row ping-pong kernel (mi_sdpa_set_kernel_choice).
int sdpa_kernel_choice();

int launch_sdpa(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream);
bool sdpa_supported(int dtype, int head_dim);

// One Y = X W^T + bias problem: X (M, K), W (N, K), Y (M, N), bias (N) or null; strides in elements.
struct LinearProblem {
    const void* x; const void* w; const void* bias; void* y;
    int M, N, K;
    long ldx, ldw, ldy;
};
constexpr int kMaxLinearProblems = 3;
struct LinearBatch { LinearProblem p[kMaxLinearProblems]; };
// Validates and launches up to kMaxLinearProblems problems as one grid.
int launch_linear(const LinearBatch& batch, int n_problems, int dtype, hipStream_t stream);

}  // namespace mi
