// Head-averaged attention map for traced forwards: map[q][k] = (1/H) sum_h softmax_h(q, k), FP32, for batch 1
// (0 in the columns of keys that a key mask hides).
//
// The flash kernels never materialise the softmax; a traced forward wants it averaged over heads. The attention
// launch leaves the base-2 log of every row's denominator (lse, per head and query row); this kernel recomputes the
// scores tile by tile and turns them into probabilities with it. One work group owns a (128 query rows x 64 keys)
// tile of the map and loops over the heads, so every map element is accumulated in one register and written once —
// no atomics, deterministic. Scores are computed transposed (S^T = K Q^T, as in the attention kernels): a lane owns
// one query row, so lse and the bias row are per-lane scalars, and holds 4 consecutive keys per accumulator group,
// which leave as 16-byte stores.
// Per head a work group reads its K tile (64 x d) and its Q rows (128 x d), both through LDS, one head ahead of the products.
#include "sdpa_common.h"

namespace mi {
namespace {

using namespace sdpa;

constexpr int kMapThreads = 256;
constexpr int kMapRows = 128;

template <typename T, int D>
__global__ void __launch_bounds__(kMapThreads, 2) attn_map_kernel(const MapDev p) {
    using G = HeadGeo<D>;
    using V8 = typename Mma<T>::v8;
    __shared__ __attribute__((aligned(16))) unsigned char Ks2[2][G::K_BYTES];   // K tiles of two consecutive heads
    __shared__ __attribute__((aligned(16))) unsigned char Qs4[kMapThreads / 64][32 * G::K_STRIDE];   // per wavefront: its 32 query rows

    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63, lq = lane & 31, lh = lane >> 5;
    const int j0 = static_cast<int>(blockIdx.x) * kBN;
    const int q0 = static_cast<int>(blockIdx.y) * kMapRows;
    const int qrow = q0 + wave * 32 + lq;
    const bool qvalid = qrow < p.Lq;
    const int qr = qvalid ? qrow : p.Lq - 1;   // rows past the end repeat the last one and are never stored
    const float* const bias_row = (p.bias && qvalid && qrow >= p.bias_q0 && j0 < p.bias_cols)
                                      ? p.bias + static_cast<long>(qrow - p.bias_q0) * p.bias_rs : nullptr;
    constexpr float kLog2e = 1.4426950408889634f;

    // the zero pad of the head dimension (columns D .. DK-1) is written once; data chunks are rewritten per head
    for (int i = tid; i < 2 * G::K_BYTES / 16; i += kMapThreads) reinterpret_cast<u32x4*>(&Ks2[0][0])[i] = u32x4{0u, 0u, 0u, 0u};

    f32x16 avg[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) avg[kb][e] = 0.f;
    // What is added to the scaled score of this lane's key (kb, e), the same for every head, fetched once: the logit
    // bias in exponent units, 0 without one, -inf for keys past the end of the sequence or hidden by the key mask
    // (their probability is then 0). The head loop is left with one fused multiply-add per score and no condition.
    f32x16 pre[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int key = j0 + 32 * kb + 8 * (e >> 2) + 4 * lh + (e & 3);
            float v = 0.f;
            if (bias_row && key < p.bias_cols) v = bias_row[key] * kLog2e;
            if (key >= p.Lk || (p.key_mask != nullptr && p.key_mask[min(key, p.Lk - 1)] == 0.f)) v = kNegInf;
            pre[kb][e] = v;
        }

    // One head's operands, requested one head ahead so that their latency passes under the previous head's products:
    // the K tile (64 x d, a few 16-byte chunks per thread, to LDS when their turn comes; rows past the last key repeat
    // it and are stored as zeros) and the wavefront's 32 query rows, fetched with full-row coalescing (a lane-per-row
    // fetch of the B operands touches 32 cache lines per instruction and made the address path the busiest unit) and
    // passed through a slice of LDS that only this wavefront uses, from which every lane picks its row's fragments
    // (8 contraction elements at 16 c + 8 lh).
    const T* const qg = static_cast<const T*>(p.q);
    const T* const kg = static_cast<const T*>(p.k);
    constexpr int NKC = (kBN * G::CPR + kMapThreads - 1) / kMapThreads;
    u32x4 kreg[NKC];
    constexpr int NQC = (32 * G::CPR + 63) / 64;
    u32x4 qn[NQC];
    float lse_n = 0.f;
    unsigned char* const Qs = Qs4[wave];
    const int wq0 = q0 + wave * 32;
    for (int i = lane; i < 32 * G::K_STRIDE / 16; i += 64) reinterpret_cast<u32x4*>(Qs)[i] = u32x4{0u, 0u, 0u, 0u};   // (the pad columns stay zero)
    auto request = [&](int h) {
#pragma unroll
        for (int i = 0; i < NKC; ++i) {
            const int idx = min(tid + kMapThreads * i, kBN * G::CPR - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            kreg[i] = *reinterpret_cast<const u32x4*>(kg + static_cast<long>(min(j0 + row, p.Lk - 1)) * p.k_rs + h * D + cc * 8);
        }
#pragma unroll
        for (int i = 0; i < NQC; ++i) {
            const int idx = min(lane + 64 * i, 32 * G::CPR - 1);
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            qn[i] = *reinterpret_cast<const u32x4*>(qg + static_cast<long>(min(wq0 + row, p.Lq - 1)) * p.q_rs + h * D + cc * 8);
        }
        lse_n = p.lse[static_cast<long>(h) * p.Lq + qr];
    };
    request(0);
    __syncthreads();   // the zeroed pads are in place before the first tile's chunks land next to them
    for (int h = 0; h < p.H; ++h) {
        unsigned char* const Ks = Ks2[h & 1];
#pragma unroll
        for (int i = 0; i < NKC; ++i) {
            const int idx = tid + kMapThreads * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < kBN * G::CPR)
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = j0 + row < p.Lk ? kreg[i] : u32x4{0u, 0u, 0u, 0u};
        }
#pragma unroll
        for (int i = 0; i < NQC; ++i) {
            const int idx = lane + 64 * i;
            const int row = idx / G::CPR, cc = idx - row * G::CPR;
            if (idx < 32 * G::CPR) *reinterpret_cast<u32x4*>(Qs + row * G::K_STRIDE + cc * 16) = qn[i];
        }
        const float lse = lse_n;
        // one barrier per head: this head's tile is complete, and every wavefront has finished the head before last,
        // whose buffer the next head's chunks will overwrite
        __syncthreads();
        V8 qf[G::KC];
#pragma unroll
        for (int c = 0; c < G::KC; ++c) qf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(Qs + lq * G::K_STRIDE + (2 * c + lh) * 16));
        if (h + 1 < p.H) request(h + 1);
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
#pragma unroll
            for (int c = 0; c < G::KC; ++c) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(Ks + (32 * kb + lq) * G::K_STRIDE + (2 * c + lh) * 16);
                sacc[kb] = Mma<T>::run(__builtin_bit_cast(V8, a), qf[c], sacc[kb]);
            }
        }
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                avg[kb][e] += __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[kb][e], p.scale_log2, pre[kb][e]) - lse);
            }
    }

    if (!qvalid) return;
    const float inv_h = 1.0f / static_cast<float>(p.H);
    float* const row = p.map + static_cast<long>(qrow) * p.map_rs;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int bb = 0; bb < 4; ++bb) {
            const int key = j0 + 32 * kb + 8 * bb + 4 * lh;
            if (key + 3 < p.Lk && (p.map_rs & 3) == 0) {
                *reinterpret_cast<f32x4*>(row + key) = f32x4{avg[kb][4 * bb] * inv_h, avg[kb][4 * bb + 1] * inv_h,
                                                             avg[kb][4 * bb + 2] * inv_h, avg[kb][4 * bb + 3] * inv_h};
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    if (key + i < p.Lk) row[key + i] = avg[kb][4 * bb + i] * inv_h;
            }
        }
}

template <typename T, int D>
int launch_map_d(const MapDev& p, hipStream_t st) {
    const dim3 grid((p.Lk + kBN - 1) / kBN, (p.Lq + kMapRows - 1) / kMapRows);
    hipLaunchKernelGGL((attn_map_kernel<T, D>), grid, dim3(kMapThreads), 0, st, p);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("mi_attention_map_avg launch: %s", hipGetErrorString(e));
    return 0;
}

template <typename T>
int launch_map_t(const MapDev& p, int head_dim, hipStream_t st) {
    switch (head_dim) {
        case 40: return launch_map_d<T, 40>(p, st);
        case 64: return launch_map_d<T, 64>(p, st);
        case 72: return launch_map_d<T, 72>(p, st);
        case 80: return launch_map_d<T, 80>(p, st);
        case 96: return launch_map_d<T, 96>(p, st);
        case 112: return launch_map_d<T, 112>(p, st);
        case 128: return launch_map_d<T, 128>(p, st);
        case 160: return launch_map_d<T, 160>(p, st);
        default: return fail("mi_attention_map_avg: head_dim %d has no kernel", head_dim);
    }
}

}  // namespace

int launch_attention_map(const MapDev& p, int dtype, int head_dim, hipStream_t stream) {
    if (dtype == MI_DTYPE_BF16) return launch_map_t<__bf16>(p, head_dim, stream);
    if (dtype == MI_DTYPE_F16) return launch_map_t<_Float16>(p, head_dim, stream);
    return fail("mi_attention_map_avg: dtype %d not supported", dtype);
}

}  // namespace mi
