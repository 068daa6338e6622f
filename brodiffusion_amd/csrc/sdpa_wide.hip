// Softmax attention for head dimensions 256, 384 and 512 on gfx950: the single wide head of a VAE mid-block
// (src/vae.cpp:259-277: one head over all 512 channels of a 64 x 64 latent; src/vae_qwenimage.cpp:322-340: 384 channels),
// through the same entry point as every other head dimension.
//
// At these widths the output accumulator of a query row (head_dim floats per lane pair) no longer fits the registers of one
// wavefront, so the head dimension is dealt out to the four wavefronts of a work group instead of the query rows: all four
// work on the SAME 32 query rows, wavefront w owns elements [w D/4, (w+1) D/4) of the head dimension. Per 64-key tile
//   1. every wavefront multiplies its quarter of the contraction: a partial score tile (K Q^T over D/4 elements);
//   2. the four partial tiles meet in LDS and every wavefront adds them in the same fixed order, so all four hold
//      bit-identical scores and run the same online softmax (same reference, same denominator, same P);
//   3. every wavefront multiplies P with its quarter of V's columns into its quarter of the output.
// K and V tiles go through registers into padded LDS, single buffered: the operator runs once per image on a few thousand
// tokens, so the kernel is written for clarity, not for the last microsecond. Masks work as everywhere (per-row visible
// key interval, kv_valid_len, key mask); cached prefixes, logit bias, lse output, packed sequences and K rotated tile by
// tile are not offered at these widths (K rotated into a scratch and Q rotated on load are).
#include "sdpa_tiles.h"

namespace mi {
namespace {

using namespace sdpa;

constexpr int kWideThreads = 256;
constexpr int kWideRows = 32;     // query rows per work group

template <int D> struct WideGeo {
    using G = HeadGeo<D>;
    static constexpr int DW = D / 4;                 // head-dim elements per wavefront
    static constexpr int KCW = DW / 16;              // its 16-element contraction chunks
    static constexpr int VBW = DW / 32;              // its 32-row blocks of O^T
    static constexpr int EX_BYTES = 4 * 2 * 16 * 64 * 4;   // four partial score tiles (2 blocks x 16 registers x 64 lanes, FP32)
    static constexpr int Q_BYTES = kWideRows * G::O_STRIDE;
    // the K tile's space also takes the staged Q rows (before the key loop), the partial score tiles (after K has been
    // read) and the staged output (after the loop)
    static constexpr int A_BYTES = G::K_BYTES > EX_BYTES ? (G::K_BYTES > Q_BYTES ? G::K_BYTES : Q_BYTES) : (EX_BYTES > Q_BYTES ? EX_BYTES : Q_BYTES);
    static constexpr int LDS_BYTES = A_BYTES + G::V_BYTES + kBN * 4;
    static_assert(D % 128 == 0, "four wavefronts with whole 32-row blocks each");
    static_assert(LDS_BYTES <= 160 * 1024, "one work group must fit the LDS of a compute unit");
};

template <typename T, int D>
__global__ void __launch_bounds__(kWideThreads) sdpa_wide_kernel(const SdpaDev p, int n_q_tiles) {
    using G = HeadGeo<D>;
    using W = WideGeo<D>;
    using GW = HeadGeo<W::DW>;            // softmax_tile rescales an accumulator of this many blocks
    using V8 = typename Mma<T>::v8;
    static_assert(GW::VB == W::VBW, "accumulator blocks per wavefront");
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    unsigned char* const Ks = smem;
    unsigned char* const Vs = smem + W::A_BYTES;
    float* const Ms = reinterpret_cast<float*>(Vs + G::V_BYTES);
    float* const Ex = reinterpret_cast<float*>(smem);

    const int bh = static_cast<int>(blockIdx.x) / n_q_tiles;
    const int qt = static_cast<int>(blockIdx.x) - bh * n_q_tiles;
    const int h = bh % p.H, b = bh / p.H;
    const int hk = h / p.kv_group;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int lane = tid & 63, lq = lane & 31, lh = lane >> 5;
    const int q0 = qt * kWideRows;
    const int qrow = q0 + lq;                         // every wavefront holds the same 32 rows
    const bool qvalid = qrow < p.Lq;
    const int d_w = wave * W::DW;                     // first head-dim element of this wavefront
    const T* const q_base = static_cast<const T*>(p.q) + b * p.q_bs + h * D;
    T* const o_base = static_cast<T*>(p.o) + b * p.o_bs + h * D;
    const unsigned char* const k_base = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.k) + b * p.k_bs + hk * D);
    const unsigned char* const v_base = reinterpret_cast<const unsigned char*>(static_cast<const T*>(p.v) + b * p.v_bs + hk * D);
    const float* const key_mask = p.key_mask ? p.key_mask + b * p.key_mask_bs : nullptr;

    int lo, hi;
    row_interval(p, b, qrow, qvalid, lo, hi);
    const WaveExtent we = wave_extent(lo, hi);        // the same in all four wavefronts

    // this wavefront's share of the Q fragments (RoPE, if any, applied while the rows are staged)
    stage_q_tile<T, D, kWideThreads, kWideRows>(smem, p, q_base, q0, tid);
    __syncthreads();
    V8 qf[W::KCW];
#pragma unroll
    for (int c = 0; c < W::KCW; ++c)
        qf[c] = __builtin_bit_cast(V8, *reinterpret_cast<const u32x4*>(smem + lq * G::O_STRIDE + (d_w + 16 * c + 8 * lh) * 2));
    __syncthreads();

    f32x16 oacc[W::VBW];
#pragma unroll
    for (int vb = 0; vb < W::VBW; ++vb)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[vb][e] = 0.f;
    SoftmaxState st;
    const float cl2 = p.scale_log2;
    const float lazy_raw = kLazyLog2 / cl2;

    const int t_begin = we.lo_min == 0x7fffffff ? 0 : we.lo_min / kBN;
    const int t_end = we.lo_min == 0x7fffffff ? 0 : (we.hi_max + kBN - 1) / kBN;
    const unsigned k_rsb = static_cast<unsigned>(p.k_rs) * 2u, v_rsb = static_cast<unsigned>(p.v_rs) * 2u;
    const int trow = (lane & 15) >> 2;
    const int tcol = 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

    for (int t = t_begin; t < t_end; ++t) {
        const int j0 = t * kBN;
        // ── K and V rows [j0, j0 + 64) into LDS; rows past the last key repeat it and are stored as zeros ──
        {
            const int last = min(p.Lk - j0, kBN) - 1;
            constexpr int NLD = G::NCH / kWideThreads;     // 16-byte pieces per thread and operand (D / 8 pieces per row)
            static_assert(G::NCH % kWideThreads == 0, "whole pieces per thread");
#pragma unroll 4
            for (int i = 0; i < NLD; ++i) {
                const int idx = tid + kWideThreads * i;
                const int row = idx / G::CPR, cc = idx - row * G::CPR;
                const unsigned long src_row = static_cast<unsigned long>(j0 + min(row, last));
                u32x4 kv = *reinterpret_cast<const u32x4*>(k_base + src_row * k_rsb + cc * 16u);
                u32x4 vv = *reinterpret_cast<const u32x4*>(v_base + src_row * v_rsb + cc * 16u);
                if (row > last) { kv = u32x4{0, 0, 0, 0}; vv = u32x4{0, 0, 0, 0}; }
                *reinterpret_cast<u32x4*>(Ks + row * G::K_STRIDE + cc * 16) = kv;
                *reinterpret_cast<u32x4*>(Vs + row * G::V_STRIDE + cc * 16) = vv;
            }
            if (key_mask && tid < kBN) Ms[tid] = j0 + tid < p.Lk ? key_mask[j0 + tid] : 0.f;
        }
        __syncthreads();

        // ── 1. partial scores over this wavefront's quarter of the head dimension ──
        f32x16 sacc[2];
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
#pragma unroll
            for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
#pragma unroll
            for (int c = 0; c < W::KCW; ++c) {
                const u32x4 a = *reinterpret_cast<const u32x4*>(Ks + (32 * kb + lq) * G::K_STRIDE + (d_w + 16 * c + 8 * lh) * 2);
                sacc[kb] = Mma<T>::run(__builtin_bit_cast(V8, a), qf[c], sacc[kb]);
            }
        }
        __syncthreads();                               // every wavefront has read the K tile: its space takes the partial tiles
        // ── 2. the four partial tiles, added in wavefront order by everybody ──
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) Ex[((wave * 2 + kb) * 16 + e) * 64 + lane] = sacc[kb][e];
        __syncthreads();
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                float s = Ex[((0 * 2 + kb) * 16 + e) * 64 + lane];
#pragma unroll
                for (int w = 1; w < 4; ++w) s += Ex[((w * 2 + kb) * 16 + e) * 64 + lane];
                sacc[kb][e] = s;
            }
        // ── softmax (identical in the four wavefronts), then 3. this wavefront's quarter of O^T += V^T P^T ──
        V8 pf[4];
        const bool interior = (j0 >= we.lo_max) && (j0 + kBN <= min(we.hi_min, p.Lk)) && (key_mask == nullptr);
        softmax_tile<T, W::DW>(sacc, pf, oacc, st, cl2, lazy_raw, !interior, j0, lo, min(hi, p.Lk), lh, key_mask ? Ms : nullptr);
#pragma unroll
        for (int c4 = 0; c4 < 4; ++c4)
#pragma unroll
            for (int vb = 0; vb < W::VBW; ++vb) {
                const unsigned char* vptr = Vs + (16 * c4 + 4 * lh + trow) * G::V_STRIDE + (d_w + 32 * vb + tcol) * 2;
                const s16x4 v_lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vptr));
                const s16x4 v_hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4*)(vptr + 8 * G::V_STRIDE));
                const s16x8 a = __builtin_shufflevector(v_lo, v_hi, 0, 1, 2, 3, 4, 5, 6, 7);
                oacc[vb] = Mma<T>::run(__builtin_bit_cast(V8, a), pf[c4], oacc[vb]);
            }
        __syncthreads();                               // tiles and partial scores are used up
    }

    const float l_tot = exchange_sum(st.l);
    const float inv = row_inverse(l_tot);
    {
        typedef T t4 __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int vb = 0; vb < W::VBW; ++vb)
#pragma unroll
            for (int bb = 0; bb < 4; ++bb) {
                t4 ov;
#pragma unroll
                for (int i = 0; i < 4; ++i) ov[i] = static_cast<T>(oacc[vb][4 * bb + i] * inv);
                *reinterpret_cast<t4*>(smem + lq * G::O_STRIDE + (d_w + 32 * vb + 8 * bb + 4 * lh) * 2) = ov;
            }
    }
    __syncthreads();
    write_output<T, D, kWideThreads>(smem, o_base, p.o_rs, q0, p.Lq, kWideRows, tid);
}

template <typename T, int D>
int launch_wide_d(const SdpaDev& p, hipStream_t stream) {
    const int n_q_tiles = (p.Lq + kWideRows - 1) / kWideRows;
    const long blocks = static_cast<long>(p.B) * p.H * n_q_tiles;
    if (blocks > 0x7fffffffL) return fail("mi_sdpa_forward: problem too large for one launch");
    static thread_local bool raised = false;
    if (!raised) {
        MI_HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&sdpa_wide_kernel<T, D>), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         WideGeo<D>::LDS_BYTES));
        raised = true;
    }
    hipLaunchKernelGGL((sdpa_wide_kernel<T, D>), dim3(static_cast<unsigned>(blocks)), dim3(kWideThreads), WideGeo<D>::LDS_BYTES, stream, p, n_q_tiles);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("sdpa_wide launch: %s", hipGetErrorString(e));
    return 0;
}

}  // namespace

bool sdpa_wide_head(int head_dim) { return head_dim == 256 || head_dim == 384 || head_dim == 512; }

int launch_sdpa_wide(const SdpaDev& p, int dtype, int head_dim, hipStream_t stream) {
    const char* what = nullptr;
    if (p.Lp > 0) what = "a cached prefix";
    else if (p.cos_k) what = "K rotated tile by tile (lend rope_k_scratch)";
    else if (p.bias) what = "a logit bias";
    else if (p.lse) what = "lse_out";
    else if (p.cu_q) what = "packed variable-length sequences";
    if (what) return fail("mi_sdpa_forward: head_dim %d does not offer %s", head_dim, what);
    if (dtype != MI_DTYPE_BF16 && dtype != MI_DTYPE_F16) return fail("mi_sdpa_forward: dtype %d not supported (fp16 = 1, bf16 = 2)", dtype);
    const bool bf = dtype == MI_DTYPE_BF16;
    switch (head_dim) {
        case 256: return bf ? launch_wide_d<__bf16, 256>(p, stream) : launch_wide_d<_Float16, 256>(p, stream);
        case 384: return bf ? launch_wide_d<__bf16, 384>(p, stream) : launch_wide_d<_Float16, 384>(p, stream);
        case 512: return bf ? launch_wide_d<__bf16, 512>(p, stream) : launch_wide_d<_Float16, 512>(p, stream);
        default: return fail("mi_sdpa_forward: head_dim %d has no kernel", head_dim);
    }
}

}  // namespace mi
