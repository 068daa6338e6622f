// TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's attention math.
//
// This file is the checker that the HIP kernels are compared against. Nothing
// in the shipped library links, loads or calls it: only tests/, the smoke check
// and the bench's cpu_baseline leg may use it.
//
// Every function cites the reference file:line it follows (paths relative to the
// reference repository root). Pinning status of each function (which independent
// check fixes it) is listed here and verified by tests/test_oracle.py:
//
//   orc_torch_randn_f32        pinned: 4 known-answer vectors of tests/test_torch_rng.cpp:44-83,
//                              and bit-equality with oracle/_ref (the reference header compiled as is)
//   orc_round_bf16 / _f16      pinned: torch.bfloat16 / torch.float16 casts (library routine)
//   orc_build_axial_rope_tables pinned: closed form cos(pos * theta^(-2p/D_a)), identity text rows
//   orc_build_qwen_rope_tables pinned: closed form on hand-built position lists
//   orc_rope_apply             math pinned by norm preservation + relative-position property;
//                              PAIR CONVENTION (adjacent vs split-half) is "parity unpinned":
//                              brotensor's rope_apply source is not in the reference tree
//   orc_sdpa                   pinned: torch float64 scaled_dot_product_attention, numpy brute force,
//                              closed forms (equal keys -> mean(V), V const -> const, key permutation),
//                              masked == trimmed, block-causal == per-segment calls == dense mask.
//                              Fully masked row -> zeros follows src/dit/common.cpp:293; what
//                              brotensor's flash kernel does there is "parity unpinned".
//   orc_linear_attn_relu       pinned: quadratic-form brute force, (S,z) additivity over token chunks
//   orc_rms_norm               pinned: torch.nn.functional.rms_norm in float64, unit-RMS invariant, scale
//                              invariance; eps placement (inside the square root) follows diffusers'
//                              RMSNorm — brotensor's own is "parity unpinned"
//   orc_geglu_exact            pinned: torch.nn.functional.gelu(approximate="none") in float64, gelu(0) = 0,
//                              gelu(x) - gelu(-x) = x
//   orc_linear                 pinned: numpy float64 matmul, identity weight, one-hot rows.
//                              WHERE the fused projection operators round their intermediates
//                              (Q, K, V, attention output to the tensor dtype) is "parity unpinned":
//                              brotensor's source is not in the reference tree
//
// Build: see oracle/Makefile (g++ -O3 -fopenmp, no dependencies).

#include <algorithm>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <random>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API extern "C" __attribute__((visibility("default")))

// ─── seeded N(0,1) input generator ──────────────────────────────────────────
// Follows include/brodiffusion/detail/torch_rng.h:34-76: MT19937 seeded with the
// low 32 bits of the seed; a uniform is the low 24 bits of a draw times 2^-24;
// blocks of 16 uniforms are Box-Muller transformed in place as 8 (u1,u2) pairs
// with u1 = 1 - d[j], u2 = d[j+8]; theta is formed in double and stored as float;
// a length that is not a multiple of 16 redraws 16 fresh uniforms for the last
// 16 elements.
ORC_API int orc_torch_randn_f32(uint64_t seed, size_t n, float* out) {
    if (n < 16) return -1;  // torch_rng.h:35-38 refuses n < 16
    std::mt19937 eng(static_cast<uint32_t>(seed));
    auto uni = [&eng]() -> float {
        return static_cast<float>(eng() & 0xFFFFFFu) * (1.0f / 16777216.0f);
    };
    for (size_t i = 0; i < n; ++i) out[i] = uni();
    auto box_muller16 = [](float* d) {
        const double two_pi = 2.0 * 3.14159265358979323846;
        for (int j = 0; j < 8; ++j) {
            const float u1 = 1.0f - d[j];
            const float u2 = d[j + 8];
            const float r = std::sqrt(-2.0f * std::log(u1));
            const float th = static_cast<float>(two_pi * static_cast<double>(u2));
            d[j] = r * std::cos(th);
            d[j + 8] = r * std::sin(th);
        }
    };
    for (size_t i = 0; i + 16 <= n; i += 16) box_muller16(out + i);
    if (n % 16 != 0) {
        float* tail = out + n - 16;
        for (int j = 0; j < 16; ++j) tail[j] = uni();
        box_muller16(tail);
    }
    return 0;
}

// ─── storage-dtype rounding (round to nearest even) ─────────────────────────
// The reference canonicalises test inputs to values representable in the GPU
// dtype and feeds the same values to both sides (tests/test_fused_parity.cpp:50-61)
// and re-rounds the traced output to BF16 (src/dit/common.cpp:318-327).
static inline uint16_t f32_to_bf16_bits(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x40u);  // NaN
    const uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return static_cast<uint16_t>(u >> 16);
}
static inline float bf16_bits_to_f32(uint16_t b) {
    uint32_t u = static_cast<uint32_t>(b) << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_f16_bits(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) {  // inf / nan
        return static_cast<uint16_t>(sign | 0x7c00u | (ax > 0x7f800000u ? 0x200u : 0u));
    }
    if (ax >= 0x477ff000u) return static_cast<uint16_t>(sign | 0x7c00u);  // rounds to inf
    if (ax < 0x33000001u) return static_cast<uint16_t>(sign);             // rounds to zero
    int exp = static_cast<int>(ax >> 23) - 127;
    uint32_t man = (ax & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t half_exp;
    if (exp < -14) {  // subnormal half
        shift = 13 + (-14 - exp);
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = static_cast<uint32_t>(exp + 15);
    }
    uint32_t q = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    if (rem > halfway || (rem == halfway && (q & 1u))) ++q;
    uint32_t out;
    if (half_exp == 0) {
        out = q;  // may carry into exponent 1: still the right encoding
    } else {
        out = ((half_exp - 1) << 10) + q;  // q includes the implicit bit (0x400)
    }
    return static_cast<uint16_t>(sign | out);
}
static inline float f16_bits_to_f32(uint16_t h) {
    const uint32_t sign = (static_cast<uint32_t>(h) & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else {
            int e = -1;
            do { ++e; man <<= 1; } while ((man & 0x400u) == 0);
            man &= 0x3ffu;
            u = sign | (static_cast<uint32_t>(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

ORC_API void orc_round_bf16(float* x, size_t n) {
    for (size_t i = 0; i < n; ++i) x[i] = bf16_bits_to_f32(f32_to_bf16_bits(x[i]));
}
ORC_API void orc_round_f16(float* x, size_t n) {
    for (size_t i = 0; i < n; ++i) x[i] = f16_bits_to_f32(f32_to_f16_bits(x[i]));
}
ORC_API void orc_f32_to_bf16_bits(const float* x, size_t n, uint16_t* out) {
    for (size_t i = 0; i < n; ++i) out[i] = f32_to_bf16_bits(x[i]);
}
ORC_API void orc_f32_to_f16_bits(const float* x, size_t n, uint16_t* out) {
    for (size_t i = 0; i < n; ++i) out[i] = f32_to_f16_bits(x[i]);
}
ORC_API void orc_bf16_bits_to_f32(const uint16_t* x, size_t n, float* out) {
    for (size_t i = 0; i < n; ++i) out[i] = bf16_bits_to_f32(x[i]);
}
ORC_API void orc_f16_bits_to_f32(const uint16_t* x, size_t n, float* out) {
    for (size_t i = 0; i < n; ++i) out[i] = f16_bits_to_f32(x[i]);
}

// ─── RoPE tables ────────────────────────────────────────────────────────────
// Flux axial tables, following src/dit/common.cpp:116-184. Axis a owns a run of
// axes[a]/2 consecutive pairs; pair p of axis a has omega = theta^(-2p/axes[a])
// computed in double; text rows [0,txt_len) are the identity rotation; image token
// (i,j) at row txt_len + i*wp + j has axial position (0, i, j). Tables are
// (txt_len + hp*wp, head_dim/2) float.
ORC_API int orc_build_axial_rope_tables(int txt_len, int hp, int wp, int head_dim, const int* axes,
                                        int n_axes, float theta, float* cos_out, float* sin_out) {
    if (head_dim % 2 != 0) return -1;
    int sum = 0;
    for (int a = 0; a < n_axes; ++a) sum += axes[a];
    if (sum != head_dim) return -1;
    const int half = head_dim / 2;
    const size_t L = static_cast<size_t>(txt_len) + static_cast<size_t>(hp) * wp;
    for (size_t i = 0; i < L * half; ++i) { cos_out[i] = 1.0f; sin_out[i] = 0.0f; }
    for (int i = 0; i < hp; ++i) {
        for (int j = 0; j < wp; ++j) {
            const size_t row = static_cast<size_t>(txt_len) + static_cast<size_t>(i) * wp + j;
            const int pos[3] = {0, i, j};
            int off = 0;
            for (int a = 0; a < n_axes; ++a) {
                const int cnt = axes[a] / 2;
                if (a < 3) {
                    for (int p = 0; p < cnt; ++p) {
                        const double omega =
                            1.0 / std::pow(static_cast<double>(theta), (2.0 * p) / static_cast<double>(axes[a]));
                        const double ang = static_cast<double>(pos[a]) * omega;
                        cos_out[row * half + off + p] = static_cast<float>(std::cos(ang));
                        sin_out[row * half + off + p] = static_cast<float>(std::sin(ang));
                    }
                }
                off += cnt;
            }
        }
    }
    return 0;
}

// Qwen-Image 3-axis tables, following src/dit/qwenimage21_forward.cpp:124-200.
// seg_kind[s] = 0 text (seg_a[s] tokens), 1 image (seg_a[s] x seg_b[s] grid); the
// target image (hp x wp) is appended after the prefix. A shared position walks
// the sequence: text token -> (p,p,p), p++; image block -> frame frozen at p,
// rows/cols centred on zero (h0 = -(h - h/2)), then p += max(h,w).
// freq of pair p of axis a = theta^(-2p/axes[a]). Returns the sequence length, or
// -1; cos_out/sin_out may be null to query the length.
ORC_API int orc_build_qwen_rope_tables(const int* seg_kind, const int* seg_a, const int* seg_b, int n_seg,
                                       int hp, int wp, int head_dim, const int* axes, double theta,
                                       float* cos_out, float* sin_out) {
    if (head_dim % 2 != 0 || axes[0] + axes[1] + axes[2] != head_dim) return -1;
    const int half = head_dim / 2;
    std::vector<int> ax[3];
    int pos = 0;
    auto add_text = [&](int n) {
        for (int i = 0; i < n; ++i) { ax[0].push_back(pos); ax[1].push_back(pos); ax[2].push_back(pos); ++pos; }
    };
    auto add_image = [&](int h, int w) {
        const int frame = pos;
        const int h0 = -(h - h / 2);
        const int w0 = -(w - w / 2);
        for (int i = 0; i < h; ++i)
            for (int j = 0; j < w; ++j) { ax[0].push_back(frame); ax[1].push_back(h0 + i); ax[2].push_back(w0 + j); }
        pos += std::max(h, w);
    };
    for (int s = 0; s < n_seg; ++s) {
        if (seg_kind[s] == 0) add_text(seg_a[s]); else add_image(seg_a[s], seg_b[s]);
    }
    add_image(hp, wp);
    const int L = static_cast<int>(ax[0].size());
    if (!cos_out || !sin_out) return L;
    std::vector<double> freq(half);
    std::vector<int> pair_axis(half);
    int off = 0;
    for (int a = 0; a < 3; ++a) {
        for (int p = 0; p < axes[a] / 2; ++p) {
            freq[off + p] = std::pow(theta, -2.0 * static_cast<double>(p) / static_cast<double>(axes[a]));
            pair_axis[off + p] = a;
        }
        off += axes[a] / 2;
    }
    for (int r = 0; r < L; ++r)
        for (int p = 0; p < half; ++p) {
            const double ang = static_cast<double>(ax[pair_axis[p]][r]) * freq[p];
            cos_out[static_cast<size_t>(r) * half + p] = static_cast<float>(std::cos(ang));
            sin_out[static_cast<size_t>(r) * half + p] = static_cast<float>(std::sin(ang));
        }
    return L;
}

// ─── RoPE apply ─────────────────────────────────────────────────────────────
// Contract of bt::rope_apply(X, cos, sin, head_dim, num_heads, out) as used at
// src/dit/common.cpp:192-193 and src/dit/qwenimage21_forward.cpp:584-585: X is
// (L, H*d); tables are (L, d/2) FP32 shared by all heads; every head's d/2 pairs are
// rotated by the row's (cos, sin). brotensor's source is not in the tree, so the
// pair convention is a parameter: split_half = 0 rotates adjacent (x[2p], x[2p+1])
// (diffusers' Flux / Qwen-Image convention, the default here), split_half = 1 rotates
// (x[p], x[p + d/2]). Arithmetic in float, as a GPU rope kernel would do it.
// round_mode: 0 keep fp32, 1 round result to bf16, 2 round result to fp16 (the
// reference's rope_apply writes the tensor's dtype, src/dit/common.cpp:192).
ORC_API void orc_rope_apply(const float* x, const float* cs, const float* sn, int L, int H, int d,
                            int split_half, int round_mode, float* out) {
    const int half = d / 2;
    const size_t D = static_cast<size_t>(H) * d;
#pragma omp parallel for schedule(static)
    for (int r = 0; r < L; ++r) {
        const float* c = cs + static_cast<size_t>(r) * half;
        const float* s = sn + static_cast<size_t>(r) * half;
        for (int h = 0; h < H; ++h) {
            const float* xi = x + static_cast<size_t>(r) * D + static_cast<size_t>(h) * d;
            float* oi = out + static_cast<size_t>(r) * D + static_cast<size_t>(h) * d;
            for (int p = 0; p < half; ++p) {
                const int i0 = split_half ? p : 2 * p;
                const int i1 = split_half ? p + half : 2 * p + 1;
                const float a = xi[i0], b = xi[i1];
                float o0 = a * c[p] - b * s[p];
                float o1 = a * s[p] + b * c[p];
                if (round_mode == 1) { o0 = bf16_bits_to_f32(f32_to_bf16_bits(o0)); o1 = bf16_bits_to_f32(f32_to_bf16_bits(o1)); }
                else if (round_mode == 2) { o0 = f16_bits_to_f32(f32_to_f16_bits(o0)); o1 = f16_bits_to_f32(f32_to_f16_bits(o1)); }
                oi[i0] = o0;
                oi[i1] = o1;
            }
        }
    }
}

// ─── softmax attention ──────────────────────────────────────────────────────
// The per-head host loop of dit::joint_attention_traced, src/dit/common.cpp:246-305,
// generalised to Lq != Lk (src/dit/qwenimage21_forward.cpp:648), a key mask
// (include/brodiffusion/dit/common.h:138-139: FP32 length-Lk, 1 valid / 0 invalid) and
// a per-query visible key interval [row_lo[i], row_hi[i]) (block-causal rule,
// include/brodiffusion/dit/qwenimage21.h:31-33) or an explicit (Lq, Lk) byte mask.
//
//   scale = 1/sqrt(d) in double                      (common.cpp:246; overridable)
//   dot accumulated in double over d                 (common.cpp:273-277)
//   optional additive bias(img rows, txt keys)       (common.cpp:279-281)
//   max-subtracted softmax in double                 (common.cpp:269-293)
//   inv = denom > 0 ? 1/denom : 0  -> empty row = 0  (common.cpp:293)
//   o += float(p) * v in float, keys in order        (common.cpp:300-302)
//   attn_avg = mean over heads of p                  (common.cpp:297, 308-312)
//
// q (Lq, H*d), k/v (Lk, H*d), out (Lq, H*d) row-major, head h in columns [h*d,(h+1)*d).
// rows: optional list of n_rows query indices to compute (others untouched), for
// sampling full-size problems. Invisible keys are skipped, which is the same as
// giving them a score of -inf.
ORC_API void orc_sdpa(const float* q, const float* k, const float* v, int Lq, int Lk, int H, int d,
                      double scale, const float* key_mask, const int* row_lo, const int* row_hi,
                      const uint8_t* dense_mask, const float* bias, int bias_q0, int bias_cols,
                      const int* rows, int n_rows, float* out, float* attn_avg, int n_threads) {
    const size_t D = static_cast<size_t>(H) * d;
    if (scale <= 0.0) scale = 1.0 / std::sqrt(static_cast<double>(d));
    const int nq = rows ? n_rows : Lq;
    std::vector<double> avg;
    if (attn_avg) avg.assign(static_cast<size_t>(Lq) * Lk, 0.0);
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#endif
    const long total = static_cast<long>(H) * nq;
#pragma omp parallel
    {
        std::vector<double> s(static_cast<size_t>(Lk));
#pragma omp for schedule(dynamic, 16)
        for (long w = 0; w < total; ++w) {
            const int h = static_cast<int>(w / nq);
            const int qi = rows ? rows[w % nq] : static_cast<int>(w % nq);
            const int hd0 = h * d;
            const float* qrow = q + static_cast<size_t>(qi) * D + hd0;
            const int lo = row_lo ? std::max(row_lo[qi], 0) : 0;
            const int hi = row_hi ? std::min(row_hi[qi], Lk) : Lk;
            const uint8_t* mrow = dense_mask ? dense_mask + static_cast<size_t>(qi) * Lk : nullptr;
            const float* brow = (bias && qi >= bias_q0) ? bias + static_cast<size_t>(qi - bias_q0) * bias_cols : nullptr;
            double smax = -std::numeric_limits<double>::infinity();
            for (int kk = 0; kk < Lk; ++kk) {
                const bool vis = kk >= lo && kk < hi && (!key_mask || key_mask[kk] != 0.0f) && (!mrow || mrow[kk]);
                if (!vis) { s[kk] = -std::numeric_limits<double>::infinity(); continue; }
                const float* krow = k + static_cast<size_t>(kk) * D + hd0;
                double dot = 0.0;
                for (int c = 0; c < d; ++c) dot += static_cast<double>(qrow[c]) * static_cast<double>(krow[c]);
                double sc = dot * scale;
                if (brow && kk < bias_cols) sc += static_cast<double>(brow[kk]);
                s[kk] = sc;
                if (sc > smax) smax = sc;
            }
            double denom = 0.0;
            for (int kk = 0; kk < Lk; ++kk) {
                const double e = (s[kk] == -std::numeric_limits<double>::infinity()) ? 0.0 : std::exp(s[kk] - smax);
                s[kk] = e;
                denom += e;
            }
            const double inv = denom > 0.0 ? 1.0 / denom : 0.0;
            float* orow = out + static_cast<size_t>(qi) * D + hd0;
            for (int c = 0; c < d; ++c) orow[c] = 0.0f;
            for (int kk = 0; kk < Lk; ++kk) {
                if (s[kk] == 0.0) continue;  // adds exactly nothing
                const double p = s[kk] * inv;
                const float pf = static_cast<float>(p);
                const float* vrow = v + static_cast<size_t>(kk) * D + hd0;
                for (int c = 0; c < d; ++c) orow[c] += pf * vrow[c];
            }
            if (attn_avg) {
                for (int kk = 0; kk < Lk; ++kk) {
                    const double p = s[kk] * inv;
                    if (p != 0.0) {
#pragma omp atomic
                        avg[static_cast<size_t>(qi) * Lk + kk] += p;
                    }
                }
            }
        }
    }
    if (attn_avg) {
        const float inv_h = 1.0f / static_cast<float>(H);
        for (size_t i = 0; i < avg.size(); ++i) attn_avg[i] = static_cast<float>(avg[i]) * inv_h;
    }
}

// Visible-key intervals for the mask modes of the attention entry points.
// Causal / windowed, following src/dit/qwenimage21_forward.cpp:8-13 and :658-663:
// with q_offset = Lk - Lq (or any offset) query row r attends keys [0, q_offset + r];
// window > 0 keeps only the last `window` of those.
ORC_API void orc_rows_causal(int Lq, int Lk, int q_offset, int window, int* row_lo, int* row_hi) {
    // The window is counted in positions, from the query's own position back: a query that sits beyond the last key
    // (q_offset + r >= Lk, outside what the reference ever calls) sees fewer than `window` keys, possibly none.
    for (int r = 0; r < Lq; ++r) {
        const int pos1 = q_offset + r + 1;
        const int hi = std::max(std::min(Lk, pos1), 0);
        const int lo = window > 0 ? std::max(0, pos1 - window) : 0;
        row_hi[r] = hi;
        row_lo[r] = std::min(lo, hi);
    }
}
// Block-causal segments, following include/brodiffusion/dit/qwenimage21.h:31-33 and the
// decomposition at src/dit/qwenimage21_forward.cpp:650-676: query rows
// [seg_q_end[s-1], seg_q_end[s]) see keys [0, seg_k_end[s]); a causal (text) segment
// additionally limits row r to keys [0, q_offset + r].
ORC_API void orc_rows_block_causal(int Lq, int Lk, int q_offset, const int* seg_q_end, const int* seg_k_end,
                                   const int* seg_causal, int n_seg, int* row_lo, int* row_hi) {
    int s = 0;
    for (int r = 0; r < Lq; ++r) {
        while (s < n_seg - 1 && r >= seg_q_end[s]) ++s;
        int hi = std::min(Lk, seg_k_end[s]);
        if (seg_causal[s]) hi = std::min(hi, q_offset + r + 1);
        row_lo[r] = 0;
        row_hi[r] = std::max(hi, 0);
    }
}
// Dense (Lq, Lk) visibility from the rule itself (qwenimage21.h:31-33): key j visible
// to query i iff i >= j or both sit in the same image block. block_id[t] < 0 marks a
// text token, otherwise the image block index; positions are joint-sequence positions,
// query row r sits at position q_offset + r.
ORC_API void orc_dense_block_causal(int Lq, int Lk, int q_offset, const int* block_id, uint8_t* mask) {
    for (int r = 0; r < Lq; ++r) {
        const int i = q_offset + r;
        for (int j = 0; j < Lk; ++j) {
            const bool same_img = block_id[i] >= 0 && block_id[i] == block_id[j];
            mask[static_cast<size_t>(r) * Lk + j] = (i >= j || same_img) ? 1 : 0;
        }
    }
}

// ─── ReLU linear attention ──────────────────────────────────────────────────
// The FP32 per-head core of SanaDenoiser::self_attention_, src/dit/sana.cpp:470-520
// (same math in src/vae_dcae.cpp:281-308), restated on token-major operands
// q/k/v (N, H*d):
//   Qr = relu(Q), Kr = relu(K)                                   (sana.cpp:477-478)
//   [S; z] = [V; 1] . Kr^T  -> S (d, d), z (d)                   (sana.cpp:480-488)
//   hid = [S; z] . Qr       -> num (d, N), den (N)               (sana.cpp:511)
//   recip = rsqrt(den + eps)^2 in FP32                           (sana.cpp:512-516)
//   out = num * recip                                            (sana.cpp:517-519)
// Matmul sums run in double and are stored as float (an FP32 matmul's exact value up
// to its own rounding). S_out (H, d, d) and z_out (H, d) are optional outputs.
ORC_API void orc_linear_attn_relu(const float* q, const float* k, const float* v, int N, int H, int d,
                                  float eps, float* out, float* S_out, float* z_out, int n_threads) {
    const size_t D = static_cast<size_t>(H) * d;
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#endif
#pragma omp parallel for schedule(dynamic, 1)
    for (int h = 0; h < H; ++h) {
        std::vector<double> S(static_cast<size_t>(d) * d, 0.0), z(d, 0.0);
        std::vector<float> kr(d);
        for (int n = 0; n < N; ++n) {
            const float* krow = k + static_cast<size_t>(n) * D + static_cast<size_t>(h) * d;
            const float* vrow = v + static_cast<size_t>(n) * D + static_cast<size_t>(h) * d;
            for (int j = 0; j < d; ++j) { kr[j] = krow[j] > 0.0f ? krow[j] : 0.0f; z[j] += kr[j]; }
            for (int i = 0; i < d; ++i) {
                const double vi = vrow[i];
                double* Si = S.data() + static_cast<size_t>(i) * d;
                for (int j = 0; j < d; ++j) Si[j] += vi * static_cast<double>(kr[j]);
            }
        }
        std::vector<float> Sf(static_cast<size_t>(d) * d), zf(d);
        for (size_t i = 0; i < Sf.size(); ++i) Sf[i] = static_cast<float>(S[i]);
        for (int j = 0; j < d; ++j) zf[j] = static_cast<float>(z[j]);
        if (S_out) std::memcpy(S_out + static_cast<size_t>(h) * d * d, Sf.data(), Sf.size() * sizeof(float));
        if (z_out) std::memcpy(z_out + static_cast<size_t>(h) * d, zf.data(), zf.size() * sizeof(float));
        std::vector<float> qr(d);
        for (int n = 0; n < N; ++n) {
            const float* qrow = q + static_cast<size_t>(n) * D + static_cast<size_t>(h) * d;
            float* orow = out + static_cast<size_t>(n) * D + static_cast<size_t>(h) * d;
            for (int j = 0; j < d; ++j) qr[j] = qrow[j] > 0.0f ? qrow[j] : 0.0f;
            double den = 0.0;
            for (int j = 0; j < d; ++j) den += static_cast<double>(zf[j]) * static_cast<double>(qr[j]);
            const float denf = static_cast<float>(den);
            const float rs = 1.0f / std::sqrt(denf + eps);
            const float recip = rs * rs;
            for (int i = 0; i < d; ++i) {
                const float* Si = Sf.data() + static_cast<size_t>(i) * d;
                double num = 0.0;
                for (int j = 0; j < d; ++j) num += static_cast<double>(Si[j]) * static_cast<double>(qr[j]);
                orow[i] = static_cast<float>(num) * recip;
            }
        }
    }
}

// ─── per-head RMS normalisation ─────────────────────────────────────────────
// bt::rms_norm_forward(X viewed as (L*heads, head_dim), gain, eps, out) as the DiT blocks use it
// (headnorm, src/dit/qwenimage21_forward.cpp:53-63; src/dit/flux.cpp:462-469):
//   y[r][j] = x[r][j] * gain[j] / sqrt(mean_j(x[r][j]^2) + eps)
// (the RMSNorm of diffusers' Flux / Qwen-Image attention processors, which the reference ports). Sums in
// double, result stored as float; x is (rows, cols), gain (cols).
ORC_API void orc_rms_norm(const float* x, const float* gain, double eps, int rows, int cols, float* out) {
#pragma omp parallel for schedule(static)
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + static_cast<size_t>(r) * cols;
        double ss = 0.0;
        for (int j = 0; j < cols; ++j) ss += static_cast<double>(xr[j]) * static_cast<double>(xr[j]);
        const double inv = 1.0 / std::sqrt(ss / cols + eps);
        for (int j = 0; j < cols; ++j)
            out[static_cast<size_t>(r) * cols + j] = static_cast<float>(static_cast<double>(xr[j]) * inv * static_cast<double>(gain[j]));
    }
}

// ─── linear layer ───────────────────────────────────────────────────────────
// Y = X W^T + bias with X (M, K), W (N, K) row-major — the torch Linear weight layout the
// reference's loaders and tests use (tests/test_unet.cpp:144-162: to_k.weight is {C, ctx_dim})
// — as computed by brotensor::linear_forward_batched_fp16 behind detail::linear_batched
// (include/brodiffusion/detail/compute.h:52-62). Sums run in double and are stored as float;
// bias may be null. The projections around attention (bt::flash_attention_qkvo_forward,
// src/unet_blocks.cpp:264-272) are this function applied four times.
ORC_API void orc_linear(const float* x, const float* w, const float* bias, int M, int N, int K, float* y, int n_threads) {
#ifdef _OPENMP
    if (n_threads > 0) omp_set_num_threads(n_threads);
#else
    (void)n_threads;
#endif
#pragma omp parallel for schedule(static)
    for (int m = 0; m < M; ++m) {
        const float* xr = x + static_cast<size_t>(m) * K;
        for (int n = 0; n < N; ++n) {
            const float* wr = w + static_cast<size_t>(n) * K;
            double acc = bias ? static_cast<double>(bias[n]) : 0.0;
            for (int k = 0; k < K; ++k) acc += static_cast<double>(xr[k]) * static_cast<double>(wr[k]);
            y[static_cast<size_t>(m) * N + n] = static_cast<float>(acc);
        }
    }
}

// ─── GEGLU ──────────────────────────────────────────────────────────────────
// brotensor::geglu_exact_forward as brodiffusion::fused_linear_geglu states it
// (include/brodiffusion/fused_transformer.h:20-29, src/fused_transformer.cu:66-68): t is (rows, 2*d_out),
// value half a = t[:, :d_out], gate half g = t[:, d_out:], out = a * 0.5 g (1 + erf(g / sqrt 2)). Double arithmetic.
ORC_API void orc_geglu_exact(const float* t, int rows, int d_out, float* out) {
    for (int r = 0; r < rows; ++r)
        for (int j = 0; j < d_out; ++j) {
            const double a = t[static_cast<size_t>(r) * 2 * d_out + j];
            const double g = t[static_cast<size_t>(r) * 2 * d_out + d_out + j];
            out[static_cast<size_t>(r) * d_out + j] = static_cast<float>(a * 0.5 * g * (1.0 + std::erf(g * 0.70710678118654752440)));
        }
}

ORC_API int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
