// Host-side operator interface of the attention path, C++20, no HIP: every computation is a call
// into the C ABI of libmi_attention.so. Names and argument order follow the brotensor operators and
// the brodiffusion wrappers the reference calls (paths in the reference repository):
//   bt::flash_attention_forward            src/dit/common.cpp:194
//   bt::flash_attention_windowed_forward   src/dit/qwenimage21_forward.cpp:662
//   bt::flash_attention_gqa_forward        src/ardy/denoiser_backbone.cpp:179
//   bt::flash_attention_varlen_forward     src/dit/krea2.cpp:574
//   bt::rope_apply / rope_apply_perhead    src/dit/common.cpp:192, src/triposplat/flow_model.cpp:374
//   dit::joint_attention                   include/brodiffusion/dit/common.h:80-88
//   dit::gqa_attention_masked              include/brodiffusion/dit/common.h:144-153
//   dit::joint_attention_traced            include/brodiffusion/dit/common.h:117-129
//   dit::build_axial_rope_tables           include/brodiffusion/dit/common.h:70-72
//   bt::flash_attention_qkvo_forward       src/unet_blocks.cpp:264-272
//   bt::flash_attention_q_with_kv_cached_forward  src/unet_blocks.cpp:311-317
//   bt::flash_attention_project_kv         src/unet.cpp:476-480
//   bt::cross_attention_forward_with_attn  src/unet_blocks.cpp:282-290
//   detail::linear_batched                 include/brodiffusion/detail/compute.h:52-62
//   headnorm + bt::rope_apply              src/dit/qwenimage21_forward.cpp:53-63, :582-585
// Precondition failures throw std::runtime_error("<op>: <message>"); a CPU tensor is refused.
#pragma once
#include <vector>

#include "tensor.h"

namespace bdamd {
namespace bt {

void flash_attention_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* d_mask,
                             int num_heads, bool causal, Tensor& out);
void flash_attention_windowed_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* d_mask,
                                      int num_heads, int window, Tensor& out);
// Grouped-query attention with an optional key mask (src/ardy/denoiser_backbone.cpp:179) and packed variable-length
// attention (src/dit/krea2.cpp:574: sequence i owns query rows [cu_q[i], cu_q[i+1]) and key rows [cu_k[i], cu_k[i+1]);
// cu_q / cu_k are device int32 arrays of n_seqs + 1 offsets).
void flash_attention_gqa_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* key_mask, int num_q_heads,
                                 int num_kv_heads, bool causal, Tensor& out);
void flash_attention_varlen_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const int32_t* cu_q, const int32_t* cu_k,
                                    int n_seqs, int max_q, int max_k, int num_heads, int head_dim, bool causal, Tensor& out);
// Pair convention of every rotation in this layer (rope_apply, rope_apply_perhead, and the rotations fused into
// joint_attention, gqa_attention_masked, joint_attention_traced and headnorm_rope): false (default) pairs adjacent
// elements (x[2p], x[2p+1]), true pairs the two halves of a head (x[p], x[p + head_dim/2]). brotensor's rope_apply has
// one fixed convention that the reference's sources do not state; a binding sets this once, to whatever brotensor does.
void set_rope_split_half(bool split_half);
bool rope_split_half();
void rope_apply(const Tensor& X, const Tensor& cos, const Tensor& sin, int head_dim, int num_heads, Tensor& out);
void rope_apply_perhead(const Tensor& X, const Tensor& cos, const Tensor& sin, int head_dim, int num_heads, Tensor& out);

// Sana's ReLU linear-attention core on token-major (N, heads*head_dim) operands
// (src/dit/sana.cpp:470-586). `state` receives the FP32 (S, z) blocks, heads x (d*d + d). `scratch` (optional,
// caller-owned like the reference's scratch tensors, sized on first use) holds partial states so that the state pass
// can spread the tokens of a head over the whole GPU.
void linear_attention_relu_forward(const Tensor& Q, const Tensor& K, const Tensor& V, int num_heads, float eps,
                                   Tensor& state, Tensor& out, bool accumulate_state = false, Tensor* scratch = nullptr);

// The same core on the reference's own operands: q, k, v and out as (heads*head_dim, N) channel-major tensors, the
// shape of q_, k_, v_ and attn_c_ in SanaDenoiser::self_attention_ (src/dit/sana.cpp:424-444, :470-586), for a binding
// that keeps the reference's projections and replaces the core alone. N must be a multiple of 8.
void linear_attention_relu_forward_channel_major(const Tensor& Q, const Tensor& K, const Tensor& V, int num_heads, float eps,
                                                 Tensor& state, Tensor& out);

// Y = X W^T + bias, W (out_features, in_features); bias may be null.
void linear_batched(const Tensor& W, const Tensor* bias, const Tensor& X, Tensor& Y);

// Attention with its projections (the U-Net spatial transformer's operators). Weights are (out_features, in_features),
// biases may be null, Ctx == nullptr is self-attention. The projections and the attention output live in a scratch
// tensor owned by the calling thread, grown on demand and kept (no allocation after warm-up, as the reference's
// persistent scratch slots, src/unet_blocks.cpp:244-249); pass `scratch` to own it instead.
void flash_attention_qkvo_forward(const Tensor& X, const Tensor* Ctx, const Tensor& Wq, const Tensor* bq,
                                  const Tensor& Wk, const Tensor* bk, const Tensor& Wv, const Tensor* bv,
                                  const Tensor& Wo, const Tensor* bo, const float* d_mask, int num_heads, bool causal,
                                  Tensor& out, Tensor* scratch = nullptr);
void flash_attention_q_with_kv_cached_forward(const Tensor& X, const Tensor& K, const Tensor& V, const Tensor& Wq,
                                              const Tensor* bq, const Tensor& Wo, const Tensor* bo, const float* d_mask,
                                              int num_heads, bool causal, Tensor& out, Tensor* scratch = nullptr);
void flash_attention_project_kv(const Tensor& ctx, const Tensor& Wk, const Tensor* bk, const Tensor& Wv, const Tensor* bv,
                                Tensor& K_out, Tensor& V_out);

// W8A16 forms (INT8 weight (out, in) + FP32 per-output-row scales (out, 1)), argument order of the brotensor operators
// the quantised U-Net calls (src/unet_blocks.cpp:238-240, :256-262, :305-310; src/unet.cpp:470-474).
void linear_forward_batched_int8w_fp16(const Tensor& W_int8, const Tensor& scales, const Tensor* bias, const Tensor& X, Tensor& Y);
void flash_attention_qkvo_int8w_fp16(const Tensor& X, const Tensor* Ctx, const Tensor& Wq, const Tensor& Wq_scales, const Tensor* bq,
                                     const Tensor& Wk, const Tensor& Wk_scales, const Tensor* bk, const Tensor& Wv,
                                     const Tensor& Wv_scales, const Tensor* bv, const Tensor& Wo, const Tensor& Wo_scales,
                                     const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out,
                                     Tensor* scratch = nullptr);
void flash_attention_q_with_kv_cached_int8w_fp16(const Tensor& X, const Tensor& K, const Tensor& V, const Tensor& Wq,
                                                 const Tensor& Wq_scales, const Tensor* bq, const Tensor& Wo, const Tensor& Wo_scales,
                                                 const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out,
                                                 Tensor* scratch = nullptr);
void flash_attention_project_kv_int8w_fp16(const Tensor& ctx, const Tensor& Wk, const Tensor& Wk_scales, const Tensor* bk,
                                           const Tensor& Wv, const Tensor& Wv_scales, const Tensor* bv, Tensor& K_out, Tensor& V_out);

// The U-Net's traced cross attention (src/unet_blocks.cpp:282-290): Q = X Wq^T, K = Ctx Wk^T, V = Ctx Wv^T (no biases),
// attention with the optional additive logit bias (FP32 (Lq, Lk)) and key mask, out = A Wo^T (no bias: the caller adds
// it), AttnAvg = the FP32 (Lq, Lk) softmax averaged over the heads. Everything stays on the device; the projected
// tensors live in a scratch this layer keeps per thread and stream.
void cross_attention_forward_with_attn(const Tensor& X, const Tensor& Ctx, const Tensor& Wq, const Tensor& Wk, const Tensor& Wv,
                                       const Tensor& Wo, const float* d_mask, const Tensor* logit_bias, int num_heads,
                                       Tensor& out, Tensor& AttnAvg);

// Multi-head self attention with the projections around it, as PixArt's self attention calls it on the reference's
// FP32 path (src/dit/pixart.cpp:325-328): qh = X Wq^T + bq, kh, vh likewise, yc = attention(qh, kh, vh) with the
// optional key mask, out = yc Wo^T + bo (biases nullable). Here for FP16 / BF16 device tensors, the same four GEMMs
// and one attention launch as flash_attention_qkvo_forward, with the intermediates in the caller's tensors. The scores
// are never materialised: `attn` is left as it is.
void mha_forward(const Tensor& X, const Tensor& Wq, const Tensor& Wk, const Tensor& Wv, const Tensor& Wo, const Tensor* bq,
                 const Tensor* bk, const Tensor* bv, const Tensor* bo, const float* d_mask, int num_heads, Tensor& qh,
                 Tensor& kh, Tensor& vh, Tensor& attn, Tensor& yc, Tensor& out);

}  // namespace bt

// The fused helpers of the SD1.5 transformer block, names and argument order of include/brodiffusion/fused_transformer.h:
//   fused_linear_geglu   Y(B, D_out) = a * gelu_exact(g), [a | g] = X W^T + b, W (2*D_out, D_in), b 2*D_out values  (:20-35)
//   add_inplace_vec      Y += X, same shape                                                                        (:50-53)
//   add_inplace_row_bias Y[i][j] += bias[j], bias holds Y.cols values in any shape                                  (:55-61)
void fused_linear_geglu(const Tensor& X, const Tensor& W, const Tensor& b, Tensor& Y);
// ... and its W8A16 overload (:37-48): W_int8 (2*D_out, D_in) INT8, W_scales (2*D_out, 1) FP32. One GEMM; the two halves are
// rounded to the tensor dtype where the reference's 16-bit (B, 2*D_out) buffer rounds them (src/fused_transformer.cu:360-396).
void fused_linear_geglu(const Tensor& X, const Tensor& W_int8, const Tensor& W_scales, const Tensor& b, Tensor& Y);
void add_inplace_vec(Tensor& Y, const Tensor& X);
void add_inplace_row_bias(Tensor& Y, const Tensor& bias);

namespace dit {

struct RopeTables {
    Tensor cos;  // (L, head_dim/2) FP32
    Tensor sin;
};
RopeTables build_axial_rope_tables(int txt_len, int hp, int wp, int head_dim, const std::vector<int>& axes_dims_rope,
                                   float theta = 10000.0f);

// One segment of a Qwen-Image prefix as the table builder sees it (include/brodiffusion/dit/qwenimage21.h: QwenImage21Segment).
struct QwenSegment {
    enum class Kind { Text, Image } kind;
    int n_tokens;   // Text
    int h, w;       // Image
};
// 3-axis RoPE tables of the joint sequence [prefix segments ; target image hp x wp]
// (QwenImage21Transformer2DModel::build_rope_tables_, src/dit/qwenimage21_forward.cpp:124-200): a shared running
// position walks the sequence; a text token sits at (p, p, p) and advances it by one; an image block freezes the frame
// axis, lays its tokens on a grid centred on zero and advances the position by max(h, w). A cached step uses the rows
// of its target tokens (row_view).
RopeTables build_qwen_rope_tables(const std::vector<QwenSegment>& prefix, int hp, int wp, int head_dim,
                                  const std::vector<int>& axes_dims_rope, float theta = 10000.0f);

// headnorm + rope_apply of the DiT blocks in one pass (src/dit/qwenimage21_forward.cpp:53-63, :582-585;
// src/dit/flux.cpp:462-469): per (row, head) RMS normalisation with `gain` (1 x head_dim or head_dim x 1), then the
// rotation (cos == sin == nullptr: normalisation only). cache_out, if given, is resized to (cache_rows, D) and receives
// the first cache_rows rows as well: the prefix rows of K on their way into the prefix cache (:587-597).
void headnorm_rope(const Tensor& X, const Tensor& gain, float eps, const Tensor* cos, const Tensor* sin, int head_dim,
                   int num_heads, Tensor& out, Tensor* cache_out = nullptr, int cache_rows = 0);

// RoPE on Q and K, then full-bidirectional attention. Q is rotated while it is loaded; K is rotated
// into Kr (resized to K's shape, holds RoPE(K) afterwards as in the reference) and read from there.
// Qr is accepted and left untouched.
void joint_attention(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor& cos, const Tensor& sin,
                     int head_dim, int num_heads, Tensor& out, Tensor& Qr, Tensor& Kr);

// joint_attention with the softmax exposed, entirely on the device (the reference downloads Q, K, V and loops on the
// host, src/dit/common.cpp:198-329): RoPE on Q and K into Qr / Kr, attention with the optional image->text steering
// bias ((L - txt_len, txt_len) FP32, added to the scaled scores of image rows against text keys), `attn_avg` = the
// (L, L) FP32 softmax averaged over the heads.
void joint_attention_traced(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor& cos, const Tensor& sin,
                            int head_dim, int num_heads, Tensor& out, Tensor& attn_avg, Tensor& Qr, Tensor& Kr,
                            int txt_len = 0, const Tensor* image_text_bias = nullptr);

void gqa_attention_masked(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor* cos, const Tensor* sin,
                          int head_dim, int num_q_heads, int num_kv_heads, const float* d_mask, Tensor& out,
                          Tensor& Qr, Tensor& Kr, Tensor& Krep, Tensor& Vrep);

// out = X * scale * row_scale (per row; row_scale: FP32 (rows, 1) / (1, rows) or null). The prefix-KV dial of the
// Qwen-Image cached step (set_prefix_kv_scale, src/dit/qwenimage21_forward.cpp:612-645): scale a copy of the cached
// prefix rows and hand the copy to block_causal_attention as k_prefix / v_prefix; the cache itself stays pristine,
// which is what makes the dial idempotent (tests/test_qwenimage21_slots.cpp:361-412).
void scale_rows(const Tensor& X, float scale, const Tensor* row_scale, Tensor& out);

// One segment of the Qwen-Image joint sequence (src/dit/qwenimage21_forward.cpp:650-676).
struct Segment {
    enum class Kind { Text, Image } kind;
    int n_tokens;
};
// Block-causal attention over [prefix ; target] in ONE launch. Q holds `q_rows` rows starting at
// joint position q_offset; keys are [k_prefix ; K] (k_prefix may be null / empty: prefill form).
// `segments` describe the query rows in order: a Text run is causal, an Image block sees every key
// up to its own end. Equals the reference's one-call-per-segment decomposition; with a single Image
// segment covering all keys it is the cached form (qwenimage21_forward.cpp:599-649).
// `dial` (optional): the prefix-KV dial of the cached step (set_prefix_kv_scale, qwenimage21_forward.cpp:606-645) applied
// inside the kernel — a factor per side on the rows of the cached prefix, optionally times a per-row FP32 weight
// ((prefix_len, 1) or (1, prefix_len)); the cache tensors are never written and no scaled copy is made.
struct PrefixDial {
    float k_scale = 1.f, v_scale = 1.f;
    const Tensor* k_rows = nullptr; const Tensor* v_rows = nullptr;
};
void block_causal_attention(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor* k_prefix,
                            const Tensor* v_prefix, const std::vector<Segment>& segments, int q_offset,
                            int num_heads, const Tensor* cos_q, const Tensor* sin_q, Tensor& out,
                            const PrefixDial* dial = nullptr);

// RMS normalisation of whole rows with a per-column gain: bt::rms_norm_forward(X, gain, eps, out) (src/dit/sana.cpp:455).
void rms_norm_rows(const Tensor& X, const Tensor& gain, float eps, Tensor& out);

// SanaDenoiser::self_attention_ (src/dit/sana.cpp:411-595) as one operator: the three bias-free projections of x_mod, the
// optional qk_norm (RMS normalisation of q and k across the full inner dimension, :449-461), the ReLU linear-attention
// core (:470-586) and the biased output projection (:587-594). The reference runs the core channel-major, (D, N), between
// a transposing projection and a transpose back; here everything from x_mod (N, D) to out (N, D) stays token-major, so
// neither transpose exists, and the core is one mi_linear_attn_relu_forward call.
// Weights are (out_features, in_features) as loaded; nq / nk (D) may be null (no qk_norm); bo may be null.
// Identity seam (:489-506, :543-552): Capture fills `ref_state` with this call's (S, z) — FP32, num_heads blocks of
// (head_dim + 1, head_dim): head_dim rows of S, then z, which is the layout of the reference's FP32 cache; Inject adds
// ref_weight * ref_state to this call's (S, z) before the queries read it and leaves ref_state untouched.
struct SanaAttnWeights {
    const Tensor* Wq; const Tensor* Wk; const Tensor* Wv;   // (D, D)
    const Tensor* nq; const Tensor* nk;                     // (D) gains of the qk_norm, or null
    const Tensor* Wo; const Tensor* bo;                     // (D, D), (D) or null
};
struct SanaAttnScratch { Tensor q, k, v, attn, state, partials; };   // caller-owned, sized on first use, reused afterwards
enum class RefMode { Off, Capture, Inject };
void sana_self_attention(const Tensor& x_mod, const SanaAttnWeights& w, int num_heads, Tensor& out, SanaAttnScratch& scratch,
                         RefMode ref_mode = RefMode::Off, Tensor* ref_state = nullptr, float ref_weight = 0.f,
                         float rms_eps = 1e-5f, float attn_eps = 1e-15f);

}  // namespace dit
}  // namespace bdamd
