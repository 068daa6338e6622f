/* mi_attention.h — flat C ABI of the MI355X (gfx950) attention library.
 *
 * This is the only boundary through which host code reaches HIP. It replaces, for
 * the attention path, the brotensor operators the reference calls
 * (paths below are relative to the reference repository root):
 *
 *   bt::flash_attention_forward            src/dit/common.cpp:194, :356, :376;
 *                                          src/dit/qwenimage21_forward.cpp:648, :667, :674;
 *                                          src/dit/pixart.cpp:340; src/dit/sana.cpp:623
 *   bt::flash_attention_windowed_forward   src/dit/qwenimage21_forward.cpp:662
 *   bt::rope_apply / rope_apply_perhead    src/dit/common.cpp:192-193;
 *                                          src/dit/qwenimage21_forward.cpp:584-585;
 *                                          src/triposplat/flow_model.cpp:374
 *   ReLU linear-attention core             src/dit/sana.cpp:470-586
 *   dit::joint_attention_traced            src/dit/common.cpp:198-329 (bias + head-averaged map on device)
 *   bt::flash_attention_qkvo_forward,      src/unet_blocks.cpp:255-327; src/unet.cpp:470-480
 *   ..._q_with_kv_cached_forward, ..._project_kv
 *   bt::linear_forward_batched_fp16        include/brodiffusion/detail/compute.h:52-62
 *
 * Conventions (the reference's own C-API conventions, include/brodiffusion/krea2_capi.h:12-18):
 *   - functions return 0 on success, -1 on failure; mi_last_error() holds the message
 *     for the calling thread; no exception crosses the boundary;
 *   - not thread-safe per stream: drive one stream from one thread;
 *   - every launch goes on the stream given in the args (NULL = the library's current
 *     stream, see mi_set_stream), performs no host synchronisation and allocates
 *     nothing, so a caller may capture it in a HIP graph.
 *
 * Tensors are 2-D row-major per batch item: rows = tokens, cols = heads * head_dim,
 * head h in columns [h*head_dim, (h+1)*head_dim). Strides are in ELEMENTS; a stride
 * of 0 means dense (row stride = heads*head_dim, batch stride = rows*row stride).
 */
#ifndef MI_ATTENTION_H
#define MI_ATTENTION_H

#include <stddef.h>
#include <stdint.h>

#define MI_API __attribute__((visibility("default")))

#ifdef __cplusplus
extern "C" {
#endif

enum { MI_DTYPE_F16 = 1, MI_DTYPE_BF16 = 2 };
enum { MI_MASK_NONE = 0, MI_MASK_CAUSAL = 1, MI_MASK_BLOCK_CAUSAL = 2 };
enum { MI_MAX_SEGMENTS = 32 };

/* Message for the most recent failure on this thread ("" if none). */
MI_API const char* mi_last_error(void);
MI_API const char* mi_version(void);

typedef struct mi_device_info_t {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t clock_khz;
    int32_t lds_bytes_per_cu;
    int32_t l2_bytes;
    int64_t hbm_bytes;
    double peak_mfma_16bit_flops; /* compute_units * clock * 4096 FLOP/clk/CU (dense fp16/bf16) */
} mi_device_info_t;
MI_API int mi_device_info(mi_device_info_t* out);

/* Calibration probe for benchmarks; no counterpart in the reference. One launch on every compute unit of a loop of
 * nothing but independent v_mfma_f32_32x32x16 instructions (`trips` trips of 8 per wavefront) on operands taken from
 * `operands` (device memory of 16-bit values of `dtype`: all zeros, N(0,1), ...). The caller times the launch with
 * events on `stream`; `flops` returns the FLOPs it performs. The sustained rate depends on the operand values because
 * the clock is power-managed, so an MFMA-bound figure quoted against the nominal peak can be read against what the
 * matrix pipes of this GPU sustain on comparable data at this moment. If `clocks` is given, work group g stores the
 * shader cycles and the 100 MHz constant-rate ticks of its loop at clocks[2g], clocks[2g + 1]
 * (cycles / ticks * 100 = MHz under this load). Writes 4096 bytes of `sink`. */
typedef struct mi_mfma_probe_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* operands;
    size_t operand_bytes;     /* >= 4096 */
    int32_t trips;
    int32_t work_groups;      /* out: work groups of the launch (2 per compute unit) */
    float* sink;
    size_t sink_bytes;        /* >= 4096 */
    uint64_t* clocks;         /* NULL, or 2 * work_groups counts (ask with a first call, or size for 2 * 2 * compute_units) */
    size_t clocks_bytes;
    double flops;             /* out */
    void* stream;
} mi_mfma_probe_args;
MI_API int mi_mfma_probe(mi_mfma_probe_args* args);

/* The library's current stream (void* is a hipStream_t). Entry points whose args carry a
 * NULL stream launch here. Mirrors brotensor's cuda_current_stream() contract
 * (src/fused_transformer.cu:38-54). */
MI_API int mi_set_stream(void* stream);
MI_API void* mi_get_stream(void);
MI_API int mi_stream_synchronize(void* stream);

/* Device memory for host code that owns no HIP of its own (the C++ Tensor type). mi_memset_async is hipMemsetAsync:
 * do not record it into a HIP graph (memset nodes have replayed wrongly on this hardware); inside a capture clear memory
 * with a kernel of your own. No operator of this library calls it. */
MI_API void* mi_malloc(size_t bytes);
MI_API int mi_free(void* ptr);
MI_API int mi_memcpy_h2d(void* dst, const void* src, size_t bytes);
MI_API int mi_memcpy_d2h(void* dst, const void* src, size_t bytes);
MI_API int mi_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream);
MI_API int mi_memset_async(void* dst, int value, size_t bytes, void* stream);

/* ── softmax attention ─────────────────────────────────────────────────────
 * O = softmax(Q K^T * scale + mask) V per (batch, head), flash style: scores never
 * reach HBM, softmax statistics and the output accumulate in FP32.
 *
 * Replaces bt::flash_attention_forward(Q,K,V,d_mask,num_heads,causal,out) and
 * bt::flash_attention_windowed_forward(Q,K,V,d_mask,num_heads,window,out), plus what
 * the reference does around them:
 *   - k_prefix/v_prefix: leading key rows read from a second buffer, so the cached
 *     prefix K/V of the Qwen-Image step (src/dit/qwenimage21_forward.cpp:599-649) is
 *     consumed in place instead of being copied into [cache ; fresh];
 *   - rope_*: RoPE applied to Q as it is loaded and to the rows of `k` (as they are loaded, or by
 *     one pass into rope_k_scratch when the caller lends one), replacing the two bt::rope_apply
 *     passes of dit::joint_attention (src/dit/common.cpp:188-196).
 *     Adjacent pairs (x[2p], x[2p+1]) or, with rope_split_half, the two halves of a head; prefix rows are taken as already rotated
 *     (the reference caches post-RoPE K, qwenimage21_forward.cpp:587-597);
 *   - block-causal segments: the per-segment calls of the prefill form
 *     (qwenimage21_forward.cpp:650-676) in one launch; key tiles no query row of a work
 *     group can see are skipped.
 *
 * Keys are indexed over the concatenation [k_prefix ; k]: Lk = prefix_len + kv_len.
 * Visibility of key j for query row r:
 *   j < kv_valid_len[b]            (if given)
 *   key_mask[b][j] != 0            (if given; FP32, 1 valid / 0 invalid,
 *                                   include/brodiffusion/dit/common.h:138-139)
 *   MI_MASK_CAUSAL:        j <= q_offset + r, and j > q_offset + r - window if window > 0
 *   MI_MASK_BLOCK_CAUSAL:  with s the segment holding r (rows [seg_q_end[s-1], seg_q_end[s])):
 *                          j < seg_k_end[s], and j <= q_offset + r if seg_causal[s]
 * A query row with no visible key produces zeros (src/dit/common.cpp:293).
 */
typedef struct mi_sdpa_args {
    uint32_t struct_size; /* = sizeof(mi_sdpa_args) */
    int32_t dtype;        /* MI_DTYPE_F16 / MI_DTYPE_BF16: type of q, k, v, o */
    const void* q;        /* (batch, q_len, heads*head_dim) */
    const void* k;        /* (batch, kv_len, heads*head_dim) */
    const void* v;
    void* o;              /* (batch, q_len, heads*head_dim) */
    const void* k_prefix; /* (batch, prefix_len, heads*head_dim) or NULL */
    const void* v_prefix;
    int32_t batch, num_heads, head_dim;
    int32_t num_kv_heads; /* 0 or num_heads: plain MHA; a divisor of num_heads: grouped-query, query head h
                             reads K/V head h / (num_heads/num_kv_heads), K/V rows are num_kv_heads*head_dim wide
                             (replaces the K/V widening copies of dit::gqa_attention_masked, src/dit/common.cpp:333-378) */
    int32_t q_len, kv_len, prefix_len;
    int64_t q_row_stride, q_batch_stride;
    int64_t k_row_stride, k_batch_stride;
    int64_t v_row_stride, v_batch_stride;
    int64_t o_row_stride, o_batch_stride;
    int64_t kp_row_stride, kp_batch_stride;
    int64_t vp_row_stride, vp_batch_stride;
    float scale;                 /* <= 0: 1/sqrt(head_dim) */
    int32_t mask_mode;           /* MI_MASK_* */
    int32_t q_offset;            /* joint-sequence position of query row 0 */
    int32_t window;              /* MI_MASK_CAUSAL only; 0 = unbounded */
    const int32_t* kv_valid_len; /* device, [batch], or NULL */
    const float* key_mask;       /* device, [batch or 1][Lk], or NULL */
    int64_t key_mask_batch_stride; /* elements; 0 = one mask shared by all batch items */
    int32_t n_segments;          /* MI_MASK_BLOCK_CAUSAL: 1..MI_MAX_SEGMENTS */
    int32_t seg_q_end[MI_MAX_SEGMENTS];
    int32_t seg_k_end[MI_MAX_SEGMENTS];
    int32_t seg_causal[MI_MAX_SEGMENTS];
    const float* rope_cos_q;     /* device FP32 (q_len, head_dim/2) or NULL */
    const float* rope_sin_q;
    const float* rope_cos_k;     /* device FP32 (kv_len, head_dim/2) or NULL; rows of `k` only */
    const float* rope_sin_k;
    int32_t rope_split_half;     /* 0: the rotation pairs adjacent elements (x[2p], x[2p+1]); 1: it pairs the two halves of a head,
                                    (x[p], x[p + head_dim/2]), as mi_rope_apply's split_half. Applies to Q as it is loaded and to the
                                    pass that rotates K into rope_k_scratch; with 1 the scratch is required when rope_cos_k is given
                                    (the tile-by-tile rotation of K exists for adjacent pairs only). Which convention brotensor's
                                    rope_apply uses cannot be read from the reference: the binding picks it per call site */
    void* rope_k_scratch;        /* device (batch, kv_len, kv_heads*head_dim) of `dtype`, dense, or NULL. With rope_cos_k:
                                    K is rotated into it by one bandwidth-bound pass and attention reads the rotated copy
                                    (fastest form); afterwards it holds RoPE(K) like the Kr scratch of dit::joint_attention
                                    (src/dit/common.cpp:193). NULL: K is rotated tile by tile as it is loaded */
    const float* logit_bias;     /* device FP32 or NULL: additive pre-softmax bias for query rows >= bias_q0 and keys
                                    < bias_cols, element (row - bias_q0, key), added to the scaled score — the image->text
                                    steering bias of dit::joint_attention_traced (src/dit/common.cpp:217-235, :279-281;
                                    joint sequence [text ; image]: bias_q0 = bias_cols = txt_len). Batch 1 */
    int32_t bias_q0, bias_cols;
    int64_t bias_row_stride;     /* elements; 0 = bias_cols */
    float* lse_out;              /* device FP32 [batch][num_heads][q_len] or NULL: receives per row the base-2 logarithm of the
                                    softmax denominator in exponent units, lse = log2 sum_k 2^(score_k*scale*log2(e) + bias*log2(e))
                                    (+inf for a row without visible keys); input of mi_attention_map_avg */
    const int32_t* cu_seqlens_q; /* device int32 [batch + 1], or NULL. With both given, the batch items are sequences of different */
    const int32_t* cu_seqlens_k; /* lengths packed along the row axis: item b owns query rows [cu_seqlens_q[b], cu_seqlens_q[b+1]) of q / o
                                    and key rows [cu_seqlens_k[b], cu_seqlens_k[b+1]) of k / v; q_len and kv_len are the LONGEST
                                    sequence (they size the launch), batch strides are ignored. bt::flash_attention_varlen_forward
                                    (q, k, v, cu_q, cu_k, n_seqs, max_q, max_k, num_heads, head_dim, causal, out),
                                    src/dit/krea2.cpp:574. MI_MASK_NONE or MI_MASK_CAUSAL (window 0; each sequence aligns its last
                                    query with its last key); no prefix, key mask, kv_valid_len, RoPE, bias */
    /* The prefix-KV dial of the Qwen-Image cached step (set_prefix_kv_scale, src/dit/qwenimage21_forward.cpp:606-645): the
       rows of k_prefix count as multiplied by prefix_k_scale, those of v_prefix by prefix_v_scale (0 = 1), and, if the
       arrays are given, row j additionally by prefix_k_row_scale[j] / prefix_v_row_scale[j] (device FP32 [prefix_len],
       shared by the batch). Nothing is copied or written: the K factor multiplies the FP32 scores of the prefix keys,
       the V factor their probabilities after the row sum is taken, inside the attention kernel (the reference scales a
       copy of the cached rows and rounds it to the storage type; mi_scale_rows + k_prefix is that dataflow). With
       scalars of exactly 1 and no arrays the call is the unscaled one bit for bit. */
    float prefix_k_scale;
    float prefix_v_scale;
    const float* prefix_k_row_scale;
    const float* prefix_v_row_scale;
    void* split_scratch;         /* device, 16-byte aligned, or NULL: lets a launch whose last round of work groups would fill
                                    only part of the GPU cut the query tiles of that round along the key axis into equal
                                    pieces for all compute units (partial results in the scratch, merged by a second small
                                    kernel). Used when at least mi_sdpa_split_scratch_bytes(args) bytes are lent and that
                                    value is not 0; results agree with the unsplit launch to rounding */
    size_t split_scratch_bytes;
    void* stream;                /* hipStream_t; NULL = library current stream */
} mi_sdpa_args;

MI_API int mi_sdpa_forward(const mi_sdpa_args* args);
/* Bytes of split_scratch with which this call (same args, split_scratch fields ignored) would split its last round;
 * 0 when it would not (masked calls, short key sequences, a last round that is nearly full, kernels without the
 * split). No reference counterpart. */
MI_API size_t mi_sdpa_split_scratch_bytes(const mi_sdpa_args* args);
/* Tuning / testing knob for the calling thread: 0 = choose the kernel by problem size (default),
 * 1 = always the 4-wavefront kernel (128 query rows per work group), 2 = always the 8-wavefront
 * kernel (256 rows; head_dim <= 128), 3 = as 2 but with register-staged tiles where the default
 * would move tiles by LDS DMA (head_dim 72 and 128). Results agree to rounding; no reference counterpart. */
MI_API int mi_sdpa_set_kernel_choice(int32_t choice);
/* 1 if (dtype, head_dim) has a compiled kernel, else 0: fp16 / bf16 at head_dim 40, 64, 72, 80, 96, 112, 128, 160, and at
 * 256, 384 and 512 (one wide head, src/vae.cpp:259-277, src/vae_qwenimage.cpp:322-340) without cached prefix, logit bias, lse_out and packed sequences. */
MI_API int mi_sdpa_supported(int32_t dtype, int32_t head_dim);

/* ── head-averaged attention map ───────────────────────────────────────────
 * map[q][k] = (1/num_heads) * sum over heads of softmax_h(q, k), FP32 (q_len, kv_len): the trace artifact of
 * dit::joint_attention_traced (src/dit/common.cpp:297, :308-312), which the reference computes in a host loop over
 * downloaded tensors, and of bt::cross_attention_forward_with_attn (src/unet_blocks.cpp:282-290). q, k as given to
 * mi_sdpa_forward (already rotated), batch 1, no mask other than key_mask; `lse` is what that call wrote to lse_out
 * with the same scale, bias and key_mask. Every element is accumulated in one register over the heads and written
 * once (no atomics). */
typedef struct mi_attention_map_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* q;           /* (q_len, heads*head_dim) */
    const void* k;           /* (kv_len, heads*head_dim) */
    const float* lse;        /* [num_heads][q_len] */
    float* map;              /* (q_len, kv_len) */
    int32_t num_heads, head_dim, q_len, kv_len;
    int64_t q_row_stride, k_row_stride, map_row_stride;
    float scale;             /* <= 0: 1/sqrt(head_dim) */
    const float* logit_bias;
    int32_t bias_q0, bias_cols;
    int64_t bias_row_stride;
    const float* key_mask;   /* null, or [kv_len]: 1 = valid, 0 = masked (those map columns are 0) */
    void* stream;
} mi_attention_map_args;
MI_API int mi_attention_map_avg(const mi_attention_map_args* args);

/* ── stand-alone RoPE ──────────────────────────────────────────────────────
 * Replaces bt::rope_apply(X,cos,sin,head_dim,num_heads,out) and
 * bt::rope_apply_perhead. Needed where the rotated tensor itself is kept (the prefix
 * cache stores post-RoPE K). Tables are FP32 (rows, head_dim/2), or
 * (rows*num_heads, head_dim/2) when per_head != 0. split_half = 0: pairs
 * (x[2p], x[2p+1]); 1: pairs (x[p], x[p+head_dim/2]). In-place (out == x) is allowed. */
typedef struct mi_rope_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* x;
    void* out;
    const float* cos;
    const float* sin;
    int32_t rows, num_heads, head_dim;
    int64_t x_row_stride, out_row_stride;
    int32_t split_half;
    int32_t per_head;
    void* stream;
} mi_rope_args;
MI_API int mi_rope_apply(const mi_rope_args* args);

/* ── per-head RMSNorm + RoPE in one pass ───────────────────────────────────
 * out = RoPE(x * rsqrt(mean over head_dim of x^2 + eps) * gain) per (row, head): what the DiT blocks do between the
 * Q/K projections and attention as two passes, bt::rms_norm_forward on the (L*heads, head_dim) view followed by
 * bt::rope_apply (headnorm, src/dit/qwenimage21_forward.cpp:53-63 and :582-585; src/dit/flux.cpp:462-469). One read
 * of x, FP32 in between, a single rounding. gain: (head_dim) of `dtype`. cos / sin: FP32 (rows, head_dim/2), pairs as
 * split_half says, or both NULL for the normalisation alone. out2 (optional): rows [0, out2_rows) are written there as well —
 * the prefix rows of K going into the prefix cache while the full K goes to attention
 * (qwenimage21_forward.cpp:587-597). In-place (out == x) is allowed. head_dim 32, 64 or 128. */
typedef struct mi_headnorm_rope_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* x;
    void* out;
    const void* gain;
    const float* cos;
    const float* sin;
    float eps;
    int32_t rows, num_heads, head_dim;
    int64_t x_row_stride, out_row_stride;
    void* out2;
    int32_t out2_rows;
    int64_t out2_row_stride;
    int32_t split_half;      /* 0: adjacent pairs (x[2p], x[2p+1]); 1: pairs (x[p], x[p + head_dim/2]) */
    void* stream;
} mi_headnorm_rope_args;
MI_API int mi_headnorm_rope(const mi_headnorm_rope_args* args);

/* ── row scaling ───────────────────────────────────────────────────────────
 * out[r][c] = x[r][c] * scale * (row_scale ? row_scale[r] : 1), one rounding. The prefix-KV dial of the Qwen-Image
 * cached step (set_prefix_kv_scale: a per-layer scalar, or per-token weights with the scalars folded in,
 * src/dit/qwenimage21_forward.cpp:612-645): the reference scales the prefix rows of its assembled [cache ; fresh]
 * copy and leaves the cache pristine; here the scaled prefix (prefix_len rows only) goes to a scratch that is then
 * passed as k_prefix / v_prefix. row_scale: device FP32 [rows] or NULL. In place (out == x) is allowed. */
typedef struct mi_scale_rows_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* x;
    void* out;
    const float* row_scale;
    float scale;
    int32_t rows, cols;
    int64_t x_row_stride, out_row_stride;
    void* stream;
} mi_scale_rows_args;
MI_API int mi_scale_rows(const mi_scale_rows_args* args);

/* ── ReLU linear attention ─────────────────────────────────────────────────
 * Per (batch, head): Kr = relu(K), Qr = relu(Q); S = V^T Kr (d x d), z = sum_n Kr (d);
 * O[n] = (S Qr[n]) / (z . Qr[n] + eps). Replaces the core of
 * SanaDenoiser::self_attention_ (src/dit/sana.cpp:470-586). Operands are token-major
 * (batch, n_tokens, heads*head_dim). The FP32 state (S, z) lives in `workspace`
 * ((batch*heads) blocks of head_dim*head_dim + head_dim floats, S row-major with rows =
 * value channel, then z): after the call it holds the (S, z) the reference captures at
 * its identity seam (sana.cpp:489-506). accumulate_state != 0 adds this call's (S, z) to
 * what the workspace already holds instead of starting from zero (the inject form).
 * `scratch` (optional, FP32, up to mi_linear_attn_scratch_bytes) lets the state pass split the
 * tokens of a head over several work groups, one partial state each, summed by a small
 * reduction: several times faster at image sizes. Without it one work group streams all
 * tokens of a (batch, head). Results are deterministic either way (no atomics). */
typedef struct mi_linear_attn_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* q;
    const void* k;
    const void* v;
    void* o;
    int32_t batch, num_heads, head_dim, n_tokens;
    int64_t q_row_stride, q_batch_stride;
    int64_t k_row_stride, k_batch_stride;
    int64_t v_row_stride, v_batch_stride;
    int64_t o_row_stride, o_batch_stride;
    float eps;
    int32_t accumulate_state;
    float accumulate_weight; /* with accumulate_state: weight w of the state found in the workspace, new state = this call's
                                (S, z) + w * old (the inject strength of the identity seam, src/dit/sana.cpp:498-505, :547-551);
                                0 means 1 */
    void* workspace;
    size_t workspace_bytes;
    void* scratch;          /* device, 16-byte aligned, or NULL */
    size_t scratch_bytes;
    int32_t form;           /* MI_LINEAR_ATTN_FORM_BY_SIZE (0): the library picks. _THREE_LAUNCHES: state per token chunk, reduction
                               of the partial states (in `scratch`), apply. _ONE_LAUNCH: the state split along its value channels,
                               every work group streams K, its slice of V, then Q, and writes its slice of O; no scratch is used.
                               A call that accumulates onto a state always takes the three launches */
    int32_t layout;         /* MI_LAYOUT_TOKEN_MAJOR (0): q, k, v, o are (batch, n_tokens, heads*head_dim), a row per token, as
                               everywhere in this header. MI_LAYOUT_CHANNEL_MAJOR: (batch, heads*head_dim, n_tokens), a row per
                               channel, head h in rows [h*head_dim, (h+1)*head_dim) — the layout in which the reference keeps
                               q_, k_, v_ and attn_c_ around its core (src/dit/sana.cpp:424-444, :470-586), so that a binding
                               which keeps the reference's projections can call the core alone. Row strides are then between
                               channel rows (0 = n_tokens), batch strides default to heads*head_dim rows; n_tokens must be a
                               multiple of 8; always one launch; accumulate_state is not offered */
    void* stream;
} mi_linear_attn_args;
enum { MI_LAYOUT_TOKEN_MAJOR = 0, MI_LAYOUT_CHANNEL_MAJOR = 1 };
enum { MI_LINEAR_ATTN_FORM_BY_SIZE = 0, MI_LINEAR_ATTN_FORM_THREE_LAUNCHES = 1, MI_LINEAR_ATTN_FORM_ONE_LAUNCH = 2 };
MI_API size_t mi_linear_attn_workspace_bytes(int32_t batch, int32_t num_heads, int32_t head_dim);
MI_API size_t mi_linear_attn_scratch_bytes(int32_t batch, int32_t num_heads, int32_t head_dim);
MI_API int mi_linear_attn_relu_forward(const mi_linear_attn_args* args);
MI_API int mi_linear_attn_supported(int32_t dtype, int32_t head_dim);
/* The same operator for callers that cannot allocate device memory and have no scratch to lend (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): the partial states of the token chunks live in a
 * static device array inside the library, MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES per GPU for the life of the process.
 * No counterpart in the reference. Same args; `scratch` / `scratch_bytes` must be NULL / 0; q, k, v, o and `workspace`
 * (the state, in and out) are still the caller's. Same kernels and, whenever 8 partial states fit the array, bit-identical
 * results to mi_linear_attn_relu_forward with a full-size scratch. A problem whose state, batch * heads * (head_dim^2 +
 * head_dim) floats, exceeds the array is refused with an error. Calls no hipMalloc / hipFree; its first call on a GPU looks
 * up the array's device address (hipGetSymbolAddress) and should happen outside a capture. All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams, two threads) race; nothing in it needs clearing between
 * calls (every partial state that is read was written by the same call). */
enum { MI_LINEAR_ATTN_STATIC_SCRATCH_BYTES = 16 * 1024 * 1024 };
MI_API int mi_linear_attn_relu_forward_static_scratch(const mi_linear_attn_args* args);

/* ── linear layer ──────────────────────────────────────────────────────────
 * Y = X W^T + bias: X (rows, in_features), W (out_features, in_features) — the layout of a
 * torch / diffusers Linear weight, which is what the reference loads (tests/test_unet.cpp:144-162) —
 * bias (out_features) of the same dtype or NULL, Y (rows, out_features). FP32 accumulation, bias added
 * in FP32, one rounding. Replaces brotensor::linear_forward_batched_fp16 as reached through
 * detail::linear_batched (include/brodiffusion/detail/compute.h:52-62). in_features and out_features
 * must be multiples of 8; strides in elements (0 = dense), multiples of 8. */
typedef struct mi_linear_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* x;
    const void* w;
    const void* bias;
    void* y;
    int32_t rows, in_features, out_features;
    int64_t x_row_stride, w_row_stride, y_row_stride;
    const float* w_scales;   /* NULL: w has `dtype`. Otherwise w is INT8 (out_features, in_features) and w_scales holds one FP32
                                scale per output feature: Y = (X Wq^T) * scale + bias, the W8A16 form
                                bt::linear_forward_batched_int8w_fp16 (src/unet_blocks.cpp:238-240; weights as
                                include/brodiffusion/detail/unet_blocks.h:28-35). The bytes are widened exactly on their way
                                to LDS and the scale is applied to the FP32 accumulator */
    void* stream;
} mi_linear_args;
MI_API int mi_linear_forward(const mi_linear_args* args);
/* Y (rows, out_features) = a * gelu_exact(g) with [a | g] = X W^T + bias, W (2*out_features, in_features) and bias
 * (2*out_features): value half first, gate half second; gelu_exact(g) = 0.5 g (1 + erf(g / sqrt 2)). The fused FF1 +
 * GEGLU of the U-Net transformer block, brodiffusion::fused_linear_geglu (include/brodiffusion/fused_transformer.h:20-35,
 * src/fused_transformer.cu:56-68): the (rows, 2*out_features) intermediate never reaches memory. Same struct as
 * mi_linear_forward. With w_scales (2*out_features values) W is INT8: the W8A16 overload of the same operator
 * (fused_transformer.h:37-48), which the reference composes from bt::linear_forward_batched_int8w_fp16 into a 16-bit
 * (rows, 2*out_features) buffer and bt::geglu_exact_forward (src/fused_transformer.cu:360-396); here both halves are
 * rounded to the tensor dtype where that buffer would round them, in registers, and the buffer does not exist. */
MI_API int mi_linear_geglu_forward(const mi_linear_args* args);
/* Y[i] += X[i] over n_elements of flat storage (brodiffusion::add_inplace_vec, fused_transformer.h:50-53) and
 * Y[r][c] += bias[c] (brodiffusion::add_inplace_row_bias, fused_transformer.h:55-61). Any element count; 16-byte
 * accesses when the addresses (and, for the bias form, cols and the row stride) allow. */
MI_API int mi_add_inplace(void* y, const void* x, int64_t n_elements, int32_t dtype, void* stream);
MI_API int mi_add_row_bias(void* y, const void* bias, int32_t rows, int32_t cols, int64_t y_row_stride, int32_t dtype, void* stream);
/* out[r][c] = x[r][c] * rsqrt(mean over c of x[r][c]^2 + eps) * gain[c]: RMS normalisation of whole rows, FP32 in between,
 * one rounding. bt::rms_norm_forward(X, gain, eps, out) as Sana-Sprint applies it to the projected q and k across the full
 * inner dimension before the head split (qk_norm, src/dit/sana.cpp:449-461). cols a multiple of 8; strides in elements
 * (0 = dense), multiples of 8; gain (cols) of `dtype`; in place (out == x) is allowed. */
MI_API int mi_rms_norm_forward(const void* x, const void* gain, void* out, int32_t rows, int32_t cols, int64_t x_row_stride,
                               int64_t out_row_stride, float eps, int32_t dtype, void* stream);

/* ── attention with its projections ────────────────────────────────────────
 * The three operators the U-Net spatial transformer calls (src/unet_blocks.cpp:255-327,
 * src/unet.cpp:470-480; also the VAE mid blocks, src/vae.cpp:268):
 *
 *   mi_flash_attention_qkvo_forward               bt::flash_attention_qkvo_forward(X, Ctx*, Wq,bq*, Wk,bk*,
 *       Q = X Wq^T + bq;  S = ctx ? ctx : X;         Wv,bv*, Wo,bo*, d_mask, num_heads, causal, out)
 *       K = S Wk^T + bk;  V = S Wv^T + bv;
 *       out = attention(Q, K, V) Wo^T + bo
 *   mi_flash_attention_q_with_kv_cached_forward   bt::flash_attention_q_with_kv_cached_forward(X, K, V, Wq,bq*,
 *       as above with K, V given (k, v)              Wo,bo*, d_mask, num_heads, causal, out)
 *   mi_flash_attention_project_kv                 bt::flash_attention_project_kv(ctx, Wk,bk*, Wv,bv*, K_out, V_out)
 *       k = ctx Wk^T + bk;  v = ctx Wv^T + bv
 *
 * Weights are (out_features, in_features) row-major, biases may be NULL. Q, K, V and the attention
 * output are rounded to `dtype` between the stages (they are tensors of that dtype in the reference too) and
 * live in `scratch`, which the caller lends: mi_flash_attention_scratch_bytes() bytes, 16-byte aligned.
 * The three projections of the qkvo form run as ONE launch, attention as one, the output projection as
 * one. Rows are batch-major: item b of x is rows [b*q_len, (b+1)*q_len); with ctx == NULL kv_len is
 * taken as q_len. head_dim = inner / num_heads must be one mi_sdpa_supported() accepts. */
typedef struct mi_attn_block_args {
    uint32_t struct_size;
    int32_t dtype;
    const void* x;     /* (batch*q_len, channels) */
    const void* ctx;   /* (batch*kv_len, ctx_channels) or NULL (self-attention) */
    const void* wq;    /* (inner, channels) */
    const void* bq;    /* (inner) or NULL */
    const void* wk;    /* (inner, ctx_channels) — (inner, channels) when ctx == NULL */
    const void* bk;
    const void* wv;
    const void* bv;
    const void* wo;    /* (out_channels, inner) */
    const void* bo;    /* (out_channels) or NULL */
    void* k;           /* (batch*kv_len, inner): input of the kv_cached form, output of project_kv, unused by qkvo */
    void* v;
    void* out;         /* (batch*q_len, out_channels) */
    int32_t batch, q_len, kv_len;
    int32_t channels, ctx_channels, inner, out_channels;
    int32_t num_heads;
    int32_t causal;    /* != 0: key j visible to query r iff j <= r + (kv_len - q_len) */
    const float* key_mask;           /* device FP32 [batch or 1][kv_len], 1 valid / 0 not, or NULL */
    int64_t key_mask_batch_stride;   /* 0 = shared */
    void* scratch;
    size_t scratch_bytes;
    const float* wq_scales;          /* each NULL (weight of `dtype`) or FP32 per-output-row scales of an INT8 weight: the */
    const float* wk_scales;          /* ..._int8w_fp16 forms of the three operators (src/unet_blocks.cpp:256-262, :305-310, */
    const float* wv_scales;          /* src/unet.cpp:470-474). The weights of one projection launch (Q/K/V) must be of one kind */
    const float* wo_scales;
    void* stream;
} mi_attn_block_args;
/* Scratch bytes of the qkvo form (with_kv != 0) or the kv_cached form (with_kv == 0); project_kv needs none. */
MI_API size_t mi_flash_attention_scratch_bytes(int32_t batch, int32_t q_len, int32_t kv_len, int32_t inner, int32_t with_kv);
MI_API int mi_flash_attention_qkvo_forward(const mi_attn_block_args* args);
MI_API int mi_flash_attention_q_with_kv_cached_forward(const mi_attn_block_args* args);
MI_API int mi_flash_attention_project_kv(const mi_attn_block_args* args);

#ifdef __cplusplus
}
#endif
#endif /* MI_ATTENTION_H */
