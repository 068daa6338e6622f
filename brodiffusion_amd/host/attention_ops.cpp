#include "attention_ops.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <unordered_map>

namespace bdamd {
namespace {

int dtype_code(const char* op, Dtype d) {
    if (d == Dtype::BF16) return MI_DTYPE_BF16;
    if (d == Dtype::FP16) return MI_DTYPE_F16;
    fail(std::string(op) + ": dtype must be FP16 or BF16 on the GPU path");
}
void need_gpu(const char* op, const Tensor& t) {
    if (t.device != Device::GPU) fail(std::string(op) + ": tensor is on the CPU; this path is GPU-only and does not copy");
    if (t.size() != 0 && t.data == nullptr) fail(std::string(op) + ": tensor has no storage");
}
void check(const char* op, int rc) {
    if (rc != 0) fail(std::string(op) + ": " + mi_last_error());
}
void init_args(mi_sdpa_args& a, const char* op, const Tensor& Q, const Tensor& K, const Tensor& V, int num_heads,
               int num_kv_heads, Tensor& out) {
    need_gpu(op, Q); need_gpu(op, K); need_gpu(op, V);
    if (num_heads <= 0 || Q.cols % num_heads != 0) fail(std::string(op) + ": D must equal head_dim * num_heads");
    const int hd = Q.cols / num_heads;
    const int dt = dtype_code(op, Q.dtype);
    if (K.dtype != Q.dtype || V.dtype != Q.dtype) fail(std::string(op) + ": Q, K, V must share one dtype");
    if (K.cols != num_kv_heads * hd || V.cols != K.cols || V.rows != K.rows)
        fail(std::string(op) + ": K and V must be (Lk, kv_heads*head_dim)");
    if (out.data == nullptr || out.rows != Q.rows || out.cols != Q.cols || out.dtype != Q.dtype)
        out.resize(Q.rows, Q.cols, Q.dtype, Q.device);
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dt;
    a.q = Q.data; a.k = K.data; a.v = V.data; a.o = out.data;
    a.batch = 1; a.num_heads = num_heads; a.head_dim = hd; a.num_kv_heads = num_kv_heads;
    a.q_len = Q.rows; a.kv_len = K.rows;
}
// Scratch that this layer owns exists once per (thread, library stream of that thread at the time of the call) and use
// (Tag): calls on one stream run in order and may share it, calls that a thread puts on different streams may overlap on
// the GPU and get one each. Grown on demand, then kept (no allocation after warm-up), and never destroyed: a destructor
// running at thread or process exit could call into a GPU runtime that is already gone.
template <typename T, typename Tag> T& per_stream() {
    static thread_local std::unordered_map<void*, T*>* m = new std::unordered_map<void*, T*>;
    T*& t = (*m)[mi_get_stream()];
    if (t == nullptr) t = new T;
    return *t;
}
// Launch with the split scratch lent when the call can use one.
void run_sdpa(const char* op, mi_sdpa_args& a) {
    struct SplitScratch;
    Tensor* const scratch = &per_stream<Tensor, SplitScratch>();
    const std::size_t need = mi_sdpa_split_scratch_bytes(&a);
    if (need > 0) {
        if (scratch->data == nullptr || scratch->bytes() < need) scratch->resize(1, static_cast<int>((need + 3) / 4), Dtype::FP32, Device::GPU);
        a.split_scratch = scratch->data;
        a.split_scratch_bytes = scratch->bytes();
    }
    check(op, mi_sdpa_forward(&a));
}
void set_rope(mi_sdpa_args& a, const char* op, const Tensor* cos, const Tensor* sin, int rows, bool for_q) {
    if (!cos && !sin) return;
    if (!cos || !sin) fail(std::string(op) + ": cos and sin must be given together");
    need_gpu(op, *cos); need_gpu(op, *sin);
    if (cos->dtype != Dtype::FP32 || sin->dtype != Dtype::FP32) fail(std::string(op) + ": RoPE tables must be FP32");
    if (cos->rows != rows || sin->rows != rows || cos->cols != a.head_dim / 2 || sin->cols != a.head_dim / 2)
        fail(std::string(op) + ": RoPE tables must be (L, head_dim/2)");
    if (for_q) { a.rope_cos_q = static_cast<const float*>(cos->data); a.rope_sin_q = static_cast<const float*>(sin->data); }
    else { a.rope_cos_k = static_cast<const float*>(cos->data); a.rope_sin_k = static_cast<const float*>(sin->data); }
}

}  // namespace

namespace bt {

void flash_attention_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* d_mask, int num_heads,
                             bool causal, Tensor& out) {
    const char* op = "flash_attention_forward";
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_heads, num_heads, out);
    a.key_mask = d_mask;
    if (causal) { a.mask_mode = MI_MASK_CAUSAL; a.q_offset = K.rows - Q.rows; }
    run_sdpa(op, a);
}

void flash_attention_windowed_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* d_mask,
                                      int num_heads, int window, Tensor& out) {
    const char* op = "flash_attention_windowed_forward";
    if (window < 0) fail(std::string(op) + ": window must be >= 0");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_heads, num_heads, out);
    a.key_mask = d_mask;
    a.mask_mode = MI_MASK_CAUSAL; a.q_offset = K.rows - Q.rows; a.window = window;
    run_sdpa(op, a);
}

void flash_attention_gqa_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const float* key_mask, int num_q_heads,
                                 int num_kv_heads, bool causal, Tensor& out) {
    const char* op = "flash_attention_gqa_forward";
    if (num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0) fail(std::string(op) + ": num_kv_heads must divide num_q_heads");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_q_heads, num_kv_heads, out);
    a.key_mask = key_mask;
    if (causal) { a.mask_mode = MI_MASK_CAUSAL; a.q_offset = K.rows - Q.rows; }
    run_sdpa(op, a);
}

void flash_attention_varlen_forward(const Tensor& Q, const Tensor& K, const Tensor& V, const int32_t* cu_q, const int32_t* cu_k,
                                    int n_seqs, int max_q, int max_k, int num_heads, int head_dim, bool causal, Tensor& out) {
    const char* op = "flash_attention_varlen_forward";
    if (!cu_q || !cu_k || n_seqs <= 0 || max_q < 0 || max_k < 0) fail(std::string(op) + ": cu_q, cu_k and a positive n_seqs are required");
    if (head_dim <= 0 || Q.cols != num_heads * head_dim) fail(std::string(op) + ": D must equal head_dim * num_heads");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_heads, num_heads, out);
    a.batch = n_seqs; a.q_len = max_q; a.kv_len = max_k;
    a.q_batch_stride = a.k_batch_stride = a.v_batch_stride = a.o_batch_stride = 8;   // ignored for packed sequences
    a.cu_seqlens_q = cu_q; a.cu_seqlens_k = cu_k;
    if (causal) a.mask_mode = MI_MASK_CAUSAL;
    run_sdpa(op, a);
}

static bool g_rope_split_half = false;
void set_rope_split_half(bool split_half) { g_rope_split_half = split_half; }
bool rope_split_half() { return g_rope_split_half; }

static void rope_impl(const char* op, const Tensor& X, const Tensor& cos, const Tensor& sin, int head_dim, int num_heads,
                      Tensor& out, bool per_head) {
    need_gpu(op, X); need_gpu(op, cos); need_gpu(op, sin);
    if (head_dim <= 0 || num_heads <= 0 || X.cols != head_dim * num_heads) fail(std::string(op) + ": D must equal head_dim * num_heads");
    const int trows = per_head ? X.rows * num_heads : X.rows;
    if (cos.dtype != Dtype::FP32 || sin.dtype != Dtype::FP32 || cos.rows != trows || sin.rows != trows ||
        cos.cols != head_dim / 2 || sin.cols != head_dim / 2)
        fail(std::string(op) + ": cos/sin must be FP32 (rows, head_dim/2)");
    if (out.data == nullptr || out.rows != X.rows || out.cols != X.cols || out.dtype != X.dtype)
        out.resize(X.rows, X.cols, X.dtype, X.device);
    mi_rope_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.x = X.data; a.out = out.data;
    a.cos = static_cast<const float*>(cos.data); a.sin = static_cast<const float*>(sin.data);
    a.rows = X.rows; a.num_heads = num_heads; a.head_dim = head_dim; a.per_head = per_head ? 1 : 0;
    a.split_half = g_rope_split_half ? 1 : 0;
    check(op, mi_rope_apply(&a));
}
void rope_apply(const Tensor& X, const Tensor& cos, const Tensor& sin, int head_dim, int num_heads, Tensor& out) {
    rope_impl("rope_apply", X, cos, sin, head_dim, num_heads, out, false);
}
void rope_apply_perhead(const Tensor& X, const Tensor& cos, const Tensor& sin, int head_dim, int num_heads, Tensor& out) {
    rope_impl("rope_apply_perhead", X, cos, sin, head_dim, num_heads, out, true);
}

void linear_attention_relu_forward(const Tensor& Q, const Tensor& K, const Tensor& V, int num_heads, float eps,
                                   Tensor& state, Tensor& out, bool accumulate_state, Tensor* scratch) {
    const char* op = "linear_attention_relu_forward";
    need_gpu(op, Q); need_gpu(op, K); need_gpu(op, V);
    if (num_heads <= 0 || Q.cols % num_heads != 0) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if (K.rows != Q.rows || V.rows != Q.rows || K.cols != Q.cols || V.cols != Q.cols || K.dtype != Q.dtype || V.dtype != Q.dtype)
        fail(std::string(op) + ": Q/K/V must share shape (N, D) and dtype");
    const int hd = Q.cols / num_heads;
    const int per_head = hd * hd + hd;
    if (accumulate_state) {
        if (state.data == nullptr || state.rows != num_heads || state.cols != per_head || state.dtype != Dtype::FP32)
            fail(std::string(op) + ": accumulate_state needs a (heads, d*d+d) FP32 state");
    } else if (state.data == nullptr || state.rows != num_heads || state.cols != per_head || state.dtype != Dtype::FP32) {
        state.resize(num_heads, per_head, Dtype::FP32, Q.device);
    }
    if (out.data == nullptr || out.rows != Q.rows || out.cols != Q.cols || out.dtype != Q.dtype)
        out.resize(Q.rows, Q.cols, Q.dtype, Q.device);
    mi_linear_attn_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, Q.dtype);
    a.q = Q.data; a.k = K.data; a.v = V.data; a.o = out.data;
    a.batch = 1; a.num_heads = num_heads; a.head_dim = hd; a.n_tokens = Q.rows;
    a.eps = eps; a.accumulate_state = accumulate_state ? 1 : 0;
    a.workspace = state.data; a.workspace_bytes = state.bytes();
    if (scratch) {
        const std::size_t need = mi_linear_attn_scratch_bytes(1, num_heads, hd);
        if (scratch->data == nullptr || scratch->bytes() < need || scratch->dtype != Dtype::FP32)
            scratch->resize(1, static_cast<int>(need / 4), Dtype::FP32, Q.device);
        a.scratch = scratch->data; a.scratch_bytes = scratch->bytes();
    }
    check(op, mi_linear_attn_relu_forward(&a));
}

void linear_attention_relu_forward_channel_major(const Tensor& Q, const Tensor& K, const Tensor& V, int num_heads, float eps,
                                                 Tensor& state, Tensor& out) {
    const char* op = "linear_attention_relu_forward_channel_major";
    need_gpu(op, Q); need_gpu(op, K); need_gpu(op, V);
    if (num_heads <= 0 || Q.rows % num_heads != 0) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if (K.rows != Q.rows || V.rows != Q.rows || K.cols != Q.cols || V.cols != Q.cols || K.dtype != Q.dtype || V.dtype != Q.dtype)
        fail(std::string(op) + ": Q/K/V must share shape (D, N) and dtype");
    const int hd = Q.rows / num_heads;
    const int per_head = hd * hd + hd;
    if (state.data == nullptr || state.rows != num_heads || state.cols != per_head || state.dtype != Dtype::FP32)
        state.resize(num_heads, per_head, Dtype::FP32, Q.device);
    if (out.data == nullptr || out.rows != Q.rows || out.cols != Q.cols || out.dtype != Q.dtype)
        out.resize(Q.rows, Q.cols, Q.dtype, Q.device);
    mi_linear_attn_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, Q.dtype);
    a.q = Q.data; a.k = K.data; a.v = V.data; a.o = out.data;
    a.batch = 1; a.num_heads = num_heads; a.head_dim = hd; a.n_tokens = Q.cols;
    a.eps = eps;
    a.layout = MI_LAYOUT_CHANNEL_MAJOR;
    a.workspace = state.data; a.workspace_bytes = state.bytes();
    check(op, mi_linear_attn_relu_forward(&a));
}

namespace {
const void* bias_ptr(const char* op, const Tensor* b, const char* name, Dtype dt, int n) {
    if (!b) return nullptr;
    need_gpu(op, *b);
    if (b->dtype != dt || b->size() != static_cast<std::size_t>(n)) fail(std::string(op) + ": " + name + " must hold " + std::to_string(n) + " values of X's dtype");
    return b->data;
}
// scales == nullptr: a weight of the activation dtype; otherwise an INT8 weight with FP32 per-output-row scales.
// Returns the scales pointer for the C ABI.
const float* need_weight(const char* op, const Tensor& W, const char* name, Dtype dt, int rows, int cols, const Tensor* scales = nullptr) {
    need_gpu(op, W);
    if (scales) {
        need_gpu(op, *scales);
        if (W.dtype != Dtype::INT8) fail(std::string(op) + ": " + name + " must be INT8");
        if (scales->dtype != Dtype::FP32 || scales->size() != static_cast<std::size_t>(W.rows))
            fail(std::string(op) + ": " + name + " scales must hold one FP32 value per output row");
    } else if (W.dtype != dt) {
        fail(std::string(op) + ": " + name + " must have X's dtype");
    }
    if ((rows >= 0 && W.rows != rows) || W.cols != cols)
        fail(std::string(op) + ": " + name + " is (" + std::to_string(W.rows) + ", " + std::to_string(W.cols) + "), expected (" +
             (rows >= 0 ? std::to_string(rows) : std::string("out")) + ", " + std::to_string(cols) + ")");
    return scales ? static_cast<const float*>(scales->data) : nullptr;
}
Tensor& thread_scratch() {
    struct BlockScratch;
    return per_stream<Tensor, BlockScratch>();
}
void lend_scratch(mi_attn_block_args& a, Tensor* scratch, bool with_kv) {
    Tensor& s = scratch ? *scratch : thread_scratch();
    const std::size_t need = mi_flash_attention_scratch_bytes(a.batch, a.q_len, a.kv_len, a.inner, with_kv ? 1 : 0);
    if (s.data == nullptr || s.bytes() < need) s.resize(1, static_cast<int>((need + 3) / 4), Dtype::FP32, Device::GPU);
    a.scratch = s.data; a.scratch_bytes = s.bytes();
}
void init_block(mi_attn_block_args& a, const char* op, const Tensor& X, const Tensor& Wq, const Tensor* bq, const Tensor& Wo,
                const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out, const Tensor* q_scales = nullptr,
                const Tensor* o_scales = nullptr) {
    need_gpu(op, X);
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.wq_scales = need_weight(op, Wq, "Wq", X.dtype, -1, X.cols, q_scales);
    a.wo_scales = need_weight(op, Wo, "Wo", X.dtype, -1, Wq.rows, o_scales);
    if (out.data == nullptr || out.rows != X.rows || out.cols != Wo.rows || out.dtype != X.dtype) out.resize(X.rows, Wo.rows, X.dtype, X.device);
    a.x = X.data; a.wq = Wq.data; a.wo = Wo.data; a.out = out.data;
    a.bq = bias_ptr(op, bq, "bq", X.dtype, Wq.rows);
    a.bo = bias_ptr(op, bo, "bo", X.dtype, Wo.rows);
    a.batch = 1; a.q_len = X.rows; a.channels = X.cols; a.inner = Wq.rows; a.out_channels = Wo.rows;
    a.num_heads = num_heads; a.causal = causal ? 1 : 0;
    a.key_mask = d_mask;
}
}  // namespace

namespace {
void linear_impl(const char* op, const Tensor& W, const Tensor* scales, const Tensor* bias, const Tensor& X, Tensor& Y) {
    need_gpu(op, X);
    const float* w_scales = need_weight(op, W, "W", X.dtype, -1, X.cols, scales);
    if (Y.data == nullptr || Y.rows != X.rows || Y.cols != W.rows || Y.dtype != X.dtype) Y.resize(X.rows, W.rows, X.dtype, X.device);
    mi_linear_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.x = X.data; a.w = W.data; a.y = Y.data;
    a.bias = bias_ptr(op, bias, "bias", X.dtype, W.rows);
    a.rows = X.rows; a.in_features = X.cols; a.out_features = W.rows;
    a.w_scales = w_scales;
    check(op, mi_linear_forward(&a));
}
}  // namespace

void linear_batched(const Tensor& W, const Tensor* bias, const Tensor& X, Tensor& Y) { linear_impl("linear_batched", W, nullptr, bias, X, Y); }
void linear_forward_batched_int8w_fp16(const Tensor& W_int8, const Tensor& scales, const Tensor* bias, const Tensor& X, Tensor& Y) {
    linear_impl("linear_forward_batched_int8w_fp16", W_int8, &scales, bias, X, Y);
}

namespace {
struct Scales { const Tensor* q; const Tensor* k; const Tensor* v; const Tensor* o; };
void qkvo_impl(const char* op, const Tensor& X, const Tensor* Ctx, const Tensor& Wq, const Tensor* bq, const Tensor& Wk,
               const Tensor* bk, const Tensor& Wv, const Tensor* bv, const Tensor& Wo, const Tensor* bo, const float* d_mask,
               int num_heads, bool causal, Tensor& out, Tensor* scratch, const Scales& sc) {
    mi_attn_block_args a;
    init_block(a, op, X, Wq, bq, Wo, bo, d_mask, num_heads, causal, out, sc.q, sc.o);
    const Tensor& S = Ctx ? *Ctx : X;
    if (Ctx) { need_gpu(op, S); if (S.dtype != X.dtype) fail(std::string(op) + ": Ctx must have X's dtype"); }
    a.wk_scales = need_weight(op, Wk, "Wk", X.dtype, Wq.rows, S.cols, sc.k);
    a.wv_scales = need_weight(op, Wv, "Wv", X.dtype, Wq.rows, S.cols, sc.v);
    a.ctx = Ctx ? S.data : nullptr;
    a.wk = Wk.data; a.wv = Wv.data;
    a.bk = bias_ptr(op, bk, "bk", X.dtype, Wq.rows);
    a.bv = bias_ptr(op, bv, "bv", X.dtype, Wq.rows);
    a.kv_len = S.rows; a.ctx_channels = S.cols;
    lend_scratch(a, scratch, true);
    check(op, mi_flash_attention_qkvo_forward(&a));
}
void kv_cached_impl(const char* op, const Tensor& X, const Tensor& K, const Tensor& V, const Tensor& Wq, const Tensor* bq,
                    const Tensor& Wo, const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out, Tensor* scratch,
                    const Scales& sc) {
    mi_attn_block_args a;
    init_block(a, op, X, Wq, bq, Wo, bo, d_mask, num_heads, causal, out, sc.q, sc.o);
    need_gpu(op, K); need_gpu(op, V);
    if (K.dtype != X.dtype || V.dtype != X.dtype || K.cols != Wq.rows || V.cols != K.cols || V.rows != K.rows)
        fail(std::string(op) + ": K and V must be (Lk, " + std::to_string(Wq.rows) + ") of X's dtype");
    a.k = K.data; a.v = V.data; a.kv_len = K.rows;
    lend_scratch(a, scratch, false);
    check(op, mi_flash_attention_q_with_kv_cached_forward(&a));
}
void project_kv_impl(const char* op, const Tensor& ctx, const Tensor& Wk, const Tensor* bk, const Tensor& Wv, const Tensor* bv,
                     Tensor& K_out, Tensor& V_out, const Scales& sc) {
    need_gpu(op, ctx);
    const float* wk_scales = need_weight(op, Wk, "Wk", ctx.dtype, -1, ctx.cols, sc.k);
    const float* wv_scales = need_weight(op, Wv, "Wv", ctx.dtype, Wk.rows, ctx.cols, sc.v);
    for (Tensor* t : {&K_out, &V_out})
        if (t->data == nullptr || t->rows != ctx.rows || t->cols != Wk.rows || t->dtype != ctx.dtype) t->resize(ctx.rows, Wk.rows, ctx.dtype, ctx.device);
    mi_attn_block_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, ctx.dtype);
    a.ctx = ctx.data; a.wk = Wk.data; a.wv = Wv.data;
    a.bk = bias_ptr(op, bk, "bk", ctx.dtype, Wk.rows);
    a.bv = bias_ptr(op, bv, "bv", ctx.dtype, Wk.rows);
    a.k = K_out.data; a.v = V_out.data;
    a.batch = 1; a.kv_len = ctx.rows; a.ctx_channels = ctx.cols; a.inner = Wk.rows;
    a.wk_scales = wk_scales; a.wv_scales = wv_scales;
    check(op, mi_flash_attention_project_kv(&a));
}
}  // namespace

void flash_attention_qkvo_forward(const Tensor& X, const Tensor* Ctx, const Tensor& Wq, const Tensor* bq, const Tensor& Wk,
                                  const Tensor* bk, const Tensor& Wv, const Tensor* bv, const Tensor& Wo, const Tensor* bo,
                                  const float* d_mask, int num_heads, bool causal, Tensor& out, Tensor* scratch) {
    qkvo_impl("flash_attention_qkvo_forward", X, Ctx, Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads, causal, out, scratch, Scales{});
}
void flash_attention_qkvo_int8w_fp16(const Tensor& X, const Tensor* Ctx, const Tensor& Wq, const Tensor& Wq_scales, const Tensor* bq,
                                     const Tensor& Wk, const Tensor& Wk_scales, const Tensor* bk, const Tensor& Wv,
                                     const Tensor& Wv_scales, const Tensor* bv, const Tensor& Wo, const Tensor& Wo_scales,
                                     const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out, Tensor* scratch) {
    qkvo_impl("flash_attention_qkvo_int8w_fp16", X, Ctx, Wq, bq, Wk, bk, Wv, bv, Wo, bo, d_mask, num_heads, causal, out, scratch,
              Scales{&Wq_scales, &Wk_scales, &Wv_scales, &Wo_scales});
}
void flash_attention_q_with_kv_cached_forward(const Tensor& X, const Tensor& K, const Tensor& V, const Tensor& Wq, const Tensor* bq,
                                              const Tensor& Wo, const Tensor* bo, const float* d_mask, int num_heads, bool causal,
                                              Tensor& out, Tensor* scratch) {
    kv_cached_impl("flash_attention_q_with_kv_cached_forward", X, K, V, Wq, bq, Wo, bo, d_mask, num_heads, causal, out, scratch, Scales{});
}
void flash_attention_q_with_kv_cached_int8w_fp16(const Tensor& X, const Tensor& K, const Tensor& V, const Tensor& Wq,
                                                 const Tensor& Wq_scales, const Tensor* bq, const Tensor& Wo, const Tensor& Wo_scales,
                                                 const Tensor* bo, const float* d_mask, int num_heads, bool causal, Tensor& out,
                                                 Tensor* scratch) {
    kv_cached_impl("flash_attention_q_with_kv_cached_int8w_fp16", X, K, V, Wq, bq, Wo, bo, d_mask, num_heads, causal, out, scratch,
                   Scales{&Wq_scales, nullptr, nullptr, &Wo_scales});
}
void flash_attention_project_kv(const Tensor& ctx, const Tensor& Wk, const Tensor* bk, const Tensor& Wv, const Tensor* bv,
                                Tensor& K_out, Tensor& V_out) {
    project_kv_impl("flash_attention_project_kv", ctx, Wk, bk, Wv, bv, K_out, V_out, Scales{});
}
void flash_attention_project_kv_int8w_fp16(const Tensor& ctx, const Tensor& Wk, const Tensor& Wk_scales, const Tensor* bk,
                                           const Tensor& Wv, const Tensor& Wv_scales, const Tensor* bv, Tensor& K_out, Tensor& V_out) {
    project_kv_impl("flash_attention_project_kv_int8w_fp16", ctx, Wk, bk, Wv, bv, K_out, V_out, Scales{nullptr, &Wk_scales, &Wv_scales, nullptr});
}

void cross_attention_forward_with_attn(const Tensor& X, const Tensor& Ctx, const Tensor& Wq, const Tensor& Wk, const Tensor& Wv,
                                       const Tensor& Wo, const float* d_mask, const Tensor* logit_bias, int num_heads,
                                       Tensor& out, Tensor& AttnAvg) {
    const char* op = "cross_attention_forward_with_attn";
    need_gpu(op, X); need_gpu(op, Ctx);
    if (Ctx.dtype != X.dtype) fail(std::string(op) + ": Ctx must have X's dtype");
    const int Lq = X.rows, Lk = Ctx.rows;
    if (num_heads <= 0 || Wq.rows % num_heads != 0) fail(std::string(op) + ": num_heads must divide the projection width");
    const float* bias = nullptr;
    if (logit_bias != nullptr) {
        need_gpu(op, *logit_bias);
        if (logit_bias->dtype != Dtype::FP32 || logit_bias->rows != Lq || logit_bias->cols != Lk) fail(std::string(op) + ": logit_bias must be FP32 (Lq, Lk)");
        bias = static_cast<const float*>(logit_bias->data);
    }
    // scratch of this layer (see per_stream): projected Q, K, V, the attention output, the denominators
    struct Work { Tensor q, k, v, a, lse; };
    Work* const w = &per_stream<Work, Work>();
    linear_impl(op, Wq, nullptr, nullptr, X, w->q);
    linear_impl(op, Wk, nullptr, nullptr, Ctx, w->k);
    linear_impl(op, Wv, nullptr, nullptr, Ctx, w->v);
    if (w->k.cols != w->q.cols || w->v.cols != w->q.cols) fail(std::string(op) + ": Wq, Wk and Wv must project to one width");
    if (w->lse.data == nullptr || w->lse.size() < static_cast<std::size_t>(num_heads) * Lq) w->lse.resize(num_heads, Lq, Dtype::FP32, Device::GPU);
    mi_sdpa_args a;
    init_args(a, op, w->q, w->k, w->v, num_heads, num_heads, w->a);
    a.key_mask = d_mask;
    a.logit_bias = bias; a.bias_q0 = 0; a.bias_cols = bias ? Lk : 0;
    a.lse_out = static_cast<float*>(w->lse.data);
    check(op, mi_sdpa_forward(&a));
    if (AttnAvg.data == nullptr || AttnAvg.rows != Lq || AttnAvg.cols != Lk || AttnAvg.dtype != Dtype::FP32) AttnAvg.resize(Lq, Lk, Dtype::FP32, X.device);
    mi_attention_map_args m;
    std::memset(&m, 0, sizeof(m));
    m.struct_size = sizeof(m);
    m.dtype = a.dtype;
    m.q = w->q.data; m.k = w->k.data; m.lse = a.lse_out; m.map = static_cast<float*>(AttnAvg.data);
    m.num_heads = num_heads; m.head_dim = a.head_dim; m.q_len = Lq; m.kv_len = Lk;
    m.logit_bias = bias; m.bias_q0 = 0; m.bias_cols = a.bias_cols;
    m.key_mask = d_mask;
    check(op, mi_attention_map_avg(&m));
    linear_impl(op, Wo, nullptr, nullptr, w->a, out);
}

void mha_forward(const Tensor& X, const Tensor& Wq, const Tensor& Wk, const Tensor& Wv, const Tensor& Wo, const Tensor* bq,
                 const Tensor* bk, const Tensor* bv, const Tensor* bo, const float* d_mask, int num_heads, Tensor& qh,
                 Tensor& kh, Tensor& vh, Tensor& attn, Tensor& yc, Tensor& out) {
    const char* op = "mha_forward";
    (void)attn;
    need_gpu(op, X);
    if (num_heads <= 0 || Wq.rows % num_heads != 0) fail(std::string(op) + ": num_heads must divide the projection width");
    if (Wk.rows != Wq.rows || Wv.rows != Wq.rows || Wo.cols != Wq.rows) fail(std::string(op) + ": Wq, Wk, Wv must project to one width, which Wo takes");
    linear_impl(op, Wq, nullptr, bq, X, qh);
    linear_impl(op, Wk, nullptr, bk, X, kh);
    linear_impl(op, Wv, nullptr, bv, X, vh);
    mi_sdpa_args a;
    init_args(a, op, qh, kh, vh, num_heads, num_heads, yc);
    a.key_mask = d_mask;
    run_sdpa(op, a);
    linear_impl(op, Wo, nullptr, bo, yc, out);
}

}  // namespace bt

namespace {
void geglu_impl(const char* op, const Tensor& X, const Tensor& W, const Tensor* scales, const Tensor& b, Tensor& Y) {
    need_gpu(op, X); need_gpu(op, W); need_gpu(op, b);
    if (scales) need_gpu(op, *scales);
    if (W.rows % 2 != 0 || W.cols != X.cols) fail(std::string(op) + ": W must be (2*D_out, D_in)");
    if (scales) {
        if (W.dtype != Dtype::INT8) fail(std::string(op) + ": W_int8 must be INT8");
        if (scales->dtype != Dtype::FP32 || scales->size() != static_cast<std::size_t>(W.rows))
            fail(std::string(op) + ": W_scales must hold one FP32 value per row of W");
    } else if (W.dtype != X.dtype) {
        fail(std::string(op) + ": W must have X's dtype");
    }
    const int d_out = W.rows / 2;
    if (b.dtype != X.dtype || b.size() != static_cast<std::size_t>(W.rows)) fail(std::string(op) + ": b must hold 2*D_out values of X's dtype");
    if (Y.data == nullptr || Y.rows != X.rows || Y.cols != d_out || Y.dtype != X.dtype) Y.resize(X.rows, d_out, X.dtype, X.device);
    mi_linear_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.x = X.data; a.w = W.data; a.bias = b.data; a.y = Y.data;
    a.w_scales = scales ? static_cast<const float*>(scales->data) : nullptr;
    a.rows = X.rows; a.in_features = X.cols; a.out_features = d_out;
    check(op, mi_linear_geglu_forward(&a));
}
}  // namespace

void fused_linear_geglu(const Tensor& X, const Tensor& W, const Tensor& b, Tensor& Y) { geglu_impl("fused_linear_geglu", X, W, nullptr, b, Y); }
void fused_linear_geglu(const Tensor& X, const Tensor& W_int8, const Tensor& W_scales, const Tensor& b, Tensor& Y) {
    geglu_impl("fused_linear_geglu(int8w)", X, W_int8, &W_scales, b, Y);
}

void add_inplace_vec(Tensor& Y, const Tensor& X) {
    const char* op = "add_inplace_vec";
    need_gpu(op, Y); need_gpu(op, X);
    if (Y.rows != X.rows || Y.cols != X.cols || Y.dtype != X.dtype) fail(std::string(op) + ": Y and X must match in shape and dtype");
    check(op, mi_add_inplace(Y.data, X.data, static_cast<int64_t>(Y.size()), dtype_code(op, Y.dtype), nullptr));
}

void add_inplace_row_bias(Tensor& Y, const Tensor& bias) {
    const char* op = "add_inplace_row_bias";
    need_gpu(op, Y); need_gpu(op, bias);
    if (bias.dtype != Y.dtype || bias.size() != static_cast<std::size_t>(Y.cols)) fail(std::string(op) + ": bias must hold Y.cols values of Y's dtype");
    check(op, mi_add_row_bias(Y.data, bias.data, Y.rows, Y.cols, 0, dtype_code(op, Y.dtype), nullptr));
}

namespace dit {

RopeTables build_axial_rope_tables(int txt_len, int hp, int wp, int head_dim, const std::vector<int>& axes, float theta) {
    if (head_dim % 2 != 0) fail("build_axial_rope_tables: head_dim must be even");
    int sum = 0;
    for (int d : axes) sum += d;
    if (sum != head_dim) fail("build_axial_rope_tables: axes_dims_rope must sum to head_dim");
    const int half = head_dim / 2;
    const std::size_t L = static_cast<std::size_t>(txt_len) + static_cast<std::size_t>(hp) * wp;
    std::vector<float> cs(L * half, 1.0f), sn(L * half, 0.0f);
    // per pair: owning axis and angular frequency theta^(-2p/D_a); positions (0, i, j)
    std::vector<int> pair_axis(half);
    std::vector<double> omega(half);
    int off = 0;
    for (std::size_t a = 0; a < axes.size(); ++a) {
        for (int p = 0; p < axes[a] / 2; ++p) {
            pair_axis[off + p] = static_cast<int>(a);
            omega[off + p] = std::pow(static_cast<double>(theta), -2.0 * p / static_cast<double>(axes[a]));
        }
        off += axes[a] / 2;
    }
    for (int i = 0; i < hp; ++i)
        for (int j = 0; j < wp; ++j) {
            const std::size_t row = static_cast<std::size_t>(txt_len) + static_cast<std::size_t>(i) * wp + j;
            for (int p = 0; p < half; ++p) {
                const int ax = pair_axis[p];
                if (ax > 2) continue;
                const double ang = (ax == 0 ? 0.0 : ax == 1 ? static_cast<double>(i) : static_cast<double>(j)) * omega[p];
                cs[row * half + p] = static_cast<float>(std::cos(ang));
                sn[row * half + p] = static_cast<float>(std::sin(ang));
            }
        }
    RopeTables t;
    t.cos = Tensor::from_host(cs.data(), static_cast<int>(L), half, Dtype::FP32);
    t.sin = Tensor::from_host(sn.data(), static_cast<int>(L), half, Dtype::FP32);
    return t;
}

RopeTables build_qwen_rope_tables(const std::vector<QwenSegment>& prefix, int hp, int wp, int head_dim,
                                  const std::vector<int>& axes, float theta) {
    if (head_dim % 2 != 0) fail("build_qwen_rope_tables: head_dim must be even");
    if (axes.size() != 3 || axes[0] + axes[1] + axes[2] != head_dim) fail("build_qwen_rope_tables: three axes_dims_rope summing to head_dim");
    // positions (frame, height, width) of every token, in sequence order
    struct Pos { int f, h, w; };
    std::vector<Pos> at;
    int cursor = 0;
    auto image = [&](int h, int w) {
        const int top = -(h - h / 2), left = -(w - w / 2);
        for (int i = 0; i < h; ++i)
            for (int j = 0; j < w; ++j) at.push_back({cursor, top + i, left + j});
        cursor += std::max(h, w);
    };
    for (const QwenSegment& s : prefix) {
        if (s.kind == QwenSegment::Kind::Text) {
            for (int i = 0; i < s.n_tokens; ++i, ++cursor) at.push_back({cursor, cursor, cursor});
        } else {
            image(s.h, s.w);
        }
    }
    image(hp, wp);
    const int half = head_dim / 2;
    const std::size_t L = at.size();
    std::vector<float> cs(L * half), sn(L * half);
    int col = 0;
    for (int a = 0; a < 3; ++a)
        for (int p = 0; p < axes[a] / 2; ++p, ++col) {
            const double omega = std::pow(static_cast<double>(theta), -2.0 * p / static_cast<double>(axes[a]));
            for (std::size_t r = 0; r < L; ++r) {
                const int x = a == 0 ? at[r].f : a == 1 ? at[r].h : at[r].w;
                const double ang = static_cast<double>(x) * omega;
                cs[r * half + col] = static_cast<float>(std::cos(ang));
                sn[r * half + col] = static_cast<float>(std::sin(ang));
            }
        }
    RopeTables t;
    t.cos = Tensor::from_host(cs.data(), static_cast<int>(L), half, Dtype::FP32);
    t.sin = Tensor::from_host(sn.data(), static_cast<int>(L), half, Dtype::FP32);
    return t;
}

void headnorm_rope(const Tensor& X, const Tensor& gain, float eps, const Tensor* cos, const Tensor* sin, int head_dim,
                   int num_heads, Tensor& out, Tensor* cache_out, int cache_rows) {
    const char* op = "headnorm_rope";
    need_gpu(op, X); need_gpu(op, gain);
    if (head_dim <= 0 || num_heads <= 0 || X.cols != head_dim * num_heads) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if (gain.dtype != X.dtype || gain.size() != static_cast<std::size_t>(head_dim)) fail(std::string(op) + ": gain must hold head_dim values of X's dtype");
    if ((cos == nullptr) != (sin == nullptr)) fail(std::string(op) + ": cos and sin must be given together");
    if (cos) {
        need_gpu(op, *cos); need_gpu(op, *sin);
        if (cos->dtype != Dtype::FP32 || sin->dtype != Dtype::FP32 || cos->rows != X.rows || sin->rows != X.rows ||
            cos->cols != head_dim / 2 || sin->cols != head_dim / 2)
            fail(std::string(op) + ": cos/sin must be FP32 (L, head_dim/2)");
    }
    if (cache_out && (cache_rows < 0 || cache_rows > X.rows)) fail(std::string(op) + ": cache_rows outside 0..L");
    if (out.data == nullptr || out.rows != X.rows || out.cols != X.cols || out.dtype != X.dtype) out.resize(X.rows, X.cols, X.dtype, X.device);
    mi_headnorm_rope_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.x = X.data; a.out = out.data; a.gain = gain.data;
    a.cos = cos ? static_cast<const float*>(cos->data) : nullptr;
    a.sin = sin ? static_cast<const float*>(sin->data) : nullptr;
    a.eps = eps;
    a.split_half = bt::rope_split_half() ? 1 : 0;
    a.rows = X.rows; a.num_heads = num_heads; a.head_dim = head_dim;
    if (cache_out && cache_rows > 0) {
        if (cache_out->data == nullptr || cache_out->rows != cache_rows || cache_out->cols != X.cols || cache_out->dtype != X.dtype)
            cache_out->resize(cache_rows, X.cols, X.dtype, X.device);
        a.out2 = cache_out->data; a.out2_rows = cache_rows;
    }
    check(op, mi_headnorm_rope(&a));
}

void joint_attention(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor& cos, const Tensor& sin, int head_dim,
                     int num_heads, Tensor& out, Tensor& /*Qr*/, Tensor& Kr) {
    const char* op = "joint_attention";
    if (head_dim <= 0 || num_heads <= 0 || Q.cols != head_dim * num_heads) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if (K.rows != Q.rows || V.rows != Q.rows || K.cols != Q.cols || V.cols != Q.cols) fail(std::string(op) + ": Q/K/V must share shape (L, D)");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_heads, num_heads, out);
    set_rope(a, op, &cos, &sin, Q.rows, true);
    set_rope(a, op, &cos, &sin, K.rows, false);
    Kr.resize(K.rows, K.cols, K.dtype, K.device);  // receives RoPE(K), as in the reference
    a.rope_k_scratch = Kr.data;
    a.rope_split_half = bt::rope_split_half() ? 1 : 0;
    run_sdpa(op, a);
}

void joint_attention_traced(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor& cos, const Tensor& sin,
                            int head_dim, int num_heads, Tensor& out, Tensor& attn_avg, Tensor& Qr, Tensor& Kr, int txt_len,
                            const Tensor* image_text_bias) {
    const char* op = "joint_attention_traced";
    bt::rope_apply(Q, cos, sin, head_dim, num_heads, Qr);
    bt::rope_apply(K, cos, sin, head_dim, num_heads, Kr);
    const int D = Q.cols, L = Q.rows;
    if (head_dim <= 0 || num_heads <= 0 || D != head_dim * num_heads) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if (K.rows != L || V.rows != L || K.cols != D || V.cols != D) fail(std::string(op) + ": Q/K/V must share shape (L, D)");
    const float* bias = nullptr;
    if (image_text_bias != nullptr) {
        if (txt_len < 0 || txt_len > L) fail(std::string(op) + ": txt_len out of range for bias");
        if (image_text_bias->dtype != Dtype::FP32) fail(std::string(op) + ": image_text_bias must be FP32");
        if (image_text_bias->rows != L - txt_len || image_text_bias->cols != txt_len) fail(std::string(op) + ": image_text_bias must be (img_len, txt_len)");
        need_gpu(op, *image_text_bias);
        if (txt_len > 0 && txt_len < L) bias = static_cast<const float*>(image_text_bias->data);
    }
    struct TracedLse;
    Tensor* const lse = &per_stream<Tensor, TracedLse>();   // scratch of this layer (see per_stream)
    if (lse->data == nullptr || lse->size() < static_cast<std::size_t>(num_heads) * L) lse->resize(num_heads, L, Dtype::FP32, Device::GPU);
    mi_sdpa_args a;
    init_args(a, op, Qr, Kr, V, num_heads, num_heads, out);
    a.logit_bias = bias; a.bias_q0 = txt_len; a.bias_cols = bias ? txt_len : 0;
    a.lse_out = static_cast<float*>(lse->data);
    check(op, mi_sdpa_forward(&a));
    if (attn_avg.data == nullptr || attn_avg.rows != L || attn_avg.cols != L || attn_avg.dtype != Dtype::FP32) attn_avg.resize(L, L, Dtype::FP32, Q.device);
    mi_attention_map_args m;
    std::memset(&m, 0, sizeof(m));
    m.struct_size = sizeof(m);
    m.dtype = a.dtype;
    m.q = Qr.data; m.k = Kr.data; m.lse = a.lse_out; m.map = static_cast<float*>(attn_avg.data);
    m.num_heads = num_heads; m.head_dim = head_dim; m.q_len = L; m.kv_len = L;
    m.logit_bias = bias; m.bias_q0 = txt_len; m.bias_cols = a.bias_cols;
    check(op, mi_attention_map_avg(&m));
}

void gqa_attention_masked(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor* cos, const Tensor* sin, int head_dim,
                          int num_q_heads, int num_kv_heads, const float* d_mask, Tensor& out, Tensor& /*Qr*/, Tensor& Kr,
                          Tensor& /*Krep*/, Tensor& /*Vrep*/) {
    const char* op = "gqa_attention_masked";
    if (num_kv_heads <= 0 || num_q_heads <= 0 || num_q_heads % num_kv_heads != 0)
        fail(std::string(op) + ": num_kv_heads must divide num_q_heads");
    if (Q.cols != head_dim * num_q_heads) fail(std::string(op) + ": D must equal head_dim * num_q_heads");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_q_heads, num_kv_heads, out);
    a.key_mask = d_mask;
    set_rope(a, op, cos, sin, Q.rows, true);
    set_rope(a, op, cos, sin, K.rows, false);
    if (cos) {
        Kr.resize(K.rows, K.cols, K.dtype, K.device);
        a.rope_k_scratch = Kr.data;
        a.rope_split_half = bt::rope_split_half() ? 1 : 0;
    }
    run_sdpa(op, a);
}

void scale_rows(const Tensor& X, float scale, const Tensor* row_scale, Tensor& out) {
    const char* op = "scale_rows";
    need_gpu(op, X);
    if (row_scale) {
        need_gpu(op, *row_scale);
        if (row_scale->dtype != Dtype::FP32 || row_scale->size() != static_cast<std::size_t>(X.rows))
            fail(std::string(op) + ": the row scale holds " + std::to_string(row_scale->size()) + " values but the tensor has " +
                 std::to_string(X.rows) + " rows");
    }
    if (out.data == nullptr || out.rows != X.rows || out.cols != X.cols || out.dtype != X.dtype) out.resize(X.rows, X.cols, X.dtype, X.device);
    mi_scale_rows_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, X.dtype);
    a.x = X.data; a.out = out.data;
    a.row_scale = row_scale ? static_cast<const float*>(row_scale->data) : nullptr;
    a.scale = scale;
    a.rows = X.rows; a.cols = X.cols;
    check(op, mi_scale_rows(&a));
}

void block_causal_attention(const Tensor& Q, const Tensor& K, const Tensor& V, const Tensor* k_prefix, const Tensor* v_prefix,
                            const std::vector<Segment>& segments, int q_offset, int num_heads, const Tensor* cos_q,
                            const Tensor* sin_q, Tensor& out, const PrefixDial* dial) {
    const char* op = "block_causal_attention";
    if (segments.empty() || segments.size() > static_cast<std::size_t>(MI_MAX_SEGMENTS))
        fail(std::string(op) + ": between 1 and 32 segments");
    mi_sdpa_args a;
    init_args(a, op, Q, K, V, num_heads, num_heads, out);
    if ((k_prefix == nullptr) != (v_prefix == nullptr)) fail(std::string(op) + ": prefix K and V must be given together");
    if (k_prefix && k_prefix->rows > 0) {
        need_gpu(op, *k_prefix); need_gpu(op, *v_prefix);
        if (k_prefix->cols != K.cols || v_prefix->cols != K.cols || v_prefix->rows != k_prefix->rows ||
            k_prefix->dtype != Q.dtype || v_prefix->dtype != Q.dtype)
            fail(std::string(op) + ": prefix K/V must be (prefix_len, D) in Q's dtype");
        a.k_prefix = k_prefix->data; a.v_prefix = v_prefix->data; a.prefix_len = k_prefix->rows;
    }
    if (dial && a.prefix_len > 0) {
        a.prefix_k_scale = dial->k_scale; a.prefix_v_scale = dial->v_scale;
        for (const Tensor* rows : {dial->k_rows, dial->v_rows}) {
            if (!rows) continue;
            need_gpu(op, *rows);
            if (rows->dtype != Dtype::FP32 || rows->size() != static_cast<std::size_t>(a.prefix_len))
                fail(std::string(op) + ": the dial's row weights must hold prefix_len FP32 values");
        }
        a.prefix_k_row_scale = dial->k_rows ? static_cast<const float*>(dial->k_rows->data) : nullptr;
        a.prefix_v_row_scale = dial->v_rows ? static_cast<const float*>(dial->v_rows->data) : nullptr;
    }
    a.mask_mode = MI_MASK_BLOCK_CAUSAL;
    a.q_offset = q_offset;
    a.n_segments = static_cast<int>(segments.size());
    int row = 0;
    for (std::size_t s = 0; s < segments.size(); ++s) {
        row += segments[s].n_tokens;
        a.seg_q_end[s] = row;
        a.seg_k_end[s] = q_offset + row;           // a segment sees every key up to its own end
        a.seg_causal[s] = segments[s].kind == Segment::Kind::Text ? 1 : 0;
    }
    if (row != Q.rows) fail(std::string(op) + ": segments must cover exactly Q's rows");
    // fresh keys get the same table rows as the queries when Q and K cover the same positions
    set_rope(a, op, cos_q, sin_q, Q.rows, true);
    if (cos_q && K.rows == Q.rows) set_rope(a, op, cos_q, sin_q, K.rows, false);
    else if (cos_q) fail(std::string(op) + ": fused RoPE needs K and Q to cover the same positions");
    run_sdpa(op, a);
}

void rms_norm_rows(const Tensor& X, const Tensor& gain, float eps, Tensor& out) {
    const char* op = "rms_norm_rows";
    need_gpu(op, X); need_gpu(op, gain);
    if (gain.dtype != X.dtype || gain.size() != static_cast<std::size_t>(X.cols)) fail(std::string(op) + ": gain must hold one value of X's dtype per column");
    if (out.data == nullptr || out.rows != X.rows || out.cols != X.cols || out.dtype != X.dtype) out.resize(X.rows, X.cols, X.dtype, X.device);
    check(op, mi_rms_norm_forward(X.data, gain.data, out.data, X.rows, X.cols, 0, 0, eps, dtype_code(op, X.dtype), nullptr));
}

void sana_self_attention(const Tensor& x_mod, const SanaAttnWeights& w, int num_heads, Tensor& out, SanaAttnScratch& sc,
                         RefMode ref_mode, Tensor* ref_state, float ref_weight, float rms_eps, float attn_eps) {
    const char* op = "sana_self_attention";
    need_gpu(op, x_mod);
    const int N = x_mod.rows, D = x_mod.cols;
    if (!w.Wq || !w.Wk || !w.Wv || !w.Wo) fail(std::string(op) + ": Wq, Wk, Wv and Wo are required");
    if (num_heads <= 0 || D % num_heads != 0) fail(std::string(op) + ": D must equal head_dim * num_heads");
    if ((w.nq == nullptr) != (w.nk == nullptr)) fail(std::string(op) + ": the qk_norm gains come as a pair");
    const int hd = D / num_heads, per_head = hd * hd + hd;
    if (ref_mode != RefMode::Off && ref_state == nullptr) fail(std::string(op) + ": capture / inject needs ref_state");
    if (ref_mode == RefMode::Inject &&
        (ref_state->data == nullptr || ref_state->rows != num_heads || ref_state->cols != per_head || ref_state->dtype != Dtype::FP32))
        fail(std::string(op) + ": inject needs a (heads, (head_dim + 1) * head_dim) FP32 ref_state");
    bt::linear_batched(*w.Wq, nullptr, x_mod, sc.q);
    bt::linear_batched(*w.Wk, nullptr, x_mod, sc.k);
    bt::linear_batched(*w.Wv, nullptr, x_mod, sc.v);
    if (w.nq) {
        rms_norm_rows(sc.q, *w.nq, rms_eps, sc.q);
        rms_norm_rows(sc.k, *w.nk, rms_eps, sc.k);
    }
    // the state this call computes lands in the caller's ref_state when capturing, else in the scratch
    Tensor& state = ref_mode == RefMode::Capture ? *ref_state : sc.state;
    if (state.data == nullptr || state.rows != num_heads || state.cols != per_head || state.dtype != Dtype::FP32)
        state.resize(num_heads, per_head, Dtype::FP32, x_mod.device);
    if (ref_mode == RefMode::Inject) {
        // the anchor stays as it is: a copy of it takes this call's (S, z) on top, weighted
        if (mi_memcpy_d2d_async(state.data, ref_state->data, state.bytes(), nullptr) != 0) fail(std::string(op) + ": " + mi_last_error());
    }
    if (sc.attn.data == nullptr || sc.attn.rows != N || sc.attn.cols != D || sc.attn.dtype != x_mod.dtype) sc.attn.resize(N, D, x_mod.dtype, x_mod.device);
    mi_linear_attn_args a;
    std::memset(&a, 0, sizeof(a));
    a.struct_size = sizeof(a);
    a.dtype = dtype_code(op, x_mod.dtype);
    a.q = sc.q.data; a.k = sc.k.data; a.v = sc.v.data; a.o = sc.attn.data;
    a.batch = 1; a.num_heads = num_heads; a.head_dim = hd; a.n_tokens = N;
    a.eps = attn_eps;
    a.accumulate_state = ref_mode == RefMode::Inject ? 1 : 0;
    a.accumulate_weight = ref_weight;
    if (ref_mode == RefMode::Inject && ref_weight == 0.f) a.accumulate_state = 0;    // weight 0: the anchor does not take part
    a.workspace = state.data; a.workspace_bytes = state.bytes();
    const std::size_t need = mi_linear_attn_scratch_bytes(1, num_heads, hd);
    if (sc.partials.data == nullptr || sc.partials.bytes() < need || sc.partials.dtype != Dtype::FP32)
        sc.partials.resize(1, static_cast<int>(need / 4), Dtype::FP32, x_mod.device);
    a.scratch = sc.partials.data; a.scratch_bytes = sc.partials.bytes();
    check(op, mi_linear_attn_relu_forward(&a));
    bt::linear_batched(*w.Wo, w.bo, sc.attn, out);
}

}  // namespace dit
}  // namespace bdamd
