// Attention with its input and output projections, and the stand-alone linear layer: host-side sequencing of the
// projection GEMM (linear.hip) and the softmax-attention kernels behind the C ABI. Three launches for the whole block:
// Q/K/V projections (one grid), attention, output projection. Nothing is allocated; intermediates live in the
// caller's scratch.
#include <cstring>

#include "internal.h"

namespace mi {
namespace {

constexpr size_t kAlign = 256;
size_t round_up(size_t n) { return (n + kAlign - 1) / kAlign * kAlign; }

struct BlockDims {
    long q_rows, kv_rows;
    int head_dim;
    size_t q_bytes, kv_bytes;
};

int check_common(const mi_attn_block_args* a, const char* op, BlockDims& d, bool needs_q) {
    if (!a) return fail("%s: null args", op);
    if (a->struct_size != sizeof(mi_attn_block_args))
        return fail("%s: struct_size %u != %zu (header mismatch)", op, a->struct_size, sizeof(mi_attn_block_args));
    if (a->dtype != MI_DTYPE_F16 && a->dtype != MI_DTYPE_BF16) return fail("%s: dtype %d is neither MI_DTYPE_F16 nor MI_DTYPE_BF16", op, a->dtype);
    if (a->batch <= 0) return fail("%s: batch must be positive", op);
    if (a->q_len < 0 || a->kv_len < 0) return fail("%s: negative length", op);
    if (a->inner <= 0 || a->inner % 8) return fail("%s: inner %d must be a positive multiple of 8", op, a->inner);
    if (needs_q) {
        if (a->num_heads <= 0 || a->inner % a->num_heads) return fail("%s: num_heads %d does not divide inner %d", op, a->num_heads, a->inner);
        d.head_dim = a->inner / a->num_heads;
        if (!sdpa_supported(a->dtype, d.head_dim)) return fail("%s: no attention kernel for dtype %d head_dim %d", op, a->dtype, d.head_dim);
    }
    const int kv_len = (needs_q && !a->ctx && !a->k) ? a->q_len : a->kv_len;
    d.q_rows = static_cast<long>(a->batch) * a->q_len;
    d.kv_rows = static_cast<long>(a->batch) * kv_len;
    if (d.q_rows > 0x7fffffffL || d.kv_rows > 0x7fffffffL) return fail("%s: too many rows", op);
    d.q_bytes = round_up(static_cast<size_t>(d.q_rows) * a->inner * 2);
    d.kv_bytes = round_up(static_cast<size_t>(d.kv_rows) * a->inner * 2);
    return 0;
}

LinearProblem problem(const void* x, const void* w, const void* bias, void* y, long M, int N, int K, const float* w_scale = nullptr) {
    LinearProblem p;
    p.x = x; p.w = w; p.bias = bias; p.y = y;
    p.w_scale = w_scale;
    p.M = static_cast<int>(M); p.N = N; p.K = K;
    p.ldx = K; p.ldw = K; p.ldy = N;
    return p;
}

int attend(const mi_attn_block_args* a, const BlockDims& d, const void* q, const void* k, const void* v, void* o, int kv_len) {
    mi_sdpa_args s;
    std::memset(&s, 0, sizeof(s));
    s.struct_size = sizeof(s);
    s.dtype = a->dtype;
    s.q = q; s.k = k; s.v = v; s.o = o;
    s.batch = a->batch; s.num_heads = a->num_heads; s.head_dim = d.head_dim;
    s.q_len = a->q_len; s.kv_len = kv_len;
    s.key_mask = a->key_mask; s.key_mask_batch_stride = a->key_mask_batch_stride;
    if (a->causal) { s.mask_mode = MI_MASK_CAUSAL; s.q_offset = kv_len - a->q_len; }
    s.stream = a->stream;
    return mi_sdpa_forward(&s);
}

}  // namespace
}  // namespace mi

using mi::fail;

extern "C" {

int mi_linear_forward(const mi_linear_args* a) {
    mi::clear_error();
    if (!a) return fail("mi_linear_forward: null args");
    if (a->struct_size != sizeof(mi_linear_args))
        return fail("mi_linear_forward: struct_size %u != %zu (header mismatch)", a->struct_size, sizeof(mi_linear_args));
    if (a->rows < 0) return fail("mi_linear_forward: negative rows");
    if (a->rows == 0) return 0;
    mi::LinearBatch b;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(a->x, a->w, a->bias, a->y, a->rows, a->out_features, a->in_features, a->w_scales);
    if (a->x_row_stride) b.p[0].ldx = a->x_row_stride;
    if (a->w_row_stride) b.p[0].ldw = a->w_row_stride;
    if (a->y_row_stride) b.p[0].ldy = a->y_row_stride;
    return mi::launch_linear(b, 1, a->dtype, mi::resolve_stream(a->stream));
}

int mi_linear_geglu_forward(const mi_linear_args* a) {
    mi::clear_error();
    if (!a) return fail("mi_linear_geglu_forward: null args");
    if (a->struct_size != sizeof(mi_linear_args))
        return fail("mi_linear_geglu_forward: struct_size %u != %zu (header mismatch)", a->struct_size, sizeof(mi_linear_args));
    if (a->rows < 0) return fail("mi_linear_geglu_forward: negative rows");
    if (a->rows == 0) return 0;
    mi::LinearBatch b;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(a->x, a->w, a->bias, a->y, a->rows, a->out_features, a->in_features, a->w_scales);
    if (a->x_row_stride) b.p[0].ldx = a->x_row_stride;
    if (a->w_row_stride) b.p[0].ldw = a->w_row_stride;
    if (a->y_row_stride) b.p[0].ldy = a->y_row_stride;
    return mi::launch_linear(b, 1, a->dtype, mi::resolve_stream(a->stream), true);
}

size_t mi_flash_attention_scratch_bytes(int32_t batch, int32_t q_len, int32_t kv_len, int32_t inner, int32_t with_kv) {
    if (batch <= 0 || q_len < 0 || kv_len < 0 || inner <= 0) return 0;
    const size_t q = mi::round_up(static_cast<size_t>(batch) * q_len * inner * 2);
    const size_t kv = mi::round_up(static_cast<size_t>(batch) * kv_len * inner * 2);
    return 2 * q + (with_kv ? 2 * kv : 0);
}

int mi_flash_attention_project_kv(const mi_attn_block_args* a) {
    mi::clear_error();
    const char* op = "mi_flash_attention_project_kv";
    mi::BlockDims d{};
    if (mi::check_common(a, op, d, false) != 0) return -1;
    if (d.kv_rows == 0) return 0;
    if (!a->ctx || !a->wk || !a->wv || !a->k || !a->v) return fail("%s: ctx, wk, wv, k and v must not be null", op);
    mi::LinearBatch b;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(a->ctx, a->wk, a->bk, a->k, d.kv_rows, a->inner, a->ctx_channels, a->wk_scales);
    b.p[1] = mi::problem(a->ctx, a->wv, a->bv, a->v, d.kv_rows, a->inner, a->ctx_channels, a->wv_scales);
    return mi::launch_linear(b, 2, a->dtype, mi::resolve_stream(a->stream));
}

int mi_flash_attention_qkvo_forward(const mi_attn_block_args* a) {
    mi::clear_error();
    const char* op = "mi_flash_attention_qkvo_forward";
    mi::BlockDims d{};
    if (a && a->k) return fail("%s: k / v are not used by this form (K and V are projected into the scratch)", op);
    if (mi::check_common(a, op, d, true) != 0) return -1;
    if (d.q_rows == 0) return 0;
    if (!a->x || !a->wq || !a->wk || !a->wv || !a->wo || !a->out) return fail("%s: x, wq, wk, wv, wo and out must not be null", op);
    const int kv_len = a->ctx ? a->kv_len : a->q_len;
    const int kv_channels = a->ctx ? a->ctx_channels : a->channels;
    const void* src = a->ctx ? a->ctx : a->x;
    const size_t need = 2 * d.q_bytes + 2 * d.kv_bytes;
    if (!a->scratch || a->scratch_bytes < need) return fail("%s: scratch of %zu bytes needed, %zu given", op, need, a->scratch ? a->scratch_bytes : size_t{0});
    if (reinterpret_cast<uintptr_t>(a->scratch) & 15u) return fail("%s: scratch must be 16-byte aligned", op);
    char* sq = static_cast<char*>(a->scratch);
    char* sa = sq + d.q_bytes;
    char* sk = sa + d.q_bytes;
    char* sv = sk + d.kv_bytes;
    hipStream_t st = mi::resolve_stream(a->stream);

    mi::LinearBatch b;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(a->x, a->wq, a->bq, sq, d.q_rows, a->inner, a->channels, a->wq_scales);
    int n = 1;
    if (d.kv_rows > 0) {
        b.p[1] = mi::problem(src, a->wk, a->bk, sk, d.kv_rows, a->inner, kv_channels, a->wk_scales);
        b.p[2] = mi::problem(src, a->wv, a->bv, sv, d.kv_rows, a->inner, kv_channels, a->wv_scales);
        n = 3;
    }
    if (mi::launch_linear(b, n, a->dtype, st) != 0) return -1;
    if (mi::attend(a, d, sq, sk, sv, sa, kv_len) != 0) return -1;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(sa, a->wo, a->bo, a->out, d.q_rows, a->out_channels, a->inner, a->wo_scales);
    return mi::launch_linear(b, 1, a->dtype, st);
}

int mi_flash_attention_q_with_kv_cached_forward(const mi_attn_block_args* a) {
    mi::clear_error();
    const char* op = "mi_flash_attention_q_with_kv_cached_forward";
    mi::BlockDims d{};
    if (a && (!a->k || !a->v) && a->kv_len > 0) return fail("%s: k and v must not be null", op);
    if (mi::check_common(a, op, d, true) != 0) return -1;
    if (d.q_rows == 0) return 0;
    if (!a->x || !a->wq || !a->wo || !a->out) return fail("%s: x, wq, wo and out must not be null", op);
    const size_t need = 2 * d.q_bytes;
    if (!a->scratch || a->scratch_bytes < need) return fail("%s: scratch of %zu bytes needed, %zu given", op, need, a->scratch ? a->scratch_bytes : size_t{0});
    if (reinterpret_cast<uintptr_t>(a->scratch) & 15u) return fail("%s: scratch must be 16-byte aligned", op);
    char* sq = static_cast<char*>(a->scratch);
    char* sa = sq + d.q_bytes;
    hipStream_t st = mi::resolve_stream(a->stream);

    mi::LinearBatch b;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(a->x, a->wq, a->bq, sq, d.q_rows, a->inner, a->channels, a->wq_scales);
    if (mi::launch_linear(b, 1, a->dtype, st) != 0) return -1;
    if (mi::attend(a, d, sq, a->k, a->v, sa, a->kv_len) != 0) return -1;
    std::memset(&b, 0, sizeof(b));
    b.p[0] = mi::problem(sa, a->wo, a->bo, a->out, d.q_rows, a->out_channels, a->inner, a->wo_scales);
    return mi::launch_linear(b, 1, a->dtype, st);
}

}  // extern "C"
