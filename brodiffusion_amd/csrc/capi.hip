// C ABI of libmi_attention.so: argument validation, error reporting, stream and memory
// helpers. All HIP calls of the library live behind these entry points.
#include <cmath>
#include <cstdio>
#include <cstring>

#include "internal.h"

namespace mi {
namespace {
thread_local char g_err[512] = "";
thread_local hipStream_t g_stream = nullptr;
thread_local int g_kernel_choice = 0;
}  // namespace

int fail(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return -1;
}
void clear_error() { g_err[0] = '\0'; }
hipStream_t resolve_stream(void* s) { return s ? static_cast<hipStream_t>(s) : g_stream; }
int sdpa_kernel_choice() { return g_kernel_choice; }
int device_cu_count() {
    static thread_local int n = 0;
    if (n == 0) {
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
            n = 256;
    }
    return n;
}

namespace {
bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
}  // namespace
}  // namespace mi

using mi::fail;

extern "C" {

const char* mi_last_error(void) { return mi::g_err; }
const char* mi_version(void) { return "mi_attention 0.1 (gfx950)"; }

int mi_device_info(mi_device_info_t* out) {
    mi::clear_error();
    if (!out) return fail("mi_device_info: null output");
    int dev = 0;
    MI_HIP_CHECK(hipGetDevice(&dev));
    hipDeviceProp_t p;
    MI_HIP_CHECK(hipGetDeviceProperties(&p, dev));
    std::memset(out, 0, sizeof(*out));
    std::snprintf(out->name, sizeof(out->name), "%s", p.name);
    std::snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
    out->compute_units = p.multiProcessorCount;
    out->clock_khz = p.clockRate;
    out->lds_bytes_per_cu = static_cast<int32_t>(p.maxSharedMemoryPerMultiProcessor);
    out->l2_bytes = p.l2CacheSize;
    out->hbm_bytes = static_cast<int64_t>(p.totalGlobalMem);
    out->peak_mfma_16bit_flops = static_cast<double>(p.multiProcessorCount) * p.clockRate * 1e3 * 4096.0;
    return 0;
}

int mi_set_stream(void* stream) { mi::clear_error(); mi::g_stream = static_cast<hipStream_t>(stream); return 0; }
void* mi_get_stream(void) { return mi::g_stream; }
int mi_stream_synchronize(void* stream) {
    mi::clear_error();
    MI_HIP_CHECK(hipStreamSynchronize(mi::resolve_stream(stream)));
    return 0;
}

void* mi_malloc(size_t bytes) {
    mi::clear_error();
    void* p = nullptr;
    const hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) { fail("mi_malloc(%zu): %s", bytes, hipGetErrorString(e)); return nullptr; }
    return p;
}
int mi_free(void* ptr) { mi::clear_error(); if (ptr) MI_HIP_CHECK(hipFree(ptr)); return 0; }
int mi_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    mi::clear_error(); MI_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice)); return 0;
}
int mi_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    mi::clear_error(); MI_HIP_CHECK(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost)); return 0;
}
int mi_memcpy_d2d_async(void* dst, const void* src, size_t bytes, void* stream) {
    mi::clear_error();
    MI_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, mi::resolve_stream(stream)));
    return 0;
}
int mi_memset_async(void* dst, int value, size_t bytes, void* stream) {
    mi::clear_error(); MI_HIP_CHECK(hipMemsetAsync(dst, value, bytes, mi::resolve_stream(stream))); return 0;
}

int mi_sdpa_set_kernel_choice(int32_t choice) {
    mi::clear_error();
    if (choice < 0 || choice > 3)
        return fail("mi_sdpa_set_kernel_choice: 0 (auto), 1 (128-row tiles), 2 (256-row ping-pong) or 3 (ping-pong, register-staged tiles)");
    mi::g_kernel_choice = choice;
    return 0;
}

int mi_sdpa_supported(int32_t dtype, int32_t head_dim) { return mi::sdpa_supported(dtype, head_dim) ? 1 : 0; }

}  // extern "C"

namespace mi {
namespace {
// Validates the arguments and fills the device-side view. Returns 0, -1 (error recorded) or 1 (nothing to do).
int prepare_sdpa(const mi_sdpa_args* a, SdpaDev& p, long& Dkv_out) {
    if (!a) return fail("mi_sdpa_forward: null args");
    if (a->struct_size != sizeof(mi_sdpa_args))
        return fail("mi_sdpa_forward: struct_size %u != %zu (header mismatch)", a->struct_size, sizeof(mi_sdpa_args));
    if (!mi::sdpa_supported(a->dtype, a->head_dim))
        return fail("mi_sdpa_forward: no kernel for dtype %d head_dim %d", a->dtype, a->head_dim);
    if (a->batch <= 0 || a->num_heads <= 0) return fail("mi_sdpa_forward: batch and num_heads must be positive");
    if (a->q_len < 0 || a->kv_len < 0 || a->prefix_len < 0) return fail("mi_sdpa_forward: negative length");
    if (a->q_len == 0) return 1;
    if (!a->q || !a->o) return fail("mi_sdpa_forward: q and o must not be null");
    if (a->kv_len > 0 && (!a->k || !a->v)) return fail("mi_sdpa_forward: k and v must not be null");
    if (a->prefix_len > 0 && (!a->k_prefix || !a->v_prefix))
        return fail("mi_sdpa_forward: prefix_len %d but k_prefix / v_prefix is null", a->prefix_len);
    const int Hkv = a->num_kv_heads > 0 ? a->num_kv_heads : a->num_heads;
    if (a->num_heads % Hkv != 0) return fail("mi_sdpa_forward: num_kv_heads %d does not divide num_heads %d", Hkv, a->num_heads);
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    const long Dkv = static_cast<long>(Hkv) * a->head_dim;
    const long Lk = static_cast<long>(a->prefix_len) + a->kv_len;
    if (Lk > 0x7fffff00L) return fail("mi_sdpa_forward: too many keys");

    std::memset(&p, 0, sizeof(p));
    Dkv_out = Dkv;
    p.q = a->q; p.k = a->k; p.v = a->v; p.o = a->o;
    p.kp = a->prefix_len > 0 ? a->k_prefix : nullptr;
    p.vp = a->prefix_len > 0 ? a->v_prefix : nullptr;
    p.B = a->batch; p.H = a->num_heads; p.Lq = a->q_len; p.Lk = static_cast<int>(Lk); p.Lp = a->prefix_len;
    p.kv_group = a->num_heads / Hkv;
    auto rs = [](int64_t s, long dense) { return s ? static_cast<long>(s) : dense; };
    p.q_rs = rs(a->q_row_stride, D); p.k_rs = rs(a->k_row_stride, Dkv); p.v_rs = rs(a->v_row_stride, Dkv);
    p.o_rs = rs(a->o_row_stride, D); p.kp_rs = rs(a->kp_row_stride, Dkv); p.vp_rs = rs(a->vp_row_stride, Dkv);
    p.q_bs = a->q_batch_stride ? a->q_batch_stride : p.q_rs * a->q_len;
    p.o_bs = a->o_batch_stride ? a->o_batch_stride : p.o_rs * a->q_len;
    p.k_bs = a->k_batch_stride ? a->k_batch_stride : p.k_rs * a->kv_len;
    p.v_bs = a->v_batch_stride ? a->v_batch_stride : p.v_rs * a->kv_len;
    p.kp_bs = a->kp_batch_stride ? a->kp_batch_stride : p.kp_rs * a->prefix_len;
    p.vp_bs = a->vp_batch_stride ? a->vp_batch_stride : p.vp_rs * a->prefix_len;
    // 16-byte vector loads: bases 16-byte aligned, strides multiples of 8 elements, row at least one head wide
    const void* ptrs[] = {a->q, a->k, a->v, a->o, p.kp, p.vp};
    for (const void* ptr : ptrs)
        if (ptr && !mi::aligned16(ptr)) return fail("mi_sdpa_forward: tensor pointers must be 16-byte aligned");
    const long strides[] = {p.q_rs, p.k_rs, p.v_rs, p.o_rs, p.kp_rs, p.vp_rs, p.q_bs, p.k_bs, p.v_bs, p.o_bs, p.kp_bs, p.vp_bs};
    for (long s : strides)
        if (s % 8 != 0) return fail("mi_sdpa_forward: strides must be multiples of 8 elements (got %ld)", s);
    if (p.q_rs < D || p.o_rs < D) return fail("mi_sdpa_forward: q/o row stride smaller than heads*head_dim %ld", D);
    if (p.k_rs < Dkv || p.v_rs < Dkv || p.kp_rs < Dkv || p.vp_rs < Dkv)
        return fail("mi_sdpa_forward: k/v row stride smaller than kv_heads*head_dim %ld", Dkv);

    const float scale = a->scale > 0.f ? a->scale : 1.0f / std::sqrt(static_cast<float>(a->head_dim));
    p.scale_log2 = scale * 1.4426950408889634f;
    p.mask_mode = a->mask_mode; p.q_offset = a->q_offset; p.window = 0;
    if (a->mask_mode == MI_MASK_CAUSAL) {
        if (a->window < 0) return fail("mi_sdpa_forward: window must be >= 0");
        p.window = a->window;
    } else if (a->mask_mode == MI_MASK_BLOCK_CAUSAL) {
        if (a->n_segments < 1 || a->n_segments > MI_MAX_SEGMENTS)
            return fail("mi_sdpa_forward: n_segments %d outside 1..%d", a->n_segments, MI_MAX_SEGMENTS);
        p.n_seg = a->n_segments;
        for (int s = 0; s < a->n_segments; ++s) {
            if (s > 0 && a->seg_q_end[s] < a->seg_q_end[s - 1])
                return fail("mi_sdpa_forward: seg_q_end must be non-decreasing");
            if (a->seg_k_end[s] < 0) return fail("mi_sdpa_forward: seg_k_end must be >= 0");
            p.seg_q_end[s] = a->seg_q_end[s]; p.seg_k_end[s] = a->seg_k_end[s]; p.seg_causal[s] = a->seg_causal[s] ? 1 : 0;
        }
        if (a->seg_q_end[a->n_segments - 1] < a->q_len)
            return fail("mi_sdpa_forward: segments cover %d query rows, q_len is %d", a->seg_q_end[a->n_segments - 1], a->q_len);
    } else if (a->mask_mode != MI_MASK_NONE) {
        return fail("mi_sdpa_forward: unknown mask_mode %d", a->mask_mode);
    }
    p.kv_valid_len = a->kv_valid_len;
    p.key_mask = a->key_mask; p.key_mask_bs = a->key_mask_batch_stride;
    if ((a->rope_cos_q == nullptr) != (a->rope_sin_q == nullptr) || (a->rope_cos_k == nullptr) != (a->rope_sin_k == nullptr))
        return fail("mi_sdpa_forward: rope cos and sin tables must be given together");
    const void* tabs[] = {a->rope_cos_q, a->rope_sin_q, a->rope_cos_k, a->rope_sin_k};
    for (const void* t : tabs)
        if (t && !mi::aligned16(t)) return fail("mi_sdpa_forward: rope tables must be 16-byte aligned");
    p.cos_q = a->rope_cos_q; p.sin_q = a->rope_sin_q; p.cos_k = a->rope_cos_k; p.sin_k = a->rope_sin_k;
    if (a->rope_split_half != 0 && a->rope_split_half != 1) return fail("mi_sdpa_forward: rope_split_half must be 0 or 1");
    p.rope_split = a->rope_split_half;
    if (p.rope_split && p.cos_k && a->kv_len > 0 && !a->rope_k_scratch)
        return fail("mi_sdpa_forward: split-half RoPE on K needs rope_k_scratch (K is rotated tile by tile for adjacent pairs only)");
    p.inv_scale = 1.0f / scale;
    if (a->logit_bias) {
        if (a->batch != 1) return fail("mi_sdpa_forward: logit_bias needs batch 1");
        if (a->bias_q0 < 0 || a->bias_cols < 0 || a->bias_cols > Lk) return fail("mi_sdpa_forward: bias_q0 / bias_cols out of range");
        p.bias = a->logit_bias; p.bias_q0 = a->bias_q0; p.bias_cols = a->bias_cols;
        p.bias_rs = a->bias_row_stride ? a->bias_row_stride : a->bias_cols;
        if (p.bias_rs < p.bias_cols) return fail("mi_sdpa_forward: bias_row_stride smaller than bias_cols");
        if (reinterpret_cast<uintptr_t>(a->logit_bias) & 3u) return fail("mi_sdpa_forward: logit_bias must be 4-byte aligned");
        p.bias_vec_ok = ((reinterpret_cast<uintptr_t>(a->logit_bias) & 15u) == 0 && p.bias_rs % 4 == 0) ? 1 : 0;
        if (a->bias_cols == 0 || a->bias_q0 >= a->q_len) p.bias = nullptr;   // nothing to add
    }
    {
        const float ks = a->prefix_k_scale != 0.f ? a->prefix_k_scale : 1.f, vs = a->prefix_v_scale != 0.f ? a->prefix_v_scale : 1.f;
        if (!std::isfinite(ks) || !std::isfinite(vs)) return fail("mi_sdpa_forward: prefix_k_scale / prefix_v_scale must be finite");
        if ((reinterpret_cast<uintptr_t>(a->prefix_k_row_scale) | reinterpret_cast<uintptr_t>(a->prefix_v_row_scale)) & 3u)
            return fail("mi_sdpa_forward: prefix row scales must be 4-byte aligned");
        if (a->prefix_len > 0 && (ks != 1.f || vs != 1.f || a->prefix_k_row_scale || a->prefix_v_row_scale)) {
            p.prefix_scaled = 1;
            p.pk_scale = ks; p.pv_scale = vs;
            p.pk_row = a->prefix_k_row_scale; p.pv_row = a->prefix_v_row_scale;
        }
    }
    if ((a->cu_seqlens_q == nullptr) != (a->cu_seqlens_k == nullptr)) return fail("mi_sdpa_forward: cu_seqlens_q and cu_seqlens_k must be given together");
    if (a->cu_seqlens_q) {
        if (a->prefix_len > 0 || a->key_mask || a->kv_valid_len || a->rope_cos_q || a->rope_cos_k || a->logit_bias || a->lse_out)
            return fail("mi_sdpa_forward: packed variable-length sequences take no prefix, key mask, kv_valid_len, RoPE, bias or lse_out");
        if (a->mask_mode == MI_MASK_BLOCK_CAUSAL || (a->mask_mode == MI_MASK_CAUSAL && a->window != 0))
            return fail("mi_sdpa_forward: packed variable-length sequences support MI_MASK_NONE and unwindowed MI_MASK_CAUSAL");
        if ((reinterpret_cast<uintptr_t>(a->cu_seqlens_q) | reinterpret_cast<uintptr_t>(a->cu_seqlens_k)) & 3u)
            return fail("mi_sdpa_forward: cu_seqlens must be 4-byte aligned");
        p.cu_q = a->cu_seqlens_q; p.cu_k = a->cu_seqlens_k;
    }
    if (a->lse_out) {
        if (reinterpret_cast<uintptr_t>(a->lse_out) & 3u) return fail("mi_sdpa_forward: lse_out must be 4-byte aligned");
        p.lse = a->lse_out;
    }
    if (a->rope_k_scratch && !mi::aligned16(a->rope_k_scratch)) return fail("mi_sdpa_forward: rope_k_scratch must be 16-byte aligned");
    if (a->split_scratch && !mi::aligned16(a->split_scratch)) return fail("mi_sdpa_forward: split_scratch must be 16-byte aligned");
    // what the wide-head kernel (head_dim 256 / 384 / 512) does not offer is refused here, before any work is enqueued
    if (mi::sdpa_wide_head(a->head_dim)) {
        const char* what = nullptr;
        if (a->prefix_len > 0) what = "a cached prefix";
        else if (p.cos_k && a->kv_len > 0 && !a->rope_k_scratch) what = "K rotated tile by tile (lend rope_k_scratch)";
        else if (p.bias) what = "a logit bias";
        else if (p.lse) what = "lse_out";
        else if (p.cu_q) what = "packed variable-length sequences";
        if (what) return fail("mi_sdpa_forward: head_dim %d does not offer %s", a->head_dim, what);
    }
    // the grid pads batch*heads to a multiple of 8 for masked calls
    const long nb = ((static_cast<long>(a->batch) * a->num_heads + 7) & ~7L) * ((a->q_len + 127) / 128);
    if (nb > 0x7fffffffL) return fail("mi_sdpa_forward: problem too large for one launch");
    return 0;
}
// K rotated into the caller's scratch is what the attention kernel reads.
void use_rotated_k(const mi_sdpa_args* a, SdpaDev& p, long Dkv) {
    p.k = a->rope_k_scratch; p.k_rs = Dkv; p.k_bs = Dkv * a->kv_len;
    p.cos_k = nullptr; p.sin_k = nullptr;
}
}  // namespace
}  // namespace mi

extern "C" {

size_t mi_sdpa_split_scratch_bytes(const mi_sdpa_args* a) {
    mi::clear_error();
    mi::SdpaDev p;
    long Dkv = 0;
    if (mi::prepare_sdpa(a, p, Dkv) != 0) return 0;
    if (p.cos_k && a->rope_k_scratch && a->kv_len > 0) mi::use_rotated_k(a, p, Dkv);
    return mi::sdpa_split_scratch_bytes(p, a->dtype, a->head_dim);
}

int mi_sdpa_forward(const mi_sdpa_args* a) {
    mi::clear_error();
    mi::SdpaDev p;
    long Dkv = 0;
    const int rc = mi::prepare_sdpa(a, p, Dkv);
    if (rc != 0) return rc < 0 ? -1 : 0;
    const int Hkv = a->num_kv_heads > 0 ? a->num_kv_heads : a->num_heads;
    if (p.cos_k && a->rope_k_scratch && a->kv_len > 0) {
        // K is rotated once into the caller's scratch (a pure HBM pass) and the attention kernel reads the
        // rotated copy: the LDS-DMA tile path stays usable and no work group repeats the rotation.
        const size_t esz = 2;
        for (int b = 0; b < a->batch; ++b) {
            mi_rope_args r;
            std::memset(&r, 0, sizeof(r));
            r.struct_size = sizeof(r);
            r.dtype = a->dtype;
            r.x = static_cast<const char*>(a->k) + static_cast<size_t>(b) * p.k_bs * esz;
            r.out = static_cast<char*>(a->rope_k_scratch) + static_cast<size_t>(b) * a->kv_len * Dkv * esz;
            r.cos = p.cos_k; r.sin = p.sin_k;
            r.rows = a->kv_len; r.num_heads = Hkv; r.head_dim = a->head_dim;
            r.x_row_stride = p.k_rs; r.out_row_stride = Dkv;
            r.split_half = a->rope_split_half;
            r.stream = mi::resolve_stream(a->stream);
            if (mi_rope_apply(&r) != 0) return -1;
        }
        mi::use_rotated_k(a, p, Dkv);
    }
    p.split_scratch = static_cast<unsigned char*>(a->split_scratch);
    p.split_scratch_bytes = a->split_scratch ? a->split_scratch_bytes : 0;
    return mi::launch_sdpa(p, a->dtype, a->head_dim, mi::resolve_stream(a->stream));
}

int mi_attention_map_avg(const mi_attention_map_args* a) {
    mi::clear_error();
    const char* op = "mi_attention_map_avg";
    if (!a) return fail("%s: null args", op);
    if (a->struct_size != sizeof(mi_attention_map_args)) return fail("%s: struct_size mismatch", op);
    // (the map kernel covers the head dimensions of the 128-row attention kernel, which writes the denominators it reads)
    if (!mi::sdpa_supported(a->dtype, a->head_dim) || mi::sdpa_wide_head(a->head_dim))
        return fail("%s: no kernel for dtype %d head_dim %d", op, a->dtype, a->head_dim);
    if (a->num_heads <= 0 || a->q_len < 0 || a->kv_len < 0) return fail("%s: bad shape", op);
    if (a->q_len == 0 || a->kv_len == 0) return 0;
    if (!a->q || !a->k || !a->lse || !a->map) return fail("%s: q, k, lse and map must not be null", op);
    const long D = static_cast<long>(a->num_heads) * a->head_dim;
    mi::MapDev p;
    std::memset(&p, 0, sizeof(p));
    p.q = a->q; p.k = a->k; p.lse = a->lse; p.map = a->map;
    p.H = a->num_heads; p.Lq = a->q_len; p.Lk = a->kv_len;
    p.q_rs = a->q_row_stride ? a->q_row_stride : D;
    p.k_rs = a->k_row_stride ? a->k_row_stride : D;
    p.map_rs = a->map_row_stride ? a->map_row_stride : a->kv_len;
    if (p.q_rs < D || p.k_rs < D || p.map_rs < a->kv_len) return fail("%s: a row stride is smaller than its row", op);
    if (p.q_rs % 8 || p.k_rs % 8) return fail("%s: q / k row strides must be multiples of 8 elements", op);
    if (!mi::aligned16(a->q) || !mi::aligned16(a->k) || !mi::aligned16(a->map)) return fail("%s: q, k and map must be 16-byte aligned", op);
    if ((reinterpret_cast<uintptr_t>(a->lse) | reinterpret_cast<uintptr_t>(a->logit_bias) | reinterpret_cast<uintptr_t>(a->key_mask)) & 3u)
        return fail("%s: lse, logit_bias and key_mask must be 4-byte aligned", op);
    const float scale = a->scale > 0.f ? a->scale : 1.0f / std::sqrt(static_cast<float>(a->head_dim));
    p.scale_log2 = scale * 1.4426950408889634f;
    if (a->logit_bias && a->bias_cols > 0 && a->bias_q0 < a->q_len) {
        if (a->bias_q0 < 0 || a->bias_cols > a->kv_len) return fail("%s: bias_q0 / bias_cols out of range", op);
        p.bias = a->logit_bias; p.bias_q0 = a->bias_q0; p.bias_cols = a->bias_cols;
        p.bias_rs = a->bias_row_stride ? a->bias_row_stride : a->bias_cols;
        if (p.bias_rs < p.bias_cols) return fail("%s: bias_row_stride smaller than bias_cols", op);
    }
    p.key_mask = a->key_mask;
    return mi::launch_attention_map(p, a->dtype, a->head_dim, mi::resolve_stream(a->stream));
}

}  // extern "C"
