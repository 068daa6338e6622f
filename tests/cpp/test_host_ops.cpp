// Parity test of the C++20 host operator layer, in the reference's test style: one executable,
// a CHECK macro that counts failures (reference: tests/test_flux_blocks.cpp:38-44).
//   test_host_ops --cpu   precondition / error-path checks that need no GPU
//   test_host_ops         the GPU parity run against the CPU checker (liboracle.so, test-only)
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "attention_ops.h"

extern "C" {
int orc_torch_randn_f32(uint64_t seed, size_t n, float* out);
void orc_round_bf16(float* x, size_t n);
void orc_f32_to_bf16_bits(const float* x, size_t n, uint16_t* out);
void orc_bf16_bits_to_f32(const uint16_t* x, size_t n, float* out);
int orc_build_axial_rope_tables(int txt_len, int hp, int wp, int head_dim, const int* axes, int n_axes, float theta,
                                float* cos_out, float* sin_out);
int orc_build_qwen_rope_tables(const int* seg_kind, const int* seg_a, const int* seg_b, int n_seg, int hp, int wp, int head_dim,
                               const int* axes, double theta, float* cos_out, float* sin_out);
void orc_rope_apply(const float* x, const float* cs, const float* sn, int L, int H, int d, int split_half, int round_mode, float* out);
void orc_sdpa(const float* q, const float* k, const float* v, int Lq, int Lk, int H, int d, double scale, const float* key_mask,
              const int* row_lo, const int* row_hi, const uint8_t* dense_mask, const float* bias, int bias_q0, int bias_cols,
              const int* rows, int n_rows, float* out, float* attn_avg, int n_threads);
void orc_rows_causal(int Lq, int Lk, int q_offset, int window, int* row_lo, int* row_hi);
void orc_rows_block_causal(int Lq, int Lk, int q_offset, const int* seg_q_end, const int* seg_k_end, const int* seg_causal,
                           int n_seg, int* row_lo, int* row_hi);
void orc_linear_attn_relu(const float* q, const float* k, const float* v, int N, int H, int d, float eps, float* out,
                          float* S_out, float* z_out, int n_threads);
void orc_rms_norm(const float* x, const float* gain, double eps, int rows, int cols, float* out);
void orc_geglu_exact(const float* t, int rows, int d_out, float* out);
void orc_linear(const float* x, const float* w, const float* bias, int M, int N, int K, float* y, int n_threads);
}

using namespace bdamd;

static int g_failures = 0;
#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) { std::printf("CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond); ++g_failures; } \
    } while (0)

template <typename F>
static bool throws_with(F&& f, const char* needle) {
    try { f(); } catch (const std::runtime_error& e) { return std::strstr(e.what(), needle) != nullptr; }
    return false;
}

static std::vector<float> randn_bf16(uint64_t seed, size_t n) {
    std::vector<float> x(n < 16 ? 16 : n);
    orc_torch_randn_f32(seed, x.size(), x.data());
    x.resize(n);
    orc_round_bf16(x.data(), n);
    return x;
}
static Tensor upload_bf16(const std::vector<float>& x, int rows, int cols) {
    std::vector<uint16_t> bits(x.size());
    orc_f32_to_bf16_bits(x.data(), x.size(), bits.data());
    return Tensor::from_host(bits.data(), rows, cols, Dtype::BF16);
}
static std::vector<float> download_bf16(const Tensor& t) {
    const std::vector<uint8_t> raw = t.to_host_bytes();
    std::vector<float> out(t.size());
    orc_bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(raw.data()), out.size(), out.data());
    return out;
}
struct Err { double rel_l2, max_abs; };
static Err compare(const std::vector<float>& ref, const std::vector<float>& got) {
    double num = 0, den = 0, mx = 0;
    for (size_t i = 0; i < ref.size(); ++i) {
        const double d = static_cast<double>(ref[i]) - got[i];
        num += d * d; den += static_cast<double>(ref[i]) * ref[i];
        if (std::fabs(d) > mx) mx = std::fabs(d);
    }
    return {std::sqrt(num / (den + 1e-300)), mx};
}
// bf16 bar of the port: rel-L2 <= 5e-3, max-abs <= 2e-2
static bool within_bf16(const Err& e) { return e.rel_l2 <= 5e-3 && e.max_abs <= 2e-2; }

static void cpu_checks() {
    float dummy[64 * 64] = {0};
    Tensor q = Tensor::view(Device::CPU, dummy, 8, 256, Dtype::BF16);
    Tensor out;
    CHECK(throws_with([&] { bt::flash_attention_forward(q, q, q, nullptr, 2, false, out); }, "flash_attention_forward: tensor is on the CPU"));
    Tensor g = Tensor::view(Device::GPU, dummy, 8, 256, Dtype::BF16);   // never dereferenced: validation fails first
    CHECK(throws_with([&] { bt::flash_attention_forward(g, g, g, nullptr, 3, false, out); }, "D must equal head_dim * num_heads"));
    Tensor k = Tensor::view(Device::GPU, dummy, 8, 128, Dtype::BF16);
    CHECK(throws_with([&] { bt::flash_attention_forward(g, k, g, nullptr, 2, false, out); }, "K and V must be"));
    Tensor f = Tensor::view(Device::GPU, dummy, 8, 256, Dtype::FP32);
    CHECK(throws_with([&] { bt::flash_attention_forward(f, f, f, nullptr, 2, false, out); }, "dtype must be FP16 or BF16"));
    CHECK(throws_with([&] { bt::flash_attention_windowed_forward(g, g, g, nullptr, 2, -1, out); }, "window must be >= 0"));
    CHECK(throws_with([&] { dit::build_axial_rope_tables(4, 2, 2, 32, {8, 8, 8}); }, "must sum to head_dim"));
    CHECK(throws_with([&] { dit::build_axial_rope_tables(4, 2, 2, 31, {15, 8, 8}); }, "head_dim must be even"));
    CHECK(throws_with([&] { dit::build_qwen_rope_tables({}, 2, 2, 32, {8, 8, 8}); }, "summing to head_dim"));
    Tensor Qr, Kr;
    CHECK(throws_with([&] { dit::joint_attention(g, k, g, f, f, 128, 2, out, Qr, Kr); }, "Q/K/V must share shape"));
    CHECK(throws_with([&] { g.row_view(4, 8); }, "rows out of range"));
    Tensor v = g.row_view(2, 4);
    CHECK(v.rows == 4 && v.data == reinterpret_cast<char*>(dummy) + 2 * 256 * 2);
}

static void gpu_checks() {
    const int H = 2, d = 128, txt = 19, hp = 6, wp = 7, L = txt + hp * wp, D = H * d;
    const std::vector<float> q = randn_bf16(7001, static_cast<size_t>(L) * D), k = randn_bf16(7002, static_cast<size_t>(L) * D),
                             v = randn_bf16(7003, static_cast<size_t>(L) * D);
    Tensor Q = upload_bf16(q, L, D), K = upload_bf16(k, L, D), V = upload_bf16(v, L, D);

    {   // joint_attention: fused RoPE == checker's explicit RoPE (rounded to bf16) + exact attention
        const std::vector<int> axes = {16, 56, 56};
        dit::RopeTables tabs = dit::build_axial_rope_tables(txt, hp, wp, d, axes);
        std::vector<float> oc(static_cast<size_t>(L) * d / 2), os(oc.size());
        orc_build_axial_rope_tables(txt, hp, wp, d, axes.data(), 3, 10000.0f, oc.data(), os.data());
        const std::vector<uint8_t> tc = tabs.cos.to_host_bytes();
        CHECK(std::memcmp(tc.data(), oc.data(), tc.size()) == 0);      // same table builder arithmetic
        Tensor out, Qr, Kr;
        dit::joint_attention(Q, K, V, tabs.cos, tabs.sin, d, H, out, Qr, Kr);
        std::vector<float> qr(q.size()), kr(k.size()), ref(q.size());
        orc_rope_apply(q.data(), oc.data(), os.data(), L, H, d, 0, 1, qr.data());
        orc_rope_apply(k.data(), oc.data(), os.data(), L, H, d, 0, 1, kr.data());
        orc_sdpa(qr.data(), kr.data(), v.data(), L, L, H, d, -1.0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr, 0,
                 ref.data(), nullptr, 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("joint_attention       rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        // determinism: bit-exact across two calls (reference: tests/test_flux_blocks.cpp:241-247)
        Tensor out2;
        dit::joint_attention(Q, K, V, tabs.cos, tabs.sin, d, H, out2, Qr, Kr);
        CHECK(out.to_host_bytes() == out2.to_host_bytes());
        // stand-alone rope_apply + flash == fused
        Tensor Qrot, Krot, out3;
        bt::rope_apply(Q, tabs.cos, tabs.sin, d, H, Qrot);
        bt::rope_apply(K, tabs.cos, tabs.sin, d, H, Krot);
        bt::flash_attention_forward(Qrot, Krot, V, nullptr, H, false, out3);
        CHECK(out.to_host_bytes() == out3.to_host_bytes());
    }
    {   // Qwen-Image 3-axis tables: host builder == checker's restatement of build_rope_tables_
        const std::vector<dit::QwenSegment> pre = {{dit::QwenSegment::Kind::Text, 5, 0, 0}, {dit::QwenSegment::Kind::Image, 0, 3, 4},
                                                   {dit::QwenSegment::Kind::Text, 2, 0, 0}};
        dit::RopeTables t = dit::build_qwen_rope_tables(pre, 2, 3, 16, {4, 6, 6});
        const int kind[3] = {0, 1, 0}, sa[3] = {5, 3, 2}, sb[3] = {0, 4, 0}, ax[3] = {4, 6, 6};
        const int Lq = orc_build_qwen_rope_tables(kind, sa, sb, 3, 2, 3, 16, ax, 10000.0, nullptr, nullptr);
        CHECK(Lq == 5 + 12 + 2 + 6 && t.cos.rows == Lq && t.cos.cols == 8);
        std::vector<float> oc(static_cast<size_t>(Lq) * 8), os(oc.size());
        orc_build_qwen_rope_tables(kind, sa, sb, 3, 2, 3, 16, ax, 10000.0, oc.data(), os.data());
        const std::vector<uint8_t> tc = t.cos.to_host_bytes(), ts = t.sin.to_host_bytes();
        CHECK(std::memcmp(tc.data(), oc.data(), tc.size()) == 0 && std::memcmp(ts.data(), os.data(), ts.size()) == 0);
    }
    {   // windowed causal vs checker
        Tensor Qs = Q.row_view(10, 30), out;
        bt::flash_attention_windowed_forward(Qs, K, V, nullptr, H, 0, out);
        std::vector<int> lo(30), hi(30);
        orc_rows_causal(30, L, L - 30, 0, lo.data(), hi.data());
        std::vector<float> ref(static_cast<size_t>(30) * D);
        orc_sdpa(q.data() + static_cast<size_t>(10) * D, k.data(), v.data(), 30, L, H, d, -1.0, nullptr, lo.data(), hi.data(), nullptr,
                 nullptr, 0, 0, nullptr, 0, ref.data(), nullptr, 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("windowed causal       rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
    }
    {   // block-causal in one launch == the reference's one call per segment, and cached == prefill rows
        const int prefix = 21;                       // text prefix kept as "cache"
        std::vector<dit::Segment> segs = {{dit::Segment::Kind::Text, prefix}, {dit::Segment::Kind::Image, L - prefix}};
        Tensor out;
        dit::block_causal_attention(Q, K, V, nullptr, nullptr, segs, 0, H, nullptr, nullptr, out);
        Tensor o_text, o_img;
        bt::flash_attention_windowed_forward(Q.row_view(0, prefix), K.row_view(0, prefix), V.row_view(0, prefix), nullptr, H, 0, o_text);
        bt::flash_attention_forward(Q.row_view(prefix, L - prefix), K, V, nullptr, H, false, o_img);
        const std::vector<uint8_t> all = out.to_host_bytes(), t = o_text.to_host_bytes(), im = o_img.to_host_bytes();
        CHECK(std::memcmp(all.data(), t.data(), t.size()) == 0);
        CHECK(std::memcmp(all.data() + t.size(), im.data(), im.size()) == 0);
        // cached form: prefix K/V from a separate buffer, target rows only
        Tensor kp = K.row_view(0, prefix), vp = V.row_view(0, prefix), o_cached;
        dit::block_causal_attention(Q.row_view(prefix, L - prefix), K.row_view(prefix, L - prefix), V.row_view(prefix, L - prefix), &kp, &vp,
                                    {{dit::Segment::Kind::Image, L - prefix}}, prefix, H, nullptr, nullptr, o_cached);
        // the key tiles restart at the prefix boundary, so the summation order differs from the one-buffer call
        const Err ec = compare(download_bf16(o_img), download_bf16(o_cached));
        std::printf("cached vs prefill     rel_l2=%.3e max_abs=%.3e\n", ec.rel_l2, ec.max_abs);
        CHECK(within_bf16(ec));
        std::vector<int> sq = {prefix, L}, sk = {prefix, L}, sc = {1, 0}, lo(L), hi(L);
        orc_rows_block_causal(L, L, 0, sq.data(), sk.data(), sc.data(), 2, lo.data(), hi.data());
        std::vector<float> ref(q.size());
        orc_sdpa(q.data(), k.data(), v.data(), L, L, H, d, -1.0, nullptr, lo.data(), hi.data(), nullptr, nullptr, 0, 0, nullptr, 0, ref.data(),
                 nullptr, 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("block-causal          rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
    }
    {   // the prefix-KV dial, as tests/test_qwenimage21_slots.cpp:361-412 exercises it: armed it changes the cached
        // step, set twice it is the same picture (the cache stays pristine), two halvings equal one quarter,
        // identity scales are the unscaled step bit for bit
        const int prefix = 21;
        Tensor kp = K.row_view(0, prefix), vp = V.row_view(0, prefix);
        Tensor Qt = Q.row_view(prefix, L - prefix), Kt = K.row_view(prefix, L - prefix), Vt = V.row_view(prefix, L - prefix);
        const std::vector<dit::Segment> seg = {{dit::Segment::Kind::Image, L - prefix}};
        auto step = [&](float ks, float vs) {
            Tensor ksc, vsc, o;
            dit::scale_rows(kp, ks, nullptr, ksc);
            dit::scale_rows(vp, vs, nullptr, vsc);
            dit::block_causal_attention(Qt, Kt, Vt, &ksc, &vsc, seg, prefix, H, nullptr, nullptr, o);
            return o.to_host_bytes();
        };
        Tensor o_plain;
        dit::block_causal_attention(Qt, Kt, Vt, &kp, &vp, seg, prefix, H, nullptr, nullptr, o_plain);
        const std::vector<uint8_t> cache_before = kp.to_host_bytes();
        const std::vector<uint8_t> plain = o_plain.to_host_bytes(), halved = step(1.0f, 0.5f), again = step(1.0f, 0.5f);
        CHECK(plain != halved);
        CHECK(halved == again);
        CHECK(step(1.0f, 1.0f) == plain);
        CHECK(kp.to_host_bytes() == cache_before);
        // composition: scaling the already halved copy by 0.5 is the quarter dial (powers of two are exact)
        Tensor vh, vq, o_q;
        dit::scale_rows(vp, 0.5f, nullptr, vh);
        dit::scale_rows(vh, 0.5f, nullptr, vq);
        dit::block_causal_attention(Qt, Kt, Vt, &kp, &vq, seg, prefix, H, nullptr, nullptr, o_q);
        CHECK(o_q.to_host_bytes() == step(1.0f, 0.25f));
        // per-token weights against the checker: keys scaled before the scores, values before the sum
        std::vector<float> wk(prefix), wv(prefix);
        for (int i = 0; i < prefix; ++i) { wk[i] = 0.5f + 0.05f * i; wv[i] = 1.5f - 0.04f * i; }
        Tensor Wk = Tensor::from_host(wk.data(), prefix, 1, Dtype::FP32), Wv = Tensor::from_host(wv.data(), prefix, 1, Dtype::FP32), ksc, vsc, o_w;
        dit::scale_rows(kp, 0.8f, &Wk, ksc);
        dit::scale_rows(vp, 1.0f, &Wv, vsc);
        dit::block_causal_attention(Qt, Kt, Vt, &ksc, &vsc, seg, prefix, H, nullptr, nullptr, o_w);
        std::vector<float> k2 = k, v2 = v;
        for (int i = 0; i < prefix; ++i)
            for (int c = 0; c < D; ++c) { k2[static_cast<size_t>(i) * D + c] *= 0.8f * wk[i]; v2[static_cast<size_t>(i) * D + c] *= wv[i]; }
        orc_round_bf16(k2.data(), static_cast<size_t>(prefix) * D);   // the scaled copy is a bf16 tensor, in the reference too
        orc_round_bf16(v2.data(), static_cast<size_t>(prefix) * D);
        std::vector<float> ref(static_cast<size_t>(L - prefix) * D);
        orc_sdpa(q.data() + static_cast<size_t>(prefix) * D, k2.data(), v2.data(), L - prefix, L, H, d, -1.0, nullptr, nullptr, nullptr, nullptr,
                 nullptr, 0, 0, nullptr, 0, ref.data(), nullptr, 0);
        const Err e = compare(ref, download_bf16(o_w));
        std::printf("prefix-KV dial        rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        CHECK(throws_with([&] { Tensor o2; dit::scale_rows(kp, 1.0f, &Wk, o2); dit::scale_rows(K, 1.0f, &Wk, o2); }, "the row scale holds 21 values"));
        // the same dial applied inside the kernel (no scaled copy): within tolerance of the checker, the cache untouched, set
        // twice the same bits, identity = the plain step, and close to the scaled-copy route it replaces
        dit::PrefixDial dial;
        dial.k_scale = 0.8f; dial.v_scale = 1.0f; dial.k_rows = &Wk; dial.v_rows = &Wv;
        Tensor o_in, o_in2, o_id;
        dit::block_causal_attention(Qt, Kt, Vt, &kp, &vp, seg, prefix, H, nullptr, nullptr, o_in, &dial);
        dit::block_causal_attention(Qt, Kt, Vt, &kp, &vp, seg, prefix, H, nullptr, nullptr, o_in2, &dial);
        CHECK(o_in.to_host_bytes() == o_in2.to_host_bytes());
        CHECK(kp.to_host_bytes() == cache_before);
        CHECK(within_bf16(compare(ref, download_bf16(o_in))));
        CHECK(within_bf16(compare(download_bf16(o_w), download_bf16(o_in))));
        const dit::PrefixDial identity;
        dit::block_causal_attention(Qt, Kt, Vt, &kp, &vp, seg, prefix, H, nullptr, nullptr, o_id, &identity);
        CHECK(o_id.to_host_bytes() == plain);
    }
    {   // ReLU linear attention, 70 x 32 (the reference's own head split) on a short sequence
        const int Hl = 70, dl = 32, N = 96, Dl = Hl * dl;
        const std::vector<float> ql = randn_bf16(7011, static_cast<size_t>(N) * Dl), kl = randn_bf16(7012, static_cast<size_t>(N) * Dl),
                                 vl = randn_bf16(7013, static_cast<size_t>(N) * Dl);
        Tensor Ql = upload_bf16(ql, N, Dl), Kl = upload_bf16(kl, N, Dl), Vl = upload_bf16(vl, N, Dl), state, out;
        Tensor scratch;
        bt::linear_attention_relu_forward(Ql, Kl, Vl, Hl, 1e-15f, state, out, false, &scratch);
        std::vector<float> ref(ql.size());
        orc_linear_attn_relu(ql.data(), kl.data(), vl.data(), N, Hl, dl, 1e-15f, ref.data(), nullptr, nullptr, 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("linear attention      rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        CHECK(state.rows == Hl && state.cols == dl * dl + dl);
        // the same values as (D, N) channel-major tensors, the reference's own layout around its core (src/dit/sana.cpp:424-444)
        auto transposed = [&](const std::vector<float>& x) {
            std::vector<float> t(x.size());
            for (int n = 0; n < N; ++n)
                for (int c = 0; c < Dl; ++c) t[static_cast<size_t>(c) * N + n] = x[static_cast<size_t>(n) * Dl + c];
            return t;
        };
        Tensor Qc = upload_bf16(transposed(ql), Dl, N), Kc = upload_bf16(transposed(kl), Dl, N), Vc = upload_bf16(transposed(vl), Dl, N), state_c, out_c;
        bt::linear_attention_relu_forward_channel_major(Qc, Kc, Vc, Hl, 1e-15f, state_c, out_c);
        CHECK(out_c.rows == Dl && out_c.cols == N);
        const Err ec = compare(transposed(ref), download_bf16(out_c));
        std::printf("linear attention (D,N) rel_l2=%.3e max_abs=%.3e\n", ec.rel_l2, ec.max_abs);
        CHECK(within_bf16(ec));
    }
    {   // traced joint attention: output and head-averaged map against the checker's restatement of the host loop
        const std::vector<int> axes = {16, 56, 56};
        dit::RopeTables tabs = dit::build_axial_rope_tables(txt, hp, wp, d, axes);
        std::vector<float> oc(static_cast<size_t>(L) * d / 2), os(oc.size());
        orc_build_axial_rope_tables(txt, hp, wp, d, axes.data(), 3, 10000.0f, oc.data(), os.data());
        std::vector<float> bias(static_cast<size_t>(L - txt) * txt);
        orc_torch_randn_f32(7301, bias.size(), bias.data());
        Tensor B = Tensor::from_host(bias.data(), L - txt, txt, Dtype::FP32), out, avg, Qr, Kr;
        dit::joint_attention_traced(Q, K, V, tabs.cos, tabs.sin, d, H, out, avg, Qr, Kr, txt, &B);
        std::vector<float> qr(q.size()), kr(k.size()), ref(q.size()), ref_avg(static_cast<size_t>(L) * L);
        orc_rope_apply(q.data(), oc.data(), os.data(), L, H, d, 0, 1, qr.data());
        orc_rope_apply(k.data(), oc.data(), os.data(), L, H, d, 0, 1, kr.data());
        orc_sdpa(qr.data(), kr.data(), v.data(), L, L, H, d, -1.0, nullptr, nullptr, nullptr, nullptr, bias.data(), txt, txt, nullptr, 0,
                 ref.data(), ref_avg.data(), 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("traced attention      rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        const std::vector<uint8_t> raw = avg.to_host_bytes();
        const float* got = reinterpret_cast<const float*>(raw.data());
        double worst = 0;
        for (size_t i = 0; i < ref_avg.size(); ++i) worst = std::fmax(worst, std::fabs(static_cast<double>(got[i]) - ref_avg[i]));
        std::printf("traced map            max_abs=%.3e\n", worst);
        CHECK(avg.rows == L && avg.cols == L && worst <= 2e-5);
        CHECK(throws_with([&] { Tensor b2 = Tensor::from_host(bias.data(), L - txt, txt - 1, Dtype::FP32);
                                dit::joint_attention_traced(Q, K, V, tabs.cos, tabs.sin, d, H, out, avg, Qr, Kr, txt, &b2); }, "(img_len, txt_len)"));
    }
    {   // the U-Net's traced cross attention: projections, logit bias + key mask, output projection, head-averaged map
        const int Lq = 200, Lk = 50, C = 128, Cc = 96, Hc = 2, dc = C / Hc;
        auto weight = [&](uint64_t seed, int rows, int cols) {
            std::vector<float> w(static_cast<size_t>(rows) * cols);
            orc_torch_randn_f32(seed, w.size(), w.data());
            for (float& x : w) x /= std::sqrt(static_cast<float>(cols));
            orc_round_bf16(w.data(), w.size());
            return w;
        };
        const std::vector<float> x = randn_bf16(7401, static_cast<size_t>(Lq) * C), ctx = randn_bf16(7402, static_cast<size_t>(Lk) * Cc);
        const std::vector<float> wq = weight(7403, C, C), wk = weight(7404, C, Cc), wv = weight(7405, C, Cc), wo = weight(7406, C, C);
        std::vector<float> bias(static_cast<size_t>(Lq) * Lk), mask(Lk, 1.f);
        orc_torch_randn_f32(7407, bias.size(), bias.data());
        mask[3] = 0.f;
        for (int j = Lk - 7; j < Lk; ++j) mask[j] = 0.f;
        Tensor X = upload_bf16(x, Lq, C), Ctx = upload_bf16(ctx, Lk, Cc), Wq = upload_bf16(wq, C, C), Wk = upload_bf16(wk, C, Cc),
               Wv = upload_bf16(wv, C, Cc), Wo = upload_bf16(wo, C, C), B = Tensor::from_host(bias.data(), Lq, Lk, Dtype::FP32),
               M = Tensor::from_host(mask.data(), 1, Lk, Dtype::FP32), out, avg;
        bt::cross_attention_forward_with_attn(X, Ctx, Wq, Wk, Wv, Wo, static_cast<const float*>(M.data), &B, Hc, out, avg);
        std::vector<float> qp(static_cast<size_t>(Lq) * C), kp(static_cast<size_t>(Lk) * C), vp(kp.size()), a(qp.size()), ref(qp.size()),
            ref_avg(static_cast<size_t>(Lq) * Lk);
        orc_linear(x.data(), wq.data(), nullptr, Lq, C, C, qp.data(), 0);
        orc_linear(ctx.data(), wk.data(), nullptr, Lk, C, Cc, kp.data(), 0);
        orc_linear(ctx.data(), wv.data(), nullptr, Lk, C, Cc, vp.data(), 0);
        orc_round_bf16(qp.data(), qp.size()); orc_round_bf16(kp.data(), kp.size()); orc_round_bf16(vp.data(), vp.size());
        orc_sdpa(qp.data(), kp.data(), vp.data(), Lq, Lk, Hc, dc, -1.0, mask.data(), nullptr, nullptr, nullptr, bias.data(), 0, Lk, nullptr, 0,
                 a.data(), ref_avg.data(), 0);
        orc_round_bf16(a.data(), a.size());
        orc_linear(a.data(), wo.data(), nullptr, Lq, C, C, ref.data(), 0);
        const Err e = compare(ref, download_bf16(out));
        std::printf("traced cross attn     rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        const std::vector<uint8_t> raw = avg.to_host_bytes();
        const float* got = reinterpret_cast<const float*>(raw.data());
        // projected Q / K elements may round the other way on the two sides (one unit in the last place), which moves a
        // probability by about that fraction
        bool ok = avg.rows == Lq && avg.cols == Lk;
        for (size_t i = 0; i < ref_avg.size() && ok; ++i) {
            ok = std::fabs(static_cast<double>(got[i]) - ref_avg[i]) <= 5e-5 + 2.0 * 0.00390625 * ref_avg[i];
            if (mask[i % Lk] == 0.f) ok = ok && got[i] == 0.f;
        }
        CHECK(ok);
        CHECK(throws_with([&] { Tensor b2 = Tensor::from_host(bias.data(), Lq, Lk - 1, Dtype::FP32);
                                bt::cross_attention_forward_with_attn(X, Ctx, Wq, Wk, Wv, Wo, nullptr, &b2, Hc, out, avg); }, "logit_bias must be FP32 (Lq, Lk)"));
    }
    {   // headnorm + RoPE in one pass, with the prefix rows also written to a cache tensor
        const std::vector<int> axes = {16, 56, 56};
        dit::RopeTables tabs = dit::build_axial_rope_tables(txt, hp, wp, d, axes);
        std::vector<float> oc(static_cast<size_t>(L) * d / 2), os(oc.size());
        orc_build_axial_rope_tables(txt, hp, wp, d, axes.data(), 3, 10000.0f, oc.data(), os.data());
        std::vector<float> gain = randn_bf16(7201, d);
        Tensor G = upload_bf16(gain, 1, d), out, cache;
        dit::headnorm_rope(K, G, 1e-6f, &tabs.cos, &tabs.sin, d, H, out, &cache, txt);
        std::vector<float> normed(k.size()), ref(k.size());
        orc_rms_norm(k.data(), gain.data(), 1e-6, L * H, d, normed.data());
        orc_rope_apply(normed.data(), oc.data(), os.data(), L, H, d, 0, 1, ref.data());
        const Err e = compare(ref, download_bf16(out));
        std::printf("headnorm + rope       rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(e.rel_l2 <= 5e-3);
        CHECK(cache.rows == txt && cache.cols == D);
        const std::vector<uint8_t> ob = out.to_host_bytes(), cb = cache.to_host_bytes();
        CHECK(std::memcmp(ob.data(), cb.data(), cb.size()) == 0);
        CHECK(throws_with([&] { Tensor o2; dit::headnorm_rope(K, Q, 1e-6f, nullptr, nullptr, d, H, o2); }, "gain must hold"));
    }
    {   // attention with its projections (SD1.5 level-0 widths: C 320, 8 heads of 40, text context 77 x 768)
        const int Lx = 100, C = 320, Hh = 8, Lc = 77, Cc = 768;
        auto scaled = [](std::vector<float> w, int fan_in) {
            for (float& x : w) x /= std::sqrt(static_cast<float>(fan_in));
            orc_round_bf16(w.data(), w.size());
            return w;
        };
        const std::vector<float> x = randn_bf16(7101, static_cast<size_t>(Lx) * C), ctx = randn_bf16(7102, static_cast<size_t>(Lc) * Cc);
        const std::vector<float> wq = scaled(randn_bf16(7103, static_cast<size_t>(C) * C), C), wk = scaled(randn_bf16(7104, static_cast<size_t>(C) * Cc), Cc),
                                 wv = scaled(randn_bf16(7105, static_cast<size_t>(C) * Cc), Cc), wo = scaled(randn_bf16(7106, static_cast<size_t>(C) * C), C),
                                 bo = randn_bf16(7107, C);
        Tensor X = upload_bf16(x, Lx, C), Ctx = upload_bf16(ctx, Lc, Cc), Wq = upload_bf16(wq, C, C), Wk = upload_bf16(wk, C, Cc),
               Wv = upload_bf16(wv, C, Cc), Wo = upload_bf16(wo, C, C), Bo = upload_bf16(bo, C, 1), out;
        bt::flash_attention_qkvo_forward(X, &Ctx, Wq, nullptr, Wk, nullptr, Wv, nullptr, Wo, &Bo, nullptr, Hh, false, out);
        auto lin = [](const std::vector<float>& a, const std::vector<float>& w, const float* b, int M, int N, int K, bool round) {
            std::vector<float> y(static_cast<size_t>(M) * N);
            orc_linear(a.data(), w.data(), b, M, N, K, y.data(), 0);
            if (round) orc_round_bf16(y.data(), y.size());
            return y;
        };
        const std::vector<float> rq = lin(x, wq, nullptr, Lx, C, C, true), rk = lin(ctx, wk, nullptr, Lc, C, Cc, true),
                                 rv = lin(ctx, wv, nullptr, Lc, C, Cc, true);
        std::vector<float> ra(rq.size());
        orc_sdpa(rq.data(), rk.data(), rv.data(), Lx, Lc, Hh, C / Hh, -1.0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr, 0, ra.data(), nullptr, 0);
        orc_round_bf16(ra.data(), ra.size());
        const std::vector<float> ref = lin(ra, wo, bo.data(), Lx, C, C, false);
        const Err e = compare(ref, download_bf16(out));
        std::printf("qkvo cross attention  rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(within_bf16(e));
        {   // mha_forward (src/dit/pixart.cpp:325-328): self attention with biased projections, intermediates visible
            const std::vector<float> bq = randn_bf16(7121, C), bk = randn_bf16(7122, C), bv = randn_bf16(7123, C);
            std::vector<float> km(Lx, 1.f);
            km[5] = 0.f; km[Lx - 1] = 0.f;
            Tensor Bq = upload_bf16(bq, 1, C), Bk = upload_bf16(bk, 1, C), Bv = upload_bf16(bv, 1, C),
                   M = Tensor::from_host(km.data(), 1, Lx, Dtype::FP32), Wks = upload_bf16(wq, C, C), qh, kh, vh, attn, yc, mo;
            bt::mha_forward(X, Wq, Wks, Wo, Wo, &Bq, &Bk, &Bv, &Bo, static_cast<const float*>(M.data), Hh, qh, kh, vh, attn, yc, mo);
            const std::vector<float> mq = lin(x, wq, bq.data(), Lx, C, C, true), mk = lin(x, wq, bk.data(), Lx, C, C, true),
                                     mvv = lin(x, wo, bv.data(), Lx, C, C, true);
            CHECK(within_bf16(compare(mq, download_bf16(qh))));
            CHECK(within_bf16(compare(mk, download_bf16(kh))));
            CHECK(within_bf16(compare(mvv, download_bf16(vh))));
            std::vector<float> ma(mq.size());
            orc_sdpa(mq.data(), mk.data(), mvv.data(), Lx, Lx, Hh, C / Hh, -1.0, km.data(), nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr, 0, ma.data(), nullptr, 0);
            orc_round_bf16(ma.data(), ma.size());
            CHECK(within_bf16(compare(ma, download_bf16(yc))));
            const Err em = compare(lin(ma, wo, bo.data(), Lx, C, C, false), download_bf16(mo));
            std::printf("mha_forward           rel_l2=%.3e max_abs=%.3e\n", em.rel_l2, em.max_abs);
            CHECK(within_bf16(em));
            CHECK(attn.data == nullptr);   // scores are never materialised
            CHECK(throws_with([&] { bt::mha_forward(X, Wq, Wks, Wo, Wo, nullptr, nullptr, nullptr, nullptr, nullptr, 7, qh, kh, vh, attn, yc, mo); },
                              "num_heads must divide"));
        }
        // K/V cache filled once, then the cached form: same kernels, same bits
        Tensor Kc, Vc, out2, own_scratch;
        bt::flash_attention_project_kv(Ctx, Wk, nullptr, Wv, nullptr, Kc, Vc);
        CHECK(Kc.rows == Lc && Kc.cols == C);
        CHECK(within_bf16(compare(rk, download_bf16(Kc))));
        bt::flash_attention_q_with_kv_cached_forward(X, Kc, Vc, Wq, nullptr, Wo, &Bo, nullptr, Hh, false, out2, &own_scratch);
        CHECK(out.to_host_bytes() == out2.to_host_bytes());
        CHECK(own_scratch.bytes() >= mi_flash_attention_scratch_bytes(1, Lx, Lc, C, 0));
        // W8A16 forms: INT8 weights with per-row scales against the checker fed the dequantised weights; the cached form
        // after project_kv equals the full form bit for bit
        {
            auto quant = [](uint64_t seed, int rows, int cols, std::vector<int8_t>& q, std::vector<float>& sc, std::vector<float>& deq) {
                std::vector<float> r(static_cast<size_t>(rows) * cols);
                orc_torch_randn_f32(seed, r.size(), r.data());
                q.resize(r.size()); sc.resize(rows); deq.resize(r.size());
                for (int i = 0; i < rows; ++i) sc[i] = (0.75f + 0.5f * static_cast<float>(i % 7) / 7.0f) / (42.0f * std::sqrt(static_cast<float>(cols)));
                for (size_t i = 0; i < r.size(); ++i) {
                    const float v = std::fmax(-127.f, std::fmin(127.f, std::nearbyint(r[i] * 42.0f)));
                    q[i] = static_cast<int8_t>(v);
                    deq[i] = v * sc[i / cols];
                }
            };
            std::vector<int8_t> qq, qk, qv, qo;
            std::vector<float> sq, sk, sv, so, dq, dk, dv, dO;
            quant(7111, C, C, qq, sq, dq); quant(7112, C, Cc, qk, sk, dk); quant(7113, C, Cc, qv, sv, dv); quant(7114, C, C, qo, so, dO);
            auto up8 = [](const std::vector<int8_t>& q, int r, int c) { return Tensor::from_host(q.data(), r, c, Dtype::INT8); };
            auto upf = [](const std::vector<float>& f, int r) { return Tensor::from_host(f.data(), r, 1, Dtype::FP32); };
            Tensor Wq8 = up8(qq, C, C), Wk8 = up8(qk, C, Cc), Wv8 = up8(qv, C, Cc), Wo8 = up8(qo, C, C);
            Tensor Sq = upf(sq, C), Sk = upf(sk, C), Sv = upf(sv, C), So = upf(so, C), o8, K8, V8, o8c;
            bt::flash_attention_qkvo_int8w_fp16(X, &Ctx, Wq8, Sq, nullptr, Wk8, Sk, nullptr, Wv8, Sv, nullptr, Wo8, So, &Bo, nullptr, Hh, false, o8);
            const std::vector<float> q8 = lin(x, dq, nullptr, Lx, C, C, true), k8 = lin(ctx, dk, nullptr, Lc, C, Cc, true), v8 = lin(ctx, dv, nullptr, Lc, C, Cc, true);
            std::vector<float> a8(q8.size());
            orc_sdpa(q8.data(), k8.data(), v8.data(), Lx, Lc, Hh, C / Hh, -1.0, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, nullptr, 0, a8.data(), nullptr, 0);
            orc_round_bf16(a8.data(), a8.size());
            const Err e8 = compare(lin(a8, dO, bo.data(), Lx, C, C, false), download_bf16(o8));
            std::printf("qkvo int8 weights     rel_l2=%.3e max_abs=%.3e\n", e8.rel_l2, e8.max_abs);
            CHECK(within_bf16(e8));
            bt::flash_attention_project_kv_int8w_fp16(Ctx, Wk8, Sk, nullptr, Wv8, Sv, nullptr, K8, V8);
            bt::flash_attention_q_with_kv_cached_int8w_fp16(X, K8, V8, Wq8, Sq, nullptr, Wo8, So, &Bo, nullptr, Hh, false, o8c);
            CHECK(o8.to_host_bytes() == o8c.to_host_bytes());
            Tensor Y8;
            bt::linear_forward_batched_int8w_fp16(Wo8, So, &Bo, X, Y8);
            CHECK(within_bf16(compare(lin(x, dO, bo.data(), Lx, C, C, false), download_bf16(Y8))));
            CHECK(throws_with([&] { bt::linear_forward_batched_int8w_fp16(Wo, So, &Bo, X, Y8); }, "must be INT8"));
        }
        // the linear layer alone
        Tensor Y;
        bt::linear_batched(Wo, &Bo, X, Y);
        CHECK(within_bf16(compare(lin(x, wo, bo.data(), Lx, C, C, false), download_bf16(Y))));
        CHECK(throws_with([&] { bt::flash_attention_qkvo_forward(X, &Ctx, Wq, nullptr, Wq, nullptr, Wv, nullptr, Wo, &Bo, nullptr, Hh, false, out); }, "Wk is (320, 320)"));
        CHECK(throws_with([&] { bt::flash_attention_qkvo_forward(X, nullptr, Wq, nullptr, Wq, nullptr, Wq, nullptr, Wo, &Bo, nullptr, 7, false, out); }, "does not divide"));
    }
    {   // the transformer block's fused helpers on the reference's own test shapes (tests/test_fused_parity.cpp:268-276)
        const int B = 40, d_in = 64, d_out = 48;
        std::vector<float> x = randn_bf16(7401, static_cast<size_t>(B) * d_in), w = randn_bf16(7402, static_cast<size_t>(2) * d_out * d_in),
                           b = randn_bf16(7403, 2 * d_out);
        for (float& e : w) e *= 0.1f;
        orc_round_bf16(w.data(), w.size());
        Tensor X = upload_bf16(x, B, d_in), W = upload_bf16(w, 2 * d_out, d_in), Bv = upload_bf16(b, 2 * d_out, 1), Y;
        fused_linear_geglu(X, W, Bv, Y);
        std::vector<float> t(static_cast<size_t>(B) * 2 * d_out), ref(static_cast<size_t>(B) * d_out);
        orc_linear(x.data(), w.data(), b.data(), B, 2 * d_out, d_in, t.data(), 0);
        orc_geglu_exact(t.data(), B, d_out, ref.data());
        const Err e = compare(ref, download_bf16(Y));
        std::printf("fused_linear_geglu    rel_l2=%.3e max_abs=%.3e\n", e.rel_l2, e.max_abs);
        CHECK(Y.rows == B && Y.cols == d_out && e.rel_l2 <= 5e-3);
        {   // the W8A16 overload: the reference's composition (INT8-weight linear into a 16-bit buffer, then GEGLU) from the
            // checker fed the dequantised weight, the buffer rounded to bf16
            std::vector<float> r(static_cast<size_t>(2) * d_out * d_in), deq(r.size()), sc(2 * d_out);
            std::vector<int8_t> q8(r.size());
            orc_torch_randn_f32(7408, r.size(), r.data());
            for (int i = 0; i < 2 * d_out; ++i) sc[i] = (0.75f + 0.5f * static_cast<float>(i % 7) / 7.0f) / (42.0f * std::sqrt(static_cast<float>(d_in)));
            for (size_t i = 0; i < r.size(); ++i) {
                const float v = std::fmax(-127.f, std::fmin(127.f, std::nearbyint(r[i] * 42.0f)));
                q8[i] = static_cast<int8_t>(v);
                deq[i] = v * sc[i / d_in];
            }
            Tensor W8 = Tensor::from_host(q8.data(), 2 * d_out, d_in, Dtype::INT8), S8 = Tensor::from_host(sc.data(), 2 * d_out, 1, Dtype::FP32), Y8;
            fused_linear_geglu(X, W8, S8, Bv, Y8);
            std::vector<float> t8(static_cast<size_t>(B) * 2 * d_out), ref8(static_cast<size_t>(B) * d_out);
            orc_linear(x.data(), deq.data(), b.data(), B, 2 * d_out, d_in, t8.data(), 0);
            orc_round_bf16(t8.data(), t8.size());
            orc_geglu_exact(t8.data(), B, d_out, ref8.data());
            const Err e8 = compare(ref8, download_bf16(Y8));
            std::printf("fused_linear_geglu i8 rel_l2=%.3e max_abs=%.3e\n", e8.rel_l2, e8.max_abs);
            CHECK(Y8.rows == B && Y8.cols == d_out && e8.rel_l2 <= 5e-3);
            CHECK(throws_with([&] { fused_linear_geglu(X, W, S8, Bv, Y8); }, "must be INT8"));
        }
        // Y += X on 10 x 37 and Y += row bias on 13 x 29: exact (one FP32 add, one rounding)
        std::vector<float> y0 = randn_bf16(7404, 370), xa = randn_bf16(7405, 370), want(370);
        for (int i = 0; i < 370; ++i) want[i] = y0[i] + xa[i];
        orc_round_bf16(want.data(), want.size());
        Tensor Ya = upload_bf16(y0, 10, 37), Xa = upload_bf16(xa, 10, 37);
        add_inplace_vec(Ya, Xa);
        CHECK(download_bf16(Ya) == want);
        std::vector<float> y1 = randn_bf16(7406, 13 * 29), rb = randn_bf16(7407, 29), want1(13 * 29);
        for (int i = 0; i < 13 * 29; ++i) want1[i] = y1[i] + rb[i % 29];
        orc_round_bf16(want1.data(), want1.size());
        Tensor Yb = upload_bf16(y1, 13, 29), Rb = upload_bf16(rb, 29, 1);
        add_inplace_row_bias(Yb, Rb);
        CHECK(download_bf16(Yb) == want1);
        CHECK(throws_with([&] { add_inplace_vec(Ya, Xa.row_view(0, 5)); }, "must match in shape"));
        CHECK(throws_with([&] { add_inplace_row_bias(Yb, Xa); }, "bias must hold"));
    }
    {   // packed variable-length attention: each sequence equals a call on its own rows; GQA wrapper equals the plain op at kv = q heads
        const std::vector<int32_t> cu = {0, 19, 19, 50, L};
        int32_t* d_cu = static_cast<int32_t*>(mi_malloc(cu.size() * sizeof(int32_t)));
        CHECK(d_cu != nullptr && mi_memcpy_h2d(d_cu, cu.data(), cu.size() * sizeof(int32_t)) == 0);
        Tensor o_var;
        bt::flash_attention_varlen_forward(Q, K, V, d_cu, d_cu, 4, L - 50, L - 50, H, d, false, o_var);
        const std::vector<uint8_t> all = o_var.to_host_bytes();
        for (size_t i = 0; i + 1 < cu.size(); ++i) {
            const int r0 = cu[i], n = cu[i + 1] - cu[i];
            if (n == 0) continue;
            Tensor o_seq;
            bt::flash_attention_forward(Q.row_view(r0, n), K.row_view(r0, n), V.row_view(r0, n), nullptr, H, false, o_seq);
            const std::vector<uint8_t> one = o_seq.to_host_bytes();
            CHECK(std::memcmp(all.data() + static_cast<size_t>(r0) * D * 2, one.data(), one.size()) == 0);
        }
        mi_free(d_cu);
        Tensor o_gqa, o_plain;
        bt::flash_attention_gqa_forward(Q, K, V, nullptr, H, H, false, o_gqa);
        bt::flash_attention_forward(Q, K, V, nullptr, H, false, o_plain);
        CHECK(o_gqa.to_host_bytes() == o_plain.to_host_bytes());
    }
    {   // SanaDenoiser::self_attention_ as one token-major operator: projections, qk_norm, linear attention, out-projection
        const int Ns = 192, Hs = 6, ds = 32, Ds = Hs * ds;
        auto weight = [&](uint64_t seed) {
            std::vector<float> wv = randn_bf16(seed, static_cast<size_t>(Ds) * Ds);
            for (float& f : wv) f /= std::sqrt(static_cast<float>(Ds));
            orc_round_bf16(wv.data(), wv.size());
            return wv;
        };
        const std::vector<float> x = randn_bf16(8101, static_cast<size_t>(Ns) * Ds);
        const std::vector<float> wq = weight(8102), wk = weight(8103), wv = weight(8104), wo = weight(8105);
        std::vector<float> bo = randn_bf16(8106, Ds), nq = randn_bf16(8107, Ds), nk = randn_bf16(8108, Ds);
        for (int i = 0; i < Ds; ++i) { nq[i] = 1.f + 0.25f * nq[i]; nk[i] = 1.f + 0.25f * nk[i]; }
        orc_round_bf16(nq.data(), nq.size()); orc_round_bf16(nk.data(), nk.size());
        const Tensor X = upload_bf16(x, Ns, Ds), Wq = upload_bf16(wq, Ds, Ds), Wk = upload_bf16(wk, Ds, Ds), Wv = upload_bf16(wv, Ds, Ds),
                     Wo = upload_bf16(wo, Ds, Ds), Bo = upload_bf16(bo, 1, Ds), Nq = upload_bf16(nq, 1, Ds), Nk = upload_bf16(nk, 1, Ds);
        const dit::SanaAttnWeights w{&Wq, &Wk, &Wv, &Nq, &Nk, &Wo, &Bo};
        dit::SanaAttnScratch sc;
        Tensor out, state;
        dit::sana_self_attention(X, w, Hs, out, sc, dit::RefMode::Capture, &state);
        // checker: the same chain, every intermediate rounded to bf16 as a tensor of the compute dtype
        auto lin = [&](const std::vector<float>& a, const std::vector<float>& wt, const float* b) {
            std::vector<float> y(static_cast<size_t>(Ns) * Ds);
            orc_linear(a.data(), wt.data(), b, Ns, Ds, Ds, y.data(), 0);
            return y;
        };
        std::vector<float> q = lin(x, wq, nullptr), k = lin(x, wk, nullptr), v = lin(x, wv, nullptr);
        orc_round_bf16(q.data(), q.size()); orc_round_bf16(k.data(), k.size()); orc_round_bf16(v.data(), v.size());
        std::vector<float> qn(q.size()), kn(k.size());
        orc_rms_norm(q.data(), nq.data(), 1e-5, Ns, Ds, qn.data()); orc_rms_norm(k.data(), nk.data(), 1e-5, Ns, Ds, kn.data());
        orc_round_bf16(qn.data(), qn.size()); orc_round_bf16(kn.data(), kn.size());
        std::vector<float> attn(q.size()), S(static_cast<size_t>(Hs) * ds * ds), z(static_cast<size_t>(Hs) * ds);
        orc_linear_attn_relu(qn.data(), kn.data(), v.data(), Ns, Hs, ds, 1e-15f, attn.data(), S.data(), z.data(), 0);
        orc_round_bf16(attn.data(), attn.size());
        const std::vector<float> ref = lin(attn, wo, bo.data());
        CHECK(within_bf16(compare(ref, download_bf16(out))));
        CHECK(state.rows == Hs && state.cols == ds * ds + ds && state.dtype == Dtype::FP32);
        // inject with weight 1 of the call's own state doubles numerator and denominator alike: same output, anchor untouched
        const std::vector<uint8_t> anchor_before = state.to_host_bytes();
        Tensor out2;
        dit::sana_self_attention(X, w, Hs, out2, sc, dit::RefMode::Inject, &state, 1.0f);
        CHECK(state.to_host_bytes() == anchor_before);
        CHECK(within_bf16(compare(ref, download_bf16(out2))));
        CHECK(throws_with([&] { dit::sana_self_attention(X, w, Hs, out2, sc, dit::RefMode::Inject, nullptr, 1.0f); }, "needs ref_state"));
        Tensor n_out;
        dit::rms_norm_rows(X, Nq, 1e-5f, n_out);
        std::vector<float> n_ref(x.size());
        orc_rms_norm(x.data(), nq.data(), 1e-5, Ns, Ds, n_ref.data());
        CHECK(compare(n_ref, download_bf16(n_out)).rel_l2 <= 5e-3);
    }
    {   // GPU-side error path: unsupported head_dim surfaces the C ABI's message
        Tensor out;
        CHECK(throws_with([&] { bt::flash_attention_forward(Q, K, V, nullptr, 8, false, out); }, "no kernel"));
    }
}

int main(int argc, char** argv) {
    const bool cpu_only = argc > 1 && std::string(argv[1]) == "--cpu";
    cpu_checks();
    if (!cpu_only) gpu_checks();
    if (g_failures == 0) std::printf("test_host_ops: OK\n");
    return g_failures == 0 ? 0 : 1;
}
