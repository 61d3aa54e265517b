// Runs on the GPU box: the C++ host mirror (include/fusor_hip.hpp) exercised with the inputs and
// assertions of the reference's own tests.
//   fusor-ml/fusor/src/composite/flash_attention.rs:207-358  (attention, CPU arm tests)
//   fusor-ml/fusor/src/cache/attention_mask.rs:88-111        (causal mask)
//   fusor-ml/fusor/src/cache/mask_cache.rs:122-175           (mask cache)
//   fusor-ml/fusor/src/cache/kv_cache.rs:74-157, tensor_cache.rs:130-186  (KV cache)
#include <cmath>
#include <cstdio>
#include <limits>
#include <vector>

#include "fusor_hip.hpp"

using namespace fusor_hip;
static int failures = 0;
#define EXPECT(cond, ...)                                             \
    do {                                                              \
        if (!(cond)) {                                                \
            failures++;                                               \
            printf("FAIL %s:%d: %s : ", __FILE__, __LINE__, #cond);   \
            printf(__VA_ARGS__);                                      \
            printf("\n");                                             \
        }                                                             \
    } while (0)

static const float NEG_INF = -std::numeric_limits<float>::infinity();

static Tensor<4> t4(const Device &d, std::vector<float> v, uint32_t a, uint32_t b, uint32_t c, uint32_t e) {
    const uint32_t shape[4] = {a, b, c, e};
    return Tensor<4>::from_slice(d, DType::F32, shape, v.data());
}
static std::vector<float> host(const Tensor<4> &t) {
    std::vector<float> h(t.numel());
    t.to_host(h.data());
    return h;
}
static std::vector<float> host2(const Tensor<2> &t) {
    std::vector<float> h(t.numel());
    t.to_host(h.data());
    return h;
}

static void test_flash_attention_cpu(const Device &d) {  // flash_attention.rs:207-239
    auto q = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), k = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), v = t4(d, {1, 2, 3, 4}, 1, 1, 2, 2);
    auto out = q.flash_attention(k, v, 1.0f / std::sqrt(2.0f));
    EXPECT(out.shape()[0] == 1 && out.shape()[1] == 1 && out.shape()[2] == 2 && out.shape()[3] == 2, "shape");
    for (float x : host(out)) EXPECT(std::isfinite(x), "non-finite %f", x);
}

static void test_flash_attention_cpu_with_mask(const Device &d) {  // :241-276
    auto q = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), k = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), v = t4(d, {1, 2, 3, 4}, 1, 1, 2, 2);
    const float m[4] = {0, NEG_INF, 0, 0};
    const uint32_t ms[2] = {2, 2};
    auto mask = Tensor<2>::from_slice(d, DType::F32, ms, m);
    auto out = host(q.flash_attention(k, v, 1.0f / std::sqrt(2.0f), std::make_pair(&mask, MaskKind::QKMask)));
    EXPECT(std::fabs(out[0] - 1.0f) < 0.01f, "row 0 should equal V[0]: %f", out[0]);
    EXPECT(std::fabs(out[1] - 2.0f) < 0.01f, "row 0 should equal V[0]: %f", out[1]);
}

// the same call with the mask's interval table computed once (AttentionMask::intervals) and passed with the tensor
static void test_flash_attention_with_mask_and_its_interval_table(const Device &d) {
    auto q = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), k = t4(d, {1, 0, 0, 1}, 1, 1, 2, 2), v = t4(d, {1, 2, 3, 4}, 1, 1, 2, 2);
    auto am = AttentionMask::causal(d, 2);
    const void *table = am.intervals();
    EXPECT(table != nullptr && table == am.intervals(), "the table is computed once");
    auto plain = host(q.flash_attention(k, v, 1.0f / std::sqrt(2.0f), std::make_pair(&am.mask(), MaskKind::QKMask)));
    auto out = host(q.flash_attention(k, v, 1.0f / std::sqrt(2.0f), std::make_pair(&am.mask(), MaskKind::QKMask), nullptr, nullptr, table));
    for (int i = 0; i < 4; i++) EXPECT(out[i] == plain[i], "element %d: %f with the table, %f without", i, out[i], plain[i]);
    EXPECT(std::fabs(out[0] - 1.0f) < 0.01f && std::fabs(out[1] - 2.0f) < 0.01f, "row 0 should equal V[0]: %f %f", out[0], out[1]);
}

static void test_flash_attention_gqa_cpu(const Device &d) {  // :278-313
    std::vector<float> q(16), k(8), v(8);
    for (int i = 0; i < 16; i++) q[i] = i * 0.1f;
    for (int i = 0; i < 8; i++) k[i] = i * 0.1f + 1.0f, v[i] = i * 0.1f + 2.0f;
    auto out = t4(d, q, 1, 4, 2, 2).flash_attention(t4(d, k, 1, 2, 2, 2), t4(d, v, 1, 2, 2, 2), 1.0f / std::sqrt(2.0f));
    EXPECT(out.shape()[1] == 4, "output keeps Q's head count");
    for (float x : host(out)) EXPECT(std::isfinite(x), "non-finite %f", x);
    // Q heads (3) not divisible by K/V heads (2): the reference asserts (:94-99)
    bool threw = false;
    try {
        t4(d, std::vector<float>(12, 0.f), 1, 3, 2, 2).flash_attention(t4(d, k, 1, 2, 2, 2), t4(d, v, 1, 2, 2, 2), 1.0f);
    } catch (const Panic &e) {
        threw = std::string(e.what()) == "Number of Q heads (3) must be divisible by number of K/V heads (2)";
    }
    EXPECT(threw, "divisibility panic with the reference's message");
}

static void test_flash_attention_cpu_with_batch_key_mask(const Device &d) {  // :315-358
    std::vector<float> q(12), k(12), v(12);
    for (int i = 0; i < 12; i++) q[i] = i * 0.1f, k[i] = i * 0.1f + 1.0f, v[i] = i * 0.1f + 2.0f;
    const float m[6] = {0, 0, 0, 0, 0, NEG_INF};
    const uint32_t ms[2] = {2, 3};
    auto mask = Tensor<2>::from_slice(d, DType::F32, ms, m);
    auto out = t4(d, q, 2, 1, 3, 2).flash_attention(t4(d, k, 2, 1, 3, 2), t4(d, v, 2, 1, 3, 2), 1.0f / std::sqrt(2.0f),
                                                    std::make_pair(&mask, MaskKind::BatchKeyMask));
    EXPECT(out.shape()[0] == 2 && out.shape()[2] == 3, "shape");
    for (float x : host(out)) EXPECT(std::isfinite(x), "non-finite %f", x);
}

static void test_attention_mask_causal(const Device &d) {  // attention_mask.rs:88-111
    auto m = host2(AttentionMask::causal(d, 3).mask());
    const float want[9] = {0, NEG_INF, NEG_INF, 0, 0, NEG_INF, 0, 0, 0};
    for (int i = 0; i < 9; i++) EXPECT(m[i] == want[i], "causal[%d] = %f", i, m[i]);
}

static void test_mask_cache(const Device &d) {  // mask_cache.rs:122-175
    MaskCache cache;
    EXPECT(cache.get_mask(3, 0, std::nullopt, d).mask().shape()[0] == 3, "3x3");
    EXPECT(cache.get_mask(5, 0, std::nullopt, d).mask().shape()[1] == 5, "5x5");
    auto padded = cache.get_mask(2, 3, std::nullopt, d);
    EXPECT(padded.mask().shape()[0] == 2 && padded.mask().shape()[1] == 5, "offset pads to [2, 5]");
    auto sw = cache.get_mask(4, 0, 2, d);
    auto m = host2(sw.mask());
    auto at = [&](int i, int j) { return m[i * 4 + j]; };
    EXPECT(at(0, 0) == 0 && at(0, 1) == NEG_INF && at(1, 0) == 0 && at(1, 1) == 0, "rows 0-1");
    EXPECT(at(2, 0) == NEG_INF && at(2, 1) == 0 && at(2, 2) == 0, "row 2");
    EXPECT(at(3, 1) == NEG_INF && at(3, 2) == 0 && at(3, 3) == 0, "row 3");
}

static void test_kv_cache(const Device &d) {  // kv_cache.rs:74-157, tensor_cache.rs:130-186
    KvCache cache(d, 2, 3);
    auto k1 = t4(d, {1, 2}, 1, 1, 1, 2), v1 = t4(d, {5, 6}, 1, 1, 1, 2);
    auto r1 = cache.append(d, k1, v1);
    EXPECT(r1.first.shape()[2] == 1 && cache.current_seq_len() == 1, "first append stores the tensor");
    auto k2 = t4(d, {3, 4}, 1, 1, 1, 2), v2 = t4(d, {7, 8}, 1, 1, 1, 2);
    auto r2 = cache.append(d, k2, v2);
    EXPECT(r2.first.shape()[2] == 2 && cache.current_seq_len() == 2, "second append");
    auto kh = host(r2.first), vh = host(r2.second);
    EXPECT(kh[0] == 1 && kh[1] == 2 && kh[2] == 3 && kh[3] == 4, "keys 1 2 3 4");
    EXPECT(vh[0] == 5 && vh[3] == 8, "values 5..8");
    // growth beyond max_sequence_len keeps the last positions (tensor_cache.rs:55-78)
    auto k3 = t4(d, {9, 10, 11, 12}, 1, 1, 2, 2), v3 = t4(d, {13, 14, 15, 16}, 1, 1, 2, 2);
    auto r3 = cache.append(d, k3, v3);
    EXPECT(r3.first.shape()[2] == 3 && cache.current_seq_len() == 3, "truncated to max_sequence_len");
    kh = host(r3.first);
    EXPECT(kh[0] == 3 && kh[1] == 4 && kh[2] == 9 && kh[5] == 12, "last three positions kept");
    cache.reset();
    EXPECT(cache.current_seq_len() == 0, "reset");
}

static void test_rope(const Device &d) {  // rope.rs:270-400 (inputs), rope.rs:46-137 (values)
    const uint32_t rows = 11, half = 32;
    std::vector<float> c(rows * half), s(rows * half), x(3 * 11 * 64);
    for (uint32_t i = 0; i < rows; i++)
        for (uint32_t j = 0; j < half; j++) {
            const float a = (float)i / std::pow(10000.0f, (float)(2 * j) / 64.0f);
            c[i * half + j] = std::cos(a);
            s[i * half + j] = std::sin(a);
        }
    for (size_t k = 0; k < x.size(); k++) x[k] = std::sin((float)(k % 64));
    RopeCache rope(d, rows, half, c.data(), s.data());
    auto t = t4(d, x, 1, 3, 11, 64);
    auto qk = rope.forward(t, t, 0);
    auto qi = rope.forward_interleaved(t, t, 0);
    auto y = host(qk.first), yi = host(qi.second);
    EXPECT(qk.first.shape()[1] == 3 && qk.first.shape()[2] == 11 && qk.first.shape()[3] == 64, "rope shape");
    int bad = 0;
    for (uint32_t h = 0; h < 3; h++)
        for (uint32_t r = 0; r < 11; r++)
            for (uint32_t i = 0; i < 32; i++) {
                const size_t base = ((size_t)h * 11 + r) * 64;
                const float cc = c[r * half + i], ss = s[r * half + i];
                // the volatile temporaries keep the host compiler from fusing the products into the sums
                volatile float a0 = x[base + i] * cc, a1 = x[base + i + 32] * ss, b0 = x[base + i + 32] * cc, b1 = x[base + i] * ss;
                if (y[base + i] != a0 - a1 || y[base + i + 32] != b0 + b1 || !std::isfinite(y[base + i])) bad++;
                volatile float e0 = x[base + 2 * i] * cc, e1 = x[base + 2 * i + 1] * ss, f0 = x[base + 2 * i] * ss, f1 = x[base + 2 * i + 1] * cc;
                if (yi[base + 2 * i] != e0 - e1 || yi[base + 2 * i + 1] != f0 + f1) bad++;
            }
    EXPECT(bad == 0, "%d rope values differ from x*cos + rotate_half(x)*sin", bad);
    // fused into the cache write: rope(k) lands in the cache, v unchanged
    KvCache cache(d, 2, 64);
    auto kv = cache.append_rope(rope.tables(0, false), t, t);
    auto kc = host(kv.first), vc = host(kv.second);
    bad = 0;
    for (size_t k = 0; k < x.size(); k++)
        if (kc[k] != y[k] || vc[k] != x[k]) bad++;
    EXPECT(bad == 0, "%d cached values differ after append_rope", bad);
}

static void test_rms_norm(const Device &d) {  // rms_norm.rs:163-186 (values), normalization.rs:351-407 (order)
    const float w2[2] = {2.0f, 2.0f};
    RmsNorm norm(d, DType::F32, 2, w2, nullptr, 1e-5f);
    auto t = t4(d, {3.0f, 4.0f, 6.0f, 8.0f}, 1, 1, 2, 2);
    auto y = host(norm.forward_generic_4d(t));
    const float rms1 = std::sqrt(12.5f);
    EXPECT(std::fabs(y[0] - 3.0f / rms1 * 2.0f) < 1e-4f && std::fabs(y[1] - 4.0f / rms1 * 2.0f) < 1e-4f, "rms norm row [3, 4]: %g %g", y[0], y[1]);
    // every step exact: squares sum to 16, mean 4, root 2; the bias is added last
    const float w4[4] = {1.0f, 3.0f, 0.5f, -7.0f}, b4[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    RmsNorm exact(d, DType::F32, 4, w4, b4, 0.0f);
    auto e = host(exact.forward_generic_4d(t4(d, {2.0f, -2.0f, 2.0f, -2.0f}, 1, 1, 1, 4)));
    EXPECT(e[0] == 2.0f && e[1] == -2.0f && e[2] == 1.5f && e[3] == 8.0f, "exact rms norm row: %g %g %g %g", e[0], e[1], e[2], e[3]);
    // fused into the rotation: at position 0 the rotation is the identity, so norm + rope == norm
    const float c0[2] = {1.0f, 1.0f}, s0[2] = {0.0f, 0.0f};
    RopeCache rope(d, 1, 2, c0, s0);
    const fhip_rms_norm n = exact.c();
    auto f = host(rope.apply(t4(d, {2.0f, -2.0f, 2.0f, -2.0f}, 1, 1, 1, 4), 0, false, std::nullopt, &n));
    EXPECT(f[0] == 2.0f && f[1] == -2.0f && f[2] == 1.5f && f[3] == 8.0f, "norm fused into rope: %g %g %g %g", f[0], f[1], f[2], f[3]);
    KvCache cache(d, 2, 8);
    auto kv = cache.append_rope(rope.tables(0, false), t4(d, {2.0f, -2.0f, 2.0f, -2.0f}, 1, 1, 1, 4), t4(d, {5.0f, 6.0f, 7.0f, 8.0f}, 1, 1, 1, 4), &n);
    auto kc = host(kv.first), vc = host(kv.second);
    EXPECT(kc[0] == 2.0f && kc[3] == 8.0f && vc[0] == 5.0f && vc[3] == 8.0f, "norm fused into the cache append");
    // q, k and v of a step prepared by one launch
    KvCache cache2(d, 2, 8);
    const uint32_t qshape[4] = {1, 1, 1, 4};
    auto q_out = Tensor<4>::empty(d, DType::F32, qshape);
    auto kv2 = cache2.qkv_rope_append(rope.tables(0, false), t4(d, {2.0f, -2.0f, 2.0f, -2.0f}, 1, 1, 1, 4), q_out,
                                      t4(d, {2.0f, -2.0f, 2.0f, -2.0f}, 1, 1, 1, 4), t4(d, {5.0f, 6.0f, 7.0f, 8.0f}, 1, 1, 1, 4), &n, nullptr);
    auto qo = host(q_out), k2 = host(kv2.first), v2 = host(kv2.second);
    EXPECT(qo[0] == 2.0f && qo[1] == -2.0f && qo[2] == 1.5f && qo[3] == 8.0f, "q normalised in the one-launch step: %g %g %g %g", qo[0], qo[1], qo[2], qo[3]);
    EXPECT(k2[0] == 2.0f && k2[1] == -2.0f && k2[3] == -2.0f && v2[0] == 5.0f && v2[3] == 8.0f, "k (no norm) and v in the one-launch step");
}

static void test_capture(const Device &d) {  // a recorded rope call replays on new contents of the same buffers
    const float c0[4] = {1.0f, 1.0f, 0.0f, 0.0f}, s0[4] = {0.0f, 0.0f, 1.0f, 1.0f};  // position 0: identity, 1: +90 degrees
    RopeCache rope(d, 2, 2, c0, s0);
    auto x = t4(d, {1.0f, 2.0f, 3.0f, 4.0f, 1.0f, 2.0f, 3.0f, 4.0f}, 1, 1, 2, 4);
    const uint32_t shape[4] = {1, 1, 2, 4};
    auto y = Tensor<4>::empty(d, DType::F32, shape);
    const fhip_rope_tables t = rope.tables(0, false);
    const fhip_tensor4 cx = x.c4(), cy = y.c4();
    Graph g = d.capture([&] { check(fhip_rope(d.stream(), &t, &cx, FHIP_F32, &cy, FHIP_F32)); });
    g.launch();
    auto h = host(y);
    // row 0 unchanged; row 1: pairs (0,2), (1,3) turned by 90 degrees: (1,3) -> (-3,1), (2,4) -> (-4,2)
    EXPECT(h[0] == 1.0f && h[3] == 4.0f && h[4] == -3.0f && h[5] == -4.0f && h[6] == 1.0f && h[7] == 2.0f,
           "captured rope: %g %g %g %g | %g %g %g %g", h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]);
    const float nx[8] = {5.0f, 6.0f, 7.0f, 8.0f, 5.0f, 6.0f, 7.0f, 8.0f};
    check(fhip_memcpy_h2d(d.stream(), cx.ptr, nx, sizeof(nx)));
    g.launch();
    h = host(y);
    EXPECT(h[0] == 5.0f && h[4] == -7.0f && h[5] == -8.0f && h[6] == 5.0f && h[7] == 6.0f, "replay on new contents: %g %g %g %g",
           h[4], h[5], h[6], h[7]);
}

// A multi-token decode step through the cache, as a turn that feeds three tokens on top of a cached context does
// (models/kalosm-llama/src/raw/mod.rs:618-620: the mask is get_mask(3, pos, None)).  With all keys equal every
// visible key weighs the same, and with V[j][d] = j the output of row r is the mean of 0 .. n_r - 1, n_r = pos + r + 1.
static void test_multi_token_step_on_a_cache(const Device &d) {
    const uint32_t H = 4, Hkv = 2, D = 64, pos = 700, n = 3;
    KvCache cache(d, 2, 4096);
    std::vector<float> k(Hkv * pos * D, 0.25f), v(Hkv * pos * D);
    for (uint32_t g = 0; g < Hkv; g++)
        for (uint32_t j = 0; j < pos; j++)
            for (uint32_t e = 0; e < D; e++) v[(g * pos + j) * D + e] = (float)j;
    cache.append(d, t4(d, k, 1, Hkv, pos, D), t4(d, v, 1, Hkv, pos, D));
    std::vector<float> kn(Hkv * n * D, 0.25f), vn(Hkv * n * D);
    for (uint32_t g = 0; g < Hkv; g++)
        for (uint32_t j = 0; j < n; j++)
            for (uint32_t e = 0; e < D; e++) vn[(g * n + j) * D + e] = (float)(pos + j);
    auto all = cache.append(d, t4(d, kn, 1, Hkv, n, D), t4(d, vn, 1, Hkv, n, D));
    EXPECT(all.first.shape()[2] == pos + n, "cache holds the context and the new rows");
    std::vector<float> q(H * n * D, 0.5f);
    auto tq = t4(d, q, 1, H, n, D);
    MaskCache masks;
    auto am = masks.get_mask(n, pos, std::nullopt, d);
    EXPECT(am.mask().shape()[0] == n && am.mask().shape()[1] == pos + n, "mask [3, pos + 3]");
    auto out_t = tq.flash_attention(all.first, all.second, 0.125f, std::make_pair(&am.mask(), MaskKind::QKMask));
    auto out = host(out_t);
    auto out_a = host(tq.flash_attention(all.first, all.second, 0.125f, std::nullopt, &*am.analytic()));
    for (uint32_t h = 0; h < H; h++)
        for (uint32_t r = 0; r < n; r++) {
            const float want = 0.5f * (float)(pos + r);  // mean of 0 .. pos + r
            const float got = out[(h * n + r) * D + 7], got_a = out_a[(h * n + r) * D + 7];
            EXPECT(std::fabs(got - want) < 1e-3f * want, "head %u row %u: %f, want %f", h, r, got, want);
            EXPECT(got == got_a, "mask tensor and analytic descriptor differ: %f vs %f", got, got_a);
        }
}

// the benchmark's calibration entry points, called through the C header
// A batched decode step whose splits are merged inside the kernel (one launch): 16 sequences x 8 KV heads = 128 units,
// 4096 keys each.  All keys equal: every key weighs the same, and with V[b][g][j][e] = j % 7 + e the output is the mean
// over j of that, whichever query it is for.
static void test_batched_decode_step_merged_inside_the_kernel(const Device &d) {
    const uint32_t B = 16, H = 32, Hkv = 8, S = 4096, D = 128;
    std::vector<float> k((size_t)B * Hkv * S * D, 0.125f), v((size_t)B * Hkv * S * D);
    for (size_t r = 0; r < (size_t)B * Hkv; r++)
        for (uint32_t j = 0; j < S; j++)
            for (uint32_t e = 0; e < D; e++) v[(r * S + j) * D + e] = (float)(j % 7) + (float)e;
    std::vector<float> q((size_t)B * H * D);
    for (size_t i = 0; i < q.size(); i++) q[i] = (float)((i * 37) % 11) * 0.1f - 0.5f;
    auto tq = t4(d, q, B, H, 1, D), tk = t4(d, k, B, Hkv, S, D), tv = t4(d, v, B, Hkv, S, D);
    fhip_attn_args a{};
    a.q = tq.c4(), a.k = tk.c4(), a.v = tv.c4(), a.out = tq.c4();
    a.dtype = a.out_dtype = FHIP_F32;
    a.scale = 0.1f;
    fhip_decode_plan_info plan{};
    check(fhip_flash_attention_decode_plan(d.stream(), &a, &plan));
    EXPECT(plan.is_decode == 1 && plan.nsplit >= 2 && plan.nsplit <= 8 && plan.kernels == 1, "plan: decode %d, %d splits, %d kernels",
           plan.is_decode, plan.nsplit, plan.kernels);
    double mean7 = 0;
    for (uint32_t j = 0; j < S; j++) mean7 += j % 7;
    mean7 /= S;
    for (int rep = 0; rep < 3; rep++) {  // the workspace's arrival counters are reused from call to call
        auto out = host(tq.flash_attention(tk, tv, 0.1f));
        float worst = 0;
        for (size_t r = 0; r < (size_t)B * H; r++)
            for (uint32_t e = 0; e < D; e++) worst = std::fmax(worst, std::fabs(out[r * D + e] - (float)(mean7 + e)));
        EXPECT(worst < 1e-3f, "call %d: output should be the mean of V over the keys, off by %g", rep, worst);
    }
}

static void test_calibrations(const Device &d) {
    const size_t cus = (size_t)d.info().compute_units;
    Buffer scratch(d, cus * 1040), data(d, 1 << 20);
    check(fhip_memset(d.stream(), data.ptr(), 0, 1 << 20));
    check(fhip_calibration_read(d.stream(), data.ptr(), 1 << 20, scratch.ptr(), cus * 1040));
    check(fhip_calibration_mfma(d.stream(), FHIP_F16, 1, 100, 50, scratch.ptr(), cus * 1040));
    check(fhip_stream_synchronize(d.stream()));
    EXPECT(fhip_calibration_mfma(d.stream(), FHIP_F32, 1, 100, 50, scratch.ptr(), cus * 1040) == FHIP_ERR_UNSUPPORTED,
           "the matrix-core loop takes 16-bit types");
}

int main() {
    try {
        Device d(0);
        test_flash_attention_cpu(d);
        test_flash_attention_cpu_with_mask(d);
        test_flash_attention_with_mask_and_its_interval_table(d);
        test_flash_attention_gqa_cpu(d);
        test_flash_attention_cpu_with_batch_key_mask(d);
        test_attention_mask_causal(d);
        test_mask_cache(d);
        test_kv_cache(d);
        test_rope(d);
        test_rms_norm(d);
        test_capture(d);
        test_multi_token_step_on_a_cache(d);
        test_batched_decode_step_merged_inside_the_kernel(d);
        test_calibrations(d);
    } catch (const std::exception &e) {
        printf("exception: %s\n", e.what());
        return 2;
    }
    printf("%s (%d failures)\n", failures ? "FAILED" : "ok", failures);
    return failures ? 1 : 0;
}
