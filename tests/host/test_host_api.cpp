// Runs the reference's own router / remap / batch-builder test vectors (src/moe_router.zig:169-439,
// src/tests/expert_remap_test.zig, src/tests/batch_builder_tests.zig) through the C++ host layer
// (dmlx_amd/host/moe.hpp) on the GPU, plus a closed-form check of the layer forward, the way the
// reference's model smoke tests use constant weights (src/tests/deepseek_v4_tests.zig:398-610).
// Built with g++ against libdmoe.so; prints "ALL HOST TESTS PASSED" and exits 0 on success.
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <set>

#include "../../dmlx_amd/host/moe.hpp"

using namespace dmoe;

static int g_failed = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);         \
            ++g_failed;                                                           \
        }                                                                         \
    } while (0)
#define NEAR(a, b, tol) EXPECT(std::fabs((double)(a) - (double)(b)) <= (tol))

static uint16_t bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float from_bf16(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

static void test_topk(const Context &ctx) {
    { // "MoERouter topkRoute selects correct top-k experts"
        auto router = MoERouter::init({4, 2, false});
        const float s[] = {0.1f, 0.9f, 0.3f, 0.7f, 0.8f, 0.2f, 0.6f, 0.4f};
        auto r = router.topkRoute(ctx, Array::fromData(ctx, s, {2, 4}, DType::float32));
        EXPECT(r.k == 2 && r.indices.shape() == std::vector<int>({2, 2}) && r.weights.shape() == std::vector<int>({2, 2}));
        auto w = r.weights.dataSlice<float>();
        NEAR(w[0] + w[1], 1.6, 1e-5);
        NEAR(w[2] + w[3], 1.4, 1e-5);
    }
    { // "MoERouter topkRoute with weight normalization"
        auto router = MoERouter::init({3, 2, true});
        const float s[] = {0.2f, 0.6f, 0.4f};
        auto r = router.topkRoute(ctx, Array::fromData(ctx, s, {1, 3}, DType::float32));
        auto w = r.weights.dataSlice<float>();
        auto idx = r.indices.dataSlice<uint32_t>();
        NEAR(w[0] + w[1], 1.0, 1e-5);
        EXPECT((idx[0] == 1 && idx[1] == 2) || (idx[0] == 2 && idx[1] == 1));
        for (int i = 0; i < 2; ++i) NEAR(w[i], s[idx[i]] / (0.6f + 0.4f), 1e-5);
    }
    { // "MoERouter config with different num_experts and top_k"
        auto router = MoERouter::init({8, 3, false});
        const float s[] = {0.1f, 0.2f, 0.8f, 0.3f, 0.9f, 0.4f, 0.7f, 0.5f};
        auto r = router.topkRoute(ctx, Array::fromData(ctx, s, {1, 8}, DType::float32));
        auto idx = r.indices.dataSlice<uint32_t>();
        auto w = r.weights.dataSlice<float>();
        std::set<uint32_t> got(idx.begin(), idx.end());
        EXPECT(got == std::set<uint32_t>({2, 4, 6}));
        for (int i = 0; i < 3; ++i) NEAR(w[i], s[idx[i]], 1e-5);
    }
}

static void test_expand_reduce(const Context &ctx) {
    const float x[] = {1, 2, 3, 4, 5, 6};
    const uint32_t di[] = {0, 1, 2, 3};
    const float dw[] = {0.6f, 0.4f, 0.7f, 0.3f};
    RouteResult route{Array::fromData(ctx, di, {2, 2}, DType::uint32), Array::fromData(ctx, dw, {2, 2}, DType::float32), 2};
    auto ex = MoERouter::expandTokens(ctx, Array::fromData(ctx, x, {2, 3}, DType::float32), route);
    EXPECT(ex.shape() == std::vector<int>({4, 3}));
    auto e = ex.dataSlice<float>();
    const float want[] = {1, 2, 3, 1, 2, 3, 4, 5, 6, 4, 5, 6};
    for (int i = 0; i < 12; ++i) NEAR(e[i], want[i], 1e-5);

    const float eo[] = {1, 0, 0, 0, 1, 0, 0, 0, 1, 1, 1, 1};
    const float rw[] = {0.7f, 0.3f, 0.4f, 0.6f};
    RouteResult r2{Array::fromData(ctx, di, {2, 2}, DType::uint32), Array::fromData(ctx, rw, {2, 2}, DType::float32), 2};
    auto red = MoERouter::reduceExperts(ctx, Array::fromData(ctx, eo, {4, 3}, DType::float32), r2).dataSlice<float>();
    const float wr[] = {0.7f, 0.3f, 0.0f, 0.6f, 0.6f, 1.0f};
    for (int i = 0; i < 6; ++i) NEAR(red[i], wr[i], 1e-5);

    // "MoERouter end-to-end route-expand-reduce": identity expert + normalised weights give x back
    auto router = MoERouter::init({4, 2, true});
    const float s[] = {0.1f, 0.5f, 0.3f, 0.1f, 0.4f, 0.1f, 0.1f, 0.4f, 0.2f, 0.2f, 0.5f, 0.1f};
    const float x3[] = {1, 2, 3, 4, 5, 6};
    auto xs = Array::fromData(ctx, x3, {3, 2}, DType::float32);
    auto r3 = router.topkRoute(ctx, Array::fromData(ctx, s, {3, 4}, DType::float32));
    auto back = MoERouter::reduceExperts(ctx, MoERouter::expandTokens(ctx, xs, r3), r3).dataSlice<float>();
    for (int i = 0; i < 6; ++i) NEAR(back[i], x3[i], 1e-4);
}

static void test_property_18(const Context &ctx) {
    // moe_router.zig:455-628, 100 random configurations
    uint64_t seed = 18;
    auto rnd = [&](uint32_t n) {
        seed = seed * 6364136223846793005ull + 1442695040888963407ull;
        return (uint32_t)((seed >> 33) % n);
    };
    const int tok[] = {1, 2, 3, 4, 5, 8}, exps[] = {4, 6, 8, 12, 16}, ks[] = {1, 2, 3, 4};
    for (int it = 0; it < 100; ++it) {
        const int T = tok[rnd(6)], E = exps[rnd(5)], K = std::min(ks[rnd(4)], E);
        const bool normalize = rnd(2);
        std::vector<float> s((size_t)T * E);
        for (auto &v : s) v = (float)rnd(10001) / 10000.0f;
        auto r = MoERouter::init({(size_t)E, (size_t)K, normalize}).topkRoute(ctx, Array::fromData(ctx, s.data(), {T, E}, DType::float32));
        auto idx = r.indices.dataSlice<uint32_t>();
        auto w = r.weights.dataSlice<float>();
        for (int t = 0; t < T; ++t) {
            std::vector<float> sorted(s.begin() + (size_t)t * E, s.begin() + (size_t)(t + 1) * E);
            std::sort(sorted.rbegin(), sorted.rend());
            float min_sel = 2.0f, sum = 0.0f;
            std::set<uint32_t> sel;
            for (int k = 0; k < K; ++k) {
                const uint32_t e = idx[(size_t)t * K + k];
                EXPECT(e < (uint32_t)E);
                sel.insert(e);
                EXPECT(s[(size_t)t * E + e] >= sorted[K - 1] - 1e-5f);
                min_sel = std::min(min_sel, s[(size_t)t * E + e]);
                sum += w[(size_t)t * K + k];
                if (!normalize) NEAR(w[(size_t)t * K + k], s[(size_t)t * E + e], 1e-5);
            }
            EXPECT((int)sel.size() == K);
            for (int e = 0; e < E; ++e)
                if (!sel.count((uint32_t)e)) EXPECT(s[(size_t)t * E + e] <= min_sel + 1e-5f);
            if (normalize) NEAR(sum, 1.0, 1e-4);
        }
    }
}

static void test_remap_smelt_batch(const Context &ctx) {
    // expert_remap_test.zig: remap {0->0, 22->1, 31->2, 87->3} on [87,0,31,0,22,0] -> [3,0,2,0,1,0]
    auto rb = ResidentExpertProvider::preloadRemap({0, 22, 31, 87}, 256);
    const uint32_t idx[] = {87, 0, 31, 0, 22, 0};
    Array d_remap = Array::fromData(ctx, rb.first.data(), {256}, DType::int32);
    Array d_idx = Array::fromData(ctx, idx, {1, 6}, DType::uint32);
    Array out(ctx, DType::uint32, {1, 6});
    check(dmoe_remap_indices((uint32_t *)out.data(), (const int32_t *)d_remap.data(), (const uint32_t *)d_idx.data(), 6, 256, ctx.stream()));
    auto got = out.dataSlice<uint32_t>();
    const uint32_t want[] = {3, 0, 2, 0, 1, 0};
    for (int i = 0; i < 6; ++i) EXPECT(got[i] == want[i]);
    EXPECT(rb.second[22] == 0.0f && rb.second[23] == -1000.0f);

    SmeltConfig sc;
    sc.enabled = true;
    sc.load_fraction = 0.2f;
    auto mask = sc.buildMask(256);
    EXPECT(std::count(mask.begin(), mask.end(), 1) == 51 && mask[0] == 1 && mask[255] == 1);
    auto remap = SmeltConfig::buildRemap(mask);
    int slot = 0;
    for (int e = 0; e < 256; ++e) EXPECT(remap[e] == (mask[e] ? slot++ : 0));

    // batch_builder: prefill requests first, then decode; positions continue each request
    Request a, b, c;
    a.state = Request::State::prefilling;
    a.prompt_tokens = {10, 11, 12, 13, 14};
    a.prefill_offset = 2;
    b.state = Request::State::decoding;
    b.prompt_tokens = {20, 21, 22};
    b.generated_tokens = {30, 31};
    c.state = Request::State::waiting;
    c.prompt_tokens = {40};
    auto br = batch_builder::build({&a, &c}, {&b});
    {
        auto db = batch_builder::buildOnDevice(ctx, {&a, &c}, {&b}, true);
        EXPECT(db.total_tokens == br.total_tokens && db.num_requests == br.num_requests);
        auto pos = db.position_ids.dataSlice<int32_t>();
        auto tok = db.batched_tokens.dataSlice<uint32_t>();
        auto msk = db.attention_mask.dataSlice<float>();
        for (size_t i = 0; i < br.total_tokens; ++i) EXPECT(pos[i] == br.position_ids[i] && tok[i] == br.batched_tokens[i]);
        const size_t T = br.total_tokens;
        EXPECT(msk[0] == 0.0f && std::isinf(msk[1]) && msk[(T - 1) * T + (T - 1)] == 0.0f);
    }
    EXPECT(br.total_tokens == 5 && br.num_requests == 3);
    EXPECT(br.batched_tokens == std::vector<uint32_t>({12, 13, 14, 40, 31}));
    EXPECT(br.position_ids == std::vector<int32_t>({2, 3, 4, 0, 4}));
    EXPECT(br.request_offsets == std::vector<int32_t>({0, 3, 4, 5}));
}

static void test_layer_closed_form(const Context &ctx) {
    // E=2, K=2, D=256, F=64, affine-4 g64 with every code 0: each dequantized weight equals its bias.
    // Then gate = up = bg * sum(x), h = silu(gate) * up, every down output = bd * sum_f(h), and the layer
    // output is (w0 + w1) * that, the same for every expert.
    const int E = 2, K = 2, D = 256, F = 64, T = 3;
    const float bg = 0.01f, bd = 0.02f;
    std::vector<uint32_t> wz_g((size_t)E * F * D / 8, 0u), wz_d((size_t)E * D * F / 8, 0u);
    std::vector<uint16_t> s_g((size_t)E * F * D / 64, bf16(0.5f)), b_g((size_t)E * F * D / 64, bf16(bg));
    std::vector<uint16_t> s_d((size_t)E * D * F / 64, bf16(0.5f)), b_d((size_t)E * D * F / 64, bf16(bd));
    QuantizedWeight gate{wz_g.data(), s_g.data(), b_g.data(), E, F, D, 64, 4, "affine"};
    QuantizedWeight up = gate;
    QuantizedWeight down{wz_d.data(), s_d.data(), b_d.data(), E, D, F, 64, 4, "affine"};
    DSV4SwitchGLU::Options opt;
    auto layer = std::make_unique<DSV4SwitchGLU>(ctx, D, F, K, gate, up, down, opt);
    ResidentExpertProvider provider;
    provider.addLayer(std::move(layer));

    std::vector<uint16_t> x((size_t)T * D);
    std::vector<double> sumx(T, 0.0);
    for (int t = 0; t < T; ++t)
        for (int d = 0; d < D; ++d) {
            float v = 0.05f * (float)((t * 7 + d * 3) % 11 - 5);
            x[(size_t)t * D + d] = bf16(v);
            sumx[t] += from_bf16(bf16(v));
        }
    std::vector<float> scores((size_t)T * E);
    for (int t = 0; t < T; ++t) {
        scores[t * 2] = 0.3f + 0.1f * t;
        scores[t * 2 + 1] = 0.6f - 0.1f * t;
    }
    DSV4MoE moe;
    moe.gate.topk = K;
    moe.gate.n_routed_experts = E;
    moe.gate.route_scale = 1.5f;
    moe.gate.scoring_func = ScoringFunc::sigmoid;
    moe.stream_provider = &provider;
    Array hidden = Array::fromData(ctx, x.data(), {1, T, D}, DType::bfloat16);
    Array out = moe.forward(ctx, hidden, Array::fromData(ctx, scores.data(), {T, E}, DType::float32));
    EXPECT(out.shape() == std::vector<int>({1, T, D}));
    auto y = out.dataSlice<uint16_t>();
    const double bgr = from_bf16(bf16(bg)), bdr = from_bf16(bf16(bd));
    for (int t = 0; t < T; ++t) {
        const double g = bgr * sumx[t], h = g / (1.0 + std::exp(-g)) * g;
        const double want = 1.5 * bdr * F * h; // renormalised weights sum to 1, times route_scale
        for (int d = 0; d < D; d += 37) NEAR(from_bf16(y[(size_t)t * D + d]), want, std::fabs(want) * 2e-2 + 1e-6);
    }
    // DSV4MoE.forward(hidden_states) as the reference declares it: the gate runs from the hidden states. Both experts
    // are selected whatever the logits are (K = E), the renormalised weights sum to one, every expert gives the same
    // output: the closed form above again
    {
        std::vector<uint16_t> wg((size_t)E * D);
        for (int e = 0; e < E; ++e)
            for (int d = 0; d < D; ++d) wg[(size_t)e * D + d] = bf16(0.01f * (float)((e * 5 + d) % 7 - 3));
        moe.gate.load(ctx, wg.data(), D);
        auto yh = moe.forward(ctx, hidden).dataSlice<uint16_t>();
        for (int t = 0; t < T; ++t) {
            const double g = bgr * sumx[t], h = g / (1.0 + std::exp(-g)) * g;
            const double want = 1.5 * bdr * F * h;
            for (int d = 0; d < D; d += 37) NEAR(from_bf16(yh[(size_t)t * D + d]), want, std::fabs(want) * 2e-2 + 1e-6);
        }
    }
    // the same step as one call from the scores on (a second handle on the same weights): the same bytes
    DSV4SwitchGLU direct(ctx, D, F, K, gate, up, down, opt);
    Array y2 = direct.forwardFromScores(ctx, hidden.reshaped({T, D}), Array::fromData(ctx, scores.data(), {T, E}, DType::float32),
                                        nullptr, nullptr, true, 1.5f);
    auto y2v = y2.dataSlice<uint16_t>();
    for (size_t i = 0; i < y.size(); ++i) EXPECT(y2v[i] == y[i]);
    // error path: an unknown layer index is reported, not ignored
    bool threw = false;
    try {
        provider.forward(ctx, 5, hidden.reshaped({T, D}), Array(ctx, DType::uint32, {T, K}), Array(ctx, DType::float32, {T, K}));
    } catch (const Error &) {
        threw = true;
    }
    EXPECT(threw);
}

// DSV4Gate.forward from the hidden states on. x = e_0 scaled: logit of expert e = 2 * W[e][0], exactly
// representable, so the selection and the sigmoid weights are known in closed form.
static void test_gate_from_hidden(Context &ctx) {
    const int T = 3, D = 64, E = 8, K = 2;
    std::vector<uint16_t> x((size_t)T * D, bf16(0.0f)), wg((size_t)E * D, bf16(0.0f));
    for (int t = 0; t < T; ++t) x[(size_t)t * D] = bf16(2.0f);
    const float w0[E] = {0.5f, -1.0f, 1.5f, 0.25f, -0.5f, 1.0f, 0.0f, -2.0f}; // logits 1, -2, 3, .5, -1, 2, 0, -4
    for (int e = 0; e < E; ++e) wg[(size_t)e * D] = bf16(w0[e]);
    DSV4Gate gate;
    gate.topk = K;
    gate.n_routed_experts = E;
    gate.route_scale = 1.0f;
    gate.scoring_func = ScoringFunc::sigmoid;
    gate.load(ctx, wg.data(), D);
    auto r = gate.forwardHidden(ctx, Array::fromData(ctx, x.data(), {T, D}, DType::bfloat16));
    auto idx = r.second.dataSlice<uint32_t>();
    auto w = r.first.dataSlice<float>();
    const double s3 = 1.0 / (1.0 + std::exp(-3.0)), s2 = 1.0 / (1.0 + std::exp(-2.0));
    for (int t = 0; t < T; ++t) {
        EXPECT(idx[t * K] == 5u && idx[t * K + 1] == 2u); // ascending score order: expert 5 (logit 2), then 2 (logit 3)
        NEAR(w[t * K], s2 / (s2 + s3), 1e-6);
        NEAR(w[t * K + 1], s3 / (s2 + s3), 1e-6);
    }
    bool threw = false;
    try {
        DSV4Gate empty;
        empty.topk = K;
        empty.forwardHidden(ctx, Array::fromData(ctx, x.data(), {T, D}, DType::bfloat16));
    } catch (const Error &) {
        threw = true;
    }
    EXPECT(threw);
}

// mhcPost on values exact in bf16: out[t,i,:] = x * post[i] + sum_j comb[j][i] * residual[j]
static void test_block_post(Context &ctx) {
    const int T = 2, H = 16, M = 2;
    std::vector<uint16_t> x((size_t)T * H), res((size_t)T * M * H);
    for (int t = 0; t < T; ++t)
        for (int d = 0; d < H; ++d) {
            x[(size_t)t * H + d] = bf16((float)(d + 1));
            for (int j = 0; j < M; ++j) res[((size_t)t * M + j) * H + d] = bf16((float)(j + 1) * (t + 1));
        }
    const std::vector<float> post = {0.5f, 2.0f, 1.0f, 0.25f};                      // [T,M]
    const std::vector<float> comb = {1.0f, 0.5f, 0.25f, 2.0f, 0.0f, 1.0f, 1.0f, 0.0f}; // [T,M,M]
    Array out = mhcPost(ctx, Array::fromData(ctx, x.data(), {T, H}, DType::bfloat16),
                        Array::fromData(ctx, res.data(), {T, M, H}, DType::bfloat16),
                        Array::fromData(ctx, post.data(), {T, M, 1}, DType::float32),
                        Array::fromData(ctx, comb.data(), {T, M, M}, DType::float32));
    auto o = out.dataSlice<uint16_t>();
    for (int t = 0; t < T; ++t)
        for (int i = 0; i < M; ++i)
            for (int d = 0; d < H; ++d) {
                float want = (float)(d + 1) * post[(size_t)t * M + i];
                for (int j = 0; j < M; ++j) want += comb[((size_t)t * M + j) * M + i] * (float)(j + 1) * (t + 1);
                EXPECT(o[((size_t)t * M + i) * H + d] == bf16(want));
            }
    Array sum = residualAdd(ctx, Array::fromData(ctx, x.data(), {T, H}, DType::bfloat16),
                            Array::fromData(ctx, x.data(), {T, H}, DType::bfloat16));
    auto sv = sum.dataSlice<uint16_t>();
    for (int d = 0; d < H; ++d) EXPECT(sv[d] == bf16(2.0f * (d + 1)));
}

// ops.gatherMm on unquantized experts with values exact in bf16: expert e is (e + 1) * [identity rows | zeros],
// so row r of the result is (rhs[r] + 1) * x[lhs[r]][0..rows)
static void test_gather_mm(Context &ctx) {
    const int E = 3, rows = 8, cols = 16, R = 5;
    std::vector<uint16_t> w((size_t)E * rows * cols, bf16(0.0f)), x((size_t)R * cols);
    for (int e = 0; e < E; ++e)
        for (int n = 0; n < rows; ++n) w[((size_t)e * rows + n) * cols + n] = bf16((float)(e + 1));
    for (int r = 0; r < R; ++r)
        for (int k = 0; k < cols; ++k) x[(size_t)r * cols + k] = bf16((float)(r * 16 + k));
    const uint32_t rhs[R] = {2, 0, 1, 1, 2}, lhs[R] = {4, 3, 2, 1, 0};
    Array wa = Array::fromData(ctx, w.data(), {E, rows, cols}, DType::bfloat16);
    Array xa = Array::fromData(ctx, x.data(), {R, cols}, DType::bfloat16);
    Array ra = Array::fromData(ctx, rhs, {R}, DType::uint32), la = Array::fromData(ctx, lhs, {R}, DType::uint32);
    auto plain = ops::gatherMm(ctx, xa, wa, nullptr, ra, false).dataSlice<uint16_t>();
    auto gathered = ops::gatherMm(ctx, xa, wa, &la, ra, false).dataSlice<uint16_t>();
    for (int r = 0; r < R; ++r)
        for (int n = 0; n < rows; ++n) {
            EXPECT(from_bf16(plain[(size_t)r * rows + n]) == (float)((rhs[r] + 1) * (r * 16 + n)));
            EXPECT(from_bf16(gathered[(size_t)r * rows + n]) == (float)((rhs[r] + 1) * (lhs[r] * 16 + n)));
        }
    const QuantizedWeight q = QuantizedWeight::unquantized(wa.data(), E, rows, cols);
    {   // the same product on a resident copy of the stack (taken from device memory)
        quantize_mod::ResidentWeight res(ctx, q, DMOE_WEIGHTS_COPY_FROM_DEVICE);
        auto again = res.gatherQmm(ctx, xa, &la, ra, false).dataSlice<uint16_t>();
        for (size_t i = 0; i < again.size(); ++i) EXPECT(again[i] == gathered[i]);
    }
    auto back = quantize_mod::dequantize(ctx, q, 1).dataSlice<uint16_t>();
    for (int i = 0; i < rows * cols; ++i) EXPECT(back[i] == w[(size_t)rows * cols + i]);
}

// the sort block of DSV4SwitchGLU.forward and the expert_remap take, on a case small enough to sort by hand:
// flat indices [2,0, 1,2, 0,2] -> rows grouped by expert with ties in flat order
static void test_sort_and_remap(Context &ctx) {
    const uint32_t idx[6] = {2, 0, 1, 2, 0, 2};
    Array ia = Array::fromData(ctx, idx, {3, 2}, DType::uint32);
    SortedRows r = sortByExpert(ctx, ia, 3);
    const uint32_t order[6] = {1, 4, 2, 0, 3, 5}, inv[6] = {3, 0, 2, 4, 1, 5}, token[6] = {0, 2, 1, 0, 1, 2};
    const uint32_t counts[3] = {2, 1, 3}, offsets[4] = {0, 2, 3, 6};
    auto o = r.order.dataSlice<uint32_t>(), iv = r.inv_order.dataSlice<uint32_t>(), tk = r.token.dataSlice<uint32_t>();
    auto cn = r.counts.dataSlice<uint32_t>(), of = r.offsets.dataSlice<uint32_t>();
    for (int i = 0; i < 6; ++i) EXPECT(o[i] == order[i] && iv[i] == inv[i] && tk[i] == token[i]);
    for (int e = 0; e < 3; ++e) EXPECT(cn[e] == counts[e]);
    for (int e = 0; e < 4; ++e) EXPECT(of[e] == offsets[e]);
    const int32_t remap[3] = {5, 0, 7};
    auto m = remapIndices(ctx, Array::fromData(ctx, remap, {3}, DType::int32), ia).dataSlice<uint32_t>();
    const uint32_t want[6] = {7, 5, 0, 7, 5, 7};
    for (int i = 0; i < 6; ++i) EXPECT(m[i] == want[i]);
}

// quantize_mod::dequantFp8 with values exact in bf16: byte 0x38 is 1.0, 0x40 is 2.0, 0xB8 is -1.0 (E4M3FN); a 3 x 5 weight
// with 2 x 2 blocks (neither dimension a whole number of blocks) and scales that are powers of two, once as f32 and
// once as E8M0 bytes
static void test_dequant_fp8(Context &ctx) {
    const int rows = 3, cols = 5, bs = 2;
    const uint8_t w[rows * cols] = {0x38, 0x40, 0xB8, 0x38, 0x40, 0x40, 0x40, 0x38, 0xB8, 0x00, 0x38, 0xB8, 0x40, 0x40, 0x38};
    const float val[rows * cols] = {1, 2, -1, 1, 2, 2, 2, 1, -1, 0, 1, -1, 2, 2, 1};
    const float sf[2 * 3] = {1.0f, 0.5f, 4.0f, 2.0f, 0.25f, 8.0f};
    const uint8_t se[2 * 3] = {127, 126, 129, 128, 125, 130};
    Array wa = Array::fromData(ctx, w, {rows, cols}, DType::uint8);
    Array fa = Array::fromData(ctx, sf, {2, 3}, DType::float32), ea = Array::fromData(ctx, se, {2, 3}, DType::uint8);
    auto a = quantize_mod::dequantFp8(ctx, wa, fa, bs).dataSlice<uint16_t>();
    auto b = quantize_mod::dequantFp8(ctx, wa, ea, bs).dataSlice<uint16_t>();
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < cols; ++c) {
            const float want = val[r * cols + c] * sf[(r / bs) * 3 + c / bs];
            EXPECT(from_bf16(a[(size_t)r * cols + c]) == want);
            EXPECT(from_bf16(b[(size_t)r * cols + c]) == want);
        }
}

int main() {
    try {
        Context ctx(0);
        test_topk(ctx);
        test_expand_reduce(ctx);
        test_property_18(ctx);
        test_remap_smelt_batch(ctx);
        test_layer_closed_form(ctx);
        test_gate_from_hidden(ctx);
        test_block_post(ctx);
        test_gather_mm(ctx);
        test_dequant_fp8(ctx);
        test_sort_and_remap(ctx);
        ctx.synchronize();
    } catch (const Error &e) {
        std::printf("dmoe::Error %d: %s\n", e.code, e.what());
        return 2;
    }
    if (g_failed) {
        std::printf("%d check(s) failed\n", g_failed);
        return 1;
    }
    std::printf("ALL HOST TESTS PASSED\n");
    return 0;
}
