// GPU tests of the C++ host shim, written the way the reference tests its own operator layer
// (tests/test_qwen.cpp, cited per case): build tiny deterministic inputs through the Buffer
// interface, run the operators, compare bytes.  The CPU oracle (oracle/zc_oracle.h) is the checker.
#include "reference_callers.hpp"
#include "../../zerocool_amd/csrc/engine/route_trace.hpp"
#include <unistd.h>
#include "../../oracle/zc_oracle.h"
#include <algorithm>
#include <bit>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <numeric>

using namespace zerocool::engine;
static int failures = 0, checks = 0;
#define CHECK(cond) do { ++checks; if (!(cond)) { ++failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)
#define CHECK_THROWS(expr) do { ++checks; bool threw = false; try { expr; } catch (const std::exception&) { threw = true; } \
    if (!threw) { ++failures; std::printf("  FAILED %s:%d: no throw: %s\n", __FILE__, __LINE__, #expr); } } while (0)
#define TEST(name) std::printf("[test] %s\n", name); std::fflush(stdout);

static MoeShape small_shape() { MoeShape s; s.hidden = 512; s.experts = 32; s.topk = 4; s.inter = 128; return s; }

// tests/test_qwen.cpp:1074-1085 at a parameterised shape, into host memory
static std::vector<std::byte> expert_fixture(const MoeShape& s, uint32_t seed, bool shared = false) {
    std::vector<std::byte> rec(s.expert_bytes(shared));
    const auto c = s.abi(); zco_config_t oc; std::memcpy(&oc, &c, sizeof oc);
    for (int p = 0; p < 3; ++p) {
        zco_linear_t l; zco_expert_linear(&oc, shared, reinterpret_cast<const uint8_t*>(rec.data()), p, &l);
        auto* w = reinterpret_cast<uint32_t*>(const_cast<void*>(l.weight));
        for (size_t i = 0; i < uint64_t(l.input) * l.output * l.bits / 32; ++i) w[i] = uint32_t(i * 2654435761u + (seed + p * 29u) * 1234567u);
        auto* sc = const_cast<uint16_t*>(l.scales); auto* bi = const_cast<uint16_t*>(l.biases);
        for (size_t i = 0; i < uint64_t(l.input / l.group) * l.output; ++i) { sc[i] = uint16_t(0x3b00 + p * 32); bi[i] = uint16_t(0xbc00 + p * 16); }
    }
    return rec;
}
static Buf to_hbm(Metal& gpu, const std::vector<std::byte>& bytes) {
    auto b = gpu.allocate(bytes.size(), AllocationClass::Expert); gpu.write(b, 0, bytes); return b;
}
static zco_config_t oracle_config(const MoeShape& s) { const auto c = s.abi(); zco_config_t oc; std::memcpy(&oc, &c, sizeof oc); return oc; }

static void test_bf16() {   // :277-283
    TEST("checked sizes and BF16 rounding");
    CHECK_THROWS(checked_add(UINT64_MAX, 1)); CHECK_THROWS(checked_mul(UINT64_MAX, 2)); CHECK(checked_mul(0, UINT64_MAX) == 0);
    CHECK(bf16(0x3f80) == 1.0f); CHECK(round_bf16(1.00390625f) == 1.0f);
    CHECK(std::isnan(round_bf16(NAN))); CHECK(std::isinf(round_bf16(INFINITY)));
}
static void test_q4_matmul() {   // :634-659
    TEST("affine Q4 matmul against a double-precision oracle, fused SwiGLU identity");
    Metal gpu; constexpr int K = 128, N = 7, T = 3;
    auto w = gpu.allocate(N * K / 2), s = gpu.allocate(N * (K / 64) * 2), b = gpu.allocate(N * (K / 64) * 2);
    auto x = gpu.zeros(T * K);
    for (int i = 0; i < N * K / 8; ++i) reinterpret_cast<uint32_t*>(w->data)[i] = 0x76543210u + uint32_t(i % 8) * 0x11111111u;
    for (int i = 0; i < N * K / 64; ++i) { reinterpret_cast<uint16_t*>(s->data)[i] = 0x3d80; reinterpret_cast<uint16_t*>(b->data)[i] = 0xbe80; }
    for (int i = 0; i < T * K; ++i) x->floats()[i] = float(i % 11 - 5) / 16;
    Linear l{{w}, {s}, {b}, K, N, 64, 0, true};
    auto result = gpu.linear(l, x, T); gpu.finish();
    for (int t = 0; t < T; ++t) for (int n = 0; n < N; ++n) {
        double sum = 0;
        for (int k = 0; k < K; ++k) {
            auto word = reinterpret_cast<uint32_t*>(w->data)[n * K / 8 + k / 8];
            sum += (double((word >> (4 * (k % 8))) & 15) / 16.0 - 0.25) * x->floats()[t * K + k];
        }
        const float want = round_bf16(float(sum));
        CHECK(std::fabs(result->floats()[t * N + n] - want) <= 1e-4f * std::fabs(want) + 1e-7f);
    }
    auto fused = gpu.gated_linear(l, l, x, T); gpu.finish();
    for (size_t i = 0; i < result->floats().size(); ++i) {
        float v = result->floats()[i];
        float y = round_bf16(1 / round_bf16(1 + round_bf16(std::exp(std::abs(v)))));
        float gate = v < 0 ? y : round_bf16(1 - y);
        CHECK(fused->floats()[i] == round_bf16(round_bf16(v * gate) * v));
    }
    auto invalid = l; invalid.bits = 3; CHECK_THROWS(gpu.linear(invalid, x, T));
    invalid = l; invalid.weight.offset = 1; CHECK_THROWS(gpu.linear(invalid, x, T));   // truncated binding, :689
    CHECK_THROWS(gpu.linear(l, x, T + 1));
    auto rows = gpu.allocate(4); reinterpret_cast<int*>(rows->data)[0] = T; CHECK_THROWS(gpu.gated_linear(l, l, x, 1, rows));
    gpu.finish();
}
static void test_route() {   // :744-754 and the refusals of :793-796
    TEST("routing selects exactly ten experts and normalises");
    Metal gpu; std::vector<float> values(512);
    for (int i = 0; i < 512; ++i) values[i] = float(i % 41) - 100;
    auto logits = gpu.upload(values), ids = gpu.allocate(40), weights = gpu.allocate(40);
    gpu.route(logits, ids, weights, 1); gpu.finish();
    std::vector<int> order(512); std::iota(order.begin(), order.end(), 0);
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return values[a] > values[b]; });
    float sum = 0;
    for (int i = 0; i < 10; ++i) { CHECK(reinterpret_cast<int*>(ids->data)[i] == order[i]); sum += weights->floats()[i]; }
    CHECK(std::fabs(sum - 1) < 1e-6f);
    CHECK_THROWS(gpu.route(logits, ids, weights, 0)); CHECK_THROWS(gpu.route(logits, ids, weights, 2)); CHECK_THROWS(gpu.route({}, ids, weights, 1));
}
static void test_moe_sum() {   // :827-842
    TEST("expert reduction preserves the reference BF16 midpoint decision");
    Metal gpu; const uint32_t H = gpu.shape().hidden;
    auto experts = gpu.zeros(10 * H), weights = gpu.zeros(10), shared = gpu.zeros(H);
    auto gate = gpu.upload(std::array<float, 1>{-1.4765625f}), out = gpu.zeros(H);
    const std::array<float, 10> values{0.00341796875f, 0.000698089599609375f, 0.037109375f, 0.034912109375f, -0.0081787109375f,
                                       0.007415771484375f, 0.01007080078125f, 0.0240478515625f, -0.045654296875f, 0.029296875f};
    const std::array<uint32_t, 10> bits{0x3e9c3eac, 0x3e0a4545, 0x3de27a41, 0x3da675fd, 0x3d91d03f, 0x3d8ff2e8, 0x3d6dd3d7, 0x3d68f8a1, 0x3d676896, 0x3d6159b8};
    for (size_t k = 0; k < 10; ++k) { experts->floats()[k * H] = values[k]; weights->floats()[k] = std::bit_cast<float>(bits[k]); }
    shared->floats()[0] = 0.0157470703125f;
    gpu.dispatch("moe_sum", {{experts}, {weights}, {shared}, {gate}, {out}}, {1}, H); gpu.finish();
    CHECK(out->floats()[0] == 0.01190185546875f);
    CHECK(std::all_of(out->floats().begin() + 1, out->floats().end(), [](float x) { return x == 0; }));
    CHECK_THROWS(gpu.dispatch("no_such_kernel", {{out}}, {1}, H));
}
static void test_direct_rows() {   // :1087-1099
    TEST("direct expert outputs preserve all destinations and reject aliasing");
    Metal gpu; const auto& s = gpu.shape(); const uint32_t H = s.hidden, I = s.inter, TopK = s.topk;
    auto record = to_hbm(gpu, expert_fixture(s, 1)); auto input = gpu.zeros(I);
    for (size_t i = 0; i < input->floats().size(); ++i) input->floats()[i] = float(int(i % 23) - 11) / 32;
    auto reference = gpu.linear(expert_linear(s, record, 2), input, 1);
    auto out = gpu.zeros((TopK + 2) * H); std::fill(out->floats().begin(), out->floats().end(), -17.0f);
    for (uint32_t pos = 0; pos < TopK; ++pos) gpu.linear_into(expert_linear(s, record, 2), input, 1, {out, (pos + 1) * H * 4ull});
    gpu.finish();
    for (uint32_t pos = 0; pos < TopK; ++pos) CHECK(std::memcmp(out->data + (pos + 1) * H * 4, reference->data, H * 4) == 0);
    for (uint32_t i = 0; i < H; ++i) { CHECK(out->floats()[i] == -17); CHECK(out->floats()[(TopK + 1) * H + i] == -17); }
    CHECK_THROWS(gpu.linear_into(expert_linear(s, record, 2), input, 1, {out, 1}));
    CHECK_THROWS(gpu.linear_into(expert_linear(s, record, 2), input, 1, {out, out->bytes - 4}));
    CHECK_THROWS(gpu.linear_into(expert_linear(s, record, 2), input, 1, {record}));
}
static void test_grouped() {   // :1188-1208
    TEST("grouped experts keep exact arithmetic and original router positions");
    Metal gpu; const auto& s = gpu.shape(); const uint32_t H = s.hidden, I = s.inter, TopK = s.topk;
    std::vector<Buf> records, reference; auto input = gpu.zeros(H);
    for (size_t i = 0; i < input->floats().size(); ++i) input->floats()[i] = float(int(i % 17) - 8) / 64;
    for (uint32_t i = 0; i < 8; ++i) {
        records.push_back(to_hbm(gpu, expert_fixture(s, i + 1)));
        auto gate = gpu.gated_linear(expert_linear(s, records.back(), 0), expert_linear(s, records.back(), 1), input, 1);
        reference.push_back(gpu.linear(expert_linear(s, records.back(), 2), gate, 1));
    }
    gpu.finish(); const std::array<uint32_t, 8> positions = {9, 1, 7, 3, 5, 0, 8, 4};
    for (size_t n : {1u, 2u, 3u, 4u, 7u, 8u}) {
        auto out = gpu.zeros(TopK * H), scratch = gpu.zeros(8 * I);
        std::fill(out->floats().begin(), out->floats().end(), -19.0f);
        gpu.grouped_experts(std::span(records).first(n), std::span(positions).first(n), input, out, scratch); gpu.finish();
        for (size_t i = 0; i < n; ++i) CHECK(std::memcmp(out->data + positions[i] * H * 4, reference[i]->data, H * 4) == 0);
        for (uint32_t p = 0; p < TopK; ++p) if (std::find(positions.begin(), positions.begin() + n, p) == positions.begin() + n)
            CHECK(std::all_of(out->floats().begin() + p * H, out->floats().begin() + (p + 1) * H, [](float v) { return v == -19; }));
        const std::array<uint32_t, 2> duplicate = {1, 1};
        CHECK_THROWS(gpu.grouped_experts(std::span(records).first(2), duplicate, input, out, scratch));
    }
}
static void test_heavy_rows() {   // :1500-1533
    TEST("heavy expert rows exercise microbatch scatter with distinct projections");
    Metal gpu; const auto& s = gpu.shape(); const uint32_t H = s.hidden, TopK = s.topk; constexpr uint32_t T = 513;
    auto record = to_hbm(gpu, expert_fixture(s, 19)); auto input = gpu.zeros(uint64_t(T) * H);
    for (size_t i = 0; i < input->floats().size(); ++i) input->floats()[i] = round_bf16(float(int((i * 7 + i / H) % 31) - 15) / 128);
    std::vector<Buf> reference; reference.reserve(T);
    for (uint32_t t = 0; t < T; ++t) {
        auto row = gpu.slice(input, uint64_t(t) * H * 4, H * 4);
        auto gate = gpu.gated_linear(expert_linear(s, record, 0), expert_linear(s, record, 1), row, 1);
        reference.push_back(gpu.linear(expert_linear(s, record, 2), gate, 1));
        if (t % 32 == 31) gpu.finish();
    }
    gpu.finish();
    auto out = gpu.zeros((uint64_t(T) * TopK + 1) * H), expected = gpu.zeros(uint64_t(T) * TopK * H);
    auto weights = gpu.zeros(uint64_t(T) * TopK), shared = gpu.zeros(uint64_t(T) * H), gate = gpu.zeros(T);
    for (auto& w : weights->floats()) w = 0.125f;
    for (bool reference_kernels : {false, true}) for (uint32_t count : {127u, 128u, 129u, 257u, 513u}) {
        KernelConfig config; if (reference_kernels) config.policy = "reference"; gpu.configure(config);
        std::memset(out->data, 0, out->bytes); std::memset(expected->data, 0, expected->bytes);
        std::memset(out->data + expected->bytes, 0xa5, H * 4);
        std::vector<int> positions;
        for (uint32_t i = 0; i < count; ++i) {
            const auto t = (i * 31) % T, p = t * TopK + (i % 9 + 1); positions.push_back(int(p));
            std::memcpy(expected->data + uint64_t(p) * H * 4, reference[t]->data, H * 4);
        }
        encode_expert_rows(gpu, record, input, out, positions, T, 128, false, 3, 4096);
        gpu.finish(); CHECK(std::memcmp(out->data, expected->data, expected->bytes) == 0);
        CHECK(std::all_of(out->data + expected->bytes, out->data + out->bytes, [](auto b) { return b == std::byte{0xa5}; }));
        auto sum = gpu.zeros(uint64_t(T) * H), want = gpu.zeros(uint64_t(T) * H);
        gpu.dispatch("moe_sum", {{out}, {weights}, {shared}, {gate}, {sum}}, {T}, H, T);
        gpu.dispatch("moe_sum", {{expected}, {weights}, {shared}, {gate}, {want}}, {T}, H, T); gpu.finish();
        CHECK(std::memcmp(sum->data, want->data, sum->bytes) == 0);
    }
    const std::array<int, 1> bad = {int(T * TopK)};
    CHECK_THROWS(encode_expert_rows(gpu, record, input, out, bad, T, 128, false, 0, 0));
}
static void test_moe_layer() {   // model.cpp:431-557 against the CPU oracle
    TEST("moe(): reference orchestration and device-resident orchestration equal the CPU oracle");
    const MoeShape s = small_shape(); Metal gpu(s); const auto oc = oracle_config(s);
    const uint64_t stride = (s.expert_bytes() + 255) / 256 * 256;
    std::vector<std::byte> all(stride * s.experts);
    for (uint32_t e = 0; e < s.experts; ++e) { auto r = expert_fixture(s, 100 + e); std::memcpy(all.data() + e * stride, r.data(), r.size()); }
    auto shared_host = expert_fixture(s, 7, true);
    auto records = to_hbm(gpu, all); auto shared_record = to_hbm(gpu, shared_host);
    std::vector<uint16_t> router(size_t(s.experts) * s.hidden), sgate(s.hidden);
    for (size_t i = 0; i < router.size(); ++i) router[i] = uint16_t(std::bit_cast<uint32_t>(round_bf16(float(int((i * 2654435761u >> 7) % 401) - 200) / 4096)) >> 16);
    for (size_t i = 0; i < sgate.size(); ++i) sgate[i] = uint16_t(std::bit_cast<uint32_t>(round_bf16(float(int(i % 37) - 18) / 512)) >> 16);
    auto router_buf = gpu.allocate(router.size() * 2, AllocationClass::Resident), sgate_buf = gpu.allocate(sgate.size() * 2, AllocationClass::Resident);
    gpu.write(router_buf, 0, std::as_bytes(std::span(router))); gpu.write(sgate_buf, 0, std::as_bytes(std::span(sgate)));
    MoeLayerWeights w;
    w.router = Linear{{router_buf}, {}, {}, s.hidden, s.experts, 64, 0, false};
    w.shared_gate = Linear{{sgate_buf}, {}, {}, s.hidden, 1, 64, 0, false};
    w.shared_record = shared_record;
    w.record = [&](uint32_t e) { return gpu.slice(records, e * stride, s.expert_bytes()); };
    for (uint32_t T : {1u, 5u, 33u}) {
        auto x = gpu.zeros(uint64_t(T) * s.hidden);
        for (size_t i = 0; i < x->floats().size(); ++i) x->floats()[i] = round_bf16(float(int((i * 40503u >> 3) % 255) - 127) / 64);
        auto a = moe(gpu, w, x, T); gpu.finish();
        auto b = moe_resident(gpu, w, records, stride, x, T);
        std::vector<float> want(size_t(T) * s.hidden);
        zco_layer_t layer{router.data(), nullptr, sgate.data(), reinterpret_cast<const uint8_t*>(shared_host.data()),
                          reinterpret_cast<const uint8_t*>(all.data()), stride};
        CHECK(zco_moe_layer(&oc, &layer, x->floats().data(), T, want.data(), nullptr, 4) == 0);
        CHECK(std::memcmp(a->data, want.data(), a->bytes) == 0);
        CHECK(std::memcmp(b->data, want.data(), b->bytes) == 0);
    }
    std::atomic<bool> cancel{true};
    auto x = gpu.zeros(s.hidden);
    CHECK_THROWS(moe(gpu, w, x, 1, &cancel));   // "generation cancelled"
    std::fill(x->floats().begin(), x->floats().end(), NAN);
    CHECK_THROWS(moe(gpu, w, x, 1));            // "invalid router output", model.cpp:459
    CHECK_THROWS(moe_resident(gpu, w, records, stride, x, 1));
    gpu.budget(gpu.allocated() + 16); CHECK_THROWS(gpu.allocate(1 << 20)); gpu.budget(0);   // "engine memory budget exceeded"
    // Metal::label + KernelConfig::profile (metal.mm:267-270): the layer's calls appear under the stages that moe() names
    KernelConfig profiled; profiled.profile = true; gpu.configure(profiled);
    std::fill(x->floats().begin(), x->floats().end(), 0.25f);
    (void)moe(gpu, w, x, 1); gpu.finish();
    const std::string stats = gpu.statistics();
    CHECK(stats.find("\"stage\": \"routed_expert\"") != std::string::npos && stats.find("\"operator\": \"gated_linear\"") != std::string::npos);
    CHECK(stats.find("\"recording\": true") != std::string::npos && stats.find("\"rows_dropped\": 0") != std::string::npos);
    gpu.configure(KernelConfig{});
    CHECK(gpu.statistics().find("\"recording\": false") != std::string::npos);
}
static void test_expert_cache() {   // :336-348 on the GPU, and moe() reading its records through leases
    TEST("expert cache: leases pin HBM slots; a layer through a few slots equals the resident layer");
    const MoeShape s = small_shape(); Metal gpu(s);
    ExpertCache cache(gpu, 1, s.topk + 2);
    const uint64_t stride = (s.expert_bytes() + 255) / 256 * 256;
    std::vector<std::byte> all(stride * s.experts);
    // the records travel through a prepared directory on disk, as they would from the reference's prepare step
    const auto dir = std::filesystem::temp_directory_path() / ("zc_engine_prepared_" + std::to_string(::getpid()));
    write_prepared_experts(dir, s, 1, [&](ExpertKey k, std::span<std::byte> into) { auto r = expert_fixture(s, 300 + k.expert); std::memcpy(into.data(), r.data(), r.size()); });
    {
        PreparedExperts prepared(dir, s);
        prepared.layer(0, all, stride);                                           // an HBM layer array's layout
        for (uint32_t e = 0; e < s.experts; ++e) prepared.expert({0, e}, cache.home({0, e}));   // the pinned home of the slot cache
        auto r = expert_fixture(s, 300 + 5);
        CHECK(std::memcmp(all.data() + 5 * stride, r.data(), r.size()) == 0 && std::memcmp(cache.home({0, 5}).data(), r.data(), r.size()) == 0);
    }
    std::filesystem::remove_all(dir);
    {
        std::vector<ExpertCache::Lease> leases;
        for (uint32_t e = 0; e < s.topk + 2; ++e) leases.push_back(cache.acquire({0, e}));
        CHECK_THROWS(cache.acquire({0, s.topk + 2}));   // "expert cache exhausted by outstanding leases; ..."
        CHECK_THROWS(cache.clear()); CHECK_THROWS(cache.resize(64));
        CHECK(std::string(leases[0].acquisition()) == "new_miss");
        auto again = cache.acquire({0, 0});
        CHECK(std::string(again.acquisition()) != "new_miss"); CHECK(again.wait()->metal == leases[0].wait()->metal);
        CHECK((leases[3].key() == ExpertKey{0, 3}));
    }
    CHECK_THROWS(cache.acquire({0, s.experts})); CHECK_THROWS(cache.acquire({1, 0}));
    auto shared_host = expert_fixture(s, 7, true);
    auto records = to_hbm(gpu, all); auto shared_record = to_hbm(gpu, shared_host);
    std::vector<uint16_t> router(size_t(s.experts) * s.hidden), sgate(s.hidden);
    for (size_t i = 0; i < router.size(); ++i) router[i] = uint16_t(std::bit_cast<uint32_t>(round_bf16(float(int((i * 2246822519u >> 9) % 401) - 200) / 4096)) >> 16);
    for (size_t i = 0; i < sgate.size(); ++i) sgate[i] = uint16_t(std::bit_cast<uint32_t>(round_bf16(float(int(i % 29) - 14) / 512)) >> 16);
    auto router_buf = gpu.allocate(router.size() * 2, AllocationClass::Resident), sgate_buf = gpu.allocate(sgate.size() * 2, AllocationClass::Resident);
    gpu.write(router_buf, 0, std::as_bytes(std::span(router))); gpu.write(sgate_buf, 0, std::as_bytes(std::span(sgate)));
    MoeLayerWeights w;
    w.router = Linear{{router_buf}, {}, {}, s.hidden, s.experts, 64, 0, false};
    w.shared_gate = Linear{{sgate_buf}, {}, {}, s.hidden, 1, 64, 0, false};
    w.shared_record = shared_record;
    std::vector<ExpertCache::Lease> held;      // pinned until the layer's GPU work has finished
    w.record = [&](uint32_t e) { held.push_back(cache.acquire({0, e})); return held.back().wait(); };
    for (uint32_t step = 0; step < 6; ++step) {
        auto x = gpu.zeros(s.hidden);
        for (size_t i = 0; i < x->floats().size(); ++i) x->floats()[i] = round_bf16(float(int(((i * 40503u + step * 977u) >> 3) % 255) - 127) / 64);
        auto a = moe(gpu, w, x, 1); gpu.finish(); held.clear();
        auto b = moe_resident(gpu, w, records, stride, x, 1);
        CHECK(std::memcmp(a->data, b->data, a->bytes) == 0);
    }
    const auto st = cache.stats();
    CHECK(st.misses >= s.topk); CHECK(st.hits + st.misses >= 6 * s.topk); CHECK(st.bytes == st.misses * s.expert_bytes());
    cache.clear(); CHECK(cache.occupancy() == 0);
    // next-layer prediction (model.cpp:437-445, 489-500): here the "next layer" has this layer's router and sees the
    // same input, so every guess is exactly what the following call demands: all of them were prefetched and none misses
    w.next_router = w.router; w.prefetch_depth = s.topk;
    w.prefetch = [&](uint32_t e) { return cache.prefetch({0, e}); };
    {
        auto x = gpu.zeros(s.hidden);
        for (size_t i = 0; i < x->floats().size(); ++i) x->floats()[i] = round_bf16(float(int((i * 2654435761u >> 7) % 255) - 127) / 64);
        const auto before = cache.stats();
        PredictionStats guess;
        auto first = moe(gpu, w, x, 1, nullptr, 128, x, &guess); gpu.finish(); held.clear();
        CHECK(guess.guesses == s.topk && guess.experts.size() == s.topk);
        const auto mid = cache.stats();
        CHECK(mid.prefetches - before.prefetches == guess.issued);        // already-resident guesses are not issued again
        auto second = moe(gpu, w, x, 1); gpu.finish(); held.clear();      // demands exactly the guessed experts
        const auto after = cache.stats();
        CHECK(after.misses == mid.misses);
        CHECK(std::memcmp(first->data, second->data, first->bytes) == 0);  // the hint never changes the arithmetic
        auto plain = moe_resident(gpu, w, records, stride, x, 1);
        CHECK(std::memcmp(first->data, plain->data, first->bytes) == 0);
        w.prefetch_depth = 3; PredictionStats shallow; cache.clear();
        moe(gpu, w, x, 1, nullptr, 128, x, &shallow); gpu.finish(); held.clear();
        CHECK(shallow.guesses == s.topk && shallow.issued <= 3);
    }
}
static void test_glue() {   // :53, :876-897, :1137-1145 and the glue of model.cpp:328-351, 651
    TEST("element-wise dispatches, the stream mix / injection and the grouped norm");
    Metal gpu; const uint32_t H = gpu.shape().hidden;
    auto x = gpu.zeros(32), y = gpu.zeros(32);
    for (int i = 0; i < 32; ++i) x->floats()[i] = round_bf16(float(i - 16) / 8);
    gpu.dispatch("binary", {{x}, {x}, {y}}, {32, 0}, 32); gpu.finish();
    for (int i = 0; i < 32; ++i) CHECK(y->floats()[i] == 2 * x->floats()[i]);
    auto edge = gpu.zeros(2), out = gpu.zeros(2); edge->floats()[0] = -6.84375f; edge->floats()[1] = 6.84375f;
    gpu.dispatch("unary", {{edge}, {out}}, {2, 0}, 2); gpu.finish();
    CHECK(out->floats()[0] == -0.00726318359375f); CHECK(out->floats()[1] == 6.84375f);   // the captured exp rounding boundary
    gpu.dispatch("unary", {{edge}, {out}}, {2, 4}, 2); gpu.finish();
    CHECK(out->floats()[1] == 6.84375f && out->floats()[0] > 0 && out->floats()[0] < 0.0011f);
    CHECK_THROWS(gpu.dispatch("unary", {{edge}, {out}}, {2, 9}, 2));
    CHECK_THROWS(gpu.dispatch("binary", {{edge}, {x}, {out}}, {32, 0}, 32));
    // four streams: mixing with unit weights averages them, injecting with zero leaves the streams alone
    const uint32_t T = 2;
    auto streams = gpu.zeros(uint64_t(T) * 4 * H), ones = gpu.zeros(uint64_t(T) * 4 * H), mixed = gpu.zeros(uint64_t(T) * H);
    for (size_t i = 0; i < streams->floats().size(); ++i) { streams->floats()[i] = round_bf16(float(int(i % 23) - 11) / 16); ones->floats()[i] = 1; }
    gpu.dispatch("hc_mix", {{streams}, {ones}, {mixed}}, {T}, H, T); gpu.finish();
    for (uint32_t t = 0; t < T; ++t) for (uint32_t d = 0; d < H; d += 97) {
        float sum = 0; for (uint32_t h = 0; h < 4; ++h) sum = round_bf16(sum + streams->floats()[(uint64_t(t) * 4 + h) * H + d]);
        CHECK(mixed->floats()[uint64_t(t) * H + d] == round_bf16(sum / 4));
    }
    auto inject = gpu.zeros(T * 4), after = gpu.zeros(uint64_t(T) * 4 * H);
    gpu.dispatch("hc_add", {{streams}, {mixed}, {inject}, {after}}, {T}, 4 * H, T); gpu.finish();
    CHECK(std::memcmp(after->data, streams->data, after->bytes) == 0);
    for (uint32_t i = 0; i < T * 4; ++i) inject->floats()[i] = float(i % 3) - 1;
    gpu.dispatch("hc_add", {{streams}, {mixed}, {inject}, {after}}, {T}, 4 * H, T); gpu.finish();
    CHECK(after->floats()[5 * H + 7] == round_bf16(streams->floats()[5 * H + 7] + round_bf16(mixed->floats()[H + 7] * inject->floats()[5])));
    // grouped RMS norm: both kernel names give the same bytes, also for a group that is not a multiple of 128
    for (auto [D, width, tokens] : std::array<std::tuple<uint32_t, uint32_t, uint32_t>, 3>{{{2560, 10240, 3}, {512, 1024, 2}, {320, 640, 1}}}) {
        auto in = gpu.zeros(uint64_t(width) * tokens), w = gpu.allocate(width * 2), a = gpu.allocate(in->bytes), b = gpu.allocate(in->bytes);
        for (size_t i = 0; i < in->floats().size(); ++i) in->floats()[i] = round_bf16(float(int(i * 7 % 61) - 30) / 10);
        for (uint32_t i = 0; i < width; ++i) reinterpret_cast<uint16_t*>(w->data)[i] = 0x3f80 + uint16_t(i % 5);
        const uint32_t threads = 32 * ((D + 127) / 128);
        gpu.dispatch("norm", {{in}, {w}, {a}}, {D, width, tokens, 0, 1}, tokens * (width / D) * 32);
        gpu.dispatch("norm_wide", {{in}, {w}, {b}}, {D, width, tokens, 0, 1}, tokens * (width / D) * threads, 1, 1, threads); gpu.finish();
        CHECK(std::memcmp(a->data, b->data, a->bytes) == 0);
        double ms = 0; for (uint32_t d = 0; d < D; ++d) ms += double(in->floats()[d]) * in->floats()[d];
        const double want = in->floats()[3] / std::sqrt(ms / D + 1e-6) * bf16(reinterpret_cast<uint16_t*>(w->data)[3]);
        CHECK(std::fabs(a->floats()[3] - want) <= std::fabs(want) / 64);
    }
    CHECK_THROWS(gpu.dispatch("norm", {{x}, {x}, {y}}, {48, 100, 1, 0, 1}, 32));
}

static void test_route_replay() {   // model.cpp:274-283, 447-448: dumped logits replayed against dumped ids
    TEST("route dumps of another machine replay through route()");
    Metal gpu; const auto& s = gpu.shape(); const uint32_t T = 5;
    std::vector<float> logits(size_t(T) * s.experts); std::vector<int> want(size_t(T) * s.topk);
    for (uint32_t t = 0; t < T; ++t) {
        for (uint32_t e = 0; e < s.experts; ++e) logits[size_t(t) * s.experts + e] = float(int((e * 37u + t * 101u) % 199) - 99) / 8;   // many exact ties
        std::vector<int> order(s.experts); std::iota(order.begin(), order.end(), 0);
        std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return logits[size_t(t) * s.experts + a] > logits[size_t(t) * s.experts + b]; });
        std::copy(order.begin(), order.begin() + s.topk, want.begin() + size_t(t) * s.topk);
    }
    const auto dir = std::filesystem::temp_directory_path() / ("zc_engine_dump_" + std::to_string(::getpid()));
    write_tensor_dump(dir, 40, "router_3", std::as_bytes(std::span(logits)));
    write_tensor_dump(dir, 40, "route_3", std::as_bytes(std::span(want)));
    CHECK(replay_route_dump(gpu, dir, 40, 3) == 0);
    std::swap(want[0], want[1]);
    write_tensor_dump(dir, 40, "route_3", std::as_bytes(std::span(want)));
    CHECK(replay_route_dump(gpu, dir, 40, 3) == 2);
    CHECK_THROWS(replay_route_dump(gpu, dir, 40, 4)); CHECK_THROWS(replay_route_dump(gpu, dir, 41, 3));
    write_tensor_dump(dir, 40, "route_3", std::as_bytes(std::span(want).first(7)));
    CHECK_THROWS(replay_route_dump(gpu, dir, 40, 3));
    std::filesystem::remove_all(dir);
}

int main() {
    test_route_replay(); test_glue(); test_bf16(); test_q4_matmul(); test_route(); test_moe_sum(); test_direct_rows(); test_grouped(); test_heavy_rows(); test_moe_layer(); test_expert_cache();
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
