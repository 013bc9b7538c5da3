// TEST HARNESS, not product code.  The two reference functions that sit ABOVE the drop-in boundary --
// encode_expert_rows (include/engine/pipeline.hpp:6-8, src/engine/pipeline.cpp:7-31) and the body of Model::moe
// (src/engine/model.cpp:431-557, without its cache, trace and timing branches) -- written against this repository's
// operator class, in the reference's order of operator calls.  An engine that swaps only the operator class keeps its own
// copies of these; the tests use them to drive the library the way that engine would, so that the reference's own tests of
// the path (tests/test_qwen.cpp:1087-1099, 1500-1600) can be restated call for call.  The library's own orchestration of
// the layer is zc_hip_moe_forward / zc_hip_stack_decode (moe_resident in engine.hpp), below the C ABI.
#pragma once
#include "../../zerocool_amd/csrc/engine/engine.hpp"
#include <algorithm>
#include <cstring>
#include <stdexcept>

namespace zerocool::engine {

struct PredictionStats { uint32_t guesses = 0, issued = 0; std::vector<int> experts; };

namespace harness {
inline Buf int_buffer(Metal& gpu, std::span<const int> values) {
    auto b = gpu.allocate(values.size_bytes());
    std::memcpy(b->data, values.data(), values.size_bytes());
    return b;
}
inline void stop_if(const std::atomic<bool>* cancel) { if (cancel && cancel->load()) throw std::runtime_error("generation cancelled"); }
}  // namespace harness

// pipeline.cpp:7-31: one expert's destination slots, `chunk` at a time: gate/up on the gathered rows, then either the down
// projection straight into the slot (one token) or down + scatter_experts.
inline void encode_expert_rows(Metal& gpu, const Buf& record, const Buf& input, const Buf& output, std::span<const int> positions,
                               uint32_t tokens, uint32_t chunk, bool direct, int layer, uint32_t offset,
                               const std::atomic<bool>* cancel = nullptr) {
    const MoeShape& s = gpu.shape();
    const uint64_t slots = uint64_t(tokens) * s.topk;
    const bool geometry_ok = chunk && chunk <= 256 && tokens && tokens <= 1024 && input && output &&
                             input->bytes >= uint64_t(tokens) * s.hidden * 4 && output->bytes >= slots * s.hidden * 4;
    if (!geometry_ok) throw std::invalid_argument("invalid expert row encoding geometry");
    if (std::any_of(positions.begin(), positions.end(), [&](int p) { return p < 0 || uint64_t(p) >= slots; }))
        throw std::invalid_argument("expert destination outside input");
    const bool into_slot = tokens == 1 && (direct || gpu.direct_rows());
    const Linear gate = expert_linear(s, record, 0), up = expert_linear(s, record, 1), down = expert_linear(s, record, 2);
    for (size_t first = 0; first < positions.size(); first += chunk) {
        harness::stop_if(cancel);
        const auto part = positions.subspan(first, std::min<size_t>(chunk, positions.size() - first));
        const uint32_t n = uint32_t(part.size());
        gpu.label("routed_expert", layer, n, offset);
        Buf gather;
        if (tokens != 1) {
            std::vector<int> rows(n);
            std::transform(part.begin(), part.end(), rows.begin(), [&](int p) { return p / int(s.topk); });
            gather = harness::int_buffer(gpu, rows);
        }
        const Buf activated = gpu.gated_linear(gate, up, input, n, gather);
        if (into_slot) { gpu.linear_into(down, activated, 1, {output, uint64_t(part[0]) * s.hidden * 4}); continue; }
        const Buf rows_out = gpu.linear(down, activated, n);
        gpu.dispatch("scatter_experts", {{rows_out}, {harness::int_buffer(gpu, part)}, {output}}, {n}, s.hidden, n);
    }
}

// model.cpp:431-557: router -> route -> (next layer's router on `predict`, model.cpp:437-445) -> ONE readback -> prefetch of
// the guesses (model.cpp:489-500) -> positions per expert (model.cpp:449-479) -> shared expert and gate (model.cpp:482-485)
// -> encode_expert_rows per selected expert in ascending id -> moe_sum (model.cpp:553-556).
inline Buf moe(Metal& gpu, const MoeLayerWeights& w, const Buf& x, uint32_t tokens, const std::atomic<bool>* cancel = nullptr,
               uint32_t chunk = 128, const Buf& predict = {}, PredictionStats* prediction = nullptr) {
    const MoeShape& s = gpu.shape();
    const uint64_t slots = uint64_t(tokens) * s.topk;
    const Buf logits = gpu.linear(w.router, x, tokens, true);
    const Buf ids = gpu.allocate(slots * 4), weights = gpu.allocate(slots * 4);
    gpu.route(logits, ids, weights, tokens);
    Buf guessed;
    if (predict && w.next_router.weight.buffer) {   // shares the readback below, never feeds the arithmetic
        if (predict->bytes < uint64_t(tokens) * s.hidden * 4) throw std::invalid_argument("invalid prediction input");
        guessed = gpu.allocate(slots * 4);
        gpu.route(gpu.linear(w.next_router, predict, tokens, true), guessed, gpu.allocate(slots * 4), tokens);
    }
    gpu.finish();
    harness::stop_if(cancel);
    if (guessed) {                                  // the first token's guesses, distinct, at most prefetch_depth issued
        PredictionStats scratch; PredictionStats& st = prediction ? *prediction : scratch;
        st = {};
        for (const int e : std::span<const int>(reinterpret_cast<const int*>(guessed->data), s.topk)) {
            if (e < 0 || e >= int(s.experts) || std::count(st.experts.begin(), st.experts.end(), e)) continue;
            const bool issued = st.experts.size() < w.prefetch_depth && w.prefetch && w.prefetch(uint32_t(e));
            st.experts.push_back(e);
            ++st.guesses;
            st.issued += issued;
        }
    }
    std::vector<std::vector<int>> positions(s.experts);
    const auto chosen = std::span<const int>(reinterpret_cast<const int*>(ids->data), size_t(slots));
    for (size_t p = 0; p < chosen.size(); ++p) {
        if (chosen[p] < 0 || chosen[p] >= int(s.experts)) throw std::runtime_error("invalid router output");
        positions[size_t(chosen[p])].push_back(int(p));
    }
    const Buf expert_out = gpu.allocate(slots * s.hidden * 4);
    const Buf shared_act = gpu.gated_linear(expert_linear(s, w.shared_record, 0, true), expert_linear(s, w.shared_record, 1, true), x, tokens);
    const Buf shared = gpu.linear(expert_linear(s, w.shared_record, 2, true), shared_act, tokens);
    const Buf gate = gpu.linear(w.shared_gate, x, tokens);
    for (uint32_t e = 0; e < s.experts; ++e) {
        if (positions[e].empty()) continue;
        harness::stop_if(cancel);
        encode_expert_rows(gpu, w.record(e), x, expert_out, positions[e], tokens, chunk, true, 0, 0, cancel);
    }
    const Buf out = gpu.allocate(uint64_t(tokens) * s.hidden * 4);
    gpu.dispatch("moe_sum", {{expert_out}, {weights}, {shared}, {gate}, {out}}, {tokens}, s.hidden, tokens);
    return out;
}

}  // namespace zerocool::engine
