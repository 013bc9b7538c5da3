// Route traces and diagnostic tensor dumps in the reference's formats, so that routing captured on another machine can
// be replayed against this library:
//  * RouteTrace: the coordinator's JSON-lines capture "qwen_route_trace_v1" (include/engine/route_trace.hpp): one
//    object per line {kind, sequence, monotonic_ns, event, request_id, forward_id, details}; the selected experts of a
//    layer travel in a "routes" event.  Same call order rules and limits (20000 events, 64 KiB per line, 16 MiB).
//  * read_route_trace: parses such a file back into committed forwards.
//  * tensor dumps: Model::trace writes <dir>/step_<offset>/<name>.bin as raw bytes (model.cpp:274-283), e.g.
//    router_<layer>.bin (fp32 logits) and route_<layer>.bin (int32 ids); write_tensor_dump / read_tensor_dump do the
//    same, replay_route_dump runs the dumped logits through Metal::route and reports whether the dumped ids come out.
#pragma once
#include "records.hpp"
#include <chrono>
#include <cstring>
#include <cstdio>
#include <fcntl.h>
#include <unistd.h>

namespace zerocool::engine {

class RouteTrace {
public:
    RouteTrace(const std::filesystem::path& path, const std::string& identity_json, uint32_t layers, uint32_t topk) : layers_(layers), topk_(topk) {
        Json::parse(identity_json);   // must be valid JSON: it is embedded verbatim
        const int fd = ::open(path.c_str(), O_WRONLY | O_CREAT | O_EXCL | O_CLOEXEC, 0600);
        if (fd < 0) throw std::runtime_error("route trace must be a new file: " + path.string());
        stream_ = ::fdopen(fd, "w");
        if (!stream_) { ::close(fd); throw std::runtime_error("cannot open route trace"); }
        try { emit("trace_begin", "{\"identity\":" + identity_json + "}"); } catch (...) { std::fclose(stream_); stream_ = nullptr; throw; }
    }
    RouteTrace(const RouteTrace&) = delete;
    ~RouteTrace() {
        if (stream_) {
            if (!terminal_) try { emit("trace_end", "{\"status\":\"incomplete\"}"); } catch (...) {}
            std::fclose(stream_);
        }
    }
    void request_begin(const std::string& name, std::span<const int> prompt, int max_tokens, bool prime) {
        if (request_ || forward_ || terminal_) throw std::logic_error("route request already active");
        request_ = true; ++request_id_;
        emit("request_begin", "{\"name\":" + quoted(name) + ",\"input_token_ids\":" + list(prompt) + ",\"max_tokens\":" + std::to_string(max_tokens) + ",\"prime\":" + (prime ? "true" : "false") + "}");
    }
    void request_end(std::span<const int> output, const std::string& reason, uint64_t reused) {
        if (!request_ || forward_ || terminal_) throw std::logic_error("route request not complete");
        emit("request_end", "{\"output_token_ids\":" + list(output) + ",\"finish_reason\":" + quoted(reason) + ",\"reused_tokens\":" + std::to_string(reused) + "}");
        request_ = false;
    }
    void begin(uint64_t session, uint32_t offset, std::span<const int> input, const std::string& phase, size_t slots) {
        if (!request_ || forward_ || terminal_ || input.empty() || offset + input.size() > 8192 || !session) throw std::logic_error("invalid route forward start");
        forward_ = true; ++forward_id_; next_layer_ = 0; offset_ = offset; tokens_ = uint32_t(input.size());
        emit("forward_begin", "{\"session_id\":" + quoted(std::to_string(session)) + ",\"offset\":" + std::to_string(offset) + ",\"tokens\":" + std::to_string(tokens_) +
                                  ",\"input_token_ids\":" + list(input) + ",\"request_phase\":" + quoted(phase) + ",\"expert_slots\":" + std::to_string(slots) + "}");
    }
    void routes(int layer, uint32_t offset, uint32_t tokens, std::span<const int> selected) {
        if (!forward_ || terminal_ || layer != next_layer_ || layer >= int(layers_) || offset != offset_ || tokens != tokens_ || selected.size() != size_t(tokens) * topk_)
            throw std::logic_error("route pass does not match active forward");
        emit("routes", "{\"layer\":" + std::to_string(layer) + ",\"routes\":" + list(selected) + "}"); ++next_layer_;
    }
    void commit(uint32_t position) {
        if (!forward_ || terminal_ || next_layer_ != int(layers_) || position != offset_ + tokens_) throw std::logic_error("route forward did not complete all layers");
        emit("forward_commit", "{\"position\":" + std::to_string(position) + "}"); forward_ = false;
    }
    void abort() { if (forward_ && !terminal_) { emit("forward_abort", "{\"captured_layers\":" + std::to_string(next_layer_) + "}"); forward_ = false; } }
    void cache_reset() { emit("cache_reset", "{}"); }
    void finish() {
        if (request_ || forward_ || terminal_) throw std::logic_error("route trace is incomplete");
        emit("trace_end", "{\"status\":\"complete\"}"); terminal_ = true;
    }
private:
    static std::string quoted(const std::string& s) {
        std::string out = "\"";
        for (unsigned char c : s) {
            if (c == '"' || c == '\\') { out += '\\'; out += char(c); }
            else if (c < 0x20) { char b[8]; std::snprintf(b, sizeof b, "\\u%04x", c); out += b; }
            else out += char(c);
        }
        return out + "\"";
    }
    static std::string list(std::span<const int> v) { std::string out = "["; for (size_t i = 0; i < v.size(); ++i) { if (i) out += ','; out += std::to_string(v[i]); } return out + "]"; }
    void emit(const char* event, const std::string& details) {
        if (sequence_ >= 20000) throw std::runtime_error("route trace event limit exceeded");
        const auto now = std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
        const std::string line = "{\"details\":" + details + ",\"event\":\"" + event + "\",\"forward_id\":" + std::to_string(forward_id_) + ",\"kind\":\"qwen_route_trace_v1\",\"monotonic_ns\":" +
                                 std::to_string(now) + ",\"request_id\":" + std::to_string(request_id_) + ",\"sequence\":" + std::to_string(sequence_ + 1) + "}\n";
        if (line.size() > 65536 || bytes_ + line.size() > (16u << 20)) throw std::runtime_error("route trace byte limit exceeded");
        if (std::fwrite(line.data(), 1, line.size(), stream_) != line.size() || std::fflush(stream_)) throw std::runtime_error("cannot flush route trace");
        ++sequence_; bytes_ += line.size();
    }
    std::FILE* stream_ = nullptr;
    uint64_t sequence_ = 0, bytes_ = 0, request_id_ = 0, forward_id_ = 0;
    uint32_t offset_ = 0, tokens_ = 0, layers_, topk_;
    int next_layer_ = 0;
    bool request_ = false, forward_ = false, terminal_ = false;
};

struct TracedForward {
    uint64_t request_id = 0, forward_id = 0;
    uint32_t offset = 0, tokens = 0;
    std::string phase;
    std::vector<std::vector<int>> routes;   // [layer][tokens * topk]
    bool committed = false;
};
struct TraceSummary { std::vector<TracedForward> forwards; bool complete = false; uint64_t events = 0; };
// Reads a route trace: every line must carry kind "qwen_route_trace_v1" and consecutive sequence numbers from 1.
inline TraceSummary read_route_trace(const std::filesystem::path& path) {
    std::FILE* f = std::fopen(path.c_str(), "r");
    if (!f) throw std::runtime_error("cannot read route trace: " + path.string());
    TraceSummary out; std::string line; int c;
    auto take = [&](const std::string& text) {
        const Json j = Json::parse(text);
        if (j.at("kind").str() != "qwen_route_trace_v1" || j.at("sequence").u64() != out.events + 1) throw std::runtime_error("route trace line out of sequence");
        ++out.events;
        const std::string& event = j.at("event").str(); const Json& d = j.at("details");
        if (event == "forward_begin") {
            TracedForward fw; fw.request_id = j.at("request_id").u64(); fw.forward_id = j.at("forward_id").u64();
            fw.offset = uint32_t(d.at("offset").u64()); fw.tokens = uint32_t(d.at("tokens").u64()); fw.phase = d.at("request_phase").str();
            out.forwards.push_back(std::move(fw));
        } else if (event == "routes") {
            if (out.forwards.empty() || d.at("layer").u64() != out.forwards.back().routes.size()) throw std::runtime_error("route pass does not match active forward");
            std::vector<int> ids; for (size_t i = 0; i < d.at("routes").size(); ++i) ids.push_back(int(std::get<double>(d.at("routes").at(i).value)));
            out.forwards.back().routes.push_back(std::move(ids));
        } else if (event == "forward_commit") { if (out.forwards.empty()) throw std::runtime_error("commit without a forward"); out.forwards.back().committed = true; }
        else if (event == "trace_end") out.complete = d.at("status").str() == "complete";
    };
    try {
        while ((c = std::fgetc(f)) != EOF) { if (c == '\n') { if (!line.empty()) take(line); line.clear(); } else line += char(c); }
        if (!line.empty()) take(line);
    } catch (...) { std::fclose(f); throw; }
    std::fclose(f);
    return out;
}

// model.cpp:274-283: <dir>/step_<offset>/<name>.bin, raw bytes
inline void write_tensor_dump(const std::filesystem::path& dir, uint32_t offset, const std::string& name, std::span<const std::byte> bytes) {
    const auto step = dir / ("step_" + std::to_string(offset));
    std::filesystem::create_directories(step);
    std::FILE* f = std::fopen((step / (name + ".bin")).c_str(), "wb");
    if (!f || std::fwrite(bytes.data(), 1, bytes.size(), f) != bytes.size() || std::fclose(f)) throw std::runtime_error("cannot write diagnostic tensor: " + name);
}
inline std::vector<std::byte> read_tensor_dump(const std::filesystem::path& dir, uint32_t offset, const std::string& name) {
    const auto path = dir / ("step_" + std::to_string(offset)) / (name + ".bin");
    std::FILE* f = std::fopen(path.c_str(), "rb");
    if (!f) throw std::runtime_error("missing diagnostic tensor: " + path.string());
    std::vector<std::byte> out(std::filesystem::file_size(path));
    const bool ok = std::fread(out.data(), 1, out.size(), f) == out.size(); std::fclose(f);
    if (!ok) throw std::runtime_error("short diagnostic tensor: " + path.string());
    return out;
}
// Runs the logits of router_<layer>.bin through Metal::route and compares the ids with route_<layer>.bin:
// the number of (token, rank) positions that differ (0 = the routing of the other machine is reproduced).
inline size_t replay_route_dump(Metal& gpu, const std::filesystem::path& dir, uint32_t offset, int layer) {
    const auto& s = gpu.shape();
    const auto logits = read_tensor_dump(dir, offset, "router_" + std::to_string(layer)), want = read_tensor_dump(dir, offset, "route_" + std::to_string(layer));
    if (logits.empty() || logits.size() % (uint64_t(s.experts) * 4) || want.size() != logits.size() / (uint64_t(s.experts) * 4) * s.topk * 4)
        throw std::invalid_argument("route dump does not match the model shape");
    const uint32_t tokens = uint32_t(logits.size() / (uint64_t(s.experts) * 4));
    auto in = gpu.allocate(logits.size()), ids = gpu.allocate(want.size()), weights = gpu.allocate(want.size());
    std::memcpy(in->data, logits.data(), logits.size());
    gpu.route(in, ids, weights, tokens); gpu.finish();
    size_t differing = 0;
    for (size_t i = 0; i < want.size() / 4; ++i) differing += reinterpret_cast<const int*>(ids->data)[i] != reinterpret_cast<const int*>(want.data())[i];
    return differing;
}

}  // namespace zerocool::engine
