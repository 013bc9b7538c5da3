// Route traces and diagnostic tensor dumps in the reference's formats, so that routing captured on another machine can
// be replayed against this library:
//  * RouteTrace: the coordinator's JSON-lines capture "qwen_route_trace_v1" (include/engine/route_trace.hpp): one
//    object per line {kind, sequence, monotonic_ns, event, request_id, forward_id, details}; the selected experts of a
//    layer travel in a "routes" event.  The format's nesting rules and limits (20000 events, 64 KiB per line, 16 MiB) hold.
//  * read_route_trace: parses such a file back into committed forwards.
//  * tensor dumps: Model::trace writes <dir>/step_<offset>/<name>.bin as raw bytes (model.cpp:274-283), e.g.
//    router_<layer>.bin (fp32 logits) and route_<layer>.bin (int32 ids); write_tensor_dump / read_tensor_dump do the
//    same, replay_route_dump runs the dumped logits through Metal::route and reports whether the dumped ids come out.
#pragma once
#include "records.hpp"
#include <chrono>
#include <cstring>
#include <cstdio>

namespace zerocool::engine {

// Writer of the capture format.  A capture is a strict nesting: trace { request { forward { routes x layers } } },
// which is kept here as one explicit stage plus the geometry of the forward that is open.  Every event goes through
// one serializer (Event), which owns the envelope fields, the limits and the flush.
class RouteTrace {
    enum class Stage { Idle, Request, Forward, Closed };
    // One line of the capture: details are appended field by field, the envelope is added when the line is written.
    class Event {
    public:
        explicit Event(const char* name) : name_(name) {}
        Event& number(const char* key, uint64_t v) { field(key) += std::to_string(v); return *this; }
        Event& flag(const char* key, bool v) { field(key) += v ? "true" : "false"; return *this; }
        Event& raw(const char* key, const std::string& json) { field(key) += json; return *this; }
        Event& text(const char* key, const std::string& v) {
            std::string& out = field(key);
            out += '"';
            for (const unsigned char c : v) {
                if (c == '"' || c == '\\') { out += '\\'; out += char(c); }
                else if (c < 0x20) { char b[8]; std::snprintf(b, sizeof b, "\\u%04x", c); out += b; }
                else out += char(c);
            }
            out += '"';
            return *this;
        }
        Event& integers(const char* key, std::span<const int> v) {
            std::string& out = field(key);
            out += '[';
            for (size_t i = 0; i < v.size(); ++i) { if (i) out += ','; out += std::to_string(v[i]); }
            out += ']';
            return *this;
        }
        const char* name() const { return name_; }
        std::string details() const { return "{" + body_ + "}"; }
    private:
        std::string& field(const char* key) { if (!body_.empty()) body_ += ','; body_ += '"'; body_ += key; body_ += "\":"; return body_; }
        const char* name_; std::string body_;
    };
    static constexpr uint64_t kMaxEvents = 20000, kMaxLine = 64u << 10, kMaxBytes = 16u << 20, kMaxContext = 8192;

public:
    RouteTrace(const std::filesystem::path& path, const std::string& identity_json, uint32_t layers, uint32_t topk) : layers_(layers), topk_(topk) {
        Json::parse(identity_json);   // embedded as it is, so it has to parse
        file_ = std::fopen(path.c_str(), "wx");   // exclusive: a capture never continues or replaces another file
        if (!file_) throw std::runtime_error("route trace must be a new file: " + path.string());
        try { write(Event("trace_begin").raw("identity", identity_json)); }
        catch (...) { std::fclose(file_); file_ = nullptr; throw; }
    }
    RouteTrace(const RouteTrace&) = delete;
    RouteTrace& operator=(const RouteTrace&) = delete;
    ~RouteTrace() {
        if (!file_) return;
        if (stage_ != Stage::Closed) { try { write(Event("trace_end").text("status", "incomplete")); } catch (...) {} }
        std::fclose(file_);
    }
    void request_begin(const std::string& name, std::span<const int> prompt, int max_tokens, bool prime) {
        expect(Stage::Idle, "a route request is already open");
        ++request_id_; stage_ = Stage::Request;
        write(Event("request_begin").text("name", name).integers("input_token_ids", prompt).raw("max_tokens", std::to_string(max_tokens)).flag("prime", prime));
    }
    void request_end(std::span<const int> output, const std::string& reason, uint64_t reused) {
        expect(Stage::Request, "no route request to end, or a forward is still open");
        write(Event("request_end").integers("output_token_ids", output).text("finish_reason", reason).number("reused_tokens", reused));
        stage_ = Stage::Idle;
    }
    void begin(uint64_t session, uint32_t offset, std::span<const int> input, const std::string& phase, size_t slots) {
        expect(Stage::Request, "a forward needs an open request and no other forward");
        if (!session || input.empty() || uint64_t(offset) + input.size() > kMaxContext) throw std::logic_error("route forward outside the context window");
        ++forward_id_; stage_ = Stage::Forward; open_ = Forward{offset, uint32_t(input.size()), 0};
        write(Event("forward_begin").text("session_id", std::to_string(session)).number("offset", offset).number("tokens", open_.tokens)
                  .integers("input_token_ids", input).text("request_phase", phase).number("expert_slots", slots));
    }
    void routes(int layer, uint32_t offset, uint32_t tokens, std::span<const int> selected) {
        expect(Stage::Forward, "routes outside a forward");
        const bool in_turn = layer >= 0 && uint32_t(layer) == open_.layers_seen && open_.layers_seen < layers_;
        if (!in_turn || offset != open_.offset || tokens != open_.tokens || selected.size() != size_t(tokens) * topk_)
            throw std::logic_error("routes do not belong to the open forward");
        write(Event("routes").number("layer", uint64_t(layer)).integers("routes", selected));
        ++open_.layers_seen;
    }
    void commit(uint32_t position) {
        expect(Stage::Forward, "commit outside a forward");
        if (open_.layers_seen != layers_ || position != open_.offset + open_.tokens) throw std::logic_error("the forward has not routed every layer");
        write(Event("forward_commit").number("position", position));
        stage_ = Stage::Request;
    }
    void abort() {   // a forward given up half way; harmless when none is open
        if (stage_ != Stage::Forward) return;
        write(Event("forward_abort").number("captured_layers", open_.layers_seen));
        stage_ = Stage::Request;
    }
    void cache_reset() { write(Event("cache_reset")); }
    void finish() {
        expect(Stage::Idle, "the route trace still has an open request");
        write(Event("trace_end").text("status", "complete"));
        stage_ = Stage::Closed;
    }

private:
    struct Forward { uint32_t offset = 0, tokens = 0, layers_seen = 0; };
    void expect(Stage wanted, const char* otherwise) const { if (stage_ != wanted) throw std::logic_error(otherwise); }
    void write(const Event& e) {
        if (written_ >= kMaxEvents) throw std::runtime_error("route trace holds its 20000 events");
        const auto now = std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now().time_since_epoch()).count();
        // keys in alphabetical order, as a sorted-key JSON writer prints them
        std::string line = "{\"details\":" + e.details() + ",\"event\":\"" + e.name() + "\",\"forward_id\":" + std::to_string(forward_id_) +
                           ",\"kind\":\"qwen_route_trace_v1\",\"monotonic_ns\":" + std::to_string(now) + ",\"request_id\":" + std::to_string(request_id_) +
                           ",\"sequence\":" + std::to_string(written_ + 1) + "}\n";
        if (line.size() > kMaxLine || bytes_ + line.size() > kMaxBytes) throw std::runtime_error("route trace is over its size limit");
        if (std::fwrite(line.data(), 1, line.size(), file_) != line.size() || std::fflush(file_) != 0) throw std::runtime_error("route trace could not be written");
        ++written_; bytes_ += line.size();
    }
    std::FILE* file_ = nullptr;
    Stage stage_ = Stage::Idle;
    Forward open_;
    uint64_t written_ = 0, bytes_ = 0, request_id_ = 0, forward_id_ = 0;
    uint32_t layers_, topk_;
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
            std::vector<int> ids; for (size_t i = 0; i < d.at("routes").size(); ++i) ids.push_back(int(d.at("routes").at(i).number()));
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
