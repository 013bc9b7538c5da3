#include "records.hpp"
#include <charconv>
#include <cmath>
#include <cstring>
#include <fcntl.h>
#include <fstream>
#include <sstream>
#include <sys/stat.h>
#include <unistd.h>

namespace zerocool::engine {
namespace {

struct Parser {
    std::string_view s; size_t i = 0;
    [[noreturn]] void fail(const char* what) const { throw std::runtime_error(std::string("invalid JSON: ") + what + " at byte " + std::to_string(i)); }
    void space() { while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r')) ++i; }
    char peek() { space(); if (i >= s.size()) fail("unexpected end"); return s[i]; }
    void expect(char c) { if (peek() != c) fail("unexpected character"); ++i; }
    bool literal(std::string_view word) { if (s.substr(i, word.size()) == word) { i += word.size(); return true; } return false; }
    std::string string() {
        expect('"'); std::string out;
        while (true) {
            if (i >= s.size()) fail("unterminated string");
            const char c = s[i++];
            if (c == '"') return out;
            if (c != '\\') { out += c; continue; }
            if (i >= s.size()) fail("unterminated escape");
            const char e = s[i++];
            switch (e) {
                case '"': case '\\': case '/': out += e; break;
                case 'n': out += '\n'; break; case 't': out += '\t'; break; case 'r': out += '\r'; break;
                case 'b': out += '\b'; break; case 'f': out += '\f'; break;
                case 'u': {
                    if (i + 4 > s.size()) fail("short unicode escape");
                    unsigned code = 0; auto r = std::from_chars(s.data() + i, s.data() + i + 4, code, 16);
                    if (r.ptr != s.data() + i + 4) fail("bad unicode escape");
                    i += 4;
                    if (code < 0x80) out += char(code);
                    else if (code < 0x800) { out += char(0xc0 | (code >> 6)); out += char(0x80 | (code & 63)); }
                    else { out += char(0xe0 | (code >> 12)); out += char(0x80 | ((code >> 6) & 63)); out += char(0x80 | (code & 63)); }
                    break;
                }
                default: fail("unknown escape");
            }
        }
    }
    Json value(int depth = 0) {
        if (depth > 64) fail("nesting too deep");
        const char c = peek();
        Json j;
        if (c == '{') {
            ++i; Json::Object o;
            if (peek() == '}') { ++i; j.value = std::move(o); return j; }
            while (true) {
                space(); std::string k = string(); expect(':'); o[std::move(k)] = value(depth + 1);
                if (peek() == ',') { ++i; continue; }
                expect('}'); break;
            }
            j.value = std::move(o);
        } else if (c == '[') {
            ++i; Json::Array a;
            if (peek() == ']') { ++i; j.value = std::move(a); return j; }
            while (true) {
                a.push_back(value(depth + 1));
                if (peek() == ',') { ++i; continue; }
                expect(']'); break;
            }
            j.value = std::move(a);
        } else if (c == '"') j.value = string();
        else if (literal("true")) j.value = true;
        else if (literal("false")) j.value = false;
        else if (literal("null")) j.value = nullptr;
        else {
            const size_t start = i;
            while (i < s.size() && (std::isdigit(static_cast<unsigned char>(s[i])) || s[i] == '-' || s[i] == '+' || s[i] == '.' || s[i] == 'e' || s[i] == 'E')) ++i;
            if (start == i) fail("unexpected character");
            const std::string text(s.substr(start, i - start));
            uint64_t whole = 0;
            const auto r = std::from_chars(text.data(), text.data() + text.size(), whole);
            if (r.ec == std::errc() && r.ptr == text.data() + text.size() && std::isdigit(static_cast<unsigned char>(text[0]))) { j.value = whole; return j; }
            char* end = nullptr;
            const double v = std::strtod(text.c_str(), &end);
            if (!end || *end) fail("bad number");
            j.value = v;
        }
        return j;
    }
};

std::string read_text(const std::filesystem::path& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("cannot read " + path.string());
    std::ostringstream out; out << f.rdbuf(); return out.str();
}
void read_at(int fd, uint64_t offset, std::span<std::byte> into) {
    size_t done = 0;
    while (done < into.size()) {
        const ssize_t n = ::pread(fd, into.data() + done, into.size() - done, off_t(offset + done));
        if (n <= 0) throw std::runtime_error("short read of an expert record");
        done += size_t(n);
    }
}
uint64_t file_size(int fd) { struct stat st{}; if (::fstat(fd, &st) != 0 || st.st_size < 0) throw std::runtime_error("cannot stat an expert file"); return uint64_t(st.st_size); }
int open_file(const std::filesystem::path& path) {
    const int fd = ::open(path.c_str(), O_RDONLY | O_CLOEXEC);
    if (fd < 0) throw std::runtime_error("missing prepared file: " + path.string());
    return fd;
}
constexpr uint64_t kAlignment = 16384;   // storage.cpp:374

struct FileIdentity { uint64_t size, device, inode, mtime_ns, ctime_ns; };
FileIdentity identity_of(const std::filesystem::path& path) {
    struct stat st{};
    if (::stat(path.c_str(), &st) != 0 || st.st_size < 0) throw std::runtime_error("missing prepared file");
    return {uint64_t(st.st_size), uint64_t(st.st_dev), uint64_t(st.st_ino),
            uint64_t(st.st_mtim.tv_sec) * 1000000000ull + uint64_t(st.st_mtim.tv_nsec),
            uint64_t(st.st_ctim.tv_sec) * 1000000000ull + uint64_t(st.st_ctim.tv_nsec)};
}
bool plain_filename(const std::string& name) { return !name.empty() && std::filesystem::path(name).filename() == name && name != "." && name != ".."; }
// Nanosecond stamps exceed 2^53.  The reference writes them as JSON integers (scripts/qwen/verify_checkpoint.py:18-22,
// read with get<uint64_t>() in storage.cpp:346-348) and so does this writer; the parser keeps such integers exactly.
// A receipt that holds them as decimal strings (what earlier versions of this library wrote) is still read.
uint64_t stamp(const Json& j) {
    if (std::holds_alternative<uint64_t>(j.value)) return j.u64();
    const std::string& s = j.str(); uint64_t v = 0;
    const auto r = std::from_chars(s.data(), s.data() + s.size(), v);
    if (r.ec != std::errc() || r.ptr != s.data() + s.size()) throw std::runtime_error("invalid time stamp in the verification receipt");
    return v;
}

}  // namespace

// ---- SHA-256
namespace {
constexpr uint32_t kRound[64] = {
    0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3,
    0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da,
    0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967, 0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13,
    0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
    0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208,
    0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
inline uint32_t rotr(uint32_t v, int n) { return (v >> n) | (v << (32 - n)); }
}  // namespace
Sha256::Sha256() : h_{0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19}, tail_{} {}
void Sha256::block(const uint8_t* p) {
    uint32_t w[64];
    for (int i = 0; i < 16; ++i) w[i] = uint32_t(p[4 * i]) << 24 | uint32_t(p[4 * i + 1]) << 16 | uint32_t(p[4 * i + 2]) << 8 | p[4 * i + 3];
    for (int i = 16; i < 64; ++i) {
        const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3), s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
        w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h_[0], b = h_[1], c = h_[2], d = h_[3], e = h_[4], f = h_[5], g = h_[6], h = h_[7];
    for (int i = 0; i < 64; ++i) {
        const uint32_t t1 = h + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + kRound[i] + w[i];
        const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
        h = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h_[0] += a; h_[1] += b; h_[2] += c; h_[3] += d; h_[4] += e; h_[5] += f; h_[6] += g; h_[7] += h;
}
void Sha256::update(std::span<const std::byte> bytes) {
    const uint8_t* p = reinterpret_cast<const uint8_t*>(bytes.data()); size_t n = bytes.size();
    size_t held = size_t(bytes_ % 64); bytes_ += n;
    if (held) {
        const size_t take = std::min(n, 64 - held);
        std::memcpy(tail_ + held, p, take); p += take; n -= take; held += take;
        if (held < 64) return;
        block(tail_);
    }
    for (; n >= 64; p += 64, n -= 64) block(p);
    std::memcpy(tail_, p, n);
}
std::string Sha256::hex() {
    const uint64_t bits = bytes_ * 8;
    size_t held = size_t(bytes_ % 64);
    tail_[held++] = 0x80;
    if (held > 56) { std::memset(tail_ + held, 0, 64 - held); block(tail_); held = 0; }
    std::memset(tail_ + held, 0, 56 - held);
    for (int i = 0; i < 8; ++i) tail_[56 + i] = uint8_t(bits >> (56 - 8 * i));
    block(tail_);
    std::string out; constexpr char digits[] = "0123456789abcdef";
    for (uint32_t v : h_) for (int s = 28; s >= 0; s -= 4) out += digits[(v >> s) & 15];
    return out;
}
std::string sha256_hex(std::string_view text) {
    Sha256 h; h.update(std::as_bytes(std::span<const char>(text.data(), text.size()))); return h.hex();
}
std::string sha256_hex_file(const std::filesystem::path& path) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("missing prepared file");
    Sha256 h; std::vector<char> buffer(1 << 20);
    while (f) { f.read(buffer.data(), std::streamsize(buffer.size())); h.update(std::as_bytes(std::span<const char>(buffer.data(), size_t(f.gcount())))); }
    return h.hex();
}

Json Json::parse(std::string_view text) { Parser p{text}; Json j = p.value(); p.space(); if (p.i != text.size()) p.fail("trailing characters"); return j; }
const Json::Object& Json::object() const { if (auto* o = std::get_if<Object>(&value)) return *o; throw std::out_of_range("JSON value is not an object"); }
const Json& Json::at(const std::string& key) const { const auto& o = object(); auto it = o.find(key); if (it == o.end()) throw std::out_of_range("missing JSON key: " + key); return it->second; }
const Json& Json::at(size_t index) const { if (auto* a = std::get_if<Array>(&value); a && index < a->size()) return (*a)[index]; throw std::out_of_range("JSON index out of range"); }
bool Json::contains(const std::string& key) const { auto* o = std::get_if<Object>(&value); return o && o->count(key); }
size_t Json::size() const { if (auto* a = std::get_if<Array>(&value)) return a->size(); if (auto* o = std::get_if<Object>(&value)) return o->size(); return 0; }
double Json::number() const {
    if (auto* w = std::get_if<uint64_t>(&value)) return double(*w);
    if (auto* d = std::get_if<double>(&value)) return *d;
    throw std::runtime_error("JSON value is not a number");
}
uint64_t Json::u64() const {
    if (auto* w = std::get_if<uint64_t>(&value)) return *w;
    if (auto* d = std::get_if<double>(&value); d && *d >= 0 && *d < 9007199254740992.0 && std::floor(*d) == *d) return uint64_t(*d);
    throw std::runtime_error("JSON value is not a non-negative integer");
}
const std::string& Json::str() const { if (auto* s = std::get_if<std::string>(&value)) return *s; throw std::runtime_error("JSON value is not a string"); }

std::array<std::pair<std::string, uint64_t>, 9> expert_layout(const MoeShape& s) {
    const zc_moe_config c = s.abi();
    std::array<std::pair<std::string, uint64_t>, 9> out;
    const char* proj[3] = {"gate_proj", "up_proj", "down_proj"};
    for (int p = 0; p < 3; ++p) {
        const uint64_t K = p < 2 ? s.hidden : s.inter, N = p < 2 ? s.inter : s.hidden, bits = p < 2 ? s.bits_gate_up : s.bits_down;
        out[3 * p] = {std::string(proj[p]) + ".weight", N * K * bits / 8};
        out[3 * p + 1] = {std::string(proj[p]) + ".scales", N * (K / s.group) * 2};
        out[3 * p + 2] = {std::string(proj[p]) + ".biases", N * (K / s.group) * 2};
    }
    uint64_t total = 0; for (auto& e : out) total += e.second;
    if (total != zc_hip_record_bytes(&c, 0)) throw std::logic_error("expert layout differs from the kernels' record size");
    return out;
}

void ExpertSource::layer(uint32_t l, std::span<std::byte> into, uint64_t stride) const {
    const uint64_t bytes = shape_.expert_bytes();
    if (stride < bytes || into.size() < stride * (shape_.experts - 1) + bytes) throw std::out_of_range("layer buffer too small");
    for (uint32_t e = 0; e < shape_.experts; ++e) expert({l, e}, into.subspan(e * stride, bytes));
}

PreparedExperts::PreparedExperts(const std::filesystem::path& dir, const MoeShape& shape, const PreparedIdentity& want) : ExpertSource(shape) {
    const std::string text = read_text(dir / "manifest.json");
    const Json m = Json::parse(text);
    identity_ = sha256_hex(text);                                                                       // storage.cpp:318-320
    const Json receipt = Json::parse(read_text(dir / "verification.json"));
    const auto text_of = [](const Json& j, const char* key) { return j.contains(key) ? j.at(key).str() : std::string(); };
    if (!m.contains("schema") || m.at("schema").u64() != 1 || text_of(m, "format") != "zc-affine-records-v1" ||
        text_of(m, "source_revision") != want.source_revision || text_of(receipt, "manifest_sha256") != identity_ ||
        text_of(receipt, "source_revision") != want.source_revision || text_of(m, "recipe") != want.recipe)
        throw std::runtime_error("unverified or incompatible prepared artifact; run the verification pass");   // storage.cpp:322-326
    if (!want.pinned_manifest_sha256.empty() && want.pinned_manifest_sha256 != identity_)
        throw std::runtime_error("prepared manifest differs from the pinned one");                      // storage.cpp:327-329
    std::map<std::string, bool> listed;
    uint64_t total = 0;
    for (size_t i = 0; i < m.at("files").size(); ++i) {                                                 // storage.cpp:337-350
        const Json& entry = m.at("files").at(i);
        const std::string& name = entry.at("path").str();
        if (!plain_filename(name) || !listed.emplace(name, true).second) throw std::runtime_error("invalid prepared filename");
        const Json& saved = receipt.at("files").at(name);
        const FileIdentity now = identity_of(dir / name);
        if (entry.at("size").u64() != now.size || saved.at("sha256").str() != entry.at("sha256").str() || saved.at("size").u64() != now.size ||
            saved.at("device").u64() != now.device || saved.at("inode").u64() != now.inode || stamp(saved.at("mtime_ns")) != now.mtime_ns ||
            stamp(saved.at("ctime_ns")) != now.ctime_ns)
            throw std::runtime_error("prepared file changed since verification: " + name);
        total += now.size;
    }
    // The reference's manifest lists more than the expert files (one per layer plus its 128 n-gram tables, storage.cpp:351);
    // what this reader needs is that the listed bytes add up and, below, that every expert range names a listed file.
    if (m.at("prepared_bytes").u64() != total) throw std::runtime_error("incomplete prepared layout");   // storage.cpp:351-354
    const auto layout = expert_layout(shape);
    if (m.at("expert_layout").size() != 9) throw std::runtime_error("incomplete prepared layout");      // storage.cpp:352-354
    uint64_t offset = 0;
    for (size_t p = 0; p < 9; ++p) {                                                                    // storage.cpp:358-367
        const Json& e = m.at("expert_layout").at(p);
        const uint64_t bits = p < 6 ? shape.bits_gate_up : shape.bits_down;
        if (e.at("name").str() != layout[p].first || e.at("offset").u64() != offset || e.at("length").u64() != layout[p].second ||
            e.at("bits").u64() != bits || e.at("group_size").u64() != shape.group)
            throw std::runtime_error("unsupported prepared expert projection");
        offset += layout[p].second;
    }
    const uint64_t bytes = shape.expert_bytes();
    stride_ = (bytes + kAlignment - 1) / kAlignment * kAlignment;
    const size_t layers = m.at("experts").size();
    if (!layers) throw std::runtime_error("incomplete prepared layout");
    std::map<std::string, bool> used;
    try {
        for (size_t l = 0; l < layers; ++l) {                                                           // storage.cpp:370-379
            const Json& e = m.at("experts").at(l);
            if (e.at("layer").u64() != l || e.at("count").u64() != shape.experts || e.at("offset").u64() != 0 || e.at("length").u64() != bytes ||
                e.at("stride").u64() != stride_ || e.at("alignment").u64() != kAlignment)
                throw std::runtime_error("unsupported prepared expert range");
            const std::string& name = e.at("file").str();
            if (!plain_filename(name)) throw std::runtime_error("invalid prepared filename");
            if (!used.emplace(name, true).second) throw std::runtime_error("duplicate prepared file range");
            if (!listed.count(name)) throw std::runtime_error("prepared expert range names an unlisted file");
            files_.push_back(open_file(dir / name));
            if (file_size(files_.back()) != stride_ * shape.experts) throw std::runtime_error("invalid prepared expert length");
        }
    } catch (...) { for (int fd : files_) ::close(fd); throw; }
}
PreparedExperts::~PreparedExperts() { for (int fd : files_) ::close(fd); }
void PreparedExperts::expert(ExpertKey key, std::span<std::byte> into) const {
    const uint64_t bytes = shape_.expert_bytes();
    if (key.layer >= files_.size() || key.expert >= shape_.experts || into.size() < bytes) throw std::out_of_range("prepared expert range");
    read_at(files_[key.layer], key.expert * stride_, into.first(bytes));
}

SafetensorsExperts::SafetensorsExperts(const std::filesystem::path& dir, const MoeShape& shape, uint32_t layers) : ExpertSource(shape) {
    struct Tensor { int file; uint64_t offset, bytes; std::vector<uint64_t> dims; std::string dtype; };
    std::map<std::string, Tensor> index;
    try {
        std::vector<std::filesystem::path> paths;
        for (const auto& entry : std::filesystem::directory_iterator(dir)) if (entry.path().extension() == ".safetensors") paths.push_back(entry.path());
        std::sort(paths.begin(), paths.end());
        for (const auto& path : paths) {
            const int fd = open_file(path); files_.push_back(fd);
            const uint64_t size = file_size(fd);
            uint64_t header = 0; std::byte raw[8];
            if (size < 8) throw std::runtime_error("invalid safetensors header");
            read_at(fd, 0, raw); std::memcpy(&header, raw, 8);
            if (header > size - 8 || header > (100ull << 20)) throw std::runtime_error("invalid safetensors header");
            std::string text(header, '\0'); read_at(fd, 8, {reinterpret_cast<std::byte*>(text.data()), text.size()});
            const Json h = Json::parse(text);
            for (const auto& [name, t] : h.object()) {
                if (name == "__metadata__") continue;
                Tensor ref{fd, 0, 0, {}, t.at("dtype").str()};
                for (size_t d = 0; d < t.at("shape").size(); ++d) ref.dims.push_back(t.at("shape").at(d).u64());
                const uint64_t begin = t.at("data_offsets").at(0).u64(), end = t.at("data_offsets").at(1).u64();
                if (end < begin || 8 + header + end > size) throw std::runtime_error("safetensors tensor outside its file");
                ref.offset = 8 + header + begin; ref.bytes = end - begin;
                index[name] = std::move(ref);
            }
        }
        const auto layout = expert_layout(shape);
        for (int p = 0; p < 9; ++p) offsets_[p + 1] = offsets_[p] + layout[p].second;
        refs_.resize(layers);
        for (uint32_t l = 0; l < layers; ++l)
            for (int p = 0; p < 9; ++p) {                                                                // storage.cpp:496-504
                const auto it = index.find("model.layers." + std::to_string(l) + ".mlp.switch_mlp." + layout[p].first);
                if (it == index.end()) throw std::runtime_error("incompatible expert layout");
                const Tensor& t = it->second;
                const uint64_t rows = p < 6 ? shape.inter : shape.hidden, cols = p < 6 ? shape.hidden : shape.inter;
                const uint64_t bits = p < 6 ? shape.bits_gate_up : shape.bits_down;
                const std::vector<uint64_t> want = {shape.experts, rows, p % 3 == 0 ? cols * bits / 32 : cols / shape.group};
                if (t.dims != want || t.dtype != (p % 3 == 0 ? "U32" : "BF16") || t.bytes != layout[p].second * shape.experts)
                    throw std::runtime_error("incompatible expert layout");
                refs_[l][p] = {t.file, t.offset, layout[p].second};
            }
    } catch (...) { for (int fd : files_) ::close(fd); throw; }
}
SafetensorsExperts::~SafetensorsExperts() { for (int fd : files_) ::close(fd); }
void SafetensorsExperts::expert(ExpertKey key, std::span<std::byte> into) const {
    if (key.layer >= refs_.size() || key.expert >= shape_.experts || into.size() < offsets_[9]) throw std::out_of_range("invalid expert load");
    for (int p = 0; p < 9; ++p) {
        const Ref& r = refs_[key.layer][p];
        read_at(r.file, r.offset + key.expert * r.row_bytes, into.subspan(offsets_[p], r.row_bytes));
    }
}

void write_prepared_experts(const std::filesystem::path& dir, const MoeShape& shape, uint32_t layers,
                            const std::function<void(ExpertKey, std::span<std::byte>)>& record, const PreparedIdentity& identity) {
    std::filesystem::create_directories(dir);
    const auto layout = expert_layout(shape);
    const uint64_t bytes = shape.expert_bytes(), stride = (bytes + kAlignment - 1) / kAlignment * kAlignment;
    std::ostringstream m;
    m << "{\n \"schema\": 1,\n \"format\": \"zc-affine-records-v1\",\n \"source_revision\": \"" << identity.source_revision
      << "\",\n \"recipe\": \"" << identity.recipe << "\",\n \"expert_layout\": [";
    std::ostringstream files; uint64_t total = 0;
    uint64_t offset = 0;
    for (size_t p = 0; p < 9; ++p) {
        m << (p ? "," : "") << "\n  {\"name\": \"" << layout[p].first << "\", \"offset\": " << offset << ", \"length\": " << layout[p].second
          << ", \"bits\": " << (p < 6 ? shape.bits_gate_up : shape.bits_down) << ", \"group_size\": " << shape.group << "}";
        offset += layout[p].second;
    }
    m << "\n ],\n \"experts\": [";
    std::vector<std::byte> buffer(stride);
    for (uint32_t l = 0; l < layers; ++l) {
        char name[32]; std::snprintf(name, sizeof name, "experts-%02u.bin", l);                        // prepare.cpp:272-273
        std::ofstream out(dir / name, std::ios::binary | std::ios::trunc);
        Sha256 digest;
        for (uint32_t e = 0; e < shape.experts; ++e) {
            std::memset(buffer.data(), 0, buffer.size());                                               // the pad after the nine pieces is zero
            record({l, e}, std::span<std::byte>(buffer).first(bytes));
            out.write(reinterpret_cast<const char*>(buffer.data()), std::streamsize(stride));
            digest.update(buffer);
        }
        out.close();
        if (!out) throw std::runtime_error("cannot write " + (dir / name).string());
        files << (l ? "," : "") << "\n  {\"path\": \"" << name << "\", \"size\": " << stride * shape.experts << ", \"sha256\": \"" << digest.hex() << "\"}";
        total += stride * shape.experts;
        m << (l ? "," : "") << "\n  {\"layer\": " << l << ", \"file\": \"" << name << "\", \"count\": " << shape.experts << ", \"offset\": 0, \"length\": " << bytes
          << ", \"stride\": " << stride << ", \"alignment\": " << kAlignment << "}";
    }
    m << "\n ],\n \"files\": [" << files.str() << "\n ],\n \"prepared_bytes\": " << total << "\n}\n";
    std::ofstream f(dir / "manifest.json", std::ios::trunc); f << m.str(); f.close();
    if (!f) throw std::runtime_error("cannot write the prepared manifest");
    verify_prepared_experts(dir);
}

void verify_prepared_experts(const std::filesystem::path& dir) {
    const std::string text = read_text(dir / "manifest.json");
    const Json m = Json::parse(text);
    std::ostringstream r;
    r << "{\n \"manifest_sha256\": \"" << sha256_hex(text) << "\",\n \"source_revision\": \"" << m.at("source_revision").str() << "\",\n \"files\": {";
    for (size_t i = 0; i < m.at("files").size(); ++i) {
        const Json& entry = m.at("files").at(i);
        const std::string& name = entry.at("path").str();
        if (!plain_filename(name)) throw std::runtime_error("invalid prepared filename");
        const FileIdentity now = identity_of(dir / name);
        const std::string digest = sha256_hex_file(dir / name);
        if (now.size != entry.at("size").u64() || digest != entry.at("sha256").str())
            throw std::runtime_error("prepared file differs from its manifest entry: " + name);
        r << (i ? "," : "") << "\n  \"" << name << "\": {\"sha256\": \"" << digest << "\", \"size\": " << now.size << ", \"device\": " << now.device
          << ", \"inode\": " << now.inode << ", \"mtime_ns\": " << now.mtime_ns << ", \"ctime_ns\": " << now.ctime_ns << "}";
    }
    r << "\n }\n}\n";
    std::ofstream f(dir / "verification.json", std::ios::trunc); f << r.str(); f.close();
    if (!f) throw std::runtime_error("cannot write the verification receipt");
}

}  // namespace zerocool::engine
