// Tests of the on-disk expert record readers (zerocool_amd/csrc/engine/records.hpp); no GPU needed.
// Follows the checks of the reference's PreparedArtifact / ExpertStore (src/engine/storage.cpp:316-394, 493-516).
#include "../../zerocool_amd/csrc/engine/route_trace.hpp"
#include <cstdio>
#include <cstring>
#include <fstream>
#include <sys/stat.h>
#include <unistd.h>

using namespace zerocool::engine;
static int checks = 0, failures = 0;
#define CHECK(cond) do { ++checks; if (!(cond)) { ++failures; std::printf("  FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond); } } while (0)
#define CHECK_THROWS(expr) do { ++checks; bool thrown = false; try { (void)(expr); } catch (const std::exception&) { thrown = true; } \
    if (!thrown) { ++failures; std::printf("  FAILED %s:%d: no exception from %s\n", __FILE__, __LINE__, #expr); } } while (0)

static std::byte value(ExpertKey k, uint64_t i) { return std::byte((k.layer * 131 + k.expert * 31 + i * 7 + (i >> 8)) & 0xff); }
static void fill(ExpertKey k, std::span<std::byte> into) { for (uint64_t i = 0; i < into.size(); ++i) into[i] = value(k, i); }
static std::string slurp(const std::filesystem::path& p) { std::ifstream f(p, std::ios::binary); return {std::istreambuf_iterator<char>(f), {}}; }
static void spit(const std::filesystem::path& p, const std::string& s) { std::ofstream f(p, std::ios::binary | std::ios::trunc); f << s; }
static std::string replaced(std::string s, const std::string& a, const std::string& b) { const auto at = s.find(a); if (at != std::string::npos) s.replace(at, a.size(), b); return s; }

int main() {
    const auto root = std::filesystem::temp_directory_path() / ("zc_records_" + std::to_string(::getpid()));
    std::filesystem::remove_all(root);
    MoeShape s; s.hidden = 512; s.experts = 8; s.topk = 2; s.inter = 128;
    const uint64_t bytes = s.expert_bytes();

    std::printf("JSON reader\n");
    const Json j = Json::parse(R"( {"a": [1, 2.5e2, {"b": "x\nA"}], "t": true, "n": null, "big": 9007199254740991} )");
    CHECK(j.at("a").size() == 3 && j.at("a").at(0).u64() == 1 && j.at("a").at(1).u64() == 250);
    CHECK(j.at("a").at(2).at("b").str() == "x\nA" && j.contains("t") && !j.contains("z") && j.at("big").u64() == 9007199254740991ull);
    CHECK_THROWS(Json::parse("{\"a\": }")); CHECK_THROWS(Json::parse("[1, 2")); CHECK_THROWS(Json::parse("{} x")); CHECK_THROWS(j.at("zz"));
    CHECK_THROWS(Json::parse("-1").u64()); CHECK_THROWS(Json::parse("1.5").u64());
    // integers beyond 2^53 are kept exactly (nanosecond time stamps, storage.cpp:346-348 reads them with get<uint64_t>())
    CHECK(Json::parse("1764000000123456789").u64() == 1764000000123456789ull && Json::parse("18446744073709551615").u64() == 18446744073709551615ull);
    CHECK(Json::parse("[-3, 7]").at(0).number() == -3.0 && Json::parse("[-3, 7]").at(1).number() == 7.0 && Json::parse("1e3").u64() == 1000);
    CHECK_THROWS(Json::parse("18446744073709551616").u64());            // one past 2^64 - 1: a double, and not an exact integer below 2^53

    std::printf("record layout\n");
    const auto layout = expert_layout(s);
    CHECK(layout[0].first == "gate_proj.weight" && layout[0].second == 128ull * 512 / 2 && layout[1].second == 128ull * 8 * 2);
    CHECK(layout[6].first == "down_proj.weight" && layout[6].second == 512ull * 128 / 2 && layout[8].second == 512ull * 2 * 2);
    MoeShape ref;   // the reference's own shape: 2,764,800 bytes at stride 2,768,896 (storage.hpp:32-33)
    CHECK(ref.expert_bytes() == 2764800 && (ref.expert_bytes() + 16383) / 16384 * 16384 == 2768896);

    std::printf("prepared directory: write, read back, reject what the reference rejects\n");
    const auto dir = root / "prepared";
    write_prepared_experts(dir, s, 2, fill);
    {
        PreparedExperts p(dir, s);
        CHECK(p.layers() == 2 && p.stride() % 16384 == 0 && p.stride() >= bytes);
        CHECK(std::filesystem::file_size(dir / "experts-01.bin") == p.stride() * s.experts);
        std::vector<std::byte> record(bytes);
        bool same = true;
        for (uint32_t l = 0; l < 2; ++l) for (uint32_t e = 0; e < s.experts; ++e) {
            p.expert({l, e}, record);
            for (uint64_t i = 0; i < bytes; i += 97) same = same && record[i] == value({l, e}, i);
            same = same && record[bytes - 1] == value({l, e}, bytes - 1);
        }
        CHECK(same);
        const uint64_t stride = (bytes + 255) / 256 * 256;                // the layout of an HBM layer array
        std::vector<std::byte> whole(stride * s.experts);
        p.layer(1, whole, stride);
        CHECK(whole[stride * 5 + 1234] == value({1, 5}, 1234) && whole[stride * 7 + bytes - 1] == value({1, 7}, bytes - 1));
        CHECK_THROWS(p.expert({2, 0}, record)); CHECK_THROWS(p.expert({0, 8}, record));
        CHECK_THROWS(p.expert({0, 0}, std::span<std::byte>(record).first(bytes - 1)));
        CHECK_THROWS(p.layer(0, std::span<std::byte>(whole).first(whole.size() - 300), stride));
        std::string pad = slurp(dir / "experts-00.bin");                  // the pad after the nine pieces is zero
        bool zero = true; for (uint64_t i = bytes; i < p.stride(); ++i) zero = zero && pad[i] == 0;
        CHECK(zero);
    }
    MoeShape other = s; other.inter = 256;
    CHECK_THROWS(PreparedExperts(dir, other));                            // "unsupported prepared expert projection"
    // Geometry refusals: the manifest is changed and the verification pass run again, so that only the named defect is left.
    const std::string manifest = slurp(dir / "manifest.json");
    const auto refused_after_verification = [&](const std::string& from, const std::string& to) {
        spit(dir / "manifest.json", replaced(manifest, from, to));
        try { verify_prepared_experts(dir); } catch (const std::exception&) { return true; }   // the pass itself may already refuse
        try { PreparedExperts p(dir, s); } catch (const std::exception&) { return true; }
        return false;
    };
    CHECK(refused_after_verification("zc-affine-records-v1", "zc-affine-records-v2"));
    CHECK(refused_after_verification("\"alignment\": 16384", "\"alignment\": 4096"));
    CHECK(refused_after_verification("\"file\": \"experts-01.bin\"", "\"file\": \"experts-00.bin\""));   // duplicate range
    CHECK(refused_after_verification("\"file\": \"experts-01.bin\"", "\"file\": \"../experts-01.bin\""));
    CHECK(refused_after_verification("\"group_size\": 64", "\"group_size\": 32"));
    spit(dir / "manifest.json", manifest); verify_prepared_experts(dir);
    { PreparedExperts again(dir, s); CHECK(again.layers() == 2); }

    std::printf("prepared directory: identity (manifest digest, verification receipt, file digests)\n");
    CHECK(sha256_hex("") == "e3b0c44298fc1c149afbf4c8996fb92427ae41e4649b934ca495991b7852b855");          // FIPS 180-4 examples
    CHECK(sha256_hex("abc") == "ba7816bf8f01cfea414140de5dae2223b00361a396177a9cb410ff61f20015ad");
    CHECK(sha256_hex("abcdbcdecdefdefgefghfghighijhijkijkljklmklmnlmnomnopnopq") == "248d6a61d20638b8e5c026930c3e6039a33ce45964ff2167f6ecedd419db06c1");
    { Sha256 h; const std::string a(1000, 'a'); for (int i = 0; i < 1000; ++i) h.update(std::as_bytes(std::span<const char>(a.data(), a.size())));
      CHECK(h.hex() == "cdc76e5c9914fb9281a1c7e284d73e67f1809a48a497200e046d39ccc7112cd0"); }              // one million 'a'
    {
        PreparedExperts p(dir, s);
        CHECK(p.identity() == sha256_hex(manifest) && p.identity().size() == 64);
        PreparedIdentity pinned; pinned.pinned_manifest_sha256 = p.identity();
        { PreparedExperts q(dir, s, pinned); CHECK(q.layers() == 2); }
        pinned.pinned_manifest_sha256[0] = pinned.pinned_manifest_sha256[0] == '0' ? '1' : '0';
        CHECK_THROWS(PreparedExperts(dir, s, pinned));                    // "prepared manifest differs from the pinned one"
        PreparedIdentity elsewhere; elsewhere.source_revision = "another-checkpoint";
        CHECK_THROWS(PreparedExperts(dir, s, elsewhere));
        PreparedIdentity recipe; recipe.recipe = "q8";
        CHECK_THROWS(PreparedExperts(dir, s, recipe));
    }
    const std::string receipt = slurp(dir / "verification.json");
    spit(dir / "manifest.json", manifest + " "); CHECK_THROWS(PreparedExperts(dir, s));            // the receipt names another manifest
    spit(dir / "manifest.json", manifest);
    { PreparedExperts again(dir, s); CHECK(again.layers() == 2); }        // the manifest's bytes decide, not its time stamps
    std::filesystem::remove(dir / "verification.json"); CHECK_THROWS(PreparedExperts(dir, s));    // never verified
    spit(dir / "verification.json", receipt);
    {   // one byte of a record file flipped in place: same size, same name
        std::fstream f(dir / "experts-00.bin", std::ios::in | std::ios::out | std::ios::binary);
        f.seekg(4321); char c = 0; f.get(c); f.seekp(4321); f.put(char(c ^ 1));
    }
    bool named = false;
    try { PreparedExperts p(dir, s); } catch (const std::exception& e) { named = std::string(e.what()) == "prepared file changed since verification: experts-00.bin"; }
    CHECK(named);
    named = false;
    try { verify_prepared_experts(dir); } catch (const std::exception& e) { named = std::string(e.what()) == "prepared file differs from its manifest entry: experts-00.bin"; }
    CHECK(named);                                                         // and a new receipt cannot be had for the changed bytes
    {
        std::fstream f(dir / "experts-00.bin", std::ios::in | std::ios::out | std::ios::binary);
        f.seekg(4321); char c = 0; f.get(c); f.seekp(4321); f.put(char(c ^ 1));
    }
    CHECK_THROWS(PreparedExperts(dir, s));                                // the bytes are back, the receipt's time stamps are stale
    verify_prepared_experts(dir);
    { PreparedExperts again(dir, s); CHECK(again.layers() == 2); }
    std::printf("prepared directory in the reference's own layout: more files than expert files, integer time stamps\n");
    {
        // What the reference's tools leave (prepare.cpp:262-300 for the manifest, storage.cpp:337-354 for what is read back):
        // "files" lists every prepared file -- the per-layer expert files AND the n-gram tables -- and the receipt holds
        // size / device / inode / mtime_ns / ctime_ns as JSON integers, with keys this reader does not know beside them.
        const auto ref_dir = root / "reference_layout";
        write_prepared_experts(ref_dir, s, 2, fill);
        spit(ref_dir / "ngram-000.bin", std::string(100, 'n')); spit(ref_dir / "ngram-001.bin", std::string(90, 'm'));
        const Json made = Json::parse(slurp(ref_dir / "manifest.json"));
        std::string m = slurp(ref_dir / "manifest.json");
        const uint64_t expert_bytes_total = made.at("prepared_bytes").u64();
        m = replaced(m, "\n ],\n \"prepared_bytes\": " + std::to_string(expert_bytes_total),
                     ",\n  {\"path\": \"ngram-000.bin\", \"size\": 100, \"sha256\": \"" + sha256_hex(std::string(100, 'n')) + "\"}"
                     ",\n  {\"path\": \"ngram-001.bin\", \"size\": 90, \"sha256\": \"" + sha256_hex(std::string(90, 'm')) + "\"}"
                     "\n ],\n \"ngrams\": [{\"order\": 0, \"file\": \"ngram-000.bin\"}, {\"order\": 1, \"file\": \"ngram-001.bin\"}],"
                     "\n \"source_files\": {\"model.safetensors\": \"00\"},\n \"prepared_bytes\": " + std::to_string(expert_bytes_total + 190));
        spit(ref_dir / "manifest.json", m);
        const Json listed = Json::parse(m);
        CHECK(listed.at("files").size() == 4 && listed.at("experts").size() == 2);
        const auto receipt_with = [&](bool integers) {
            std::string r = "{\n  \"schema\": 1,\n  \"verified_at\": 1764000000,\n  \"manifest_sha256\": \"" + sha256_hex(m) + "\",\n  \"source_revision\": \"synthetic\",\n  \"files\": {";
            for (size_t i = 0; i < listed.at("files").size(); ++i) {
                const std::string name = listed.at("files").at(i).at("path").str();
                struct stat st{}; ::stat((ref_dir / name).c_str(), &st);
                const std::string mt = std::to_string(uint64_t(st.st_mtim.tv_sec) * 1000000000ull + uint64_t(st.st_mtim.tv_nsec));
                const std::string ct = std::to_string(uint64_t(st.st_ctim.tv_sec) * 1000000000ull + uint64_t(st.st_ctim.tv_nsec));
                const std::string q = integers ? "" : "\"";
                r += std::string(i ? "," : "") + "\n    \"" + name + "\": {\n      \"size\": " + std::to_string(st.st_size) + ",\n      \"device\": " + std::to_string(st.st_dev) +
                     ",\n      \"inode\": " + std::to_string(st.st_ino) + ",\n      \"mtime_ns\": " + q + mt + q + ",\n      \"ctime_ns\": " + q + ct + q +
                     ",\n      \"sha256\": \"" + listed.at("files").at(i).at("sha256").str() + "\"\n    }";
            }
            return r + "\n  }\n}\n";
        };
        spit(ref_dir / "verification.json", receipt_with(true));
        {
            PreparedExperts p(ref_dir, s);
            std::vector<std::byte> record(bytes);
            p.expert({1, 6}, record);
            CHECK(p.layers() == 2 && record[777] == value({1, 6}, 777));
        }
        spit(ref_dir / "verification.json", receipt_with(false));       // stamps as decimal strings: still read
        { PreparedExperts p(ref_dir, s); CHECK(p.layers() == 2); }
        // an integer stamp that is off by one nanosecond is a changed file: no rounding through a double hides it
        struct stat st{}; ::stat((ref_dir / "ngram-001.bin").c_str(), &st);
        const uint64_t mt = uint64_t(st.st_mtim.tv_sec) * 1000000000ull + uint64_t(st.st_mtim.tv_nsec);
        const std::string good = receipt_with(true);
        spit(ref_dir / "verification.json", replaced(good, "\"mtime_ns\": " + std::to_string(mt) + ",\n      \"ctime_ns\"", "\"mtime_ns\": " + std::to_string(mt + 1) + ",\n      \"ctime_ns\""));
        if (mt > (1ull << 53)) CHECK_THROWS(PreparedExperts(ref_dir, s));
        // the receipt this library writes holds integers too
        verify_prepared_experts(ref_dir);
        const Json own = Json::parse(slurp(ref_dir / "verification.json"));
        CHECK(std::holds_alternative<uint64_t>(own.at("files").at("ngram-000.bin").at("mtime_ns").value));
        { PreparedExperts p(ref_dir, s); CHECK(p.layers() == 2); }
        // an expert range that names a file the manifest does not list is still refused
        spit(ref_dir / "manifest.json", replaced(m, "\"path\": \"experts-01.bin\"", "\"path\": \"experts-1.bin\""));
        std::filesystem::copy_file(ref_dir / "experts-01.bin", ref_dir / "experts-1.bin");
        verify_prepared_experts(ref_dir);
        CHECK_THROWS(PreparedExperts(ref_dir, s));
    }
    std::filesystem::resize_file(dir / "experts-01.bin", std::filesystem::file_size(dir / "experts-01.bin") - 1); CHECK_THROWS(PreparedExperts(dir, s));
    CHECK_THROWS(verify_prepared_experts(dir));
    std::filesystem::remove(dir / "experts-01.bin"); CHECK_THROWS(PreparedExperts(dir, s));
    CHECK_THROWS(PreparedExperts(root / "nowhere", s));

    std::printf("safetensors checkpoint: nine stacked tensors per layer gathered into records\n");
    const auto ckpt = root / "checkpoint"; std::filesystem::create_directories(ckpt);
    {
        // layer 0 in one file, layer 1 in another; tensor data = for each piece, the experts' slices back to back
        for (uint32_t l = 0; l < 2; ++l) {
            std::string header = "{\"__metadata__\": {\"format\": \"pt\"}", data; uint64_t at = 0, piece_at = 0;
            for (int p = 0; p < 9; ++p) {
                const uint64_t rows = p < 6 ? s.inter : s.hidden, cols = p < 6 ? s.hidden : s.inter, len = layout[p].second;
                header += ", \"model.layers." + std::to_string(l) + ".mlp.switch_mlp." + layout[p].first + "\": {\"dtype\": \"" + (p % 3 == 0 ? "U32" : "BF16") +
                          "\", \"shape\": [" + std::to_string(s.experts) + ", " + std::to_string(rows) + ", " + std::to_string(p % 3 == 0 ? cols / 8 : cols / 64) +
                          "], \"data_offsets\": [" + std::to_string(at) + ", " + std::to_string(at + len * s.experts) + "]}";
                for (uint32_t e = 0; e < s.experts; ++e) for (uint64_t i = 0; i < len; ++i) data += char(value({l, e}, piece_at + i));
                at += len * s.experts; piece_at += len;
            }
            header += "}";
            const uint64_t n = header.size(); std::string file(8, '\0'); std::memcpy(file.data(), &n, 8);
            spit(ckpt / ("model-0000" + std::to_string(l + 1) + ".safetensors"), file + header + data);
        }
        SafetensorsExperts c(ckpt, s, 2);
        std::vector<std::byte> record(bytes); bool same = true;
        for (uint32_t l = 0; l < 2; ++l) for (uint32_t e = 0; e < s.experts; e += 3) {
            c.expert({l, e}, record);
            for (uint64_t i = 0; i < bytes; i += 61) same = same && record[i] == value({l, e}, i);
        }
        CHECK(same);                                                      // byte-identical to the prepared record of the same expert
        CHECK_THROWS(c.expert({2, 0}, record));
        CHECK_THROWS(SafetensorsExperts(ckpt, s, 3));                     // layer 2 is not there
        CHECK_THROWS(SafetensorsExperts(ckpt, other, 2));                 // shapes differ
    }
    std::printf("route trace: the reference's call-order rules, and a round trip through the reader\n");
    {
        const auto path = root / "routes.jsonl";
        const uint32_t L = 3, K = 2;
        {
            RouteTrace t(path, "{\"model\": \"test\", \"layers\": 3}", L, K);
            CHECK_THROWS(RouteTrace(path, "{}", L, K));                    // must be a new file
            const int prompt[3] = {5, 6, 7}, one[1] = {9};
            CHECK_THROWS(t.begin(1, 0, prompt, "prefill", 16));            // no request yet
            t.request_begin("a \"quoted\" name", prompt, 4, false);
            CHECK_THROWS(t.request_begin("again", prompt, 4, false));
            t.begin(77, 0, prompt, "prefill", 16);
            const int r0[6] = {1, 2, 3, 4, 5, 6}, r1[6] = {6, 5, 4, 3, 2, 1}, r2[6] = {0, 1, 0, 1, 0, 1};
            CHECK_THROWS(t.routes(1, 0, 3, r0));                           // layers in order
            CHECK_THROWS(t.routes(0, 0, 3, std::span<const int>(r0, 5)));  // tokens * topk ids
            t.routes(0, 0, 3, r0); t.routes(1, 0, 3, r1);
            CHECK_THROWS(t.commit(3));                                     // a layer is missing
            t.routes(2, 0, 3, r2); CHECK_THROWS(t.commit(4)); t.commit(3);
            t.begin(77, 3, one, "decode", 16); const int d[2] = {7, 8}; t.routes(0, 3, 1, d); t.abort();
            CHECK_THROWS(t.finish());                                      // the request is still open
            t.request_end(one, "stop", 0); t.cache_reset(); t.finish();
        }
        const TraceSummary sum = read_route_trace(path);
        CHECK(sum.complete && sum.events == 13 && sum.forwards.size() == 2);
        CHECK(sum.forwards[0].committed && sum.forwards[0].tokens == 3 && sum.forwards[0].phase == "prefill" && sum.forwards[0].routes.size() == 3);
        CHECK(sum.forwards[0].routes[1] == (std::vector<int>{6, 5, 4, 3, 2, 1}) && !sum.forwards[1].committed && sum.forwards[1].routes.size() == 1);
        spit(root / "broken.jsonl", replaced(slurp(path), "\"sequence\":3", "\"sequence\":4")); CHECK_THROWS(read_route_trace(root / "broken.jsonl"));
        { RouteTrace open_ended(root / "open.jsonl", "{}", L, K); }
        CHECK(!read_route_trace(root / "open.jsonl").complete);           // closed without finish(): "incomplete"
        const float logits[4] = {1, 2, 3, 4};
        write_tensor_dump(root / "dump", 12, "router_0", std::as_bytes(std::span(logits)));
        const auto back = read_tensor_dump(root / "dump", 12, "router_0");
        CHECK(back.size() == 16 && std::memcmp(back.data(), logits, 16) == 0 && std::filesystem::exists(root / "dump" / "step_12" / "router_0.bin"));
        CHECK_THROWS(read_tensor_dump(root / "dump", 12, "route_0"));
    }
    std::filesystem::remove_all(root);
    std::printf("%d checks, %d failures\n", checks, failures);
    return failures ? 1 : 0;
}
