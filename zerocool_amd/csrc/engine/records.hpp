// Expert records on disk, as the reference stores them:
//  * PreparedExperts: the "zc-affine-records-v1" directory written by the reference's prepare step
//    (src/engine/prepare.cpp:268-300): manifest.json + one experts-NN.bin per layer holding `experts` records at a
//    fixed stride (record bytes rounded up to 16384), each record the nine pieces gate/up/down x weight/scales/biases
//    back to back and zero padded.  Reader after PreparedArtifact (src/engine/storage.cpp:316-394).
//  * SafetensorsExperts: the checkpoint itself, nine stacked tensors per layer
//    (model.layers.L.mlp.switch_mlp.{gate,up,down}_proj.{weight,scales,biases}, first dimension = expert); a record
//    is gathered from nine slices (ExpertStore, src/engine/storage.cpp:493-516).
// Both hand out records byte-identical to what the kernels expect (zc_hip_expert_linear), so a record read here can
// be written straight into ExpertCache::home() or an HBM layer array.  No GPU is needed to use this file's classes.
// The prepared directory carries its identity as the reference's does (storage.cpp:316-349): manifest.json names the
// source revision, the recipe and every file with its size and SHA-256; verification.json is the receipt of a
// verification pass (the manifest's own SHA-256, the source revision, and per file the digest, size, device, inode,
// mtime and ctime seen then).  PreparedExperts refuses a directory whose manifest, receipt and files disagree.
#pragma once
#include "engine.hpp"
#include <filesystem>
#include <map>
#include <variant>

namespace zerocool::engine {

// A small JSON value: what manifest.json and a safetensors header need.
struct Json {
    using Array = std::vector<Json>;
    using Object = std::map<std::string, Json>;
    // A number written as a plain run of digits is kept exactly (nanosecond stamps, sizes and offsets exceed 2^53);
    // everything else numeric (a sign, a fraction, an exponent) is a double.
    std::variant<std::nullptr_t, bool, double, std::string, Array, Object, uint64_t> value;
    static Json parse(std::string_view text);
    const Json& at(const std::string& key) const;      // std::out_of_range when absent or not an object
    const Json& at(size_t index) const;
    bool contains(const std::string& key) const;
    size_t size() const;
    uint64_t u64() const;                               // std::runtime_error unless a non-negative integer
    double number() const;                              // either kind of number; std::runtime_error otherwise
    const std::string& str() const;
    const Object& object() const;
};

// SHA-256 (FIPS 180-4), streaming; hex() gives 64 lowercase digits and may be called once.
class Sha256 {
public:
    Sha256();
    void update(std::span<const std::byte> bytes);
    std::string hex();
private:
    void block(const uint8_t* p);
    uint32_t h_[8]; uint8_t tail_[64]; uint64_t bytes_ = 0;
};
std::string sha256_hex(std::string_view text);
std::string sha256_hex_file(const std::filesystem::path& path);

// What a prepared directory must say about where it comes from.  The reference compiles these in (ModelRevision, the
// recipe name and the manifest digest pinned in its model lock, storage.cpp:322-329); here the caller names them.
struct PreparedIdentity {
    std::string source_revision = "synthetic";
    std::string recipe = "q4-control-lossless";
    std::string pinned_manifest_sha256;     // empty: any verified manifest of this revision and recipe
};

class ExpertSource {
public:
    virtual ~ExpertSource() = default;
    virtual uint32_t layers() const = 0;
    virtual void expert(ExpertKey key, std::span<std::byte> into) const = 0;   // into.size() >= record bytes
    // every record of a layer, `stride` bytes apart (the layout of an HBM layer array and of ExpertCache's home)
    void layer(uint32_t layer, std::span<std::byte> into, uint64_t stride) const;
    const MoeShape& shape() const { return shape_; }
protected:
    explicit ExpertSource(const MoeShape& shape) : shape_(shape) {}
    MoeShape shape_;
};

class PreparedExperts final : public ExpertSource {
public:
    PreparedExperts(const std::filesystem::path& dir, const MoeShape& shape, const PreparedIdentity& identity = {});
    ~PreparedExperts() override;
    const std::string& identity() const { return identity_; }                  // SHA-256 of manifest.json (storage.cpp:318-320)
    uint32_t layers() const override { return uint32_t(files_.size()); }
    uint64_t stride() const { return stride_; }
    void expert(ExpertKey key, std::span<std::byte> into) const override;      // storage.cpp:391-394
private:
    std::vector<int> files_;
    uint64_t stride_ = 0;
    std::string identity_;
};

class SafetensorsExperts final : public ExpertSource {
public:
    // every *.safetensors file of the directory is indexed; `layers` consecutive layers starting at 0 must be complete
    SafetensorsExperts(const std::filesystem::path& dir, const MoeShape& shape, uint32_t layers);
    ~SafetensorsExperts() override;
    uint32_t layers() const override { return uint32_t(refs_.size()); }
    void expert(ExpertKey key, std::span<std::byte> into) const override;      // storage.cpp:507-516
private:
    struct Ref { int file; uint64_t offset, row_bytes; };
    std::vector<std::array<Ref, 9>> refs_;
    std::array<uint64_t, 10> offsets_{};
    std::vector<int> files_;
};

// The nine pieces of a record in file order with their byte lengths (prepare.cpp:262-266, storage.cpp:355-368).
std::array<std::pair<std::string, uint64_t>, 9> expert_layout(const MoeShape& shape);
// Writes a prepared directory (manifest.json + experts-NN.bin) from a record generator, as the reference's prepare
// step does from a checkpoint (prepare.cpp:268-300): used to convert synthetic or gathered records, and by the tests.
// Ends with a verification pass, so the directory is ready to open.
void write_prepared_experts(const std::filesystem::path& dir, const MoeShape& shape, uint32_t layers,
                            const std::function<void(ExpertKey, std::span<std::byte>)>& record, const PreparedIdentity& identity = {});
// The verification pass (the reference's `prepare_storage.py --verify`): re-reads every file the manifest names, compares
// size and SHA-256 with the manifest and writes the receipt verification.json.  std::runtime_error when a file differs.
void verify_prepared_experts(const std::filesystem::path& dir);

}  // namespace zerocool::engine
