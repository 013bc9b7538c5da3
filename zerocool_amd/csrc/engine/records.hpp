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
// The reference also pins file digests and a verification receipt (storage.cpp:318-353); that integrity layer is not
// part of this reader: geometry and sizes are checked, contents are not hashed.
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
    std::variant<std::nullptr_t, bool, double, std::string, Array, Object> value;
    static Json parse(std::string_view text);
    const Json& at(const std::string& key) const;      // std::out_of_range when absent or not an object
    const Json& at(size_t index) const;
    bool contains(const std::string& key) const;
    size_t size() const;
    uint64_t u64() const;                               // std::runtime_error unless a non-negative integer
    const std::string& str() const;
    const Object& object() const;
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
    PreparedExperts(const std::filesystem::path& dir, const MoeShape& shape);
    ~PreparedExperts() override;
    uint32_t layers() const override { return uint32_t(files_.size()); }
    uint64_t stride() const { return stride_; }
    void expert(ExpertKey key, std::span<std::byte> into) const override;      // storage.cpp:391-394
private:
    std::vector<int> files_;
    uint64_t stride_ = 0;
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
void write_prepared_experts(const std::filesystem::path& dir, const MoeShape& shape, uint32_t layers,
                            const std::function<void(ExpertKey, std::span<std::byte>)>& record);

}  // namespace zerocool::engine
