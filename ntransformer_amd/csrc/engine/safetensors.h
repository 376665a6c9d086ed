// engine/safetensors.h -- reader of a model folder: config.json + model.safetensors.
// The tensor file is mapped read-only (8-byte little-endian header length, that many bytes of JSON: name -> dtype, shape, data_offsets; then the data);
// nothing of it is executed or copied until a tensor is uploaded.  The GGUF counterpart is engine/gguf.h.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <vector>
#include "json.h"

namespace nt {

struct StTensor {
    std::string dtype;            // "BF16", "F32", "F16", "I32", ...
    std::vector<int64_t> shape;
    const uint8_t* data = nullptr;
    size_t nbytes = 0;
    int64_t numel() const { int64_t n = 1; for (auto d : shape) n *= d; return n; }
};

class ModelFolder {
public:
    ModelFolder() = default;
    ~ModelFolder();
    ModelFolder(const ModelFolder&) = delete;
    ModelFolder& operator=(const ModelFolder&) = delete;
    // 0 or a negative NTK_E_* (error() says what)
    int open(const std::string& dir);
    const Json& config() const { return config_; }
    const StTensor* tensor(const std::string& name) const;
    const std::map<std::string, StTensor>& tensors() const { return tensors_; }
    const std::string& error() const { return err_; }
    // true if `path` is a folder that holds a config.json
    static bool looks_like(const std::string& path);
    // the "architecture" string of path/config.json ("" if unreadable)
    static std::string architecture_of(const std::string& path);

private:
    Json config_;
    std::map<std::string, StTensor> tensors_;
    void* map_ = nullptr;
    size_t map_bytes_ = 0;
    std::string err_;
};

}  // namespace nt
