// qm_safetensors.hpp — reader of the safetensors container: 8-byte little-endian header length,
// a JSON object {name: {dtype, shape, data_offsets}, "__metadata__": ...}, then the tensor bytes.
// Follows what SafeFile / ModelWeights check (R17:4020-4099): header inside the file, every
// tensor's range inside the data section and equal to elements * sizeof(dtype); a model
// directory is the union of its *.safetensors files, tensors are looked up by name suffix.
#ifndef QM_SAFETENSORS_HPP
#define QM_SAFETENSORS_HPP

#include <cstdint>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

namespace qm_engine {

struct IoError : std::runtime_error { using std::runtime_error::runtime_error; };
struct TensorError : std::runtime_error { using std::runtime_error::runtime_error; };

struct TensorView {
    std::string name, dtype;
    std::vector<int64_t> shape;
    const uint8_t* data = nullptr;
    uint64_t bytes = 0;
    uint64_t elements() const {
        uint64_t n = 1;
        for (int64_t d : shape) n *= static_cast<uint64_t>(d);
        return n;
    }
};

// Bytes per element of a safetensors dtype name; throws TensorError for an unknown one.
size_t dtype_size(const std::string& dtype);

class SafeFile {
public:
    explicit SafeFile(const std::string& path);
    ~SafeFile();
    SafeFile(const SafeFile&) = delete;
    SafeFile& operator=(const SafeFile&) = delete;
    const std::map<std::string, TensorView>& tensors() const { return tensors_; }

private:
    int fd_ = -1;
    uint8_t* map_ = nullptr;
    size_t size_ = 0;
    std::map<std::string, TensorView> tensors_;
};

class ModelDirectory {
public:
    explicit ModelDirectory(const std::string& directory);
    // The one tensor whose name ends in `suffix`; nullptr if none; TensorError if several.
    const TensorView* maybe_suffix(const std::string& suffix) const;
    const TensorView& suffix(const std::string& suffix) const;

private:
    std::vector<std::unique_ptr<SafeFile>> files_;
    std::map<std::string, const TensorView*> index_;
};

}  // namespace qm_engine
#endif
