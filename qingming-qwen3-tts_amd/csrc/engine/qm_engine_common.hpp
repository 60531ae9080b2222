// qm_engine_common.hpp — what the engine shell's translation units share: constants of the model family,
// error plumbing of the C ABI, the owner of a device allocation and a BF16 tensor on the device.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../../include/qm_attn.h"
#include "../../../include/qm_engine.h"
#include "qm_safetensors.hpp"

namespace qm_engine {

constexpr int kHidden = 2048;          // R17:14625
constexpr int kHeadDim = 128;          // kHeadDimRequired, R17:14629
constexpr float kEpsilon = 1.0e-6f;    // kRmsEpsilon, R17:7965
constexpr float kScale = 0.08838834764831845f;   // 1 / sqrt(128), R17:7966

struct ApiError : std::runtime_error {
    int32_t code;
    ApiError(int32_t c, const std::string& what) : std::runtime_error(what), code(c) {}
};

// text of the calling thread's last failure (qm_engine_last_error)
std::string& last_error();

inline void hip_check(hipError_t e, const char* what) {
    if (e != hipSuccess) throw ApiError(QM_ERR_HIP_BASE - static_cast<int32_t>(e), std::string(what) + ": " + hipGetErrorString(e));
}
inline void op_check(int32_t rc, const char* what) {
    if (rc != QM_OK) throw ApiError(rc, std::string(what) + ": " + qm_error_string(rc));
}

// Owner of one device allocation (DeviceBuffer, R17:7968-8020).
class DeviceBuffer {
public:
    DeviceBuffer() = default;
    explicit DeviceBuffer(size_t bytes) : bytes_(bytes) {
        if (bytes) hip_check(hipMalloc(&pointer_, bytes), "device allocation");
    }
    ~DeviceBuffer() {
        if (pointer_) (void)hipFree(pointer_);
    }
    DeviceBuffer(DeviceBuffer&& o) noexcept : pointer_(o.pointer_), bytes_(o.bytes_) { o.pointer_ = nullptr; o.bytes_ = 0; }
    DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
        if (this != &o) {
            if (pointer_) (void)hipFree(pointer_);
            pointer_ = o.pointer_; bytes_ = o.bytes_;
            o.pointer_ = nullptr; o.bytes_ = 0;
        }
        return *this;
    }
    DeviceBuffer(const DeviceBuffer&) = delete;
    DeviceBuffer& operator=(const DeviceBuffer&) = delete;
    uint16_t* u16() const { return static_cast<uint16_t*>(pointer_); }
    void* raw() const { return pointer_; }
    size_t bytes() const { return bytes_; }

private:
    void* pointer_ = nullptr;
    size_t bytes_ = 0;
};

// A BF16 tensor on the device (GpuParam, R17:14639-14683); absent optional tensors give nullptr.
struct Param {
    DeviceBuffer buffer;
    std::vector<int64_t> shape;
    bool present = false;
    Param() = default;
    Param(const TensorView& t, hipStream_t upload) : buffer(static_cast<size_t>(t.elements()) * 2), shape(t.shape), present(true) {
        if (t.dtype != "BF16") throw TensorError("expected BF16 tensor: " + t.name);
        hip_check(hipMemcpyAsync(buffer.raw(), t.data, buffer.bytes(), hipMemcpyHostToDevice, upload), "weight upload");
    }
    const uint16_t* data() const { return present ? buffer.u16() : nullptr; }
};

// Declared after the object that owns the mapped checkpoint files and therefore destroyed before it, also when an
// exception unwinds: the uploads still in flight on the stream read from those mappings.
struct StreamDrain {
    hipStream_t stream;
    explicit StreamDrain(hipStream_t s) : stream(s) {}
    StreamDrain(const StreamDrain&) = delete;
    StreamDrain& operator=(const StreamDrain&) = delete;
    ~StreamDrain() { (void)hipStreamSynchronize(stream); }
};

// Runs f, turning exceptions into codes.
template <typename F>
inline int32_t guarded(F&& f) {
    try {
        f();
        return QM_OK;
    } catch (const ApiError& e) {
        last_error() = e.what();
        return e.code;
    } catch (const IoError& e) {
        last_error() = e.what();
        return QM_ERR_IO;
    } catch (const TensorError& e) {
        last_error() = e.what();
        return QM_ERR_TENSOR;
    } catch (const std::exception& e) {
        last_error() = e.what();
        return QM_ERR_ARGUMENT;
    }
}

}  // namespace qm_engine
