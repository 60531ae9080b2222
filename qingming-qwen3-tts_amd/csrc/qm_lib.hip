// qm_lib.hip — library identification and error strings of the C ABI.

#include "qm_device.h"
#include "qm_host.h"

#include <atomic>

namespace qm {

// f2bf (one v_cvt_pk_bf16_f32) against the reference's integer sequence (R17:15040-15056: NaNs quieted, else add 0x7fff +
// the lowest kept bit and shift) for the `count` bit patterns from `first` on; mismatches are counted.
__global__ void bf16_rounding_check_kernel(uint32_t first, uint32_t count, unsigned long long* mismatches) {
    unsigned long long bad = 0;
    for (uint64_t i = static_cast<uint64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count;
         i += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
        const uint32_t bits = first + static_cast<uint32_t>(i);
        uint32_t want = bits;
        if ((bits & 0x7fffffffU) > 0x7f800000U) {
            want = (bits >> 16) | 0x0040U;
        } else {
            want += 0x7fffU + ((bits >> 16) & 1U);
            want >>= 16;
        }
        bad += f2bf(__uint_as_float(bits)) != static_cast<uint16_t>(want);
    }
    if (bad) atomicAdd(mismatches, bad);
}

}  // namespace qm

extern "C" int32_t qm_selftest_bf16_rounding(uint32_t first_bits, uint32_t count, uint64_t* mismatches_dev, void* hip_stream) {
    if (!mismatches_dev) return QM_ERR_NULL;
    if (count == 0) return QM_OK;
    hipLaunchKernelGGL(qm::bf16_rounding_check_kernel, dim3(2048), dim3(256), 0, static_cast<hipStream_t>(hip_stream), first_bits, count,
                       reinterpret_cast<unsigned long long*>(mismatches_dev));
    return qm::launch_status();
}

extern "C" int32_t qm_abi_version(void) { return 2; }

extern "C" const char* qm_target_arch(void) { return "gfx950"; }

extern "C" const char* qm_error_string(int32_t code) {
    switch (code) {
        case QM_OK: return "ok";
        case QM_ERR_NULL: return "required pointer is NULL";
        case QM_ERR_GEOMETRY: return "unsupported head/page geometry or misaligned pointer";
        case QM_ERR_SLOT_RANGE: return "cache position beyond the capacity of the page table";
        case QM_ERR_WORKSPACE: return "workspace missing, misaligned or too small";
        case QM_ERR_ARGUMENT: return "invalid argument";
        case QM_ERR_NO_DEVICE: return "no usable gfx950 device";
        case QM_ERR_STATUS: return "a kernel reported a status bit (bad page, bad position, key-split or frame timeout)";
        default: break;
    }
    if (code <= QM_ERR_HIP_BASE) return hipGetErrorString(static_cast<hipError_t>(QM_ERR_HIP_BASE - code));
    return "unknown error";
}

namespace qm {

namespace {
std::atomic<int32_t> g_options[QM_OPT_COUNT] = {
    {1},   // QM_OPT_PREFILL_SCORE_ROUNDING
    {0},   // QM_OPT_DECODE_TILES_PER_BLOCK (0 = chosen from the problem size)
    {0},   // QM_OPT_PREFILL_KERNEL (0 = interleaved waves, 1 = four uniform waves)
    {0},   // QM_OPT_DECODE_STREAMING_LOADS (0 = chosen from the bytes of context, 1 = plain loads, 2 = non-temporal loads)
    {0},   // QM_OPT_PREDICTOR_LOOP_KERNEL (0 = matrix cores, 1 = the reference's exact summation chain)
    {0},   // QM_OPT_PREDICTOR_FRAME_OPERATORS (0 = the frame's M = 1 steps as one launch, 1 = operator by operator)
    {0},   // QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT (0 = the kernel's own bound)
    {0},   // QM_OPT_LINEAR_ROWS_KERNEL (0 = matrix cores for 16 or more token rows, 1 = always the exact chain)
    {0},   // QM_OPT_TALKER_LAYER_OPERATORS (0 = two launches per layer, 2 = three, 1 = operator by operator)
};

// a thread's own values: -1 = none, the process-wide value applies
struct ThreadOptions {
    int32_t value[QM_OPT_COUNT];
    ThreadOptions() {
        for (int32_t& v : value) v = -1;
    }
};
thread_local ThreadOptions t_options;

int32_t check_option(int32_t option, int32_t value) {
    if (option < 0 || option >= QM_OPT_COUNT) return QM_ERR_ARGUMENT;
    if (value < 0) return QM_ERR_ARGUMENT;
    if (option == QM_OPT_DECODE_TILES_PER_BLOCK && value > 4096) return QM_ERR_ARGUMENT;
    return QM_OK;
}
}  // namespace

int32_t option_value(int32_t option) {
    const int32_t own = t_options.value[option];
    return own >= 0 ? own : g_options[option].load(std::memory_order_relaxed);
}

}  // namespace qm

extern "C" int32_t qm_set_option(int32_t option, int32_t value) {
    const int32_t rc = qm::check_option(option, value);
    if (rc != QM_OK) return rc;
    qm::g_options[option].store(value, std::memory_order_relaxed);
    return QM_OK;
}

extern "C" int32_t qm_set_thread_option(int32_t option, int32_t value) {
    if (value == -1) {                                   // back to the process-wide value
        if (option < 0 || option >= QM_OPT_COUNT) return QM_ERR_ARGUMENT;
        qm::t_options.value[option] = -1;
        return QM_OK;
    }
    const int32_t rc = qm::check_option(option, value);
    if (rc != QM_OK) return rc;
    qm::t_options.value[option] = value;
    return QM_OK;
}

extern "C" int32_t qm_get_option(int32_t option, int32_t* value) {
    if (!value) return QM_ERR_NULL;
    if (option < 0 || option >= QM_OPT_COUNT) return QM_ERR_ARGUMENT;
    *value = qm::option_value(option);
    return QM_OK;
}
