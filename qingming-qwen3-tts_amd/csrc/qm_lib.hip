// qm_lib.hip — library identification and error strings of the C ABI.

#include "qm_host.h"

#include <atomic>

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
