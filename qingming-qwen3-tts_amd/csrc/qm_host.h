// qm_host.h — host-side argument validation shared by the C-ABI entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

#include "../../include/qm_attn.h"

namespace qm {

inline int32_t hip_code(hipError_t e) {
    return e == hipSuccess ? QM_OK : QM_ERR_HIP_BASE - static_cast<int32_t>(e);
}

// Geometry rules of qm_kv_cache; `single_page` relaxes the page_size % 16 rule for the
// reference's flat one-page layout.
inline int32_t check_cache(const qm_kv_cache* c, int32_t max_pages) {
    if (!c) return QM_ERR_NULL;
    if (!c->k_pool || !c->v_pool) return QM_ERR_NULL;
    if (c->head_dim != 128 || c->stride_token != 128) return QM_ERR_GEOMETRY;
    if (c->kv_heads <= 0 || c->page_size <= 0 || c->n_pages <= 0 || max_pages <= 0)
        return QM_ERR_GEOMETRY;
    if ((c->page_size % 16) != 0 && max_pages != 1) return QM_ERR_GEOMETRY;
    if ((c->stride_page % 8) != 0 || (c->stride_head % 8) != 0) return QM_ERR_GEOMETRY;
    if (c->stride_head < 0 || c->stride_page < 0) return QM_ERR_GEOMETRY;
    if ((reinterpret_cast<uintptr_t>(c->k_pool) & 15) || (reinterpret_cast<uintptr_t>(c->v_pool) & 15))
        return QM_ERR_GEOMETRY;
    return QM_OK;
}

inline int64_t cache_capacity(const qm_kv_cache* c, int32_t max_pages) {
    return static_cast<int64_t>(c->page_size) * max_pages;
}

inline int32_t check_group(int32_t q_heads, int32_t kv_heads) {
    if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads) return QM_ERR_GEOMETRY;
    return QM_OK;
}

// Process-wide tuning options (qm_set_option); defined with the library's other global entry points.
int32_t option_value(int32_t option);

// Raises a kernel's dynamic LDS limit once per (kernel, device); safe to call from several host
// threads and for several devices of one process.  `done` is the caller's static table.
constexpr int kMaxDevices = 64;
inline int32_t ensure_dynamic_lds(const void* kernel, int bytes, std::atomic<bool> (&done)[kMaxDevices]) {
    int dev = 0;
    const hipError_t e0 = hipGetDevice(&dev);
    if (e0 != hipSuccess) return hip_code(e0);
    if (dev >= 0 && dev < kMaxDevices && done[dev].load(std::memory_order_acquire)) return QM_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return hip_code(e);
    if (dev >= 0 && dev < kMaxDevices) done[dev].store(true, std::memory_order_release);
    return QM_OK;
}

inline int32_t launch_status() { return hip_code(hipGetLastError()); }

// Whether a kernel all of whose `blocks` blocks must be resident at once (they wait for one another) can be launched
// on `hip_stream`: blocks_per_cu (the occupancy the runtime reports for the kernel) times the compute units the
// stream's kernels may use — the device's, or fewer if the stream was created with a CU mask — must hold them all.
// On a stream that is confined to a part of the chip the blocks left over would never start and the ones running
// would wait for them until their bounded waits give up.  (What other streams' kernels occupy at the moment of the
// launch cannot be asked: such a kernel needs the chip to itself for its duration.)
inline int32_t resident_blocks_fit(void* hip_stream, int device, int blocks_per_cu, int blocks, bool* fits) {
    int compute_units = 0;
    const hipError_t e = hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) return hip_code(e);
    uint32_t mask[32] = {};
    int usable = compute_units;
    if (hipExtStreamGetCUMask(static_cast<hipStream_t>(hip_stream), 32, mask) == hipSuccess) {
        int bits = 0;
        for (int w = 0; w < 32; ++w) bits += __builtin_popcount(mask[w]);
        if (bits > 0 && bits < usable) usable = bits;
    } else {
        (void)hipGetLastError();      // a stream that cannot be asked (mid-capture, say) counts as unmasked
    }
    *fits = static_cast<int64_t>(blocks_per_cu) * usable >= blocks;
    return QM_OK;
}

}  // namespace qm
