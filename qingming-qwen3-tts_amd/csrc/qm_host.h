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

}  // namespace qm
