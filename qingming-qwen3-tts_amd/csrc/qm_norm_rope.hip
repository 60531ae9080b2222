// qm_norm_rope.hip — per-head QK-RMSNorm + RoPE + KV append for gfx950.
//
// One 64-lane wave owns one 128-wide head; lane l holds dimensions l and l+64, which
// are exactly the rotate_half partners, so RoPE needs no cross-lane traffic.  The sum of
// squares is reduced in the order of the reference's 32-lane shuffle trees
// (R17:15059-15148) so that, with a correctly rounded 1/sqrt, every output bit equals the
// CPU restatement of R17:15365-15526.  All bf16 roundings of the reference are kept.
//
// HBM traffic per head: 256 B in, 256 B out (+256 B V in / 256 B V out for K heads);
// the operator is launch-latency bound, not bandwidth bound.

#include "qm_device.h"
#include "qm_host.h"
#include "qm_norm_rope_head.h"

namespace qm {

// grid (q_heads + kv_heads, n_streams), block 64.
__global__ __launch_bounds__(64) void qk_norm_rope_append_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ k, const uint16_t* __restrict__ v,
    const uint16_t* __restrict__ q_norm_w, const uint16_t* __restrict__ k_norm_w,
    const uint16_t* __restrict__ cos_rows, const uint16_t* __restrict__ sin_rows,
    int rope_by_position, uint16_t* __restrict__ q_rotated,
    qm_kv_cache cache, const int32_t* __restrict__ page_table, int max_pages,
    const int32_t* __restrict__ positions, int fixed_position,
    int q_heads, float epsilon, uint32_t* status) {
    request_arguments(q, k, v, q_norm_w, k_norm_w, cos_rows, sin_rows, rope_by_position, q_rotated, cache, page_table, max_pages,
                      positions, fixed_position, q_heads, epsilon, status);
    const int lane = threadIdx.x;
    const int slot = blockIdx.x;
    const int stream = blockIdx.y;
    const bool is_query = slot < q_heads;
    const int head = is_query ? slot : slot - q_heads;
    const int position = positions ? positions[stream] : fixed_position;
    const int32_t* table = page_table ? page_table + static_cast<int64_t>(stream) * max_pages : nullptr;

    // A stream whose slot cannot be addressed is skipped as a whole (query included) so
    // that a bad position never produces a half-updated step.
    if (position < 0 || position / cache.page_size >= max_pages) {
        if (lane == 0 && status) atomicOr(status, QM_STATUS_BAD_POSITION);
        return;
    }
    const int page = position / cache.page_size;
    const int phys = table ? table[page] : page;
    if (phys < 0 || phys >= cache.n_pages) {
        if (lane == 0 && status) atomicOr(status, QM_STATUS_BAD_PAGE);
        return;
    }

    const int64_t rope_row = rope_by_position ? position : stream;
    const uint16_t* cosv = cos_rows + rope_row * kDim;
    const uint16_t* sinv = sin_rows + rope_row * kDim;

    if (is_query) {
        const int64_t base = (static_cast<int64_t>(stream) * q_heads + head) * kDim;
        const HeadPair r = norm_rope_head(q[base + lane], q[base + lane + 64], q_norm_w, cosv, sinv,
                                          epsilon, lane);
        q_rotated[base + lane] = r.lo;
        q_rotated[base + lane + 64] = r.hi;
        return;
    }
    const int64_t base = (static_cast<int64_t>(stream) * cache.kv_heads + head) * kDim;
    const HeadPair r = norm_rope_head(k[base + lane], k[base + lane + 64], k_norm_w, cosv, sinv,
                                      epsilon, lane);
    const int64_t dst = static_cast<int64_t>(phys) * cache.stride_page
                      + static_cast<int64_t>(head) * cache.stride_head
                      + static_cast<int64_t>(position - page * cache.page_size) * kDim;
    cache.k_pool[dst + lane] = r.lo;
    cache.k_pool[dst + lane + 64] = r.hi;
    // V is appended as it is: no norm, no rotation (R17:15515-15524).
    cache.v_pool[dst + lane] = v[base + lane];
    cache.v_pool[dst + lane + 64] = v[base + lane + 64];
}

// Prefill front half: rows*heads independent heads, four per block.
__global__ __launch_bounds__(256) void norm_rope_rows_kernel(
    const uint16_t* __restrict__ in, const uint16_t* __restrict__ norm_w,
    const uint16_t* __restrict__ cos_rows, const uint16_t* __restrict__ sin_rows,
    uint16_t* __restrict__ out, int64_t total_heads, int heads, float epsilon) {
    request_arguments(in, norm_w, cos_rows, sin_rows, out, total_heads, heads, epsilon);
    const int lane = threadIdx.x & 63;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (item >= total_heads) return;
    const int64_t row = item / heads;
    const int64_t base = item * kDim;
    const HeadPair r = norm_rope_head(in[base + lane], in[base + lane + 64], norm_w,
                                      cos_rows + row * kDim, sin_rows + row * kDim, epsilon, lane);
    out[base + lane] = r.lo;
    out[base + lane + 64] = r.hi;
}

// The prompt pass's query and key heads in one grid: item = row * (q_heads + kv_heads) + head, the first q_heads of a
// row its query heads; every head as norm_rope_rows_kernel forms it.
__global__ __launch_bounds__(256) void qk_norm_rope_rows_kernel(
    const uint16_t* __restrict__ q_in, const uint16_t* __restrict__ k_in, const uint16_t* __restrict__ q_norm_w,
    const uint16_t* __restrict__ k_norm_w, const uint16_t* __restrict__ cos_rows, const uint16_t* __restrict__ sin_rows,
    uint16_t* __restrict__ q_out, uint16_t* __restrict__ k_out, int64_t total_heads, int q_heads, int kv_heads, float epsilon) {
    request_arguments(q_in, k_in, q_norm_w, k_norm_w, cos_rows, sin_rows, q_out, k_out, total_heads, q_heads, kv_heads, epsilon);
    const int lane = threadIdx.x & 63;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (item >= total_heads) return;
    const int per_row = q_heads + kv_heads;
    const int64_t row = item / per_row;
    const int head = static_cast<int>(item - row * per_row);
    const bool is_query = head < q_heads;
    const uint16_t* in = is_query ? q_in : k_in;
    uint16_t* out = is_query ? q_out : k_out;
    const int64_t base = is_query ? (row * q_heads + head) * kDim : (row * kv_heads + (head - q_heads)) * kDim;
    const HeadPair r = norm_rope_head(in[base + lane], in[base + lane + 64], is_query ? q_norm_w : k_norm_w,
                                      cos_rows + row * kDim, sin_rows + row * kDim, epsilon, lane);
    out[base + lane] = r.lo;
    out[base + lane + 64] = r.hi;
}

// [rows][kv_heads][128] -> pages; one thread moves 16 bytes of K and 16 bytes of V.
__global__ __launch_bounds__(256) void scatter_kv_kernel(
    const uint16_t* __restrict__ key, const uint16_t* __restrict__ value,
    qm_kv_cache cache, const int32_t* __restrict__ page_table, int max_pages,
    int64_t total_chunks, int first_position, uint32_t* status) {
    request_arguments(key, value, cache, page_table, max_pages, total_chunks, first_position, status);
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= total_chunks) return;
    const int chunk = static_cast<int>(idx & 15);
    const int64_t t = idx >> 4;
    const int head = static_cast<int>(t % cache.kv_heads);
    const int token = first_position + static_cast<int>(t / cache.kv_heads);
    const int page = token / cache.page_size;
    const int phys = page_table ? page_table[page] : page;
    if (phys < 0 || phys >= cache.n_pages) {        // (validated on the host for NULL tables)
        if (status && chunk == 0) atomicOr(status, QM_STATUS_BAD_PAGE);
        return;
    }
    const int64_t dst = static_cast<int64_t>(phys) * cache.stride_page
                      + static_cast<int64_t>(head) * cache.stride_head
                      + static_cast<int64_t>(token - page * cache.page_size) * kDim + chunk * 8;
    const uint4 kv = *reinterpret_cast<const uint4*>(key + idx * 8);
    const uint4 vv = *reinterpret_cast<const uint4*>(value + idx * 8);
    *reinterpret_cast<uint4*>(cache.k_pool + dst) = kv;
    *reinterpret_cast<uint4*>(cache.v_pool + dst) = vv;
}

}  // namespace qm

extern "C" int32_t qm_qk_norm_rope_kv_append(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t q_heads, int32_t cache_position, float epsilon, void* hip_stream) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_row || !sin_row || !q_rotated)
        return QM_ERR_NULL;
    int32_t rc = qm::check_cache(cache, max_pages);
    if (rc != QM_OK) return rc;
    if (q_heads <= 0) return QM_ERR_GEOMETRY;
    // The reference's host-side overflow guard (R17:16844-16847, 17114-17117).
    if (cache_position < 0 || cache_position >= qm::cache_capacity(cache, max_pages))
        return QM_ERR_SLOT_RANGE;
    if (!page_table && cache_position / cache->page_size >= cache->n_pages) return QM_ERR_SLOT_RANGE;
    hipLaunchKernelGGL(qm::qk_norm_rope_append_kernel, dim3(q_heads + cache->kv_heads, 1), dim3(64),
                       0, static_cast<hipStream_t>(hip_stream),
                       q, k, v, q_norm_w, k_norm_w, cos_row, sin_row, 0, q_rotated, *cache,
                       page_table, max_pages, static_cast<const int32_t*>(nullptr), cache_position,
                       q_heads, epsilon, static_cast<uint32_t*>(nullptr));
    return qm::launch_status();
}

extern "C" int32_t qm_qk_norm_rope_kv_append_ragged(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows, int32_t rope_by_position,
    uint16_t* q_rotated,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    const int32_t* positions, int32_t n_streams,
    int32_t q_heads, float epsilon, uint32_t* status_dev, void* hip_stream) {
    if (!q || !k || !v || !q_norm_w || !k_norm_w || !cos_rows || !sin_rows || !q_rotated
        || !positions || !page_table)
        return QM_ERR_NULL;
    int32_t rc = qm::check_cache(cache, max_pages);
    if (rc != QM_OK) return rc;
    if (q_heads <= 0) return QM_ERR_GEOMETRY;
    if (n_streams < 0 || n_streams > 65535) return QM_ERR_ARGUMENT;
    if (n_streams == 0) return QM_OK;
    hipLaunchKernelGGL(qm::qk_norm_rope_append_kernel, dim3(q_heads + cache->kv_heads, n_streams),
                       dim3(64), 0, static_cast<hipStream_t>(hip_stream),
                       q, k, v, q_norm_w, k_norm_w, cos_rows, sin_rows, rope_by_position, q_rotated,
                       *cache, page_table, max_pages, positions, 0, q_heads, epsilon, status_dev);
    return qm::launch_status();
}

extern "C" int32_t qm_norm_rope_rows(
    const uint16_t* in, const uint16_t* norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows,
    uint16_t* out, int32_t rows, int32_t heads, float epsilon, void* hip_stream) {
    if (!in || !cos_rows || !sin_rows || !out) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    if (rows == 0) return QM_OK;
    const int64_t total = static_cast<int64_t>(rows) * heads;
    const int64_t blocks = (total + 3) / 4;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::norm_rope_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream),
                       in, norm_w, cos_rows, sin_rows, out, total, heads, epsilon);
    return qm::launch_status();
}

extern "C" int32_t qm_qk_norm_rope_rows(
    const uint16_t* q_in, const uint16_t* k_in, const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_rows, const uint16_t* sin_rows, uint16_t* q_out, uint16_t* k_out,
    int32_t rows, int32_t q_heads, int32_t kv_heads, float epsilon, void* hip_stream) {
    if (!q_in || !k_in || !cos_rows || !sin_rows || !q_out || !k_out) return QM_ERR_NULL;
    if (rows < 0 || q_heads <= 0 || kv_heads <= 0) return QM_ERR_ARGUMENT;
    if (rows == 0) return QM_OK;
    const int64_t total = static_cast<int64_t>(rows) * (static_cast<int64_t>(q_heads) + kv_heads);
    const int64_t blocks = (total + 3) / 4;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::qk_norm_rope_rows_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream),
                       q_in, k_in, q_norm_w, k_norm_w, cos_rows, sin_rows, q_out, k_out, total, q_heads, kv_heads, epsilon);
    return qm::launch_status();
}

extern "C" int32_t qm_scatter_kv(
    const uint16_t* key, const uint16_t* value,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    int32_t rows, int32_t first_position, uint32_t* status_dev, void* hip_stream) {
    if (!key || !value) return QM_ERR_NULL;
    int32_t rc = qm::check_cache(cache, max_pages);
    if (rc != QM_OK) return rc;
    if (rows < 0 || first_position < 0) return QM_ERR_ARGUMENT;
    if (static_cast<int64_t>(first_position) + rows > qm::cache_capacity(cache, max_pages))
        return QM_ERR_SLOT_RANGE;
    if (!page_table && rows > 0
        && (first_position + rows - 1) / cache->page_size >= cache->n_pages)
        return QM_ERR_SLOT_RANGE;
    if ((reinterpret_cast<uintptr_t>(key) & 15) || (reinterpret_cast<uintptr_t>(value) & 15))
        return QM_ERR_GEOMETRY;
    if (rows == 0) return QM_OK;
    const int64_t chunks = static_cast<int64_t>(rows) * cache->kv_heads * 16;
    const int64_t blocks = (chunks + 255) / 256;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::scatter_kv_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream),
                       key, value, *cache, page_table, max_pages, chunks, first_position, status_dev);
    return qm::launch_status();
}
