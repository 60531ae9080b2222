// qm_predictor_layout.hip — the three BHSD layout operators in front of the code predictor's staged
// attention of step 0 (call site R17:13663-13699): transpose [rows][heads][128] -> [heads][rows][128]
// (R17:8366-8400), RoPE over a BHSD tensor (R17:8403-8488) and the copy of BHSD rows into the
// [8][16][128] cache (R17:8491-8529).  A handful of head vectors each: launch latency, nothing else.
//
// One 64-lane wave owns one 128-wide head vector; lane l holds dimensions l and l + 64, the
// rotate_half partners, so RoPE needs no cross-lane traffic (as in qm_norm_rope_head.h).

#include "qm_device.h"
#include "qm_host.h"
#include "qm_norm_rope_head.h"

namespace qm {

constexpr int kPredictorCacheRows = 16;   // kMaxCache, R17:7964
constexpr int kPredictorKvHeads = 8;      // kKvHeads, R17:7956

// item = head * rows + sequence (the reference's index / 128); four items per block.
__global__ __launch_bounds__(256) void predictor_rope_bhsd_kernel(
    const uint16_t* __restrict__ in, const uint16_t* __restrict__ cos_rows,
    const uint16_t* __restrict__ sin_rows, uint16_t* __restrict__ out, int64_t items, int rows) {
    const int lane = threadIdx.x & 63;
    const int64_t item = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (item >= items) return;
    const int64_t sequence = item % rows;
    const int64_t base = item * kDim;
    const HeadPair r = norm_rope_head(in[base + lane], in[base + lane + 64], nullptr,
                                      cos_rows + sequence * kDim, sin_rows + sequence * kDim, 0.0f, lane);
    out[base + lane] = r.lo;
    out[base + lane + 64] = r.hi;
}

// One thread moves 16 bytes.  chunk index = ((head * rows + sequence) * 16 + piece).
__global__ __launch_bounds__(256) void predictor_update_cache_kernel(
    const uint16_t* __restrict__ source, uint16_t* __restrict__ cache, int64_t chunks, int rows, int start) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= chunks) return;
    const int piece = static_cast<int>(idx & 15);
    const int64_t t = idx >> 4;
    const int64_t sequence = t % rows;
    const int64_t head = t / rows;
    const int64_t dst = (head * kPredictorCacheRows + start + sequence) * kDim + piece * 8;
    *reinterpret_cast<uint4*>(cache + dst) = *reinterpret_cast<const uint4*>(source + idx * 8);
}

// chunk index over the BSHD input: ((sequence * heads + head) * 16 + piece).
__global__ __launch_bounds__(256) void predictor_transpose_kernel(
    const uint16_t* __restrict__ in, uint16_t* __restrict__ out, int64_t chunks, int rows, int heads) {
    const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= chunks) return;
    const int piece = static_cast<int>(idx & 15);
    const int64_t t = idx >> 4;
    const int64_t head = t % heads;
    const int64_t sequence = t / heads;
    const int64_t dst = (head * rows + sequence) * kDim + piece * 8;
    *reinterpret_cast<uint4*>(out + dst) = *reinterpret_cast<const uint4*>(in + idx * 8);
}

inline bool misaligned16(const void* a, const void* b) {
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) != 0;
}

}  // namespace qm

extern "C" int32_t qm_predictor_transpose(const uint16_t* input, uint16_t* output, int32_t rows, int32_t heads,
                                          void* hip_stream) {
    if (!input || !output) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    if (input == output) return QM_ERR_ARGUMENT;
    if (qm::misaligned16(input, output)) return QM_ERR_GEOMETRY;
    if (rows == 0) return QM_OK;
    const int64_t chunks = static_cast<int64_t>(rows) * heads * 16;
    const int64_t blocks = (chunks + 255) / 256;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::predictor_transpose_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), input, output, chunks, rows, heads);
    return qm::launch_status();
}

extern "C" int32_t qm_predictor_rope_bhsd(const uint16_t* input, const uint16_t* cos_rows, const uint16_t* sin_rows,
                                          uint16_t* output, int32_t rows, int32_t heads, void* hip_stream) {
    if (!input || !cos_rows || !sin_rows || !output) return QM_ERR_NULL;
    if (rows < 0 || heads <= 0) return QM_ERR_ARGUMENT;
    if (rows == 0) return QM_OK;
    const int64_t items = static_cast<int64_t>(rows) * heads;
    const int64_t blocks = (items + 3) / 4;
    if (blocks > 0x7fffffffLL) return QM_ERR_ARGUMENT;
    hipLaunchKernelGGL(qm::predictor_rope_bhsd_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), input, cos_rows, sin_rows, output, items, rows);
    return qm::launch_status();
}

extern "C" int32_t qm_predictor_update_cache(const uint16_t* source, uint16_t* cache, int32_t rows, int32_t start,
                                             void* hip_stream) {
    if (!source || !cache) return QM_ERR_NULL;
    if (rows < 0 || start < 0) return QM_ERR_ARGUMENT;
    // The reference has no guard here; its callers keep start + rows <= kMaxCache (R17:13593-13596).
    if (static_cast<int64_t>(start) + rows > qm::kPredictorCacheRows) return QM_ERR_SLOT_RANGE;
    if (qm::misaligned16(source, cache)) return QM_ERR_GEOMETRY;
    if (rows == 0) return QM_OK;
    const int64_t chunks = static_cast<int64_t>(qm::kPredictorKvHeads) * rows * 16;
    const int64_t blocks = (chunks + 255) / 256;
    hipLaunchKernelGGL(qm::predictor_update_cache_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(hip_stream), source, cache, chunks, rows, start);
    return qm::launch_status();
}
