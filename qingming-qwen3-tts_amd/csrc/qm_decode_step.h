// qm_decode_step.h — the fused decode step as the library's other sources launch it: with or without its merge launch.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include "../../include/qm_attn.h"

namespace qm {

constexpr int kDecodeMergeRound = 32;   // split records the merge takes per round of loads

// What a decode step launched without its merge leaves for whoever combines the splits: `splits` records of
// (acc[G][128], max[G], sum[G]) floats per kv head, `max_splits` apart, kv head h at records + h * max_splits * that.
// records == NULL: the context was a single split and the split kernel has written context_out itself.
struct DecodeSplitInfo {
    const float* records;
    int splits;
    int max_splits;
};

// qm_decode_step_fused; with `unmerged` the merge launch is left out and *unmerged says where the records are.
int32_t decode_step(
    const uint16_t* q, const uint16_t* k, const uint16_t* v,
    const uint16_t* q_norm_w, const uint16_t* k_norm_w,
    const uint16_t* cos_row, const uint16_t* sin_row,
    uint16_t* q_rotated_out,
    const qm_kv_cache* cache, const int32_t* page_table, int32_t max_pages,
    uint16_t* context_out,
    int32_t q_heads, int32_t position, int32_t sliding_window, float scale, float epsilon,
    void* workspace, size_t workspace_bytes, uint32_t* status_dev, void* hip_stream, DecodeSplitInfo* unmerged);

}  // namespace qm
