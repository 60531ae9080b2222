// qm_predictor_params.h — launch parameters shared by the two kernels of the code predictor's attention loop.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qm {

constexpr int kPredRows = 16;     // kMaxCache of the reference (R17:7963)
constexpr int kPredThreads = 256;

struct PredictorParams {
    const uint16_t* q;        // [units][rows][16][128]
    const uint16_t* k;        // [units][rows][8][128]
    const uint16_t* v;        // [units][rows][8][128]
    const uint16_t* q_norm_w; // [n_layers][128]
    const uint16_t* k_norm_w; // [n_layers][128]
    const uint16_t* cos_rows; // [rows][128]
    const uint16_t* sin_rows; // [rows][128]
    uint16_t* out;            // [units][rows][16][128]
    uint16_t* k_cache_out;    // [units][8][16][128] or NULL
    uint16_t* v_cache_out;    // [units][8][16][128] or NULL
    int64_t unit_base;        // index of the first unit of this launch (layer = unit % n_layers)
    int n_layers;
    int rows;
    float epsilon;
    // STAGED mode (the reference's six-kernel attention, R17:13300-13386): q is already rotated and
    // laid out [16][rows][128]; k, v point at the [8][16][128] caches; row r sees the keys
    // j < key_length with (causal ? j <= r : true).
    int key_length;
    int causal;
};

// The loop on the matrix cores (qm_predictor_mfma.hip): one launch for all `units`.
int32_t launch_predictor_loop_mfma(const PredictorParams& prm, int64_t units, hipStream_t stream);

}  // namespace qm
