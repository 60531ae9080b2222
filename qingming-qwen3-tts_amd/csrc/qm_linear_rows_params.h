// qm_linear_rows_params.h — launch parameters shared by the two kernels behind qm_linear_rows / qm_gate_up_swiglu_rows.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qm {

struct LinearRowsParams {
    const uint16_t* input;        // [rows][reduction]
    const uint16_t* weight[2];    // [columns][reduction]; [1] = the up matrix (DUAL)
    const uint16_t* bias;         // [columns] or NULL
    const uint16_t* residual;     // [rows][columns] or NULL
    uint16_t* output;             // [rows][columns]
    int rows, columns, reduction;
    int columns_per_block;        // 8 or 4 (4: the two halves of the block take four token rows each)
    // (matrix cores, few token rows) the reduction cut into reduction_parts pieces, one block each: the fp32 sums of
    // piece z go to partials[z] ([rows][columns]; a gate/up pair: gate plane, then up plane) and a second launch adds the
    // pieces in order and rounds.  1: every block takes the whole reduction and rounds its sums itself.
    int reduction_parts;
    float* partials;
    // (matrix cores, no gate/up pair) up to three linears of the same input in one grid: the column tiles of linear g
    // start at tile group_first_tile[g] (group 0 at 0), and a block of group g > 0 takes weight / bias / output / columns
    // from group_*[g - 1] instead of the fields above.  groups = 1: one linear.
    int groups;
    int group_first_tile[2];
    const uint16_t* group_weight[2];
    const uint16_t* group_bias[2];
    uint16_t* group_output[2];
    int group_columns[2];
};

// The row linears on the matrix cores (qm_linear_rows_mfma.hip).  `dual`: weight[0] / weight[1] are the gate and up
// matrices and the epilogue is SwiGLU.  Needs columns % 128 == 0 and reduction % 128 == 0 (checked by the caller).
int32_t launch_rows_mfma(const LinearRowsParams& prm, bool dual, hipStream_t stream);

// Into how many pieces launch_rows_mfma cuts the reduction when it is given a workspace for the partial sums (a pure
// function of the shape), and the bytes that workspace must hold (0: the shape is not cut).
int rows_mfma_reduction_parts(int rows, int columns, int reduction, bool dual);
size_t rows_mfma_workspace_bytes(int rows, int columns, int reduction, bool dual);

}  // namespace qm
