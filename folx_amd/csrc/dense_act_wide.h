// Wide dense layer + activation (N > 128): internal interface between the two source files
// behind folx_hip_dense_act_fwdlap.
#pragma once
#include "common.h"

// Workspace the wide path needs, or a negative error code when the shape is not one it takes.
int64_t folx_dense_act_wide_ws_bytes(int64_t R, int32_t P, int32_t K, int32_t N);

int folx_dense_act_wide(hipStream_t st, int32_t act, float param, const float* x, const float* jac, const float* lap,
                        const float* W, const float* bias, float* y, float* y_jac, float* y_lap, int64_t R,
                        int32_t P, int32_t K, int32_t N, void* workspace, int64_t workspace_bytes);
