// Launch geometry of the many-row GEMM of linear.hip as plain host functions, so that a host test can walk the
// shapes (tests/cpp/test_launch_plans.cpp).
#ifndef GLM_LINEAR_PLAN_H
#define GLM_LINEAR_PLAN_H

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace glm_attn {

constexpr int kGemmTile = 128;  // output features and input rows per workgroup of gemm_f16_kernel
constexpr int kGemmK = 64;      // input features per step
constexpr int kSplitKMax = 8;   // shares of the input features at most

// Steps [*step0, *step1) of kGemmK input features that share kz of ksplit takes: the shares tile [0, K / kGemmK) in
// order, and none is empty as long as ksplit <= K / kGemmK.
__host__ __device__ inline void splitk_step_range(int K, int ksplit, int kz, int *step0, int *step1) {
    const int64_t steps = K / kGemmK;
    *step0 = (int)(steps * kz / ksplit);
    *step1 = (int)(steps * (kz + 1) / ksplit);
}

// Shares of the input features for a call of `rows` rows: more than one only for a single tile of rows against
// fewer feature tiles than the GPU has CUs, and only as many as the scratch (scratch_bytes, fp32 [share][row][feature])
// holds.
inline int plan_splitk(int rows, int N, int K, int num_cus, size_t scratch_bytes) {
    const int f_tiles = (N + kGemmTile - 1) / kGemmTile;
    int ksplit = 1;
    if (rows <= kGemmTile && scratch_bytes > 0 && f_tiles < num_cus) {
        ksplit = num_cus / f_tiles;
        if (ksplit > kSplitKMax) ksplit = kSplitKMax;
        if (ksplit > K / kGemmK) ksplit = K / kGemmK;
        if (ksplit < 1) ksplit = 1;
        if (sizeof(float) * (size_t)ksplit * (size_t)rows * (size_t)N > scratch_bytes) ksplit = 1;
    }
    return ksplit;
}

}  // namespace glm_attn
#endif
