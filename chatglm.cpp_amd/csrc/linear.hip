// Linear (chatglm.cpp:418-426) for the projections either side of the attention path: y = x W^T + b with
// W fp16 [out][in] (x rounded to fp16, fp32 accumulation: ggml_mul_mat with an fp16 src0) or fp32.
//
//   gemv_f16_kernel     up to 8 input rows: a bandwidth kernel over W.  A workgroup owns 16 output features,
//                       its 8 waves split the input features; W rows are the A operand of
//                       v_mfma_f32_16x16x32_f16 (16 features x 32 inputs per 16-byte-per-lane load), the
//                       input rows, rounded to fp16 into LDS once per workgroup, are its 16 columns.
//   more rows           a plain GEMM: the rows are rounded to fp16 (round_rows_kernel) and hipBLASLt multiplies
//                       (fp16 x fp16, fp32 accumulation and output, bias in its epilogue).
//   gemm_f16_kernel     the same GEMM for shapes hipBLASLt has no algorithm for: 128 x 128 x 64 tiles of
//                       v_mfma_f32_32x32x16_f16, both operands copied straight from global memory into swizzled,
//                       double-buffered LDS.
//   linear_generic_kernel  any shape, fp32 or fp16 weights: one wave per output element.
#include <hipblaslt/hipblaslt.h>

#include <cstdlib>
#include <mutex>
#include <new>
#include <vector>

#include "glm_attn_internal.h"
#include "glm_block.h"
#include "glm_linear.h"
#include "linear_plan.h"
#include "linear_quant.h"

namespace glm_attn {

namespace {

__device__ inline floatx4 mfma16(half8 a, half8 b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
__device__ inline floatx16 mfma32(half8 a, half8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// ---------------------------------------------------------------- few rows: bandwidth kernel over W

constexpr int GV_WAVES = 8;
constexpr int GV_BATCH = 16;     // 32-input steps a wave keeps in flight (16 x 16 bytes per lane)
constexpr int GV_XPAD = 8;       // halfs added to an input row in LDS: rows 16 bytes apart in the banks

struct GemvArgs {
    const __half *W;
    const float *bias;
    const float *x;
    int rows, K, N, feats;
    float *y;
    // optional work of the same launch (glm_linear_fusion)
    const float *norm_weight;
    float norm_eps;
    const float *up;
    int activation;
    const float *residual;
    float residual_scale;
    // second layer of a gated pair (glm_linear_forward_glu): y = act(x W^T + bias) * (x W2^T + bias2)
    const __half *W2;
    const float *bias2;
};

// A workgroup owns `feats` (<= 16 NBLK) consecutive output features, as NBLK blocks of 16 MFMA rows of which
// the last may be partly used: with feats = ceil(N / CUs) every CU gets the same share of W, which matters
// because the launch is as long as its busiest CU.
//
// PRO: what turns x into the input rows on their way into LDS: nothing, RMSNorm (every workgroup recomputes the
// row's mean square: x comes from L2 and is tiny next to W), or act(x) * up.
//
// GLU (with NBLK = 1): the workgroup streams the same 16 features of two weight tensors, half the loads in flight
// for each, and writes act(gate) * up: BasicGLU::forward's first three nodes (chatglm.cpp:465-473) in one launch.
//
// WAVES: 8, or 16 for launches of one workgroup per CU over long rows (the down projection), which otherwise have
// half the loads in flight per CU that a launch of two resident workgroups per CU has.
template <int NBLK, int PRO, bool GLU, int WAVES = GV_WAVES>
__global__ __launch_bounds__(WAVES * 64, NBLK == 1 ? 4 : 2) void gemv_f16_kernel(GemvArgs a) {
    static_assert(!GLU || NBLK == 1, "a gated pair is one block of each tensor");
    constexpr int NB = GLU ? 2 : NBLK;                    // 16-row blocks of weights per workgroup
    constexpr int BATCH = GLU ? GV_BATCH / 2 : GV_BATCH;  // steps in flight per block
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    __shared__ double sm_red[8][WAVES];  // [input row][wave]
    const int rows = a.rows, K = a.K, N = a.N, feats = a.feats;
    __half *x16 = reinterpret_cast<__half *>(smem);  // [rows][K + GV_XPAD]
    float(*sm_acc)[NB * 16][17] =
        reinterpret_cast<float(*)[NB * 16][17]>(smem + (((size_t)rows * (K + GV_XPAD) * 2 + 15) & ~(size_t)15));

    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    const int j = lane & 15, c = lane >> 4;
    const int f0 = blockIdx.x * feats;
    const int steps = K >> 5;
    const int s_begin = (int)((int64_t)w * steps / WAVES), s_end = (int)((int64_t)(w + 1) * steps / WAVES);
    const int xpitch = K + GV_XPAD;
    bool live[NB];          // this lane's feature of block b exists
    const __half *wrow[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) {
        const int f = GLU ? j : b * 16 + j;
        live[b] = f < feats && f0 + f < N;
        wrow[b] = (GLU && b == 1 ? a.W2 : a.W) + (int64_t)(live[b] ? f0 + f : 0) * K + c * 8;
    }

    // A wave multiplies only its own share of the input features, so it stages only that share of the input rows
    // (rounded to fp16) in LDS and no workgroup barrier stands between its loads and its products.  The loads of
    // the input go out first (they come from L2), the wave's first batch of W right behind them.
    const int k_begin = s_begin * 32, k_len4 = (s_end - s_begin) * 8;  // this wave's inputs: first, count / 4
    const int n4 = rows * k_len4;
    auto load_x = [&](int base, floatx4(&v)[4], floatx4(&v2)[4], int(&off)[4]) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx4 = base + u * 64 + lane;
            const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};
            const int r = idx4 < n4 ? idx4 / k_len4 : -1;
            off[u] = r;
            const int64_t g = (int64_t)r * K + k_begin + (idx4 - r * k_len4) * 4;
            v[u] = r >= 0 ? *reinterpret_cast<const floatx4 *>(a.x + g) : zero4;
            if (PRO == GLM_LINEAR_PRO_GATED_ACT) {
                v2[u] = r >= 0 ? *reinterpret_cast<const floatx4 *>(a.up + g) : zero4;
            }
        }
    };
    auto store_x = [&](int base, const floatx4(&v)[4], const int(&off)[4]) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const int idx4 = base + u * 64 + lane;
            if (off[u] >= 0) {
                const int k = k_begin + (idx4 - off[u] * k_len4) * 4;
                half4 h = {(_Float16)v[u][0], (_Float16)v[u][1], (_Float16)v[u][2], (_Float16)v[u][3]};
                *reinterpret_cast<half4 *>(x16 + off[u] * xpitch + k) = h;
            }
        }
    };
    auto gate_x = [&](floatx4(&v)[4], const floatx4(&v2)[4]) {
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float g = a.activation == GLM_BLOCK_ACT_GELU ? gelu_value(v[u][e]) : silu_value(v[u][e]);
                v[u][e] = __fmul_rn(v2[u][e], g);
            }
        }
    };
    const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    auto load_w = [&](int s0, half8(&wf)[NB][BATCH]) {
#pragma unroll
        for (int b = 0; b < NB; b++) {
#pragma unroll
            for (int i = 0; i < BATCH; i++) {
                if (s0 + i < s_end) {
                    wf[b][i] = live[b] ? *reinterpret_cast<const half8 *>(wrow[b] + (int64_t)(s0 + i) * 32) : zero;
                }
            }
        }
    };
    floatx4 xv[4], xv2[4];
    int row_of[4];  // input row of each of the four loads, -1: none
    load_x(0, xv, xv2, row_of);
    half8 wf[NB][BATCH];
    load_w(s_begin, wf);
    if (PRO == GLM_LINEAR_PRO_RMS_NORM) {
        // The host admits this form only when a wave's share of all rows fits one round of loads (n4 <= 256): the
        // values stay in registers between the sum of squares and the scaling.  The waves' sums of a row meet in
        // LDS: the only workgroup barrier of this prologue.
        for (int r = 0; r < rows; r++) {
            double s2 = 0.0;
#pragma unroll
            for (int u = 0; u < 4; u++) {
                // opaque to the optimiser, which would otherwise compute all squares as doubles ahead of the loop
                // over the rows and keep them in 32 registers that the weights in flight need
                asm volatile("" : "+v"(xv[u]));
                if (row_of[u] == r) {
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        s2 += (double)__fmul_rn(xv[u][e], xv[u][e]);
                    }
                }
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) {
                s2 += __shfl_xor(s2, off);
            }
            if (lane == 0) {
                sm_red[r][w] = s2;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
        // the norm's weights are fetched only now: held across the reduction they would not fit the registers
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (row_of[u] >= 0) {
                double tot = 0.0;
#pragma unroll
                for (int i = 0; i < WAVES; i++) {
                    tot += sm_red[row_of[u]][i];
                }
                const float scale = 1.0f / sqrtf((float)(tot / K) + a.norm_eps);
                int k = k_begin + (u * 64 + lane - row_of[u] * k_len4) * 4;
                asm volatile("" : "+v"(k) : "v"(scale));  // keeps the compiler from hoisting the load
                const floatx4 nw = *reinterpret_cast<const floatx4 *>(a.norm_weight + k);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    xv[u][e] = __fmul_rn(__fmul_rn(xv[u][e], scale), nw[e]);
                }
            }
        }
    }
    if (PRO == GLM_LINEAR_PRO_GATED_ACT) {
        gate_x(xv, xv2);
    }
    store_x(0, xv, row_of);
    for (int base = 256; base < n4; base += 256) {  // not reached with RMS_NORM
        load_x(base, xv, xv2, row_of);
        if (PRO == GLM_LINEAR_PRO_GATED_ACT) {
            gate_x(xv, xv2);
        }
        store_x(base, xv, row_of);
    }
    // the wave reads back what its own lanes wrote: LDS operations of one wave complete in order
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");

    floatx4 acc[NB];
#pragma unroll
    for (int b = 0; b < NB; b++) {
        acc[b] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const __half *xrow = x16 + (j < rows ? j : 0) * xpitch + c * 8;
    for (int s0 = s_begin; s0 < s_end; s0 += BATCH) {
#pragma unroll
        for (int i = 0; i < BATCH; i++) {
            if (s0 + i < s_end) {
                half8 xf = *reinterpret_cast<const half8 *>(xrow + (s0 + i) * 32);
                xf = j < rows ? xf : zero;
#pragma unroll
                for (int b = 0; b < NB; b++) {
                    acc[b] = mfma16(wf[b][i], xf, acc[b]);
                }
            }
        }
        if (s0 + BATCH < s_end) {
            load_w(s0 + BATCH, wf);
        }
    }
    // acc[b][r] = feature 16 b + 4 c + r, input row j, over this wave's share of the input features
#pragma unroll
    for (int b = 0; b < NB; b++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            sm_acc[w][b * 16 + 4 * c + r][j] = acc[b][r];
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    constexpr int NF = GLU ? 16 : NBLK * 16;  // output features of the workgroup
    for (int idx = tid; idx < NF * 16; idx += WAVES * 64) {
        const int f = idx % NF, r = idx / NF;  // consecutive threads: consecutive features of one row
        float sum = 0.f, sum2 = 0.f;
#pragma unroll
        for (int ww = 0; ww < WAVES; ww++) {
            sum += sm_acc[ww][f][r];
            if (GLU) {
                sum2 += sm_acc[ww][16 + f][r];
            }
        }
        if (r < rows && f < feats && f0 + f < N) {
            const int64_t o = (int64_t)r * N + f0 + f;
            float v = a.bias ? sum + a.bias[f0 + f] : sum;
            if (GLU) {
                const float u = a.bias2 ? sum2 + a.bias2[f0 + f] : sum2;
                v = __fmul_rn(u, a.activation == GLM_BLOCK_ACT_GELU ? gelu_value(v) : silu_value(v));
            }
            if (a.residual) {
                v = __fadd_rn(v, __fmul_rn(a.residual[o], a.residual_scale));
            }
            a.y[o] = v;
        }
    }
}

// ---------------------------------------------------------------- many rows: MFMA GEMM

constexpr int GM_TILE = kGemmTile;  // output features and input rows per workgroup
constexpr int GM_K = kGemmK;        // input features per step
constexpr int GM_WAVES = 4;
constexpr int GM_THREADS = GM_WAVES * 64;

// LDS rows of 64 halfs (8 chunks of 16 bytes) are filled by global_load_lds_dwordx4, which rules out row
// padding; chunk c of row r is stored at position c ^ swz(r) instead, which keeps the 16-byte fragment
// reads of a wave off each other's banks.
__device__ inline int gm_swz(int row) { return (row >> 1) & 7; }

// Copies rows row0 .. row0 + 127 (clamped to n_rows - 1), inputs k0 .. k0 + 63 of a [n_rows][K] fp16 matrix.
__device__ inline void gm_fetch(const __half *M, int n_rows, int K, int row0, int k0, int w, int lane,
                                __half (*dst)[GM_K]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int blk = i * GM_WAVES + w;  // 1 KiB of LDS: 8 rows
        const int row = blk * 8 + (lane >> 3), pos = lane & 7;
        int grow = row0 + row;
        grow = grow < n_rows ? grow : n_rows - 1;
        const __half *src = M + (int64_t)grow * K + k0 + (pos ^ gm_swz(row)) * 8;
        __builtin_amdgcn_global_load_lds(src, &dst[blk * 8][0], 16, 0, 0);
    }
}

// x fp32 -> fp16, what ggml_mul_mat does to src1 for an fp16 src0
__global__ void round_rows_kernel(const float *x, __half *x16, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const floatx4 v = *reinterpret_cast<const floatx4 *>(x + i * 4);
        half4 h = {(_Float16)v[0], (_Float16)v[1], (_Float16)v[2], (_Float16)v[3]};
        *reinterpret_cast<half4 *>(x16 + i * 4) = h;
    }
}

// The same pass with the work of the graph node in front of the GEMM folded in: the fp32 result of that node is
// never written, its fp16 rounding (what the GEMM reads) is.  RMSNorm (chatglm.cpp:437-442): one workgroup per row,
// sum of squares in double, (x * scale) * weight.
__global__ __launch_bounds__(256) void rms_rows_f16_kernel(const float *x, const float *weight, float eps, int K,
                                                           __half *x16) {
    __shared__ double sm[4];
    const float *xr = x + (int64_t)blockIdx.x * K;
    __half *o = x16 + (int64_t)blockIdx.x * K;
    const int tid = threadIdx.x;
    double s2 = 0.0;
    for (int i = tid * 4; i < K; i += 1024) {
        const floatx4 v = *reinterpret_cast<const floatx4 *>(xr + i);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            s2 += (double)__fmul_rn(v[e], v[e]);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        s2 += __shfl_xor(s2, off);
    }
    if ((tid & 63) == 0) sm[tid >> 6] = s2;
    __syncthreads();
    const double tot = sm[0] + sm[1] + sm[2] + sm[3];
    const float scale = 1.0f / sqrtf((float)(tot / K) + eps);
    for (int i = tid * 4; i < K; i += 1024) {
        const floatx4 v = *reinterpret_cast<const floatx4 *>(xr + i);
        const floatx4 w = *reinterpret_cast<const floatx4 *>(weight + i);
        half4 h;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            h[e] = (_Float16)__fmul_rn(__fmul_rn(v[e], scale), w[e]);
        }
        *reinterpret_cast<half4 *>(o + i) = h;
    }
}

// act(x) * up, the middle of BasicGLU::forward (chatglm.cpp:465-473), rounded to fp16
__global__ void gated_rows_f16_kernel(const float *x, const float *up, int activation, __half *x16, int64_t n4) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        const floatx4 v = *reinterpret_cast<const floatx4 *>(x + i * 4);
        const floatx4 u = *reinterpret_cast<const floatx4 *>(up + i * 4);
        half4 h;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const float g = activation == GLM_BLOCK_ACT_GELU ? gelu_value(v[e]) : silu_value(v[e]);
            h[e] = (_Float16)__fmul_rn(u[e], g);
        }
        *reinterpret_cast<half4 *>(x16 + i * 4) = h;
    }
}

// Y^T tile = W tile (features on MFMA rows) x X^T tile (input rows on MFMA columns).  Waves: 2 x 2, each
// 64 features x 64 input rows = 2 x 2 blocks of 32 x 32.
// `residual` (or null) has y's shape and may be y itself: a lane reads its 4 values right before it writes the same 4.
// gridDim.z > 1 (a few rows against a weight with too few feature tiles to fill the chip): workgroup z takes share z
// of the input features and leaves its sums, without bias or residual, in part[z][row][feature] for
// splitk_reduce_kernel.
__global__ __launch_bounds__(GM_THREADS, 2) void gemm_f16_kernel(const __half *W, const float *bias, const __half *x16,
                                                                 int rows, int K, int N, float *y, const float *residual,
                                                                 float residual_scale, float *part) {
    __shared__ __attribute__((aligned(1024))) __half Ws[2][GM_TILE][GM_K];
    __shared__ __attribute__((aligned(1024))) __half Xs[2][GM_TILE][GM_K];
    const int tid = threadIdx.x, lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, c = lane >> 5;
    const int wf = w & 1, wr = w >> 1;  // feature half, row half of the tile
    const int f0 = blockIdx.x * GM_TILE, r0 = blockIdx.y * GM_TILE;

    floatx16 acc[2][2];
#pragma unroll
    for (int fb = 0; fb < 2; fb++) {
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                acc[fb][rb][e] = 0.f;
            }
        }
    }
    const int ksplit = gridDim.z, kz = blockIdx.z;
    int step0, step1;
    splitk_step_range(K, ksplit, kz, &step0, &step1);
    const int n_steps = step1 - step0;
    if (n_steps <= 0) {
        return;  // (never: the host gives no share fewer than one step)
    }
    W += step0 * GM_K;
    x16 += step0 * GM_K;
    gm_fetch(W, N, K, f0, 0, w, lane, Ws[0]);
    gm_fetch(x16, rows, K, r0, 0, w, lane, Xs[0]);
    for (int step = 0; step < n_steps; step++) {
        const int buf = step & 1;
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();  // this step's tiles have landed for every wave; nobody reads the other buffer any more
        if (step + 1 < n_steps) {
            gm_fetch(W, N, K, f0, (step + 1) * GM_K, w, lane, Ws[buf ^ 1]);
            gm_fetch(x16, rows, K, r0, (step + 1) * GM_K, w, lane, Xs[buf ^ 1]);
        }
        half8 a[2][4], b[2][4];
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int arow = wf * 64 + h * 32 + n, brow = wr * 64 + h * 32 + n;
#pragma unroll
            for (int ks = 0; ks < 4; ks++) {
                a[h][ks] = *reinterpret_cast<const half8 *>(&Ws[buf][arow][((2 * ks + c) ^ gm_swz(arow)) << 3]);
                b[h][ks] = *reinterpret_cast<const half8 *>(&Xs[buf][brow][((2 * ks + c) ^ gm_swz(brow)) << 3]);
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ks++) {
#pragma unroll
            for (int fb = 0; fb < 2; fb++) {
#pragma unroll
                for (int rb = 0; rb < 2; rb++) {
                    acc[fb][rb] = mfma32(a[fb][ks], b[rb][ks], acc[fb][rb]);
                }
            }
        }
    }
    // acc[fb][rb][4 b + e] = feature f0 + wf*64 + fb*32 + 8 b + 4 c + e, input row r0 + wr*64 + rb*32 + n
#pragma unroll
    for (int rb = 0; rb < 2; rb++) {
        const int row = r0 + wr * 64 + rb * 32 + n;
        if (row < rows) {
#pragma unroll
            for (int fb = 0; fb < 2; fb++) {
#pragma unroll
                for (int b4 = 0; b4 < 4; b4++) {
                    const int f = f0 + wf * 64 + fb * 32 + 8 * b4 + 4 * c;
                    if (f < N) {  // N is a multiple of 4 on this path
                        floatx4 v = {acc[fb][rb][4 * b4], acc[fb][rb][4 * b4 + 1], acc[fb][rb][4 * b4 + 2],
                                     acc[fb][rb][4 * b4 + 3]};
                        if (ksplit > 1) {
                            *reinterpret_cast<floatx4 *>(part + ((int64_t)kz * rows + row) * N + f) = v;
                            continue;
                        }
                        if (bias) {
                            v += *reinterpret_cast<const floatx4 *>(bias + f);
                        }
                        if (residual) {
                            const floatx4 r = *reinterpret_cast<const floatx4 *>(residual + (int64_t)row * N + f);
#pragma unroll
                            for (int e = 0; e < 4; e++) {
                                v[e] = __fadd_rn(v[e], __fmul_rn(r[e], residual_scale));
                            }
                        }
                        *reinterpret_cast<floatx4 *>(y + (int64_t)row * N + f) = v;
                    }
                }
            }
        }
    }
}

// y = sum over the shares of part (in the order of the shares) + bias + residual * scale, four values per thread
__global__ void splitk_reduce_kernel(const float *part, int ksplit, int rows, int N, const float *bias,
                                     const float *residual, float residual_scale, float *y) {
    const int64_t n4 = (int64_t)rows * N / 4;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n4; i += (int64_t)gridDim.x * blockDim.x) {
        floatx4 v = *reinterpret_cast<const floatx4 *>(part + i * 4);
        for (int z = 1; z < ksplit; z++) {
            v += *reinterpret_cast<const floatx4 *>(part + (int64_t)z * rows * N + i * 4);
        }
        if (bias) {
            v += *reinterpret_cast<const floatx4 *>(bias + (i * 4) % N);
        }
        if (residual) {
            const floatx4 r = *reinterpret_cast<const floatx4 *>(residual + i * 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
                v[e] = __fadd_rn(v[e], __fmul_rn(r[e], residual_scale));
            }
        }
        *reinterpret_cast<floatx4 *>(y + i * 4) = v;
    }
}

// ---------------------------------------------------------------- any shape, fp32 or fp16 weights

template <bool F16>
__global__ void linear_generic_kernel(const void *weight, const float *bias, const float *x, int rows, int K, int N,
                                      float *y) {
    const int lane = threadIdx.x & 63;
    const int64_t n_out = (int64_t)rows * N;
    const int64_t wave0 = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int64_t n_waves = ((int64_t)gridDim.x * blockDim.x) >> 6;
    for (int64_t idx = wave0; idx < n_out; idx += n_waves) {
        const int r = (int)(idx / N), o = (int)(idx - (int64_t)r * N);
        float sum = 0.f;
        for (int k = lane; k < K; k += 64) {
            float wv, xv = x[(int64_t)r * K + k];
            if (F16) {
                wv = __half2float(static_cast<const __half *>(weight)[(int64_t)o * K + k]);
                xv = __half2float(__float2half_rn(xv));
            } else {
                wv = static_cast<const float *>(weight)[(int64_t)o * K + k];
            }
            sum = __builtin_fmaf(wv, xv, sum);
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            sum += __shfl_xor(sum, off);
        }
        if (lane == 0) {
            y[idx] = bias ? sum + bias[o] : sum;
        }
    }
}

}  // namespace

}  // namespace glm_attn

// ---------------------------------------------------------------- C ABI

// One hipBLASLt handle and one workspace per device, made at the first glm_linear_create on that device.
struct LtDevice {
    hipblasLtHandle_t handle = nullptr;
    void *workspace = nullptr;
    size_t workspace_bytes = 0;
};
// One staging buffer per device for the inputs rounded to fp16 ahead of a GEMM, as large as the largest
// max_rows x in_features of the layers created on the device so far.  It only grows, at glm_linear_create
// (which synchronises the device), and is kept until the process ends.
struct RowStaging {
    __half *x16 = nullptr;
    size_t bytes = 0;
};
static RowStaging g_staging[64];
// Likewise one fp16 buffer per device that a block-quantised weight is expanded into ahead of a GEMM, as large as
// the largest quantised weight of the layers created on the device so far.
static RowStaging g_dequant[64];
// And one fp32 buffer per device for the shares of a GEMM that is cut along the input features (a few rows
// against a weight with fewer feature tiles than the GPU has CUs): kSplitKMax x 128 rows x out_features.
static RowStaging g_splitk[64];
using glm_attn::kSplitKMax;
static std::mutex g_lt_mutex;
static LtDevice g_lt[64];

struct LtPlan {  // what hipBLASLt needs for one row count
    int rows;
    bool usable;
    hipblasLtMatrixLayout_t lb, lc;
    hipblasLtMatmulAlgo_t algo;
};

struct glm_linear {
    glm_linear_desc desc;
    LtDevice *lt;
    hipblasLtMatmulDesc_t lt_desc;
    hipblasLtMatrixLayout_t lt_la;
    std::vector<LtPlan> plans;
    void *weight;
    float *bias;
    bool owns_weight, owns_bias;
    int num_cus;
    RowStaging *staging;  // the device's staging of the rounded input for the GEMM (max_rows > 8 only)
    bool quant;           // block-quantised weight: `weight` holds ggml blocks until glm_linear_commit
    bool committed;
    glm_attn::QuantPlanes q;
    RowStaging *dequant;  // the device's fp16 expansion buffer (quantised weights only)
    RowStaging *splitk;   // the device's buffer for the shares of a GEMM cut along the input features, or null
    int max_rows;
    int last_hip_error;
};

namespace {

size_t weight_bytes(const glm_linear_desc &d) {
    if (glm_attn::quant_type_known(d.weight_dtype)) {
        return glm_attn::quant_raw_bytes(d.weight_dtype, d.out_features, d.in_features);
    }
    return (size_t)d.in_features * (size_t)d.out_features * (d.weight_dtype == GLM_LINEAR_F16 ? 2 : 4);
}

// grows one of the per-device buffers to `need` bytes; the caller holds g_lt_mutex
// Bytes kept free behind a buffer that becomes an operand of a library GEMM, in case one of its kernels fetches
// ahead of the last tile it uses.
constexpr size_t kOperandSlack = 4096;

hipError_t grow(RowStaging &stg, size_t need) {
    need += kOperandSlack;
    if (need <= stg.bytes) return hipSuccess;
    hipError_t e = hipDeviceSynchronize();  // earlier launches may still read the buffer being replaced
    if (e != hipSuccess) return e;
    if (stg.x16) (void)hipFree(stg.x16);
    stg.x16 = nullptr;
    stg.bytes = 0;
    e = hipMalloc((void **)&stg.x16, need);
    if (e == hipSuccess) stg.bytes = need;
    return e;
}

void free_linear(glm_linear *l) {
    if (!l) return;
    for (LtPlan &p : l->plans) {
        if (p.lb) (void)hipblasLtMatrixLayoutDestroy(p.lb);
        if (p.lc) (void)hipblasLtMatrixLayoutDestroy(p.lc);
    }
    if (l->lt_la) (void)hipblasLtMatrixLayoutDestroy(l->lt_la);
    if (l->lt_desc) (void)hipblasLtMatmulDescDestroy(l->lt_desc);
    if (l->owns_weight && l->weight) (void)hipFree(l->weight);
    if (l->owns_bias && l->bias) (void)hipFree(l->bias);
    if (l->q.levels) (void)hipFree(l->q.levels);
    if (l->q.scales) (void)hipFree(l->q.scales);
    if (l->q.mins) (void)hipFree(l->q.mins);
    delete l;
}

// The device's hipBLASLt handle and workspace, or null: then the library's own GEMM kernel runs, which is the
// default.  hipBLASLt is used only when the environment holds GLM_LINEAR_HIPBLASLT=1 at glm_linear_create: two
// timing programs that drove many-row calls through it ended in GPU memory faults whose cause was never shown.
LtDevice *lt_device(int device) {
    if (device < 0 || device >= 64) return nullptr;
    const char *lt = getenv("GLM_LINEAR_HIPBLASLT");
    if (!lt || lt[0] != '1') return nullptr;
    std::lock_guard<std::mutex> lock(g_lt_mutex);
    LtDevice &d = g_lt[device];
    if (!d.handle) {
        hipblasLtHandle_t h = nullptr;
        if (hipblasLtCreate(&h) != HIPBLAS_STATUS_SUCCESS) return nullptr;
        void *ws = nullptr;
        const size_t bytes = (size_t)32 << 20;
        if (hipMalloc(&ws, bytes) != hipSuccess) {
            (void)hipblasLtDestroy(h);
            return nullptr;
        }
        d.handle = h;
        d.workspace = ws;
        d.workspace_bytes = bytes;
    }
    return &d;
}

// Y^T (N x rows, ld N) = W^T-view * X16: in hipBLASLt's column-major terms A = W as K x N (ld K) transposed,
// B = X16 as K x rows (ld K), C = D = Y as N x rows (ld N); the bias vector runs along D's rows.
bool lt_setup(glm_linear *l) {
    const int K = l->desc.in_features, N = l->desc.out_features;
    if (hipblasLtMatmulDescCreate(&l->lt_desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return false;
    const hipblasOperation_t ta = HIPBLAS_OP_T, tb = HIPBLAS_OP_N;
    bool ok = hipblasLtMatmulDescSetAttribute(l->lt_desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ta, sizeof(ta)) ==
                  HIPBLAS_STATUS_SUCCESS &&
              hipblasLtMatmulDescSetAttribute(l->lt_desc, HIPBLASLT_MATMUL_DESC_TRANSB, &tb, sizeof(tb)) ==
                  HIPBLAS_STATUS_SUCCESS;
    if (ok && l->bias) {
        const hipblasLtEpilogue_t epi = HIPBLASLT_EPILOGUE_BIAS;
        const hipDataType bt = HIP_R_32F;
        const void *bp = l->bias;
        ok = hipblasLtMatmulDescSetAttribute(l->lt_desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epi, sizeof(epi)) ==
                 HIPBLAS_STATUS_SUCCESS &&
             hipblasLtMatmulDescSetAttribute(l->lt_desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bp, sizeof(bp)) ==
                 HIPBLAS_STATUS_SUCCESS &&
             hipblasLtMatmulDescSetAttribute(l->lt_desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bt, sizeof(bt)) ==
                 HIPBLAS_STATUS_SUCCESS;
    }
    ok = ok && hipblasLtMatrixLayoutCreate(&l->lt_la, HIP_R_16F, K, N, K) == HIPBLAS_STATUS_SUCCESS;
    return ok;
}

// The plan for this row count, made on first use (a handful of distinct row counts per model).
LtPlan *lt_plan(glm_linear *l, int rows) {
    for (LtPlan &p : l->plans) {
        if (p.rows == rows) return &p;
    }
    const int K = l->desc.in_features, N = l->desc.out_features;
    LtPlan p;
    p.rows = rows;
    p.usable = false;
    p.lb = p.lc = nullptr;
    if (hipblasLtMatrixLayoutCreate(&p.lb, HIP_R_16F, K, rows, K) == HIPBLAS_STATUS_SUCCESS &&
        hipblasLtMatrixLayoutCreate(&p.lc, HIP_R_32F, N, rows, N) == HIPBLAS_STATUS_SUCCESS) {
        hipblasLtMatmulPreference_t pref = nullptr;
        if (hipblasLtMatmulPreferenceCreate(&pref) == HIPBLAS_STATUS_SUCCESS) {
            const size_t ws = l->lt->workspace_bytes;
            hipblasLtMatmulHeuristicResult_t res;
            int found = 0;
            if (hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &ws, sizeof(ws)) ==
                    HIPBLAS_STATUS_SUCCESS &&
                hipblasLtMatmulAlgoGetHeuristic(l->lt->handle, l->lt_desc, l->lt_la, p.lb, p.lc, p.lc, pref, 1, &res,
                                                &found) == HIPBLAS_STATUS_SUCCESS &&
                found > 0 && res.state == HIPBLAS_STATUS_SUCCESS && res.workspaceSize <= ws) {
                p.algo = res.algo;
                p.usable = true;
            }
            (void)hipblasLtMatmulPreferenceDestroy(pref);
        }
    }
    l->plans.push_back(p);
    return &l->plans.back();
}

}  // namespace

extern "C" {

int glm_linear_create(const glm_linear_desc *desc, glm_linear **out_linear) {
    if (!desc || !out_linear || desc->struct_size != (int32_t)sizeof(glm_linear_desc)) return GLM_ATTN_EINVAL;
    if (desc->in_features <= 0 || desc->out_features <= 0 || desc->max_rows < 0) return GLM_ATTN_EINVAL;
    const bool quant = glm_attn::quant_type_known(desc->weight_dtype);
    if (desc->weight_dtype != GLM_LINEAR_F32 && desc->weight_dtype != GLM_LINEAR_F16 && !quant) return GLM_ATTN_EUNSUPPORTED;
    if (quant && desc->in_features % 32 != 0) return GLM_ATTN_EINVAL;  // ggml's blocks hold 32 inputs
    if (quant && (desc->device < 0 || desc->device >= 64)) return GLM_ATTN_EINVAL;
    if (!desc->use_bias && desc->bias) return GLM_ATTN_EINVAL;
    if (desc->weight_bytes < 0 || (desc->weight_bytes > 0 && !desc->weight)) return GLM_ATTN_EINVAL;
    if (desc->weight && desc->weight_bytes > 0 && (uint64_t)desc->weight_bytes < (uint64_t)weight_bytes(*desc)) {
        return GLM_ATTN_EINVAL;  // the kernels would read past the caller's allocation
    }
    if (hipSetDevice(desc->device) != hipSuccess) return GLM_ATTN_EHIP;
    glm_linear *l = new (std::nothrow) glm_linear();
    if (!l) return GLM_ATTN_ENOMEM;
    l->desc = *desc;
    l->max_rows = desc->max_rows > 0 ? desc->max_rows : 1;
    l->weight = desc->weight;
    l->bias = desc->bias;
    l->owns_weight = l->owns_bias = false;
    l->staging = nullptr;
    l->dequant = nullptr;
    l->splitk = nullptr;
    l->quant = quant;
    l->committed = !quant;
    memset(&l->q, 0, sizeof(l->q));
    l->last_hip_error = 0;
    {
        hipDeviceProp_t prop;
        l->num_cus = hipGetDeviceProperties(&prop, desc->device) == hipSuccess && prop.multiProcessorCount > 0
                         ? prop.multiProcessorCount
                         : 256;
    }
    l->lt = nullptr;
    l->lt_desc = nullptr;
    l->lt_la = nullptr;
#define LINEAR_TRY(expr)                                                        \
    do {                                                                        \
        hipError_t e_ = (expr);                                                 \
        if (e_ != hipSuccess) {                                                 \
            free_linear(l);                                                     \
            return e_ == hipErrorOutOfMemory ? GLM_ATTN_ENOMEM : GLM_ATTN_EHIP; \
        }                                                                       \
    } while (0)
    if (!l->weight) {
        LINEAR_TRY(hipMalloc(&l->weight, weight_bytes(*desc) + kOperandSlack));
        l->owns_weight = true;
        LINEAR_TRY(hipMemset(l->weight, 0, weight_bytes(*desc)));
    }
    if (desc->use_bias && !l->bias) {
        LINEAR_TRY(hipMalloc((void **)&l->bias, sizeof(float) * (size_t)desc->out_features));
        l->owns_bias = true;
        LINEAR_TRY(hipMemset(l->bias, 0, sizeof(float) * (size_t)desc->out_features));
    }
    if (quant) {
        glm_attn::quant_plan(&l->q, desc->weight_dtype, desc->out_features, desc->in_features);
        LINEAR_TRY(hipMalloc((void **)&l->q.levels, glm_attn::quant_levels_bytes(l->q)));
        LINEAR_TRY(hipMemset(l->q.levels, 0, glm_attn::quant_levels_bytes(l->q)));
        LINEAR_TRY(hipMalloc((void **)&l->q.scales, glm_attn::quant_scales_bytes(l->q)));
        LINEAR_TRY(hipMemset(l->q.scales, 0, glm_attn::quant_scales_bytes(l->q)));
        if (desc->weight_dtype == GLM_LINEAR_Q4_1 || desc->weight_dtype == GLM_LINEAR_Q5_1) {
            LINEAR_TRY(hipMalloc((void **)&l->q.mins, glm_attn::quant_scales_bytes(l->q)));
            LINEAR_TRY(hipMemset(l->q.mins, 0, glm_attn::quant_scales_bytes(l->q)));
        }
        LINEAR_TRY(glm_attn::quant_set_attributes());
        std::lock_guard<std::mutex> lock(g_lt_mutex);
        LINEAR_TRY(grow(g_dequant[desc->device], sizeof(__half) * (size_t)desc->out_features * (size_t)desc->in_features));
        l->dequant = &g_dequant[desc->device];
    }
    if (desc->weight_dtype == GLM_LINEAR_F16 || quant) {
        const void *kernels[] = {
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_NONE, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<2, GLM_LINEAR_PRO_NONE, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_RMS_NORM, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<2, GLM_LINEAR_PRO_RMS_NORM, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_GATED_ACT, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<2, GLM_LINEAR_PRO_GATED_ACT, false>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_NONE, true>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_RMS_NORM, true>),
            reinterpret_cast<const void *>(glm_attn::gemv_f16_kernel<1, GLM_LINEAR_PRO_NONE, false, 16>)};
        for (const void *k : kernels) {
            LINEAR_TRY(hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024));
        }
        if (l->max_rows > 8) {
            if (desc->device < 0 || desc->device >= 64) {
                free_linear(l);
                return GLM_ATTN_EINVAL;
            }
            std::lock_guard<std::mutex> lock(g_lt_mutex);
            LINEAR_TRY(grow(g_staging[desc->device], sizeof(__half) * (size_t)l->max_rows * (size_t)desc->in_features));
            l->staging = &g_staging[desc->device];
            if ((desc->out_features + glm_attn::GM_TILE - 1) / glm_attn::GM_TILE < l->num_cus) {
                const size_t r = l->max_rows < glm_attn::GM_TILE ? l->max_rows : glm_attn::GM_TILE;
                LINEAR_TRY(grow(g_splitk[desc->device], sizeof(float) * kSplitKMax * r * (size_t)desc->out_features));
                l->splitk = &g_splitk[desc->device];
            }
        }
    }
    if ((desc->weight_dtype == GLM_LINEAR_F16 || quant) && l->max_rows > 8) {
        // A borrowed fp16 weight goes to hipBLASLt only if the caller has stated a size that leaves the slack an
        // owned weight gets: without it a library kernel that fetches ahead of its last tile would read past the
        // caller's allocation.  (A quantised weight is expanded into the library's own buffer.)
        const bool slack_known = l->owns_weight || quant ||
                                 (uint64_t)desc->weight_bytes >= (uint64_t)weight_bytes(*desc) + kOperandSlack;
        l->lt = slack_known ? lt_device(desc->device) : nullptr;
        if (l->lt && !lt_setup(l)) {
            l->lt = nullptr;
        }
    }
    LINEAR_TRY(hipDeviceSynchronize());
#undef LINEAR_TRY
    *out_linear = l;
    return GLM_ATTN_OK;
}

void glm_linear_destroy(glm_linear *linear) {
    if (!linear) return;
    (void)hipSetDevice(linear->desc.device);
    (void)hipDeviceSynchronize();
    free_linear(linear);
}

int glm_linear_params(const glm_linear *linear, void **weight, float **bias) {
    if (!linear) return GLM_ATTN_EINVAL;
    if (weight) *weight = linear->weight;
    if (bias) *bias = linear->bias;
    return GLM_ATTN_OK;
}

// l2: the up projection of a gated pair (then l is the gate projection), or NULL
static int linear_forward_impl(glm_linear *l, glm_linear *l2, const glm_linear_fusion *fu, const float *x, int32_t rows,
                               float *y, void *stream_) {
    using namespace glm_attn;
    if (!l || !x || !y || rows <= 0) return GLM_ATTN_EINVAL;
    if (rows > l->max_rows) return GLM_ATTN_ERANGE;
    if (l2) {
        if (!fu || l2->desc.in_features != l->desc.in_features || l2->desc.out_features != l->desc.out_features ||
            l2->desc.device != l->desc.device ||
            (fu->activation != GLM_BLOCK_ACT_GELU && fu->activation != GLM_BLOCK_ACT_SILU) ||
            fu->prologue == GLM_LINEAR_PRO_GATED_ACT) {
            return GLM_ATTN_EINVAL;
        }
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int K = l->desc.in_features, N = l->desc.out_features;
    bool need_dequant = false;
    if (l->quant) {
        if (!l->committed) return GLM_ATTN_EINVAL;  // glm_linear_commit has not run
        if (l2 && (!l2->quant || !l2->committed || l2->desc.weight_dtype != l->desc.weight_dtype)) return GLM_ATTN_EINVAL;
        const bool xy_aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y)) & 15) == 0;
        if (xy_aligned && quant_gemv_fits(l->q, rows)) {
            // one token: the integer kernel, with whatever it can take into its launch
            const float *norm_weight = nullptr;
            if (fu) {
                if (fu->struct_size != (int32_t)sizeof(glm_linear_fusion)) return GLM_ATTN_EINVAL;
                if (fu->prologue == GLM_LINEAR_PRO_RMS_NORM) {
                    if (!fu->norm_weight) return GLM_ATTN_EINVAL;
                    norm_weight = fu->norm_weight;
                } else if (fu->prologue == GLM_LINEAR_PRO_GATED_ACT) {
                    return GLM_ATTN_EUNSUPPORTED;  // the gate is taken by glm_linear_forward_glu for these types
                } else if (fu->prologue != GLM_LINEAR_PRO_NONE) {
                    return GLM_ATTN_EINVAL;
                }
                const bool plain = !norm_weight && !l2;  // a residual at most
                if ((!plain && !quant_gemv_fused_fits(rows)) || (reinterpret_cast<uintptr_t>(norm_weight) & 15) != 0) {
                    return GLM_ATTN_EUNSUPPORTED;
                }
            }
            launch_quant_gemv(l->q, l->bias, x, rows, y, fu ? fu->residual : nullptr, fu ? fu->residual_scale : 0.f,
                              norm_weight, fu ? fu->norm_eps : 0.f, l2 ? &l2->q : nullptr, l2 ? l2->bias : nullptr,
                              fu ? fu->activation : 0, l->num_cus, stream);
            const hipError_t qe = hipGetLastError();
            if (qe != hipSuccess) {
                l->last_hip_error = (int)qe;
                return GLM_ATTN_EHIP;
            }
            return GLM_ATTN_OK;
        }
        if (l2) return GLM_ATTN_EUNSUPPORTED;
        // many rows: the weight is expanded to fp16 and the fp16 paths below run on the expansion
        need_dequant = true;
    }
    const void *weight = l->quant ? static_cast<const void *>(l->dequant->x16) : l->weight;
    const bool f16 = l->desc.weight_dtype == GLM_LINEAR_F16 || l->quant;
    bool aligned = ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(y) |
                     reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(l->bias)) & 15) == 0;
    int pro = GLM_LINEAR_PRO_NONE;
    if (fu) {
        if (fu->struct_size != (int32_t)sizeof(glm_linear_fusion)) return GLM_ATTN_EINVAL;
        pro = fu->prologue;
        if (pro == GLM_LINEAR_PRO_RMS_NORM) {
            if (!fu->norm_weight) return GLM_ATTN_EINVAL;
            aligned = aligned && (reinterpret_cast<uintptr_t>(fu->norm_weight) & 15) == 0;
        } else if (pro == GLM_LINEAR_PRO_GATED_ACT) {
            if (!fu->up || (fu->activation != GLM_BLOCK_ACT_GELU && fu->activation != GLM_BLOCK_ACT_SILU)) {
                return GLM_ATTN_EINVAL;
            }
            aligned = aligned && (reinterpret_cast<uintptr_t>(fu->up) & 15) == 0;
        } else if (pro != GLM_LINEAR_PRO_NONE) {
            return GLM_ATTN_EINVAL;
        }
    }
    hipError_t e = hipSuccess;
    const size_t x_lds = (((size_t)rows * (K + GV_XPAD) * 2 + 15) & ~(size_t)15);
    if (l2) {
        aligned = aligned && ((reinterpret_cast<uintptr_t>(l2->weight) | reinterpret_cast<uintptr_t>(l2->bias)) & 15) == 0;
    }
    const bool gemv = !l->quant && f16 && aligned && K % GM_K == 0 && N % 4 == 0 && rows <= 8 && x_lds <= 66 * 1024 &&
                      (!l2 || l2->desc.weight_dtype == GLM_LINEAR_F16);
    // the GEMM takes the prologues as its input-rounding pass and the residual as its C operand
    const bool gemm = !gemv && f16 && aligned && K % GM_K == 0 && N % 4 == 0 && l->staging && !l2 &&
                      (!fu || !fu->residual || (reinterpret_cast<uintptr_t>(fu->residual) & 15) == 0);
    // RMS_NORM in the bandwidth kernel: a wave's share of all rows (at most ceil(K / 32 / waves) steps of 32 a row)
    // in 4 x 64 loads of 4
    if (fu && !gemm &&
        (!gemv || (pro == GLM_LINEAR_PRO_RMS_NORM && (int64_t)rows * ((K / 32 + GV_WAVES - 1) / GV_WAVES) > 32))) {
        return GLM_ATTN_EUNSUPPORTED;
    }
    // the shared per-device buffers hold what this call writes into them (they only grow, at glm_linear_create)
    if (gemm && sizeof(__half) * (size_t)rows * (size_t)K > l->staging->bytes) return GLM_ATTN_ERANGE;
    if (need_dequant && sizeof(__half) * (size_t)N * (size_t)K > l->dequant->bytes) return GLM_ATTN_ERANGE;
    if (need_dequant) {
        launch_dequant_f16(l->q, l->dequant->x16, stream);
    }
    if (gemv) {
        // 16 features per workgroup, unless that leaves a last round of workgroups for a few CUs only:
        // then every CU gets the same number of features (up to 32) in one round
        const int tiles = (N + 15) / 16;
        int feats = 16;
        if (!l2 && tiles > l->num_cus && tiles < 2 * l->num_cus) {
            feats = (N + l->num_cus - 1) / l->num_cus;
        }
        const int n_wg = (N + feats - 1) / feats;
        GemvArgs ga;
        ga.W = static_cast<const __half *>(weight);
        ga.bias = l->bias;
        ga.x = x;
        ga.rows = rows;
        ga.K = K;
        ga.N = N;
        ga.feats = feats;
        ga.y = y;
        ga.norm_weight = fu ? fu->norm_weight : nullptr;
        ga.norm_eps = fu ? fu->norm_eps : 0.f;
        ga.up = fu ? fu->up : nullptr;
        ga.activation = fu ? fu->activation : 0;
        ga.residual = fu ? fu->residual : nullptr;
        ga.residual_scale = fu ? fu->residual_scale : 0.f;
        ga.W2 = l2 ? static_cast<const __half *>(l2->weight) : nullptr;
        ga.bias2 = l2 ? l2->bias : nullptr;
        const int nblk = feats <= 16 ? 1 : 2;
        // one workgroup per CU or less and at least a full batch of loads per wave even at 16 waves
        const bool wide = !l2 && nblk == 1 && pro == GLM_LINEAR_PRO_NONE && n_wg <= l->num_cus &&
                          K / 32 >= 16 * GV_BATCH;
        const int waves = wide ? 16 : GV_WAVES;
        const size_t lds = x_lds + sizeof(float) * waves * (l2 ? 2 : nblk) * 16 * 17;
        const dim3 grid(n_wg), block(waves * 64);
#define GEMV_LAUNCH(NB, PR) hipLaunchKernelGGL((gemv_f16_kernel<NB, PR, false>), grid, block, lds, stream, ga)
        if (l2) {
            if (pro == GLM_LINEAR_PRO_RMS_NORM) {
                hipLaunchKernelGGL((gemv_f16_kernel<1, GLM_LINEAR_PRO_RMS_NORM, true>), grid, block, lds, stream, ga);
            } else {
                hipLaunchKernelGGL((gemv_f16_kernel<1, GLM_LINEAR_PRO_NONE, true>), grid, block, lds, stream, ga);
            }
        } else if (wide) {
            hipLaunchKernelGGL((gemv_f16_kernel<1, GLM_LINEAR_PRO_NONE, false, 16>), grid, block, lds, stream, ga);
        } else if (nblk == 1) {
            if (pro == GLM_LINEAR_PRO_RMS_NORM) GEMV_LAUNCH(1, GLM_LINEAR_PRO_RMS_NORM);
            else if (pro == GLM_LINEAR_PRO_GATED_ACT) GEMV_LAUNCH(1, GLM_LINEAR_PRO_GATED_ACT);
            else GEMV_LAUNCH(1, GLM_LINEAR_PRO_NONE);
        } else {
            if (pro == GLM_LINEAR_PRO_RMS_NORM) GEMV_LAUNCH(2, GLM_LINEAR_PRO_RMS_NORM);
            else if (pro == GLM_LINEAR_PRO_GATED_ACT) GEMV_LAUNCH(2, GLM_LINEAR_PRO_GATED_ACT);
            else GEMV_LAUNCH(2, GLM_LINEAR_PRO_NONE);
        }
#undef GEMV_LAUNCH
    } else if (gemm) {
        const int64_t n4 = (int64_t)rows * K / 4;
        const int blocks = (int)((n4 + 255) / 256 < 2048 ? (n4 + 255) / 256 : 2048);
        if (pro == GLM_LINEAR_PRO_RMS_NORM) {
            hipLaunchKernelGGL(rms_rows_f16_kernel, dim3(rows), dim3(256), 0, stream, x, fu->norm_weight, fu->norm_eps, K,
                               l->staging->x16);
        } else if (pro == GLM_LINEAR_PRO_GATED_ACT) {
            hipLaunchKernelGGL(gated_rows_f16_kernel, dim3(blocks), dim3(256), 0, stream, x, fu->up, fu->activation,
                               l->staging->x16, n4);
        } else {
            hipLaunchKernelGGL(round_rows_kernel, dim3(blocks), dim3(256), 0, stream, x, l->staging->x16, n4);
        }
        const float *residual = fu ? fu->residual : nullptr;
        LtPlan *plan = l->lt ? lt_plan(l, rows) : nullptr;
        bool done = false;
        if (plan && plan->usable) {
            // D = A B + beta C (+ bias): the residual sum is the C operand
            const float alpha = 1.f, beta = residual ? fu->residual_scale : 0.f;
            const void *cmat = residual ? static_cast<const void *>(residual) : static_cast<const void *>(y);
            done = hipblasLtMatmul(l->lt->handle, l->lt_desc, &alpha, weight, l->lt_la, l->staging->x16, plan->lb, &beta,
                                   cmat, plan->lc, y, plan->lc, &plan->algo, l->lt->workspace, l->lt->workspace_bytes,
                                   stream) == HIPBLAS_STATUS_SUCCESS;
            if (!done) {
                plan->usable = false;  // not again for this row count
            }
        }
        if (!done) {
            // One tile of rows against fewer feature tiles than CUs: cut along the input features as well, so
            // that the weight is streamed by the whole chip (a prompt of 20 tokens is bound by that stream).
            const int f_tiles = (N + GM_TILE - 1) / GM_TILE;
            const int ksplit = plan_splitk(rows, N, K, l->num_cus, l->splitk ? l->splitk->bytes : 0);
            const float rscale = residual ? fu->residual_scale : 0.f;
            float *part = ksplit > 1 ? reinterpret_cast<float *>(l->splitk->x16) : nullptr;
            hipLaunchKernelGGL(gemm_f16_kernel, dim3(f_tiles, (rows + GM_TILE - 1) / GM_TILE, ksplit), dim3(GM_THREADS), 0,
                               stream, static_cast<const __half *>(weight), l->bias, l->staging->x16, rows, K, N, y,
                               residual, rscale, part);
            if (ksplit > 1) {
                const int64_t o4 = (int64_t)rows * N / 4;
                const int rb = (int)((o4 + 255) / 256 < 1024 ? (o4 + 255) / 256 : 1024);
                hipLaunchKernelGGL(splitk_reduce_kernel, dim3(rb), dim3(256), 0, stream, part, ksplit, rows, N, l->bias,
                                   residual, rscale, y);
            }
        }
    } else {
        const int64_t n_out = (int64_t)rows * N;
        const int blocks = (int)((n_out + 3) / 4 < 4096 ? (n_out + 3) / 4 : 4096);
        if (f16) {
            hipLaunchKernelGGL(linear_generic_kernel<true>, dim3(blocks), dim3(256), 0, stream, weight, l->bias, x,
                               rows, K, N, y);
        } else {
            hipLaunchKernelGGL(linear_generic_kernel<false>, dim3(blocks), dim3(256), 0, stream, l->weight, l->bias, x,
                               rows, K, N, y);
        }
    }
    e = hipGetLastError();
    if (e != hipSuccess) {
        l->last_hip_error = (int)e;
        return GLM_ATTN_EHIP;
    }
    return GLM_ATTN_OK;
}

int glm_linear_commit(glm_linear *l, void *stream_) {
    if (!l) return GLM_ATTN_EINVAL;
    if (!l->quant) return GLM_ATTN_OK;
    if (!l->weight) return GLM_ATTN_EINVAL;  // the blocks have been released by an earlier commit
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    glm_attn::launch_repack(l->q, l->weight, stream);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
        l->last_hip_error = (int)e;
        return GLM_ATTN_EHIP;
    }
    if (l->owns_weight) {
        (void)hipFree(l->weight);
        l->weight = nullptr;
        l->owns_weight = false;
    }
    l->committed = true;
    return GLM_ATTN_OK;
}

int glm_linear_forward(glm_linear *l, const float *x, int32_t rows, float *y, void *stream) {
    return linear_forward_impl(l, nullptr, nullptr, x, rows, y, stream);
}

int glm_linear_forward_fused(glm_linear *l, const glm_linear_fusion *fusion, const float *x, int32_t rows, float *y,
                             void *stream) {
    if (!fusion) return GLM_ATTN_EINVAL;
    return linear_forward_impl(l, nullptr, fusion, x, rows, y, stream);
}

int glm_linear_forward_glu(glm_linear *gate, glm_linear *up, const glm_linear_fusion *fusion, const float *x,
                           int32_t rows, float *y, void *stream) {
    if (!fusion || !up) return GLM_ATTN_EINVAL;
    return linear_forward_impl(gate, up, fusion, x, rows, y, stream);
}

int glm_linear_last_hip_error(const glm_linear *linear) { return linear ? linear->last_hip_error : 0; }

}  // extern "C"
