// Read kernels that do nothing but load: what this GPU gives a launch shaped like the decode kernel's
// (one workgroup per CU, every load of the launch issued up front), with the arithmetic, the exchange
// between workgroups and the output taken away; and loops of matrix instructions: what the matrix pipes give
// the prefill kernel.  bench.py --ceiling times them; they are no part of the attention path and are built
// into a library of their own (libglm_bench.so).
#include "glm_attn_internal.h"
#include "glm_bench.h"

namespace glm_attn {
namespace {

constexpr int D = kFastHeadSize;

__device__ inline int tile_key(int T, int rho) { return (T >> 1) * 32 + (rho >> 2) * 8 + (T & 1) * 4 + (rho & 3); }

// One launch reads kvh * L * D * 2 halfs from `base` ([kvh][L][D] then [kvh][D][L], the layout of one
// layer's caches) with grid (L / 256, kvh) and 8 waves per workgroup, 16 loads of 16 bytes per lane.
//   PATTERN 0: the bytes in address order (wave = 16 KiB contiguous).
//   PATTERN 1: as the decode kernel does: waves 0..3 the K rows of one 64-key tile each in MFMA operand
//              order, waves 4..7 the V columns of 32 head dims over the workgroup's 256 keys.
template <int PATTERN>
__global__ __launch_bounds__(512) void read_kernel(const __half *base, int L, int kvh, float *sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, c = lane >> 4;
    const int g = blockIdx.y, split = blockIdx.x;
    half8 r[16];
    if (PATTERN == 0) {
        const __half *p = base + ((int64_t)(g * gridDim.x + split) * 8 + wave) * (16 * 512);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            r[i] = *reinterpret_cast<const half8 *>(p + i * 512 + lane * 8);
        }
    } else {
        const __half *Kg = base + (int64_t)g * L * D;
        const __half *Vg = base + (int64_t)kvh * L * D + (int64_t)g * D * L;
        if (wave < 4) {
            const int key0 = (split * 4 + wave) * 64;
#pragma unroll
            for (int T = 0; T < 4; T++) {
                const __half *row = Kg + (int64_t)(key0 + tile_key(T, j)) * D + c * 8;
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    r[T * 4 + t] = *reinterpret_cast<const half8 *>(row + t * 32);
                }
            }
        } else {
            const int w = wave - 4, key0 = split * 256;
#pragma unroll
            for (int jb = 0; jb < 2; jb++) {
                const __half *row = Vg + (int64_t)(w * 32 + jb * 16 + j) * L;
#pragma unroll
                for (int ks = 0; ks < 8; ks++) {
                    r[jb * 8 + ks] = *reinterpret_cast<const half8 *>(row + key0 + ks * 32 + c * 8);
                }
            }
        }
    }
    half8 acc = r[0];
#pragma unroll
    for (int i = 1; i < 16; i++) {
        acc += r[i];
    }
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e++) {
        s += (float)acc[e];
    }
    if (s == 123456.75f) {
        sink[0] = s;  // never: keeps the loads alive
    }
}

// One launch over the whole buffer, eight loads in flight per lane.
__global__ __launch_bounds__(256) void stream_kernel(const uint4 *p, size_t n16, float *sink) {
    uint4 acc = {0u, 0u, 0u, 0u};
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i + 7 * stride < n16; i += 8 * stride) {
        uint4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            v[u] = p[i + u * stride];
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            acc.x ^= v[u].x;
            acc.y ^= v[u].y;
            acc.z ^= v[u].z;
            acc.w ^= v[u].w;
        }
    }
    for (; i < n16; i += stride) {
        acc.x ^= p[i].x;
    }
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345679u) {
        sink[0] = 1.f;  // practically never: keeps the loads alive
    }
}

__global__ void empty_kernel(float *sink, int never) {
    if (never == 12345 && threadIdx.x == 77) {
        sink[0] = 1.f;
    }
}

// ---- the same bytes asked for in other ways: what shape of launch, how many loads in flight per wave and
// which cache policy bits read fastest.  One launch reads `bytes` contiguous bytes with bytes / (W * NL KiB)
// workgroups of W waves, every lane NL loads of 16 bytes, all issued before the one wait.
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

// POL 0: plain, 1: nt (non-temporal), 2: sc1, 3: sc0 sc1 nt.  The result register of every load is used after
// the wait in the kernel, so it stays reserved while the load is on its way.
template <int POL>
__device__ inline void ld_policy(uintx4 &r, const void *p) {
    if (POL == 0) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(r) : "v"(p) : "memory");
    if (POL == 1) asm volatile("global_load_dwordx4 %0, %1, off nt" : "=v"(r) : "v"(p) : "memory");
    if (POL == 2) asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(r) : "v"(p) : "memory");
    if (POL == 3) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1 nt" : "=v"(r) : "v"(p) : "memory");
}

template <int POL, int W, int NL>
__global__ __launch_bounds__(W * 64) void sweep_kernel(const char *base, float *sink) {
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    uintx4 r[NL];
    const char *p = base + (size_t)blockIdx.x * (W * NL * 1024) + (size_t)w * (NL * 1024) + lane * 16;
#pragma unroll
    for (int i = 0; i < NL; i++) {
        ld_policy<POL>(r[i], p + i * 1024);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    unsigned int acc = 0;
#pragma unroll
    for (int i = 0; i < NL; i++) {
        asm volatile("" : "+v"(r[i]));
        acc ^= r[i][0] ^ r[i][1] ^ r[i][2] ^ r[i][3];
    }
    if (acc == 0x12345679u) {
        sink[0] = 1.f;  // practically never: keeps the loads alive
    }
}

// The same through LDS: global_load_lds_dwordx4 drops the 64 lanes' 16 bytes at consecutive LDS addresses and
// needs no registers.  W * NL KiB of LDS per workgroup.  POL 0: plain, 1: nt.
template <int POL, int W, int NL>
__global__ __launch_bounds__(W * 64) void sweep_lds_kernel(const char *base, float *sink) {
    extern __shared__ char lds[];
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const char *p = base + (size_t)blockIdx.x * (W * NL * 1024) + (size_t)w * (NL * 1024);
    const uint32_t lds0 = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds) + w * NL * 1024;
#pragma unroll
    for (int i = 0; i < NL; i++) {
        const uint32_t dst = lds0 + i * 1024;
        const uint32_t off = i * 1024 + lane * 16;
        if (POL == 0) {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         : : "s"(dst), "v"(off), "s"(p) : "memory");
        } else {
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                         : : "s"(dst), "v"(off), "s"(p) : "memory");
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const unsigned int acc = *reinterpret_cast<unsigned int *>(lds + threadIdx.x * 4);
    if (acc == 0x12345679u) {
        sink[0] = 1.f;  // practically never
    }
}

template <int POL, int W, int NL>
hipError_t launch_sweep(const char *base, size_t bytes, float *sink, hipStream_t st) {
    hipLaunchKernelGGL((sweep_kernel<POL, W, NL>), dim3((unsigned int)(bytes / ((size_t)W * NL * 1024))), dim3(W * 64), 0,
                       st, base, sink);
    return hipGetLastError();
}
template <int POL, int W, int NL>
hipError_t launch_sweep_lds(const char *base, size_t bytes, float *sink, hipStream_t st) {
    constexpr int kLds = W * NL * 1024;
    static bool raised = false;  // more than 64 KiB of LDS wants the limit raised once
    if (!raised) {
        hipError_t e = hipFuncSetAttribute((const void *)sweep_lds_kernel<POL, W, NL>,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, kLds);
        if (e != hipSuccess) return e;
        raised = true;
    }
    hipLaunchKernelGGL((sweep_lds_kernel<POL, W, NL>), dim3((unsigned int)(bytes / ((size_t)W * NL * 1024))), dim3(W * 64),
                       kLds, st, base, sink);
    return hipGetLastError();
}
template <int POL>
hipError_t launch_sweep_shape(int waves, int loads, int through_lds, const char *base, size_t bytes, float *sink,
                              hipStream_t st, bool *known) {
    *known = true;
    if (through_lds) {
        constexpr int P2 = POL > 1 ? 0 : POL;
        if (POL > 1) {
            *known = false;
            return hipSuccess;
        }
        if (waves == 8 && loads == 16) return launch_sweep_lds<P2, 8, 16>(base, bytes, sink, st);
        if (waves == 4 && loads == 16) return launch_sweep_lds<P2, 4, 16>(base, bytes, sink, st);
        if (waves == 4 && loads == 32) return launch_sweep_lds<P2, 4, 32>(base, bytes, sink, st);
        *known = false;
        return hipSuccess;
    }
    if (waves == 8 && loads == 16) return launch_sweep<POL, 8, 16>(base, bytes, sink, st);
    if (waves == 4 && loads == 16) return launch_sweep<POL, 4, 16>(base, bytes, sink, st);
    if (waves == 4 && loads == 32) return launch_sweep<POL, 4, 32>(base, bytes, sink, st);
    if (waves == 16 && loads == 8) return launch_sweep<POL, 16, 8>(base, bytes, sink, st);
    if (waves == 8 && loads == 8) return launch_sweep<POL, 8, 8>(base, bytes, sink, st);
    if (waves == 4 && loads == 8) return launch_sweep<POL, 4, 8>(base, bytes, sink, st);
    if (waves == 16 && loads == 16) return launch_sweep<POL, 16, 16>(base, bytes, sink, st);
    *known = false;
    return hipSuccess;
}

}  // namespace
}  // namespace glm_attn

using namespace glm_attn;

namespace glm_attn {
namespace {

// Loops of nothing but matrix instructions on operands with random bits, two waves per SIMD on every CU:
// what the matrix pipes of this GPU sustain at the clock its power management grants them.
//   SHAPE 0: v_mfma_f32_32x32x16_f16, four independent accumulators
//   SHAPE 1: v_mfma_f32_16x16x32_f16, eight independent accumulators
//   MIX    : the attention kernel's diet beside them: one 16-byte-per-lane LDS read per matrix instruction's
//            worth of 32x32x16 work, and per four such instructions 21 vector instructions, 4 of them v_exp_f32
template <int SHAPE, int MIX>
__global__ __launch_bounds__(256, 2) void mfma_loop_kernel(const half8 *in, float *sink, int iters) {
    __shared__ half8 lds[2048];  // 32 KiB
    for (int i = threadIdx.x; i < 2048; i += 256) {
        lds[i] = in[i];
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    half8 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        a[i] = in[i * 64 + lane];
        b[i] = in[256 + i * 64 + lane];
    }
    floatx16 c32[4];
    floatx4 c16[8];
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            c32[i][r] = 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        c16[i] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        v[i] = (float)in[512 + lane][i];
    }
    int at = lane;
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int g = 0; g < 8; g++) {
            if (MIX) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    a[i] = lds[(at + g * 64 + i * 512) & 2047];
                }
            }
            if (SHAPE == 0) {
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    c32[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[i], b[i], c32[i], 0, 0, 0);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    c16[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[i >> 1], b[(i & 1) * 2 + (i >> 2)], c16[i], 0, 0, 0);
                }
            }
            if (MIX) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = __builtin_fmaf(v[e], 1.4426950f, -v[e + 4]);
                    x = __builtin_amdgcn_exp2f(x);
                    v[e + 4] = fmaxf(v[e + 4], x) * 0.5f;
                    v[e] = __builtin_fmaf(v[e], 0.999f, x) + 0.001f;
                }
            }
        }
        at += 7;
    }
    float acc = 0.f;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        acc += v[i] + c16[i][0] + c16[i][1] + c16[i][2] + c16[i][3];
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            acc += c32[i][r];
        }
    }
    if (acc == 12345.678f) {
        *sink = acc;
    }
}

}  // namespace
}  // namespace glm_attn

extern "C" int glm_bench_mfma(int pattern, const void *operands, size_t operand_bytes, int32_t iters, float *sink,
                              void *stream, double *flops) {
    using namespace glm_attn;
    if (!operands || !sink || iters <= 0 || operand_bytes < 2048 * sizeof(half8)) return GLM_ATTN_EINVAL;
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
        return GLM_ATTN_EHIP;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half8 *in = static_cast<const half8 *>(operands);
    const dim3 grid(2 * cus), block(256);
    switch (pattern) {
    case GLM_BENCH_MFMA_32X32X16:
        hipLaunchKernelGGL((mfma_loop_kernel<0, 0>), grid, block, 0, st, in, sink, iters);
        break;
    case GLM_BENCH_MFMA_16X16X32:
        hipLaunchKernelGGL((mfma_loop_kernel<1, 0>), grid, block, 0, st, in, sink, iters);
        break;
    case GLM_BENCH_MFMA_32X32X16_MIX:
        hipLaunchKernelGGL((mfma_loop_kernel<0, 1>), grid, block, 0, st, in, sink, iters);
        break;
    case GLM_BENCH_MFMA_16X16X32_MIX:
        hipLaunchKernelGGL((mfma_loop_kernel<1, 1>), grid, block, 0, st, in, sink, iters);
        break;
    default:
        return GLM_ATTN_EINVAL;
    }
    if (flops) {
        // per wave and iteration: 8 groups of 4 x 32x32x16 (or 8 x 16x16x32) = 8 x 131072 multiply-adds x 2
        *flops = (double)grid.x * 4.0 * iters * 8.0 * 4.0 * 32.0 * 32.0 * 16.0 * 2.0;
    }
    return hipGetLastError() == hipSuccess ? GLM_ATTN_OK : GLM_ATTN_EHIP;
}

extern "C" int glm_bench_read_sweep(int policy, int32_t waves, int32_t loads, int32_t through_lds, const void *base,
                                    size_t bytes, float *sink, void *stream) {
    if (!base || !sink || waves <= 0 || loads <= 0) return GLM_ATTN_EINVAL;
    const size_t per_wg = (size_t)waves * loads * 1024;
    if (bytes < per_wg || bytes % per_wg != 0 || bytes / per_wg > 0x7fffffffu) return GLM_ATTN_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const char *b = static_cast<const char *>(base);
    bool known = false;
    hipError_t e = hipSuccess;
    switch (policy) {
    case GLM_BENCH_POLICY_PLAIN:
        e = launch_sweep_shape<0>(waves, loads, through_lds, b, bytes, sink, st, &known);
        break;
    case GLM_BENCH_POLICY_NT:
        e = launch_sweep_shape<1>(waves, loads, through_lds, b, bytes, sink, st, &known);
        break;
    case GLM_BENCH_POLICY_SC1:
        e = launch_sweep_shape<2>(waves, loads, through_lds, b, bytes, sink, st, &known);
        break;
    case GLM_BENCH_POLICY_SC0_SC1_NT:
        e = launch_sweep_shape<3>(waves, loads, through_lds, b, bytes, sink, st, &known);
        break;
    default:
        return GLM_ATTN_EINVAL;
    }
    if (!known) return GLM_ATTN_EUNSUPPORTED;
    return e == hipSuccess ? GLM_ATTN_OK : GLM_ATTN_EHIP;
}

extern "C" int glm_bench_read(int pattern, const void *base, int32_t cache_rows, int32_t kv_heads, size_t bytes,
                              float *sink, void *stream) {
    if (!base || !sink) return GLM_ATTN_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    switch (pattern) {
    case GLM_BENCH_READ_LINEAR:
    case GLM_BENCH_READ_DECODE_PATTERN: {
        if (cache_rows <= 0 || cache_rows % 256 || kv_heads <= 0) return GLM_ATTN_EINVAL;
        if (bytes < (size_t)2 * kv_heads * cache_rows * D * sizeof(__half)) return GLM_ATTN_ERANGE;
        const dim3 grid(cache_rows / 256, kv_heads), block(512);
        if (pattern == GLM_BENCH_READ_LINEAR) {
            hipLaunchKernelGGL(read_kernel<0>, grid, block, 0, st, static_cast<const __half *>(base), cache_rows,
                               kv_heads, sink);
        } else {
            hipLaunchKernelGGL(read_kernel<1>, grid, block, 0, st, static_cast<const __half *>(base), cache_rows,
                               kv_heads, sink);
        }
        break;
    }
    case GLM_BENCH_READ_STREAM:
        if (bytes < 16) return GLM_ATTN_EINVAL;
        hipLaunchKernelGGL(stream_kernel, dim3(4096), dim3(256), 0, st, static_cast<const uint4 *>(base), bytes / 16,
                           sink);
        break;
    case GLM_BENCH_EMPTY:
        hipLaunchKernelGGL(empty_kernel, dim3(256), dim3(512), 0, st, sink, 0);
        break;
    default:
        return GLM_ATTN_EINVAL;
    }
    return hipGetLastError() == hipSuccess ? GLM_ATTN_OK : GLM_ATTN_EHIP;
}
