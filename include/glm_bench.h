/*
 * Measurement aids for `bench.py --ceiling`, in a library of their own (libglm_bench.so; the drop-in library
 * libglm_attn.so exports none of them).  They have no counterpart in the reference
 * and are no part of the attention path: kernels that only load, shaped like a launch of the decode
 * kernel, so that the read rate this GPU gives such a launch can be measured beside the kernel's own, and
 * loops of matrix instructions, so that what the matrix pipes sustain can be measured beside the prefill kernel.
 */
#ifndef GLM_BENCH_H
#define GLM_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum glm_bench_pattern {
    GLM_BENCH_READ_LINEAR = 0,         /* one layer's caches (2 kv_heads cache_rows 128 halfs) in address order */
    GLM_BENCH_READ_DECODE_PATTERN = 1, /* the same bytes as the decode kernel asks for them: K rows, V columns */
    GLM_BENCH_READ_STREAM = 2,         /* `bytes` bytes in one long launch */
    GLM_BENCH_EMPTY = 3                /* a launch of 256 workgroups that does nothing */
};

/* Launches one read kernel on `stream` (hipStream_t).  For patterns 0 and 1 `base` is a device buffer laid
   out like one layer's caches ([kv_heads][cache_rows][128] then [kv_heads][128][cache_rows], fp16), cache_rows
   a multiple of 256, and `bytes` its size; one workgroup of 8 waves per 256 cache rows and KV head.
   `sink` is a device float that is never written in practice.  Returns a glm_attn status. */
int glm_bench_read(int pattern, const void *base, int32_t cache_rows, int32_t kv_heads, size_t bytes, float *sink,
                   void *stream);

enum glm_bench_policy {
    GLM_BENCH_POLICY_PLAIN = 0,     /* global_load_dwordx4 */
    GLM_BENCH_POLICY_NT = 1,        /* ... nt: non-temporal, the lines are not kept in the caches */
    GLM_BENCH_POLICY_SC1 = 2,       /* ... sc1: performed at the device's coherence point */
    GLM_BENCH_POLICY_SC0_SC1_NT = 3 /* ... sc0 sc1 nt */
};

/* Launches one read of `bytes` contiguous bytes at `base` (device) with bytes / (waves x loads KiB) workgroups of
   `waves` waves, every lane `loads` loads of 16 bytes issued up front under the given policy; through_lds != 0:
   the loads go straight to LDS (global_load_lds_dwordx4; policies PLAIN and NT).  `bytes` must be a multiple of
   waves x loads KiB.  GLM_ATTN_EUNSUPPORTED for a (waves, loads) pair the library has no kernel for: it has
   (8,16) (4,16) (4,32) (16,8) (8,8) (4,8) (16,16), through LDS (8,16) (4,16) (4,32). */
int glm_bench_read_sweep(int policy, int32_t waves, int32_t loads, int32_t through_lds, const void *base, size_t bytes,
                         float *sink, void *stream);

enum glm_bench_mfma_pattern {
    GLM_BENCH_MFMA_32X32X16 = 0,     /* nothing but v_mfma_f32_32x32x16_f16, two waves per SIMD on every CU */
    GLM_BENCH_MFMA_16X16X32 = 1,     /* nothing but v_mfma_f32_16x16x32_f16 */
    GLM_BENCH_MFMA_32X32X16_MIX = 2, /* with the attention kernel's diet beside them: an LDS read of 16 bytes per
                                        lane per 32x32x16 and 21 vector instructions (4 v_exp_f32) per four */
    GLM_BENCH_MFMA_16X16X32_MIX = 3
};

/* Launches one loop of matrix instructions on `stream`: 2 workgroups of 4 waves per CU, `iters` iterations of
   32 32x32x16 (or 64 16x16x32) instructions per wave.  `operands`: at least 32 KiB of device memory holding
   fp16 values (finite ones, or the timing measures exception paths).  *flops (may be NULL) receives the
   floating-point operations of the launch.  Returns a glm_attn status. */
int glm_bench_mfma(int pattern, const void *operands, size_t operand_bytes, int32_t iters, float *sink, void *stream,
                   double *flops);

#ifdef __cplusplus
}
#endif
#endif /* GLM_BENCH_H */
