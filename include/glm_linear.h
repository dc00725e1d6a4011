/*
 * glm_linear.h — C ABI of the Linear layers either side of the attention path, in libglm_attn.so (gfx950).
 *
 * Replaces li-plus/chatglm.cpp's Linear (chatglm.h:362-377, chatglm.cpp:418-426):
 *
 *     y[r][o] = sum_i weight[o][i] * x[r][i] + bias[o]
 *
 * as BasicAttention uses it for query_key_value (chatglm.cpp:629) and dense (chatglm.cpp:719).  Weights are
 * fp16 or fp32, row-major [out_features][in_features] (ggml ne = {in_features, out_features}); the bias is fp32.
 * With fp16 weights the input rows are rounded to fp16 before the products, which accumulate in fp32: what
 * ggml_mul_mat does for an fp16 src0.
 *
 * Block-quantised weights (Q4_0, Q4_1, Q5_0, Q5_1, Q8_0; in_features a multiple of 32): the weight tensor is
 * ggml's blocks, [out_features][in_features / 32] blocks of 18, 20, 22, 24 or 34 bytes, exactly the bytes of a
 * model file.  After the blocks are in place, glm_linear_commit rearranges them into the layout the kernels read
 * (and releases the block buffer if the library owns it); forward calls before that fail with GLM_ATTN_EINVAL.
 * For up to 8 rows the input rows are quantised to 8 bits per block of 32 and the products are exact integer sums
 * scaled per block (ggml's quantize_row_q8_0 / q8_1 and vec_dot_<type>_q8); for more rows the weight is expanded to
 * fp16 and the fp16 GEMM runs (input rounded to fp16, not quantised), as ggml's GPU backends do for batches.  The
 * expansion goes into one buffer per device, as large as the largest quantised weight created on it: such calls
 * on one device must not overlap on different streams.
 *
 * Calls with more than 8 rows are plain GEMMs (fp16 x fp16, fp32 accumulation and output) on the library's own MFMA
 * kernel after the rows have been rounded.  With GLM_LINEAR_HIPBLASLT=1 in the environment when the layer is created
 * they go to hipBLASLt instead (bias epilogue; the own kernel for shapes it has no algorithm for): faster, but off
 * by default, because two timing programs that drove it ended in GPU memory faults whose cause was never shown; a
 * caller-owned fp16 weight takes that branch only when weight_bytes states at least 4096 bytes beyond the tensor.
 *
 * All pointers named "device" are HIP device pointers; calls are asynchronous on the given stream.  Status
 * codes are those of glm_attn.h (0 = ok, negative = error; glm_attn_strerror names them).
 */
#ifndef GLM_LINEAR_H
#define GLM_LINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct glm_linear glm_linear;

/* Same numeric values as ggml_type (GGML_TYPE_F32 = 0, GGML_TYPE_F16 = 1, GGML_TYPE_Q4_0 = 2, ...): the types the
   reference's converter writes (chatglm_cpp/convert.py:37-44) and its Linear test runs (chatglm_test.cpp:424-428). */
typedef enum glm_linear_dtype {
    GLM_LINEAR_F32 = 0,
    GLM_LINEAR_F16 = 1,
    GLM_LINEAR_Q4_0 = 2,
    GLM_LINEAR_Q4_1 = 3,
    GLM_LINEAR_Q5_0 = 6,
    GLM_LINEAR_Q5_1 = 7,
    GLM_LINEAR_Q8_0 = 8
} glm_linear_dtype;

/* Replaces the constructor arguments of Linear (chatglm.h:365-367) and ModelContext::dtype. */
typedef struct glm_linear_desc {
    int32_t struct_size;  /* sizeof(glm_linear_desc), checked */
    int32_t in_features;
    int32_t out_features;
    int32_t weight_dtype; /* glm_linear_dtype */
    int32_t use_bias;     /* 0: no bias tensor (the reference's use_bias = false) */
    int32_t max_rows;     /* most input rows of any call; 0 means 1.  Above 8 it sizes the fp16 staging of the input
                             (max_rows x in_features x 2 bytes) and, for weights of fewer 128-feature tiles than the
                             GPU has CUs, the fp32 partial sums of calls cut along the input features (up to
                             8 x min(max_rows, 128) x out_features x 4 bytes): one buffer of each kind per device,
                             shared by all layers: calls with more than 8 rows on one device must not overlap on
                             different streams */
    int32_t device;       /* HIP device ordinal */
    void *weight;         /* optional caller-owned device tensor [out_features][in_features] (quantised types:
                             ggml blocks); NULL: the library allocates (zero-filled) and the caller fills it
                             through glm_linear_params */
    float *bias;          /* optional caller-owned device tensor [out_features]; NULL: as for weight */
    int64_t weight_bytes; /* bytes the caller's allocation holds from `weight` on, or 0 if not stated (and with a NULL
                             weight): a value below out_features x in_features elements (quantised types: blocks) is
                             refused with GLM_ATTN_EINVAL before any device call */
} glm_linear_desc;

/* Linear::Linear (chatglm.h:365-367). */
int glm_linear_create(const glm_linear_desc *desc, glm_linear **out_linear);

/* Frees what the object owns (not caller-owned tensors).  Synchronises the device. */
void glm_linear_destroy(glm_linear *linear);

/* Device pointers of the parameters: the public members Linear::weight and Linear::bias (chatglm.h:375-376).
   *bias is NULL for a layer without bias. */
int glm_linear_params(const glm_linear *linear, void **weight, float **bias);

/* To be called once the weight is in place (after ggml_backend_tensor_set in the reference's load_state_dict,
   chatglm.cpp:1113-1119): a no-op for fp32 and fp16 weights; for block-quantised weights it rearranges the blocks
   into the kernels' layout, synchronises the stream and, if the library owns the block buffer, frees it (then
   glm_linear_params reports a NULL weight).  May be called again after the caller has changed a caller-owned
   block buffer. */
int glm_linear_commit(glm_linear *linear, void *stream);

/* Linear::forward (chatglm.cpp:418-426).  x: device fp32 [rows][in_features]; y: device fp32
   [rows][out_features]; x and y must not overlap.  rows <= max_rows.  stream: hipStream_t (NULL = default). */
int glm_linear_forward(glm_linear *linear, const float *x, int32_t rows, float *y, void *stream);

/* What the one-token path can do in the same launch as the product, instead of separate launches before and after
   it.  No counterpart in the reference, whose graph has one node per operation; results are those of the separate
   entry points (glm_block_rms_norm / glm_block_gated_activation before, glm_attn_scale_add after). */
typedef enum glm_linear_prologue {
    GLM_LINEAR_PRO_NONE = 0,
    GLM_LINEAR_PRO_RMS_NORM = 1, /* input = RMSNorm(x): chatglm.cpp:437-442 feeding chatglm.cpp:629 or the MLP */
    GLM_LINEAR_PRO_GATED_ACT = 2 /* input = act(x) * up: the middle of BasicGLU::forward, chatglm.cpp:465-473 */
} glm_linear_prologue;

typedef struct glm_linear_fusion {
    int32_t struct_size;      /* sizeof(glm_linear_fusion), checked */
    int32_t prologue;         /* glm_linear_prologue */
    const float *norm_weight; /* RMS_NORM: device [in_features] */
    float norm_eps;           /* RMS_NORM */
    int32_t activation;       /* GATED_ACT and glm_linear_forward_glu: glm_block_activation (0 GELU, 1 SILU) */
    const float *up;          /* GATED_ACT: device [rows][in_features] */
    const float *residual;    /* NULL, or device [rows][out_features]: y = (x W^T + b) + residual * residual_scale,
                                 the residual sums of chatglm.h:488-503 and chatglm.cpp:1070-1087; may be y itself */
    float residual_scale;
} glm_linear_fusion;

/* glm_linear_forward with the operations named by *fusion folded into it.  Up to 8 rows: done inside the one launch
   of the bandwidth kernel.  More rows: the prologue takes the place of the pass that rounds the input to fp16 for
   the GEMM (its fp32 result is never written) and the residual is the GEMM's C operand.  GLM_ATTN_EUNSUPPORTED when
   the call would take neither path (fp32 weights, odd shapes, unaligned pointers), for block-quantised weights and
   up to 8 rows with GATED_ACT (glm_linear_forward_glu takes the gate) or with RMS_NORM at more than 2 rows, or, for
   fp16 weights and up to 8 rows with RMS_NORM,
   when rows * ceil(in_features / 256) > 32 (rows * in_features > 8192 for the usual widths): the caller then uses
   the separate entry points. */
int glm_linear_forward_fused(glm_linear *linear, const glm_linear_fusion *fusion, const float *x, int32_t rows,
                             float *y, void *stream);

/* The first three nodes of BasicGLU::forward (chatglm.cpp:465-473) for the one-token path in one launch:
       y = act(gate(x)) * up(x)
   gate and up: two layers of the same shape on the same device, both with fp16 weights or both block-quantised
   with the same type.  fusion->activation names act; fusion->prologue may be NONE or RMS_NORM (the post-attention
   norm, applied to x first); a residual is added last as in glm_linear_forward_fused.  GLM_ATTN_EUNSUPPORTED for
   more than 8 rows (2 for block-quantised weights) and wherever the bandwidth kernel is not taken: the caller then
   runs the two projections with glm_linear_forward_fused and gives the gate to the projection that follows. */
int glm_linear_forward_glu(glm_linear *gate, glm_linear *up, const glm_linear_fusion *fusion, const float *x,
                           int32_t rows, float *y, void *stream);

/* hipError_t of the last failed HIP call of this object (0 if none). */
int glm_linear_last_hip_error(const glm_linear *linear);

#ifdef __cplusplus
}
#endif
#endif /* GLM_LINEAR_H */
