/*
 * glm_attn.h — C ABI of libglm_attn.so: the KV-cache attention path of chatglm.cpp on MI355X (gfx950).
 *
 * The library replaces what li-plus/chatglm.cpp builds as a ggml graph in
 * BasicAttention::forward (chatglm.cpp:620-721) between the two Linear layers:
 *
 *     rope(q, k)  ->  append K into k_cache[kvh][L][d], V into v_cache[kvh][d][L] at nvt + n_past
 *                 ->  softmax(q K^T / sqrt(d) + mask) V  over cache positions [0, nvt + n_past + qlen)
 *
 * with L = max_length + num_virtual_tokens, both caches fp16, the reference's layouts
 * (chatglm.h:452-455, 470-471).  All pointers named "device" are HIP device pointers; every call
 * is asynchronous on the given stream and ordered like any other work on it; nothing here
 * synchronises the stream.  One context serves one caller thread at a time (the reference's
 * ModelContext is not re-entrant either, chatglm.cpp:728-729); separate contexts are independent.
 *
 * Every entry point returns a glm_attn_status (0 = ok, negative = error) and never throws.
 */
#ifndef GLM_ATTN_H
#define GLM_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct glm_attn_ctx glm_attn_ctx;

typedef enum glm_attn_status {
    GLM_ATTN_OK = 0,
    GLM_ATTN_EINVAL = -1,       /* null pointer, non-positive size, heads not divisible, bad enum value */
    GLM_ATTN_ERANGE = -2,       /* nvt + n_past + qlen > cache rows, layer out of range, qlen > max_qlen */
    GLM_ATTN_ENOMEM = -3,       /* device or host allocation failed */
    GLM_ATTN_EHIP = -4,         /* a HIP call failed; see glm_attn_last_hip_error */
    GLM_ATTN_EUNSUPPORTED = -5, /* shape outside what the kernels are written for */
    GLM_ATTN_ESTATIC = -6       /* beyond the fixed size of glm_attn_decode_static's exchange memory */
} glm_attn_status;

/* Same numeric values as the reference's enum class RopeType (chatglm.h:93-99). */
typedef enum glm_attn_rope_type {
    GLM_ATTN_ROPE_GPTJ = 0,       /* whole head, adjacent pairs (apply_rotary_emb_basic, chatglm.cpp:523-537) */
    GLM_ATTN_ROPE_NEOX = 2,       /* whole head, pairs (i, i + d/2) */
    GLM_ATTN_ROPE_CHATGLM = 4,    /* ChatGLM-6B 2-D rope: NEOX on each half (apply_rotary_emb_glm, :539-574) */
    GLM_ATTN_ROPE_CHATGLM2 = 8,   /* ChatGLM2/3/4: adjacent pairs on dims [0, d/2) (apply_rotary_emb_glm2, :576-601) */
    GLM_ATTN_ROPE_DISABLED = 10000
} glm_attn_rope_type;

/* Same order as the reference's enum class AttentionMaskType (chatglm.h:101-104). */
typedef enum glm_attn_mask_type {
    GLM_ATTN_MASK_CAUSAL = 0,  /* ggml_diag_mask_inf(nvt + n_past), chatglm.cpp:696-697 */
    GLM_ATTN_MASK_CHATGLM = 1  /* additive fp32 mask tensor [qlen][kvlen], chatglm.cpp:699 */
} glm_attn_mask_type;

typedef enum glm_attn_mask_rule {
    /* The reference masks only when n_past == 0 (chatglm.cpp:689): a multi-token call at
       n_past > 0 attends to every key, including later tokens of the same call. */
    GLM_ATTN_MASK_RULE_REFERENCE = 0,
    /* Extension without a counterpart in the reference: causal mask with offset for every n_past
       (key c is visible to token t iff c <= nvt + n_past + t); the mask tensor is ignored. */
    GLM_ATTN_MASK_RULE_CAUSAL_OFFSET = 1
} glm_attn_mask_rule;

/* Replaces the constructor arguments of BasicAttention (chatglm.h:443-455) and the per-model
   allocation of all layers' caches in one buffer (BasicModel::build_layers, chatglm.h:618-630). */
typedef struct glm_attn_desc {
    int32_t struct_size;          /* sizeof(glm_attn_desc), checked */
    int32_t num_layers;           /* one k_cache / v_cache pair per layer */
    int32_t num_attention_heads;  /* h */
    int32_t num_key_value_heads;  /* kvh, divides h; q head hh reads group hh / (h / kvh) */
    int32_t head_size;            /* d */
    int32_t max_length;           /* cache rows L = max_length + num_virtual_tokens */
    int32_t num_virtual_tokens;   /* p-tuning prefix length nvt (0 if none) */
    int32_t rope_type;            /* glm_attn_rope_type */
    float rope_theta;             /* frequency base; CHATGLM ignores it and uses 10000 like the reference */
    int32_t attn_mask_type;       /* glm_attn_mask_type */
    int32_t interleaved_qkv;      /* 1: qkv row is [h][3][d] (ChatGLM-6B), needs kvh == h (chatglm.cpp:636-644) */
    int32_t mask_rule;            /* glm_attn_mask_rule */
    int32_t max_qlen;             /* largest qlen of any call; 0 means max_length */
    int32_t device;               /* HIP device ordinal */
    void *kv_buffer;              /* optional caller-owned device slab of glm_attn_kv_bytes() bytes, 256-byte
                                     aligned; NULL: the library allocates (and zero-fills) its own */
} glm_attn_desc;

/* Fills desc with the ChatGLM2/3/4 defaults (32 heads, 2 groups, d 128, CHATGLM2 rope, causal). */
void glm_attn_default_desc(glm_attn_desc *desc);

/* Bytes of the KV slab: num_layers * 2 * kvh * L * d * 2, layer l at offset l * 2 * kvh*L*d*2,
   K first ([kvh][L][d]), then V ([kvh][d][L]). */
size_t glm_attn_kv_bytes(const glm_attn_desc *desc);

/* Builds the context: KV slab, the rope cos/sin table (host libm, fp32 recurrence of ggml's rope),
   scratch for fp16 queries and split partials.  Replaces BasicAttention's constructor and
   ModelContext's kv buffer (chatglm.h:331-348, 443-455). */
int glm_attn_create(const glm_attn_desc *desc, glm_attn_ctx **out_ctx);

/* Frees everything the context owns (not a caller-owned kv_buffer).  Synchronises the device. */
void glm_attn_destroy(glm_attn_ctx *ctx);

/* The three views of the fused projection in their general form (chatglm.cpp:636-653: ggml_view_3d with a byte
   offset, nb[1] between heads and nb[2] between tokens): q head i of a token starts q_offset + i * head_stride
   floats into the token's row, k and v heads likewise from k_offset and v_offset; the stride between tokens stays
   the qkv_row_stride of each call (0 there = the smallest stride that holds all three views).  glm_attn_create
   sets the two layouts the reference builds (plain: offsets 0, h d, (h + kvh) d, stride d; interleaved_qkv:
   0, d, 2 d, stride 3 d); this call replaces them for every later call of the context.  head_stride >= d.
   When an offset or the stride is not a multiple of 4 floats, one-token calls take the two-launch path
   (glm_attn_decode returns GLM_ATTN_EUNSUPPORTED). */
int glm_attn_set_qkv_views(glm_attn_ctx *ctx, int64_t q_offset, int64_t k_offset, int64_t v_offset,
                           int64_t head_stride);

/* Device pointers of one layer's caches: k_cache fp16 [kvh][L][d], v_cache fp16 [kvh][d][L]
   (the public members BasicAttention::k_cache / v_cache, chatglm.h:470-471). */
int glm_attn_cache_ptrs(const glm_attn_ctx *ctx, int32_t layer, void **k_cache, void **v_cache);

/*
 * BasicAttention::forward (chatglm.cpp:620-721) without query_key_value (:629) and dense (:719).
 *
 *   qkv             device fp32 [qlen][qkv_row_stride], the output of the fused QKV projection:
 *                   q heads, then k heads, then v heads (or [h][3][d] when interleaved_qkv);
 *                   qkv_row_stride in floats, 0 = (h + 2 kvh) d.  Not modified.
 *   attention_mask  device fp32 [qlen][nvt + n_past + qlen] or NULL; read only for
 *                   GLM_ATTN_MASK_CHATGLM at n_past == 0 under the reference mask rule.
 *   position_ids    device int32 [qlen] ([2 qlen] for GLM_ATTN_ROPE_CHATGLM: positions, then block
 *                   positions); may be NULL when position_ids_host is given and qlen == 1, or when
 *                   rope is disabled.
 *   position_ids_host  optional host copy of the same ids (the reference builds them on the host,
 *                   chatglm.cpp:1148-1152, 1324-1325).  For qlen == 1 they travel as kernel
 *                   arguments, which takes a dependent device load off the decode critical path.
 *   out             device fp32 [qlen][h d] (the context layer the reference feeds to dense).
 *   stream          hipStream_t (NULL = default stream).
 *
 * Errors: EINVAL for null/shape errors, ERANGE when nvt + n_past + qlen exceeds the cache rows
 * (the reference does not check this and would write out of bounds).
 */
int glm_attn_forward(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                     const float *attention_mask, const int32_t *position_ids, const int32_t *position_ids_host,
                     int32_t qlen, int32_t n_past, float *out, void *stream);

/* The first half of forward alone: rope on q and k, then the K and V appends (chatglm.cpp:655-675).
   Leaves the roped, scaled fp16 queries in the context's scratch. */
int glm_attn_rope_append(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                         const int32_t *position_ids, int32_t qlen, int32_t n_past, void *stream);

/* The second half of forward alone: attention of the queries that the last glm_attn_rope_append of this
   context left in its scratch (same qlen and n_past) over the cache, masked as forward masks
   (chatglm.cpp:678-717).  rope_append followed by attend is forward for qlen > 1, launch for launch. */
int glm_attn_attend(glm_attn_ctx *ctx, int32_t layer, const float *attention_mask, int32_t qlen, int32_t n_past,
                    float *out, void *stream);

/* forward for qlen == 1 through the fused split-KV kernel: rope, append, attention and the merge of
   the split partials in one launch.  EUNSUPPORTED unless d == 128, h / kvh <= 16 and L % 8 == 0. */
int glm_attn_decode(glm_attn_ctx *ctx, int32_t layer, const float *qkv, const int32_t *position_ids,
                    const int32_t *position_ids_host, int32_t n_past, float *out, void *stream);

/* glm_attn_decode for callers that cannot allocate device memory and want no allocation of the library's
   behind their call either (code under HIP graph capture, tight serving loops, harnesses that forbid
   hipMalloc).  It has no counterpart in the reference.  Same arguments, same kernel and same result as
   glm_attn_decode, but the split partials and the hand-over words of the launch live in a device array
   that is part of the library's code object (2.2 MB on every GPU the library runs on, held until the
   process ends) instead of in memory of the context; the call itself allocates and frees nothing.
   Limit: at most 32 KV groups (GLM_ATTN_ESTATIC beyond), at most 256 workgroups per launch (the split
   count is cut to fit).  All calls on one GPU share that GPU's array, whatever their context: calls that
   overlap in time on one GPU (two streams, two threads) race and give wrong results; calls in stream
   order on one stream at a time are fine, also from different contexts in turn.  Nothing needs to be
   cleared between calls: what a launch reads of the array it has written itself, under a stamp that no
   earlier launch used. */
int glm_attn_decode_static(glm_attn_ctx *ctx, int32_t layer, const float *qkv, const int32_t *position_ids,
                           const int32_t *position_ids_host, int32_t n_past, float *out, void *stream);

/* forward through rope+append and the MFMA prefill kernel.  Same shape limits as decode. */
int glm_attn_prefill(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                     const float *attention_mask, const int32_t *position_ids, int32_t qlen, int32_t n_past,
                     float *out, void *stream);

/* BasicModel::load_prefix_cache for one layer (chatglm.h:580-615): past_kv is device fp16
   [2][kvh][nvt][d] (keys, then values); it is copied to cache positions [0, nvt), V transposed. */
int glm_attn_load_prefix_cache(glm_attn_ctx *ctx, int32_t layer, const void *past_kv, void *stream);

/* Graph-input producers, host side (ChatGLM2ForCausalLM::set_graph_inputs chatglm.cpp:1319-1327,
   ChatGLMForCausalLM::set_graph_inputs chatglm.cpp:1127-1154).  Outputs are host arrays. */
int glm_attn_position_ids_glm2(int32_t qlen, int32_t n_past, int32_t *out /* [qlen] */);
int glm_attn_position_ids_glm(int32_t qlen, int32_t n_past, int32_t n_ctx, int32_t *out /* [2 qlen] */);
int glm_attn_attention_mask_glm(int32_t qlen, int32_t kvlen, float *out /* [qlen][kvlen] */);

/* out[i] = a[i] * alpha + b[i] over n fp32 elements (device pointers; out may be a or b): the residual
   arithmetic around the attention, ggml_add_inplace in BasicBlock::forward (chatglm.h:488-503) and
   ggml_scale_inplace + ggml_add_inplace in GLMBlock::forward (chatglm.cpp:1070-1087). */
int glm_attn_scale_add(float *out, const float *a, float alpha, const float *b, int64_t n, void *stream);

/* Bit 0 of *flags is set when a kernel of this context met a position id outside the rope table
   [0, max_length + nvt) and clamped it.  Synchronises the context's device to read the word. */
int glm_attn_device_flags(glm_attn_ctx *ctx, uint32_t *flags);

/* The workgroups of the decode kernel wait for each other before they merge their partial results.
   The wait is bounded: a workgroup whose wait runs out exits and the last workgroup to arrive does
   its share, so the kernel always ends and the result is always complete, only later.  This sets
   the bound (default 100 us; 0 makes every workgroup but the last leave at once, which is how the
   tests drive the slow path).  No counterpart in the reference. */
int glm_attn_set_spin_limit_us(glm_attn_ctx *ctx, int64_t microseconds);

/* hipError_t of the last failed HIP call of this context (0 if none). */
int glm_attn_last_hip_error(const glm_attn_ctx *ctx);

const char *glm_attn_strerror(int status);

/* "glm_attn x.y (gfx950)" */
const char *glm_attn_version(void);

#ifdef __cplusplus
}
#endif
#endif /* GLM_ATTN_H */
