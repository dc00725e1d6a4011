// C-ABI layer of libglm_attn.so: context set-up, argument checks and kernel dispatch.
// Entry points are documented in include/glm_attn.h.
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <new>
#include <vector>

#include "glm_attn_internal.h"

using namespace glm_attn;

struct glm_attn_ctx {
    glm_attn_desc desc;
    Shape shape;
    QkvLayout layout;  // row_stride filled per call
    int64_t row_extent;  // floats of a row that the three views reach: the default row stride
    bool views_aligned;  // offsets and head stride are multiples of 4 floats: the 16-byte loads of the decode kernel
    RopeSpec rope;
    float scale;
    int max_qlen;
    bool fast;  // d == 128, G <= 16, cache rows % 8 == 0: the MFMA kernels apply
    int num_cus;
    size_t layer_halfs;  // halfs per layer in the slab (K then V)
    __half *kv;
    bool own_kv;
    float2 *rope_table;
    __half *q16;         // [h][max_qlen][d]
    int32_t *pos_stage;  // device copy of host position ids, [2 max_qlen]
    float *part;         // decode partials
    float *prefill_part; // partials of a prefill cut along the keys (see AttendArgs::split_scratch), or null
    int64_t prefill_floats;
    int max_splits;
    void *sync_mem;      // hand-over words of the decode kernel (see DecodeArgs)
    DecodeGroupSync *sync;
    unsigned long long *claim;
    long long spin_ticks;
    uint32_t *flags;
    int last_hip_error;
};

namespace {

// ---- exchange memory of glm_attn_decode_static: the split partials and hand-over words of one decode
// launch, for callers that must not allocate.  One copy per device, there from the moment the library is
// loaded until the process ends; every call on a device uses that device's copy.
constexpr int kStaticMaxGroups = 32;  // KV groups
constexpr int kStaticMaxParts = 256;  // (group, split) partials of one launch = workgroups of the launch
struct StaticScratch {
    DecodeGroupSync sync[kStaticMaxGroups];
    unsigned long long claim[kStaticMaxGroups][kDecodeMaxSplits];
    float part[(size_t)kStaticMaxParts * kDecodePartFloats];
};
constexpr int kMaxDevices = 64;

}  // namespace

// 2.2 MB.  In host code this name is a stand-in for the symbol, not a device address: the address on a
// device comes from hipGetSymbolAddress (scratch_on_device below), and only that is handed to kernels.
static __device__ __align__(256) unsigned char scratch[sizeof(StaticScratch)];

namespace {

StaticScratch *g_scratch_ptr[kMaxDevices];  // per device, null until asked for

// The address of `scratch` on the current device (which must be `device`).
hipError_t scratch_on_device(int device, StaticScratch **out) {
    *out = nullptr;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        if (!p) return hipErrorInvalidSymbol;
        g_scratch_ptr[device] = static_cast<StaticScratch *>(p);
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

#define HIP_TRY(ctx, expr)                         \
    do {                                           \
        hipError_t e_ = (expr);                    \
        if (e_ != hipSuccess) {                    \
            if (ctx) (ctx)->last_hip_error = (int)e_; \
            return GLM_ATTN_EHIP;                  \
        }                                          \
    } while (0)

int check_desc(const glm_attn_desc *d) {
    if (!d || d->struct_size != (int32_t)sizeof(glm_attn_desc)) return GLM_ATTN_EINVAL;
    if (d->num_layers <= 0 || d->num_attention_heads <= 0 || d->num_key_value_heads <= 0 || d->head_size <= 0 ||
        d->max_length <= 0 || d->num_virtual_tokens < 0 || d->max_qlen < 0) {
        return GLM_ATTN_EINVAL;
    }
    if (d->num_attention_heads % d->num_key_value_heads != 0) return GLM_ATTN_EINVAL;
    // chatglm.cpp:637: "interleaved qkv is not supported for GQA"
    if (d->interleaved_qkv && d->num_attention_heads != d->num_key_value_heads) return GLM_ATTN_EINVAL;
    switch (d->rope_type) {
    case GLM_ATTN_ROPE_GPTJ:
    case GLM_ATTN_ROPE_NEOX:
        if (d->head_size % 2) return GLM_ATTN_EINVAL;
        break;
    case GLM_ATTN_ROPE_CHATGLM:
    case GLM_ATTN_ROPE_CHATGLM2:
        if (d->head_size % 4) return GLM_ATTN_EINVAL;
        break;
    case GLM_ATTN_ROPE_DISABLED:
        break;
    default:  // chatglm.cpp:615-616 "Unknown rope type"
        return GLM_ATTN_EINVAL;
    }
    if (d->attn_mask_type != GLM_ATTN_MASK_CAUSAL && d->attn_mask_type != GLM_ATTN_MASK_CHATGLM) return GLM_ATTN_EINVAL;
    if (d->mask_rule != GLM_ATTN_MASK_RULE_REFERENCE && d->mask_rule != GLM_ATTN_MASK_RULE_CAUSAL_OFFSET) {
        return GLM_ATTN_EINVAL;
    }
    if (d->head_size > 256) return GLM_ATTN_EUNSUPPORTED;
    return GLM_ATTN_OK;
}

struct DeviceGuard {
    int prev = -1;
    bool ok = false;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) == hipSuccess && hipSetDevice(dev) == hipSuccess) ok = true;
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

// ggml's rope keeps the angle in an fp32 recurrence (theta *= theta_scale) and calls the host libm;
// a closed form or device transcendentals would change K-cache bits, so the table is built here.
std::vector<float> build_rope_table(int n_dims, float base, int positions) {
    const int pairs = n_dims / 2;
    std::vector<float> t((size_t)positions * pairs * 2);
    const float theta_scale = powf(base, -2.0f / (float)n_dims);
    for (int p = 0; p < positions; p++) {
        float theta = (float)p;
        float *row = t.data() + (size_t)p * pairs * 2;
        for (int i = 0; i < pairs; i++) {
            row[2 * i + 0] = cosf(theta);
            row[2 * i + 1] = sinf(theta);
            theta *= theta_scale;
        }
    }
    return t;
}

void free_ctx(glm_attn_ctx *c) {
    if (!c) return;
    if (c->own_kv && c->kv) (void)hipFree(c->kv);
    if (c->rope_table) (void)hipFree(c->rope_table);
    if (c->q16) (void)hipFree(c->q16);
    if (c->prefill_part) (void)hipFree(c->prefill_part);
    if (c->pos_stage) (void)hipFree(c->pos_stage);
    if (c->part) (void)hipFree(c->part);
    if (c->sync_mem) (void)hipFree(c->sync_mem);
    if (c->flags) (void)hipFree(c->flags);
    delete c;
}

__half *layer_k(const glm_attn_ctx *c, int layer) { return c->kv + (size_t)layer * c->layer_halfs; }
__half *layer_v(const glm_attn_ctx *c, int layer) {
    return c->kv + (size_t)layer * c->layer_halfs + c->layer_halfs / 2;
}

int check_call(const glm_attn_ctx *c, int layer, int qlen, int n_past) {
    if (!c) return GLM_ATTN_EINVAL;
    if (qlen <= 0 || n_past < 0) return GLM_ATTN_EINVAL;
    if (layer < 0 || layer >= c->desc.num_layers) return GLM_ATTN_ERANGE;
    if (qlen > c->max_qlen) return GLM_ATTN_ERANGE;
    if ((int64_t)c->desc.num_virtual_tokens + n_past + qlen > c->shape.L) return GLM_ATTN_ERANGE;
    return GLM_ATTN_OK;
}

QkvLayout call_layout(const glm_attn_ctx *c, int64_t row_stride) {
    QkvLayout l = c->layout;
    l.row_stride = row_stride > 0 ? row_stride : c->row_extent;
    return l;
}

// One past the last float of a row that the views (offsets, head stride) reach.
int64_t views_extent(const Shape &s, int64_t q_off, int64_t k_off, int64_t v_off, int64_t head_stride) {
    const int64_t q_end = q_off + (int64_t)(s.h - 1) * head_stride + s.d;
    const int64_t k_end = k_off + (int64_t)(s.kvh - 1) * head_stride + s.d;
    const int64_t v_end = v_off + (int64_t)(s.kvh - 1) * head_stride + s.d;
    return q_end > k_end ? (q_end > v_end ? q_end : v_end) : (k_end > v_end ? k_end : v_end);
}

// Which keys a call masks: (causal flag, additive mask pointer).  chatglm.cpp:689-707.
int resolve_mask(const glm_attn_ctx *c, int n_past, const float *attention_mask, int *causal, const float **mask) {
    *causal = 0;
    *mask = nullptr;
    if (c->desc.mask_rule == GLM_ATTN_MASK_RULE_CAUSAL_OFFSET) {
        *causal = 1;
        return GLM_ATTN_OK;
    }
    if (n_past != 0) return GLM_ATTN_OK;  // the reference applies no mask to a continuation
    if (c->desc.attn_mask_type == GLM_ATTN_MASK_CAUSAL) {
        *causal = 1;
    } else {
        if (!attention_mask) return GLM_ATTN_EINVAL;
        *mask = attention_mask;
    }
    return GLM_ATTN_OK;
}

bool aligned16(const void *p) { return ((uintptr_t)p & 15u) == 0; }

int stage_positions(glm_attn_ctx *c, const int32_t *position_ids, const int32_t *position_ids_host, int qlen,
                    hipStream_t stream, const int32_t **dev_pos) {
    *dev_pos = position_ids;
    if (c->rope.pairs == 0) return GLM_ATTN_OK;
    if (position_ids) return GLM_ATTN_OK;
    if (!position_ids_host) return GLM_ATTN_EINVAL;
    const int n = (c->desc.rope_type == GLM_ATTN_ROPE_CHATGLM) ? 2 * qlen : qlen;
    HIP_TRY(c, hipMemcpyAsync(c->pos_stage, position_ids_host, sizeof(int32_t) * (size_t)n, hipMemcpyHostToDevice,
                              stream));
    *dev_pos = c->pos_stage;
    return GLM_ATTN_OK;
}

int do_rope_append(glm_attn_ctx *c, int layer, const float *qkv, int64_t row_stride, const int32_t *dev_pos, int qlen,
                   int n_past, hipStream_t stream) {
    if (row_stride > 0 && row_stride < c->row_extent) return GLM_ATTN_EINVAL;  // rows would run into each other
    RopeAppendArgs ra;
    ra.qkv = qkv;
    ra.lay = call_layout(c, row_stride);
    ra.rope = c->rope;
    ra.s = c->shape;
    ra.position_ids = dev_pos;
    ra.qlen = qlen;
    ra.p0 = c->desc.num_virtual_tokens + n_past;
    ra.scale = c->scale;
    ra.q16 = c->q16;
    ra.k_cache = layer_k(c, layer);
    ra.v_cache = layer_v(c, layer);
    ra.flags = c->flags;
    HIP_TRY(c, launch_rope_append(ra, stream));
    return GLM_ATTN_OK;
}

AttendArgs make_attend(glm_attn_ctx *c, int layer, int qlen, int n_past, int causal, const float *mask, float *out) {
    AttendArgs aa;
    aa.s = c->shape;
    aa.q16 = c->q16;
    aa.k_cache = layer_k(c, layer);
    aa.v_cache = layer_v(c, layer);
    aa.mask = mask;
    aa.causal = causal;
    aa.qlen = qlen;
    aa.p0 = c->desc.num_virtual_tokens + n_past;
    aa.kvs = aa.p0 + qlen;
    aa.out = out;
    aa.split_scratch = c->prefill_part;
    aa.split_floats = c->prefill_floats;
    return aa;
}

// `shared`: null, or the device's static exchange memory to use in place of the context's own
int do_decode(glm_attn_ctx *c, int layer, const float *qkv, const int32_t *position_ids,
              const int32_t *position_ids_host, int n_past, float *out, hipStream_t stream,
              StaticScratch *shared = nullptr) {
    DecodeArgs da;
    da.qkv = qkv;
    da.lay = call_layout(c, 0);
    da.rope = c->rope;
    da.s = c->shape;
    da.position_ids = position_ids;
    da.pos0 = 0;
    da.pos1 = 0;
    da.pos_from_args = 0;
    if (c->rope.pairs > 0) {
        if (position_ids_host) {
            da.pos_from_args = 1;
            da.pos0 = position_ids_host[0];
            da.pos1 = (c->desc.rope_type == GLM_ATTN_ROPE_CHATGLM) ? position_ids_host[1] : 0;
        } else if (!position_ids) {
            return GLM_ATTN_EINVAL;
        }
    }
    da.p0 = c->desc.num_virtual_tokens + n_past;
    da.scale = c->scale;
    da.k_cache = layer_k(c, layer);
    da.v_cache = layer_v(c, layer);
    const DecodePlan pl = plan_decode(da.p0, c->shape.kvh, c->num_cus, c->max_splits, shared ? kStaticMaxParts : 0);
    da.nsplit = pl.nsplit;
    da.tiles_q = pl.tiles_q;
    da.tiles_r = pl.tiles_r;
    da.part = shared ? shared->part : c->part;
    da.out = out;
    da.flags = c->flags;
    da.sync = shared ? shared->sync : c->sync;
    da.claim = shared ? &shared->claim[0][0] : c->claim;
    da.spin_ticks = c->spin_ticks;
    da.stamp_groups = shared ? 1 : 0;
    HIP_TRY(c, launch_decode(da, stream));
    return GLM_ATTN_OK;
}

// out = a * alpha + b; the product and the sum are rounded separately, like ggml's scale followed by add
__global__ void scale_add_kernel(float *out, const float *a, float alpha, const float *b, int64_t n) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
        out[i] = __fadd_rn(__fmul_rn(a[i], alpha), b[i]);
    }
}

}  // namespace

extern "C" {

void glm_attn_default_desc(glm_attn_desc *d) {
    if (!d) return;
    memset(d, 0, sizeof(*d));
    d->struct_size = (int32_t)sizeof(glm_attn_desc);
    d->num_layers = 1;
    d->num_attention_heads = 32;
    d->num_key_value_heads = 2;
    d->head_size = 128;
    d->max_length = 2048;
    d->num_virtual_tokens = 0;
    d->rope_type = GLM_ATTN_ROPE_CHATGLM2;
    d->rope_theta = 10000.f;
    d->attn_mask_type = GLM_ATTN_MASK_CAUSAL;
    d->interleaved_qkv = 0;
    d->mask_rule = GLM_ATTN_MASK_RULE_REFERENCE;
    d->max_qlen = 0;
    d->device = 0;
    d->kv_buffer = nullptr;
}

size_t glm_attn_kv_bytes(const glm_attn_desc *d) {
    if (check_desc(d) != GLM_ATTN_OK) return 0;
    const size_t L = (size_t)d->max_length + (size_t)d->num_virtual_tokens;
    return (size_t)d->num_layers * 2u * (size_t)d->num_key_value_heads * L * (size_t)d->head_size * sizeof(__half);
}

int glm_attn_create(const glm_attn_desc *desc, glm_attn_ctx **out_ctx) {
    if (!out_ctx) return GLM_ATTN_EINVAL;
    *out_ctx = nullptr;
    int rc = check_desc(desc);
    if (rc != GLM_ATTN_OK) return rc;
    if (desc->kv_buffer && ((uintptr_t)desc->kv_buffer & 255u)) return GLM_ATTN_EINVAL;

    glm_attn_ctx *c = new (std::nothrow) glm_attn_ctx();
    if (!c) return GLM_ATTN_ENOMEM;
    memset(c, 0, sizeof(*c));
    c->desc = *desc;
    Shape &s = c->shape;
    s.h = desc->num_attention_heads;
    s.kvh = desc->num_key_value_heads;
    s.d = desc->head_size;
    s.G = s.h / s.kvh;
    s.L = desc->max_length + desc->num_virtual_tokens;
    c->scale = 1.f / sqrtf((float)s.d);  // chatglm.cpp:686
    c->max_qlen = desc->max_qlen > 0 ? desc->max_qlen : desc->max_length;
    if (desc->interleaved_qkv) {  // chatglm.cpp:636-644
        c->layout.head_stride = 3 * s.d;
        c->layout.q_off = 0;
        c->layout.k_off = s.d;
        c->layout.v_off = 2 * s.d;
    } else {  // chatglm.cpp:645-653
        c->layout.head_stride = s.d;
        c->layout.q_off = 0;
        c->layout.k_off = s.h * s.d;
        c->layout.v_off = (s.h + s.kvh) * s.d;
    }
    c->row_extent = views_extent(s, c->layout.q_off, c->layout.k_off, c->layout.v_off, c->layout.head_stride);
    c->views_aligned = ((c->layout.q_off | c->layout.k_off | c->layout.v_off | c->layout.head_stride) & 3) == 0;
    c->fast = (s.d == kFastHeadSize) && (s.G <= kMaxGroupHeads) && (s.L % 8 == 0);
    c->layer_halfs = 2u * (size_t)s.kvh * (size_t)s.L * (size_t)s.d;

    DeviceGuard guard(desc->device);
    if (!guard.ok) {
        delete c;
        return GLM_ATTN_EHIP;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, desc->device) != hipSuccess) {
        delete c;
        return GLM_ATTN_EHIP;
    }
    c->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    {
        // set-up is where the address of the static exchange memory on this device is looked up
        StaticScratch *unused;
        if (scratch_on_device(desc->device, &unused) != hipSuccess) {
            delete c;
            return GLM_ATTN_EHIP;
        }
    }

#define CREATE_TRY(expr)                               \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) {                        \
            free_ctx(c);                               \
            return e_ == hipErrorOutOfMemory ? GLM_ATTN_ENOMEM : GLM_ATTN_EHIP; \
        }                                              \
    } while (0)

    const size_t kv_bytes = glm_attn_kv_bytes(desc);
    if (desc->kv_buffer) {
        c->kv = static_cast<__half *>(desc->kv_buffer);
        c->own_kv = false;
    } else {
        CREATE_TRY(hipMalloc((void **)&c->kv, kv_bytes));
        c->own_kv = true;
        CREATE_TRY(hipMemset(c->kv, 0, kv_bytes));
    }

    // rope table (chatglm.cpp:534-535, 563-564, 593-594 give n_dims and the base per rope type)
    int n_dims = 0;
    float base = desc->rope_theta;
    switch (desc->rope_type) {
    case GLM_ATTN_ROPE_GPTJ:
    case GLM_ATTN_ROPE_NEOX:
        n_dims = s.d;
        break;
    case GLM_ATTN_ROPE_CHATGLM2:
        n_dims = s.d / 2;
        break;
    case GLM_ATTN_ROPE_CHATGLM:
        n_dims = s.d / 2;
        base = 10000.f;  // ggml_rope_inplace has no base argument
        break;
    default:
        n_dims = 0;
    }
    c->rope.type = desc->rope_type;
    c->rope.pairs = n_dims / 2;
    c->rope.table_positions = s.L;
    c->rope.table = nullptr;
    if (c->rope.pairs > 0) {
        std::vector<float> t = build_rope_table(n_dims, base, s.L);
        CREATE_TRY(hipMalloc((void **)&c->rope_table, t.size() * sizeof(float)));
        CREATE_TRY(hipMemcpy(c->rope_table, t.data(), t.size() * sizeof(float), hipMemcpyHostToDevice));
        c->rope.table = c->rope_table;
    }

    CREATE_TRY(hipMalloc((void **)&c->q16, (size_t)s.h * (size_t)c->max_qlen * (size_t)s.d * sizeof(__half)));
    CREATE_TRY(hipMalloc((void **)&c->pos_stage, sizeof(int32_t) * 2u * (size_t)c->max_qlen));
    c->max_splits = c->num_cus / s.kvh > 0 ? c->num_cus / s.kvh : 1;
    if (c->max_splits > kDecodeMaxSplits) c->max_splits = kDecodeMaxSplits;
    {
        // [kvh] counters, then [kvh][kDecodeMaxSplits] claims (u64)
        const size_t bytes = (size_t)s.kvh * (sizeof(DecodeGroupSync) + kDecodeMaxSplits * sizeof(unsigned long long));
        CREATE_TRY(hipMalloc(&c->sync_mem, bytes));
        CREATE_TRY(hipMemset(c->sync_mem, 0, bytes));
        c->sync = static_cast<DecodeGroupSync *>(c->sync_mem);
        c->claim = reinterpret_cast<unsigned long long *>(c->sync + s.kvh);
        c->spin_ticks = 100 * 100;  // 100 us at the 100 MHz constant clock
    }
    {
        // the lines of the partials carry launch stamps, which are never 0: begin with none that matches
        const size_t bytes = sizeof(float) * (size_t)s.kvh * c->max_splits * kDecodePartFloats;
        CREATE_TRY(hipMalloc((void **)&c->part, bytes));
        CREATE_TRY(hipMemset(c->part, 0, bytes));
    }
    c->prefill_part = nullptr;
    c->prefill_floats = 0;
    if (c->fast && c->max_qlen > 1) {
        // room for the partials of a short chunk against a long cache: 2048 (share, token) pairs of all heads
        c->prefill_floats = 2048 * ((int64_t)s.h * s.d + 2 * (int64_t)s.h);
        CREATE_TRY(hipMalloc((void **)&c->prefill_part, sizeof(float) * (size_t)c->prefill_floats));
    }
    CREATE_TRY(hipMalloc((void **)&c->flags, sizeof(uint32_t)));
    CREATE_TRY(hipMemset(c->flags, 0, sizeof(uint32_t)));
    CREATE_TRY(hipDeviceSynchronize());
#undef CREATE_TRY
    *out_ctx = c;
    return GLM_ATTN_OK;
}

void glm_attn_destroy(glm_attn_ctx *ctx) {
    if (!ctx) return;
    DeviceGuard guard(ctx->desc.device);
    (void)hipDeviceSynchronize();
    free_ctx(ctx);
}

int glm_attn_set_qkv_views(glm_attn_ctx *ctx, int64_t q_offset, int64_t k_offset, int64_t v_offset,
                           int64_t head_stride) {
    if (!ctx) return GLM_ATTN_EINVAL;
    const Shape &s = ctx->shape;
    if (q_offset < 0 || k_offset < 0 || v_offset < 0 || head_stride < s.d) return GLM_ATTN_EINVAL;
    const int64_t extent = views_extent(s, q_offset, k_offset, v_offset, head_stride);
    if (extent > 0x7fffffff) return GLM_ATTN_ERANGE;  // the kernels keep the offsets in 32 bits
    ctx->layout.q_off = (int)q_offset;
    ctx->layout.k_off = (int)k_offset;
    ctx->layout.v_off = (int)v_offset;
    ctx->layout.head_stride = (int)head_stride;
    ctx->row_extent = extent;
    ctx->views_aligned = ((q_offset | k_offset | v_offset | head_stride) & 3) == 0;
    return GLM_ATTN_OK;
}

int glm_attn_cache_ptrs(const glm_attn_ctx *ctx, int32_t layer, void **k_cache, void **v_cache) {
    if (!ctx) return GLM_ATTN_EINVAL;
    if (layer < 0 || layer >= ctx->desc.num_layers) return GLM_ATTN_ERANGE;
    if (k_cache) *k_cache = layer_k(ctx, layer);
    if (v_cache) *v_cache = layer_v(ctx, layer);
    return GLM_ATTN_OK;
}

int glm_attn_rope_append(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                         const int32_t *position_ids, int32_t qlen, int32_t n_past, void *stream) {
    int rc = check_call(ctx, layer, qlen, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!qkv || (ctx->rope.pairs > 0 && !position_ids)) return GLM_ATTN_EINVAL;
    DeviceGuard guard(ctx->desc.device);
    return do_rope_append(ctx, layer, qkv, qkv_row_stride, position_ids, qlen, n_past, (hipStream_t)stream);
}

int glm_attn_decode(glm_attn_ctx *ctx, int32_t layer, const float *qkv, const int32_t *position_ids,
                    const int32_t *position_ids_host, int32_t n_past, float *out, void *stream) {
    int rc = check_call(ctx, layer, 1, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!qkv || !out) return GLM_ATTN_EINVAL;
    if (!ctx->fast || !aligned16(qkv) || !ctx->views_aligned) return GLM_ATTN_EUNSUPPORTED;
    DeviceGuard guard(ctx->desc.device);
    return do_decode(ctx, layer, qkv, position_ids, position_ids_host, n_past, out, (hipStream_t)stream);
}

int glm_attn_decode_static(glm_attn_ctx *ctx, int32_t layer, const float *qkv, const int32_t *position_ids,
                           const int32_t *position_ids_host, int32_t n_past, float *out, void *stream) {
    int rc = check_call(ctx, layer, 1, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!qkv || !out) return GLM_ATTN_EINVAL;
    if (!ctx->fast || !aligned16(qkv) || !ctx->views_aligned) return GLM_ATTN_EUNSUPPORTED;
    if (ctx->shape.kvh > kStaticMaxGroups) return GLM_ATTN_ESTATIC;
    DeviceGuard guard(ctx->desc.device);
    StaticScratch *shared;
    HIP_TRY(ctx, scratch_on_device(ctx->desc.device, &shared));  // looked up in glm_attn_create: no work here
    return do_decode(ctx, layer, qkv, position_ids, position_ids_host, n_past, out, (hipStream_t)stream, shared);
}

int glm_attn_prefill(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                     const float *attention_mask, const int32_t *position_ids, int32_t qlen, int32_t n_past,
                     float *out, void *stream) {
    int rc = check_call(ctx, layer, qlen, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!qkv || !out || (ctx->rope.pairs > 0 && !position_ids)) return GLM_ATTN_EINVAL;
    if (!ctx->fast || !aligned16(out)) return GLM_ATTN_EUNSUPPORTED;
    int causal;
    const float *mask;
    rc = resolve_mask(ctx, n_past, attention_mask, &causal, &mask);
    if (rc != GLM_ATTN_OK) return rc;
    DeviceGuard guard(ctx->desc.device);
    hipStream_t st = (hipStream_t)stream;
    rc = do_rope_append(ctx, layer, qkv, qkv_row_stride, position_ids, qlen, n_past, st);
    if (rc != GLM_ATTN_OK) return rc;
    AttendArgs aa = make_attend(ctx, layer, qlen, n_past, causal, mask, out);
    HIP_TRY(ctx, launch_prefill(aa, ctx->num_cus, st));
    return GLM_ATTN_OK;
}

int glm_attn_attend(glm_attn_ctx *ctx, int32_t layer, const float *attention_mask, int32_t qlen, int32_t n_past,
                    float *out, void *stream) {
    int rc = check_call(ctx, layer, qlen, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!out) return GLM_ATTN_EINVAL;
    int causal;
    const float *mask;
    rc = resolve_mask(ctx, n_past, attention_mask, &causal, &mask);
    if (rc != GLM_ATTN_OK) return rc;
    DeviceGuard guard(ctx->desc.device);
    AttendArgs aa = make_attend(ctx, layer, qlen, n_past, causal, mask, out);
    if (ctx->fast && aligned16(out)) {
        HIP_TRY(ctx, launch_prefill(aa, ctx->num_cus, (hipStream_t)stream));
    } else {
        HIP_TRY(ctx, launch_attend_generic(aa, (hipStream_t)stream));
    }
    return GLM_ATTN_OK;
}

int glm_attn_forward(glm_attn_ctx *ctx, int32_t layer, const float *qkv, int64_t qkv_row_stride,
                     const float *attention_mask, const int32_t *position_ids, const int32_t *position_ids_host,
                     int32_t qlen, int32_t n_past, float *out, void *stream) {
    int rc = check_call(ctx, layer, qlen, n_past);
    if (rc != GLM_ATTN_OK) return rc;
    if (!qkv || !out) return GLM_ATTN_EINVAL;
    if (ctx->rope.pairs > 0 && !position_ids && !position_ids_host) return GLM_ATTN_EINVAL;
    int causal;
    const float *mask;
    rc = resolve_mask(ctx, n_past, attention_mask, &causal, &mask);
    if (rc != GLM_ATTN_OK) return rc;
    DeviceGuard guard(ctx->desc.device);
    hipStream_t st = (hipStream_t)stream;

    // one token, nothing to mask: the fused split-KV kernel
    if (qlen == 1 && ctx->fast && !mask && aligned16(qkv) && ctx->views_aligned) {
        return do_decode(ctx, layer, qkv, position_ids, position_ids_host, n_past, out, st);
    }
    const int32_t *dev_pos;
    rc = stage_positions(ctx, position_ids, position_ids_host, qlen, st, &dev_pos);
    if (rc != GLM_ATTN_OK) return rc;
    const bool mfma = ctx->fast && aligned16(out);
    rc = do_rope_append(ctx, layer, qkv, qkv_row_stride, dev_pos, qlen, n_past, st);
    if (rc != GLM_ATTN_OK) return rc;
    AttendArgs aa = make_attend(ctx, layer, qlen, n_past, causal, mask, out);
    if (mfma) {
        HIP_TRY(ctx, launch_prefill(aa, ctx->num_cus, st));
    } else {
        HIP_TRY(ctx, launch_attend_generic(aa, st));
    }
    return GLM_ATTN_OK;
}

int glm_attn_load_prefix_cache(glm_attn_ctx *ctx, int32_t layer, const void *past_kv, void *stream) {
    if (!ctx || !past_kv) return GLM_ATTN_EINVAL;
    if (layer < 0 || layer >= ctx->desc.num_layers) return GLM_ATTN_ERANGE;
    DeviceGuard guard(ctx->desc.device);
    HIP_TRY(ctx, launch_prefix_copy(static_cast<const __half *>(past_kv), layer_k(ctx, layer), layer_v(ctx, layer),
                                    ctx->shape, ctx->desc.num_virtual_tokens, (hipStream_t)stream));
    return GLM_ATTN_OK;
}

int glm_attn_position_ids_glm2(int32_t qlen, int32_t n_past, int32_t *out) {
    if (qlen < 0 || !out) return GLM_ATTN_EINVAL;
    for (int32_t i = 0; i < qlen; i++) out[i] = n_past + i;  // chatglm.cpp:1324-1325
    return GLM_ATTN_OK;
}

int glm_attn_position_ids_glm(int32_t qlen, int32_t n_past, int32_t n_ctx, int32_t *out) {
    if (qlen < 0 || !out) return GLM_ATTN_EINVAL;
    for (int32_t i = 0; i < qlen; i++) {  // chatglm.cpp:1148-1152
        const int32_t p = n_past + i;
        out[i] = p < n_ctx - 2 ? p : n_ctx - 2;
        out[qlen + i] = p - (n_ctx - 2) > 0 ? p - (n_ctx - 2) : 0;
    }
    return GLM_ATTN_OK;
}

int glm_attn_attention_mask_glm(int32_t qlen, int32_t kvlen, float *out) {
    if (qlen < 0 || kvlen <= 0 || !out) return GLM_ATTN_EINVAL;
    for (int64_t i = 0; i < (int64_t)qlen * kvlen; i++) out[i] = 0.f;  // chatglm.cpp:1133
    for (int32_t i = 0; i < qlen - 1; i++) out[(int64_t)i * kvlen + (kvlen - 1)] = -INFINITY;  // :1135-1137
    return GLM_ATTN_OK;
}

int glm_attn_device_flags(glm_attn_ctx *ctx, uint32_t *flags) {
    if (!ctx || !flags) return GLM_ATTN_EINVAL;
    DeviceGuard guard(ctx->desc.device);
    HIP_TRY(ctx, hipDeviceSynchronize());
    HIP_TRY(ctx, hipMemcpy(flags, ctx->flags, sizeof(uint32_t), hipMemcpyDeviceToHost));
    // slices of a decode output that their owners left behind and nobody redid
    std::vector<DecodeGroupSync> sync((size_t)ctx->shape.kvh);
    HIP_TRY(ctx, hipMemcpy(sync.data(), ctx->sync, sync.size() * sizeof(DecodeGroupSync), hipMemcpyDeviceToHost));
    for (const DecodeGroupSync &g : sync) {
        if (g.lost != 0) *flags |= kFlagMergeIncomplete;
    }
    // ... and the same count of the device's static exchange memory (glm_attn_decode_static), which every
    // context on the device shares: a slice lost there is reported to all of them
    if (ctx->shape.kvh <= kStaticMaxGroups) {
        StaticScratch *shared = nullptr;
        HIP_TRY(ctx, scratch_on_device(ctx->desc.device, &shared));
        HIP_TRY(ctx, hipMemcpy(sync.data(), shared->sync, sync.size() * sizeof(DecodeGroupSync), hipMemcpyDeviceToHost));
        for (const DecodeGroupSync &g : sync) {
            if (g.lost != 0) *flags |= kFlagMergeIncomplete;
        }
    }
    return GLM_ATTN_OK;
}

int glm_attn_set_spin_limit_us(glm_attn_ctx *ctx, int64_t microseconds) {
    if (!ctx || microseconds < 0) return GLM_ATTN_EINVAL;
    ctx->spin_ticks = microseconds * 100;  // wall_clock64() counts at 100 MHz
    return GLM_ATTN_OK;
}

int glm_attn_last_hip_error(const glm_attn_ctx *ctx) { return ctx ? ctx->last_hip_error : 0; }

const char *glm_attn_strerror(int status) {
    switch (status) {
    case GLM_ATTN_OK:
        return "ok";
    case GLM_ATTN_EINVAL:
        return "invalid argument";
    case GLM_ATTN_ERANGE:
        return "out of range (layer, qlen, or nvt + n_past + qlen beyond the cache rows)";
    case GLM_ATTN_ENOMEM:
        return "out of memory";
    case GLM_ATTN_EHIP:
        return "HIP runtime error";
    case GLM_ATTN_EUNSUPPORTED:
        return "shape not supported by this entry point";
    case GLM_ATTN_ESTATIC:
        return "more KV groups than the static exchange memory of glm_attn_decode_static has room for (32)";
    default:
        return "unknown status";
    }
}

int glm_attn_scale_add(float *out, const float *a, float alpha, const float *b, int64_t n, void *stream) {
    if (!out || !a || !b || n < 0) return GLM_ATTN_EINVAL;
    if (n == 0) return GLM_ATTN_OK;
    const int blocks = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
    hipLaunchKernelGGL(scale_add_kernel, dim3(blocks), dim3(256), 0, static_cast<hipStream_t>(stream), out, a, alpha, b,
                       n);
    return hipGetLastError() == hipSuccess ? GLM_ATTN_OK : GLM_ATTN_EHIP;
}

const char *glm_attn_version(void) { return "glm_attn 0.1 (gfx950)"; }

}  // extern "C"
