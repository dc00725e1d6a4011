// Host-side C++ mirror of the reference's attention surface; see chatglm_attn.h.
#include "chatglm_attn.h"

#include <hip/hip_runtime.h>

#include <cstring>

namespace chatglm {

#define CHATGLM_CHECK_HIP(call)                                                       \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        CHATGLM_CHECK(e_ == hipSuccess) << "HIP error: " << hipGetErrorString(e_);    \
    } while (0)

#define CHATGLM_CHECK_ATTN(call)                                                                 \
    do {                                                                                         \
        int s_ = (call);                                                                         \
        CHATGLM_CHECK(s_ == GLM_ATTN_OK) << #call << " failed: " << glm_attn_strerror(s_);       \
    } while (0)

size_t dtype_size(DType t) {
    switch (t) {
    case DType::F32:
    case DType::I32:
        return 4;
    case DType::F16:
        return 2;
    case DType::Q4_0:
        return 18;
    case DType::Q4_1:
        return 20;
    case DType::Q5_0:
        return 22;
    case DType::Q5_1:
        return 24;
    case DType::Q8_0:
        return 34;
    }
    return 0;
}

int dtype_block_elems(DType t) {
    switch (t) {
    case DType::Q4_0:
    case DType::Q4_1:
    case DType::Q5_0:
    case DType::Q5_1:
    case DType::Q8_0:
        return 32;
    default:
        return 1;
    }
}

static void set_shape(Tensor *t, DType type, int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3) {
    t->type = type;
    t->ne[0] = ne0;
    t->ne[1] = ne1;
    t->ne[2] = ne2;
    t->ne[3] = ne3;
    t->nb[0] = dtype_size(type);
    t->nb[1] = t->nb[0] * (size_t)(ne0 / dtype_block_elems(type));  // rows of whole blocks, as in ggml
    for (int i = 2; i < 4; i++) {
        t->nb[i] = t->nb[i - 1] * (size_t)t->ne[i - 1];
    }
}

// ---------------------------------------------------------------------------------------------------
ModelContext::ModelContext(int device_, size_t arena_bytes, size_t layer_zone_bytes)
    : device(device_), stream(nullptr) {
    CHATGLM_CHECK_HIP(hipSetDevice(device));
    hipStream_t st;
    CHATGLM_CHECK_HIP(hipStreamCreate(&st));
    stream = st;
    const size_t sizes[3] = {arena_bytes, layer_zone_bytes, layer_zone_bytes};
    for (int z = 0; z < 3; z++) {
        if (sizes[z]) {
            CHATGLM_CHECK_HIP(hipMalloc((void **)&zones_[z].base, sizes[z]));
            zones_[z].bytes = sizes[z];
        }
    }
}

void ModelContext::reserve(size_t arena_bytes, size_t layer_zone_bytes) {
    reset();
    const size_t sizes[3] = {arena_bytes, layer_zone_bytes, layer_zone_bytes};
    CHATGLM_CHECK_HIP(hipSetDevice(device));
    for (int z = 0; z < 3; z++) {
        if (sizes[z] > zones_[z].bytes) {
            if (zones_[z].base) {
                CHATGLM_CHECK_HIP(hipFree(zones_[z].base));
                zones_[z].base = nullptr;
                zones_[z].bytes = 0;
            }
            CHATGLM_CHECK_HIP(hipMalloc((void **)&zones_[z].base, sizes[z]));
            zones_[z].bytes = sizes[z];
        }
    }
}

void ModelContext::begin_layer(int i) {
    if (zones_[1].bytes) {
        zone_ = 1 + (i & 1);
        zones_[zone_].used = 0;
    }
}

ModelContext::~ModelContext() {
    (void)hipSetDevice(device);
    if (attn) {
        glm_attn_destroy(attn);
    }
    if (stream) {
        (void)hipStreamSynchronize((hipStream_t)stream);
        (void)hipStreamDestroy((hipStream_t)stream);
    }
    for (Zone &z : zones_) {
        if (z.base) {
            (void)hipFree(z.base);
        }
    }
}

Tensor *ModelContext::new_tensor(DType type, int64_t ne0, int64_t ne1, int64_t ne2, int64_t ne3) {
    auto t = std::make_unique<Tensor>();
    set_shape(t.get(), type, ne0, ne1, ne2, ne3);
    const size_t bytes = (t->nbytes() + 255) & ~(size_t)255;
    Zone &z = zones_[zone_];
    CHATGLM_CHECK(z.used + bytes <= z.bytes) << "tensor arena exhausted (zone " << zone_ << ", " << z.bytes << " bytes)";
    t->data = z.base + z.used;
    z.used += bytes;
    tensors_.push_back(std::move(t));
    return tensors_.back().get();
}

void ModelContext::reset() {
    // the stream may still read arena tensors of the previous forward
    synchronize();
    tensors_.clear();
    for (Zone &z : zones_) {
        z.used = 0;
    }
    zone_ = 0;
}

void ModelContext::tensor_set(Tensor *t, const void *host, size_t offset, size_t nbytes) {
    CHATGLM_CHECK(offset + nbytes <= t->nbytes()) << "tensor_set out of range";
    CHATGLM_CHECK_HIP(hipMemcpyAsync((char *)t->data + offset, host, nbytes, hipMemcpyHostToDevice, (hipStream_t)stream));
    CHATGLM_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));  // the host buffer may be reused at once
}

void ModelContext::tensor_get(const Tensor *t, void *host, size_t offset, size_t nbytes) {
    CHATGLM_CHECK(offset + nbytes <= t->nbytes()) << "tensor_get out of range";
    CHATGLM_CHECK_HIP(hipMemcpyAsync(host, (const char *)t->data + offset, nbytes, hipMemcpyDeviceToHost, (hipStream_t)stream));
    CHATGLM_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
}

void ModelContext::synchronize() { CHATGLM_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream)); }

int ModelContext::register_layer(const glm_attn_desc &desc, std::shared_ptr<Tensor> k, std::shared_ptr<Tensor> v) {
    CHATGLM_CHECK(attn == nullptr) << "layers must be constructed before the KV buffer is allocated";
    if (!layers_.empty()) {
        const glm_attn_desc &a = layers_.front().desc;
        CHATGLM_CHECK(a.num_attention_heads == desc.num_attention_heads &&
                      a.num_key_value_heads == desc.num_key_value_heads && a.head_size == desc.head_size &&
                      a.max_length == desc.max_length && a.num_virtual_tokens == desc.num_virtual_tokens &&
                      a.rope_type == desc.rope_type && a.rope_theta == desc.rope_theta &&
                      a.attn_mask_type == desc.attn_mask_type && a.interleaved_qkv == desc.interleaved_qkv)
            << "all layers of a model share one attention configuration";
    }
    layers_.push_back(LayerRecord{desc, std::move(k), std::move(v)});
    return (int)layers_.size() - 1;
}

void ModelContext::alloc_kv() {
    if (attn) {
        return;
    }
    CHATGLM_CHECK(!layers_.empty()) << "no attention layer was constructed";
    glm_attn_desc desc = layers_.front().desc;
    desc.num_layers = (int32_t)layers_.size();
    desc.device = device;
    CHATGLM_CHECK_ATTN(glm_attn_create(&desc, &attn));
    for (size_t i = 0; i < layers_.size(); i++) {
        void *k = nullptr, *v = nullptr;
        CHATGLM_CHECK_ATTN(glm_attn_cache_ptrs(attn, (int32_t)i, &k, &v));
        layers_[i].k_cache->data = k;
        layers_[i].v_cache->data = v;
    }
}

// ---------------------------------------------------------------------------------------------------
Linear::Linear(ModelContext *mctx, int in_features, int out_features, bool use_bias, Tensor *tied_weight) {
    CHATGLM_CHECK(mctx->dtype != DType::I32) << "Linear weights are F32, F16 or one of ggml's block-quantised types";
    CHATGLM_CHECK(in_features % dtype_block_elems(mctx->dtype) == 0) << "in_features must be whole blocks of 32";
    glm_linear_desc desc;
    memset(&desc, 0, sizeof(desc));
    desc.struct_size = (int32_t)sizeof(desc);
    desc.in_features = in_features;
    desc.out_features = out_features;
    desc.weight_dtype = (int32_t)mctx->dtype;  // the same numbers as ggml_type
    desc.use_bias = use_bias ? 1 : 0;
    desc.max_rows = mctx->max_rows;
    desc.device = mctx->device;
    if (tied_weight) {
        CHATGLM_CHECK(tied_weight->type == mctx->dtype && tied_weight->ne[0] == in_features &&
                      tied_weight->ne[1] == out_features && tied_weight->data)
            << "tied weight must be an allocated [out_features, in_features] tensor of the context's dtype";
        desc.weight = tied_weight->data;
        desc.weight_bytes = (int64_t)tied_weight->nbytes();
    }
    glm_linear *raw = nullptr;
    CHATGLM_CHECK_ATTN(glm_linear_create(&desc, &raw));
    impl_ = std::shared_ptr<glm_linear>(raw, glm_linear_destroy);
    void *w = nullptr;
    float *b = nullptr;
    CHATGLM_CHECK_ATTN(glm_linear_params(raw, &w, &b));
    weight_ = std::make_shared<Tensor>();
    set_shape(weight_.get(), mctx->dtype, in_features, out_features, 1, 1);
    weight_->data = w;
    weight = weight_.get();
    if (use_bias) {
        bias_ = std::make_shared<Tensor>();
        set_shape(bias_.get(), DType::F32, out_features, 1, 1, 1);
        bias_->data = b;
        bias = bias_.get();
    }
}

Tensor *Linear::forward(ModelContext *mctx, Tensor *input) const {
    CHATGLM_CHECK(impl_) << "Linear was not constructed with a ModelContext";
    CHATGLM_CHECK(input && input->type == DType::F32 && input->ne[0] == in_features())
        << "input must be fp32 [seqlen, " << in_features() << "]";
    const int rows = (int)(input->ne[1] * input->ne[2] * input->ne[3]);
    Tensor *out = mctx->new_tensor(DType::F32, out_features(), input->ne[1], input->ne[2], input->ne[3]);
    const int st = glm_linear_forward(impl_.get(), static_cast<const float *>(input->data), rows,
                                      static_cast<float *>(out->data), mctx->stream);
    CHATGLM_CHECK(st == GLM_ATTN_OK) << "glm_linear_forward failed: " << glm_attn_strerror(st) << " (rows " << rows
                                     << ", max_rows " << mctx->max_rows << ")";
    return out;
}

void Linear::commit(ModelContext *mctx) {
    CHATGLM_CHECK(impl_) << "Linear was not constructed with a ModelContext";
    CHATGLM_CHECK_ATTN(glm_linear_commit(impl_.get(), mctx->stream));
    void *w = nullptr;
    CHATGLM_CHECK_ATTN(glm_linear_params(impl_.get(), &w, nullptr));
    weight_->data = w;
}

static glm_linear_fusion make_fusion(const Fused &f) {
    glm_linear_fusion fu;
    std::memset(&fu, 0, sizeof(fu));
    fu.struct_size = (int32_t)sizeof(fu);
    if (f.norm) {
        fu.prologue = GLM_LINEAR_PRO_RMS_NORM;
        fu.norm_weight = static_cast<const float *>(f.norm->weight->data);
        fu.norm_eps = f.norm->eps;
    }
    if (f.gate_up) {
        fu.prologue = GLM_LINEAR_PRO_GATED_ACT;
        fu.up = static_cast<const float *>(f.gate_up->data);
        fu.activation = f.act == ActivationType::GELU ? GLM_BLOCK_ACT_GELU : GLM_BLOCK_ACT_SILU;
    }
    if (f.residual) {
        fu.residual = static_cast<const float *>(f.residual->data);
        fu.residual_scale = f.residual_scale;
    }
    return fu;
}

Tensor *Linear::forward(ModelContext *mctx, Tensor *input, const Fused &f) const {
    if (!f.norm && !f.residual && !f.gate_up) {
        return forward(mctx, input);
    }
    CHATGLM_CHECK(!(f.norm && f.gate_up)) << "a projection takes a norm or a gate in front, not both";
    CHATGLM_CHECK(!f.gate_up || f.gate_up->nelements() == input->nelements()) << "gate and up differ in size";
    CHATGLM_CHECK(impl_) << "Linear was not constructed with a ModelContext";
    CHATGLM_CHECK(input && input->type == DType::F32 && input->ne[0] == in_features())
        << "input must be fp32 [seqlen, " << in_features() << "]";
    CHATGLM_CHECK(!f.norm || !f.norm->inplace) << "an in-place norm cannot run inside the projection";
    const int rows = (int)(input->ne[1] * input->ne[2] * input->ne[3]);
    CHATGLM_CHECK(!f.residual || f.residual->nelements() == (int64_t)rows * out_features()) << "residual shape";
    const size_t mark = mctx->arena_mark();
    Tensor *out = mctx->new_tensor(DType::F32, out_features(), input->ne[1], input->ne[2], input->ne[3]);
    const glm_linear_fusion fu = make_fusion(f);
    const int st = glm_linear_forward_fused(impl_.get(), &fu, static_cast<const float *>(input->data), rows,
                                            static_cast<float *>(out->data), mctx->stream);
    if (st == GLM_ATTN_OK) {
        return out;
    }
    CHATGLM_CHECK(st == GLM_ATTN_EUNSUPPORTED) << "glm_linear_forward_fused failed: " << glm_attn_strerror(st);
    mctx->arena_release(mark);
    Tensor *in = f.norm ? f.norm->forward(mctx, input) : input;
    if (f.gate_up) {
        in = mctx->new_tensor(DType::F32, input->ne[0], input->ne[1], input->ne[2], input->ne[3]);
        CHATGLM_CHECK_ATTN(glm_block_gated_activation(static_cast<const float *>(input->data),
                                                      static_cast<const float *>(f.gate_up->data), input->nelements(),
                                                      f.act == ActivationType::GELU ? GLM_BLOCK_ACT_GELU : GLM_BLOCK_ACT_SILU,
                                                      static_cast<float *>(in->data), mctx->stream));
    }
    out = forward(mctx, in);
    return f.residual ? scale_add(mctx, f.residual, f.residual_scale, out) : out;
}

// device storage of a parameter tensor, owned by the tensor's shared_ptr
static std::shared_ptr<Tensor> new_parameter(ModelContext *mctx, DType type, int64_t ne0) {
    CHATGLM_CHECK_HIP(hipSetDevice(mctx->device));
    void *p = nullptr;
    CHATGLM_CHECK_HIP(hipMalloc(&p, (size_t)ne0 * dtype_size(type)));
    CHATGLM_CHECK_HIP(hipMemset(p, 0, (size_t)ne0 * dtype_size(type)));
    std::shared_ptr<Tensor> t(new Tensor(), [](Tensor *x) {
        (void)hipFree(x->data);
        delete x;
    });
    set_shape(t.get(), type, ne0, 1, 1, 1);
    t->data = p;
    return t;
}

static Tensor *norm_output(ModelContext *mctx, Tensor *input, bool inplace) {
    return inplace ? input : mctx->new_tensor(DType::F32, input->ne[0], input->ne[1], input->ne[2], input->ne[3]);
}

LayerNorm::LayerNorm(ModelContext *mctx, int normalized_shape, bool inplace_, float eps_)
    : inplace(inplace_), eps(eps_) {
    weight_ = new_parameter(mctx, DType::F32, normalized_shape);
    bias_ = new_parameter(mctx, DType::F32, normalized_shape);
    weight = weight_.get();
    bias = bias_.get();
}

Tensor *LayerNorm::forward(ModelContext *mctx, Tensor *input) const {
    CHATGLM_CHECK(weight && input && input->type == DType::F32 && input->ne[0] == weight->ne[0])
        << "input must be fp32 [seqlen, normalized_shape]";
    Tensor *out = norm_output(mctx, input, inplace);
    CHATGLM_CHECK_ATTN(glm_block_layer_norm(static_cast<const float *>(input->data),
                                            static_cast<const float *>(weight->data),
                                            static_cast<const float *>(bias->data), eps,
                                            (int32_t)(input->nelements() / input->ne[0]), (int32_t)input->ne[0],
                                            static_cast<float *>(out->data), mctx->stream));
    return out;
}

RMSNorm::RMSNorm(ModelContext *mctx, int normalized_shape, bool inplace_, float eps_) : inplace(inplace_), eps(eps_) {
    weight_ = new_parameter(mctx, DType::F32, normalized_shape);
    weight = weight_.get();
}

Tensor *RMSNorm::forward(ModelContext *mctx, Tensor *input) const {
    CHATGLM_CHECK(weight && input && input->type == DType::F32 && input->ne[0] == weight->ne[0])
        << "input must be fp32 [seqlen, normalized_shape]";
    Tensor *out = norm_output(mctx, input, inplace);
    CHATGLM_CHECK_ATTN(glm_block_rms_norm(static_cast<const float *>(input->data),
                                          static_cast<const float *>(weight->data), eps,
                                          (int32_t)(input->nelements() / input->ne[0]), (int32_t)input->ne[0],
                                          static_cast<float *>(out->data), mctx->stream));
    return out;
}

static int32_t activation_code(ActivationType a) {
    return a == ActivationType::GELU ? GLM_BLOCK_ACT_GELU : GLM_BLOCK_ACT_SILU;
}

Tensor *BasicMLP::forward(ModelContext *mctx, Tensor *hidden_states, const Fused &f) const {
    Fused in, out;
    in.norm = f.norm;
    out.residual = f.residual;
    out.residual_scale = f.residual_scale;
    hidden_states = dense_h_to_4h.forward(mctx, hidden_states, in);
    float *h = static_cast<float *>(hidden_states->data);
    CHATGLM_CHECK_ATTN(
        glm_block_activation_forward(h, hidden_states->nelements(), activation_code(hidden_act), h, mctx->stream));
    return dense_4h_to_h.forward(mctx, hidden_states, out);
}

Tensor *BasicGLU::forward(ModelContext *mctx, Tensor *hidden_states, const Fused &f) const {
    CHATGLM_CHECK(hidden_states && hidden_states->type == DType::F32 && hidden_states->ne[0] == gate_proj.in_features())
        << "input must be fp32 [seqlen, hidden_size]";
    Fused in, out;
    in.norm = f.norm;
    out.residual = f.residual;
    out.residual_scale = f.residual_scale;
    const int rows = (int)(hidden_states->ne[1] * hidden_states->ne[2] * hidden_states->ne[3]);
    // chatglm.cpp:465-473: act(gate_proj(x)) * up_proj(x), in one launch where the library can
    const size_t mark = mctx->arena_mark();
    Tensor *mid = mctx->new_tensor(DType::F32, gate_proj.out_features(), hidden_states->ne[1], hidden_states->ne[2],
                                   hidden_states->ne[3]);
    glm_linear_fusion fu = make_fusion(in);
    fu.activation = activation_code(hidden_act);
    const int st = glm_linear_forward_glu(gate_proj.handle(), up_proj.handle(), &fu,
                                          static_cast<const float *>(hidden_states->data), rows,
                                          static_cast<float *>(mid->data), mctx->stream);
    if (st != GLM_ATTN_OK) {
        CHATGLM_CHECK(st == GLM_ATTN_EUNSUPPORTED) << "glm_linear_forward_glu failed: " << glm_attn_strerror(st);
        // more than a token or two: three GEMMs; the norm rides in front of the first two, the gate in front of
        // the third, the residual behind it
        mctx->arena_release(mark);
        Tensor *gate = gate_proj.forward(mctx, hidden_states, in);
        out.gate_up = up_proj.forward(mctx, hidden_states, in);
        out.act = hidden_act;
        return down_proj.forward(mctx, gate, out);
    }
    return down_proj.forward(mctx, mid, out);
}

Tensor *scale_add(ModelContext *mctx, Tensor *a, float alpha, Tensor *b) {
    CHATGLM_CHECK(a && b && a->type == DType::F32 && b->type == DType::F32 && a->nelements() == b->nelements())
        << "scale_add needs two fp32 tensors of one size";
    Tensor *out = mctx->new_tensor(DType::F32, a->ne[0], a->ne[1], a->ne[2], a->ne[3]);
    CHATGLM_CHECK_ATTN(glm_attn_scale_add(static_cast<float *>(out->data), static_cast<const float *>(a->data), alpha,
                                          static_cast<const float *>(b->data), a->nelements(), mctx->stream));
    return out;
}

// ---------------------------------------------------------------------------------------------------
BasicAttention::BasicAttention(ModelContext *mctx, int hidden_size_, int num_attention_heads_,
                               int num_key_value_heads_, int max_length_, bool use_qkv_bias, bool use_dense_bias,
                               bool interleaved_qkv_, RopeType rope_type_, float rope_theta_,
                               AttentionMaskType attn_mask_type_, int num_virtual_tokens_)
    : num_attention_heads(num_attention_heads_), num_key_value_heads(num_key_value_heads_),
      interleaved_qkv(interleaved_qkv_), rope_type(rope_type_), rope_theta(rope_theta_),
      attn_mask_type(attn_mask_type_), num_virtual_tokens(num_virtual_tokens_), hidden_size(hidden_size_),
      max_length(max_length_) {
    CHATGLM_CHECK(num_attention_heads > 0 && hidden_size % num_attention_heads == 0) << "bad head count";
    // chatglm.h:449-451
    query_key_value = Linear(mctx, hidden_size, hidden_size + 2 * (hidden_size / num_attention_heads) * num_key_value_heads,
                             use_qkv_bias);
    dense = Linear(mctx, hidden_size, hidden_size, use_dense_bias);
    const int head_size = hidden_size / num_attention_heads;
    // chatglm.h:452-455: k_cache ne = [d, L, kvh], v_cache ne = [L, d, kvh], both F16
    k_cache_ = std::make_shared<Tensor>();
    v_cache_ = std::make_shared<Tensor>();
    set_shape(k_cache_.get(), DType::F16, head_size, max_length + num_virtual_tokens, num_key_value_heads, 1);
    set_shape(v_cache_.get(), DType::F16, max_length + num_virtual_tokens, head_size, num_key_value_heads, 1);
    k_cache = k_cache_.get();
    v_cache = v_cache_.get();

    glm_attn_desc desc;
    glm_attn_default_desc(&desc);
    desc.num_attention_heads = num_attention_heads;
    desc.num_key_value_heads = num_key_value_heads;
    desc.head_size = head_size;
    desc.max_length = max_length;
    desc.num_virtual_tokens = num_virtual_tokens;
    desc.rope_type = (int32_t)rope_type;
    desc.rope_theta = rope_theta;
    desc.attn_mask_type = attn_mask_type == AttentionMaskType::CAUSAL ? GLM_ATTN_MASK_CAUSAL : GLM_ATTN_MASK_CHATGLM;
    desc.interleaved_qkv = interleaved_qkv ? 1 : 0;
    layer_id = mctx->register_layer(desc, k_cache_, v_cache_);
}

Tensor *BasicAttention::forward(ModelContext *mctx, Tensor *hidden_states, Tensor *attention_mask,
                                Tensor *position_ids, int n_past, const Fused &f) const {
    Fused in, out;
    in.norm = f.norm;
    out.residual = f.residual;
    out.residual_scale = f.residual_scale;
    Tensor *qkv = query_key_value.forward(mctx, hidden_states, in);  // chatglm.cpp:629
    Tensor *context_layer = attend(mctx, qkv, attention_mask, position_ids, n_past);
    return dense.forward(mctx, context_layer, out);  // chatglm.cpp:719
}

Tensor *BasicAttention::attend(ModelContext *mctx, Tensor *qkv, Tensor *attention_mask, Tensor *position_ids,
                               int n_past, const int32_t *position_ids_host) const {
    CHATGLM_CHECK(layer_id >= 0) << "attention layer was not constructed with a ModelContext";
    const int head_size = hidden_size / num_attention_heads;
    const int64_t width = (int64_t)(num_attention_heads + 2 * num_key_value_heads) * head_size;
    CHATGLM_CHECK(qkv && qkv->type == DType::F32 && qkv->ne[0] == width) << "qkv must be fp32 [s][(h + 2 kvh) d]";
    const int qlen = (int)qkv->ne[1];
    // chatglm.cpp:637
    CHATGLM_CHECK(!interleaved_qkv || num_attention_heads == num_key_value_heads)
        << "interleaved qkv is not supported for GQA";
    if (rope_type != RopeType::DISABLED) {
        const int64_t want = rope_type == RopeType::CHATGLM ? 2 * qlen : qlen;  // chatglm.cpp:1144-1145, 1321-1322
        CHATGLM_CHECK(position_ids && position_ids->type == DType::I32 && position_ids->ne[0] == want)
            << "invalid position ids size " << (position_ids ? position_ids->ne[0] : -1);
    }
    mctx->alloc_kv();
    Tensor *out = mctx->new_tensor(DType::F32, hidden_size, qlen);  // [s, #h * d], chatglm.cpp:717
    const int st = glm_attn_forward(mctx->attn, layer_id, static_cast<const float *>(qkv->data),
                                    (int64_t)(qkv->nb[1] / sizeof(float)),
                                    attention_mask ? static_cast<const float *>(attention_mask->data) : nullptr,
                                    position_ids ? static_cast<const int32_t *>(position_ids->data) : nullptr,
                                    position_ids_host, qlen, n_past, static_cast<float *>(out->data), mctx->stream);
    CHATGLM_CHECK(st == GLM_ATTN_OK) << "glm_attn_forward failed: " << glm_attn_strerror(st) << " (layer " << layer_id
                                     << ", qlen " << qlen << ", n_past " << n_past << ")";
    return out;
}

// ---------------------------------------------------------------------------------------------------
std::vector<int32_t> glm2_position_ids(int qlen, int n_past) {
    std::vector<int32_t> v((size_t)qlen);
    CHATGLM_CHECK_ATTN(glm_attn_position_ids_glm2(qlen, n_past, v.data()));
    return v;
}

std::vector<int32_t> glm_position_ids(int qlen, int n_past, int n_ctx) {
    std::vector<int32_t> v((size_t)qlen * 2);
    CHATGLM_CHECK_ATTN(glm_attn_position_ids_glm(qlen, n_past, n_ctx, v.data()));
    return v;
}

std::vector<float> glm_attention_mask(int qlen, int kvlen) {
    std::vector<float> v((size_t)qlen * kvlen);
    CHATGLM_CHECK_ATTN(glm_attn_attention_mask_glm(qlen, kvlen, v.data()));
    return v;
}

void load_prefix_cache(ModelContext *mctx, const BasicAttention &attn, const Tensor *past_key_values) {
    CHATGLM_CHECK(past_key_values && past_key_values->type == DType::F16) << "past_key_values must be fp16";
    mctx->alloc_kv();
    CHATGLM_CHECK_ATTN(glm_attn_load_prefix_cache(mctx->attn, attn.layer_id, past_key_values->data, mctx->stream));
}

}  // namespace chatglm
