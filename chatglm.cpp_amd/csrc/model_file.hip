// Reader of the reference's "ggml" model files (include/glm_model_file.h) and the embedding lookup that
// consumes the first tensor of such a file (glm_block_embedding, include/glm_block.h).
//
// The file is mapped read-only and parsed once at open: header, config record (three layouts), tokenizer byte
// range, then the tensor records to the end of the file (chatglm.cpp:357-391, 1754-1848).  Every read is bounds
// checked against the mapping, which the reference does not do: a truncated file is an error here, not a fault.
#include <fcntl.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <string>
#include <unordered_map>
#include <vector>

#include "glm_attn.h"
#include "glm_block.h"
#include "glm_model_file.h"

namespace {

thread_local std::string g_last_error;

int fail(int status, const char *fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof(buf), fmt, ap);
    va_end(ap);
    g_last_error = buf;
    return status;
}

// a tensor name as it may appear in a message: the file is outside input, its bytes need not be text
std::string printable(const std::string &name) {
    std::string out = name.substr(0, 80);
    for (char &ch : out) {
        if (ch < 0x20 || ch > 0x7e) ch = '?';
    }
    return out;
}

// ggml's block-quantised layouts: 32 elements per block (ggml-common.h block_q4_0 ... block_q8_0)
bool type_traits(int32_t dtype, int64_t *block_elems, int64_t *block_bytes) {
    switch (dtype) {
        case GLM_MODEL_F32: *block_elems = 1; *block_bytes = 4; return true;
        case GLM_MODEL_F16: *block_elems = 1; *block_bytes = 2; return true;
        case GLM_MODEL_Q4_0: *block_elems = 32; *block_bytes = 2 + 16; return true;
        case GLM_MODEL_Q4_1: *block_elems = 32; *block_bytes = 2 + 2 + 16; return true;
        case GLM_MODEL_Q5_0: *block_elems = 32; *block_bytes = 2 + 4 + 16; return true;
        case GLM_MODEL_Q5_1: *block_elems = 32; *block_bytes = 2 + 2 + 4 + 16; return true;
        case GLM_MODEL_Q8_0: *block_elems = 32; *block_bytes = 2 + 32; return true;
        default: return false;
    }
}

struct TensorRecord {
    std::string name;
    int32_t dtype, ndim;
    int64_t ne[4];
    int64_t offset, nbytes;
};

// the three record layouts, all of 4-byte fields (chatglm.h:49-86)
struct RecordV1 {
    int32_t dtype, vocab_size, hidden_size, num_attention_heads, num_hidden_layers, intermediate_size, max_length,
        bos_token_id, eos_token_id, pad_token_id, sep_token_id;
};
struct RecordV1GQA {
    RecordV1 base;
    int32_t num_key_value_heads;
};
struct RecordV2 {
    int32_t dtype, vocab_size, hidden_size, num_attention_heads, num_key_value_heads, num_hidden_layers,
        intermediate_size;
    float norm_eps;
    int32_t num_virtual_tokens;
    float rope_theta;
    int32_t max_length, eos_token_id, pad_token_id;
};

}  // namespace

struct glm_model_file {
    char *data = nullptr;
    size_t size = 0;
    glm_model_config config;
    std::vector<TensorRecord> tensors;
    std::unordered_map<std::string, int> by_name;
    // pinned staging for uploads, allocated at the first upload
    void *staging = nullptr;
    size_t staging_bytes = 0;
};

namespace {

struct Cursor {
    const char *data;
    size_t size, pos;
    bool take(void *dst, size_t n) {
        if (n > size - pos) return false;
        memcpy(dst, data + pos, n);
        pos += n;
        return true;
    }
    template <typename T>
    bool read(T *v) { return take(v, sizeof(T)); }
};

void derive_config(glm_model_config *c) {
    // ModelConfig::ModelConfig (chatglm.h:121-138)
    if (c->model_type == GLM_MODEL_CHATGLM) {
        c->hidden_act = GLM_BLOCK_ACT_GELU;
        c->use_qkv_bias = 1;
        c->use_dense_bias = 1;
        c->interleaved_qkv = 1;
        c->tie_word_embeddings = 1;
        c->rope_type = GLM_ATTN_ROPE_CHATGLM;
        c->attn_mask_type = GLM_ATTN_MASK_CHATGLM;
    } else {
        c->hidden_act = GLM_BLOCK_ACT_SILU;
        c->use_qkv_bias = 1;
        c->use_dense_bias = 0;
        c->interleaved_qkv = 0;
        c->tie_word_embeddings = 0;
        c->rope_type = GLM_ATTN_ROPE_CHATGLM2;
        c->attn_mask_type = GLM_ATTN_MASK_CAUSAL;
    }
}

void from_v1(glm_model_config *c, const RecordV1 &r, int32_t kvh) {
    // chatglm.h:140-153: norm_eps 1e-5, rope_theta 10000, no virtual tokens (chatglm.cpp:1779,1802)
    c->dtype = r.dtype;
    c->vocab_size = r.vocab_size;
    c->hidden_size = r.hidden_size;
    c->num_attention_heads = r.num_attention_heads;
    c->num_key_value_heads = kvh;
    c->num_hidden_layers = r.num_hidden_layers;
    c->intermediate_size = r.intermediate_size;
    c->norm_eps = 1e-5f;
    c->rope_theta = 10000.f;
    c->num_virtual_tokens = 0;
    c->max_length = r.max_length;
    c->bos_token_id = r.bos_token_id;
    c->eos_token_id = r.eos_token_id;
    c->pad_token_id = r.pad_token_id;
    c->sep_token_id = r.sep_token_id;
}

void from_v2(glm_model_config *c, const RecordV2 &r) {
    // chatglm.h:155-160
    c->dtype = r.dtype;
    c->vocab_size = r.vocab_size;
    c->hidden_size = r.hidden_size;
    c->num_attention_heads = r.num_attention_heads;
    c->num_key_value_heads = r.num_key_value_heads;
    c->num_hidden_layers = r.num_hidden_layers;
    c->intermediate_size = r.intermediate_size;
    c->norm_eps = r.norm_eps;
    c->rope_theta = r.rope_theta;
    c->num_virtual_tokens = r.num_virtual_tokens;
    c->max_length = r.max_length;
    c->bos_token_id = -1;
    c->eos_token_id = r.eos_token_id;
    c->pad_token_id = r.pad_token_id;
    c->sep_token_id = -1;
}

int parse(glm_model_file *f) {
    Cursor cur{f->data, f->size, 0};
    char magic[4];
    if (!cur.take(magic, 4) || memcmp(magic, "ggml", 4) != 0) {
        return fail(GLM_ATTN_EINVAL, "model file is broken (bad magic)");  // chatglm.cpp:1769
    }
    glm_model_config &c = f->config;
    memset(&c, 0, sizeof(c));
    c.struct_size = (int32_t)sizeof(c);
    if (!cur.read(&c.model_type) || !cur.read(&c.version)) return fail(GLM_ATTN_EINVAL, "model file is truncated (header)");
    bool ok = true;
    if (c.model_type == GLM_MODEL_CHATGLM) {
        if (c.version == 1) {
            RecordV1 r;
            ok = cur.read(&r);
            if (ok) from_v1(&c, r, r.num_attention_heads);
        } else if (c.version == 2) {
            RecordV2 r;
            ok = cur.read(&r);
            if (ok) from_v2(&c, r);
        } else {
            return fail(GLM_ATTN_EINVAL, "only support version 1 or 2 for now but got %d", c.version);
        }
    } else if (c.model_type == GLM_MODEL_CHATGLM2 || c.model_type == GLM_MODEL_CHATGLM3) {
        if (c.version == 1) {
            RecordV1GQA r;
            ok = cur.read(&r);
            if (ok) from_v1(&c, r.base, r.num_key_value_heads);
        } else if (c.version == 2) {
            RecordV2 r;
            ok = cur.read(&r);
            if (ok) from_v2(&c, r);
        } else {
            return fail(GLM_ATTN_EINVAL, "only support version 1 or 2 for now but got %d", c.version);
        }
    } else if (c.model_type == GLM_MODEL_CHATGLM4) {
        if (c.version != 2) return fail(GLM_ATTN_EINVAL, "only support version 2 for now but got %d", c.version);
        RecordV2 r;
        ok = cur.read(&r);
        if (ok) from_v2(&c, r);
    } else {
        return fail(GLM_ATTN_EINVAL, "invalid model type %d", c.model_type);  // chatglm.cpp:1845
    }
    if (!ok) return fail(GLM_ATTN_EINVAL, "model file is truncated (config record)");
    derive_config(&c);
    if (c.vocab_size <= 0 || c.hidden_size <= 0 || c.num_attention_heads <= 0 || c.num_key_value_heads <= 0 ||
        c.num_hidden_layers <= 0 || c.intermediate_size <= 0 || c.max_length <= 0 || c.num_virtual_tokens < 0 ||
        c.hidden_size % c.num_attention_heads != 0) {
        return fail(GLM_ATTN_EINVAL, "model file is broken (config record holds impossible sizes)");
    }
    int32_t tok_size = 0;
    if (!cur.read(&tok_size) || tok_size < 0 || (size_t)tok_size > cur.size - cur.pos) {
        return fail(GLM_ATTN_EINVAL, "model file is truncated (tokenizer data)");
    }
    c.tokenizer_offset = (int64_t)cur.pos;
    c.tokenizer_size = tok_size;
    cur.pos += (size_t)tok_size;

    // "assume state dict is stored at the back of file" (chatglm.cpp:362)
    while (cur.pos < cur.size) {
        TensorRecord t;
        int32_t name_size = 0;
        if (!cur.read(&name_size) || name_size <= 0 || (size_t)name_size > cur.size - cur.pos) {
            return fail(GLM_ATTN_EINVAL, "model file is broken (tensor name at byte %zu)", cur.pos);
        }
        t.name.assign(cur.data + cur.pos, (size_t)name_size);
        cur.pos += (size_t)name_size;
        if (!cur.read(&t.ndim) || t.ndim <= 0 || t.ndim > 4) {  // chatglm.cpp:371
            return fail(GLM_ATTN_EINVAL, "model file is broken (tensor %s: bad number of dimensions)", printable(t.name).c_str());
        }
        for (int i = 0; i < 4; i++) t.ne[i] = 1;
        for (int i = t.ndim - 1; i >= 0; i--) {  // outermost first in the file, ne[0] innermost
            int32_t n = 0;
            if (!cur.read(&n) || n <= 0) {
                return fail(GLM_ATTN_EINVAL, "model file is broken (tensor %s: bad shape)", printable(t.name).c_str());
            }
            t.ne[i] = n;
        }
        int64_t block_elems = 0, block_bytes = 0;
        if (!cur.read(&t.dtype) || !type_traits(t.dtype, &block_elems, &block_bytes)) {
            return fail(GLM_ATTN_EINVAL, "model file is broken (tensor %s: unknown ggml type)", printable(t.name).c_str());
        }
        if (t.ne[0] % block_elems != 0) {
            return fail(GLM_ATTN_EINVAL, "model file is broken (tensor %s: row of %lld elements in blocks of %lld)",
                        printable(t.name).c_str(), (long long)t.ne[0], (long long)block_elems);
        }
        // ggml_nbytes of a contiguous tensor.  Every factor comes from the file: a product that does not
        // fit 63 bits must not wrap into a size that passes the check against the mapping below.
        t.nbytes = t.ne[0] / block_elems;
        bool overflow = __builtin_mul_overflow(t.nbytes, block_bytes, &t.nbytes);
        for (int i = 1; i < 4; i++) {
            overflow = overflow || __builtin_mul_overflow(t.nbytes, t.ne[i], &t.nbytes);
        }
        if (overflow) {
            return fail(GLM_ATTN_EINVAL, "model file is broken (tensor %s: bad shape)", printable(t.name).c_str());
        }
        t.offset = (int64_t)((cur.pos + 15) & ~(size_t)15);                            // chatglm.cpp:381-382
        if ((size_t)t.offset > cur.size || (size_t)t.nbytes > cur.size - (size_t)t.offset) {
            return fail(GLM_ATTN_EINVAL, "model file is truncated (data of tensor %s)", printable(t.name).c_str());
        }
        cur.pos = (size_t)(t.offset + t.nbytes);
        f->by_name.emplace(t.name, (int)f->tensors.size());
        f->tensors.push_back(std::move(t));
    }
    return GLM_ATTN_OK;
}

void fill_tensor(const TensorRecord &t, glm_model_tensor *out) {
    out->dtype = t.dtype;
    out->ndim = t.ndim;
    out->reserved = 0;
    for (int i = 0; i < 4; i++) out->ne[i] = t.ne[i];
    out->offset = t.offset;
    out->nbytes = t.nbytes;
    out->name = t.name.c_str();
}

constexpr size_t kStagingBytes = 32u << 20;

}  // namespace

extern "C" {

const char *glm_model_file_last_error(void) { return g_last_error.c_str(); }

int glm_model_file_open(const char *path, glm_model_file **out_file) {
    if (!path || !out_file) return fail(GLM_ATTN_EINVAL, "null argument");
    *out_file = nullptr;
    const int fd = open(path, O_RDONLY);
    if (fd < 0) return fail(GLM_ATTN_EINVAL, "cannot open file %s: %s", path, strerror(errno));  // chatglm.cpp:300
    struct stat sb;
    if (fstat(fd, &sb) != 0) {
        const int e = errno;
        close(fd);
        return fail(GLM_ATTN_EINVAL, "cannot stat file %s: %s", path, strerror(e));
    }
    if (sb.st_size < 12) {
        close(fd);
        return fail(GLM_ATTN_EINVAL, "model file is broken (%lld bytes)", (long long)sb.st_size);
    }
    void *data = mmap(nullptr, (size_t)sb.st_size, PROT_READ, MAP_SHARED, fd, 0);
    const int map_errno = errno;
    close(fd);
    if (data == MAP_FAILED) return fail(GLM_ATTN_ENOMEM, "cannot map file %s: %s", path, strerror(map_errno));
    glm_model_file *f = new (std::nothrow) glm_model_file();
    if (!f) {
        munmap(data, (size_t)sb.st_size);
        return fail(GLM_ATTN_ENOMEM, "out of memory");
    }
    f->data = static_cast<char *>(data);
    f->size = (size_t)sb.st_size;
    const int st = parse(f);
    if (st != GLM_ATTN_OK) {
        glm_model_file_close(f);
        return st;
    }
    *out_file = f;
    return GLM_ATTN_OK;
}

void glm_model_file_close(glm_model_file *f) {
    if (!f) return;
    if (f->staging) (void)hipHostFree(f->staging);
    if (f->data) munmap(f->data, f->size);
    delete f;
}

int glm_model_file_config(const glm_model_file *f, glm_model_config *out) {
    if (!f || !out) return fail(GLM_ATTN_EINVAL, "null argument");
    if (out->struct_size != (int32_t)sizeof(glm_model_config)) return fail(GLM_ATTN_EINVAL, "glm_model_config.struct_size");
    *out = f->config;
    return GLM_ATTN_OK;
}

int glm_model_file_data(const glm_model_file *f, const void **out_data, int64_t *out_size) {
    if (!f || !out_data || !out_size) return fail(GLM_ATTN_EINVAL, "null argument");
    *out_data = f->data;
    *out_size = (int64_t)f->size;
    return GLM_ATTN_OK;
}

int glm_model_file_tensor_count(const glm_model_file *f) { return f ? (int)f->tensors.size() : 0; }

int glm_model_file_tensor(const glm_model_file *f, int32_t index, glm_model_tensor *out) {
    if (!f || !out) return fail(GLM_ATTN_EINVAL, "null argument");
    if (out->struct_size != (int32_t)sizeof(glm_model_tensor)) return fail(GLM_ATTN_EINVAL, "glm_model_tensor.struct_size");
    if (index < 0 || index >= (int32_t)f->tensors.size()) return fail(GLM_ATTN_ERANGE, "tensor index %d of %zu", index, f->tensors.size());
    fill_tensor(f->tensors[(size_t)index], out);
    return GLM_ATTN_OK;
}

int glm_model_file_find(const glm_model_file *f, const char *name, glm_model_tensor *out) {
    if (!f || !name || !out) return fail(GLM_ATTN_EINVAL, "null argument");
    if (out->struct_size != (int32_t)sizeof(glm_model_tensor)) return fail(GLM_ATTN_EINVAL, "glm_model_tensor.struct_size");
    auto it = f->by_name.find(name);
    if (it == f->by_name.end()) return fail(GLM_ATTN_ERANGE, "no tensor named %s", name);
    fill_tensor(f->tensors[(size_t)it->second], out);
    out->reserved = it->second;  // its index, for glm_model_file_upload
    return GLM_ATTN_OK;
}

int glm_model_file_upload(const glm_model_file *cf, int32_t index, int64_t src_offset, int64_t nbytes, void *device_dst,
                          void *stream_) {
    glm_model_file *f = const_cast<glm_model_file *>(cf);
    if (!f || !device_dst) return fail(GLM_ATTN_EINVAL, "null argument");
    if (index < 0 || index >= (int32_t)f->tensors.size()) return fail(GLM_ATTN_ERANGE, "tensor index %d of %zu", index, f->tensors.size());
    const TensorRecord &t = f->tensors[(size_t)index];
    if (src_offset < 0 || nbytes < 0 || src_offset > t.nbytes || nbytes > t.nbytes - src_offset) {
        return fail(GLM_ATTN_ERANGE, "bytes [%lld, %lld) of tensor %s, which holds %lld", (long long)src_offset,
                    (long long)(src_offset + nbytes), t.name.c_str(), (long long)t.nbytes);
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (!f->staging) {
        // two halves: one is filled from the mapping while the other is on its way to the device
        if (hipHostMalloc(&f->staging, kStagingBytes, hipHostMallocDefault) != hipSuccess) {
            f->staging = nullptr;
            return fail(GLM_ATTN_ENOMEM, "cannot allocate %zu bytes of pinned memory", kStagingBytes);
        }
        f->staging_bytes = kStagingBytes;
    }
    const size_t half = f->staging_bytes / 2;
    hipEvent_t done[2] = {nullptr, nullptr};
    for (auto &e : done) {
        if (hipEventCreateWithFlags(&e, hipEventDisableTiming) != hipSuccess) return fail(GLM_ATTN_EHIP, "hipEventCreate failed");
    }
    const char *src = f->data + t.offset + src_offset;
    char *dst = static_cast<char *>(device_dst);
    int status = GLM_ATTN_OK;
    bool used[2] = {false, false};
    int which = 0;
    for (int64_t off = 0; off < nbytes; off += (int64_t)half, which ^= 1) {
        const size_t n = (size_t)std::min<int64_t>((int64_t)half, nbytes - off);
        char *stage = static_cast<char *>(f->staging) + (size_t)which * half;
        if (used[which] && hipEventSynchronize(done[which]) != hipSuccess) {
            status = fail(GLM_ATTN_EHIP, "hipEventSynchronize failed");
            break;
        }
        memcpy(stage, src + off, n);
        if (hipMemcpyAsync(dst + off, stage, n, hipMemcpyHostToDevice, stream) != hipSuccess ||
            hipEventRecord(done[which], stream) != hipSuccess) {
            status = fail(GLM_ATTN_EHIP, "copy of tensor %s to the device failed: %s", t.name.c_str(),
                          hipGetErrorString(hipGetLastError()));
            break;
        }
        used[which] = true;
    }
    if (hipStreamSynchronize(stream) != hipSuccess && status == GLM_ATTN_OK) {
        status = fail(GLM_ATTN_EHIP, "copy of tensor %s to the device failed", printable(t.name).c_str());
    }
    for (auto &e : done) (void)hipEventDestroy(e);
    return status;
}

}  // extern "C"

// ---------------------------------------------------------------- embedding lookup

namespace {

// ggml_get_rows (Embedding::forward, chatglm.cpp:413-416): out[t][:] = float(weight[ids[t]][:]).
// One workgroup per token; ids outside [0, rows) give a row of NaN rather than a stray read.
template <bool F16>
__global__ __launch_bounds__(256) void embedding_kernel(const void *weight, const int32_t *ids, int64_t rows, int dim,
                                                        float *out) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    float *o = out + (int64_t)t * dim;
    if (id < 0 || id >= rows) {
        for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = __builtin_nanf("");
        return;
    }
    if (F16) {
        const __half *w = static_cast<const __half *>(weight) + id * dim;
        for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = __half2float(w[i]);
    } else {
        const float *w = static_cast<const float *>(weight) + id * dim;
        for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = w[i];
    }
}

// The same over ggml's block-quantised rows (dequantize_row_<type> of ggml-quants.c): one thread per element, which
// reads its block's scale (and minimum, and fifth bit) straight from the 18..34-byte block.
__global__ __launch_bounds__(256) void embedding_quant_kernel(const uint8_t *weight, int type, int block_bytes,
                                                              const int32_t *ids, int64_t rows, int dim, float *out) {
    const int t = blockIdx.x;
    const int64_t id = ids[t];
    float *o = out + (int64_t)t * dim;
    if (id < 0 || id >= rows) {
        for (int i = threadIdx.x; i < dim; i += blockDim.x) o[i] = __builtin_nanf("");
        return;
    }
    const uint8_t *row = weight + id * (int64_t)(dim / 32) * block_bytes;
    for (int i = threadIdx.x; i < dim; i += blockDim.x) {
        const uint8_t *b = row + (int64_t)(i / 32) * block_bytes;
        const int e = i % 32;
        const float d = __half2float(__ushort_as_half((uint16_t)(b[0] | (b[1] << 8))));
        float m = 0.f;
        int off = 2, level;
        if (type == GLM_MODEL_Q4_1 || type == GLM_MODEL_Q5_1) {
            m = __half2float(__ushort_as_half((uint16_t)(b[2] | (b[3] << 8))));
            off = 4;
        }
        if (type == GLM_MODEL_Q8_0) {
            level = (int8_t)b[2 + e];
        } else {
            int high = 0;
            if (type == GLM_MODEL_Q5_0 || type == GLM_MODEL_Q5_1) {
                high = ((b[off + e / 8] >> (e % 8)) & 1) << 4;
                off += 4;
            }
            level = (e < 16 ? b[off + e] & 0x0F : b[off + e - 16] >> 4) | high;
            if (type == GLM_MODEL_Q4_0) level -= 8;
            if (type == GLM_MODEL_Q5_0) level -= 16;
        }
        o[i] = __fadd_rn(__fmul_rn((float)level, d), m);
    }
}

}  // namespace

extern "C" int glm_block_embedding(const void *weight, int32_t weight_dtype, int64_t num_embeddings, int32_t dim,
                                   const int32_t *ids, int32_t n_ids, float *out, void *stream) {
    if (!weight || !ids || !out || num_embeddings <= 0 || dim <= 0 || n_ids <= 0) return GLM_ATTN_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    int64_t block_elems = 0, block_bytes = 0;
    if (!type_traits(weight_dtype, &block_elems, &block_bytes)) return GLM_ATTN_EUNSUPPORTED;
    if (block_elems == 32) {
        if (dim % 32 != 0) return GLM_ATTN_EINVAL;
        hipLaunchKernelGGL(embedding_quant_kernel, dim3(n_ids), dim3(256), 0, st, static_cast<const uint8_t *>(weight),
                           weight_dtype, (int)block_bytes, ids, num_embeddings, dim, out);
    } else if (weight_dtype == GLM_MODEL_F16) {
        hipLaunchKernelGGL(embedding_kernel<true>, dim3(n_ids), dim3(256), 0, st, weight, ids, num_embeddings, dim, out);
    } else {
        hipLaunchKernelGGL(embedding_kernel<false>, dim3(n_ids), dim3(256), 0, st, weight, ids, num_embeddings, dim, out);
    }
    return hipGetLastError() == hipSuccess ? GLM_ATTN_OK : GLM_ATTN_EHIP;
}
