// Times whole forwards of a GLM-4-9B-shaped model through the C++ mirror of the reference's model classes
// (chatglm_model.h), random fp16 weights and caches made on the device: what BaseModelForCausalLM::
// generate_next_token (chatglm.cpp:757-831) does per token minus the sampling, i.e. ids in, logits on the host.
// Prints one JSON object.
//
// usage: bench_model [--dtype f16|f32|q4_0|q4_1|q5_0|q5_1|q8_0] [--layers N] [--n-past N] [--tokens N] [--warmup N]
//                    [--prompt N] [--followup N]
// --followup N: also time one forward of N new tokens on top of n_past cached ones (a follow-up message in a
// long conversation)
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "chatglm_model.h"

using namespace chatglm;

namespace {

// counter-based values in [-scale, scale) + offset, fp16 or fp32
template <typename T>
__global__ void fill_kernel(T *p, size_t n, uint32_t seed, float scale, float offset) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t x = (uint32_t)i * 2654435761u ^ (uint32_t)(i >> 32) * 40503u ^ seed;
        x ^= x >> 16;
        x *= 0x7feb352du;
        x ^= x >> 15;
        x *= 0x846ca68bu;
        x ^= x >> 16;
        p[i] = (T)(((float)(x >> 8) * (1.f / 8388608.f) - 1.f) * scale + offset);
    }
}

// ggml blocks with a fixed scale (and minimum) and random levels
__global__ void fill_blocks_kernel(uint8_t *p, size_t n_blocks, int block_bytes, int head_bytes, bool has_min,
                                   uint32_t seed, float scale) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_blocks; i += (size_t)gridDim.x * blockDim.x) {
        uint8_t *b = p + i * block_bytes;
        const uint16_t d = __half_as_ushort(__float2half(scale)), m = __half_as_ushort(__float2half(-8.f * scale));
        b[0] = (uint8_t)d;
        b[1] = (uint8_t)(d >> 8);
        if (has_min) {
            b[2] = (uint8_t)m;
            b[3] = (uint8_t)(m >> 8);
        }
        uint32_t x = (uint32_t)i * 2654435761u ^ seed;
        for (int k = has_min ? 4 : 2; k < block_bytes; k++) {
            x ^= x << 13;
            x ^= x >> 17;
            x ^= x << 5;
            b[k] = (uint8_t)(x >> 11);
        }
        (void)head_bytes;
    }
}

uint32_t g_seed = 1;

void fill(Tensor *t, float scale, float offset = 0.f) {
    if (!t) return;
    const size_t n = (size_t)t->nelements();
    const int blocks = (int)std::min<size_t>((n + 255) / 256, 65536);
    if (dtype_is_quantized(t->type)) {
        const bool has_min = t->type == DType::Q4_1 || t->type == DType::Q5_1;
        // levels of Q8_0 span -128..127, of the 4- and 5-bit types 16 or 32 steps: scales that give weights of ~scale
        const float step = t->type == DType::Q8_0 ? scale / 127.f : (t->type == DType::Q4_0 || t->type == DType::Q4_1) ? scale / 8.f : scale / 16.f;
        hipLaunchKernelGGL(fill_blocks_kernel, dim3((unsigned)std::min<size_t>((n / 32 + 255) / 256, 65536)), dim3(256), 0,
                           0, static_cast<uint8_t *>(t->data), n / 32, (int)dtype_size(t->type), 0, has_min, g_seed++, step);
    } else if (t->type == DType::F16) {
        hipLaunchKernelGGL(fill_kernel<__half>, dim3(blocks), dim3(256), 0, 0, static_cast<__half *>(t->data), n, g_seed++, scale, offset);
    } else {
        hipLaunchKernelGGL(fill_kernel<float>, dim3(blocks), dim3(256), 0, 0, static_cast<float *>(t->data), n, g_seed++, scale, offset);
    }
}

double now_ms() {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

}  // namespace

int main(int argc, char **argv) {
    int layers = 40, n_past = 32767, tokens = 20, warmup = 3, prompt = 2048, followup = 0;
    std::string dtype_name = "f16";
    int ggml_dtype = GLM_MODEL_F16;
    for (int i = 1; i + 1 < argc; i += 2) {
        const std::string k = argv[i];
        const int v = atoi(argv[i + 1]);
        if (k == "--dtype") {
            dtype_name = argv[i + 1];
            const char *names[] = {"f32", "f16", "q4_0", "q4_1", "", "", "q5_0", "q5_1", "q8_0"};
            ggml_dtype = -1;
            for (int t = 0; t < 9; t++) {
                if (dtype_name == names[t]) ggml_dtype = t;
            }
            if (ggml_dtype < 0) {
                fprintf(stderr, "unknown dtype %s\n", argv[i + 1]);
                return 2;
            }
        } else if (k == "--layers") layers = v;
        else if (k == "--n-past") n_past = v;
        else if (k == "--tokens") tokens = v;
        else if (k == "--warmup") warmup = v;
        else if (k == "--prompt") prompt = v;
        else if (k == "--followup") followup = v;
        else {
            fprintf(stderr, "unknown option %s\n", argv[i]);
            return 2;
        }
    }
    try {
        // GLM-4-9B (config.json of THUDM/glm-4-9b-chat as convert.py:292-323 records it)
        glm_model_config rec;
        memset(&rec, 0, sizeof(rec));
        rec.struct_size = (int32_t)sizeof(rec);
        rec.model_type = GLM_MODEL_CHATGLM4;
        rec.version = 2;
        rec.dtype = ggml_dtype;
        rec.vocab_size = 151552;
        rec.hidden_size = 4096;
        rec.num_attention_heads = 32;
        rec.num_key_value_heads = 2;
        rec.num_hidden_layers = layers;
        rec.intermediate_size = 13696;
        rec.norm_eps = 1.5625e-07f;
        rec.hidden_act = GLM_BLOCK_ACT_SILU;
        rec.use_qkv_bias = 1;
        rec.rope_type = GLM_ATTN_ROPE_CHATGLM2;
        rec.rope_theta = 5000000.f;
        rec.attn_mask_type = GLM_ATTN_MASK_CAUSAL;
        rec.max_length = ((std::max(std::max(n_past + warmup + tokens + 1, prompt), n_past + followup) + 7) / 8) * 8;
        ModelConfig config(rec);
        ChatGLM4ForCausalLM model(config);
        fill(model.transformer.word_embeddings.weight, 0.05f);
        for (auto &l : model.transformer.layers) {
            fill(l.input_layernorm.weight, 0.1f, 1.f);
            fill(l.attention.query_key_value.weight, 0.02f);
            fill(l.attention.query_key_value.bias, 0.1f);
            fill(l.attention.dense.weight, 0.02f);
            fill(l.post_attention_layernorm.weight, 0.1f, 1.f);
            fill(l.mlp.gate_proj.weight, 0.02f);
            fill(l.mlp.up_proj.weight, 0.02f);
            fill(l.mlp.down_proj.weight, 0.01f);
            fill(l.attention.k_cache, 1.f);
            fill(l.attention.v_cache, 1.f);
        }
        fill(model.transformer.final_layernorm.weight, 0.1f, 1.f);
        fill(model.lm_head.weight, 0.02f);
        if (hipDeviceSynchronize() != hipSuccess) {
            fprintf(stderr, "fill failed\n");
            return 3;
        }
        for (auto &l : model.transformer.layers) {  // what load_state_dict does after the uploads
            l.attention.query_key_value.commit(model.context());
            l.attention.dense.commit(model.context());
            l.mlp.gate_proj.commit(model.context());
            l.mlp.up_proj.commit(model.context());
            l.mlp.down_proj.commit(model.context());
        }
        model.lm_head.commit(model.context());

        std::vector<int> ids((size_t)n_past + std::max(warmup + tokens + 1, followup));
        for (size_t i = 0; i < ids.size(); i++) ids[i] = (int)((i * 7919u + 13u) % (size_t)config.vocab_size);
        double decode_ms = 0.0;
        bool finite = true;
        for (int t = 0; t < warmup + tokens; t++) {
            std::vector<int> seen(ids.begin(), ids.begin() + n_past + t + 1);
            const double t0 = now_ms();
            std::vector<float> logits = model.forward_graph_compute(seen, n_past + t, n_past, true);
            const double t1 = now_ms();
            if (t >= warmup) decode_ms += t1 - t0;
            for (size_t i = 0; i < logits.size(); i += 997) finite = finite && std::isfinite(logits[i]);
        }
        decode_ms /= tokens;

        double prefill_ms = 0.0;
        if (prompt > 0) {
            std::vector<int> seen(ids.begin(), ids.begin() + prompt);
            model.forward_graph_compute(seen, 0, prompt, true);  // warm-up: arenas grow
            const double t0 = now_ms();
            std::vector<float> logits = model.forward_graph_compute(seen, 0, prompt, true);
            prefill_ms = now_ms() - t0;
            for (size_t i = 0; i < logits.size(); i += 997) finite = finite && std::isfinite(logits[i]);
        }
        double followup_ms = 0.0;
        if (followup > 0) {
            std::vector<int> seen(ids.begin(), ids.begin() + n_past + followup);
            model.forward_graph_compute(seen, n_past, n_past + followup, false);  // warm-up
            const double t0 = now_ms();
            std::vector<float> logits = model.forward_graph_compute(seen, n_past, n_past + followup, false);
            followup_ms = now_ms() - t0;
            for (size_t i = 0; i < logits.size(); i += 997) finite = finite && std::isfinite(logits[i]);
        }
        const double bytes_per_weight = dtype_is_quantized(config.dtype)
                                            ? (double)dtype_size(config.dtype) / 32.0
                                            : (double)dtype_size(config.dtype);
        const double weight_bytes =
            bytes_per_weight * ((double)layers * ((4608.0 + 4096.0 + 3 * 13696.0) * 4096.0) + 151552.0 * 4096.0);  // + LM head
        const double cache_bytes = (double)layers * 2.0 * 2 * 128 * (n_past + 1) * 2.0;
        printf("{\"workload\": \"GLM-4-9B-shaped model, %d layers, %s weights, ids in -> logits on the host, eager "
               "launches through the C++ mirror of the reference's model classes\", \"n_past\": %d, "
               "\"decode_ms_per_token\": %.4f, \"decode_tokens_per_s\": %.2f, \"decode_hbm_gbs\": %.1f, "
               "\"decode_bytes_per_token\": %.0f, \"prefill_tokens\": %d, \"prefill_ms\": %.3f, "
               "\"prefill_tokens_per_s\": %.1f, \"followup_tokens\": %d, \"followup_ms\": %.3f, \"finite\": %s}\n",
               layers, dtype_name.c_str(), n_past, decode_ms, 1000.0 / decode_ms, (weight_bytes + cache_bytes) / decode_ms / 1e6,
               weight_bytes + cache_bytes, prompt, prefill_ms, prompt > 0 ? prompt / prefill_ms * 1000.0 : 0.0, followup, followup_ms,
               finite ? "true" : "false");
    } catch (const std::exception &e) {
        fprintf(stderr, "exception: %s\n", e.what());
        return 3;
    }
    return 0;
}
