#!/usr/bin/env python3
"""Writes tests/golden/reference_converter/: bytes made by the reference's own converter.

The reference holds no model-file fixture and no quantised-block fixture, and nothing else in its tree pins
the byte layout of its "ggml" model files or of the blocks its quantisers write.  This script imports
/root/reference/chatglm_cpp/convert.py (by path, in the build container only: the reference does not travel
with the tests) and lets it write

  quant_blocks.npz   seeded fp32 tensors and the blocks quantize_q4_0 / q4_1 / q5_0 / q5_1 / q8_0 make of them
                     (convert.py:54-131);
  *.bin + *.npz      tiny ChatGLM (v1), ChatGLM2, ChatGLM3 (with a p-tuning prefix) and ChatGLM4 shaped model
                     files written by the converters' own convert() = magic, model type, dump_config,
                     dump_tokenizer, dump_model -> dump_state_dict -> dump_tensor (convert.py:133-396), from stub
                     model / tokenizer objects that carry exactly the attributes the converters read; the .npz
                     beside each file holds the tensors that went in.

The committed files are the fixtures; the tests (tests/test_reference_converter_goldens.py) never import the
reference.  Run: python tests/golden/make_model_file_goldens.py
"""
import importlib.util
import os
import sys
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "reference_converter")
REF = "/root/reference/chatglm_cpp/convert.py"


def load_reference_converter():
    spec = importlib.util.spec_from_file_location("reference_convert", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def rng_tensor(rng, *shape, scale=0.1):
    return torch.from_numpy((rng.standard_normal(shape) * scale).astype(np.float32))


def quant_goldens(ref):
    rng = np.random.default_rng(20241125)
    x = (rng.standard_normal((12, 128)) * np.exp(rng.uniform(-4, 2, size=(12, 1)))).astype(np.float32)
    x[3, :32] = np.linspace(-1.0, 1.0, 32, dtype=np.float32)  # evenly spaced: values on rounding ties
    x[4, 32:64] = np.abs(x[4, 32:64]) + 0.5                   # one-sided block
    x[5, 64:96] = -np.abs(x[5, 64:96]) - 0.25
    out = {"x": x}
    t = torch.from_numpy(x)
    for name in ("q4_0", "q4_1", "q5_0", "q5_1", "q8_0"):
        blocks = getattr(ref, "quantize_" + name)(t.clone())
        out[name] = blocks.numpy().view(np.uint8).copy()
    np.savez(os.path.join(OUT, "quant_blocks.npz"), **out)
    print("quant_blocks.npz:", {k: v.shape for k, v in out.items()})


class StubModel:
    def __init__(self, config, state, prefix_encoder=None):
        self.config = config
        self._state = state
        if prefix_encoder is not None:
            self.transformer = types.SimpleNamespace(prefix_encoder=prefix_encoder)

    def state_dict(self):
        return dict(self._state)


def glm2_state(rng, cfg):
    h, heads, groups, layers, ffn, vocab = (cfg.hidden_size, cfg.num_attention_heads, cfg.multi_query_group_num,
                                            cfg.num_layers, cfg.ffn_hidden_size, cfg.padded_vocab_size)
    d = cfg.kv_channels
    st = {"transformer.embedding.word_embeddings.weight": rng_tensor(rng, vocab, h)}
    for i in range(layers):
        p = f"transformer.encoder.layers.{i}."
        st[p + "input_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
        st[p + "self_attention.query_key_value.weight"] = rng_tensor(rng, h + 2 * groups * d, h)
        st[p + "self_attention.query_key_value.bias"] = rng_tensor(rng, h + 2 * groups * d)
        st[p + "self_attention.dense.weight"] = rng_tensor(rng, h, h)
        st[p + "post_attention_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
        st[p + "mlp.dense_h_to_4h.weight"] = rng_tensor(rng, 2 * ffn, h)
        st[p + "mlp.dense_4h_to_h.weight"] = rng_tensor(rng, h, ffn)
    st["transformer.encoder.final_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
    st["transformer.output_layer.weight"] = rng_tensor(rng, vocab, h)
    return st


def glm2_config(**over):
    cfg = types.SimpleNamespace(
        add_bias_linear=False, add_qkv_bias=True, apply_residual_connection_post_layernorm=False, kv_channels=8,
        num_attention_heads=4, hidden_size=32, multi_query_attention=True, original_rope=True, post_layer_norm=True,
        rmsnorm=True, padded_vocab_size=48, multi_query_group_num=2, num_layers=2, ffn_hidden_size=64,
        layernorm_epsilon=1e-5, seq_length=128, eos_token_id=2, pad_token_id=0)
    for k, v in over.items():
        setattr(cfg, k, v)
    return cfg


def convert_to_bytes(converter, model, tokenizer, ggml_type):
    """The converter writes tensors with numpy's tofile, which wants a real file."""
    path = os.path.join(OUT, "_convert.tmp")
    with open(path, "wb") as f:
        converter.convert(f, model, tokenizer, ggml_type)
    with open(path, "rb") as f:
        blob = f.read()
    os.remove(path)
    return blob


def save(name, blob, state=None, state_name=None):
    """The file as <name>.bin; the tensors that went in as <state_name>.npz (one per family: several files are
    made from the same tensors with different weight types)."""
    with open(os.path.join(OUT, name + ".bin"), "wb") as f:
        f.write(blob)
    if state is not None:
        np.savez(os.path.join(OUT, state_name + ".npz"),
                 **{k: (v.numpy().view(np.uint16) if v.dtype == torch.float16 else v.float().numpy())
                    for k, v in state.items()})
    print(f"{name}.bin: {len(blob)} bytes")


def file_goldens(ref):
    rng = np.random.default_rng(7)
    sp_tok = types.SimpleNamespace(tokenizer=types.SimpleNamespace(
        sp_model=types.SimpleNamespace(serialized_model_proto=lambda: b"\x0a\x05stub sentencepiece model bytes")))

    # ChatGLM2, f16 and q4_0 (convert.py:288-370)
    cfg = glm2_config()
    st = glm2_state(rng, cfg)
    for dtype in ("F16", "Q4_0", "Q4_1", "Q5_0"):
        save("glm2_" + dtype.lower(), convert_to_bytes(ref.ChatGLM2Converter, StubModel(cfg, st), sp_tok,
                                                       ref.GGMLType[dtype]), st, "glm2_state")

    # ChatGLM3 with a p-tuning prefix (convert.py:212-222, 334-343), rope_ratio, missing pad token
    cfg = glm2_config(pre_seq_len=3, rope_ratio=50, pad_token_id=None)
    st = glm2_state(rng, cfg)
    table = rng_tensor(rng, cfg.pre_seq_len, cfg.num_layers * 2 * cfg.multi_query_group_num * cfg.kv_channels, scale=1.0)
    model = StubModel(cfg, st, prefix_encoder=lambda tokens: table[tokens])
    blob = convert_to_bytes(ref.ChatGLM3Converter, model, sp_tok, ref.GGMLType.F16)
    st_out = dict(st)
    st_out["past_key_values"] = ref.get_prefix_cache(model.transformer.prefix_encoder, cfg.pre_seq_len, cfg.num_layers,
                                                     cfg.multi_query_group_num, cfg.kv_channels)
    save("glm3_ptuning_f16", blob, st_out, "glm3_ptuning_state")

    # ChatGLM4, f32 weights and q8_0; the tokenizer is the text of a vocabulary file (convert.py:380-385)
    vocab_path = os.path.join(OUT, "_vocab.tmp")
    with open(vocab_path, "wb") as vf:
        vf.write(b"IQ== 0\nIg== 1\nIw== 2\n")
    tk_tok = types.SimpleNamespace(vocab_file=vocab_path)
    cfg = glm2_config(eos_token_id=39)
    for dtype in ("F32", "Q8_0"):  # the tensors of the ChatGLM3 file, without the prefix
        save("glm4_" + dtype.lower(), convert_to_bytes(ref.ChatGLM4Converter, StubModel(cfg, st), tk_tok,
                                                       ref.GGMLType[dtype]))
    os.remove(vocab_path)

    # ChatGLM v1 (convert.py:225-286): tied head, biases everywhere, q5_1 weights
    cfg = types.SimpleNamespace(position_encoding_2d=True, hidden_size=32, inner_hidden_size=128, vocab_size=40,
                                num_attention_heads=4, num_layers=2, layernorm_epsilon=1e-5, pre_seq_len=None,
                                max_sequence_length=64, eos_token_id=5, pad_token_id=3, quantization_bit=0)
    h, inter = cfg.hidden_size, cfg.inner_hidden_size
    st = {"transformer.word_embeddings.weight": rng_tensor(rng, cfg.vocab_size, h)}
    st["lm_head.weight"] = st["transformer.word_embeddings.weight"]
    for i in range(cfg.num_layers):
        p = f"transformer.layers.{i}."
        st[p + "input_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
        st[p + "input_layernorm.bias"] = rng_tensor(rng, h)
        st[p + "attention.query_key_value.weight"] = rng_tensor(rng, 3 * h, h)
        st[p + "attention.query_key_value.bias"] = rng_tensor(rng, 3 * h)
        st[p + "attention.dense.weight"] = rng_tensor(rng, h, h)
        st[p + "attention.dense.bias"] = rng_tensor(rng, h)
        st[p + "post_attention_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
        st[p + "post_attention_layernorm.bias"] = rng_tensor(rng, h)
        st[p + "mlp.dense_h_to_4h.weight"] = rng_tensor(rng, inter, h)
        st[p + "mlp.dense_h_to_4h.bias"] = rng_tensor(rng, inter)
        st[p + "mlp.dense_4h_to_h.weight"] = rng_tensor(rng, h, inter)
        st[p + "mlp.dense_4h_to_h.bias"] = rng_tensor(rng, h)
    st["transformer.final_layernorm.weight"] = rng_tensor(rng, h, scale=1.0)
    st["transformer.final_layernorm.bias"] = rng_tensor(rng, h)
    v1_tok = types.SimpleNamespace(sp_tokenizer=types.SimpleNamespace(text_tokenizer=types.SimpleNamespace(
        sp=types.SimpleNamespace(serialized_model_proto=lambda: b"\x0a\x03v1 stub model"))))
    for dtype in ("F16", "Q5_1"):
        save("glm1_" + dtype.lower(), convert_to_bytes(ref.ChatGLMConverter, StubModel(cfg, st), v1_tok,
                                                       ref.GGMLType[dtype]),
             {k: v for k, v in st.items() if k != "lm_head.weight"}, "glm1_state")


def main():
    if not os.path.exists(REF):
        sys.exit(f"{REF} is not here: the goldens can only be made where the reference is")
    os.makedirs(OUT, exist_ok=True)
    ref = load_reference_converter()
    quant_goldens(ref)
    file_goldens(ref)


if __name__ == "__main__":
    main()
