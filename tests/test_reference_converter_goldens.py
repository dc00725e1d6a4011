"""Bytes that the reference's own converter wrote (tests/golden/reference_converter/, made by
tests/golden/make_model_file_goldens.py from chatglm_cpp/convert.py in the build container) against

  * tests/quant_numpy.py: the same blocks, byte for byte, from the same seeded tensors (convert.py:54-131);
  * tests/model_file_writer.py: the same files, byte for byte, from the same tensors (convert.py:133-396);
  * the model-file reader of the library (include/glm_model_file.h): config records, tensor records, payloads;
  * the oracle's dequantiser: the values of the reference-written blocks.

These fixtures are what pins the "ggml" file layout and the quantised block layouts: the tests here never
import the reference.  No GPU."""
import os
import struct
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.join(os.path.dirname(HERE), "oracle"))

from __graft_entry__ import load_package  # noqa: E402

pkg = load_package()
import glm_oracle as orc  # noqa: E402
import model_file_writer as mw  # noqa: E402
import quant_numpy as qn  # noqa: E402

GOLD = os.path.join(HERE, "golden", "reference_converter")
QTYPES = {"q4_0": qn.Q4_0, "q4_1": qn.Q4_1, "q5_0": qn.Q5_0, "q5_1": qn.Q5_1, "q8_0": qn.Q8_0}
GGML = {"f32": mw.F32, "f16": mw.F16, **QTYPES}


@pytest.mark.parametrize("name", sorted(QTYPES))
def test_quantised_blocks_of_the_reference_converter(name):
    g = np.load(os.path.join(GOLD, "quant_blocks.npz"))
    x, want = g["x"], g[name]
    mine = qn.quantize(QTYPES[name], x)
    assert mine.reshape(want.shape).tobytes() == want.tobytes(), f"{name}: blocks differ from the converter's"
    # what the blocks stand for: the oracle's dequantiser reads the reference's bytes
    vals = orc.dequantize(QTYPES[name], np.ascontiguousarray(want.reshape(x.shape[0], -1)))
    assert np.allclose(vals, qn.dequantize(QTYPES[name], want.reshape(x.shape[0], -1)), rtol=0, atol=1e-6)
    step = {"q4_0": 1 / 8, "q4_1": 1 / 15, "q5_0": 1 / 16, "q5_1": 1 / 31, "q8_0": 1 / 127}[name]
    blocks = x.reshape(-1, 32)
    span = np.abs(blocks).max(axis=1, keepdims=True) * (2 if name in ("q4_1", "q5_1") else 1)
    # half a step, a whole one where the asymmetric 4- and 5-bit grids clamp the far end of a block
    assert np.all(np.abs(vals.reshape(-1, 32) - blocks) <= span * step * 1.01 + 1e-3 * span)


# file, family state, model type, converter family, weight type, config as the converter's dump_config packs it
GLM2_CFG = dict(vocab_size=48, hidden_size=32, num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=2,
                intermediate_size=64, norm_eps=1e-5, num_virtual_tokens=0, rope_theta=10000.0, max_length=128,
                eos_token_id=2, pad_token_id=0)
GLM1_CFG = dict(vocab_size=40, hidden_size=32, num_attention_heads=4, num_key_value_heads=4, num_hidden_layers=2,
                intermediate_size=128, norm_eps=1e-5, num_virtual_tokens=0, rope_theta=10000.0, max_length=64,
                eos_token_id=5, pad_token_id=3)
FILES = [
    ("glm2_f16", "glm2_state", 2, "f16", GLM2_CFG, b"\x0a\x05stub sentencepiece model bytes"),
    ("glm2_q4_0", "glm2_state", 2, "q4_0", GLM2_CFG, b"\x0a\x05stub sentencepiece model bytes"),
    ("glm2_q4_1", "glm2_state", 2, "q4_1", GLM2_CFG, b"\x0a\x05stub sentencepiece model bytes"),
    ("glm2_q5_0", "glm2_state", 2, "q5_0", GLM2_CFG, b"\x0a\x05stub sentencepiece model bytes"),
    ("glm3_ptuning_f16", "glm3_ptuning_state", 3, "f16",
     dict(GLM2_CFG, num_virtual_tokens=3, rope_theta=500000.0, pad_token_id=-1), b"\x0a\x05stub sentencepiece model bytes"),
    ("glm4_f32", "glm3_ptuning_state", 4, "f32", dict(GLM2_CFG, eos_token_id=39), b"IQ== 0\nIg== 1\nIw== 2\n"),
    ("glm4_q8_0", "glm3_ptuning_state", 4, "q8_0", dict(GLM2_CFG, eos_token_id=39), b"IQ== 0\nIg== 1\nIw== 2\n"),
    ("glm1_f16", "glm1_state", 1, "f16", GLM1_CFG, b"\x0a\x03v1 stub model"),
    ("glm1_q5_1", "glm1_state", 1, "q5_1", GLM1_CFG, b"\x0a\x03v1 stub model"),
]


def expected_tensors(state, model_type, wtype, cfg):
    """(name, payload array / QuantTensor, ggml type) in file order, as dump_state_dict decides them
    (convert.py:166-205): the prefix in F16, 2-d weights in the file's type, 1-d tensors in F32."""
    names = mw.glm1_weight_names(cfg["num_hidden_layers"]) if model_type == 1 else \
        mw.glm2_weight_names(cfg["num_hidden_layers"], cfg["num_virtual_tokens"] > 0)
    out = []
    for n in names:
        a = state[n]
        if n == "past_key_values":
            out.append((n, a.view(np.uint16), mw.F16))  # stored as the fp16 bit patterns
        elif a.ndim == 2:
            t = GGML[wtype]
            if t == mw.F32:
                out.append((n, a.astype(np.float32), t))
            elif t == mw.F16:
                out.append((n, a.astype(np.float16), t))
            else:
                out.append((n, mw.QuantTensor(qn.quantize(t, a), a.shape, t), t))
        else:
            out.append((n, a.astype(np.float32), mw.F32))
    return out


@pytest.mark.parametrize("fname,sname,model_type,wtype,cfg,tok", FILES, ids=[f[0] for f in FILES])
def test_files_of_the_reference_converter(tmp_path, fname, sname, model_type, wtype, cfg, tok):
    want = open(os.path.join(GOLD, fname + ".bin"), "rb").read()
    state = np.load(os.path.join(GOLD, sname + ".npz"))
    tensors = expected_tensors(state, model_type, wtype, cfg)

    # 1. the test writer restates the converter: the same bytes
    mine = mw.write_model_file(str(tmp_path / "mine.bin"), model_type, mw.pack_config_v2(GGML[wtype], **cfg), tok, tensors)
    assert len(mine) == len(want)
    assert mine == want, f"{fname}: first difference at byte {next(i for i in range(len(want)) if mine[i] != want[i])}"

    # 2. the library's reader on the converter's bytes
    with pkg.ModelFile(os.path.join(GOLD, fname + ".bin")) as f:
        c = f.config().as_dict()
        for k, v in cfg.items():
            assert c[k] == pytest.approx(v), k
        assert (c["model_type"], c["version"], c["dtype"]) == (model_type, 2, GGML[wtype])
        assert want[c["tokenizer_offset"]:c["tokenizer_offset"] + c["tokenizer_size"]] == tok
        if model_type == 1:  # ModelConfig for ChatGLM-6B (chatglm.h:121-129)
            assert (c["hidden_act"], c["use_qkv_bias"], c["use_dense_bias"], c["interleaved_qkv"],
                    c["tie_word_embeddings"], c["rope_type"], c["attn_mask_type"]) == (0, 1, 1, 1, 1, 4, 1)
        else:
            assert (c["hidden_act"], c["use_qkv_bias"], c["use_dense_bias"], c["interleaved_qkv"],
                    c["tie_word_embeddings"], c["rope_type"], c["attn_mask_type"]) == (1, 1, 0, 0, 0, 8, 0)
        assert len(f) == len(tensors)
        for i, (name, array, ggml_type) in enumerate(tensors):
            t = f.tensor(i)
            assert t.name.decode() == name and t.dtype == ggml_type and t.ndim == array.ndim
            assert list(t.ne)[:array.ndim] == list(array.shape)[::-1]
            payload = array.blocks.tobytes() if isinstance(array, mw.QuantTensor) else array.tobytes()
            assert t.offset % 16 == 0 and t.nbytes == len(payload)
            assert f.host_bytes(t) == payload, name
        last = f.tensor(len(f) - 1)
        assert last.offset + last.nbytes == len(want)


def test_config_record_layout_of_the_reference_converter():
    """The 14 fields behind magic and model type, as struct.pack("iiiiiiiififiii", ...) laid them out."""
    want = open(os.path.join(GOLD, "glm3_ptuning_f16.bin"), "rb").read()
    assert want[:4] == b"ggml" and struct.unpack_from("i", want, 4) == (3,)
    fields = struct.unpack_from("iiiiiiiififiii", want, 8)
    assert fields[:8] == (2, 1, 48, 32, 4, 2, 2, 64)
    assert fields[8] == pytest.approx(1e-5) and fields[9] == 3 and fields[10] == pytest.approx(500000.0)
    assert fields[11:] == (128, 2, -1)
