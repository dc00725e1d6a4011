"""The model-file reader (include/glm_model_file.h) against files written in the converter's layout
(tests/model_file_writer.py follows chatglm_cpp/convert.py): header, the three config records and what ModelConfig
derives from them (chatglm.h:106-160), tensor records with their 16-byte alignment (chatglm.cpp:357-391), and the
checks on broken files.  No GPU: everything up to the upload is host code.

The reference ships no model file to read; the byte layout is pinned by tests/test_reference_converter_goldens.py,
where the writer used here reproduces files of the reference's own converter byte for byte and the reader parses
them."""
import os
import struct
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
sys.path.insert(0, os.path.dirname(HERE))

from __graft_entry__ import load_package  # noqa: E402

pkg = load_package()
import model_file_writer as mw  # noqa: E402

GLM4 = dict(vocab_size=96, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, num_hidden_layers=2,
            intermediate_size=80, norm_eps=1.5625e-07, num_virtual_tokens=0, rope_theta=5000000.0, max_length=48,
            eos_token_id=7, pad_token_id=3)


def glm4_file(tmp_path, weight_type=mw.F16, tokenizer=b"tiktoken vocabulary bytes", cfg=GLM4, model_type=4):
    tensors = mw.random_state_dict(cfg, mw.glm2_weight_names(cfg["num_hidden_layers"], cfg["num_virtual_tokens"] > 0),
                                   mw.glm2_shapes, 5, weight_type)
    path = str(tmp_path / "model.bin")
    blob = mw.write_model_file(path, model_type, mw.pack_config_v2(weight_type, **cfg), tokenizer, tensors)
    return path, blob, tensors


def test_version_2_record_and_tensor_records(tmp_path):
    path, blob, tensors = glm4_file(tmp_path)
    with pkg.ModelFile(path) as f:
        c = f.config().as_dict()
        for k, v in GLM4.items():
            assert c[k] == pytest.approx(v), k
        assert (c["model_type"], c["version"], c["dtype"]) == (4, 2, mw.F16)
        # ModelConfig's constructor for everything but ChatGLM-6B (chatglm.h:130-137), record V2 (:155-160)
        assert (c["hidden_act"], c["use_qkv_bias"], c["use_dense_bias"], c["interleaved_qkv"],
                c["tie_word_embeddings"], c["rope_type"], c["attn_mask_type"]) == (1, 1, 0, 0, 0, 8, 0)
        assert (c["bos_token_id"], c["sep_token_id"]) == (-1, -1)
        assert blob[c["tokenizer_offset"]:c["tokenizer_offset"] + c["tokenizer_size"]] == b"tiktoken vocabulary bytes"
        assert len(f) == len(tensors)
        for i, (name, array, ggml_type) in enumerate(tensors):
            t = f.tensor(i)
            assert t.name.decode() == name and t.dtype == ggml_type and t.ndim == array.ndim
            assert list(t.ne)[:array.ndim] == list(array.shape)[::-1]  # ggml order: innermost first
            assert list(t.ne)[array.ndim:] == [1] * (4 - array.ndim)
            assert t.offset % 16 == 0 and t.nbytes == array.nbytes
            assert f.host_bytes(t) == array.tobytes()  # bit-exact payload at the aligned offset
            found = f.find(name)
            assert found.offset == t.offset and found.reserved == i
        assert f.find("no.such.tensor") is None
        # the records tile the file: the last one ends at the end of the file
        last = f.tensor(len(f) - 1)
        assert last.offset + last.nbytes == len(blob)
        assert pkg.lib().glm_model_file_tensor(f.handle, len(f), None) == pkg.EINVAL
        t = pkg.ModelTensor()
        t.struct_size = 8
        assert pkg.lib().glm_model_file_tensor(f.handle, 0, t) == pkg.EINVAL
    assert pkg.lib().glm_model_file_tensor_count(None) == 0


def test_version_1_records(tmp_path):
    # ChatGLM-6B: ConfigRecordV1, kv heads = heads, eps 1e-5, theta 10000 (chatglm.h:140-146, chatglm.cpp:1779)
    cfg1 = dict(vocab_size=80, hidden_size=32, num_attention_heads=4, num_hidden_layers=1, intermediate_size=128,
                max_length=24, bos_token_id=5, eos_token_id=6, pad_token_id=3, sep_token_id=-1)
    full = dict(cfg1, num_key_value_heads=4)
    tensors = mw.random_state_dict(full, mw.glm1_weight_names(1), mw.glm1_shapes, 2, mw.F32)
    path = str(tmp_path / "glm1.bin")
    mw.write_model_file(path, 1, mw.pack_config_v1(mw.F32, **cfg1), b"sp", tensors)
    with pkg.ModelFile(path) as f:
        c = f.config().as_dict()
        for k, v in cfg1.items():
            assert c[k] == v, k
        assert c["num_key_value_heads"] == 4 and c["norm_eps"] == pytest.approx(1e-5) and c["rope_theta"] == 10000.0
        assert c["num_virtual_tokens"] == 0
        # ChatGLM-6B flags (chatglm.h:121-129)
        assert (c["hidden_act"], c["use_qkv_bias"], c["use_dense_bias"], c["interleaved_qkv"],
                c["tie_word_embeddings"], c["rope_type"], c["attn_mask_type"]) == (0, 1, 1, 1, 1, 4, 1)
        assert len(f) == len(tensors)
    # ChatGLM2 with the GQA record (chatglm.h:148-153)
    cfg2 = dict(vocab_size=80, hidden_size=32, num_attention_heads=4, num_hidden_layers=1, intermediate_size=48,
                max_length=24, bos_token_id=-1, eos_token_id=2, pad_token_id=0, sep_token_id=-1)
    full = dict(cfg2, num_key_value_heads=2, num_virtual_tokens=0)
    tensors = mw.random_state_dict(full, mw.glm2_weight_names(1), mw.glm2_shapes, 3, mw.F16)
    path = str(tmp_path / "glm2.bin")
    mw.write_model_file(path, 2, mw.pack_config_v1(mw.F16, num_key_value_heads=2, **cfg2), b"", tensors)
    with pkg.ModelFile(path) as f:
        c = f.config().as_dict()
        assert c["num_key_value_heads"] == 2 and c["version"] == 1 and c["rope_type"] == 8 and c["tokenizer_size"] == 0
        assert len(f) == len(tensors)


def test_quantised_records_have_ggml_sizes(tmp_path):
    # block sizes of ggml's q4_0, q4_1, q5_0, q5_1, q8_0: 18, 20, 22, 24, 34 bytes per 32 elements
    tensors = [("w%d" % t, np.zeros((6, 64), np.float32), t) for t in (2, 3, 6, 7, 8)]
    path = str(tmp_path / "q.bin")
    mw.write_model_file(path, 4, mw.pack_config_v2(2, **GLM4), b"", tensors)
    with pkg.ModelFile(path) as f:
        assert [f.tensor(i).nbytes for i in range(5)] == [6 * 2 * n for n in (18, 20, 22, 24, 34)]


def test_prefix_cache_record(tmp_path):
    cfg = dict(GLM4, num_virtual_tokens=5)
    path, _, tensors = glm4_file(tmp_path, cfg=cfg, model_type=3)
    with pkg.ModelFile(path) as f:
        t = f.find("past_key_values")  # [l * 2, #h, v, d] fp16 (convert.py:212-222)
        assert t.dtype == mw.F16 and list(t.ne) == [16, 5, 2, 4] and t.reserved == 0
        assert f.config().num_virtual_tokens == 5


def test_broken_files_are_errors_with_the_reference_messages(tmp_path):
    path, blob, _ = glm4_file(tmp_path)

    def open_error(data):
        p = str(tmp_path / "broken.bin")
        open(p, "wb").write(data)
        with pytest.raises(pkg.GlmAttnError) as e:
            pkg.ModelFile(p)
        return str(e.value)

    assert "bad magic" in open_error(b"gguf" + blob[4:])                      # chatglm.cpp:1769
    assert "invalid model type" in open_error(blob[:4] + struct.pack("i", 9) + blob[8:])  # :1845
    assert "only support version 2" in open_error(blob[:8] + struct.pack("i", 1) + blob[12:])  # :1827
    v3 = blob[:4] + struct.pack("i", 2) + struct.pack("i", 3) + blob[12:]
    assert "only support version 1 or 2 for now but got 3" in open_error(v3)  # :1806
    assert "truncated" in open_error(blob[:40])
    assert "truncated" in open_error(blob[:-5])          # data of the last tensor cut short
    assert "truncated" in open_error(blob[:len(blob) - GLM4["vocab_size"] * 64 * 2 - 3])
    with pytest.raises(pkg.GlmAttnError) as e:
        pkg.ModelFile(str(tmp_path / "missing.bin"))
    assert "cannot open file" in str(e.value)            # chatglm.cpp:300
    bad_dims = bytearray(blob)
    with pkg.ModelFile(path) as f:
        first = f.tensor(0)
        name_len = len(first.name)
        hdr = f.config().tokenizer_offset + f.config().tokenizer_size
    struct.pack_into("i", bad_dims, hdr + 4 + name_len, 5)  # ndim = 5 (chatglm.cpp:371)
    assert "dimensions" in open_error(bytes(bad_dims))
    # a shape whose byte count does not fit 64 bits must not wrap into a size that fits the file:
    # 4 dims of 2^31 - 1 fp32 elements = 2^126 bytes (2^62 elements would wrap to a small count)
    rec = struct.pack("i", 1) + b"w" + struct.pack("i" * 6, 4, 0x7fffffff, 0x7fffffff, 0x7fffffff, 0x7fffffff, 0)
    assert "bad shape" in open_error(blob[:hdr] + rec + b"\0" * 64)
    # 2^31-1 * 2^31-1 * 2 * 2 elements of fp16: 2^65 bytes, which is 2^1 modulo 2^64
    rec = struct.pack("i", 1) + b"w" + struct.pack("i" * 6, 4, 0x40000000, 0x40000000, 4, 2, 1)
    assert "bad shape" in open_error(blob[:hdr] + rec + b"\0" * 64)


def test_mutated_files_never_crash_the_reader(tmp_path):
    """A model file is outside input: whatever bytes it holds, opening it either works or fails with a message.
    Truncations at every kind of boundary and random byte changes in the header and the records' metadata."""
    path, blob, _ = glm4_file(tmp_path, weight_type=mw.F32)
    with pkg.ModelFile(path) as f:
        meta_end = f.tensor(0).offset  # end of the first record's metadata
        offsets = [f.tensor(i).offset for i in range(len(f))]
    rng = np.random.default_rng(7)
    cases = [blob[:n] for n in list(range(0, 120)) + [meta_end - 1, meta_end, meta_end + 1] + [o - 3 for o in offsets[1:]]]
    for _ in range(300):
        b = bytearray(blob)
        for _ in range(int(rng.integers(1, 4))):
            # header, config record, tokenizer length, or the metadata of a record
            region = int(rng.integers(0, 3))
            if region == 0:
                pos = int(rng.integers(0, meta_end))
            else:
                start = offsets[int(rng.integers(1, len(offsets)))]
                pos = max(0, start - int(rng.integers(1, 90)))
            b[pos] = int(rng.integers(0, 256))
        cases.append(bytes(b))
    opened = failed = 0
    p = str(tmp_path / "mutated.bin")
    for data in cases:
        open(p, "wb").write(data)
        try:
            with pkg.ModelFile(p) as f:
                n = len(f)
                for i in range(n):
                    t = f.tensor(i)
                    assert 0 <= t.offset and t.offset + t.nbytes <= len(data)  # every record lies inside the file
                f.config()
            opened += 1
        except pkg.GlmAttnError as e:
            assert str(e)
            failed += 1
    assert failed > 100 and opened + failed == len(cases)
