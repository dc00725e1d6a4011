"""Model files end to end: a file in the converter's layout (tests/model_file_writer.py) is loaded by the C++
mirror of the reference's model classes (chatglm.cpp_amd/host/chatglm_model.h: the model half of
Pipeline::Pipeline, chatglm.cpp:1754-1848, and load_state_dict, :1090-1121, 1250-1313), the reference's generation
protocol is run on the device (prompt, then one token at a time), and every forward's logits are compared with the
same model composed from the CPU oracle's modules (tests/model_host.py).

The reference holds no model-file fixture (its end-to-end tests need downloaded checkpoints, chatglm_test.cpp:
1060-1495), so the file format is pinned by the converter's source alone and the values by the oracle, whose
modules are pinned by the reference's block and module fixtures."""
import os
import struct
import subprocess
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
sys.path.insert(0, HERE)
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))
RUNNER = os.path.join(HERE, "cpp", "test_model_file")

import model_file_writer as mw  # noqa: E402


def read_logits(path):
    buf = open(path, "rb").read()
    out, off = [], 0
    while off < len(buf):
        rows, vocab = struct.unpack_from("ii", buf, off)
        off += 8
        out.append(np.frombuffer(buf, np.float32, rows * vocab, off).reshape(rows, vocab).copy())
        off += rows * vocab * 4
    return out


def run_case(tmp_path, model_type, cfg, config_bytes, tensors, ids, n_prompt, all_rows, max_length=-1, tol=4e-3,
             path=None):
    """path: an existing model file that holds `tensors` (else one is written in the converter's layout)."""
    from model_host import OracleModel

    if path is None:
        path = str(tmp_path / "model.bin")
        mw.write_model_file(path, model_type, config_bytes, b"tokenizer bytes", tensors)
    out_path = str(tmp_path / "logits.bin")
    print("running", os.path.basename(RUNNER), "model_type", model_type, flush=True)
    r = subprocess.run([RUNNER, path, out_path, str(max_length), str(n_prompt), str(int(all_rows))] + [str(i) for i in ids],
                       capture_output=True, text=True, timeout=240)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    got = read_logits(out_path)
    full = dict(cfg, model_type=model_type)
    if max_length > 0:
        full["max_length"] = max_length
    oracle = OracleModel(full, {name: a for name, a, _ in tensors})
    n_past, worst = 0, 0.0
    assert len(got) == len(ids) - n_prompt + 1
    for step, end in enumerate(range(n_prompt, len(ids) + 1)):
        decoding = not (all_rows and n_past == 0)
        ref = np.atleast_2d(oracle.forward(ids[:end], n_past, n_prompt, decoding))
        assert got[step].shape == ref.shape, (got[step].shape, ref.shape)
        err = np.abs(got[step] - ref)
        bound = tol + tol * np.abs(ref)
        worst = max(worst, float((err / bound).max()))
        assert (err <= bound).all(), f"forward {step}: max err {err.max():.3e}, largest logit {np.abs(ref).max():.3f}"
        assert np.abs(ref).max() > 0.05  # the comparison is not one of zeros
        n_past = end
    print(f"worst error / tolerance: {worst:.3f}")


GLM4 = dict(vocab_size=160, hidden_size=256, num_attention_heads=2, num_key_value_heads=1, num_hidden_layers=3,
            intermediate_size=320, norm_eps=1.5625e-07, num_virtual_tokens=0, rope_theta=5000000.0, max_length=64,
            eos_token_id=7, pad_token_id=3)


@pytest.mark.gpu
@pytest.mark.parametrize("all_rows", [False, True])
def test_glm4_f16_file_runs_the_mfma_and_fused_paths(tmp_path, all_rows):
    assert os.path.exists(RUNNER), "tests/cpp/test_model_file is not built (run __graft_entry__.build())"
    tensors = mw.random_state_dict(GLM4, mw.glm2_weight_names(3), mw.glm2_shapes, 11, mw.F16)
    ids = [3, 17, 150, 42, 9, 77, 101, 5]
    run_case(tmp_path, 4, GLM4, mw.pack_config_v2(mw.F16, **GLM4), tensors, ids, 5, all_rows, max_length=32)


@pytest.mark.gpu
def test_glm4_f16_prompt_of_more_than_8_tokens(tmp_path):
    """The prompt takes the GEMM path of every Linear, with norms, gate and residuals folded into it."""
    tensors = mw.random_state_dict(GLM4, mw.glm2_weight_names(3), mw.glm2_shapes, 15, mw.F16)
    ids = list(range(30, 50)) + [7, 8]
    run_case(tmp_path, 4, GLM4, mw.pack_config_v2(mw.F16, **GLM4), tensors, ids, 20, True, max_length=32)


@pytest.mark.gpu
def test_glm3_f16_file_with_a_prefix_cache(tmp_path):
    cfg = dict(GLM4, num_key_value_heads=2, num_virtual_tokens=4, rope_theta=10000.0, norm_eps=1e-5)
    tensors = mw.random_state_dict(cfg, mw.glm2_weight_names(3, True), mw.glm2_shapes, 12, mw.F16)
    run_case(tmp_path, 3, cfg, mw.pack_config_v2(mw.F16, **cfg), tensors, [1, 2, 3, 4, 5, 6], 3, False)


@pytest.mark.gpu
def test_glm2_f32_file_with_the_version_1_record(tmp_path):
    rec = dict(vocab_size=80, hidden_size=64, num_attention_heads=4, num_hidden_layers=2, intermediate_size=96,
               max_length=24, bos_token_id=-1, eos_token_id=2, pad_token_id=0, sep_token_id=-1)
    cfg = dict(rec, num_key_value_heads=2, num_virtual_tokens=0, norm_eps=1e-5, rope_theta=10000.0)
    tensors = mw.random_state_dict(cfg, mw.glm2_weight_names(2), mw.glm2_shapes, 13, mw.F32)
    run_case(tmp_path, 2, cfg, mw.pack_config_v1(mw.F32, num_key_value_heads=2, **rec), tensors,
             [5, 6, 7, 8, 70, 71, 72], 4, False)


@pytest.mark.gpu
@pytest.mark.parametrize("weight_type", [mw.F32, mw.F16])
def test_glm1_file_tied_lm_head_mask_and_2d_positions(tmp_path, weight_type):
    rec = dict(vocab_size=96, hidden_size=128, num_attention_heads=4, num_hidden_layers=2, intermediate_size=512,
               max_length=24, bos_token_id=90, eos_token_id=91, pad_token_id=3, sep_token_id=-1)
    cfg = dict(rec, num_key_value_heads=4, num_virtual_tokens=0, norm_eps=1e-5, rope_theta=10000.0)
    tensors = mw.random_state_dict(cfg, mw.glm1_weight_names(2), mw.glm1_shapes, 14, weight_type)
    run_case(tmp_path, 1, cfg, mw.pack_config_v1(weight_type, **rec), tensors, [10, 11, 12, 13, 90, 20, 21], 5, False)


@pytest.mark.gpu
@pytest.mark.parametrize("qtype", [2, 3, 6, 7, 8])
def test_glm4_block_quantised_files(tmp_path, qtype):
    """q4_0 (the converter's default), q4_1, q5_0, q5_1, q8_0: the blocks the converter's quantisers write go to the
    device as they are, embedding table included; every Linear runs ggml's integer path (at most 8 rows here).

    The tolerance is ten times that of the fp16 files: the input rows of every Linear are rounded to 8-bit levels, so
    a difference in the last bits of an activation (the attention's tolerance, the order of a sum) now and then moves
    a level by one, which is 1/127 of the block's largest value; the reference's own tolerances for these types
    are 0.2 to 2.0 on a single Linear (chatglm_test.cpp:424-428)."""
    tensors = mw.random_state_dict(GLM4, mw.glm2_weight_names(3), mw.glm2_shapes, 20 + qtype, qtype)
    ids = [3, 17, 150, 42, 9, 77, 101]
    run_case(tmp_path, 4, GLM4, mw.pack_config_v2(qtype, **GLM4), tensors, ids, 4, False, max_length=32, tol=4e-2)


@pytest.mark.gpu
def test_glm1_q4_0_file_with_the_tied_lm_head(tmp_path):
    rec = dict(vocab_size=96, hidden_size=128, num_attention_heads=4, num_hidden_layers=2, intermediate_size=512,
               max_length=24, bos_token_id=90, eos_token_id=91, pad_token_id=3, sep_token_id=-1)
    cfg = dict(rec, num_key_value_heads=4, num_virtual_tokens=0, norm_eps=1e-5, rope_theta=10000.0)
    tensors = mw.random_state_dict(cfg, mw.glm1_weight_names(2), mw.glm1_shapes, 31, 2)
    run_case(tmp_path, 1, cfg, mw.pack_config_v1(2, **rec), tensors, [10, 11, 12, 13, 90, 20, 21], 5, False, tol=4e-2)


@pytest.mark.gpu
def test_a_prompt_of_more_than_8_tokens_takes_the_expanded_weights(tmp_path):
    tensors = mw.random_state_dict(GLM4, mw.glm2_weight_names(3), mw.glm2_shapes, 41, 8)
    ids = list(range(20, 32)) + [5, 6]
    run_case(tmp_path, 4, GLM4, mw.pack_config_v2(8, **GLM4), tensors, ids, 12, False, max_length=32, tol=4e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("fname", ["glm2_f16", "glm3_ptuning_f16", "glm4_q8_0", "glm1_q5_1", "glm2_q4_0"])
def test_files_written_by_the_reference_converter_run_end_to_end(tmp_path, fname):
    """tests/golden/reference_converter/*.bin are bytes of chatglm_cpp/convert.py itself (see
    tests/golden/make_model_file_goldens.py): loaded by the C++ model classes, run on the device, compared with the
    oracle-composed model built from the tensors that went into the converter."""
    import test_reference_converter_goldens as gold

    _, sname, model_type, wtype, cfg, _ = next(f for f in gold.FILES if f[0] == fname)
    state = np.load(os.path.join(gold.GOLD, sname + ".npz"))
    tensors = gold.expected_tensors(state, model_type, wtype, cfg)
    tol = 4e-3 if wtype in ("f16", "f32") else 4e-2
    run_case(tmp_path, model_type, cfg, None, tensors, [3, 17, 30, 22, 9, 1], 3, False, tol=tol,
             path=os.path.join(gold.GOLD, fname + ".bin"))
