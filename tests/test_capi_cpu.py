"""CPU-side checks of the C-ABI library: it loads, exports every symbol include/glm_attn.h declares,
and rejects bad descriptors before touching a device.  No kernel is launched here."""
import ctypes
import os
import re
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
from __graft_entry__ import load_package  # noqa: E402

pkg = load_package()


def declared_symbols(header="glm_attn.h", prefix="glm_attn_"):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = pkg.lib()
    names = declared_symbols()
    assert len(names) >= 18
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/glm_attn.h but not exported"
    assert sorted(pkg.SYMBOLS) == names  # the Python binding covers the whole header
    assert b"gfx950" in lib.glm_attn_version()


def test_desc_defaults_and_kv_bytes():
    d = pkg.make_desc()
    assert (d.num_attention_heads, d.num_key_value_heads, d.head_size) == (32, 2, 128)
    assert d.rope_type == pkg.ROPE_CHATGLM2 and d.attn_mask_type == pkg.MASK_CAUSAL
    d.num_layers, d.max_length = 40, 32768
    assert pkg.lib().glm_attn_kv_bytes(ctypes.byref(d)) == 40 * 2 * 2 * 32768 * 128 * 2  # 1.34 GB
    d.num_virtual_tokens = 5
    assert pkg.lib().glm_attn_kv_bytes(ctypes.byref(d)) == 40 * 2 * 2 * 32773 * 128 * 2


def test_bad_descriptors_are_rejected_without_a_device():
    def status(**kw):
        d = pkg.make_desc(**kw)
        h = ctypes.c_void_p()
        st = pkg.lib().glm_attn_create(ctypes.byref(d), ctypes.byref(h))
        assert not h.value
        return st

    assert status(num_attention_heads=30, num_key_value_heads=4) == pkg.EINVAL   # heads not divisible
    assert status(interleaved_qkv=1) == pkg.EINVAL            # chatglm.cpp:637: interleaved needs kvh == h
    assert status(rope_type=3) == pkg.EINVAL                  # chatglm.cpp:615-616: unknown rope type
    assert status(max_length=0) == pkg.EINVAL
    assert status(struct_size=8) == pkg.EINVAL
    assert status(head_size=512) == pkg.EUNSUPPORTED
    assert status(attn_mask_type=7) == pkg.EINVAL
    assert pkg.lib().glm_attn_create(None, None) == pkg.EINVAL
    assert pkg.lib().glm_attn_forward(None, 0, None, 0, None, None, None, 1, 0, None, None) == pkg.EINVAL


def test_host_side_producers_match_the_oracle():
    import glm_oracle as orc

    for qlen, n_past, n_ctx in [(3, 0, 3), (1, 3, 3), (1, 4, 3), (128, 896, 897), (1, 1030, 897)]:
        out = np.zeros(2 * qlen, dtype=np.int32)
        assert pkg.lib().glm_attn_position_ids_glm(qlen, n_past, n_ctx, out.ctypes.data) == 0
        assert np.array_equal(out, orc.position_ids_glm(qlen, n_past, n_ctx))
        out = np.zeros(qlen, dtype=np.int32)
        assert pkg.lib().glm_attn_position_ids_glm2(qlen, n_past, out.ctypes.data) == 0
        assert np.array_equal(out, orc.position_ids_glm2(qlen, n_past))
    m = np.zeros((5, 9), dtype=np.float32)
    assert pkg.lib().glm_attn_attention_mask_glm(5, 9, m.ctypes.data) == 0
    assert np.array_equal(m, orc.attention_mask_glm(5, 9))


def test_strerror_covers_every_status():
    msgs = {pkg.lib().glm_attn_strerror(s) for s in (0, -1, -2, -3, -4, -5)}
    assert len(msgs) == 6 and b"unknown status" not in msgs
    assert pkg.lib().glm_attn_strerror(-99) == b"unknown status"


def test_library_exports_every_symbol_of_the_linear_header():
    lib = pkg.lib()
    names = [n for n in declared_symbols("glm_linear.h", "glm_linear_") if n not in ("glm_linear_fusion",)]
    assert len(names) == 8
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/glm_linear.h but not exported"
    assert sorted(pkg.LINEAR_SYMBOLS) == names


def test_bad_linear_descriptors_are_rejected_without_a_device():
    h = ctypes.c_void_p()
    d = pkg.make_linear_desc(64, 32)
    d.struct_size = 4
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    d = pkg.make_linear_desc(0, 32)
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    d = pkg.make_linear_desc(64, 32, weight_dtype=10)  # GGML_TYPE_Q2_K: not implemented
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EUNSUPPORTED
    d = pkg.make_linear_desc(48, 32, weight_dtype=8)  # GGML_TYPE_Q8_0 holds blocks of 32 inputs
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    # a caller-owned weight whose stated allocation is shorter than what the kernels read (64 x 32 fp16 = 4096 B;
    # Q8_0: 2 blocks of 34 B per feature) is refused before any device call; a size without a weight as well
    d = pkg.make_linear_desc(64, 32, weight=0x1000, weight_bytes=4095)
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    d = pkg.make_linear_desc(64, 32, weight_dtype=8, weight=0x1000, weight_bytes=32 * 2 * 34 - 1)
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    d = pkg.make_linear_desc(64, 32, weight_bytes=4096)
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    d = pkg.make_linear_desc(64, 32, weight=0x1000, weight_bytes=-1)
    assert pkg.lib().glm_linear_create(ctypes.byref(d), ctypes.byref(h)) == pkg.EINVAL
    assert pkg.lib().glm_linear_commit(None, None) == pkg.EINVAL
    assert pkg.lib().glm_linear_forward(None, None, 1, None, None) == pkg.EINVAL


def test_library_exports_every_symbol_of_the_block_header():
    lib = pkg.lib()
    names = declared_symbols("glm_block.h", "glm_block_")
    names = [n for n in names if n != "glm_block_activation"]  # the enum's typedef name, not a function
    assert len(names) == 5
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/glm_block.h but not exported"
    assert sorted(pkg.BLOCK_SYMBOLS) == names
    assert lib.glm_block_rms_norm(None, None, 1e-5, 1, 64, None, None) == pkg.EINVAL
    assert lib.glm_block_gated_activation(1, None, 4, pkg.ACT_SILU, 1, None) == pkg.EINVAL
    assert lib.glm_block_activation_forward(1, 4, 7, 1, None) == pkg.EINVAL  # no such activation


def test_bench_library_exports_every_symbol_of_the_bench_header_and_the_drop_in_none():
    lib = pkg.bench_lib()
    names = declared_symbols("glm_bench.h", "glm_bench_")
    names = [n for n in names if n not in ("glm_bench_pattern", "glm_bench_policy", "glm_bench_mfma_pattern")]
    assert names == ["glm_bench_mfma", "glm_bench_read", "glm_bench_read_sweep"]
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/glm_bench.h but not exported by libglm_bench.so"
        assert not hasattr(pkg.lib(), n), f"{n} is a measurement aid and must not be exported by libglm_attn.so"
    assert sorted(pkg.BENCH_SYMBOLS) == names
    assert lib.glm_bench_read(pkg.BENCH_READ_LINEAR, None, 256, 2, 0, None, None) == pkg.EINVAL
    assert lib.glm_bench_mfma(pkg.BENCH_MFMA_32X32X16, None, 0, 1, None, None, None) == pkg.EINVAL
    # shapes are checked before anything is launched
    assert lib.glm_bench_read_sweep(pkg.BENCH_POLICY_NT, 8, 16, 0, None, 1 << 25, None, None) == pkg.EINVAL
    assert lib.glm_bench_read_sweep(pkg.BENCH_POLICY_NT, 8, 16, 0, 1, 1000, 1, None) == pkg.EINVAL


def test_library_exports_every_symbol_of_the_model_file_header():
    lib = pkg.lib()
    names = declared_symbols("glm_model_file.h", "glm_model_file_")
    assert len(names) == 9
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/glm_model_file.h but not exported"
    assert sorted(pkg.MODEL_FILE_SYMBOLS) == names
    assert lib.glm_model_file_open(None, None) == pkg.EINVAL
    assert lib.glm_block_embedding(None, 1, 8, 8, None, 1, None, None) == pkg.EINVAL


def test_decode_launch_stamps_on_the_host(tmp_path):
    """tests/cpp/test_decode_stamp.cpp: the stamp arithmetic of the decode kernel's exchange, compiled for the
    host from the kernel's own header (a stamp is never 0, the count skips the one that would be)."""
    import subprocess

    exe = str(tmp_path / "test_decode_stamp")
    src = os.path.join(ROOT, "tests", "cpp", "test_decode_stamp.cpp")
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "chatglm.cpp_amd", "csrc")]
    subprocess.run(["/opt/rocm/bin/hipcc", "-O1", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", src, "-o", exe] + inc,
                   check=True, capture_output=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr


def test_launch_geometry_on_the_host(tmp_path):
    """tests/cpp/test_launch_plans.cpp: the functions that choose the grids of the decode and prefill kernels
    (splits, tiles per workgroup, shares of the key range, partials), compiled for the host from the kernels' own
    header and walked over many shapes: every extent a launch derives from them stays inside its buffer."""
    import subprocess

    exe = str(tmp_path / "test_launch_plans")
    src = os.path.join(ROOT, "tests", "cpp", "test_launch_plans.cpp")
    inc = ["-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "chatglm.cpp_amd", "csrc")]
    subprocess.run(["/opt/rocm/bin/hipcc", "-O1", "-std=c++17", "-x", "hip", "--offload-arch=gfx950", src, "-o", exe] + inc,
                   check=True, capture_output=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
