"""ctypes binding of libglm_attn.so (include/glm_attn.h).

The library is the product; this module only declares its entry points for Python callers (tests,
benchmark).  There is no fallback: if the shared library is missing, loading raises.
"""
import ctypes
import os
import subprocess

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "libglm_attn.so")
CSRC = os.path.join(_PKG, "csrc")

OK, EINVAL, ERANGE, ENOMEM, EHIP, EUNSUPPORTED, ESTATIC = 0, -1, -2, -3, -4, -5, -6
ROPE_GPTJ, ROPE_NEOX, ROPE_CHATGLM, ROPE_CHATGLM2, ROPE_DISABLED = 0, 2, 4, 8, 10000
MASK_CAUSAL, MASK_CHATGLM = 0, 1
MASK_RULE_REFERENCE, MASK_RULE_CAUSAL_OFFSET = 0, 1

# every symbol include/glm_attn.h declares
SYMBOLS = [
    "glm_attn_default_desc", "glm_attn_kv_bytes", "glm_attn_create", "glm_attn_destroy", "glm_attn_set_qkv_views", "glm_attn_cache_ptrs",
    "glm_attn_forward", "glm_attn_rope_append", "glm_attn_attend", "glm_attn_decode", "glm_attn_decode_static", "glm_attn_prefill",
    "glm_attn_load_prefix_cache", "glm_attn_position_ids_glm2", "glm_attn_position_ids_glm",
    "glm_attn_attention_mask_glm", "glm_attn_scale_add", "glm_attn_device_flags", "glm_attn_set_spin_limit_us", "glm_attn_last_hip_error", "glm_attn_strerror",
    "glm_attn_version",
]
LINEAR_SYMBOLS = [
    "glm_linear_create", "glm_linear_destroy", "glm_linear_params", "glm_linear_forward", "glm_linear_forward_fused",
    "glm_linear_forward_glu", "glm_linear_commit", "glm_linear_last_hip_error",
]
PRO_NONE, PRO_RMS_NORM, PRO_GATED_ACT = 0, 1, 2
LINEAR_F32, LINEAR_F16 = 0, 1
LINEAR_Q4_0, LINEAR_Q4_1, LINEAR_Q5_0, LINEAR_Q5_1, LINEAR_Q8_0 = 2, 3, 6, 7, 8
BLOCK_SYMBOLS = [
    "glm_block_rms_norm", "glm_block_layer_norm", "glm_block_activation_forward", "glm_block_gated_activation",
    "glm_block_embedding",
]
MODEL_FILE_SYMBOLS = [
    "glm_model_file_open", "glm_model_file_close", "glm_model_file_last_error", "glm_model_file_config",
    "glm_model_file_data", "glm_model_file_tensor_count", "glm_model_file_tensor", "glm_model_file_find",
    "glm_model_file_upload",
]
BENCH_SYMBOLS = ["glm_bench_mfma", "glm_bench_read", "glm_bench_read_sweep"]
BENCH_POLICY_PLAIN, BENCH_POLICY_NT, BENCH_POLICY_SC1, BENCH_POLICY_SC0_SC1_NT = 0, 1, 2, 3
BENCH_MFMA_32X32X16, BENCH_MFMA_16X16X32, BENCH_MFMA_32X32X16_MIX, BENCH_MFMA_16X16X32_MIX = 0, 1, 2, 3
BENCH_READ_LINEAR, BENCH_READ_DECODE_PATTERN, BENCH_READ_STREAM, BENCH_EMPTY = 0, 1, 2, 3
MODEL_F32, MODEL_F16, MODEL_Q4_0, MODEL_Q4_1, MODEL_Q5_0, MODEL_Q5_1, MODEL_Q8_0 = 0, 1, 2, 3, 6, 7, 8


class ModelConfig(ctypes.Structure):
    """glm_model_config of include/glm_model_file.h."""
    _fields_ = [(n, ctypes.c_int32) for n in (
        "struct_size", "model_type", "version", "dtype", "vocab_size", "hidden_size", "num_attention_heads",
        "num_key_value_heads", "num_hidden_layers", "intermediate_size")] + [
        ("norm_eps", ctypes.c_float)] + [(n, ctypes.c_int32) for n in (
            "hidden_act", "use_qkv_bias", "use_dense_bias", "interleaved_qkv", "tie_word_embeddings", "rope_type")] + [
        ("rope_theta", ctypes.c_float)] + [(n, ctypes.c_int32) for n in (
            "attn_mask_type", "num_virtual_tokens", "max_length", "bos_token_id", "eos_token_id", "pad_token_id",
            "sep_token_id")] + [("tokenizer_offset", ctypes.c_int64), ("tokenizer_size", ctypes.c_int64)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_ if n != "struct_size"}


class ModelTensor(ctypes.Structure):
    """glm_model_tensor of include/glm_model_file.h."""
    _fields_ = [
        ("struct_size", ctypes.c_int32), ("dtype", ctypes.c_int32), ("ndim", ctypes.c_int32),
        ("reserved", ctypes.c_int32), ("ne", ctypes.c_int64 * 4), ("offset", ctypes.c_int64),
        ("nbytes", ctypes.c_int64), ("name", ctypes.c_char_p),
    ]
ACT_GELU, ACT_SILU = 0, 1


class LinearDesc(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_int32),
        ("in_features", ctypes.c_int32),
        ("out_features", ctypes.c_int32),
        ("weight_dtype", ctypes.c_int32),
        ("use_bias", ctypes.c_int32),
        ("max_rows", ctypes.c_int32),
        ("device", ctypes.c_int32),
        ("weight", ctypes.c_void_p),
        ("bias", ctypes.c_void_p),
        ("weight_bytes", ctypes.c_int64),
    ]


class LinearFusion(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_int32),
        ("prologue", ctypes.c_int32),
        ("norm_weight", ctypes.c_void_p),
        ("norm_eps", ctypes.c_float),
        ("activation", ctypes.c_int32),
        ("up", ctypes.c_void_p),
        ("residual", ctypes.c_void_p),
        ("residual_scale", ctypes.c_float),
    ]


def make_fusion(prologue=0, norm_weight=None, norm_eps=1e-5, activation=1, up=None, residual=None,
                residual_scale=1.0):
    f = LinearFusion()
    f.struct_size = ctypes.sizeof(LinearFusion)
    f.prologue, f.norm_weight, f.norm_eps = prologue, norm_weight, norm_eps
    f.activation, f.up, f.residual, f.residual_scale = activation, up, residual, residual_scale
    return f


class Desc(ctypes.Structure):
    _fields_ = [
        ("struct_size", ctypes.c_int32),
        ("num_layers", ctypes.c_int32),
        ("num_attention_heads", ctypes.c_int32),
        ("num_key_value_heads", ctypes.c_int32),
        ("head_size", ctypes.c_int32),
        ("max_length", ctypes.c_int32),
        ("num_virtual_tokens", ctypes.c_int32),
        ("rope_type", ctypes.c_int32),
        ("rope_theta", ctypes.c_float),
        ("attn_mask_type", ctypes.c_int32),
        ("interleaved_qkv", ctypes.c_int32),
        ("mask_rule", ctypes.c_int32),
        ("max_qlen", ctypes.c_int32),
        ("device", ctypes.c_int32),
        ("kv_buffer", ctypes.c_void_p),
    ]


def build(verbose=False):
    """Compile libglm_attn.so for gfx950 with the Makefile in csrc/ (hipcc cross-compiles without a GPU)."""
    r = subprocess.run(["make", "-C", CSRC, "-j8", "-B"], capture_output=True, text=True)
    if verbose or r.returncode != 0:
        print(r.stdout[-4000:])
        print(r.stderr[-4000:])
    if r.returncode != 0:
        raise RuntimeError("building libglm_attn.so failed")
    return LIB_PATH


_lib = None

# The instrumented build (csrc/Makefile, target `timeline`): the same library whose decode and prefill kernels
# leave clock readings per wave.  For finding where the time of a launch goes, never for timing it.
TIMELINE_LIB_PATH = os.path.join(_PKG, "libglm_attn_timeline.so")
TIMELINE_SLOTS = 4096  # waves recorded (kTimelineSlots)
# index -> what the wave had just done when it read the clock; slot = workgroup * 8 + wave, waves 0-3 of a
# decode workgroup are score waves, 4-7 output waves
DECODE_STAMPS = {
    "score": [(10, "wave started"), (5, "own work entered"), (8, "query loads issued"), (0, "K tile loads issued"),
              (1, "queries in LDS (and the new key)"), (2, "maxes of the last round left"),
              (3, "probabilities of the last round left"), (6, "first look at the others' lines"),
              (13, "polling entered (last pass)"), (15, "last poll's loads back"), (12, "all lines in (last pass)"),
              (11, "quads folded and written (last block)"), (7, "slice done")],
    "output": [(10, "wave started"), (0, "V column loads issued"), (3, "probabilities seen"), (4, "second product done"),
               (5, "lines issued")],
}
PREFILL_STAMPS = [(0, "wave started"), (1, "first copies issued"), (2, "first tiles landed"), (3, "first product done"),
                  (8, "1st tile of the group done"), (9, "2nd tile done"), (10, "4th tile done"), (4, "tile loop done"),
                  (5, "last second product done"), (6, "the two groups merged"), (7, "output stores issued")]


def use_timeline_build():
    """Makes lib() load the instrumented library.  Call before anything else of this module."""
    global LIB_PATH
    if _lib is not None:
        raise RuntimeError("the library is already loaded")
    LIB_PATH = TIMELINE_LIB_PATH


def read_timeline(kind):
    """Clock readings (100 MHz ticks) of the launches since the last call: array [TIMELINE_SLOTS][16] of int64, zero
    where a wave left none.  kind: "decode" or "prefill".  Only with the instrumented library."""
    import numpy as np

    fn = getattr(lib(), f"glm_attn_debug_{kind}_timeline", None)
    if fn is None:
        raise RuntimeError("timeline readings need the instrumented library: call use_timeline_build() first")
    fn.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
    fn.restype = ctypes.c_int
    n = TIMELINE_SLOTS * 16
    buf = (ctypes.c_ulonglong * n)()
    rc = fn(buf, n)
    if rc != 0:
        raise RuntimeError(f"glm_attn_debug_{kind}_timeline: hip error {rc}")
    return np.frombuffer(buf, dtype=np.uint64).reshape(TIMELINE_SLOTS, 16).astype(np.int64)


def summarise_timeline(t, stamps, rows):
    """Per stamp: waves that left one, and min / mean / max in us since the first wave of the launch started.
    rows: boolean mask over the slots (e.g. the score waves)."""
    start_idx = stamps[0][0]
    used = (t[:, start_idx] > 0) & rows
    if not used.any():
        return []
    t0 = t[(t[:, start_idx] > 0), start_idx].min()
    out = []
    for idx, name in stamps:
        v = t[used, idx]
        v = v[v >= t0]
        if v.size == 0:
            continue
        us = (v - t0) / 100.0
        out.append({"stamp": name, "waves": int(v.size), "min_us": round(float(us.min()), 2),
                    "mean_us": round(float(us.mean()), 2), "max_us": round(float(us.max()), 2)})
    return out


BENCH_LIB_PATH = os.path.join(_PKG, "libglm_bench.so")
_bench_lib = None


def bench_lib():
    """The measurement aids of include/glm_bench.h (libglm_bench.so): read kernels and loops of matrix
    instructions that bench.py --ceiling times beside the kernels of the path.  No part of the drop-in library."""
    global _bench_lib
    if _bench_lib is not None:
        return _bench_lib
    if not os.path.exists(BENCH_LIB_PATH):
        raise RuntimeError(f"{BENCH_LIB_PATH} is missing: build it with __graft_entry__.build()")
    c = ctypes
    P = c.c_void_p
    L = c.CDLL(BENCH_LIB_PATH)
    L.glm_bench_read.argtypes = [c.c_int, P, c.c_int32, c.c_int32, c.c_size_t, P, P]
    L.glm_bench_read.restype = c.c_int
    L.glm_bench_read_sweep.argtypes = [c.c_int, c.c_int32, c.c_int32, c.c_int32, P, c.c_size_t, P, P]
    L.glm_bench_read_sweep.restype = c.c_int
    L.glm_bench_mfma.argtypes = [c.c_int, P, c.c_size_t, c.c_int32, P, P, c.POINTER(c.c_double)]
    L.glm_bench_mfma.restype = c.c_int
    _bench_lib = L
    return L


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: build it with __graft_entry__.build() (there is no fallback path)")
    L = ctypes.CDLL(LIB_PATH)
    c = ctypes
    P = c.c_void_p
    descp = c.POINTER(Desc)
    L.glm_attn_default_desc.argtypes = [descp]
    L.glm_attn_default_desc.restype = None
    L.glm_attn_kv_bytes.argtypes = [descp]
    L.glm_attn_kv_bytes.restype = c.c_size_t
    L.glm_attn_create.argtypes = [descp, c.POINTER(P)]
    L.glm_attn_create.restype = c.c_int
    L.glm_attn_destroy.argtypes = [P]
    L.glm_attn_destroy.restype = None
    L.glm_attn_set_qkv_views.argtypes = [P, c.c_int64, c.c_int64, c.c_int64, c.c_int64]
    L.glm_attn_set_qkv_views.restype = c.c_int
    L.glm_attn_cache_ptrs.argtypes = [P, c.c_int32, c.POINTER(P), c.POINTER(P)]
    L.glm_attn_cache_ptrs.restype = c.c_int
    L.glm_attn_forward.argtypes = [P, c.c_int32, P, c.c_int64, P, P, P, c.c_int32, c.c_int32, P, P]
    L.glm_attn_forward.restype = c.c_int
    L.glm_attn_rope_append.argtypes = [P, c.c_int32, P, c.c_int64, P, c.c_int32, c.c_int32, P]
    L.glm_attn_rope_append.restype = c.c_int
    L.glm_attn_attend.argtypes = [P, c.c_int32, P, c.c_int32, c.c_int32, P, P]
    L.glm_attn_attend.restype = c.c_int
    L.glm_attn_decode.argtypes = [P, c.c_int32, P, P, P, c.c_int32, P, P]
    L.glm_attn_decode.restype = c.c_int
    L.glm_attn_decode_static.argtypes = [P, c.c_int32, P, P, P, c.c_int32, P, P]
    L.glm_attn_decode_static.restype = c.c_int
    L.glm_attn_prefill.argtypes = [P, c.c_int32, P, c.c_int64, P, P, c.c_int32, c.c_int32, P, P]
    L.glm_attn_prefill.restype = c.c_int
    L.glm_attn_load_prefix_cache.argtypes = [P, c.c_int32, P, P]
    L.glm_attn_load_prefix_cache.restype = c.c_int
    L.glm_attn_position_ids_glm2.argtypes = [c.c_int32, c.c_int32, P]
    L.glm_attn_position_ids_glm2.restype = c.c_int
    L.glm_attn_position_ids_glm.argtypes = [c.c_int32, c.c_int32, c.c_int32, P]
    L.glm_attn_position_ids_glm.restype = c.c_int
    L.glm_attn_attention_mask_glm.argtypes = [c.c_int32, c.c_int32, P]
    L.glm_attn_attention_mask_glm.restype = c.c_int
    L.glm_attn_scale_add.argtypes = [P, P, c.c_float, P, c.c_int64, P]
    L.glm_attn_scale_add.restype = c.c_int
    L.glm_attn_device_flags.argtypes = [P, c.POINTER(c.c_uint32)]
    L.glm_attn_device_flags.restype = c.c_int
    L.glm_attn_set_spin_limit_us.argtypes = [P, c.c_int64]
    L.glm_attn_set_spin_limit_us.restype = c.c_int
    L.glm_attn_last_hip_error.argtypes = [P]
    L.glm_attn_last_hip_error.restype = c.c_int
    L.glm_attn_strerror.argtypes = [c.c_int]
    L.glm_attn_strerror.restype = c.c_char_p
    L.glm_attn_version.argtypes = []
    L.glm_attn_version.restype = c.c_char_p
    L.glm_linear_create.argtypes = [c.POINTER(LinearDesc), c.POINTER(P)]
    L.glm_linear_create.restype = c.c_int
    L.glm_linear_destroy.argtypes = [P]
    L.glm_linear_destroy.restype = None
    L.glm_linear_params.argtypes = [P, c.POINTER(P), c.POINTER(P)]
    L.glm_linear_params.restype = c.c_int
    L.glm_linear_forward.argtypes = [P, P, c.c_int32, P, P]
    L.glm_linear_forward.restype = c.c_int
    L.glm_linear_forward_fused.argtypes = [P, c.POINTER(LinearFusion), P, c.c_int32, P, P]
    L.glm_linear_forward_fused.restype = c.c_int
    L.glm_linear_commit.argtypes = [P, P]
    L.glm_linear_commit.restype = c.c_int
    L.glm_linear_forward_glu.argtypes = [P, P, c.POINTER(LinearFusion), P, c.c_int32, P, P]
    L.glm_linear_forward_glu.restype = c.c_int
    L.glm_linear_last_hip_error.argtypes = [P]
    L.glm_linear_last_hip_error.restype = c.c_int
    L.glm_block_rms_norm.argtypes = [P, P, c.c_float, c.c_int32, c.c_int32, P, P]
    L.glm_block_rms_norm.restype = c.c_int
    L.glm_block_layer_norm.argtypes = [P, P, P, c.c_float, c.c_int32, c.c_int32, P, P]
    L.glm_block_layer_norm.restype = c.c_int
    L.glm_block_activation_forward.argtypes = [P, c.c_int64, c.c_int32, P, P]
    L.glm_block_activation_forward.restype = c.c_int
    L.glm_block_gated_activation.argtypes = [P, P, c.c_int64, c.c_int32, P, P]
    L.glm_block_gated_activation.restype = c.c_int
    L.glm_block_embedding.argtypes = [P, c.c_int32, c.c_int64, c.c_int32, P, c.c_int32, P, P]
    L.glm_block_embedding.restype = c.c_int
    L.glm_model_file_open.argtypes = [c.c_char_p, c.POINTER(P)]
    L.glm_model_file_open.restype = c.c_int
    L.glm_model_file_close.argtypes = [P]
    L.glm_model_file_close.restype = None
    L.glm_model_file_last_error.argtypes = []
    L.glm_model_file_last_error.restype = c.c_char_p
    L.glm_model_file_config.argtypes = [P, c.POINTER(ModelConfig)]
    L.glm_model_file_config.restype = c.c_int
    L.glm_model_file_data.argtypes = [P, c.POINTER(P), c.POINTER(c.c_int64)]
    L.glm_model_file_data.restype = c.c_int
    L.glm_model_file_tensor_count.argtypes = [P]
    L.glm_model_file_tensor_count.restype = c.c_int
    L.glm_model_file_tensor.argtypes = [P, c.c_int32, c.POINTER(ModelTensor)]
    L.glm_model_file_tensor.restype = c.c_int
    L.glm_model_file_find.argtypes = [P, c.c_char_p, c.POINTER(ModelTensor)]
    L.glm_model_file_find.restype = c.c_int
    L.glm_model_file_upload.argtypes = [P, c.c_int32, c.c_int64, c.c_int64, P, P]
    L.glm_model_file_upload.restype = c.c_int
    _lib = L
    return L


class GlmAttnError(RuntimeError):
    def __init__(self, status, what):
        self.status = status
        super().__init__(f"{what}: {lib().glm_attn_strerror(status).decode()} (status {status})")


def strerror(status):
    return lib().glm_attn_strerror(status).decode()


def check(status, what):
    if status != OK:
        raise GlmAttnError(status, what)


def make_desc(**kw):
    d = Desc()
    lib().glm_attn_default_desc(ctypes.byref(d))
    for k, v in kw.items():
        if not hasattr(d, k):
            raise AttributeError(k)
        setattr(d, k, v)
    return d


class Context:
    """Owns one glm_attn_ctx.  Pointers are raw device addresses (ints), e.g. torch.Tensor.data_ptr()."""

    def __init__(self, **desc_fields):
        self.desc = make_desc(**desc_fields)
        h = ctypes.c_void_p()
        check(lib().glm_attn_create(ctypes.byref(self.desc), ctypes.byref(h)), "glm_attn_create")
        self.handle = h

    def close(self):
        if getattr(self, "handle", None):
            lib().glm_attn_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def cache_rows(self):
        return self.desc.max_length + self.desc.num_virtual_tokens

    def cache_ptrs(self, layer):
        k, v = ctypes.c_void_p(), ctypes.c_void_p()
        check(lib().glm_attn_cache_ptrs(self.handle, layer, ctypes.byref(k), ctypes.byref(v)), "glm_attn_cache_ptrs")
        return k.value, v.value

    def forward(self, layer, qkv_ptr, qlen, n_past, out_ptr, position_ids_ptr=None, position_ids_host=None,
                attention_mask_ptr=None, qkv_row_stride=0, stream=None):
        hp = None
        if position_ids_host is not None:
            hp = (ctypes.c_int32 * len(position_ids_host))(*[int(x) for x in position_ids_host])
        return lib().glm_attn_forward(self.handle, layer, qkv_ptr, qkv_row_stride, attention_mask_ptr,
                                      position_ids_ptr, ctypes.cast(hp, ctypes.c_void_p) if hp is not None else None,
                                      qlen, n_past, out_ptr, stream)

    def set_qkv_views(self, q_offset, k_offset, v_offset, head_stride):
        return lib().glm_attn_set_qkv_views(self.handle, q_offset, k_offset, v_offset, head_stride)

    def rope_append(self, layer, qkv_ptr, position_ids_ptr, qlen, n_past, qkv_row_stride=0, stream=None):
        return lib().glm_attn_rope_append(self.handle, layer, qkv_ptr, qkv_row_stride, position_ids_ptr, qlen, n_past,
                                          stream)

    def attend(self, layer, qlen, n_past, out_ptr, attention_mask_ptr=None, stream=None):
        return lib().glm_attn_attend(self.handle, layer, attention_mask_ptr, qlen, n_past, out_ptr, stream)

    def decode(self, layer, qkv_ptr, n_past, out_ptr, position_ids_ptr=None, position_ids_host=None, stream=None):
        hp = None
        if position_ids_host is not None:
            hp = (ctypes.c_int32 * len(position_ids_host))(*[int(x) for x in position_ids_host])
        return lib().glm_attn_decode(self.handle, layer, qkv_ptr, position_ids_ptr,
                                     ctypes.cast(hp, ctypes.c_void_p) if hp is not None else None, n_past, out_ptr,
                                     stream)

    def decode_static(self, layer, qkv_ptr, n_past, out_ptr, position_ids_ptr=None, position_ids_host=None,
                      stream=None):
        hp = None
        if position_ids_host is not None:
            hp = (ctypes.c_int32 * len(position_ids_host))(*[int(x) for x in position_ids_host])
        return lib().glm_attn_decode_static(self.handle, layer, qkv_ptr, position_ids_ptr,
                                            ctypes.cast(hp, ctypes.c_void_p) if hp is not None else None, n_past,
                                            out_ptr, stream)

    def prefill(self, layer, qkv_ptr, position_ids_ptr, qlen, n_past, out_ptr, attention_mask_ptr=None,
                qkv_row_stride=0, stream=None):
        return lib().glm_attn_prefill(self.handle, layer, qkv_ptr, qkv_row_stride, attention_mask_ptr,
                                      position_ids_ptr, qlen, n_past, out_ptr, stream)

    def load_prefix_cache(self, layer, past_kv_ptr, stream=None):
        return lib().glm_attn_load_prefix_cache(self.handle, layer, past_kv_ptr, stream)

    def device_flags(self):
        f = ctypes.c_uint32(0)
        check(lib().glm_attn_device_flags(self.handle, ctypes.byref(f)), "glm_attn_device_flags")
        return f.value

    def set_spin_limit_us(self, us):
        check(lib().glm_attn_set_spin_limit_us(self.handle, int(us)), "glm_attn_set_spin_limit_us")

    def last_hip_error(self):
        return lib().glm_attn_last_hip_error(self.handle)


def make_linear_desc(in_features, out_features, weight_dtype=LINEAR_F16, use_bias=True, max_rows=1, device=0,
                     weight=None, bias=None, weight_bytes=0):
    d = LinearDesc()
    d.struct_size = ctypes.sizeof(LinearDesc)
    d.in_features, d.out_features = in_features, out_features
    d.weight_dtype, d.use_bias, d.max_rows, d.device = weight_dtype, int(bool(use_bias)), max_rows, device
    d.weight, d.bias, d.weight_bytes = weight, bias, weight_bytes
    return d


class Linear:
    """Owns one glm_linear (Linear of chatglm.h:362-377).  Pointers are raw device addresses (ints)."""

    def __init__(self, in_features, out_features, **kw):
        self.desc = make_linear_desc(in_features, out_features, **kw)
        h = ctypes.c_void_p()
        check(lib().glm_linear_create(ctypes.byref(self.desc), ctypes.byref(h)), "glm_linear_create")
        self.handle = h

    def close(self):
        if getattr(self, "handle", None):
            lib().glm_linear_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def params(self):
        w, b = ctypes.c_void_p(), ctypes.c_void_p()
        check(lib().glm_linear_params(self.handle, ctypes.byref(w), ctypes.byref(b)), "glm_linear_params")
        return w.value, b.value

    def forward(self, x_ptr, rows, y_ptr, stream=None):
        return lib().glm_linear_forward(self.handle, x_ptr, rows, y_ptr, stream)

    def forward_fused(self, fusion, x_ptr, rows, y_ptr, stream=None):
        return lib().glm_linear_forward_fused(self.handle, ctypes.byref(fusion), x_ptr, rows, y_ptr, stream)

    def commit(self, stream=None):
        check(lib().glm_linear_commit(self.handle, stream), "glm_linear_commit")

    def forward_glu(self, up, fusion, x_ptr, rows, y_ptr, stream=None):
        """self is the gate projection: y = act(self(x)) * up(x) in one launch."""
        return lib().glm_linear_forward_glu(self.handle, up.handle, ctypes.byref(fusion), x_ptr, rows, y_ptr, stream)

    def last_hip_error(self):
        return lib().glm_linear_last_hip_error(self.handle)


class ModelFile:
    """A mapped "ggml" model file (include/glm_model_file.h): config, tensor records, uploads."""

    def __init__(self, path):
        self.handle = ctypes.c_void_p()
        st = lib().glm_model_file_open(os.fsencode(path), ctypes.byref(self.handle))
        if st != 0:
            raise GlmAttnError(st, "glm_model_file_open: " + lib().glm_model_file_last_error().decode(errors="replace"))

    def close(self):
        if self.handle:
            lib().glm_model_file_close(self.handle)
            self.handle = ctypes.c_void_p()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def config(self):
        c = ModelConfig()
        c.struct_size = ctypes.sizeof(ModelConfig)
        check(lib().glm_model_file_config(self.handle, ctypes.byref(c)), "glm_model_file_config")
        return c

    def __len__(self):
        return lib().glm_model_file_tensor_count(self.handle)

    def tensor(self, index):
        t = ModelTensor()
        t.struct_size = ctypes.sizeof(ModelTensor)
        check(lib().glm_model_file_tensor(self.handle, index, ctypes.byref(t)), "glm_model_file_tensor")
        return t

    def find(self, name):
        t = ModelTensor()
        t.struct_size = ctypes.sizeof(ModelTensor)
        st = lib().glm_model_file_find(self.handle, name.encode(), ctypes.byref(t))
        return None if st == ERANGE else (check(st, "glm_model_file_find"), t)[1]

    def host_bytes(self, t):
        """The tensor's data in the mapping, as a bytes copy."""
        base, size = ctypes.c_void_p(), ctypes.c_int64()
        check(lib().glm_model_file_data(self.handle, ctypes.byref(base), ctypes.byref(size)), "glm_model_file_data")
        return ctypes.string_at(base.value + t.offset, t.nbytes)

    def upload(self, index, device_ptr, src_offset=0, nbytes=None, stream=None):
        if nbytes is None:
            nbytes = self.tensor(index).nbytes - src_offset
        return lib().glm_model_file_upload(self.handle, index, src_offset, nbytes, device_ptr, stream)
