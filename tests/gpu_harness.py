"""Shared plumbing of the GPU parity tests: device buffers come from torch, every computation goes
through the C-ABI of libglm_attn.so, and the CPU oracle is the checker."""
import ctypes
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import glm_oracle as orc  # noqa: E402
from __graft_entry__ import load_package  # noqa: E402

pkg = load_package()

ATOL, RTOL = 2e-3, 1e-3  # attention output tolerance of the path (fp32 output, fp16 cache)


_hip = None


def hip_memcpy_dtod(dst_ptr, src_ptr, nbytes):
    """Device-to-device copy between raw pointers (for memory the library owns), after a device synchronise."""
    global _hip
    import torch

    torch.cuda.synchronize()
    if _hip is None:
        _hip = ctypes.CDLL(os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so"))
        _hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        _hip.hipMemcpy.restype = ctypes.c_int
    rc = _hip.hipMemcpy(dst_ptr, src_ptr, nbytes, 3)  # hipMemcpyDeviceToDevice
    assert rc == 0, f"hipMemcpy failed with {rc}"


def assert_close(out, ref, what=""):
    """allclose with the reference test's rule (chatglm_test.cpp:36-40): |a-b| < atol + rtol |b|."""
    out = np.asarray(out, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    assert out.shape == ref.shape, (out.shape, ref.shape)
    assert np.all(np.isfinite(out)), f"{what}: non-finite output"
    err = np.abs(out - ref)
    bad = err >= ATOL + RTOL * np.abs(ref)
    assert not bad.any(), (f"{what}: {bad.sum()} of {bad.size} elements differ, max abs {err.max():.3e}, "
                           f"max rel {np.max(err / (np.abs(ref) + 1e-30)):.3e}")
    return float(err.max())


class Pair:
    """One GPU context and one oracle state with the same configuration and the same cache contents."""

    def __init__(self, num_layers=1, h=32, kvh=2, d=128, max_length=2048, nvt=0, rope_type=orc.ROPE_CHATGLM2,
                 rope_theta=10000.0, mask_type=orc.MASK_CAUSAL, interleaved=False, mask_rule=0, max_qlen=0,
                 cache_fill=0, device="cuda:0"):
        import torch

        self.torch = torch
        self.dev = torch.device(device)
        self.h, self.kvh, self.d, self.nvt = h, kvh, d, nvt
        self.interleaved = bool(interleaved)
        self.L = max_length + nvt
        self.num_layers = num_layers
        self.rope_type = rope_type
        self.ocfg = orc.make_cfg(num_attention_heads=h, num_key_value_heads=kvh, head_size=d, max_length=max_length,
                                 num_virtual_tokens=nvt, rope_type=rope_type, rope_theta=rope_theta,
                                 attn_mask_type=mask_type, interleaved_qkv=interleaved,
                                 mask_continuation=bool(mask_rule))
        self.layer_halfs = 2 * kvh * self.L * d
        # the slab lives in a torch tensor so that tests can read the caches back without extra API
        self.kv = torch.full((num_layers * self.layer_halfs,), cache_fill, dtype=torch.int16, device=self.dev)
        self.ctx = pkg.Context(num_layers=num_layers, num_attention_heads=h, num_key_value_heads=kvh, head_size=d,
                               max_length=max_length, num_virtual_tokens=nvt, rope_type=rope_type,
                               rope_theta=rope_theta, attn_mask_type=mask_type, interleaved_qkv=int(interleaved),
                               mask_rule=mask_rule, max_qlen=max_qlen, kv_buffer=self.kv.data_ptr())
        self.ref_k = []
        self.ref_v = []
        for _ in range(num_layers):
            k, v = orc.new_caches(self.ocfg, fill=cache_fill & 0xFFFF)
            self.ref_k.append(k)
            self.ref_v.append(v)
        self.width = (h + 2 * kvh) * d

    def close(self):
        self.ctx.close()

    # ---- cache access
    def gpu_caches(self, layer):
        t = self.kv[layer * self.layer_halfs:(layer + 1) * self.layer_halfs].cpu().numpy().view(np.uint16)
        half = self.layer_halfs // 2
        return t[:half].reshape(self.kvh, self.L, self.d), t[half:].reshape(self.kvh, self.d, self.L)

    def set_caches(self, layer, k_bits, v_bits):
        """Same fp16 bit patterns into the oracle's and the GPU's caches."""
        torch = self.torch
        self.ref_k[layer][...] = k_bits
        self.ref_v[layer][...] = v_bits
        flat = np.concatenate([self.ref_k[layer].reshape(-1), self.ref_v[layer].reshape(-1)]).view(np.int16)
        self.kv[layer * self.layer_halfs:(layer + 1) * self.layer_halfs] = torch.from_numpy(flat).to(self.dev)

    def fill_past(self, layer, n_past, seed):
        """Positions [nvt, nvt + n_past) of both caches from N(0,1) rounded to fp16; the rest keeps its fill."""
        p0, p1 = self.nvt, self.nvt + n_past
        k = self.ref_k[layer].copy()
        v = self.ref_v[layer].copy()
        k[:, p0:p1, :] = orc.randn_f16_bits(seed, 1, self.kvh * n_past * self.d).reshape(self.kvh, n_past, self.d)
        v[:, :, p0:p1] = orc.randn_f16_bits(seed, 2, self.kvh * self.d * n_past).reshape(self.kvh, self.d, n_past)
        self.set_caches(layer, k, v)

    def assert_caches_equal(self, layer, what=""):
        gk, gv = self.gpu_caches(layer)
        nk = int(np.count_nonzero(gk != self.ref_k[layer]))
        nv = int(np.count_nonzero(gv != self.ref_v[layer]))
        assert nk == 0 and nv == 0, f"{what}: cache mismatch, {nk} K and {nv} V halfs differ"

    # ---- positions and masks as the reference's set_graph_inputs makes them
    def positions(self, qlen, n_past, n_ctx=None):
        if self.rope_type == orc.ROPE_CHATGLM:
            return orc.position_ids_glm(qlen, n_past, n_ctx if n_ctx is not None else n_past + qlen)
        return orc.position_ids_glm2(qlen, n_past)

    def mask_for(self, qlen, n_past):
        if self.ocfg.attn_mask_type == orc.MASK_CHATGLM and n_past == 0 and not self.ocfg.mask_continuation:
            return orc.attention_mask_glm(qlen, self.nvt + n_past + qlen)
        return None

    # ---- one call through both implementations
    def forward(self, layer, qkv, n_past, pos=None, mask=None, host_pos=False, entry="forward", n_ctx=None,
                oracle_rows=None, use_default_mask=True, row_pad=0, views=None, default_row_stride=False):
        """row_pad > 0: the device copy of qkv gets that many floats of NaN behind every row and the call is
        made with qkv_row_stride = width + row_pad (entries "forward", "prefill" and "rope_append").
        views = (q_offset, k_offset, v_offset, head_stride, row_stride): the context has been given these views
        (set_qkv_views); the device copy of qkv is laid out accordingly, NaN wherever no view reaches;
        default_row_stride: the call passes qkv_row_stride = 0 (the views' own extent) instead of row_stride."""
        torch = self.torch
        qlen = qkv.shape[0]
        if pos is None:
            pos = self.positions(qlen, n_past, n_ctx)
        if mask is None and use_default_mask:
            mask = self.mask_for(qlen, n_past)
        qkv_ref = qkv.copy()
        if oracle_rows is None:
            ref = orc.attention_forward(self.ocfg, qkv_ref, pos, n_past, self.ref_k[layer], self.ref_v[layer],
                                        attention_mask=mask)
        else:
            orc.rope_inplace(self.ocfg, qkv_ref, pos)
            orc.append(self.ocfg, qkv_ref, n_past, self.ref_k[layer], self.ref_v[layer])
            ref = orc.attend(self.ocfg, qkv_ref, n_past, self.ref_k[layer], self.ref_v[layer], attention_mask=mask,
                             rows=oracle_rows)
        stride = 0
        if views is not None:
            q_off, k_off, v_off, hs, stride = views
            laid = np.full((qlen, stride), np.nan, dtype=np.float32)
            std = qkv.reshape(qlen, -1)
            d = self.d
            if self.interleaved:  # the oracle's row is [h][3][d]
                src = lambda which, i: std[:, (3 * i + which) * d:(3 * i + which + 1) * d]
            else:
                base = (0, self.h * d, (self.h + self.kvh) * d)
                src = lambda which, i: std[:, base[which] + i * d:base[which] + (i + 1) * d]
            for which, off, n in ((0, q_off, self.h), (1, k_off, self.kvh), (2, v_off, self.kvh)):
                for i in range(n):
                    laid[:, off + i * hs:off + i * hs + d] = src(which, i)
            qkv_d = torch.from_numpy(laid).to(self.dev)
            if default_row_stride:
                stride = 0
        elif row_pad:
            padded = np.full((qlen, self.width + row_pad), np.nan, dtype=np.float32)
            padded[:, :self.width] = qkv
            qkv_d = torch.from_numpy(padded).to(self.dev)
            stride = self.width + row_pad
        else:
            qkv_d = torch.from_numpy(qkv).to(self.dev)
        pos_d = torch.from_numpy(np.ascontiguousarray(pos, dtype=np.int32)).to(self.dev)
        mask_d = None if mask is None else torch.from_numpy(np.ascontiguousarray(mask, dtype=np.float32)).to(self.dev)
        out_d = torch.full((qlen, self.h * self.d), float("nan"), dtype=torch.float32, device=self.dev)
        mp = None if mask_d is None else mask_d.data_ptr()
        if entry == "forward":
            st = self.ctx.forward(layer, qkv_d.data_ptr(), qlen, n_past, out_d.data_ptr(),
                                  position_ids_ptr=None if host_pos else pos_d.data_ptr(),
                                  position_ids_host=pos if host_pos else None, attention_mask_ptr=mp,
                                  qkv_row_stride=stride)
        elif entry == "rope_append":  # the first half alone: caches only, no output
            st = self.ctx.rope_append(layer, qkv_d.data_ptr(), pos_d.data_ptr(), qlen, n_past, qkv_row_stride=stride)
        elif entry == "rope_append+attend":  # the two halves of forward as two calls
            st = self.ctx.rope_append(layer, qkv_d.data_ptr(), pos_d.data_ptr(), qlen, n_past, qkv_row_stride=stride)
            pkg.check(st, "glm_attn_rope_append")
            st = self.ctx.attend(layer, qlen, n_past, out_d.data_ptr(), attention_mask_ptr=mp)
        elif entry == "decode":
            st = self.ctx.decode(layer, qkv_d.data_ptr(), n_past, out_d.data_ptr(),
                                 position_ids_ptr=None if host_pos else pos_d.data_ptr(),
                                 position_ids_host=pos if host_pos else None)
        elif entry == "decode_static":
            st = self.ctx.decode_static(layer, qkv_d.data_ptr(), n_past, out_d.data_ptr(),
                                        position_ids_ptr=None if host_pos else pos_d.data_ptr(),
                                        position_ids_host=pos if host_pos else None)
        elif entry == "prefill":
            st = self.ctx.prefill(layer, qkv_d.data_ptr(), pos_d.data_ptr(), qlen, n_past, out_d.data_ptr(),
                                  attention_mask_ptr=mp, qkv_row_stride=stride)
        else:
            raise ValueError(entry)
        pkg.check(st, f"glm_attn_{entry}")
        torch.cuda.synchronize()
        return out_d.cpu().numpy(), ref, qkv_ref

    def random_qkv(self, qlen, seed):
        return orc.randn_f32(seed, 0, qlen * self.width).reshape(qlen, self.width)
