"""GPU parity: every call goes through the C-ABI of libglm_attn.so and is compared with the CPU oracle
on the same seeded inputs.  K and V caches must match bit for bit over the whole layer; the attention
output must satisfy |gpu - oracle| < 2e-3 + 1e-3 |oracle|."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import gpu_harness

    return gpu_harness


def test_config0_decode_at_512(H):
    """ChatGLM3-6B layer, one token at n_past = 512, max_length 2048."""
    p = H.Pair(max_length=2048)
    p.fill_past(0, 512, seed=0xC0FFEE)
    qkv = p.random_qkv(1, seed=0xC0FFEE + 7)
    for host_pos in (True, False):
        p.fill_past(0, 512, seed=0xC0FFEE)
        out, ref, _ = p.forward(0, qkv, 512, host_pos=host_pos)
        p.assert_caches_equal(0, "cfg0")
        H.assert_close(out, ref, "cfg0 decode")
    assert p.ctx.device_flags() == 0
    p.close()


@pytest.mark.parametrize("n_past", [0, 1, 63, 64, 65, 127, 128, 129, 1000, 2047])
def test_decode_tile_boundaries(H, n_past):
    p = H.Pair(max_length=2048, cache_fill=0x7E00)  # NaN in every slot that was never written
    p.fill_past(0, n_past, seed=11 + n_past)
    qkv = p.random_qkv(1, seed=500 + n_past)
    out, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode")
    p.assert_caches_equal(0, f"decode n_past={n_past}")
    H.assert_close(out, ref, f"decode n_past={n_past}")
    p.close()


def test_decode_sequence_through_persistent_cache(H):
    p = H.Pair(max_length=512)
    n0 = 70
    qkv = p.random_qkv(n0, seed=1)
    out, ref, _ = p.forward(0, qkv, 0)
    H.assert_close(out, ref, "prefill")
    for step in range(12):
        qkv = p.random_qkv(1, seed=100 + step)
        out, ref, _ = p.forward(0, qkv, n0 + step, host_pos=bool(step % 2))
        H.assert_close(out, ref, f"decode step {step}")
    p.assert_caches_equal(0, "after 12 decode steps")
    p.close()


@pytest.mark.parametrize("qlen", [1, 2, 31, 32, 33, 127, 128, 129, 300])
def test_prefill_causal_from_empty_cache(H, qlen):
    p = H.Pair(max_length=512, cache_fill=0x7E00)
    qkv = p.random_qkv(qlen, seed=qlen)
    out, ref, _ = p.forward(0, qkv, 0)
    p.assert_caches_equal(0, f"prefill q={qlen}")
    H.assert_close(out, ref, f"prefill q={qlen}")
    p.close()


@pytest.mark.parametrize("qlen,n_past", [(5, 300), (64, 64), (130, 333), (2, 1)])
def test_continuation_is_unmasked_like_the_reference(H, qlen, n_past):
    p = H.Pair(max_length=512, cache_fill=0x7E00)
    p.fill_past(0, n_past, seed=3)
    qkv = p.random_qkv(qlen, seed=4)
    out, ref, _ = p.forward(0, qkv, n_past)
    p.assert_caches_equal(0, "continuation")
    H.assert_close(out, ref, "continuation")
    p.close()


@pytest.mark.parametrize("max_length,qlen,n_past", [(200, 200, 0), (200, 72, 128), (72, 72, 0), (40, 40, 0),
                                                    (40, 8, 32), (136, 136, 0), (136, 3, 133)])
def test_prefill_where_the_cache_ends_inside_a_tile(H, max_length, qlen, n_past):
    """Cache lengths that are no multiple of the 64-key tile: the copy of the last tile has rows and columns that do
    not exist and must neither read outside the cache nor let what it reads instead (NaN-filled slots) through."""
    p = H.Pair(max_length=max_length, cache_fill=0x7E00)
    if n_past:
        p.fill_past(0, n_past, seed=11)
    qkv = p.random_qkv(qlen, seed=12)
    out, ref, _ = p.forward(0, qkv, n_past)
    p.assert_caches_equal(0, f"L={max_length} q={qlen} n_past={n_past}")
    H.assert_close(out, ref, f"L={max_length} q={qlen} n_past={n_past}")
    p.close()


@pytest.mark.parametrize("h,kvh,max_length,qlen,n_past,mask_rule", [
    (32, 2, 4096, 5, 3000, 0),      # a short follow-up against a long history: cut into 16 shares
    (32, 2, 4096, 130, 3900, 0),    # two token tiles, the cache almost full
    (32, 2, 4096, 20, 2000, 1),     # the same with the causal-offset rule: shares that end at the diagonal
    (32, 2, 8192, 300, 7000, 1),    # three token tiles, fewer shares (the partials have to fit)
    (32, 32, 2048, 128, 896, 0),    # 32 KV heads, 128 tokens at 896: two shares
    (32, 2, 1024, 7, 1000, 0),      # 16 tiles: the last share odd and short
    (32, 2, 4096, 2, 4000, 0),      # two tokens: 32 rows of a group in one tile, 62 tiles
    (32, 2, 4096, 9, 3000, 1),      # 144 rows per group: two row tiles, the second one mostly padding
    (32, 2, 4096, 64, 100, 1),      # 64 tokens x 16 heads = 8 row tiles per group, few keys: no cut
    (32, 4, 2048, 33, 1500, 0),     # groups of 8 heads
])
def test_short_chunk_against_a_long_cache_is_cut_along_the_keys(H, h, kvh, max_length, qlen, n_past, mask_rule):
    """Few token tiles and many key tiles: the MFMA kernel runs as several shares of the key range plus a merge."""
    p = H.Pair(h=h, kvh=kvh, max_length=max_length, mask_rule=mask_rule, cache_fill=0x7E00)
    p.fill_past(0, n_past, seed=21)
    qkv = p.random_qkv(qlen, seed=22)
    out, ref, _ = p.forward(0, qkv, n_past)
    p.assert_caches_equal(0, f"q={qlen} n_past={n_past}")
    H.assert_close(out, ref, f"q={qlen} n_past={n_past}")
    p.close()


@pytest.mark.parametrize("qlen,n_past", [(5, 300), (130, 333), (1, 17)])
def test_causal_offset_extension(H, qlen, n_past):
    p = H.Pair(max_length=512, mask_rule=1, cache_fill=0x7E00)
    p.fill_past(0, n_past, seed=5)
    qkv = p.random_qkv(qlen, seed=6)
    out, ref, _ = p.forward(0, qkv, n_past)
    p.assert_caches_equal(0, "causal offset")
    H.assert_close(out, ref, "causal offset")
    p.close()


def test_glm1_mha_2d_rope_and_mask(H):
    """ChatGLM-6B shape: 32 KV heads, interleaved qkv, 2-D NEOX rope, additive mask at n_past = 0."""
    orc = H.orc
    p = H.Pair(h=32, kvh=32, max_length=256, rope_type=orc.ROPE_CHATGLM, mask_type=orc.MASK_CHATGLM,
               interleaved=True, cache_fill=0x7E00)
    n0 = 100
    qkv = p.random_qkv(n0, seed=21)
    out, ref, _ = p.forward(0, qkv, 0, n_ctx=n0)
    p.assert_caches_equal(0, "glm1 prefill")
    H.assert_close(out, ref, "glm1 prefill")
    qkv = p.random_qkv(20, seed=22)
    out, ref, _ = p.forward(0, qkv, n0, n_ctx=n0)  # continuation chunk, unmasked
    H.assert_close(out, ref, "glm1 chunk")
    for step in range(4):
        qkv = p.random_qkv(1, seed=30 + step)
        out, ref, _ = p.forward(0, qkv, n0 + 20 + step, n_ctx=n0, host_pos=bool(step % 2))
        H.assert_close(out, ref, f"glm1 decode {step}")
    p.assert_caches_equal(0, "glm1 end")
    p.close()


@pytest.mark.parametrize("rope_type", [0, 2, 10000])
def test_full_head_rope_types(H, rope_type):
    p = H.Pair(max_length=256, rope_type=rope_type, cache_fill=0x7E00)
    qkv = p.random_qkv(40, seed=rope_type + 1)
    out, ref, _ = p.forward(0, qkv, 0)
    p.assert_caches_equal(0, f"rope {rope_type} prefill")
    H.assert_close(out, ref, f"rope {rope_type} prefill")
    qkv = p.random_qkv(1, seed=rope_type + 2)
    out, ref, _ = p.forward(0, qkv, 40, host_pos=True)
    p.assert_caches_equal(0, f"rope {rope_type} decode")
    H.assert_close(out, ref, f"rope {rope_type} decode")
    p.close()


@pytest.mark.parametrize("h,kvh,d,L", [(8, 2, 4, 13), (8, 8, 4, 8), (4, 2, 64, 100), (6, 3, 32, 50), (40, 2, 128, 64)])
def test_generic_kernel_shapes(H, h, kvh, d, L):
    """Head sizes and cache lengths the MFMA kernels are not written for take the generic kernel."""
    p = H.Pair(h=h, kvh=kvh, d=d, max_length=L, cache_fill=0x7E00)
    n0 = min(5, L - 3)
    qkv = p.random_qkv(n0, seed=h * d)
    out, ref, _ = p.forward(0, qkv, 0)
    H.assert_close(out, ref, "generic prefill")
    for step in range(3):
        qkv = p.random_qkv(1, seed=h * d + 1 + step)
        out, ref, _ = p.forward(0, qkv, n0 + step, host_pos=bool(step % 2))
        H.assert_close(out, ref, f"generic decode {step}")
    p.assert_caches_equal(0, "generic")
    p.close()


def test_prefix_cache_and_virtual_tokens(H):
    orc = H.orc
    nvt = 8
    p = H.Pair(max_length=248, nvt=nvt, cache_fill=0x7E00)
    import torch

    past = orc.randn_f16_bits(77, 0, 2 * p.kvh * nvt * p.d).reshape(2, p.kvh, nvt, p.d)
    orc.load_prefix_cache(p.ocfg, past, p.ref_k[0], p.ref_v[0])
    past_d = torch.from_numpy(past.view(np.int16)).to(p.dev)
    H.pkg.check(p.ctx.load_prefix_cache(0, past_d.data_ptr()), "load_prefix_cache")
    torch.cuda.synchronize()
    p.assert_caches_equal(0, "prefix")
    qkv = p.random_qkv(33, seed=78)
    out, ref, _ = p.forward(0, qkv, 0)
    H.assert_close(out, ref, "prefix prefill")
    qkv = p.random_qkv(1, seed=79)
    out, ref, _ = p.forward(0, qkv, 33, host_pos=True)
    H.assert_close(out, ref, "prefix decode")
    p.assert_caches_equal(0, "prefix end")
    p.close()


def test_layers_are_independent(H):
    p = H.Pair(num_layers=3, max_length=256)
    for layer in range(3):
        p.fill_past(layer, 100 + layer, seed=layer)
    for layer in (2, 0, 1):
        qkv = p.random_qkv(1, seed=40 + layer)
        out, ref, _ = p.forward(layer, qkv, 100 + layer, host_pos=True)
        H.assert_close(out, ref, f"layer {layer}")
    for layer in range(3):
        p.assert_caches_equal(layer, f"layer {layer}")
    p.close()


def test_position_out_of_table_sets_flag(H):
    p = H.Pair(max_length=64)
    qkv = p.random_qkv(2, seed=1)
    pos = np.array([5, 1000], dtype=np.int32)
    import torch

    qkv_d = torch.from_numpy(qkv).to(p.dev)
    pos_d = torch.from_numpy(pos).to(p.dev)
    out_d = torch.empty(2, p.h * p.d, dtype=torch.float32, device=p.dev)
    H.pkg.check(p.ctx.forward(0, qkv_d.data_ptr(), 2, 0, out_d.data_ptr(), position_ids_ptr=pos_d.data_ptr()), "fwd")
    assert p.ctx.device_flags() & 1
    p.close()


@pytest.mark.parametrize("entry", ["forward", "prefill", "rope_append"])
@pytest.mark.parametrize("interleaved,kvh,rope_type", [(False, 2, None), (True, 32, "glm1")])
def test_padded_qkv_rows(H, entry, interleaved, kvh, rope_type):
    """qkv_row_stride > width: the rows of the fused projection are views into a wider buffer (the views of
    chatglm.cpp:636-653 carry their own row stride); what lies between the rows is NaN here."""
    kw = dict(kvh=kvh, max_length=512, interleaved=interleaved)
    if rope_type == "glm1":
        kw.update(rope_type=H.orc.ROPE_CHATGLM, mask_type=H.orc.MASK_CHATGLM)
    p = H.Pair(**kw)
    p.fill_past(0, 100, seed=3)
    for qlen, n_past in ((37, 100), (5, 137)):
        qkv = p.random_qkv(qlen, seed=40 + qlen)
        out, ref, _ = p.forward(0, qkv, n_past, entry=entry, row_pad=24, n_ctx=300)
        p.assert_caches_equal(0, f"{entry} with padded rows")
        if entry != "rope_append":
            H.assert_close(out, ref, f"{entry} with padded rows, qlen {qlen}")
    p.close()


def test_range_errors(H):
    p = H.Pair(max_length=64)
    import torch

    qkv_d = torch.zeros(4, p.width, device=p.dev)
    out_d = torch.zeros(4, p.h * p.d, device=p.dev)
    pos_d = torch.zeros(4, dtype=torch.int32, device=p.dev)
    c = p.ctx
    assert c.forward(0, qkv_d.data_ptr(), 4, 61, out_d.data_ptr(), position_ids_ptr=pos_d.data_ptr()) == H.pkg.ERANGE
    assert c.forward(1, qkv_d.data_ptr(), 1, 0, out_d.data_ptr(), position_ids_ptr=pos_d.data_ptr()) == H.pkg.ERANGE
    assert c.forward(0, None, 1, 0, out_d.data_ptr(), position_ids_ptr=pos_d.data_ptr()) == H.pkg.EINVAL
    assert c.forward(0, qkv_d.data_ptr(), 1, 0, out_d.data_ptr()) == H.pkg.EINVAL  # no positions at all
    p.close()


@pytest.mark.parametrize("n_past", [700, 2047])
def test_decode_slow_path_when_workgroups_do_not_wait(H, n_past):
    """With a zero wait bound a wave gives up on its first look, flags its slice and looks once more; slices that
    are still missing then are redone by the workgroups that finish later: the result must not change."""
    p = H.Pair(max_length=2048)
    p.ctx.set_spin_limit_us(0)
    p.fill_past(0, n_past, seed=n_past)
    for rep in range(3):
        qkv = p.random_qkv(1, seed=900 + rep)
        p.fill_past(0, n_past, seed=n_past)
        out, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode")
        p.assert_caches_equal(0, "slow path")
        H.assert_close(out, ref, f"slow path rep {rep}")
    assert p.ctx.device_flags() == 0  # every slice was written in the end, by its owner's second look or by a sweep
    p.close()


def test_decode_repeated_launches_reuse_the_handover_state(H):
    p = H.Pair(num_layers=2, max_length=4096)
    p.fill_past(0, 4000, seed=1)
    p.fill_past(1, 3000, seed=2)
    for rep in range(6):
        layer = rep % 2
        n_past = (4000, 3000)[layer] + rep // 2
        qkv = p.random_qkv(1, seed=1000 + rep)
        out, ref, _ = p.forward(layer, qkv, n_past, host_pos=True)
        H.assert_close(out, ref, f"rep {rep}")
    p.assert_caches_equal(0)
    p.assert_caches_equal(1)
    p.close()


# The merge across workgroups changes shape with the number of splits (split lanes per line 1..16; 1, 2, 4 or 8
# lines per lane and block, up to four quads per block, 16 lines per lane as two blocks) and with the group size
# (padding heads).
@pytest.mark.parametrize("h,kvh,max_length,n_past", [
    (32, 2, 8192, 100),    # 2 tiles: one workgroup per group, no exchange
    (32, 2, 8192, 200),    # 4 tiles: the same, a full round
    (32, 2, 8192, 300),    # 5 splits of one tile
    (128, 128, 1024, 600), # 2 splits (2 CUs per group) of 5 tiles: two rounds in a workgroup
    (64, 64, 2048, 1000),  # 4 splits of 4 tiles
    (32, 2, 8192, 500),    # 8
    (32, 2, 8192, 1000),   # 16
    (32, 2, 8192, 1500),   # 24
    (32, 2, 8192, 3000),   # 47: three lines per lane, code for four
    (32, 2, 8192, 4095),   # 64
    (32, 2, 8192, 5000),   # 79: five lines per lane, code for eight
    (32, 2, 8192, 8191),   # 128
    (32, 32, 2048, 1000),  # one head per group, 8 splits
    (8, 2, 4096, 3000),    # four heads per group
    (16, 1, 16384, 16383), # 256 splits: 16 lines per lane, two blocks of eight
])
def test_decode_merge_geometries(H, h, kvh, max_length, n_past):
    p = H.Pair(h=h, kvh=kvh, max_length=max_length, cache_fill=0x7E00)
    p.fill_past(0, n_past, seed=21 + n_past)
    for rep in range(2):  # the second launch meets the first one's lines in the exchange buffer
        qkv = p.random_qkv(1, seed=600 + n_past + rep)
        p.fill_past(0, n_past, seed=21 + n_past)
        out, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode")
        p.assert_caches_equal(0, f"decode h={h} kvh={kvh} n_past={n_past}")
        H.assert_close(out, ref, f"decode h={h} kvh={kvh} n_past={n_past} rep {rep}")
    assert p.ctx.device_flags() == 0
    p.close()


@pytest.mark.parametrize("n_past", [200, 3000, 4095, 8191])
def test_decode_slow_path_geometries(H, n_past):
    p = H.Pair(max_length=8192)
    p.ctx.set_spin_limit_us(0)
    for rep in range(2):
        qkv = p.random_qkv(1, seed=950 + rep)
        p.fill_past(0, n_past, seed=n_past)
        out, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode")
        p.assert_caches_equal(0, "slow path")
        H.assert_close(out, ref, f"slow path n_past={n_past} rep {rep}")
    assert p.ctx.device_flags() == 0
    p.close()
