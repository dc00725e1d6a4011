"""glm_attn_attend (the second half of forward as a call of its own) and glm_attn_set_qkv_views (the three views of
the fused projection in their general form, chatglm.cpp:636-653), against the oracle through the C-ABI.  The file
name makes pytest collect these after the tests of forward / decode / prefill themselves: with `pytest -x` a
failure in a newer entry point then does not hide the tests of the path every caller uses."""
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import gpu_harness

    return gpu_harness


@pytest.mark.parametrize("kw,qlen,n_past", [
    (dict(kvh=2, max_length=512), 37, 0),       # causal prompt, MFMA kernel
    (dict(kvh=2, max_length=512), 5, 137),      # unmasked continuation
    (dict(kvh=32, max_length=512, rope_type="glm1"), 20, 0),  # v1 additive mask
    (dict(h=4, kvh=2, d=64, max_length=40), 7, 3),            # generic kernel
])
def test_rope_append_then_attend_is_forward(H, kw, qlen, n_past):
    """glm_attn_rope_append followed by glm_attn_attend does what glm_attn_forward does (chatglm.cpp:655-717)."""
    kw = dict(kw)
    if kw.get("rope_type") == "glm1":
        kw.update(rope_type=H.orc.ROPE_CHATGLM, mask_type=H.orc.MASK_CHATGLM)
    p = H.Pair(**kw)
    if n_past:
        p.fill_past(0, n_past, seed=5)
    qkv = p.random_qkv(qlen, seed=60 + qlen)
    out, ref, _ = p.forward(0, qkv, n_past, entry="rope_append+attend", n_ctx=300)
    p.assert_caches_equal(0, "rope_append + attend")
    H.assert_close(out, ref, f"rope_append + attend, qlen {qlen}")
    p.close()


@pytest.mark.parametrize("shape,views", [
    # k heads first, then v heads, a gap, then the q heads, every head in a slot of d + 8 floats (all 16-byte aligned)
    (dict(kvh=2, max_length=512), "kv_first_padded_heads"),
    # the interleaved layout [h][3][d] spelled out as views on a context created with the plain layout
    (dict(kvh=32, max_length=512), "interleaved_as_views"),
    # offsets that are not multiples of 4 floats: one-token calls take the two-launch path
    (dict(kvh=2, max_length=512), "unaligned"),
    (dict(h=4, kvh=2, d=64, max_length=40), "kv_first_padded_heads"),  # generic kernel
])
def test_general_qkv_views(H, shape, views):
    """glm_attn_set_qkv_views: the three views of chatglm.cpp:636-653 with any offsets and head stride."""
    p = H.Pair(**shape)
    h, kvh, d = p.h, p.kvh, p.d
    if views == "kv_first_padded_heads":
        hs = d + 8
        v = (2 * kvh * hs + 16, 0, kvh * hs, hs)
    elif views == "interleaved_as_views":
        v = (0, d, 2 * d, 3 * d)
    else:
        hs = d + 2
        v = (1, h * hs + 3, (h + kvh) * hs + 5, hs)
    extent = max(v[0] + (h - 1) * v[3] + d, v[1] + (kvh - 1) * v[3] + d, v[2] + (kvh - 1) * v[3] + d)
    assert p.ctx.set_qkv_views(*v) == 0
    n_past = 0
    for qlen in (19, 1, 1, 7):
        qkv = p.random_qkv(qlen, seed=70 + qlen + n_past)
        for stride in (0, extent + 12):
            if stride and qlen == 1:
                continue
            if n_past:
                p.fill_past(0, n_past, seed=9 + n_past)
            out, ref, _ = p.forward(0, qkv, n_past, n_ctx=300, views=v + (stride or extent,),
                                    default_row_stride=(stride == 0))
            p.assert_caches_equal(0, f"views {views}, qlen {qlen}")
            H.assert_close(out, ref, f"views {views}, qlen {qlen}, row stride {stride}")
        n_past += qlen
    if views == "unaligned":
        import torch

        x = torch.zeros(extent, device=p.dev)
        o = torch.zeros(h * d, device=p.dev)
        assert p.ctx.decode(0, x.data_ptr(), n_past, o.data_ptr(), position_ids_host=[n_past]) == H.pkg.EUNSUPPORTED
    # a row stride that lets rows run into each other is refused
    import torch

    x = torch.zeros(4 * extent, device=p.dev)
    o = torch.zeros(2, h * d, device=p.dev)
    pos = torch.zeros(2, dtype=torch.int32, device=p.dev)
    assert p.ctx.forward(0, x.data_ptr(), 2, n_past, o.data_ptr(), position_ids_ptr=pos.data_ptr(),
                         qkv_row_stride=extent - 4) == H.pkg.EINVAL
    p.close()
