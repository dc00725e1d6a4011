"""glm_attn_decode_static (the split partials in a static device array, nothing allocated) against
glm_attn_decode on the same inputs, through the C-ABI: two calls in a row, the second with a smaller
input, and contexts of different shapes taking turns on the one array."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def H():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import gpu_harness

    return gpu_harness


def both(H, p, n_past, seed):
    """One token at n_past through both entry points from the same cache state; returns the two outputs."""
    qkv = p.random_qkv(1, seed=seed)
    p.fill_past(0, n_past, seed=n_past)
    out_a, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode")
    p.assert_caches_equal(0, "decode")
    p.fill_past(0, n_past, seed=n_past)
    out_b, ref_b, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode_static")
    p.assert_caches_equal(0, "decode_static")
    H.assert_close(out_b, ref, f"decode_static vs oracle at n_past={n_past}")
    H.assert_close(out_b, out_a, f"decode_static vs decode at n_past={n_past}")
    return out_a, out_b


def test_two_calls_in_a_row_the_second_smaller(H):
    p = H.Pair(max_length=8192, cache_fill=0x7E00)
    a1, b1 = both(H, p, 8191, seed=11)  # 128 splits per group
    a2, b2 = both(H, p, 700, seed=12)   # 11 splits: most of the array keeps the first call's lines
    # same kernel, same split geometry, lines folded in index order: the same bits
    assert np.array_equal(a1, b1) and np.array_equal(a2, b2)
    assert p.ctx.device_flags() == 0
    p.close()


def test_contexts_of_different_shapes_take_turns(H):
    p = H.Pair(max_length=4096)
    q = H.Pair(h=8, kvh=8, max_length=2048)  # one head per group, 8 groups: other regions of the array
    for rep in range(3):
        both(H, p, 3000 + rep, seed=21 + rep)
        both(H, q, 1500 + rep, seed=31 + rep)
    p.close()
    q.close()


def test_more_groups_than_the_array_has_room_for(H):
    import torch

    p = H.Pair(h=64, kvh=64, max_length=256)
    qkv_d = torch.zeros(p.width, device=p.dev)
    out_d = torch.zeros(p.h * p.d, device=p.dev)
    st = p.ctx.decode_static(0, qkv_d.data_ptr(), 10, out_d.data_ptr(), position_ids_host=[10])
    assert st == H.pkg.ESTATIC
    assert "32" in H.pkg.strerror(st)
    p.close()


@pytest.mark.parametrize("kw,n_past", [
    (dict(max_length=8192), 700),            # 11 splits of one tile, 12 quads a slice
    (dict(max_length=8192), 8191),           # 128 splits, one quad a slice
    (dict(h=8, kvh=8, max_length=2048), 1500),  # one head per group: grouped stamps of 8 groups side by side
    (dict(h=8, kvh=2, max_length=4096), 3000),  # four heads per group
])
def test_static_slow_path_when_workgroups_do_not_wait(H, kw, n_past):
    """The give-up / redo path of the exchange (wait bound 0: every wave gives up on its first look, flags its slice,
    and the workgroups that finish later redo what is still missing) on the static array: grouped stamps, the shared
    claim words.  Every kernel exits normally; the result must not change and nothing may be reported lost."""
    p = H.Pair(**kw)
    p.ctx.set_spin_limit_us(0)
    for rep in range(3):
        qkv = p.random_qkv(1, seed=700 + rep)
        p.fill_past(0, n_past, seed=n_past)
        out, ref, _ = p.forward(0, qkv, n_past, host_pos=True, entry="decode_static")
        p.assert_caches_equal(0, "static slow path")
        H.assert_close(out, ref, f"static slow path rep {rep}")
    assert p.ctx.device_flags() == 0  # the static array's own count of lost slices is part of the flags
    p.close()
