"""The format in which the decode kernel's workgroups exchange their partial results (csrc/attn_decode.hip,
pack_piece): O / sum as fp16 and the base-2 log-sum-exp as fp32, per (split, head).  A numpy model of that exchange
against the exact softmax-weighted sum in float64: the rounding of the lines costs at most 2^-11 (fp16's half unit in
the last place, relative) of the largest partial that carries weight, well inside the 2e-3 + 1e-3 |ref| of the parity
tests.  This pins the error bound the format is chosen for, not the kernel's code (the GPU parity tests do that)."""
import numpy as np
import pytest


def exact_and_exchanged(scores, values, nsplit):
    """scores [keys] (natural-log units), values [keys][dims] fp16-representable; keys dealt out to nsplit splits."""
    keys = scores.shape[0]
    s64 = scores.astype(np.float64)
    w = np.exp(s64 - s64.max())
    exact = (w[:, None] * values.astype(np.float64)).sum(0) / w.sum()
    bounds = np.linspace(0, keys, nsplit + 1).astype(int)
    lse, part = [], []
    for a, b in zip(bounds[:-1], bounds[1:]):
        if a == b:
            lse.append(np.float32(-np.inf))
            part.append(np.zeros(values.shape[1], dtype=np.float16))
            continue
        m = s64[a:b].max()
        e = np.exp(s64[a:b] - m)
        o = (e[:, None] * values[a:b].astype(np.float64)).sum(0) / e.sum()
        part.append(o.astype(np.float32).astype(np.float16))          # what a line carries
        lse.append(np.float32(m * np.log2(np.e) + np.log2(e.sum())))  # ... and the log-sum-exp beside it
    lse = np.array(lse, dtype=np.float32)
    part = np.array(part)
    wgt = np.exp2((lse - lse.max()).astype(np.float32)).astype(np.float32)  # the fold, fp32
    merged = (wgt[:, None] * part.astype(np.float32)).sum(0, dtype=np.float32) / wgt.sum(dtype=np.float32)
    return exact, merged, part, wgt


@pytest.mark.parametrize("nsplit", [2, 8, 47, 128])
@pytest.mark.parametrize("kind", ["gaussian", "peaked", "wide_range"])
def test_fp16_lines_cost_at_most_half_an_fp16_ulp_of_the_partials(nsplit, kind):
    rng = np.random.default_rng(nsplit * 7 + len(kind))
    keys, dims = 128 * nsplit, 16
    values = rng.standard_normal((keys, dims)).astype(np.float16)
    if kind == "gaussian":
        scores = rng.standard_normal(keys).astype(np.float32)
    elif kind == "peaked":
        scores = rng.standard_normal(keys).astype(np.float32)
        scores[rng.integers(keys)] += 30.0  # one key takes nearly all the weight
    else:
        scores = (rng.standard_normal(keys) * 25.0).astype(np.float32)  # splits differ by hundreds of log2 units
    exact, merged, part, wgt = exact_and_exchanged(scores, values, nsplit)
    carrying = np.abs(part.astype(np.float64))[wgt > 2.0 ** -20]
    bound = 2.0 ** -11 * carrying.max() + 1e-6
    err = np.abs(merged.astype(np.float64) - exact)
    assert err.max() <= bound, (err.max(), bound)
    # and that is inside the parity bar with room to spare
    assert np.all(err < 0.5 * (2e-3 + 1e-3 * np.abs(exact)))


def test_a_split_without_keys_carries_no_weight():
    scores = np.zeros(8, dtype=np.float32)
    values = np.ones((8, 4), dtype=np.float16)
    exact, merged, part, wgt = exact_and_exchanged(scores, values, 16)  # 8 of the 16 splits are empty
    assert np.count_nonzero(wgt) == 8
    assert np.allclose(merged, 1.0)
