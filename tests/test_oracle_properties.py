"""Property tests (hypothesis) of the CPU oracle on randomly drawn shapes and values.

The fixed-seed pins (tests/test_oracle_gemm.py, tests/test_oracle_rowops.py) check the oracle against
independent routines on chosen inputs; these draw shapes, strides of values and scales at random and check
relations that must hold for every input: exact integer accumulators against python integers, linearity,
the two rounding modes at most one step apart, clamp bounds, batch independence, LayerNorm's invariance
under shifts and its zero-mean / unit-variance output, the softmax row sum, the tanh-GELU odd-part identity.
"""
import numpy as np
import pytest
from hypothesis import HealthCheck, given, settings
from hypothesis import strategies as st

import oracle as O

SET = settings(max_examples=60, deadline=None, suppress_health_check=[HealthCheck.too_slow, HealthCheck.data_too_large])

dims = st.tuples(st.integers(1, 24), st.integers(1, 24), st.integers(1, 96))
seeds = st.integers(0, 2**31 - 1)


def _ops(seed, M, N, K, lo=-128):
    g = np.random.default_rng(seed)
    return g.integers(lo, 128, size=(M, K), dtype=np.int8), g.integers(lo, 128, size=(N, K), dtype=np.int8), g


@SET
@given(dims, seeds)
def test_int32_accumulator_is_the_exact_integer_product(d, seed):
    M, N, K = d
    a, w, g = _ops(seed, M, N, K)
    bias = g.integers(-2**24, 2**24, size=N, dtype=np.int32)
    got = O.linear_a8_w8_b32_o32(a, w, bias)
    want = [[sum(int(a[m, k]) * int(w[n, k]) for k in range(K)) + int(bias[n]) for n in range(N)] for m in range(M)]
    assert got.dtype == np.int32 and got.tolist() == want


@SET
@given(dims, seeds)
def test_accumulator_is_linear_in_the_activations(d, seed):
    M, N, K = d
    _, w, g = _ops(seed, M, N, K)
    a = g.integers(-60, 61, size=(M, K), dtype=np.int8)
    a2 = g.integers(-60, 61, size=(M, K), dtype=np.int8)
    s = O.linear_a8_w8_b32_o32((a.astype(np.int16) + a2).astype(np.int8), w, None)
    assert np.array_equal(s, O.linear_a8_w8_b32_o32(a, w, None) + O.linear_a8_w8_b32_o32(a2, w, None))
    # and the BMM of a batch is its slices' linears
    b3 = O.bmm_s8t_s8n_s32t(np.stack([a, a2]), np.stack([w, w]))
    assert np.array_equal(b3[0], O.linear_a8_w8_b32_o32(a, w, None)) and np.array_equal(b3[1], O.linear_a8_w8_b32_o32(a2, w, None))


@SET
@given(dims, seeds, st.floats(1e-4, 0.5), st.floats(0.0, 2.0))
def test_int8_epilogues_round_and_clamp(d, seed, alpha, beta):
    M, N, K = d
    a, w, g = _ops(seed, M, N, K)
    b8 = g.integers(-127, 128, size=N, dtype=np.int8)
    alpha, beta = np.float32(alpha), np.float32(beta)
    acc = O.linear_a8_w8_b32_o32(a, w, None)
    v = (alpha * acc.astype(np.float32)) + (beta * b8.astype(np.float32))          # fp32, each step rounded
    rne = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta)
    assert np.array_equal(rne, np.clip(np.rint(v), -128, 127).astype(np.int8))     # numpy's rint is half-to-even
    tr = O.linear_a8_w8_b8_o8(a, w, b8, alpha, beta, round_mode=O.TRUNC)
    assert np.array_equal(tr, np.clip(np.trunc(v), -128, 127).astype(np.int8))
    assert np.abs(rne.astype(int) - tr.astype(int)).max() <= 1                     # the literal Triton cast is one step away at most
    relu = O.linear_relu_a8_w8_b8_o8(a, w, b8, alpha, beta)
    assert np.array_equal(relu, np.maximum(rne, 0))
    f = O.linear_a8_w8_bfp32_ofp32(a, w, b8.astype(np.float32), alpha, beta)
    assert np.array_equal(f, v)


@SET
@given(st.integers(1, 12), st.integers(2, 700), seeds, st.floats(-50, 50), st.floats(0.01, 30))
def test_layernorm_q_statistics_and_shift_invariance(rows, cols, seed, shift, spread):
    g = np.random.default_rng(seed)
    x = (g.standard_normal((rows, cols)) * spread).astype(np.float32)
    ones, zeros = np.ones(cols, np.float32), np.zeros(cols, np.float32)
    q, mean, rstd = O.layernorm_q(x, ones * 20, zeros, 1e-5, return_stats=True)
    x64 = x.astype(np.float64)
    assert np.allclose(mean, x64.mean(-1), rtol=1e-4, atol=1e-4 * spread)
    assert np.allclose(rstd, 1 / np.sqrt(x64.var(-1) + 1e-5), rtol=1e-4)
    # normalised rows: mean 0 and variance 1 before the affine part (here scaled by 20, then rounded)
    y = q.astype(np.float64) / 20
    if cols >= 64:
        assert np.abs(y.mean(-1)).max() < 0.05 and np.abs(y.std(-1) - 1).max() < 0.1
    # a constant added to a row changes nothing but rounding boundaries
    q2 = O.layernorm_q(x + np.float32(shift), ones * 20, zeros, 1e-5)
    diff = np.abs(q.astype(int) - q2.astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.05
    assert q.min() >= -128 and q.max() <= 127


@SET
@given(st.integers(1, 6), st.integers(1, 300), seeds, st.floats(0.0, 2.0), st.booleans())
def test_softmax_q_rows(rows, cols, seed, scale, causal):
    g = np.random.default_rng(seed)
    x = g.integers(-128, 128, size=(rows, cols), dtype=np.int8)
    q_len = rows if (causal and rows <= cols) else 0
    p = O.softmax_q(x, scale, causal_q_len=q_len)
    assert p.min() >= 0 and p.max() <= 127
    for r in range(rows):
        lim = cols if not q_len else min(cols, r + cols - rows + 1)
        assert (p[r, lim:] == 0).all()
        # each entry is within half a step of 127 * softmax, so the row sums to 127 within lim / 2
        assert abs(int(p[r, :lim].astype(int).sum()) - 127) <= lim / 2 + 1
        # the largest score takes the largest probability; equal scores take equal probabilities
        xs = x[r, :lim]
        assert p[r, np.argmax(xs)] == p[r, :lim].max()
        order = np.argsort(xs, kind="stable")
        assert (np.diff(p[r, :lim][order].astype(int)) >= 0).all()


@SET
@given(st.lists(st.floats(-12, 12, width=32), min_size=1, max_size=200), st.floats(0.5, 40))
def test_gelu_q_identities(xs, scale):
    x = np.array(xs, np.float32)
    s = np.float32(scale)
    g = O.gelu_f32(x, np.float32(1.0))
    assert np.allclose(g - O.gelu_f32(-x, np.float32(1.0)), x, atol=2e-6 * max(1.0, np.abs(x).max()))   # gelu(x) - gelu(-x) = x
    assert (O.gelu_f32(np.zeros(3, np.float32), s) == 0).all()
    q = O.gelu_q(x, s)
    assert np.array_equal(q, np.clip(np.rint(O.gelu_f32(x, s)), -128, 127).astype(np.int8))
    order = np.argsort(x[x > 1], kind="stable")
    assert (np.diff(q[x > 1][order].astype(int)) >= 0).all()                                            # increasing right of the dip
