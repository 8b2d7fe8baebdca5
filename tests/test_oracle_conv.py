"""Pins oracle/refconv.c (the CPU restatement of test/ReferenceConvolutions.cpp)
without running the reference: the reference's own closed-form table and its
padded-vs-unpadded self-consistency tests, scipy's textbook routines, sliding-
window brute force, and inner-product adjoint identities.  A dropped term, a
flipped kernel, a transposed operand or a wrong pad offset fails at least one.
"""
import itertools

import numpy as np
import pytest
from scipy.signal import convolve2d, correlate2d

from fbcunn_amd import synth


def _pad(x, pt, pb, pl, pr):
    return np.pad(x, ((0, 0), (0, 0), (pt, pb), (pl, pr)))


def _scipy_fprop(x, w, stride, padding):
    xp = _pad(x, *padding).astype(np.float64)
    B, P = x.shape[:2]
    F = w.shape[0]
    outs = []
    for b in range(B):
        row = []
        for f in range(F):
            acc = sum(correlate2d(xp[b, p], w[f, p].astype(np.float64), mode="valid")
                      for p in range(P))
            row.append(acc[::stride[0], ::stride[1]])
        outs.append(row)
    return np.array(outs)


# --- reference fixture: test/ConvolutionTest.cpp:1316-1374 -------------------
def test_full_convolution_ones_table(oracle):
    """ones(7x7) fully convolved with ones(3x3) is the 9x9 '1 2 3 3 ...' table
    the reference's CuFFT_updateGradInput_fixed test spells out."""
    edge = np.array([1, 2, 3, 3, 3, 3, 3, 2, 1], np.float32)
    expected = np.outer(edge, edge)
    # spot values copied from the reference's table
    assert expected[0, 0] == 1 and expected[1, 1] == 4 and expected[4, 4] == 9
    assert expected[0, 7] == 2 and expected[3, 0] == 3 and expected[3, 1] == 6
    got = oracle.convolution_full(np.ones((1, 1, 7, 7), np.float32),
                                  np.ones((1, 1, 3, 3), np.float32))
    assert got.shape == (1, 1, 9, 9)
    np.testing.assert_array_equal(got[0, 0], expected)


# --- scipy as the textbook routine ------------------------------------------
CASES = [
    # B, P, F, H, W, kH, kW, stride, padding(t,b,l,r)
    (2, 3, 4, 8, 9, 3, 2, (1, 1), (0, 0, 0, 0)),
    (2, 2, 3, 7, 7, 3, 3, (1, 1), (1, 1, 1, 1)),
    (1, 3, 2, 9, 6, 5, 4, (1, 1), (2, 1, 0, 3)),
    (2, 2, 2, 6, 6, 4, 4, (2, 2), (0, 0, 0, 0)),
    (2, 2, 2, 6, 6, 4, 4, (2, 2), (2, 4, 0, 2)),
    (1, 1, 1, 10, 6, 4, 2, (3, 2), (0, 0, 0, 0)),
]


@pytest.mark.parametrize("case", CASES)
def test_fprop_vs_scipy(oracle, case):
    B, P, F, H, W, kH, kW, stride, padding = case
    x = synth.uniform(11, (B, P, H, W))
    w = synth.uniform(12, (F, P, kH, kW))
    got = oracle.cross_correlation_valid(x, w, stride, padding)
    want = _scipy_fprop(x, w, stride, padding)
    assert got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)


@pytest.mark.parametrize("case", CASES)
def test_bprop_vs_scipy(oracle, case):
    B, P, F, H, W, kH, kW, stride, padding = case
    pt, pb, pl, pr = padding
    oR = (H + pt + pb - kH) // stride[0] + 1
    oC = (W + pl + pr - kW) // stride[1] + 1
    g = synth.uniform(13, (B, F, oR, oC))
    w = synth.uniform(14, (F, P, kH, kW))
    got = oracle.convolution_full(g, w, stride, padding)
    assert got.shape == (B, P, H, W)
    # stride s full convolution = stride-1 full convolution of the zero-stuffed gradient
    up = np.zeros((B, F, (oR - 1) * stride[0] + 1, (oC - 1) * stride[1] + 1))
    up[:, :, ::stride[0], ::stride[1]] = g
    for b in range(B):
        for p in range(P):
            full = sum(convolve2d(up[b, f], w[f, p].astype(np.float64), mode="full")
                       for f in range(F))
            want = full[pt:pt + H, pl:pl + W]
            np.testing.assert_allclose(got[b, p], want, rtol=0, atol=2e-5)


@pytest.mark.parametrize("case", CASES)
def test_accgrad_vs_scipy(oracle, case):
    B, P, F, H, W, kH, kW, stride, padding = case
    pt, pb, pl, pr = padding
    oR = (H + pt + pb - kH) // stride[0] + 1
    oC = (W + pl + pr - kW) // stride[1] + 1
    x = synth.uniform(15, (B, P, H, W))
    g = synth.uniform(16, (B, F, oR, oC))
    scale = 0.333
    got = oracle.cross_correlation_reverse_valid(x, g, stride, scale, padding)
    assert got.shape == (F, P, kH, kW)
    xp = _pad(x, *padding).astype(np.float64)
    up = np.zeros((B, F, (oR - 1) * stride[0] + 1, (oC - 1) * stride[1] + 1))
    up[:, :, ::stride[0], ::stride[1]] = g
    for f in range(F):
        for p in range(P):
            want = scale * sum(correlate2d(xp[b, p], up[b, f], mode="valid") for b in range(B))
            np.testing.assert_allclose(got[f, p], want, rtol=0, atol=5e-5)


# --- brute force with sliding windows (a different formula shape) -------------
def test_fprop_bruteforce_windows(oracle):
    B, P, F, H, W, k, pad = 2, 3, 2, 6, 5, 3, 2
    x = synth.uniform(21, (B, P, H, W))
    w = synth.uniform(22, (F, P, k, k))
    xp = _pad(x, pad, pad, pad, pad).astype(np.float64)
    o = H + 2 * pad - k + 1, W + 2 * pad - k + 1
    want = np.zeros((B, F) + o)
    for r in range(o[0]):
        for c in range(o[1]):
            win = xp[:, :, r:r + k, c:c + k]                     # B,P,k,k
            want[:, :, r, c] = np.einsum("bpij,fpij->bf", win, w.astype(np.float64))
    got = oracle.cross_correlation_valid(x, w, (1, 1), (pad,) * 4)
    np.testing.assert_allclose(got, want, rtol=0, atol=2e-5)


def test_special_cases(oracle):
    # 1x1 kernel: a per-pixel matrix product over planes
    x = synth.uniform(31, (2, 4, 5, 5))
    w = synth.uniform(32, (3, 4, 1, 1))
    got = oracle.cross_correlation_valid(x, w)
    want = np.einsum("bphw,fp->bfhw", x.astype(np.float64), w[:, :, 0, 0].astype(np.float64))
    np.testing.assert_allclose(got, want, atol=1e-5)
    # delta kernel at (i,j): a shifted copy
    d = np.zeros((1, 1, 3, 3), np.float32)
    d[0, 0, 2, 1] = 1.0
    x = synth.uniform(33, (1, 1, 6, 6))
    got = oracle.cross_correlation_valid(x, d)
    np.testing.assert_array_equal(got[0, 0], x[0, 0, 2:6, 1:5])


# --- adjoint identities: pin bprop and accGrad against fprop ------------------
@pytest.mark.parametrize("case", CASES)
def test_adjoint_identities(oracle, case):
    B, P, F, H, W, kH, kW, stride, padding = case
    x = synth.uniform(41, (B, P, H, W))
    w = synth.uniform(42, (F, P, kH, kW))
    y = oracle.cross_correlation_valid(x, w, stride, padding)
    g = synth.uniform(43, y.shape)
    gi = oracle.convolution_full(g, w, stride, padding)
    gw = oracle.cross_correlation_reverse_valid(x, g, stride, 1.0, padding)
    lhs = np.vdot(y.astype(np.float64), g.astype(np.float64))
    assert abs(lhs - np.vdot(x.astype(np.float64), gi.astype(np.float64))) < 1e-4 * max(1, abs(lhs))
    assert abs(lhs - np.vdot(w.astype(np.float64), gw.astype(np.float64))) < 1e-4 * max(1, abs(lhs))


# --- the reference's own self-consistency test, test/ConvolutionTest.cpp:982-1089
def _linear_tensor(shape):
    """makeTestTensor(sizes): 0.1*l + 0.2*k + 0.3*j + 0.4*i (test/TestUtils.cpp:92-112)."""
    l, k, j, i = np.meshgrid(*[np.arange(s) for s in shape], indexing="ij")
    return (np.float32(0.1) * l + np.float32(0.2) * k + np.float32(0.3) * j
            + np.float32(0.4) * i).astype(np.float32)


RAP = dict(batch=2, P=2, H=6, W=6, F=2, k=4, stride=2)  # kRAPParams(2,2,6,6,2,4,2)


def _rap_cases():
    for i, j, k, l in itertools.product(range(3), repeat=4):
        for rs in (1, RAP["stride"]):
            for cs in (1, RAP["stride"]):
                yield (i * rs, j * rs, k * cs, l * cs), (rs, cs)


def test_reference_asymmetric_padding_update_output(oracle):
    x = _linear_tensor((RAP["batch"], RAP["P"], RAP["H"], RAP["W"]))
    w = _linear_tensor((RAP["F"], RAP["P"], RAP["k"], RAP["k"]))
    for pad, (rs, cs) in _rap_cases():
        base = oracle.cross_correlation_valid(x, w, (rs, cs))
        padded = oracle.cross_correlation_valid(x, w, (rs, cs), pad)
        t, b, l, r = pad[0] // rs, pad[1] // rs, pad[2] // cs, pad[3] // cs
        narrowed = padded[:, :, t:padded.shape[2] - b, l:padded.shape[3] - r]
        np.testing.assert_array_equal(narrowed, base)
        # and the padded border equals the convolution of an explicitly padded input
        np.testing.assert_allclose(
            padded, oracle.cross_correlation_valid(_pad(x, *pad), w, (rs, cs)), atol=1e-5)


def test_reference_asymmetric_padding_update_grad_input(oracle):
    w = _linear_tensor((RAP["F"], RAP["P"], RAP["k"], RAP["k"]))
    for pad, (rs, cs) in _rap_cases():
        oR = (RAP["H"] - RAP["k"]) // rs + 1
        oC = (RAP["W"] - RAP["k"]) // cs + 1
        g = _linear_tensor((RAP["batch"], RAP["F"], oR, oC))
        base = oracle.convolution_full(g, w, (rs, cs))
        gp = _pad(g, pad[0] // rs, pad[1] // rs, pad[2] // cs, pad[3] // cs)
        got = oracle.convolution_full(gp, w, (rs, cs), pad)
        np.testing.assert_allclose(got, base, rtol=1e-5, atol=1e-5)


def test_reference_asymmetric_padding_acc_grad(oracle):
    x = _linear_tensor((RAP["batch"], RAP["P"], RAP["H"], RAP["W"]))
    for pad, (rs, cs) in _rap_cases():
        oR = (RAP["H"] - RAP["k"]) // rs + 1
        oC = (RAP["W"] - RAP["k"]) // cs + 1
        g = _linear_tensor((RAP["batch"], RAP["F"], oR, oC))
        base = oracle.cross_correlation_reverse_valid(x, g, (rs, cs), 0.333)
        gp = _pad(g, pad[0] // rs, pad[1] // rs, pad[2] // cs, pad[3] // cs)
        got = oracle.cross_correlation_reverse_valid(x, gp, (rs, cs), 0.333, pad)
        np.testing.assert_allclose(got, base, rtol=1e-5, atol=1e-5)


# --- argument errors the reference throws ------------------------------------
def test_argument_errors(oracle):
    x = np.zeros((1, 2, 4, 4), np.float32)
    with pytest.raises(ValueError):
        oracle.cross_correlation_valid(x, np.zeros((1, 3, 2, 2), np.float32))   # planes mismatch
    with pytest.raises(ValueError):
        oracle.cross_correlation_valid(x, np.zeros((1, 2, 5, 5), np.float32))   # filter > input
    with pytest.raises(ValueError):
        oracle.cross_correlation_valid(x, np.zeros((1, 2, 3, 3), np.float32), (2, 2))  # illegal stride
    with pytest.raises(ValueError):
        oracle.cross_correlation_valid(x, np.zeros((1, 2, 2, 2), np.float32), (0, 1))


# --- bias loops, test/BiasTest.cpp:83-130 ------------------------------------
def test_bias_loops(oracle):
    g = synth.uniform(51, (3, 4, 5, 6))
    bias = np.arange(4, dtype=np.float32)           # makeBiasTensor: bias[i] = i
    out = oracle.bias_update_output(g, bias)
    np.testing.assert_array_equal(out, g + bias[None, :, None, None])
    gb = oracle.bias_acc_grad_parameters(g, 0.5)
    np.testing.assert_allclose(gb, 0.5 * g.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-5)
    # assignment, not accumulation: a second call gives the same values
    np.testing.assert_array_equal(gb, oracle.bias_acc_grad_parameters(g, 0.5))


def test_is_within_semantics(oracle):
    assert oracle.is_within(1.0, 1.0, 1e-5)
    assert oracle.is_within(float("nan"), float("nan"), 1e-5)
    assert oracle.is_within(float("inf"), float("inf"), 1e-5)
    assert not oracle.is_within(float("inf"), float("-inf"), 1e-5)
    assert oracle.is_within(1.0, 1.0 + 0.9e-5, 1e-5)        # |a-b| <= 0.5*rel*(|a|+|b|)
    assert not oracle.is_within(1.0, 1.0 + 1.2e-5, 1e-5)
    assert oracle.is_within(0.0, 4e-6, 1e-5)                # near zero: absolute 0.5*rel
    assert not oracle.is_within(0.0, 6e-6, 1e-5)


# --- regression fixture for the CPU-runnable configuration --------------------
def test_config1_fixture(oracle):
    """batch 4, 16 -> 16 planes, 32x32, 5x5, no padding, seed 1001 (written by
    tests/golden/make_config1.py from this oracle: guards against drift and
    differing float summation order across machines and compilers)."""
    import os
    ref = np.load(os.path.join(os.path.dirname(__file__), "golden", "config1_fprop.npy"))
    x = synth.uniform(1001, (4, 16, 32, 32), stream=0)
    w = synth.uniform(1001, (16, 16, 5, 5), stream=1)
    got = oracle.cross_correlation_valid(x, w)
    assert got.shape == (4, 16, 28, 28)
    np.testing.assert_array_equal(got, ref)
