"""Pins the oracle's naive DFT / inverse DFT / per-frequency contraction:
the known-answer vectors the reference's cuFFT tests hold (test/FFTTest.cpp),
numpy.fft as the library routine, round trips, and the composition
IDFT(contract(DFT, DFT)) == the CPU convolution oracle for all three passes
(which pins the conjugate placement and the crop offsets).
"""
import numpy as np
import pytest

from fbcunn_amd import synth


def _variable(shape):
    """makeTestTensor(sizes): 0.1*l + 0.2*k + 0.3*j + 0.4*i, (l,k,j,i) = (batch, plane, row, col)."""
    l, k, j, i = np.meshgrid(*[np.arange(s) for s in shape], indexing="ij")
    return (0.1 * l + 0.2 * k + 0.3 * j + 0.4 * i).astype(np.float32)


def _cplx(a):
    return a[..., 0] + 1j * a[..., 1]


# ---- known answers held by test/FFTTest.cpp ---------------------------------
def test_fft_2x2_constant(oracle):                       # FFTTest.cpp:197-228
    out = _cplx(oracle.dft2d_r2c(np.ones((1, 2, 2), np.float32), 2, 2))[0]
    np.testing.assert_allclose(out, [[4, 0], [0, 0]], atol=1e-6)


def test_fft_2x2_variable(oracle):                       # FFTTest.cpp:262-298
    x = _variable((1, 1, 2, 2))[0]
    out = _cplx(oracle.dft2d_r2c(x, 2, 2))[0]
    np.testing.assert_allclose(out, [[1.4, -0.8], [-0.6, 0.0]], atol=1e-6)


def test_fft_1x2_constant_padded_to_4x2(oracle):         # FFTTest.cpp:339-376
    out = _cplx(oracle.dft2d_r2c(np.ones((1, 1, 2), np.float32), 4, 2))[0]
    np.testing.assert_allclose(out, [[2, 0], [2, 0], [2, 0], [2, 0]], atol=1e-6)


def test_fft_2x2_constant_padded_to_3x4(oracle):         # FFTTest.cpp:415-466
    out = _cplx(oracle.dft2d_r2c(np.ones((1, 2, 2), np.float32), 3, 4))[0]
    want = np.array([[4, 2 - 2j, 0],
                     [1 - 1.732051j, -0.366025 - 1.366025j, 0],
                     [1 + 1.732051j, 1.366025 + 0.366025j, 0]])
    np.testing.assert_allclose(out, want, atol=5e-5)


def test_fft_2x2_constant_padded_to_4x3_batched(oracle):  # FFTTest.cpp:468-525
    out = _cplx(oracle.dft2d_r2c(np.ones((15, 2, 2), np.float32), 4, 3))
    want = np.array([[4, 1 - 1.732051j],
                     [2 - 2j, -0.366025 - 1.366025j],
                     [0, 0],
                     [2 + 2j, 1.366025 - 0.366025j]])
    for pl in range(15):
        np.testing.assert_allclose(out[pl], want, atol=5e-5)


def test_fft_1d_4_variable_padded_to_8(oracle):          # FFTTest.cpp:637-686
    x = _variable((1, 1, 1, 4))[0]
    out = _cplx(oracle.dft2d_r2c(x, 1, 8))[0, 0]
    want = np.array([2.4, -0.565685 - 1.931371j, -0.8 + 0.8j, 0.565685 - 0.331371j, -0.8])
    np.testing.assert_allclose(out, want, atol=2e-6)


# ---- numpy.fft as the library routine ----------------------------------------
@pytest.mark.parametrize("h,w,n,pu,pl", [(5, 5, 8, 0, 0), (6, 7, 8, 1, 1), (13, 13, 16, 1, 1),
                                         (27, 27, 32, 2, 2), (3, 4, 16, 0, 2)])
def test_dft_vs_numpy(oracle, h, w, n, pu, pl):
    x = synth.uniform(61, (3, h, w))
    canvas = np.zeros((3, n, n))
    canvas[:, pu:pu + h, pl:pl + w] = x
    want = np.fft.rfft2(canvas)
    got = _cplx(oracle.dft2d_r2c(x, n, n, pu, pl))
    np.testing.assert_allclose(got, want, atol=2e-5)
    # Hermitian/central symmetry of a real signal's spectrum on the stored columns 0 and n/2
    for v in (0, n // 2):
        np.testing.assert_allclose(got[:, 1:, v], np.conj(got[:, :0:-1, v]), atol=2e-5)
    # DC bin is the plain sum
    np.testing.assert_allclose(got[:, 0, 0].real, x.astype(np.float64).sum(axis=(1, 2)), atol=2e-5)


@pytest.mark.parametrize("h,w,n,pu,pl", [(8, 8, 8, 0, 0), (5, 6, 8, 2, 1), (13, 13, 16, 1, 1)])
def test_inverse_vs_numpy_and_round_trip(oracle, h, w, n, pu, pl):
    full = synth.uniform(62, (2, n, n))
    spec = oracle.dft2d_r2c(full, n, n)
    got = oracle.idft2d_c2r(spec, h, w, n, pu, pl)
    want = np.fft.irfft2(_cplx(spec), s=(n, n)) * (n * n)      # unnormalised
    np.testing.assert_allclose(got, want[:, pu:pu + h, pl:pl + w], atol=2e-4)
    # round trip: IDFT(DFT(x)) / n^2 = x on the cropped window
    np.testing.assert_allclose(got / (n * n), full[:, pu:pu + h, pl:pl + w], atol=2e-6)


# ---- composition equals the convolution oracle (the maths of the three passes)
def _to_plane_major(spec, d0, d1):
    planes, n, nh, _ = spec.shape
    return spec.reshape(d0, d1, n * nh, 2)


@pytest.mark.parametrize("B,P,F,H,W,k,pad,n", [(2, 3, 2, 6, 6, 3, 1, 8), (1, 2, 3, 11, 9, 5, 2, 16),
                                               (2, 2, 2, 8, 8, 3, 0, 8)])
def test_frequency_pipeline_equals_convolution(oracle, B, P, F, H, W, k, pad, n):
    x = synth.uniform(71, (B, P, H, W))
    w = synth.uniform(72, (F, P, k, k))
    oH, oW = H + 2 * pad - k + 1, W + 2 * pad - k + 1
    g = synth.uniform(73, (B, F, oH, oW))
    scale = 0.5
    X = _to_plane_major(oracle.dft2d_r2c(x.reshape(B * P, H, W), n, n, pad, pad), B, P)
    Wf = _to_plane_major(oracle.dft2d_r2c(w.reshape(F * P, k, k), n, n), F, P)
    G = _to_plane_major(oracle.dft2d_r2c(g.reshape(B * F, oH, oW), n, n), B, F)
    inv = 1.0 / (n * n)

    O = oracle.freq_contract(0, X, Wf, B, P, F, inv)
    out = oracle.idft2d_c2r(O.reshape(B * F, n, n // 2 + 1, 2), oH, oW, n).reshape(B, F, oH, oW)
    np.testing.assert_allclose(out, oracle.cross_correlation_valid(x, w, (1, 1), (pad,) * 4), atol=2e-5)

    GI = oracle.freq_contract(1, G, Wf, B, P, F, inv)
    gin = oracle.idft2d_c2r(GI.reshape(B * P, n, n // 2 + 1, 2), H, W, n, pad, pad).reshape(B, P, H, W)
    np.testing.assert_allclose(gin, oracle.convolution_full(g, w, (1, 1), (pad,) * 4), atol=2e-5)

    GW = oracle.freq_contract(2, G, X, B, P, F, scale * inv)
    gw = oracle.idft2d_c2r(GW.reshape(F * P, n, n // 2 + 1, 2), k, k, n).reshape(F, P, k, k)
    np.testing.assert_allclose(
        gw, oracle.cross_correlation_reverse_valid(x, g, (1, 1), scale, (pad,) * 4), atol=5e-5)


def test_contraction_single_plane_is_pointwise(oracle):
    a = synth.uniform(81, (1, 1, 10, 2))
    b = synth.uniform(82, (1, 1, 10, 2))
    ca, cb = _cplx(a)[0, 0], _cplx(b)[0, 0]
    np.testing.assert_allclose(_cplx(oracle.freq_contract(0, a, b, 1, 1, 1, 1.0))[0, 0], ca * np.conj(cb), atol=1e-6)
    np.testing.assert_allclose(_cplx(oracle.freq_contract(1, a, b, 1, 1, 1, 1.0))[0, 0], ca * cb, atol=1e-6)
    np.testing.assert_allclose(_cplx(oracle.freq_contract(2, a, b, 1, 1, 1, 1.0))[0, 0], np.conj(ca) * cb, atol=1e-6)
