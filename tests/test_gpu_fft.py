"""GPU parity of the batched 2-D real<->complex FFT kernels, called through the
C ABI (fbfc_fft2d / fbfc_ifft2d via nn.FFTWrapper), against the oracle's naive
DFT on sampled planes and numpy.fft on all planes (the oracle's DFT is itself
pinned against numpy.fft and the reference's cuFFT vectors in
tests/test_oracle_fft.py).

Tolerance: |err| <= 5e-6 * max|expected| (the reference compares fbfft with cuFFT
at 4e-7 * max per element for sizes up to 128, test/test_FFTModule.lua:13; the
sums here have up to 4096 float32 terms).
"""
import numpy as np
import pytest
import torch

from fbcunn_amd import synth
from gpu_util import dev, freq_major_to_planes, host, planes_to_freq_major

pytestmark = pytest.mark.gpu
TOL = 5e-6


@pytest.fixture(scope="module")
def nn():
    from fbcunn_amd import nn as mod
    return mod


CASES = [
    # N, planes, h, w, padU, padL
    (2, 300, 2, 2, 0, 0), (2, 5, 1, 2, 1, 0), (4, 300, 4, 4, 0, 0), (4, 7, 3, 2, 1, 2),   # one lane per plane
    (8, 5, 8, 8, 0, 0), (8, 130, 3, 3, 0, 0), (8, 64, 5, 6, 2, 1),
    (16, 7, 13, 13, 1, 1), (16, 96, 16, 16, 0, 0), (16, 33, 3, 3, 0, 0), (16, 40, 10, 12, 3, 2),
    (32, 3, 27, 27, 2, 2), (32, 48, 32, 32, 0, 0), (32, 17, 5, 5, 0, 0), (32, 35, 20, 28, 5, 1),
    (64, 9, 55, 55, 4, 4), (64, 16, 64, 64, 0, 0), (64, 5, 9, 9, 0, 0), (64, 11, 33, 40, 7, 10),
    (64, 19, 16, 16, 0, 0), (64, 3, 1, 16, 0, 0), (64, 8, 11, 2, 0, 0), (64, 4, 9, 9, 1, 0),   # small planes: zero inputs skipped
    (64, 37, 47, 47, 0, 0), (64, 50, 21, 35, 3, 5), (64, 41, 9, 9, 0, 0), (32, 70, 27, 27, 2, 2), (16, 200, 13, 13, 1, 1),   # several workgroups, ragged last one
    (64, 23, 63, 63, 1, 1), (64, 18, 1, 63, 63, 0), (32, 19, 31, 1, 0, 31),   # planes that touch the canvas border
    (128, 5, 100, 100, 3, 7), (128, 9, 128, 128, 0, 0), (128, 6, 11, 11, 0, 0), (128, 3, 70, 127, 20, 1),
]


def _canvas(x, n, pu, pl):
    c = np.zeros((x.shape[0], n, n))
    c[:, pu:pu + x.shape[1], pl:pl + x.shape[2]] = x
    return c


@pytest.mark.parametrize("n,planes,h,w,pu,pl", CASES)
def test_forward_matches_dft(nn, oracle, n, planes, h, w, pu, pl):
    x = synth.uniform(100 + n, (planes, h, w))
    freq = torch.full((n, n // 2 + 1, planes, 2), float("nan"), device="cuda")
    nn.FFTWrapper("fbfft", pl, pu).fft(dev(x), freq)
    got = freq_major_to_planes(host(freq))
    want = np.fft.rfft2(_canvas(x, n, pu, pl))
    scale = np.abs(want).max()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * scale
    # oracle's naive DFT on a few planes (first, last = ragged tail of the last workgroup)
    pick = sorted({0, planes // 2, planes - 1})
    o = oracle.dft2d_r2c(x[pick], n, n, pu, pl)
    oc = o[..., 0] + 1j * o[..., 1]
    assert np.abs(got[pick] - oc).max() <= TOL * scale
    # columns 0 and N/2 of a real signal's spectrum are Hermitian in the row frequency
    for v in (0, n // 2):
        assert np.abs(got[:, 1:, v] - np.conj(got[:, :0:-1, v])).max() <= TOL * scale


@pytest.mark.parametrize("n,planes,h,w,pu,pl", CASES)
def test_inverse_matches_idft(nn, oracle, n, planes, h, w, pu, pl):
    full = synth.uniform(200 + n, (planes, n, n))
    spec = np.fft.rfft2(full.astype(np.float64))
    freq = dev(planes_to_freq_major(spec))
    out = torch.full((planes, h, w), float("nan"), device="cuda")
    nn.FFTWrapper("fbfft", pl, pu).ffti(out, freq)
    got = host(out)
    want = full[:, pu:pu + h, pl:pl + w].astype(np.float64) * (n * n)   # unnormalised inverse
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * np.abs(want).max() * 4
    pick = sorted({0, planes - 1})
    sp32 = np.stack([spec.real, spec.imag], -1).astype(np.float32)[pick]
    o = oracle.idft2d_c2r(sp32, h, w, n, pu, pl)
    assert np.abs(got[pick] - o).max() <= TOL * np.abs(want).max() * 4


def test_inverse_n32_many_planes(nn):
    """More than two rounds of workgroups: the N = 32 inverse switches to its two-phase variant."""
    n, distinct, reps, h, w, pu, pl = 32, 129, 130, 27, 25, 2, 3
    full = synth.uniform(77, (distinct, n, n))
    spec = np.tile(np.fft.rfft2(full.astype(np.float64)), (reps, 1, 1))
    planes = distinct * reps
    out = torch.full((planes, h, w), float("nan"), device="cuda")
    nn.FFTWrapper("fbfft", pl, pu).ffti(out, dev(planes_to_freq_major(spec)))
    got = host(out)
    want = np.tile(full[:, pu:pu + h, pl:pl + w].astype(np.float64) * (n * n), (reps, 1, 1))
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * np.abs(want).max() * 4


def test_inverse_adds_bias_per_plane(nn):
    n, B, F, h = 16, 3, 5, 13
    full = synth.uniform(31, (B * F, n, n))
    freq = dev(planes_to_freq_major(np.fft.rfft2(full.astype(np.float64))))
    bias = synth.uniform(32, (F,), -0.1, 0.1)
    plain = torch.empty((B * F, h, h), device="cuda")
    biased = torch.empty((B * F, h, h), device="cuda")
    w = nn.FFTWrapper("fbfft")
    w.ffti(plain, freq)
    w.ffti(biased, freq, bias=dev(bias))
    want = host(plain).reshape(B, F, h, h) + bias[None, :, None, None]
    np.testing.assert_allclose(host(biased).reshape(B, F, h, h), want, rtol=0, atol=1e-4)


def test_linearity_and_shift(nn):
    """FFT(a x + b y) = a FFT(x) + b FFT(y); moving the plane by (padU, padL)
    multiplies the spectrum by the shift phase."""
    n, planes, h = 32, 20, 20
    x, y = synth.uniform(41, (planes, h, h)), synth.uniform(42, (planes, h, h))
    f = lambda a, pu=0, pl=0: host(nn.FFTWrapper("fbfft", pl, pu).fft(
        dev(a), torch.empty((n, n // 2 + 1, planes, 2), device="cuda")))
    fx, fy, fz = f(x), f(y), f((2 * x - 3 * y).astype(np.float32))
    scale = np.abs(fz).max()
    assert np.abs(fz - (2 * fx - 3 * fy)).max() <= 1e-5 * scale
    pu, pl = 5, 9
    shifted = freq_major_to_planes(f(x, pu, pl))
    ky = np.arange(n)[:, None]
    kx = np.arange(n // 2 + 1)[None, :]
    phase = np.exp(-2j * np.pi * (ky * pu + kx * pl) / n)
    assert np.abs(shifted - freq_major_to_planes(fx) * phase).max() <= 1e-5 * scale


def test_config2_round_trip_8192_planes(nn, oracle):
    """8192 planes of 32x32: IFFT(FFT(x)) / 1024 reproduces x, and the forward
    transform matches the naive DFT on 64 sampled planes."""
    n, planes = 32, 8192
    x = synth.uniform(1002, (planes, n, n))
    xd = dev(x)
    freq = torch.empty((n, n // 2 + 1, planes, 2), device="cuda")
    back = torch.empty((planes, n, n), device="cuda")
    w = nn.FFTWrapper("fbfft")
    w.fft(xd, freq)
    w.ffti(back, freq)
    err = float((back / (n * n) - xd).abs().max())
    assert err <= 1e-5 * float(np.abs(x).max())
    pick = np.linspace(0, planes - 1, 64).astype(int)
    got = host(freq[:, :, torch.from_numpy(pick).cuda(), :])
    got = freq_major_to_planes(got)
    o = oracle.dft2d_r2c(x[pick], n, n)
    oc = o[..., 0] + 1j * o[..., 1]
    assert np.abs(got - oc).max() <= TOL * np.abs(oc).max()


def test_fft_argument_errors(nn):
    x = torch.zeros((4, 20, 20), device="cuda")
    with pytest.raises(nn.FbfcError) as e:          # plane + pad does not fit
        nn.FFTWrapper("fbfft", 0, 15).fft(x, torch.empty((32, 17, 4, 2), device="cuda"))
    assert "fit" in e.value.message
    with pytest.raises(nn.FbfcError) as e:          # unsupported size, like fbfft's error code
        nn.FFTWrapper("fbfft").fft(x, torch.empty((24, 13, 4, 2), device="cuda"))
    assert e.value.code == 2


# One transform dimension: the sizes and batch sizes of the reference's module test
# (test/test_FFTModule.lua:170-193), plus padded rows.
CASES_1D = [(n, rows, n, 0) for n in (2, 4, 8, 16, 32, 64, 128) for rows in (1, 127, 437)] + \
           [(8, 33, 5, 2), (32, 1000, 27, 3), (128, 64, 100, 28), (16, 2, 1, 15)] + \
           [(8, 5000, 4, 4), (16, 100001, 12, 4), (32, 70000, 32, 0), (32, 513, 31, 1), (64, 33333, 64, 0),
            (64, 300, 60, 4), (64, 129, 62, 1), (128, 10001, 128, 0), (128, 129, 3, 125), (128, 65, 64, 64)]


@pytest.mark.parametrize("n,rows,m,pl", CASES_1D)
def test_1d_forward_and_inverse(nn, oracle, n, rows, m, pl):
    x = synth.uniform(300 + n + rows, (rows, m))
    canvas = np.zeros((rows, n))
    canvas[:, pl:pl + m] = x
    want = np.fft.rfft(canvas)
    freq = torch.full((rows, n // 2 + 1, 2), float("nan"), device="cuda")
    w = nn.FFTWrapper("fbfft", pl, 0)
    w.fft(dev(x), freq)
    # sizes from 32 on run a row over 2, 4 or 8 lanes with cross-lane butterflies
    assert ("rfft1d_split_kernel" in w.lastKernel()) == (n >= 32)
    got = host(freq)
    got = got[..., 0] + 1j * got[..., 1]
    scale = max(np.abs(want).max(), 1e-30)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * scale
    # the oracle's naive DFT of the rows as 1 x n planes
    pick = sorted({0, rows - 1})
    o = oracle.dft2d_r2c(x[pick].reshape(len(pick), 1, m), 1, n, 0, pl)
    assert np.abs(got[pick] - (o[..., 0] + 1j * o[..., 1]).reshape(len(pick), -1)).max() <= TOL * scale
    # unnormalised inverse of an arbitrary real row's spectrum, read back at the padding offset
    full = synth.uniform(400 + n + rows, (rows, n))
    spec = np.fft.rfft(full.astype(np.float64))
    fr = dev(np.stack([spec.real, spec.imag], -1).astype(np.float32))
    out = torch.full((rows, m), float("nan"), device="cuda")
    w.ffti(out, fr)
    back = host(out)
    wantb = full[:, pl:pl + m].astype(np.float64) * n
    assert np.isfinite(back).all()
    assert np.abs(back - wantb).max() <= 4 * TOL * np.abs(wantb).max()


@pytest.mark.parametrize("n", [8, 32, 64, 128])
def test_1d_rows_that_do_not_start_on_16_bytes(nn, n):
    """Row lengths that are multiples of four floats take 16-byte pieces only if the tensor itself starts on
    a 16-byte boundary; a view one float into a buffer takes the 4-byte path and gives the same numbers."""
    rows = 777
    x = synth.uniform(500 + n, (rows, n))
    buf = torch.zeros(rows * n + 1, device="cuda")
    buf[1:] = dev(x).reshape(-1)
    view = buf[1:].view(rows, n)
    assert view.data_ptr() % 16 == 4
    w = nn.FFTWrapper("fbfft")
    fa = torch.empty((rows, n // 2 + 1, 2), device="cuda")
    fb = torch.empty_like(fa)
    w.fft(dev(x), fa)
    w.fft(view, fb)
    assert torch.equal(fa, fb)
    want = np.fft.rfft(x.astype(np.float64))
    got = host(fa)
    assert np.abs(got[..., 0] + 1j * got[..., 1] - want).max() <= TOL * np.abs(want).max()
    out_a = torch.empty((rows, n), device="cuda")
    out_buf = torch.full((rows * n + 1,), float("nan"), device="cuda")
    w.ffti(out_a, fa)
    w.ffti(out_buf[1:].view(rows, n), fa)
    assert torch.equal(out_a.reshape(-1), out_buf[1:])
    assert torch.isnan(out_buf[0])
    assert np.abs(host(out_a) / n - x).max() <= 1e-5 * np.abs(x).max()
    # spectra that start 8 bytes into a buffer are read one complex number at a time, not two
    fbuf = torch.zeros(fa.numel() + 2, device="cuda")
    fbuf[2:] = fa.reshape(-1)
    fview = fbuf[2:].view(rows, n // 2 + 1, 2)
    assert fview.data_ptr() % 16 == 8
    out_c = torch.empty((rows, n), device="cuda")
    w.ffti(out_c, fview)
    assert torch.equal(out_a, out_c)
    w.ffti(out_buf[1:].view(rows, n), fview)
    assert torch.equal(out_a.reshape(-1), out_buf[1:])


def test_1d_round_trip_and_timed_mode(nn):
    n, rows = 64, 4096
    x = synth.uniform(77, (rows, n))
    freq = torch.empty((rows, n // 2 + 1, 2), device="cuda")
    back = torch.empty((rows, n), device="cuda")
    w = nn.FFTWrapper("fbfft", 0, 0, "timed")
    w.fft(dev(x), freq)
    assert w.lastTiming["ms"] > 0 and w.lastTiming["GNlogN/s"] > 0
    w.ffti(back, freq)
    assert np.abs(host(back) / n - x).max() <= 1e-5 * np.abs(x).max()


def test_1d_errors(nn):
    from fbcunn_amd._lib import FbfcError, ERR_UNSUPPORTED_SIZE, ERR_INVALID_ARGUMENT
    w = nn.FFTWrapper("fbfft")
    with pytest.raises(FbfcError) as e:
        w.fft(torch.zeros(3, 256, device="cuda"), torch.zeros(3, 129, 2, device="cuda"))
    assert e.value.code == ERR_UNSUPPORTED_SIZE
    with pytest.raises(FbfcError) as e:
        nn.FFTWrapper("fbfft", 5, 0).fft(torch.zeros(3, 6, device="cuda"), torch.zeros(3, 5, 2, device="cuda"))
    assert e.value.code == ERR_INVALID_ARGUMENT


def test_plane_count_beyond_the_32_bit_row_offsets_is_refused(nn):
    """The kernels address one frequency row with 32-bit offsets: a plane count whose row would pass
    2 GiB is refused before anything is launched (no buffer of that size is touched)."""
    from fbcunn_amd._lib import FbfcError, lib
    import ctypes
    small = torch.zeros(1024, device="cuda")
    planes = (1 << 31) // (5 * 8) + 1          # N = 8: (N/2+1) * planes * 8 bytes >= 2^31
    rc = lib().fbfc_fft2d(ctypes.c_void_p(small.data_ptr()), planes, 1, 1, 0, 0, 8,
                          ctypes.c_void_p(small.data_ptr()), ctypes.c_void_p(0))
    assert rc != 0 and b"invalid" in lib().fbfc_last_error().lower()
    rc = lib().fbfc_ifft2d(ctypes.c_void_p(small.data_ptr()), planes, 1, 1, 0, 0, 8,
                           ctypes.c_void_p(small.data_ptr()), ctypes.c_void_p(0), 1, ctypes.c_void_p(0))
    assert rc != 0
    torch.cuda.synchronize()


# ---- the reference's own buffer layout (nn.FFTWrapper level) -------------------------------------
def _reference_layout(full, n):
    """complex (planes, N, N) full spectrum X[ky][kx] -> the (planes, N/2+1, N) buffer fbfft leaves:
    buf[a][c] = X[ky = a][kx = c] for 8 <= N <= 32, buf[a][c] = X[ky = c][kx = a] otherwise
    (test/test_FFTModule.lua:238-241, 267-269)."""
    if 8 <= n <= 32:
        return full[:, :n // 2 + 1, :]
    return np.transpose(full, (0, 2, 1))[:, :n // 2 + 1, :]


PLANES_CASES = [(4, 7, 3, 2, 1, 2), (8, 33, 5, 6, 2, 1), (16, 200, 13, 13, 1, 1), (32, 70, 27, 27, 2, 2),
                (32, 48, 32, 32, 0, 0), (64, 37, 55, 55, 4, 4), (64, 41, 9, 9, 0, 0), (128, 5, 100, 100, 3, 7)]


@pytest.mark.parametrize("n,planes,h,w,pu,pl", PLANES_CASES)
def test_forward_in_the_reference_layout(nn, oracle, n, planes, h, w, pu, pl):
    x = synth.uniform(300 + n, (planes, h, w))
    freq = torch.full((planes, n // 2 + 1, n, 2), float("nan"), device="cuda")
    nn.FFTWrapper("fbfft", pl, pu, layout="planes").fft(dev(x), freq)
    got = host(freq)
    got = got[..., 0] + 1j * got[..., 1]
    full = np.fft.fft2(_canvas(x, n, pu, pl))
    want = _reference_layout(full, n)
    scale = np.abs(want).max()
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * scale
    # the oracle's naive DFT gives X[ky][kx <= N/2]; the other half follows from X[-ky][-kx] = conj X[ky][kx]
    pick = sorted({0, planes - 1})
    o = oracle.dft2d_r2c(x[pick], n, n, pu, pl)
    half = o[..., 0] + 1j * o[..., 1]                       # (len(pick), N, N/2+1)
    fullo = np.zeros((len(pick), n, n), complex)
    fullo[:, :, :n // 2 + 1] = half
    for kx in range(n // 2 + 1, n):
        fullo[:, :, kx] = np.conj(half[:, (-np.arange(n)) % n, n - kx])
    assert np.abs(got[pick] - _reference_layout(fullo, n)).max() <= TOL * scale


@pytest.mark.parametrize("n,planes,h,w,pu,pl", PLANES_CASES)
def test_inverse_in_the_reference_layout(nn, n, planes, h, w, pu, pl):
    full = synth.uniform(400 + n, (planes, n, n))
    spec = _reference_layout(np.fft.fft2(full.astype(np.float64)), n)
    buf = dev(np.stack([spec.real, spec.imag], -1).astype(np.float32))
    out = torch.full((planes, h, w), float("nan"), device="cuda")
    nn.FFTWrapper("fbfft", pl, pu, layout="planes").ffti(out, buf)
    want = full[:, pu:pu + h, pl:pl + w].astype(np.float64) * (n * n)
    got = host(out)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * np.abs(want).max() * 4


def test_round_trip_in_the_reference_layout(nn):
    """fft then ffti / N^2 on (batch, planes, N, N) tensors with two batch dimensions, as
    test/test_FFTModule.lua:247-262 runs it."""
    n = 32
    x = synth.uniform(55, (3, 5, n, n))
    xd = dev(x)
    freq = torch.empty((3, 5, n // 2 + 1, n, 2), device="cuda")
    w = nn.FFTWrapper("fbfft", layout="planes")
    w.fft(xd, freq, 2)
    back = torch.empty_like(xd)
    w.ffti(back, freq, 2)
    assert np.abs(host(back) / (n * n) - x).max() <= 1e-5 * np.abs(x).max()


@pytest.mark.parametrize("n,planes", [(8, 40), (16, 70), (32, 33), (64, 21), (64, 9), (128, 5)])
def test_inverse_takes_its_input_as_the_spectrum_of_a_real_plane(nn, n, planes):
    """What the header documents for a buffer that is not exactly Hermitian (rounding breaks the symmetry of
    a product of spectra): the entries (ky > N/2, kx in {0, N/2}) are not read -- garbage there, NaN included,
    leaves every output bit unchanged, in the frequency-major and in the reference's plane-major layout --
    and every other entry is used as given: an imaginary part eps in the four self-conjugate entries moves
    the result by at most 4 eps (the transform is linear and unnormalised), it is not filtered out."""
    h = w = n - 3
    x = synth.uniform(700 + n, (planes, n, n))
    spec = np.fft.rfft2(x.astype(np.float64))                    # (planes, N, N/2+1): X[ky][kx]
    clean = planes_to_freq_major(spec)
    dirty = clean.copy()                                          # (N, N/2+1, planes, 2)
    for kx in (0, n // 2):
        dirty[n // 2 + 1:, kx] = np.nan
    eps = 1e-2
    tilted = clean.copy()
    for kx in (0, n // 2):
        for ky in (0, n // 2):
            tilted[ky, kx, :, 1] = eps
    outs = []
    for buf in (clean, dirty, tilted):
        out = torch.full((planes, h, w), float("nan"), device="cuda")
        nn.FFTWrapper("fbfft", 1, 2).ffti(out, dev(buf))
        outs.append(host(out))
    assert np.isfinite(outs[0]).all()
    assert np.array_equal(outs[0], outs[1])
    want = x[:, 2:2 + h, 1:1 + w].astype(np.float64) * (n * n)
    assert np.abs(outs[0] - want).max() <= TOL * np.abs(want).max() * 4
    assert np.isfinite(outs[2]).all()
    assert np.abs(outs[2] - outs[0]).max() <= 4 * eps * 1.01 + TOL * np.abs(want).max()
    # plane-major: the same entries of X, wherever the reference's half plane keeps them
    full = np.fft.fft2(x.astype(np.float64))
    ref_clean = _reference_layout(full, n)
    ref_dirty = ref_clean.copy()
    bad = np.zeros((n, n), bool)                                  # [ky][kx] entries that are not used
    for kx in (0, n // 2):
        bad[n // 2 + 1:, kx] = True
    bad_ref = _reference_layout(np.broadcast_to(bad, (1, n, n)), n)[0]
    ref_dirty[:, bad_ref] = np.nan
    outs = []
    for spec_ref in (ref_clean, ref_dirty):
        buf = dev(np.stack([spec_ref.real, spec_ref.imag], -1).astype(np.float32))
        out = torch.full((planes, h, w), float("nan"), device="cuda")
        nn.FFTWrapper("fbfft", 1, 2, layout="planes").ffti(out, buf)
        outs.append(host(out))
    assert np.isfinite(outs[0]).all()
    assert np.array_equal(outs[0], outs[1])


def test_tiny_transforms_log_their_launch(nn):
    w = nn.FFTWrapper("fbfft")
    for n in (2, 4):
        x = dev(synth.uniform(n, (300, n, n)))
        freq = torch.empty((n, n // 2 + 1, 300, 2), device="cuda")
        w.fft(x, freq)
        assert w.lastKernel().startswith("rfft2d_tiny_kernel<%d> grid=" % n)
        w.ffti(x, freq)
        assert w.lastKernel().startswith("irfft2d_tiny_kernel<%d> grid=" % n)
