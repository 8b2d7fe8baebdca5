"""GPU parity of the per-frequency complex contraction (fbfc_transpose_mm, the
replacement of transposeMMFFI) against the oracle's frequency-domain triple loop
and numpy einsum, for the three conjugation modes the reference uses, ragged
sizes and the accumulate flag.  Tolerance 2e-5 * max|expected| (float32 MFMA
accumulation of up to 256 products)."""
import numpy as np
import pytest
import torch

from fbcunn_amd import synth
from gpu_util import dev, host

pytestmark = pytest.mark.gpu
TOL = 2e-5


@pytest.fixture(scope="module")
def nn():
    from fbcunn_amd import nn as mod
    return mod


def _c(a):
    return a[..., 0].astype(np.float64) + 1j * a[..., 1].astype(np.float64)


SHAPES = [  # Q, m, n, k
    (5, 64, 64, 16), (3, 128, 64, 64), (4, 32, 32, 32), (7, 1, 1, 1), (6, 3, 5, 7),
    (2, 65, 33, 17), (3, 70, 130, 40), (2, 64, 256, 96), (9, 16, 16, 4), (2, 100, 20, 129),
    # small aligned problems take the split-K kernel (M, N multiples of 32, K of 64)
    (4, 32, 32, 64), (2, 96, 160, 128), (3, 128, 128, 128), (5, 64, 32, 192), (144, 128, 128, 128),
    # a few rounds of 64x64 tiles with a ragged last one: whole rounds as LDS-direct tiles, the
    # left-over frequencies as split blocks, in one launch
    (70, 128, 128, 64), (300, 64, 64, 128), (33, 192, 128, 64),
    # ragged M or N with K a multiple of 16: the register-fed kernel with its edge lanes masked
    (130, 16, 128, 128), (7, 128, 3, 64), (9, 3, 5, 16), (40, 100, 120, 64), (5, 33, 31, 32), (3, 1, 1, 16), (11, 70, 130, 48),
    # one to four rounds of tiles whose last round is more than half full (or full): whole tiles throughout
    (60, 128, 256, 128), (130, 128, 128, 32), (64, 128, 128, 128),
    # N a multiple of 96 but not of 64 and at least 1024 64x96 blocks: 64x32 tiles by two waves
    (1024, 64, 96, 16), (260, 128, 288, 32), (1100, 64, 96, 48),
]


@pytest.mark.parametrize("Q,m,n,k", SHAPES)
@pytest.mark.parametrize("mode", ["fprop", "bprop", "accgrad"])
def test_transpose_mm(nn, mode, Q, m, n, k):
    ca, cb = (mode == "accgrad"), (mode == "fprop")
    A = synth.uniform(1, (Q, k, m, 2) if ca else (Q, m, k, 2))
    B = synth.uniform(2, (Q, n, k, 2) if cb else (Q, k, n, 2))
    C = torch.full((Q, m, n, 2), float("nan"), device="cuda")
    nn.transposeMM(dev(A), dev(B), C, 0.25, ca, cb, False)
    got = _c(host(C))
    a, b = _c(A), _c(B)
    if mode == "fprop":
        want = 0.25 * np.einsum("qmk,qnk->qmn", a, np.conj(b))
    elif mode == "bprop":
        want = 0.25 * np.einsum("qmk,qkn->qmn", a, b)
    else:
        want = 0.25 * np.einsum("qkm,qkn->qmn", np.conj(a), b)
    assert np.isfinite(got).all()
    assert np.abs(got - want).max() <= TOL * np.abs(want).max()


@pytest.mark.parametrize("Q,m,n,k", [(3, 40, 50, 20), (3, 64, 96, 64), (70, 128, 128, 64)])
def test_accumulate_flag(nn, Q, m, n, k):
    A, B = synth.uniform(3, (Q, m, k, 2)), synth.uniform(4, (Q, k, n, 2))
    C0 = synth.uniform(5, (Q, m, n, 2))
    C = dev(C0)
    nn.transposeMM(dev(A), dev(B), C, 1.0, False, False, True)
    want = _c(C0) + np.einsum("qmk,qkn->qmn", _c(A), _c(B))
    assert np.abs(_c(host(C)) - want).max() <= TOL * np.abs(want).max()


@pytest.mark.parametrize("pass_", [0, 1, 2])
def test_against_oracle_contraction(nn, oracle, pass_):
    """Same numbers as the oracle's restatement of the reference's one-thread
    frequency-domain kernels, after moving from plane-major to frequency-major."""
    nB, nP, nF, Q = 6, 5, 4, 12
    to_fm = lambda x: np.ascontiguousarray(np.transpose(x, (2, 0, 1, 3)))   # (d0,d1,Q,2) -> (Q,d0,d1,2)
    I = synth.uniform(6, (nB, nP, Q, 2))
    W = synth.uniform(7, (nF, nP, Q, 2))
    G = synth.uniform(8, (nB, nF, Q, 2))
    alpha = 1.0 / 64
    if pass_ == 0:
        want = oracle.freq_contract(0, I, W, nB, nP, nF, alpha)
        C = torch.empty((Q, nB, nF, 2), device="cuda")
        nn.transposeMM(dev(to_fm(I)), dev(to_fm(W)), C, alpha, False, True, False)
    elif pass_ == 1:
        want = oracle.freq_contract(1, G, W, nB, nP, nF, alpha)
        C = torch.empty((Q, nB, nP, 2), device="cuda")
        nn.transposeMM(dev(to_fm(G)), dev(to_fm(W)), C, alpha, False, False, False)
    else:
        want = oracle.freq_contract(2, G, I, nB, nP, nF, alpha)
        C = torch.empty((Q, nF, nP, 2), device="cuda")
        nn.transposeMM(dev(to_fm(G)), dev(to_fm(I)), C, alpha, True, False, False)
    got = np.transpose(host(C), (1, 2, 0, 3))
    assert np.abs(got - want).max() <= TOL * np.abs(want).max()


@pytest.mark.parametrize("shape,kernel", [((3, 128, 128, 128), "cgemm_splitk_kernel"), ((70, 128, 128, 64), "cgemm_hybrid_kernel"),
                                          ((300, 64, 64, 128), "cgemm_hybrid_kernel"), ((60, 128, 256, 128), "cgemm_ldsdirect_kernel"),
                                          ((130, 128, 128, 32), "cgemm_ldsdirect_kernel"), ((64, 128, 128, 128), "cgemm_ldsdirect_kernel"),
                                          ((300, 128, 128, 64), "cgemm_ldsdirect_kernel"), ((6, 3, 5, 7), "cgemm_freq_kernel"),
                                          ((130, 16, 128, 128), "cgemm_splitk_kernel"), ((130, 128, 3, 128), "cgemm_splitk_kernel"),
                                          ((2112, 64, 250, 96), "cgemm_freq_kernel")])
def test_which_kernel_a_shape_takes(nn, shape, kernel):
    """The shape rule of the contraction: few tiles -> register-fed blocks with K shared by the waves; a few rounds
    of tiles with a thin last round -> tiles plus split blocks in one launch; otherwise whole tiles; ragged sizes ->
    the bounds-checked kernel."""
    from fbcunn_amd import _lib
    Q, m, n, k = shape
    A = torch.zeros((Q, m, k, 2), device="cuda")
    B = torch.zeros((Q, n, k, 2), device="cuda")
    C = torch.empty((Q, m, n, 2), device="cuda")
    nn.transposeMM(A, B, C, 1.0, False, True, False)
    assert _lib.lib().fbfc_last_launch().decode().startswith(kernel)


def test_both_conjugations_rejected(nn):
    t = torch.zeros((1, 2, 2, 2), device="cuda")
    with pytest.raises(nn.FbfcError) as e:
        nn.transposeMM(t, t, t.clone(), 1.0, True, True, False)
    assert e.value.code == 3


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_transpose_mm_on_the_reference_operand_layout(nn, mode):
    """src/MM.cu:14-24, 54-73: operands are (d0, d1, N/2+1, N, 2) buffers, plane-major."""
    f1, f2, m, n, k = 9, 16, 20, 12, 7
    rng = np.random.RandomState(5 + mode)
    cplx = lambda *shape: rng.uniform(-1, 1, shape) + 1j * rng.uniform(-1, 1, shape)
    conj_a, conj_b = mode == 2, mode == 0
    A = cplx(k, m, f1, f2) if conj_a else cplx(m, k, f1, f2)
    B = cplx(n, k, f1, f2) if conj_b else cplx(k, n, f1, f2)
    C0 = cplx(m, n, f1, f2)
    if mode == 0:
        want = np.einsum("mkxy,nkxy->mnxy", A, np.conj(B))
    elif mode == 1:
        want = np.einsum("mkxy,knxy->mnxy", A, B)
    else:
        want = np.einsum("kmxy,knxy->mnxy", np.conj(A), B)
    pack = lambda z: dev(np.stack([z.real, z.imag], -1).astype(np.float32))
    for accumulate in (False, True):
        Cd = pack(C0)
        nn.transposeMM(pack(A), pack(B), Cd, 0.5, conj_a, conj_b, accumulate, layout="planes")
        got = host(Cd)
        got = got[..., 0] + 1j * got[..., 1]
        exp = 0.5 * want + (C0 if accumulate else 0)
        assert np.abs(got - exp).max() <= 2e-5 * np.abs(exp).max()


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_contraction_clock_probe(nn, mode):
    """The measurement variant of the tile kernel (in the probe library): same product as transposeMM (it runs the same tile code),
    and a shader clock between the chip's idle and peak clocks."""
    Q, m, n, k = 40, 128, 64, 64
    A = synth.uniform(5, (Q, k, m, 2) if mode == 2 else (Q, m, k, 2))
    B = synth.uniform(6, (Q, n, k, 2) if mode == 0 else (Q, k, n, 2))
    C = torch.full((Q, m, n, 2), float("nan"), device="cuda")
    want = torch.empty_like(C)
    nn.transposeMM(dev(A), dev(B), want, 1.0, mode == 2, mode == 0, False)
    from fbcunn_amd import probe
    mhz = probe.contractionClock(mode, dev(A), dev(B), C, launches=5)
    assert 300.0 < mhz < 2600.0, mhz
    got, ref = _c(host(C)), _c(host(want))
    assert np.isfinite(got).all()
    assert np.abs(got - ref).max() <= TOL * np.abs(ref).max()
    with pytest.raises(ValueError):
        probe.contractionClock(mode, dev(A)[:, :, :40].contiguous() if mode != 2 else dev(A)[:, :40].contiguous(),
                               dev(B)[:, :, :40].contiguous() if mode == 0 else dev(B)[:, :40].contiguous(), C)
