"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def max_rel(got, want):
    """max |got - want| / max |want| : the north-star criterion (bound 1e-3)."""
    return float(np.max(np.abs(got.astype(np.float64) - want)) / max(np.max(np.abs(want)), 1e-30))


def rel_l2(got, want):
    """||got - want|| / ||want|| : the reference's own metric (test/test_FFT.lua:239-250, bound 1e-4)."""
    d = got.astype(np.float64) - want
    return float(np.sqrt((d * d).sum()) / max(np.sqrt((np.asarray(want, np.float64) ** 2).sum()), 1e-30))


def freq_major_to_planes(freq):
    """(N, N/2+1, planes, 2) float -> complex (planes, N, N/2+1)."""
    c = freq[..., 0] + 1j * freq[..., 1]
    return np.transpose(c, (2, 0, 1))


def planes_to_freq_major(c):
    """complex (planes, N, N/2+1) -> float32 (N, N/2+1, planes, 2)."""
    t = np.transpose(c, (1, 2, 0))
    return np.ascontiguousarray(np.stack([t.real, t.imag], axis=-1).astype(np.float32))
