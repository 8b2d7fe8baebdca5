"""CPU-only checks of the shipped library: it loads, exports every symbol the
header declares, and its host-side planning follows the reference's rules.  No
compute entry point is called here."""
import os
import re

import pytest

from fbcunn_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "fbfftconv.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(fbfc_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 18
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    handle = _lib.lib()                       # raises if the .so is missing
    for name in declared:
        assert hasattr(handle, name), name
    assert b"gfx950" in handle.fbfc_version()


def test_probe_library_is_separate_from_the_shipped_one():
    """include/fbfftconv_probe.h declares the measurement library's one symbol: libfbfftconv_probe.so
    exports it and the shipped library does not."""
    from fbcunn_amd import probe
    header = open(os.path.join(ROOT, "include", "fbfftconv_probe.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(fbfc_[a-z0-9_]+)\s*\(", header))
    assert declared == {"fbfc_probe_contraction_clock"}
    for name in declared:
        assert hasattr(probe.lib(), name)
        assert not hasattr(_lib.lib(), name)


def test_backward_buffers_are_reported():
    info = _q(batch=128, in_planes=64, out_planes=64, in_h=27, in_w=27, k_h=5, k_w=5, pad_h=2, pad_w=2)
    assert info.backward_freq_bytes == info.input_freq_bytes + info.weight_freq_bytes
    assert _q(in_h=112, in_w=112, tile_h=32, tile_w=32).backward_freq_bytes == 0
    assert _lib.lib().fbfc_plan_prepare_backward(None) == _lib.ERR_INVALID_ARGUMENT


def test_planes_layout_entries_validate_before_launching():
    """Every argument of the plane-major entry points is checked before the first kernel is launched
    (no GPU needed to see the refusals)."""
    import ctypes
    L = _lib.lib()
    ok, odd = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    assert L.fbfc_ifft2d_planes(ok, 4, 9, 8, 0, 0, 8, ok, ok, None) == _lib.ERR_INVALID_ARGUMENT
    assert b"must fit" in L.fbfc_last_error()
    assert L.fbfc_ifft2d_planes(odd, 4, 8, 8, 0, 0, 8, ok, ok, None) == _lib.ERR_INVALID_ARGUMENT
    assert L.fbfc_fft2d_planes(ok, 4, 8, 8, 0, 0, 8, odd, ok, None) == _lib.ERR_INVALID_ARGUMENT
    assert L.fbfc_transpose_mm_planes(ok, odd, ok, 1, 4, 4, 4, ctypes.c_float(1.0), 0, 0, 0, ok, None) == _lib.ERR_INVALID_ARGUMENT
    assert L.fbfc_transpose_mm_planes(ok, ok, ok, 1, 4, 4, 4, ctypes.c_float(1.0), 1, 1, 0, ok, None) == _lib.ERR_UNSUPPORTED_DIMENSION


def _q(**kw):
    base = dict(batch=2, in_planes=3, out_planes=4, in_h=13, in_w=13, k_h=3, k_w=3,
                stride_h=1, stride_w=1, pad_h=1, pad_w=1)
    base.update(kw)
    return _lib.plan_query(**base)


# FFT size = nextPowerOf2(max(H+2pU, W+2pL, kH, kW, oH, oW)), fbcunn/SpatialConvolutionFFT.lua:947-956
@pytest.mark.parametrize("kw,n,q,o", [
    (dict(batch=128, in_planes=64, out_planes=64, in_h=27, in_w=27, k_h=5, k_w=5, pad_h=2, pad_w=2), 32, 544, 27),
    (dict(batch=128, in_planes=128, out_planes=128, in_h=13, in_w=13, k_h=3, k_w=3, pad_h=1, pad_w=1), 16, 144, 13),
    (dict(batch=64, in_planes=96, out_planes=256, in_h=55, in_w=55, k_h=9, k_w=9, pad_h=4, pad_w=4), 64, 2112, 55),
    (dict(batch=4, in_planes=16, out_planes=16, in_h=32, in_w=32, k_h=5, k_w=5, pad_h=0, pad_w=0), 32, 544, 28),
    (dict(in_h=3, in_w=3, k_h=2, k_w=2, pad_h=0, pad_w=0), 8, 40, 2),      # tiny: canvas rounded up to 8
    (dict(in_h=16, in_w=9, k_h=3, k_w=3, pad_h=1, pad_w=0), 32, 544, 16),   # square canvas from the larger side
    (dict(in_h=100, in_w=90, k_h=5, k_w=5, pad_h=2, pad_w=2), 128, 8320, 100),
])
def test_plan_sizes(kw, n, q, o):
    info = _q(**kw)
    assert (info.fft_size, info.n_freq, info.out_h) == (n, q, o)


def test_plan_buffer_bytes_match_reference_layout():
    # (d0, d1, N/2+1, N, 2) floats per buffer, fbcunn/SpatialConvolutionFFT.lua:710-721
    info = _q(batch=128, in_planes=64, out_planes=64, in_h=27, in_w=27, k_h=5, k_w=5, pad_h=2, pad_w=2)
    assert info.input_freq_bytes == 128 * 64 * 17 * 32 * 2 * 4
    assert info.weight_freq_bytes == 64 * 64 * 17 * 32 * 2 * 4
    assert info.output_freq_bytes == 128 * 64 * 17 * 32 * 2 * 4


@pytest.mark.parametrize("kw,code,text", [
    (dict(stride_h=2), _lib.ERR_INVALID_ARGUMENT, "stride-1"),
    (dict(stride_w=3), _lib.ERR_INVALID_ARGUMENT, "stride-1"),
    (dict(pad_h=3), _lib.ERR_INVALID_ARGUMENT, "Padding must be smaller than kernel"),
    (dict(pad_w=5), _lib.ERR_INVALID_ARGUMENT, "Padding must be smaller than kernel"),
    (dict(batch=0), _lib.ERR_INVALID_ARGUMENT, "positive"),
    (dict(in_h=2, in_w=2, k_h=5, k_w=5, pad_h=0, pad_w=0), _lib.ERR_INVALID_ARGUMENT, "kernel larger"),
    (dict(in_h=200, in_w=100), _lib.ERR_UNSUPPORTED_SIZE, "not supported"),
    (dict(in_h=2000, in_w=5), _lib.ERR_UNSUPPORTED_SIZE, "Too large"),
])
def test_plan_rejections(kw, code, text):
    with pytest.raises(_lib.FbfcError) as e:
        _q(**kw)
    assert e.value.code == code
    assert text in e.value.message


def test_plan_refuses_more_planes_than_one_launch_addresses():
    """One launch addresses a frequency row of the spectrum with 32-bit offsets: the limit is checked
    when the plan is made and the message carries the numbers."""
    n = 64
    lim = (2 ** 31 - 1) // ((n // 2 + 1) * 8)
    ok = _q(batch=lim // 4096, in_planes=4096, out_planes=16, in_h=55, in_w=55, k_h=9, k_w=9, pad_h=4, pad_w=4)
    assert ok.fft_size == n
    with pytest.raises(_lib.FbfcError) as e:
        _q(batch=lim // 4096 + 1, in_planes=4096, out_planes=16, in_h=55, in_w=55, k_h=9, k_w=9, pad_h=4, pad_w=4)
    assert e.value.code == _lib.ERR_UNSUPPORTED_SIZE
    assert str(lim) in e.value.message and "input planes" in e.value.message
    with pytest.raises(_lib.FbfcError) as e:
        _q(batch=2, in_planes=8192, out_planes=8192, in_h=100, in_w=100, k_h=3, k_w=3, pad_h=1, pad_w=1)
    assert e.value.code == _lib.ERR_UNSUPPORTED_SIZE and "output planes x input planes" in e.value.message
    with pytest.raises(_lib.FbfcError) as e:    # tiles multiply the batch
        _q(batch=4096, in_planes=512, out_planes=64, in_h=224, in_w=224, tile_h=16, tile_w=16)
    assert e.value.code == _lib.ERR_UNSUPPORTED_SIZE and "batch x tiles" in e.value.message


def test_debug_knob_validates_its_argument():
    assert _lib.lib().fbfc_debug_force_contraction_kernel(3) == _lib.ERR_INVALID_ARGUMENT
    assert _lib.lib().fbfc_debug_force_contraction_kernel(-1) == _lib.OK
    assert _lib.lib().fbfc_debug_force_spectrum_streaming(0) == _lib.ERR_INVALID_ARGUMENT
    assert _lib.lib().fbfc_debug_force_spectrum_streaming(-1) == _lib.OK


def test_misaligned_complex_buffers_are_refused():
    """Complex buffers are accessed as 8-byte (re, im) pairs: a pointer that is not 8-byte aligned is an
    argument error, found before any launch (no GPU needed)."""
    import ctypes
    L = _lib.lib()
    ok, odd = ctypes.c_void_p(0x1000), ctypes.c_void_p(0x1004)
    assert L.fbfc_fft2d(ok, 4, 8, 8, 0, 0, 8, odd, None) == _lib.ERR_INVALID_ARGUMENT
    assert b"aligned" in L.fbfc_last_error()
    assert L.fbfc_ifft2d(odd, 4, 8, 8, 0, 0, 8, ok, None, 1, None) == _lib.ERR_INVALID_ARGUMENT
    assert L.fbfc_transpose_mm(ok, odd, ok, 1, 4, 4, 4, ctypes.c_float(1.0), 0, 0, 0, None) == _lib.ERR_INVALID_ARGUMENT


def test_scratch_size_query():
    assert _lib.lib().fbfc_bias_grad_scratch_bytes(128, 64) >= 64 * 4
    assert _lib.lib().fbfc_bias_grad_scratch_bytes(0, 64) == 0


# Tiled planning (fbcunn/SpatialConvolutionFFTTiled.lua:521-537): windows of the tile size,
# tile - kernel + 1 apart; the FFT is the next power of two of the tile.
@pytest.mark.parametrize("kw,tile,n,tiles", [
    (dict(in_h=112, in_w=112), (32, 32), 32, (4, 4)),          # o = 112, step 30
    (dict(in_h=224, in_w=224), (32, 32), 32, (8, 8)),          # o = 224, step 30
    (dict(in_h=56, in_w=56), (16, 16), 16, (4, 4)),            # o = 56, step 14
    (dict(in_h=45, in_w=52), (10, 14), 16, (6, 5)),            # steps 8 and 12
    (dict(in_h=20, in_w=20, k_h=5, k_w=5, pad_h=0, pad_w=0), (8, 8), 8, (4, 4)),   # o = 16, step 4
])
def test_tiled_plan_sizes(kw, tile, n, tiles):
    info = _q(**dict(kw, tile_h=tile[0], tile_w=tile[1]))
    assert info.fft_size == n and (info.tiles_h, info.tiles_w) == tiles
    q = n * (n // 2 + 1)
    assert info.n_freq == q
    # buffers hold batch * tiles planes (tiles of the output, or of gradInput if those are more)
    assert info.output_freq_bytes >= q * 2 * tiles[0] * tiles[1] * 4 * 8
    assert _q(**kw).tiles_h == 1 if max(kw["in_h"], kw["in_w"]) <= 126 else True


@pytest.mark.parametrize("kw,tile,code,text", [
    (dict(in_h=20, in_w=20, k_h=5, k_w=5, pad_h=0, pad_w=0), (4, 4), _lib.ERR_INVALID_ARGUMENT,
     "Tiling cannot be smaller than kernel"),
    (dict(in_h=20, in_w=20), (32, 32), _lib.ERR_INVALID_ARGUMENT, "Tile size too large (32x32) for output (20x20)"),
    (dict(in_h=100, in_w=100), (64, 64), _lib.ERR_UNSUPPORTED_SIZE, "tile FFT size"),
    (dict(in_h=100, in_w=100, stride_h=2), (16, 16), _lib.ERR_INVALID_ARGUMENT, "stride-1"),
    (dict(in_h=100, in_w=100), (16, 0), _lib.ERR_INVALID_ARGUMENT, "both tile sizes"),
])
def test_tiled_plan_rejections(kw, tile, code, text):
    with pytest.raises(_lib.FbfcError) as e:
        _q(**dict(kw, tile_h=tile[0], tile_w=tile[1]))
    assert e.value.code == code
    assert text in e.value.message


def test_tiled_plan_accepts_images_too_large_for_one_fft():
    with pytest.raises(_lib.FbfcError):
        _q(in_h=224, in_w=224)
    assert _q(in_h=224, in_w=224, tile_h=32, tile_w=32).fft_size == 32
