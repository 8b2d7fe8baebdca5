"""fbcunn_amd: the FFT-convolution path of fbcunn, built for MI355X (gfx950).

Only the path behind nn.SpatialConvolutionFBFFT / nn.SpatialConvolutionFBFFTGemm, its
tiled variants and the tuning front fbnn.SpatialConvolution exists here.  `nn` and `fbnn`
mirror the reference's Lua module names; importing them needs the built library
(python -m fbcunn_amd.build) and raises otherwise.
"""
__all__ = ["synth"]


def __getattr__(name):
    if name == "nn":
        from . import modules
        return modules
    if name == "fbnn":
        from . import tuned
        return tuned
    raise AttributeError(name)
