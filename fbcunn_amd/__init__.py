"""fbcunn_amd: the FFT-convolution path of fbcunn, built for MI355X (gfx950).

Only the path behind nn.SpatialConvolutionFBFFT / nn.SpatialConvolutionFBFFTGemm
exists here.  `nn` mirrors the reference's Lua module names; importing it needs
the built library (python -m fbcunn_amd.build) and raises otherwise.
"""
__all__ = ["synth"]


def __getattr__(name):
    if name == "nn":
        from . import modules
        return modules
    raise AttributeError(name)
