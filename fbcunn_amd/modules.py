"""Host-side mirror of the reference's Lua modules for the FFT-convolution path.

Same names, constructor arguments, fields and call protocol as
nn.SpatialConvolutionFBFFT / nn.SpatialConvolutionFBFFTGemm
(fbcunn/SpatialConvolutionFBFFT.lua, fbcunn/SpatialConvolutionFBFFTGemm.lua,
base class fbcunn/SpatialConvolutionFFT.lua) and nn.FFTWrapper
(fbcunn/FFTWrapper.lua).  All arithmetic happens in libfbfftconv.so; torch is
used only to own device memory and to name the current stream.
"""
import ctypes
import math

import torch

from . import _lib
from ._lib import ConvDesc, FbfcError, PlanInfo, check, lib

__all__ = ["SpatialConvolutionFFT", "SpatialConvolutionFBFFT", "SpatialConvolutionFBFFTGemm", "SpatialConvolutionDirect",
           "SpatialConvolutionFFTTiled", "SpatialConvolutionFFTTiledSync", "SpatialConvolutionFFTTiledAsync",
           "SpatialConvolutionFFTTiledIterated", "FFTWrapper", "transposeMM", "updateOutputBias", "accGradParametersBias", "FbfcError"]


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _check_tensor(t, name, ndim=None, strided=False):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("%s: CUDA support only!" % name)   # the reference's assert message
    if t.dtype != torch.float32:
        raise TypeError("%s must be float32" % name)
    if ndim is not None and t.dim() != ndim:
        raise ValueError("%s must be %d-D" % (name, ndim))
    if not strided and not t.is_contiguous():
        raise ValueError("%s must be contiguous" % name)


class _Plan:
    """RAII holder of one fbfc_plan."""

    def __init__(self, desc, tile=None, iterated=False):
        self.handle = ctypes.c_void_p(0)
        if tile is None:
            check(lib().fbfc_plan_create(ctypes.byref(desc), ctypes.byref(self.handle)))
        elif iterated:
            check(lib().fbfc_plan_create_tiled_iterated(ctypes.byref(desc), tile[0], tile[1], ctypes.byref(self.handle)))
        else:
            check(lib().fbfc_plan_create_tiled(ctypes.byref(desc), tile[0], tile[1], ctypes.byref(self.handle)))
        self.info = PlanInfo()
        check(lib().fbfc_plan_get_info(self.handle, ctypes.byref(self.info)))
        self.backward_state = None   # None: not asked yet; True: prepared; False: no room (two halves)

    def prepare_backward(self):
        """The extra buffers of the one-grid-per-stage backward(), made once and outside the pass.  With no
        room for them backward() runs as its two halves (same results); any other failure raises."""
        if self.backward_state is None:
            rc = lib().fbfc_plan_prepare_backward(self.handle)
            if rc not in (_lib.OK, _lib.ERR_OUT_OF_MEMORY):
                check(rc)
            self.backward_state = rc == _lib.OK
        return self.backward_state

    def close(self):
        if self.handle:
            lib().fbfc_plan_destroy(self.handle)
            self.handle = ctypes.c_void_p(0)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class SpatialConvolutionDirect:
    """The direct (spatial-domain) convolution, in the role cudnn.SpatialConvolution plays next to the
    reference's FFT modules: non-FFT candidate of the tuning front (fbcunn/SpatialConvolution.lua:259-269),
    fallback for layers the FFT path cannot run (fbcunn/SpatialConvolutionFFT.lua:323-393) and the
    result the self-check compares with (:91-133).  Any stride.  accGradParameters assigns gradWeight
    and gradBias, like the FFT modules here."""

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padW=0, padH=0, device="cuda", init=True):
        self.nInputPlane, self.nOutputPlane = nInputPlane, nOutputPlane
        self.kW, self.kH, self.dW, self.dH, self.padW, self.padH = kW, kH, dW, dH, padW, padH
        self.device = torch.device(device)
        self.weight = torch.empty(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.bias = torch.empty(nOutputPlane, device=self.device)
        self.gradWeight = torch.zeros(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.gradBias = torch.zeros(nOutputPlane, device=self.device)
        self.output = None
        self.gradInput = None
        if init:   # init=False: the caller hands in its own parameters; the random stream is left alone
            stdv = 1.0 / math.sqrt(kW * kH * nInputPlane)
            self.weight.uniform_(-stdv, stdv)
            self.bias.uniform_(-stdv, stdv)

    def _desc(self, input):
        _check_tensor(input, "input", 4)
        if input.size(1) != self.nInputPlane:
            raise ValueError("input has %d planes, module expects %d" % (input.size(1), self.nInputPlane))
        return ConvDesc(input.size(0), self.nInputPlane, self.nOutputPlane, input.size(2), input.size(3),
                        self.kH, self.kW, self.dH, self.dW, self.padH, self.padW)

    def _out_shape(self, input):
        return (input.size(0), self.nOutputPlane, (input.size(2) + 2 * self.padH - self.kH) // self.dH + 1,
                (input.size(3) + 2 * self.padW - self.kW) // self.dW + 1)

    def updateOutput(self, input):
        d = self._desc(input)
        shape = self._out_shape(input)
        if self.output is None or tuple(self.output.shape) != shape:
            self.output = torch.empty(shape, device=input.device)
        check(lib().fbfc_direct_update_output(ctypes.byref(d), _ptr(input), _ptr(self.weight), _ptr(self.bias),
                                              _ptr(self.output), _stream()))
        return self.output

    forward = updateOutput

    def updateGradInput(self, input, gradOutput):
        d = self._desc(input)
        _check_tensor(gradOutput, "gradOutput", 4)
        if tuple(gradOutput.shape) != self._out_shape(input):
            raise ValueError("gradOutput has the wrong shape")
        if self.gradInput is None or self.gradInput.shape != input.shape:
            self.gradInput = torch.empty_like(input)
        check(lib().fbfc_direct_update_grad_input(ctypes.byref(d), _ptr(gradOutput), _ptr(self.weight),
                                                  _ptr(self.gradInput), _stream()))
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1.0):
        d = self._desc(input)
        _check_tensor(gradOutput, "gradOutput", 4)
        if tuple(gradOutput.shape) != self._out_shape(input):
            raise ValueError("gradOutput has the wrong shape")
        nbytes = lib().fbfc_bias_grad_scratch_bytes(input.size(0), self.nOutputPlane)
        scratch = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=input.device)
        check(lib().fbfc_direct_acc_grad_parameters(ctypes.byref(d), _ptr(input), _ptr(gradOutput),
                                                    _ptr(self.gradWeight), _ptr(self.gradBias),
                                                    ctypes.c_float(scale), _ptr(scratch), _stream()))

    def backward(self, input, gradOutput, scale=1.0):
        self.updateGradInput(input, gradOutput)
        self.accGradParameters(input, gradOutput, scale)
        return self.gradInput

    def cleanupBuffers(self):
        pass


class SpatialConvolutionFFT:
    """Module state and protocol of nn.SpatialConvolutionFFT
    (fbcunn/SpatialConvolutionFFT.lua:150-316, 405-416)."""

    # relative-L2 bound of the self-check (fbcunn/SpatialConvolutionFFT.lua:15)
    prec = 2e-5

    memoryReuseNone = "none"
    memoryReuseInput = "input"
    memoryReuseOutput = "output"
    memoryReuseWeight = "weight"
    memoryReuseAll = "all"
    _REUSE_BITS = {"none": _lib.REUSE_NONE, "input": _lib.REUSE_INPUT, "output": _lib.REUSE_OUTPUT,
                   "weight": _lib.REUSE_WEIGHT, "all": _lib.REUSE_ALL}

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padLeft=0, padUp=0,
                 memoryReusePolicy=None, numCudaStreams=None, device="cuda"):
        for v in (nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp):
            if not isinstance(v, int):
                raise TypeError("module dimensions must be numbers")
        self.nInputPlane, self.nOutputPlane = nInputPlane, nOutputPlane
        self.kW, self.kH = kW, kH
        self.dW, self.dH = dW, dH
        self.padLeft, self.padUp = padLeft, padUp
        self.padRight, self.padDown = padLeft, padUp
        if self.dW != 1 or self.dH != 1:
            raise ValueError("fft only supports stride-1 convolutions atm")
        if not (self.padUp < self.kH and self.padLeft < self.kW):
            raise ValueError("Padding must be smaller than kernel")
        if memoryReusePolicy is None:
            memoryReusePolicy = [self.memoryReuseNone]
        if isinstance(memoryReusePolicy, str):
            memoryReusePolicy = [memoryReusePolicy]
        self.memoryReusePolicy = list(memoryReusePolicy)
        self._reuse_bits = 0
        for p in self.memoryReusePolicy:
            if p not in self._REUSE_BITS:
                raise ValueError("unknown memory reuse policy " + str(p))
            self._reuse_bits |= self._REUSE_BITS[p]
        self.numCudaStreams = numCudaStreams or 16  # kept for signature parity; one stream is used
        self.device = torch.device(device)
        self.weight = torch.empty(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.bias = torch.empty(nOutputPlane, device=self.device)
        self.gradWeight = torch.zeros(nOutputPlane, nInputPlane, kH, kW, device=self.device)
        self.gradBias = torch.zeros(nOutputPlane, device=self.device)
        self.output = None
        self.gradInput = None
        self.timed = False
        # the reference's debugging hook (fbcunn/SpatialConvolutionFFT.lua:160-161, 91-133): with
        # cudnnDebug set every pass is run again through the direct convolution and cudnnChecks turns
        # False when they differ by more than `prec` in relative L2
        self.cudnnDebug = False
        self.cudnnChecks = True
        self.printDebugLevel = -1
        self._plans = {}
        self.reset()

    def debugVSCUDNN(self, pass_name, got, run_direct):
        """Compares `got` with what the direct path computes for the same pass (run_direct(module) ->
        tensor); ||direct - got|| / ||direct|| must not exceed self.prec."""
        other = getattr(self, "_direct_ref", None)
        if other is None:   # made once per module, without drawing from the caller's random stream
            other = SpatialConvolutionDirect(self.nInputPlane, self.nOutputPlane, self.kW, self.kH, self.dW, self.dH,
                                             self.padLeft, self.padUp, device=self.device, init=False)
            self._direct_ref = other
        other.weight, other.bias = self.weight, self.bias
        want = run_direct(other).double()
        norm = math.sqrt(float(torch.dot(want.flatten(), want.flatten())) + 1e-8)
        err = float((want - got.double()).norm()) / norm
        ok = bool(torch.isfinite(got).all()) and err <= self.prec
        if not ok:
            print("%s error %s %g %g" % (type(self).__name__, pass_name, err, self.prec))
        elif self.printDebugLevel >= 0:
            print("%s debug vs direct check passes %s %g" % (type(self).__name__, pass_name, err))
        self.cudnnChecks = self.cudnnChecks and ok
        return ok

    # -- parameters ---------------------------------------------------------------
    def reset(self, stdv=None):
        """uniform(-stdv, stdv), stdv = 1/sqrt(kW*kH*nInputPlane) (SpatialConvolutionFFT.lua:271-289)."""
        if stdv is not None:
            stdv = stdv * math.sqrt(3)
        else:
            stdv = 1.0 / math.sqrt(self.kW * self.kH * self.nInputPlane)
        self.weight.uniform_(-stdv, stdv)
        self.bias.uniform_(-stdv, stdv)

    def zeroGradParameters(self):
        self.gradWeight.zero_()
        self.gradBias.zero_()

    def parameters(self):
        return [self.weight, self.bias], [self.gradWeight, self.gradBias]

    # -- planning -------------------------------------------------------------------
    def _plan_for(self, batch, in_h, in_w):
        key = (batch, in_h, in_w)
        plan = self._plans.get(key)
        if plan is None:
            desc = ConvDesc(batch, self.nInputPlane, self.nOutputPlane, in_h, in_w, self.kH, self.kW,
                            self.dH, self.dW, self.padUp, self.padLeft)
            plan = _Plan(desc, self._tile(), self._iterated())
            if self._reuse_bits:
                check(lib().fbfc_plan_set_reuse(plan.handle, self._reuse_bits))
            self._plans[key] = plan
        check(lib().fbfc_plan_set_timed(plan.handle, int(self.timed)))  # reps per stage, 0 = off
        return plan

    def _tile(self):
        """(tileSizeH, tileSizeW) of a tiled module, None otherwise."""
        return None

    def _iterated(self):
        """Whether the passes run as the fused kernels of nn.SpatialConvolutionFFTTiledIterated."""
        return False

    def _check_input(self, input):
        _check_tensor(input, "input", 4)
        if input.size(1) != self.nInputPlane:
            raise ValueError("input has %d planes, module expects %d" % (input.size(1), self.nInputPlane))

    def stageKernels(self, input):
        """What each stage of the last pass on this input shape launched (dict stage -> string)."""
        plan = self._plan_for(input.size(0), input.size(2), input.size(3))
        out = {}
        for i, name in enumerate(_lib.STAGE_NAMES):
            buf = ctypes.create_string_buffer(200)
            check(lib().fbfc_plan_stage_kernel(plan.handle, i, buf, len(buf)))
            if buf.value:
                out[name] = buf.value.decode()
        return out

    def stageTimes(self, input):
        """Mean ms per launch of each stage of the last pass run with self.timed = reps > 0 (dict)."""
        plan = self._plan_for(input.size(0), input.size(2), input.size(3))
        ms = (ctypes.c_float * len(_lib.STAGE_NAMES))()
        check(lib().fbfc_plan_stage_ms(plan.handle, ms, len(_lib.STAGE_NAMES)))
        return dict(zip(_lib.STAGE_NAMES, [float(x) for x in ms]))

    # -- nn.Module protocol -----------------------------------------------------------
    def updateOutput(self, input):
        self._check_input(input)
        B, _, H, W = input.shape
        plan = self._plan_for(B, H, W)
        shape = (B, self.nOutputPlane, plan.info.out_h, plan.info.out_w)
        # allocated once, like the reference (SpatialConvolutionFFT.lua:435-441), but
        # re-made when the shape changes instead of silently keeping the old size
        if self.output is None or tuple(self.output.shape) != shape:
            self.output = torch.empty(shape, device=input.device)
        check(lib().fbfc_update_output(plan.handle, _ptr(input), _ptr(self.weight), _ptr(self.bias),
                                       _ptr(self.output), _stream()))
        if self.cudnnDebug:
            self.debugVSCUDNN("updateOutput", self.output, lambda m: m.updateOutput(input))
        return self.output

    forward = updateOutput

    def updateGradInput(self, input, gradOutput):
        self._check_input(input)
        _check_tensor(gradOutput, "gradOutput", 4)
        B, _, H, W = input.shape
        plan = self._plan_for(B, H, W)
        if tuple(gradOutput.shape) != (B, self.nOutputPlane, plan.info.out_h, plan.info.out_w):
            raise ValueError("gradOutput has the wrong shape")
        if self.gradInput is None or self.gradInput.shape != input.shape:
            self.gradInput = torch.empty_like(input)
        check(lib().fbfc_update_grad_input(plan.handle, _ptr(gradOutput), _ptr(self.weight),
                                           _ptr(self.gradInput), _stream()))
        if self.cudnnDebug:
            self.debugVSCUDNN("updateGradInput", self.gradInput, lambda m: m.updateGradInput(input, gradOutput))
        return self.gradInput

    def accGradParameters(self, input, gradOutput, scale=1.0):
        """gradWeight and gradBias are overwritten, as in the reference's FBFFT path
        (accumulate=false, SpatialConvolutionFBFFT.lua:337-349)."""
        self._check_input(input)
        _check_tensor(gradOutput, "gradOutput", 4)
        B, _, H, W = input.shape
        plan = self._plan_for(B, H, W)
        if tuple(gradOutput.shape) != (B, self.nOutputPlane, plan.info.out_h, plan.info.out_w):
            raise ValueError("gradOutput has the wrong shape")
        check(lib().fbfc_acc_grad_parameters(plan.handle, _ptr(input), _ptr(gradOutput),
                                             _ptr(self.gradWeight), _ptr(self.gradBias),
                                             ctypes.c_float(scale), _stream()))
        if self.cudnnDebug:
            def both(m):
                m.accGradParameters(input, gradOutput, scale)
                return torch.cat([m.gradWeight.flatten(), m.gradBias.flatten()])
            self.debugVSCUDNN("accGradParameters", torch.cat([self.gradWeight.flatten(), self.gradBias.flatten()]), both)

    def backward(self, input, gradOutput, scale=1.0):
        """updateGradInput + accGradParameters sharing FFT(gradOutput)
        (SpatialConvolutionFFT.lua:405-416)."""
        self._check_input(input)
        _check_tensor(gradOutput, "gradOutput", 4)
        B, _, H, W = input.shape
        plan = self._plan_for(B, H, W)
        if tuple(gradOutput.shape) != (B, self.nOutputPlane, plan.info.out_h, plan.info.out_w):
            raise ValueError("gradOutput has the wrong shape")
        if self.gradInput is None or self.gradInput.shape != input.shape:
            self.gradInput = torch.empty_like(input)
        plan.prepare_backward()   # allocates on the first call for this shape only (see prepareBackward)
        check(lib().fbfc_backward(plan.handle, _ptr(input), _ptr(gradOutput), _ptr(self.weight),
                                  _ptr(self.gradInput), _ptr(self.gradWeight), _ptr(self.gradBias),
                                  ctypes.c_float(scale), _stream()))
        return self.gradInput

    def prepareBackward(self, input):
        """Allocates what backward() on inputs of this shape needs, so that backward() itself allocates
        nothing (call it before capturing backward() into a graph).  True if the one-grid-per-stage form
        will run, False if there was no room and backward() will run as its two passes."""
        self._check_input(input)
        return self._plan_for(input.size(0), input.size(2), input.size(3)).prepare_backward()

    def cleanupBuffers(self):
        for plan in self._plans.values():
            plan.close()
        self._plans = {}


class SpatialConvolutionFBFFT(SpatialConvolutionFFT):
    """nn.SpatialConvolutionFBFFT (fbcunn/SpatialConvolutionFBFFT.lua)."""
    fftImplementation = "fbfft"


class SpatialConvolutionFBFFTGemm(SpatialConvolutionFFT):
    """nn.SpatialConvolutionFBFFTGemm (fbcunn/SpatialConvolutionFBFFTGemm.lua).  The
    reference differs from FBFFT only in HOW the per-frequency contraction is
    done (explicit transposes + cuBLAS Cgemm); here both modules share the one
    frequency-major MFMA contraction, which is the layout that variant builds."""
    fftImplementation = "fbfft"


class SpatialConvolutionFFTTiled(SpatialConvolutionFBFFT):
    """nn.SpatialConvolutionFFTTiled (fbcunn/SpatialConvolutionFFTTiled.lua:260-330): the image is
    convolved window by window with FFTs of the tile size (default 16) instead of one FFT that
    covers the whole image.  Constructor arguments in the reference's order."""

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padLeft=0, padUp=0,
                 tileSizeW=None, tileSizeH=None, memoryReusePolicy=None, numCudaStreams=None, device="cuda"):
        for v in (tileSizeW, tileSizeH):
            if v is not None and not isinstance(v, int):
                raise TypeError("tile sizes must be numbers")
        self.tileSizeH = tileSizeH or 16
        self.tileSizeW = tileSizeW or 16
        super().__init__(nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp, memoryReusePolicy,
                         numCudaStreams, device)

    def _tile(self):
        return (self.tileSizeH, self.tileSizeW)


class SpatialConvolutionFFTTiledSync(SpatialConvolutionFFTTiled):
    """nn.SpatialConvolutionFFTTiledSync (fbcunn/SpatialConvolutionFFTTiledSync.lua): in the
    reference one tile after the other on one stream; here all tiles go through each stage in a
    single launch, so the Sync / Async / Iterated variants are one implementation."""


class SpatialConvolutionFFTTiledAsync(SpatialConvolutionFFTTiled):
    """nn.SpatialConvolutionFFTTiledAsync (fbcunn/SpatialConvolutionFFTTiledAsync.lua)."""


class SpatialConvolutionFFTTiledIterated(SpatialConvolutionFFTTiled):
    """nn.SpatialConvolutionFFTTiledIterated (fbcunn/SpatialConvolutionFFTTiledIterated.lua): every pass is
    one fused kernel per tile block (window transforms, product over the contracted planes, inverse
    transform) that never writes a spectrum of a feature map to memory.  Like the reference's module
    (:47-48) it overrides any memory reuse policy with "none"."""

    def __init__(self, nInputPlane, nOutputPlane, kW, kH, dW=1, dH=1, padLeft=0, padUp=0,
                 tileSizeW=None, tileSizeH=None, memoryReusePolicy=None, numCudaStreams=None, device="cuda"):
        super().__init__(nInputPlane, nOutputPlane, kW, kH, dW, dH, padLeft, padUp, tileSizeW, tileSizeH,
                         None, numCudaStreams, device)

    def _iterated(self):
        return True


class FFTWrapper:
    """nn.FFTWrapper with the fbfft backend (fbcunn/FFTWrapper.lua:53-132).

    Two transform dimensions: time (..., h, w) real, frequency a float tensor of shape
    (N, N/2+1, planes, 2), frequency-major.  One transform dimension: time (..., n) real,
    frequency (rows, N/2+1, 2) as in the reference.  ffti is unnormalised.  With timed set,
    every call is measured (1 skipped + 1 timed run, src/fft/FFTWrapperLua.cpp:106-134) and
    `lastTiming` holds {"ms", "GNlogN/s"} computed like the reference's log line (:137-152)."""

    def __init__(self, cufft=None, padLeft=0, padUp=0, timed=False, layout="frequency"):
        if cufft not in (None, "fbfft", False, 0):
            raise ValueError("only the fbfft implementation exists in this build")
        if layout not in ("frequency", "planes"):
            raise ValueError("layout must be 'frequency' or 'planes'")
        self.padLeft, self.padUp = padLeft, padUp
        self.timed = bool(timed)
        self.lastTiming = None
        # "planes": the reference's own 2-D buffer, (planes..., N/2+1, N, 2), first frequency axis
        # halved and laid out as fbfft leaves it (test/test_FFTModule.lua:238-241)
        self.layout = layout
        self._workspace = None

    def _planes_workspace(self, planes, n, device):
        nbytes = lib().fbfc_planes_layout_workspace_bytes(planes, n)
        if self._workspace is None or self._workspace.numel() * 4 < nbytes or self._workspace.device != device:
            self._workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=device)
        return self._workspace

    def _dims_planes(self, time, frequency):
        _check_tensor(time, "time")
        _check_tensor(frequency, "frequency")
        if frequency.dim() < 4 or frequency.size(-1) != 2:
            raise ValueError("frequency must be (planes..., N/2+1, N, 2)")
        n = frequency.size(-2)
        if frequency.size(-3) != n // 2 + 1:
            raise ValueError("frequency must be (planes..., N/2+1, N, 2)")
        planes = frequency.numel() // (2 * n * (n // 2 + 1))
        h, w = time.size(-2), time.size(-1)
        if time.numel() != planes * h * w:
            raise ValueError("time and frequency disagree on the number of planes")
        return n, planes, h, w

    @staticmethod
    def _dims(time, frequency):
        _check_tensor(time, "time")
        _check_tensor(frequency, "frequency")
        if frequency.dim() == 3:                       # one transform dimension
            rows, nh = frequency.size(0), frequency.size(1)
            if frequency.size(2) != 2 or nh < 2:
                raise ValueError("frequency must be (rows, N/2+1, 2)")
            n = 2 * (nh - 1)
            if time.numel() != rows * time.size(-1):
                raise ValueError("time and frequency disagree on the number of rows")
            return 1, n, rows, 1, time.size(-1)
        if frequency.dim() != 4:
            raise ValueError("frequency must be (rows, N/2+1, 2) or (N, N/2+1, planes, 2)")
        n = frequency.size(0)
        planes = frequency.size(2)
        if frequency.size(1) != n // 2 + 1 or frequency.size(3) != 2:
            raise ValueError("frequency must be (N, N/2+1, planes, 2)")
        h, w = time.size(-2), time.size(-1)
        if time.numel() != planes * h * w:
            raise ValueError("time and frequency disagree on the number of planes")
        return 2, n, planes, h, w

    def lastKernel(self):
        """What the last transform called from this thread launched ("<kernel> grid=<work-items>")."""
        return lib().fbfc_last_launch().decode()

    def _run(self, call, dims, n, batches):
        if not self.timed:
            call()
            return
        call()                                           # skipped trial
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        call()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        size = float(batches) * (n ** dims) * (1.0 + dims * math.log(n))   # the reference's formula
        self.lastTiming = {"ms": ms, "GNlogN/s": size / 1e9 / (ms * 1e-3) if ms > 0 else float("inf")}

    def fft(self, time, frequency, batchDims=None):
        if self.layout == "planes" and frequency.dim() >= 4:
            n, planes, h, w = self._dims_planes(time, frequency)
            ws = self._planes_workspace(planes, n, time.device)
            self._run(lambda: check(lib().fbfc_fft2d_planes(_ptr(time), planes, h, w, self.padUp, self.padLeft, n,
                                                            _ptr(frequency), _ptr(ws), _stream())), 2, n, planes)
            return frequency
        dims, n, planes, h, w = self._dims(time, frequency)
        if dims == 1:
            self._run(lambda: check(lib().fbfc_fft1d(_ptr(time), planes, w, self.padLeft, n, _ptr(frequency),
                                                     _stream())), 1, n, planes)
        else:
            self._run(lambda: check(lib().fbfc_fft2d(_ptr(time), planes, h, w, self.padUp, self.padLeft, n,
                                                     _ptr(frequency), _stream())), 2, n, planes)
        return frequency

    def ffti(self, time, frequency, batchDims=None, bias=None):
        if self.layout == "planes" and frequency.dim() >= 4:
            if bias is not None:
                raise ValueError("the plane-major inverse adds no bias")
            n, planes, h, w = self._dims_planes(time, frequency)
            ws = self._planes_workspace(planes, n, time.device)
            self._run(lambda: check(lib().fbfc_ifft2d_planes(_ptr(frequency), planes, h, w, self.padUp, self.padLeft,
                                                             n, _ptr(time), _ptr(ws), _stream())), 2, n, planes)
            return time
        dims, n, planes, h, w = self._dims(time, frequency)
        if dims == 1:
            self._run(lambda: check(lib().fbfc_ifft1d(_ptr(frequency), planes, w, self.padLeft, n, _ptr(time),
                                                      _stream())), 1, n, planes)
        else:
            period = bias.numel() if bias is not None else 1
            self._run(lambda: check(lib().fbfc_ifft2d(_ptr(frequency), planes, h, w, self.padUp, self.padLeft, n,
                                                      _ptr(time), _ptr(bias), period, _stream())), 2, n, planes)
        return time


def transposeMM(A, B, C, invNorm, conjugateTransposeA, conjugateTransposeB, accumulate, layout="frequency"):
    """transposeMMFFI (src/MM.cu:54-73).  layout "frequency": operands (Q, rows, cols, 2);
    layout "planes": the reference's own (rows, cols, f1, f2, 2) buffers, Q = f1 * f2."""
    if layout == "planes":
        for t, nme in ((A, "A"), (B, "B"), (C, "C")):
            _check_tensor(t, nme, 5)
        m, n = C.size(0), C.size(1)
        Q = C.size(2) * C.size(3)
        k = A.size(0) if conjugateTransposeA else A.size(1)
        exp_a = (k, m) if conjugateTransposeA else (m, k)
        exp_b = (n, k) if conjugateTransposeB else (k, n)
        if tuple(A.shape[:2]) != exp_a or tuple(B.shape[:2]) != exp_b or \
                tuple(A.shape[2:]) != tuple(C.shape[2:]) or tuple(B.shape[2:]) != tuple(C.shape[2:]):
            raise ValueError("operand shapes do not match: A %s B %s C %s" % (tuple(A.shape), tuple(B.shape), tuple(C.shape)))
        nbytes = lib().fbfc_transpose_mm_planes_workspace_bytes(Q, m, n, k)
        ws = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=C.device)
        check(lib().fbfc_transpose_mm_planes(_ptr(A), _ptr(B), _ptr(C), Q, m, n, k, ctypes.c_float(invNorm),
                                             int(bool(conjugateTransposeA)), int(bool(conjugateTransposeB)),
                                             int(bool(accumulate)), _ptr(ws), _stream()))
        return C
    for t, nme in ((A, "A"), (B, "B"), (C, "C")):
        _check_tensor(t, nme, 4)
    Q, m, n = C.size(0), C.size(1), C.size(2)
    k = A.size(1) if conjugateTransposeA else A.size(2)
    exp_a = (Q, k, m, 2) if conjugateTransposeA else (Q, m, k, 2)
    exp_b = (Q, n, k, 2) if conjugateTransposeB else (Q, k, n, 2)
    if tuple(A.shape) != exp_a or tuple(B.shape) != exp_b:
        raise ValueError("operand shapes do not match: A %s B %s C %s" % (tuple(A.shape), tuple(B.shape), tuple(C.shape)))
    check(lib().fbfc_transpose_mm(_ptr(A), _ptr(B), _ptr(C), Q, m, n, k, ctypes.c_float(invNorm),
                                  int(bool(conjugateTransposeA)), int(bool(conjugateTransposeB)),
                                  int(bool(accumulate)), _stream()))
    return C


def updateOutputBias(output, bias):
    """updateOutputBiasFFI (src/ConvolutionBias.cu:256-260); like the reference's kernel it takes
    non-contiguous tensors (test/BiasTest.cpp:38-63)."""
    _check_tensor(output, "output", 4, strided=True)
    _check_tensor(bias, "bias", 1, strided=True)
    B, F, h, w = output.shape
    if output.is_contiguous() and bias.is_contiguous():
        check(lib().fbfc_update_output_bias(_ptr(output), _ptr(bias), B, F, h, w, _stream()))
    else:
        check(lib().fbfc_update_output_bias_strided(_ptr(output), _ptr(bias), B, F, h, w, *output.stride(),
                                                    bias.stride(0), _stream()))
    return output


def accGradParametersBias(gradOutput, gradBias, scale=1.0):
    """accGradParametersBiasFFI (src/ConvolutionBias.cu:262-274): gradBias is assigned.  Takes
    non-contiguous tensors (test/BiasTest.cpp:186-222)."""
    _check_tensor(gradOutput, "gradOutput", 4, strided=True)
    _check_tensor(gradBias, "gradBias", 1, strided=True)
    B, F, h, w = gradOutput.shape
    nbytes = lib().fbfc_bias_grad_scratch_bytes(B, F)
    scratch = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=gradOutput.device)
    if gradOutput.is_contiguous() and gradBias.is_contiguous():
        check(lib().fbfc_acc_grad_parameters_bias(_ptr(gradOutput), _ptr(gradBias), ctypes.c_float(scale),
                                                  B, F, h, w, _ptr(scratch), _stream()))
    else:
        check(lib().fbfc_acc_grad_parameters_bias_strided(_ptr(gradOutput), _ptr(gradBias), ctypes.c_float(scale),
                                                          B, F, h, w, *gradOutput.stride(), gradBias.stride(0),
                                                          _ptr(scratch), _stream()))
    return gradBias
