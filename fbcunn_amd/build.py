"""Builds fbcunn_amd/libfbfftconv.so (HIP kernels + C ABI) for gfx950 with hipcc, and beside it the
measurement library libfbfftconv_probe.so (an instrumented copy of the contraction kernel for bench.py;
the shipped library is compiled without it).

    python -m fbcunn_amd.build            # compile and link
    python -m fbcunn_amd.build --report   # also print register/LDS use per kernel
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libfbfftconv.so")
PROBE_LIB = os.path.join(HERE, "libfbfftconv_probe.so")
# (source, object name, extra flags) of the measurement library
PROBE_SOURCES = [("cgemm_kernels.hip", "cgemm_kernels_probe.o", ["-DFBFC_PROBES"]),
                 ("probe_clock.cpp", "probe_clock.o", ["-DFBFC_PROBES"])]
SOURCES = ["api.cpp", "fft_kernels.hip", "fft_large.hip", "fft_small.hip", "cgemm_kernels.hip", "bias_kernels.hip", "bias_noalloc.hip", "layout_kernels.hip", "direct_kernels.hip", "fused_kernels.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-x", "hip",
    # packed fp32 VALU forms are switched off for every device function
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


# Per-file flags.  fft_large.hip: with common-code sinking the two role branches of the inverse kernel
# end in one store through a pointer that selects between two register arrays, which forces both
# into scratch memory.
# The FFT files are compiled without implicit contraction of a multiply and an add into one operation (every
# multiply-add they want is written as one): which pairs the compiler fuses can differ between two
# instantiations of one kernel, and the staging variants of a transform must give the same bits.
NO_CONTRACT = ["-ffp-contract=off"]
EXTRA_FLAGS = {"fft_large.hip": ["-mllvm", "-simplifycfg-sink-common=false"] + NO_CONTRACT,
               "fft_kernels.hip": NO_CONTRACT, "fft_small.hip": NO_CONTRACT, "fused_kernels.hip": NO_CONTRACT}


def _compile(src, report, obj=None, extra=()):
    out = os.path.join(OBJ, obj or os.path.splitext(src)[0] + ".o")
    cmd = [HIPCC] + FLAGS + EXTRA_FLAGS.get(src, []) + list(extra) + ["-c", os.path.join(CSRC, src), "-o", out]
    if report:
        cmd.append("-Rpass-analysis=kernel-resource-usage")
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed on %s:\n%s" % (src, r.stderr))
    return out, r.stderr


def build(report=False):
    os.makedirs(OBJ, exist_ok=True)
    with ThreadPoolExecutor(max_workers=6) as ex:
        probe = [ex.submit(_compile, src, False, obj, extra) for src, obj, extra in PROBE_SOURCES]
        results = list(ex.map(lambda s: _compile(s, report), SOURCES))
        probe_objs = [f.result()[0] for f in probe]
    objs = [o for o, _ in results]
    for lib, parts in ((LIB, objs), (PROBE_LIB, probe_objs)):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + parts
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n%s" % r.stderr)
    if report:
        for _, err in results:
            keep = [l for l in err.splitlines()
                    if any(k in l for k in ("Function Name", "VGPRs:", "AGPRs", "ScratchSize", "Occupancy",
                                            "LDS Size", "SGPRs:"))]
            print("\n".join(keep))
    return LIB


if __name__ == "__main__":
    print(build(report="--report" in sys.argv))
