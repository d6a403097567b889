"""Builds the native parts of the package in-tree with hipcc for gfx950.

* ``csrc/libmi355_quant.so``  - the HIP kernels behind the C ABI of ``include/mi355_quant.h``
* ``csrc/libmi355_npu_ops.so`` - the torch operator library registering ``torch.ops.npu.*``

Usage: ``python pytorch_amd/build.py`` (compiles every time it is called; run it as a script, because
importing the package requires the libraries this builds).
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
KERNEL_LIB = os.path.join(CSRC, "libmi355_quant.so")
OPS_LIB = os.path.join(CSRC, "libmi355_npu_ops.so")
KERNEL_SOURCES = ["dynamic_quant.hip", "dynamic_quant_asym.hip", "quant_matmul.hip", "quant_matmul_decode.hip", "weight_quant_matmul.hip", "weight_quant_gemm.hip", "weight_quant_kpacked.hip", "weight_quant_kpacked_decode.hip", "weight_quant_kmajor_decode.hip", "weight_quant_decode.hip", "weight_quant_gemm4.hip", "weight_quant_repack.hip", "swiglu.hip", "anti_quant.hip", "unpack_int4.hip", "quantize.hip", "tuning.hip", "device_probe.hip"]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=off: the dequantising epilogues must round every operation separately.
# packed-fp32-ops off: packed FP32 instructions are kept out of generated code on this platform.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
                "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
                "-Wno-pass-failed",
                # MFMA accumulators stay in ordinary vector registers.  Left to itself the compiler puts them into the
                # accumulation registers whenever a kernel may use 512 registers per lane, and then moves them to and
                # fro around every vector instruction that touches them (the per-group folds) and, for arrays of
                # accumulators in loops, around the MFMAs themselves (a register-only probe: 27 clocks per MFMA
                # instead of 17, and scratch spills in four streaming kernels).
                "-mllvm", "-amdgpu-mfma-vgpr-form"]


# Per-file additions (none at present).
EXTRA_FLAGS = {}


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(verbose: bool = False) -> str:
    objs = []

    def compile_one(src):
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        out = _run([HIPCC, *DEVICE_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(compile_one, KERNEL_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", KERNEL_LIB, *objs])
    # a kernel whose host stub the compiler silently dropped would only fail at load time
    undefined = [l for l in _run(["nm", "-u", KERNEL_LIB]).splitlines() if "mi355" in l]
    if undefined:
        raise RuntimeError("unresolved kernel symbols in %s:\n%s" % (KERNEL_LIB, "\n".join(undefined)))
    return KERNEL_LIB


def build_ops(verbose: bool = False) -> str:
    """torch operator library: host-only C++ against libtorch + the C ABI."""
    import torch
    from torch.utils import cpp_extension as ce

    inc = []
    for p in ce.include_paths(device_type="cuda"):
        inc += ["-I", p]
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-unused-command-line-argument",
           "-I", os.path.join(HERE, "..", "include"), *inc,
           os.path.join(CSRC, "npu_ops.cpp"), "-o", OPS_LIB,
           "-L", torch_lib, "-L", CSRC, "-lc10", "-ltorch_cpu", "-ltorch", "-lc10_hip", "-ltorch_hip", "-lmi355_quant",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    return OPS_LIB


def build_all(verbose: bool = False) -> None:
    build_kernels(verbose)
    if os.path.exists(os.path.join(CSRC, "npu_ops.cpp")):
        build_ops(verbose)


if __name__ == "__main__":
    build_all(verbose=True)
    print("built:", KERNEL_LIB, OPS_LIB if os.path.exists(OPS_LIB) else "")
    sys.exit(0)
