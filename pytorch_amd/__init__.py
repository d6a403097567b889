"""MI355X-native quantized-inference operators behind torch_npu's operator names.

Importing this package loads the gfx950 kernel library (C ABI, ``include/mi355_quant.h``) and
the torch operator library that registers ``torch.ops.npu.npu_dynamic_quant``,
``npu_quant_matmul``, ``npu_weight_quant_batchmatmul`` and ``npu_swiglu``, then re-exports
every ``torch.ops.npu.*`` operator as an attribute of the package, the way torch_npu does
(torch_npu/_init/core/_exports.py:45-51), so ``pytorch_amd.npu_quant_matmul(...)`` is a drop-in
for ``torch_npu.npu_quant_matmul(...)``.

There is no CPU or eager-PyTorch fallback: if the native libraries are missing the import
fails, and the operators only accept tensors on the GPU.
"""
from __future__ import annotations

import os as _os

import torch as _torch

_CSRC = _os.path.join(_os.path.dirname(_os.path.abspath(__file__)), "csrc")
KERNEL_LIBRARY = _os.path.join(_CSRC, "libmi355_quant.so")
OPS_LIBRARY = _os.path.join(_CSRC, "libmi355_npu_ops.so")

for _p in (KERNEL_LIBRARY, OPS_LIBRARY):
    if not _os.path.exists(_p):
        raise ImportError(f"{_p} is missing: build the native libraries first with `python pytorch_amd/build.py` "
                          "(hipcc, --offload-arch=gfx950)")

_torch.ops.load_library(OPS_LIBRARY)

__all__ = []


def _export_npu_ops() -> None:
    # every operator registered in the "npu" namespace becomes an attribute of the package
    names = sorted({n.split("::", 1)[1].split(".", 1)[0] for n in _torch._C._dispatch_get_all_op_names()
                    if n.startswith("npu::")})
    for _name in names:
        globals()[_name] = getattr(_torch.ops.npu, _name)
        __all__.append(_name)


_export_npu_ops()

from . import contrib  # noqa: E402,F401
from . import flops  # noqa: E402,F401  (registers the FLOP formulas of the matmul operators)
from .prepare import prepare_quant_matmul_weight, prepare_weight_quant_weight  # noqa: E402,F401


def check_device_status() -> None:
    """Waits for the streams the operators have launched on and raises RuntimeError if a kernel reported a failure
    through the status word of its workspace (a bounded wait for another workgroup's partial sums ran out; the outputs of
    that launch hold NaN).  The workspaces concerned are cleared, so the operators can be used again afterwards.  The
    reference reports device-side failures the same way, at the caller's next synchronisation
    (torch_npu/csrc/framework/OpParamMaker.cpp:541-571)."""
    import ctypes as _ctypes
    failures = _ctypes.CDLL(OPS_LIBRARY).mi355_npu_check_workspaces()
    if failures:
        raise RuntimeError(f"mi355: {failures} workspace(s) hold a device-side failure report (a bounded wait for split-K "
                           "partial sums ran out; the outputs of that launch hold NaN); the workspaces have been cleared")


__all__.append("check_device_status")
