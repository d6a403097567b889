"""Explicit one-time weight pre-layout, the counterpart of casting a weight to the device's private format before
deployment (torch_npu's modules rely on such a cast, e.g. torch_npu/optim/npu_fused_optim_base.py:49)."""
from __future__ import annotations

import torch

from . import _capi

__all__ = ["prepare_quant_matmul_weight", "prepare_weight_quant_weight"]


def prepare_quant_matmul_weight(x2: torch.Tensor) -> torch.Tensor:
    """Return a tensor that is equal to ``x2`` (int8, logical ``[..., K, N]``) and can be passed to ``npu_quant_matmul``
    in its place, but whose storage is K-major (``[..., N, K]`` contiguous, i.e. strides ``(1, K)`` in the last two
    dimensions): the layout the int8 GEMM reads directly.  A weight that is contiguous along N is otherwise transposed
    into the workspace on every call (about 16 us for 45 MB).  Weights that are already K-major (the transposed view
    the contrib modules pass) are returned unchanged."""
    if x2.dtype != torch.int8 or x2.dim() < 2:
        raise ValueError(f"prepare_quant_matmul_weight expects an int8 weight with at least two dimensions, got {x2.dtype} {tuple(x2.shape)}")
    K, N = x2.shape[-2], x2.shape[-1]
    if x2.stride(-2) == 1 and x2.stride(-1) == K and (x2.dim() == 2 or x2.transpose(-1, -2).is_contiguous()):
        return x2
    flat = x2.reshape(-1, K, N)
    if flat.stride(-1) != 1:
        flat = flat.contiguous()
    out = torch.stack([_capi.transpose_int8(flat[b]) for b in range(flat.shape[0])]) if flat.shape[0] != 1 else \
        _capi.transpose_int8(flat[0]).unsqueeze(0)
    return out.reshape(*x2.shape[:-2], N, K).transpose(-1, -2)


def prepare_weight_quant_weight(weight: torch.Tensor) -> torch.Tensor:
    """Return a tensor equal to the int8 ``weight`` (logical ``[K, N]``) of ``npu_weight_quant_batchmatmul`` whose storage
    is ``[N, K]`` contiguous (strides ``(1, K)``): the layout ``LinearWeightQuant`` keeps and passes as a transposed view
    (torch_npu/contrib/module/linear_weight_quant.py:71,106).  With at most 32 activation rows and one scale per column
    that layout takes the decode kernel that splits K inside a workgroup (configuration 3: 41-45 us against 48-50 for a
    weight contiguous along N).  Weights already stored that way, and int32 words of int4 values, are returned
    unchanged."""
    if weight.dim() != 2:
        raise ValueError(f"prepare_weight_quant_weight expects a two-dimensional weight, got {tuple(weight.shape)}")
    if weight.dtype != torch.int8:
        return weight
    K, N = weight.shape
    if weight.stride(0) == 1 and weight.stride(1) == K:
        return weight
    src = weight if weight.stride(1) == 1 else weight.contiguous()
    return _capi.transpose_int8(src).t()
