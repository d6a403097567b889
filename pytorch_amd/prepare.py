"""Explicit one-time weight pre-layout, the counterpart of casting a weight to the device's private format before
deployment (torch_npu's modules rely on such a cast, e.g. torch_npu/optim/npu_fused_optim_base.py:49)."""
from __future__ import annotations

import torch

from . import _capi

__all__ = ["prepare_quant_matmul_weight", "prepare_weight_quant_weight", "padded_row_bytes"]

# Weight rows of exactly 4096 bytes are the one pitch at which the decode kernels (at most 64 / 32 activation rows, K
# split over the wavefronts of a workgroup) read measurably slower than they could: rows 4096 bytes apart put the eight
# wavefronts' slices of sixteen rows on few memory channels.  One cache line of padding per row removes it
# (int8 [28672, 4096] at 16 rows: 23.5 -> 19.9 us; through the operator 23.0 -> 21.0).  Pitches of 2048, 6144, 8192, 12288,
# 14336 and 16384 bytes measured the same with and without padding, so only this one is padded.
_PADDED_PITCHES = {4096: 128}


def padded_row_bytes(row_bytes: int) -> int:
    """Row pitch in bytes that the prepared K-major layouts use for rows of ``row_bytes`` bytes."""
    return row_bytes + _PADDED_PITCHES.get(row_bytes, 0)


def _k_major(nk: torch.Tensor, row_pad: bool) -> torch.Tensor:
    """``nk``: contiguous ``[N, K]`` int8.  Returns a ``[N, K]`` tensor with the prepared row pitch."""
    N, K = nk.shape
    pitch = padded_row_bytes(K) if row_pad else K
    if pitch == K:
        return nk
    store = torch.empty((N, pitch), dtype=nk.dtype, device=nk.device)
    store[:, K:].zero_()
    out = store[:, :K]
    out.copy_(nk)
    return out


def prepare_quant_matmul_weight(x2: torch.Tensor, row_pad: bool = True) -> torch.Tensor:
    """Return a tensor that is equal to ``x2`` (int8, logical ``[..., K, N]``) and can be passed to ``npu_quant_matmul``
    in its place, but whose storage is K-major (``[..., N, K]``, i.e. stride 1 along K): the layout the int8 GEMM reads
    directly.  A weight that is contiguous along N is otherwise transposed into the workspace on every call (about
    17 us for 45 MB).  With ``row_pad`` a two-dimensional weight whose rows are 4096 bytes gets a row pitch of 4224
    (see ``_PADDED_PITCHES``).  Weights that already have the prepared layout are returned unchanged."""
    if x2.dtype != torch.int8 or x2.dim() < 2:
        raise ValueError(f"prepare_quant_matmul_weight expects an int8 weight with at least two dimensions, got {x2.dtype} {tuple(x2.shape)}")
    K, N = x2.shape[-2], x2.shape[-1]
    want_pitch = padded_row_bytes(K) if row_pad and x2.dim() == 2 else K
    if x2.stride(-2) == 1 and x2.stride(-1) == want_pitch and (x2.dim() == 2 or x2.transpose(-1, -2).is_contiguous()):
        return x2
    if x2.dim() == 2 and x2.stride(0) == 1 and x2.stride(1) >= K:                  # K-major already: only the pitch changes
        return _k_major(x2.t().contiguous() if x2.stride(1) != K else x2.t(), row_pad).t()
    flat = x2.reshape(-1, K, N)
    if flat.stride(-1) != 1:
        flat = flat.contiguous()
    out = torch.stack([_capi.transpose_int8(flat[b]) for b in range(flat.shape[0])]) if flat.shape[0] != 1 else \
        _capi.transpose_int8(flat[0]).unsqueeze(0)
    if x2.dim() == 2:
        return _k_major(out[0], row_pad).t()
    return out.reshape(*x2.shape[:-2], N, K).transpose(-1, -2)


def prepare_weight_quant_weight(weight: torch.Tensor, row_pad: bool = True) -> torch.Tensor:
    """Return a tensor equal to the int8 ``weight`` (logical ``[K, N]``) of ``npu_weight_quant_batchmatmul`` whose storage
    is ``[N, K]`` contiguous (strides ``(1, K)``): the layout ``LinearWeightQuant`` keeps and passes as a transposed view
    (torch_npu/contrib/module/linear_weight_quant.py:71,106).  With at most 32 activation rows and one scale per column
    that layout takes the decode kernel that splits K inside a workgroup (configuration 3: 41-45 us against 48-50 for a
    weight contiguous along N).  With ``row_pad`` rows of 4096 bytes get a pitch of 4224 (see ``_PADDED_PITCHES``).
    Weights already stored that way, and int32 words of int4 values, are returned unchanged."""
    if weight.dim() != 2:
        raise ValueError(f"prepare_weight_quant_weight expects a two-dimensional weight, got {tuple(weight.shape)}")
    if weight.dtype != torch.int8:
        return weight
    K, N = weight.shape
    want_pitch = padded_row_bytes(K) if row_pad else K
    if weight.stride(0) == 1 and weight.stride(1) == want_pitch:
        return weight
    if weight.stride(0) == 1 and weight.stride(1) >= K:                             # [N, K] already: only the pitch changes
        return _k_major(weight.t().contiguous() if weight.stride(1) != K else weight.t(), row_pad).t()
    src = weight if weight.stride(1) == 1 else weight.contiguous()
    return _k_major(_capi.transpose_int8(src), row_pad).t()
