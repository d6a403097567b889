"""Explicit one-time weight pre-layout, the counterpart of casting a weight to the device's private format before
deployment (torch_npu's modules rely on such a cast, e.g. torch_npu/optim/npu_fused_optim_base.py:49)."""
from __future__ import annotations

import torch

from . import _capi

__all__ = ["prepare_quant_matmul_weight", "prepare_weight_quant_weight", "padded_row_bytes"]

# Row pitches at which the weight-streaming kernels read measurably slower than they could, and the padding (bytes per
# row) that removes it.  Rows 4096 bytes apart put the slices that the wavefronts of a decode workgroup read at the same
# time on few memory channels; one or two cache lines of padding per row spread them.  Measured at 16 rows, int8 stored
# [N, K]: K = 4096: 23.5 -> 19.9 us (N = 28672), K = 11008: 24.2 -> 22.7; int4 words along N, [4096, 14336 / 8] (7168
# bytes per row): 10.3 -> 9.5 us at one row, 32.8 -> 30.3 at 128.  Pitches of 2048, 5120, 6144, 8192, 12288, 14336, 16384
# and 28672 bytes measured within 2 % with and without padding (and some paddings 9-13 % slower), so only the measured
# cases are padded.
_PADDED_PITCHES = {4096: 128, 11008: 256, 7168: 256}


def padded_row_bytes(row_bytes: int) -> int:
    """Row pitch in bytes that the prepared K-major layouts use for rows of ``row_bytes`` bytes."""
    return row_bytes + _PADDED_PITCHES.get(row_bytes, 0)


def _k_major(nk: torch.Tensor, row_pad: bool) -> torch.Tensor:
    """``nk``: contiguous two-dimensional tensor.  Returns an equal tensor with the prepared row pitch."""
    rows, cols = nk.shape
    esz = nk.element_size()
    pitch = padded_row_bytes(cols * esz) // esz if row_pad else cols
    if pitch == cols:
        return nk
    store = torch.empty((rows, pitch), dtype=nk.dtype, device=nk.device)
    store[:, cols:].zero_()
    out = store[:, :cols]
    out.copy_(nk)
    return out


def prepare_quant_matmul_weight(x2: torch.Tensor, row_pad: bool = True) -> torch.Tensor:
    """Return a tensor that is equal to ``x2`` (int8, logical ``[..., K, N]``) and can be passed to ``npu_quant_matmul``
    in its place, but whose storage is K-major (``[..., N, K]``, i.e. stride 1 along K): the layout the int8 GEMM reads
    directly.  A weight that is contiguous along N is otherwise transposed into the workspace on every call (about
    17 us for 45 MB).  With ``row_pad`` a two-dimensional weight whose row pitch is in ``_PADDED_PITCHES`` is padded (rows of 4096
    bytes get a pitch of 4224).  Weights that already have the prepared layout are returned unchanged."""
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
    weight contiguous along N).  With ``row_pad`` rows whose pitch is in ``_PADDED_PITCHES`` are padded (int8 rows of
    4096 bytes get a pitch of 4224; int32 words of int4 values along N keep their layout and only get the padding).
    Weights already stored that way are returned unchanged."""
    if weight.dim() != 2:
        raise ValueError(f"prepare_weight_quant_weight expects a two-dimensional weight, got {tuple(weight.shape)}")
    if weight.dtype == torch.int32 and weight.stride(1) == 1 and row_pad:
        # int4 words along N: the layout stays, rows whose pitch is in the table are padded
        pitch = padded_row_bytes(weight.shape[1] * 4) // 4
        if weight.stride(0) == pitch:
            return weight
        return _k_major(weight.contiguous(), True) if pitch != weight.shape[1] else weight
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
