"""Weight-only quantized linear layer on top of ``torch.ops.npu.npu_weight_quant_batchmatmul``.

Counterpart of torch_npu/contrib/module/linear_weight_quant.py:98-109: ``weight`` is stored
``[out_features, in_features]`` and handed over as its transposed view; two-dimensional
antiquant parameters (per-group, stored ``[N, G]``) are handed over transposed as well.
"""
from __future__ import annotations

import torch
from torch import nn

__all__ = ["LinearWeightQuant"]


class LinearWeightQuant(nn.Module):
    def __init__(self, in_features, out_features, bias: bool = True, device=None, dtype=None,
                 antiquant_offset: bool = False, quant_scale: bool = False, quant_offset: bool = False,
                 antiquant_group_size: int = 0, inner_precise: int = 0, weight_dtype=None) -> None:
        super().__init__()
        frozen = lambda *shape: nn.Parameter(torch.empty(*shape, device=device), requires_grad=False)  # noqa: E731
        self.weight = frozen((out_features, in_features))
        self.antiquant_scale = frozen(out_features)
        for name, present in (("antiquant_offset", antiquant_offset), ("quant_scale", quant_scale),
                              ("quant_offset", quant_offset), ("bias", bias)):
            if present:
                setattr(self, name, frozen(out_features))
            else:
                self.register_parameter(name, None)
        self.antiquant_group_size = antiquant_group_size
        self.inner_precise = inner_precise
        self.weight_dtype = weight_dtype

    @staticmethod
    def _as_group_major(param):
        return param.transpose(-1, -2) if param is not None and param.dim() == 2 else param

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return torch.ops.npu.npu_weight_quant_batchmatmul(
            x, self.weight.transpose(-1, -2), self._as_group_major(self.antiquant_scale),
            self._as_group_major(self.antiquant_offset), self.quant_scale, self.quant_offset, self.bias,
            self.antiquant_group_size, self.inner_precise, weight_dtype=self.weight_dtype)
