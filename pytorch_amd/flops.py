"""FLOP formulas of the matmul operators for ``torch.utils.flop_counter.FlopCounterMode``.

The reference counts a (batched) matmul as 2 * M * K * N (torch_npu/profiler/_flops_formulas.py:319-329); the
quantised matmuls are registered with the same formula, with N taken from the logical weight shape (a packed
int4 weight holds eight columns per int32 word).
"""
from __future__ import annotations

from math import prod

import torch
from torch.utils.flop_counter import register_flop_formula


def _matmul_flops(x_shape, k: int, n: int) -> int:
    return int(2 * prod(x_shape[:-1]) * k * n)


@register_flop_formula(torch.ops.npu.npu_quant_matmul)
def quant_matmul_flops(x1_shape, x2_shape, *args, out_shape=None, **kwargs) -> int:
    batch = prod(out_shape[:-2]) if out_shape is not None and len(out_shape) > 2 else prod(x1_shape[:-2])
    return int(2 * batch * x1_shape[-2] * x1_shape[-1] * x2_shape[-1])


@register_flop_formula(torch.ops.npu.npu_weight_quant_batchmatmul, get_raw=True)
def weight_quant_batchmatmul_flops(x, weight, *args, out_val=None, **kwargs) -> int:
    n = weight.shape[-1] * (8 if weight.dtype == torch.int32 else 1)
    return _matmul_flops(tuple(x.shape), int(x.shape[-1]), int(n))
