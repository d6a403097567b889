"""Seeded synthetic inputs for the benchmark configurations of the quantized-operator path.

All tensors are produced on the CPU from ``torch.Generator().manual_seed(seed)`` so that
the CPU golden and the GPU kernels see identical bits; callers move them to the device.
"""
from __future__ import annotations

import torch


def _gen(seed: int) -> torch.Generator:
    return torch.Generator().manual_seed(int(seed))


def pack_int4(w4: torch.Tensor) -> torch.Tensor:
    """int8 values in [-8, 7], shape [..., N] -> int32 [..., N/8]; element i of a word sits in
    bits [4i, 4i+3] (nibble order of test/custom_ops/test_npu_anti_quant.py:12-24)."""
    assert w4.shape[-1] % 8 == 0
    n = (w4.to(torch.int64) & 0xF).reshape(*w4.shape[:-1], w4.shape[-1] // 8, 8)
    shifts = torch.arange(8, dtype=torch.int64) * 4
    word = (n << shifts).sum(-1)
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32)


def dynamic_quant_input(seed: int = 0, rows: int = 2048, cols: int = 4096, dtype=torch.bfloat16):
    """x ~ N(0,1) with 0.1 % of the entries scaled x50 as outliers."""
    g = _gen(seed)
    x = torch.randn(rows, cols, generator=g)
    mask = torch.rand(rows, cols, generator=g) < 1e-3
    x = torch.where(mask, x * 50.0, x)
    return x.to(dtype)


def quant_matmul_inputs(seed: int = 0, M: int = 1024, K: int = 4096, N: int = 11008, *,
                        weight_nk: bool = False, bias: bool = True):
    """W8A8 inputs.  ``weight_nk`` stores the weight as [N, K] and returns its transposed
    view (logical [K, N], strides (1, K)) as torch_npu/contrib/module/linear_quant.py:110 does."""
    g = _gen(seed)
    x1 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    x2 = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8)
    if weight_nk:
        x2 = x2.t().contiguous().t()
    ps = torch.rand(M, generator=g) * 9e-3 + 1e-3
    s = torch.rand(N, generator=g) * 9e-3 + 1e-3
    b = (torch.randn(N, generator=g) * 0.02).to(torch.bfloat16) if bias else None
    return {"x1": x1, "x2": x2, "pertoken_scale": ps, "scale": s, "bias": b}


def w8a16_inputs(seed: int = 0, M: int = 16, K: int = 8192, N: int = 28672, *, weight_nk: bool = False):
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8)
    if weight_nk:
        w = w.t().contiguous().t()
    scale = (torch.rand(N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
    offset = (torch.rand(N, generator=g) * 8.0 - 4.0).to(torch.bfloat16)
    return {"x": x, "weight": w, "antiquant_scale": scale, "antiquant_offset": offset}


def w4a16_inputs(seed: int = 0, M: int = 1, K: int = 4096, N: int = 14336, group_size: int = 128):
    g = _gen(seed)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w4 = torch.randint(-8, 8, (K, N), generator=g, dtype=torch.int8)
    G = K // group_size
    scale = (torch.rand(G, N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
    offset = (torch.rand(G, N, generator=g) * 4.0 - 2.0).to(torch.bfloat16)
    return {"x": x, "weight": pack_int4(w4), "weight_int4_values": w4, "antiquant_scale": scale,
            "antiquant_offset": offset, "antiquant_group_size": group_size}


def mlp_inputs(seed: int = 0, M: int = 64, hidden: int = 4096, inter: int = 14336):
    """Llama-3-8B-shaped W8A8 decoder MLP, random init.  Weights are stored [N, K] as the
    contrib modules store them; ``w_gate_up`` stacks gate then up along N."""
    g = _gen(seed)
    x = torch.randn(M, hidden, generator=g).to(torch.bfloat16)
    w_gu = torch.randint(-127, 128, (2 * inter, hidden), generator=g, dtype=torch.int8)
    w_d = torch.randint(-127, 128, (hidden, inter), generator=g, dtype=torch.int8)
    s_gu = torch.rand(2 * inter, generator=g) * 9e-3 + 1e-3
    s_d = torch.rand(hidden, generator=g) * 9e-3 + 1e-3
    return {"x": x, "w_gate_up": w_gu, "w_down": w_d, "scale_gate_up": s_gu, "scale_down": s_d}
