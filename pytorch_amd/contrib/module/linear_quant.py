"""W8A8 linear layers on top of ``torch.ops.npu.npu_quant_matmul``.

Counterparts of torch_npu/contrib/module/linear_quant.py:96-112 (``LinearQuant``) and
linear_a8w8_quant.py:87-120 (``LinearA8W8Quant``, the deprecated twin that validates dtypes
explicitly).  Parameter names, shapes and defaults are the reference's so a state dict moves
over unchanged: ``weight`` is stored ``[out_features, in_features]`` and reaches the operator
as its transposed view, i.e. logical ``[K, N]`` with strides ``(1, K)``.
"""
from __future__ import annotations

import warnings

import torch
from torch import nn

from ._prepared import PreparedCopiesMixin

__all__ = ["LinearQuant", "LinearA8W8Quant"]


class _QuantLinearBase(PreparedCopiesMixin, nn.Module):
    _validate_dtypes = False
    _prepared_attrs = ("_prepared_i8",)

    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, offset: bool = False,
                 pertoken_scale: bool = False, device=None, dtype=None, output_dtype=None) -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.output_dtype = output_dtype
        frozen = lambda t: nn.Parameter(t, requires_grad=False)  # noqa: E731
        self.weight = frozen(torch.empty((out_features, in_features)))
        self.scale = frozen(torch.empty(out_features))
        optional = {
            "offset": (offset, torch.float32),
            "pertoken_scale": (pertoken_scale, torch.float32),
            "bias": (bias, torch.int32),
        }
        for name, (present, dt) in optional.items():
            if present:
                setattr(self, name, frozen(torch.empty(out_features, dtype=dt)))
            else:
                self.register_parameter(name, None)

    def _check_dtypes(self, x: torch.Tensor) -> None:
        pair = (x.dtype, self.weight.dtype)
        if pair not in ((torch.int8, torch.int8), (torch.int32, torch.int32)):
            raise ValueError("input and weight should be both torch.int32 or both torch.int8 datatype, "
                             f"but now input is {x.dtype}, weight is {self.weight.dtype}.")
        if not self._validate_dtypes:
            return
        rules = (
            ("scale", self.scale, (torch.int64, torch.float32, torch.bfloat16),
             "scale should be torch.int64, torch.float32 or torch.bfloat16 datatype, "),
            ("offset", self.offset, (torch.float32,), "offset should be torch.float32 datatype, "),
            ("bias", self.bias, (torch.int32, torch.bfloat16, torch.float16, torch.float32),
             "bias should be torch.int32, torch.bfloat16, torch.float16 or torch.float32 datatype, "),
            ("pertoken_scale", self.pertoken_scale, (torch.float32,), "pertoken_scale should be torch.float32 datatype, "),
        )
        for _, tensor, allowed, text in rules:
            if tensor is not None and tensor.dtype not in allowed:
                raise ValueError(text + f"but now it is {tensor.dtype}.")
        if self.output_dtype is not None and self.output_dtype not in (torch.int8, torch.float16, torch.bfloat16):
            raise ValueError("output_dtype should be torch.int8, torch.float16 or torch.bfloat16, "
                             f"but now it is {self.output_dtype}.")

    def prepare_(self) -> "_QuantLinearBase":
        """One-time pre-layout for inference (optional).  A4W4: a weight stored as int32 words of eight int4 values is
        widened to int8 ``[out_features, in_features]`` once, so that a forward pass widens only the activations before
        the int8 GEMM instead of the weight as well.  W8A8 with ``in_features`` = 4096: the weight is copied into rows
        with a padded pitch (``pytorch_amd.prepare.padded_row_bytes``), which the decode kernels read 8-15 % faster.
        The parameter the module exposes (and its state_dict) stays as it is; the copy is a plain attribute that costs
        the int8 weight's size.  Moving, casting or reloading the module drops the copy; call this again afterwards,
        and after changing the weight in place."""
        self._prepared_i8 = None
        from ...prepare import prepare_quant_matmul_weight
        if self.weight.dtype == torch.int32:
            from ... import _capi
            self._prepared_i8 = prepare_quant_matmul_weight(_capi.unpack_int4(self.weight.data).t()).t()
        elif self.weight.dtype == torch.int8:
            prepared = prepare_quant_matmul_weight(self.weight.data.t()).t()
            if prepared.data_ptr() != self.weight.data_ptr():
                self._prepared_i8 = prepared
        return self

    def forward(self, linear_quant_input: torch.Tensor) -> torch.Tensor:
        self._check_dtypes(linear_quant_input)
        weight = self.weight
        prepared = getattr(self, "_prepared_i8", None)
        if prepared is not None and linear_quant_input.dtype == torch.int32:
            from ... import _capi
            x = linear_quant_input
            words = x.shape[-1]
            linear_quant_input = _capi.unpack_int4(x.reshape(-1, words).contiguous()).view(*x.shape[:-1], words * 8)
            weight = prepared
        elif prepared is not None and linear_quant_input.dtype == torch.int8 and self.weight.dtype == torch.int8:
            weight = prepared
        scale = self.scale
        # a float32 scale is packed with npu_trans_quant_param when there is no pertoken_scale and the output is int8
        # (output_dtype None) or float16 (linear_quant.py:104-108)
        if (self.pertoken_scale is None and scale.dtype == torch.float32
                and self.output_dtype not in (torch.bfloat16, torch.int32)):
            scale = torch.ops.npu.npu_trans_quant_param(scale, self.offset)
        return torch.ops.npu.npu_quant_matmul(linear_quant_input, weight.transpose(-2, -1), scale,
                                              offset=self.offset, pertoken_scale=self.pertoken_scale, bias=self.bias,
                                              output_dtype=self.output_dtype)


class LinearQuant(_QuantLinearBase):
    """``y = dequant(x_int8 @ weight_int8.T)``; see the module docstring."""


class LinearA8W8Quant(_QuantLinearBase):
    """Deprecated alias of :class:`LinearQuant` that validates parameter dtypes before the call."""
    _validate_dtypes = True

    def __init__(self, *args, **kwargs) -> None:
        warnings.warn("LinearA8W8Quant is deprecated and will be removed in a future version. "
                      "Use LinearQuant instead.", FutureWarning)
        super().__init__(*args, **kwargs)
