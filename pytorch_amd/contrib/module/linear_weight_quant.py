"""Weight-only quantized linear layer on top of ``torch.ops.npu.npu_weight_quant_batchmatmul``.

Counterpart of torch_npu/contrib/module/linear_weight_quant.py:98-109: ``weight`` is stored
``[out_features, in_features]`` and handed over as its transposed view; two-dimensional
antiquant parameters (per-group, stored ``[N, G]``) are handed over transposed as well.

An int4 weight is stored ``[out_features, in_features / 8]`` int32, so its transposed view holds the words along
K; the operator has a kernel for that layout.  The layout the streaming and tiled kernels read fastest at decode
sizes is the other one (words along N, row-major ``[G, N]`` parameters): ``prepare_()`` builds that copy once, the
counterpart of casting a weight to the device's private format before deployment.
"""
from __future__ import annotations

import torch
from torch import nn

from ._prepared import PreparedCopiesMixin

__all__ = ["LinearWeightQuant"]


class LinearWeightQuant(PreparedCopiesMixin, nn.Module):
    _prepared_attrs = ("_prepared",)

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

    @torch.no_grad()
    def prepare_(self) -> "LinearWeightQuant":
        """One-time repack for inference (optional): an int4 weight is rewritten with its words along N and per-group
        parameters are made row-major ``[G, N]``, the layout the decode kernels stream fastest; an int8 weight with
        ``in_features`` = 4096 is copied into rows with a padded pitch.  The parameters the
        module exposes (and its state_dict) stay as they are; the prepared copies are plain attributes, so they cost
        the weight's size again.  Moving, casting or reloading the module drops them; call this again afterwards, and
        after changing a parameter in place."""
        self._prepared = None
        if self.weight.dtype == torch.int8:
            # rows of 4096 bytes get a padded pitch (pytorch_amd.prepare.padded_row_bytes); other weights stay as they are
            from ...prepare import prepare_weight_quant_weight
            kn = prepare_weight_quant_weight(self.weight.data.t())
            if kn.data_ptr() != self.weight.data_ptr():
                self._prepared = (kn, self._as_group_major(self.antiquant_scale), self._as_group_major(self.antiquant_offset))
            return self
        if self.weight.dtype != torch.int32:
            return self
        w = self.weight                                             # [N, K/8], word j of a row holds k = 8j..8j+7
        shifts = torch.arange(8, device=w.device, dtype=torch.int64) * 4
        nib = (w.to(torch.int64).unsqueeze(-1) >> shifts) & 0xF     # [N, K/8, 8] raw nibbles
        kn = nib.reshape(w.shape[0], -1).t().contiguous()           # [K, N]
        words = (kn.reshape(kn.shape[0], -1, 8) << shifts).sum(-1)  # [K, N/8]: word j of a row holds n = 8j..8j+7
        prepared_w = words.to(torch.int32)                          # wraps modulo 2**32: bit 31 becomes the sign
        from ...prepare import prepare_weight_quant_weight
        prepared_w = prepare_weight_quant_weight(prepared_w)        # row padding where the pitch calls for it
        group_major = lambda t: None if t is None else self._as_group_major(t).contiguous()  # noqa: E731
        self._prepared = (prepared_w, group_major(self.antiquant_scale), group_major(self.antiquant_offset))
        return self

    @staticmethod
    def _as_group_major(param):
        return param.transpose(-1, -2) if param is not None and param.dim() == 2 else param

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        prepared = getattr(self, "_prepared", None)
        if prepared is not None and self.weight.dtype == torch.int32 and self.antiquant_group_size == 128:
            # 2 to 32 rows: the decode kernel for the module's own storage (words along K) is the faster one
            # (int4 [14336, 4096/8], 8 / 32 rows: 9.8 / 15.4 us against 10.3 / 17.2 on the repacked copy)
            rows = x.numel() // x.shape[-1] if x.shape[-1] else 0
            if 2 <= rows <= 32:
                prepared = None
        if prepared is not None:
            weight, scale, offset = prepared
            return torch.ops.npu.npu_weight_quant_batchmatmul(x, weight, scale, offset, self.quant_scale, self.quant_offset,
                                                              self.bias, self.antiquant_group_size, self.inner_precise,
                                                              weight_dtype=self.weight_dtype)
        return torch.ops.npu.npu_weight_quant_batchmatmul(
            x, self.weight.transpose(-1, -2), self._as_group_major(self.antiquant_scale),
            self._as_group_major(self.antiquant_offset), self.quant_scale, self.quant_offset, self.bias,
            self.antiquant_group_size, self.inner_precise, weight_dtype=self.weight_dtype)
