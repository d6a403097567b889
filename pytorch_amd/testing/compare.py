"""Comparison rules for operator outputs.

``rtol_failures`` / ``assert_rtol_equal`` restate the element rule of
``TestCase.assertRtolEqual`` (torch_npu/testing/testcase.py:158-227): an element fails
only if it violates BOTH the absolute and the relative bound, and the comparison as a
whole fails only if more than ``size * prec`` elements fail.

``bf16_gate`` is the acceptance gate for bf16 (and float16) outputs of this operator path:
  * at least 99.9 % of the elements lie within one unit in the last place (of the output type) of the
    float32 golden value, counted strictly on the number line of the output type (``within_1ulp_strict``).
    ``floor=True`` selects the looser count (``within_1ulp``) in which elements that cancel to almost
    nothing (|golden| below 1/256 of the root mean square of the golden values) are judged by the unit of
    that floor magnitude; both fractions are always returned, and
  * no element is off by more than 1e-2 relative to max(|a|, |b|) unless its absolute error is below four
    units in the last place of the root mean square of the golden values (values that cancel to ~0 carry
    the rounding of their much larger terms, so they are judged on that absolute scale, which follows
    the data instead of being a fixed constant).
"""
from __future__ import annotations

import numpy as np
import torch


def _np(a):
    if isinstance(a, torch.Tensor):
        a = a.detach().cpu()
        if a.dtype in (torch.bfloat16, torch.float16):
            a = a.float()
        a = a.numpy()
    return np.asarray(a)


def rtol_failures(x, y, prec: float = 1e-4) -> int:
    x = _np(x).astype(np.float64)
    y = _np(y).astype(np.float64)
    d = np.abs(x - y)
    denom = np.maximum(np.abs(x), np.abs(y)) + np.finfo(np.float64).tiny
    return int(np.count_nonzero((d > prec) & (d / denom > prec)))


def assert_rtol_equal(x, y, prec: float = 1e-4, prec16: float = 1e-3) -> None:
    xa, ya = _np(x), _np(y)
    if xa.shape != ya.shape:
        raise AssertionError(f"shape error: {xa.shape} vs {ya.shape}")
    tx = x.dtype if hasattr(x, "dtype") else xa.dtype
    ty = y.dtype if hasattr(y, "dtype") else ya.dtype
    if tx != ty:
        raise AssertionError(f"dtype error: {tx} vs {ty}")
    p = prec16 if tx in (torch.float16, torch.bfloat16, np.float16) else prec
    bad = rtol_failures(xa, ya, p)
    if bad > xa.size * p:
        raise AssertionError(f"result error: {bad} of {xa.size} elements outside tolerance {p}")


def _bf16_line(t: torch.Tensor) -> np.ndarray:
    u = t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16).astype(np.int32)
    return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)


def bf16_gate(out_bf16: torch.Tensor, golden_f32: torch.Tensor, *, min_within_1ulp: float = 0.999,
              max_rel: float = 1e-2, floor: bool = False) -> dict:
    """Return the gate statistics; raise AssertionError when the gate is not met.

    ``golden_f32`` is the unrounded float32 golden.  "Within one ulp" is measured on the
    bf16 number line between ``out`` and the golden rounded to bf16 (distance <= 1)."""
    assert out_bf16.dtype in (torch.bfloat16, torch.float16)     # the same gate serves float16 outputs (fp16 ulps)
    g32 = golden_f32.detach().cpu().float()
    o = out_bf16.detach().cpu()
    dist = np.abs(_bf16_line(o) - _bf16_line(g32.to(out_bf16.dtype)))
    exact = float(np.count_nonzero(dist == 0)) / max(dist.size, 1)
    of = o.float().numpy().astype(np.float64)
    gf = g32.numpy().astype(np.float64)
    # one unit in the last place at the magnitude of the (rounded) golden value, not below the cancellation floor
    gr = g32.to(out_bf16.dtype).float().numpy().astype(np.float64)
    finite = np.isfinite(gr)
    rms = float(np.sqrt(np.mean(np.square(gr[finite])))) if finite.any() else 0.0
    mant_bits = 7 if out_bf16.dtype == torch.bfloat16 else 10
    mag = np.maximum(np.abs(np.where(finite, gr, 0.0)), max(rms / 256.0, np.finfo(np.float64).tiny))
    ulp = np.exp2(np.floor(np.log2(mag)) - mant_bits)
    near = (dist <= 1) | (np.abs(of - gr) <= ulp * (1 + 1e-9))
    within = float(np.count_nonzero(near)) / max(dist.size, 1)
    strict = float(np.count_nonzero(dist <= 1)) / max(dist.size, 1)
    d = np.abs(of - gf)
    denom = np.maximum(np.abs(of), np.abs(gf)) + np.finfo(np.float64).tiny
    # an absolute escape for elements near the cancellation floor: four ulps of the golden's rms, never more than 1e-2
    abs_escape = min(1e-2, 4.0 * float(np.exp2(np.floor(np.log2(max(rms, np.finfo(np.float64).tiny))) - mant_bits)))
    bad = int(np.count_nonzero((d > abs_escape) & (d / denom > max_rel)))
    stats = {"within_1ulp_strict": strict, "within_1ulp": within, "bit_identical": exact,
             "max_ulp": int(dist.max()) if dist.size else 0, "abs_or_rel_failures": bad, "n": int(dist.size)}
    if not np.all(np.isfinite(of) == np.isfinite(gf)):
        raise AssertionError(f"non-finite mismatch: {stats}")
    if (within if floor else strict) < min_within_1ulp or bad:
        raise AssertionError(f"bf16 gate not met ({'floor' if floor else 'strict'} count): {stats}")
    return stats
