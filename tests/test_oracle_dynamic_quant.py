"""Pins oracle.dynamic_quant: library evaluation (torch), exact rational arithmetic,
hand-typed round-half-even answers and invariants of symmetric per-token quantisation."""
from fractions import Fraction

import numpy as np
import pytest
import torch

from pytorch_amd.testing import workloads


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_matches_torch_float32_evaluation(golden):
    x = workloads.dynamic_quant_input(seed=0, rows=64, cols=4096)
    y, s = golden.dynamic_quant(_bits(x))
    xf = x.float()
    scale = xf.abs().amax(-1) / 127.0
    yt = torch.round(xf / scale[:, None]).clamp(-127, 127).to(torch.int8)
    assert np.array_equal(s, scale.numpy())
    assert np.array_equal(y, yt.numpy())
    # the sample must actually contain exact .5 ties, or half-even is not exercised
    q = (xf / scale[:, None])
    assert int(((q - torch.floor(q)) == 0.5).sum()) > 0


def test_fp16_input_matches_torch(golden):
    g = torch.Generator().manual_seed(3)
    x = (torch.randn(16, 1024, generator=g) * 3).to(torch.float16)
    y, s = golden.dynamic_quant(_bits(x), in_dtype="fp16")
    xf = x.float()
    scale = xf.abs().amax(-1) / 127.0
    assert np.array_equal(s, scale.numpy())
    assert np.array_equal(y, torch.round(xf / scale[:, None]).clamp(-127, 127).to(torch.int8).numpy())


def _rne_f32(fr: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) binary32 of a positive rational in the normal range."""
    assert fr > 0
    e = 0
    while fr >= 2:
        fr /= 2
        e += 1
    while fr < 1:
        fr *= 2
        e -= 1
    m = fr * (1 << 23)           # in [2^23, 2^24)
    lo = m.numerator // m.denominator
    rem = m - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)):
        lo += 1
    return np.float32(float(lo) * 2.0 ** (e - 23))


def _rint_half_even(fr: Fraction) -> int:
    lo = fr.numerator // fr.denominator
    rem = fr - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)):
        lo += 1
    return lo


def test_exact_rational_arithmetic(golden):
    """scale = RN(amax/127), q = RN(x/scale), y = rint_half_even(q) with every step done in
    exact rational arithmetic and rounded by hand."""
    x = workloads.dynamic_quant_input(seed=5, rows=4, cols=512)
    y, s = golden.dynamic_quant(_bits(x))
    xf = x.float().numpy()
    for r in range(xf.shape[0]):
        amax = Fraction(float(np.abs(xf[r]).max()))
        sc = _rne_f32(amax / 127)
        assert sc == s[r]
        for j in range(xf.shape[1]):
            v = Fraction(float(xf[r, j]))
            if v == 0:
                assert y[r, j] == 0
                continue
            q = Fraction(float(_rne_f32(abs(v) / Fraction(float(sc)))))
            k = _rint_half_even(q)
            assert y[r, j] == (k if v > 0 else -k), (r, j)


def test_known_answers_half_even(golden):
    # amax = 127 -> scale exactly 1.0, so y = rint_half_even(x)
    vals = [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5, 126.5, -126.5, 0.0, 0.25, 0.75, -3.5, 100.5, 101.5]
    want = [127, 0, 2, 2, 0, -2, -2, 4, 126, -126, 0, 0, 1, -4, 100, 102]
    x = torch.tensor([vals], dtype=torch.bfloat16)
    assert x.float().tolist()[0] == vals  # all representable in bf16
    y, s = golden.dynamic_quant(_bits(x))
    assert s[0] == np.float32(1.0)
    assert y[0].tolist() == want


def test_zero_row_and_shapes(golden):
    x = torch.zeros(3, 5, 16, dtype=torch.bfloat16)
    x[1, 2, 3] = 2.0
    y, s = golden.dynamic_quant(_bits(x))
    assert y.shape == (3, 5, 16) and s.shape == (3, 5) and y.dtype == np.int8 and s.dtype == np.float32
    assert s[0, 0] == 0 and not y[0].any()
    assert y[1, 2, 3] == 127 and s[1, 2] == np.float32(2.0) / np.float32(127.0)


@pytest.mark.parametrize("seed", [0, 1])
def test_invariants(golden, seed):
    x = workloads.dynamic_quant_input(seed=seed, rows=128, cols=2048)
    y, s = golden.dynamic_quant(_bits(x))
    xf = x.float().numpy()
    assert (np.abs(y.astype(np.int32)).max(-1) == 127).all()          # every row reaches +-127
    err = np.abs(y.astype(np.float64) * s[:, None].astype(np.float64) - xf)
    # half-step reconstruction bound; the quotient itself carries one rounding (|q| <= 127)
    assert (err <= s[:, None] * (0.5 + 127 * 2.0 ** -23)).all()
    y2, s2 = golden.dynamic_quant(_bits(-x))                             # odd symmetry
    assert np.array_equal(s2, s) and np.array_equal(y2, -y)
    y3, s3 = golden.dynamic_quant(_bits(x * 4))                          # power-of-two scaling is exact
    assert np.array_equal(y3, y) and np.array_equal(s3, s * 4)


def test_smooth_scales(golden):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(8, 256, generator=g).to(torch.bfloat16)
    sm = (torch.rand(256, generator=g) + 0.5).to(torch.bfloat16)
    y, s = golden.dynamic_quant(_bits(x), smooth_u16=_bits(sm))
    xf = x.float() * sm.float()
    scale = xf.abs().amax(-1) / 127.0
    assert np.array_equal(s, scale.numpy())
    assert np.array_equal(y, torch.round(xf / scale[:, None]).clamp(-127, 127).to(torch.int8).numpy())


def test_per_expert_smooth_scales(golden):
    """group_index: rows below a running total take that expert's scales.  Checked against a torch float32 evaluation
    with the scales gathered per row, with an empty expert, and with totals that stop short of the row count."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(12, 128, generator=g).to(torch.bfloat16)
    sm = (torch.rand(4, 128, generator=g) + 0.5).to(torch.bfloat16)
    for totals, expert_of_row in [([3, 3, 8, 12], [0] * 3 + [2] * 5 + [3] * 4), ([5, 7, 9, 10], [0] * 5 + [1] * 2 + [2] * 2 + [3] * 3)]:
        y, s = golden.dynamic_quant_grouped(_bits(x), _bits(sm), totals)
        xf = x.float() * sm.float()[torch.tensor(expert_of_row)]
        scale = xf.abs().amax(-1) / 127.0
        assert np.array_equal(s, scale.numpy())
        assert np.array_equal(y, torch.round(xf / scale[:, None]).clamp(-127, 127).to(torch.int8).numpy())


def test_int4_output_hand_computed_and_torch(golden):
    """dst_type=torch.quint4x2: scale = max|x| / 7, codes rint(x / scale), eight to a word with the first column in the
    low nibble.  A row typed by hand (scale 1; ties 3.5 -> 4, 2.5 -> 2, +-0.5 -> 0; -7 is nibble 9) and a torch float32
    evaluation unpacked with the oracle's own unpack_int4 (whose nibble order the reference pins)."""
    row = torch.tensor([[7.0, -7.0, 3.5, 2.5, 0.5, -0.5, 1.0, 0.0]], dtype=torch.bfloat16)
    y, s = golden.dynamic_quant_int4(_bits(row))
    assert s.tolist() == [1.0] and y.dtype == np.int32 and y.shape == (1, 1)
    assert int(y.view(np.uint32)[0, 0]) == 0x01002497
    g = torch.Generator().manual_seed(8)
    x = (torch.randn(16, 256, generator=g) * 2).to(torch.bfloat16)
    x[3] = 0
    sm = (torch.rand(256, generator=g) + 0.5).to(torch.bfloat16)
    for smooth in (None, sm):
        y, s = golden.dynamic_quant_int4(_bits(x), smooth_u16=None if smooth is None else _bits(smooth))
        xf = x.float() if smooth is None else x.float() * smooth.float()
        scale = xf.abs().amax(-1) / 7.0
        assert np.array_equal(s, scale.numpy())
        want = torch.where(scale[:, None] > 0, torch.round(xf / scale[:, None]), torch.zeros(())).to(torch.int8).numpy()
        assert np.array_equal(golden.unpack_int4(y), want) and want.min() == -7 and want.max() == 7


# ------------------------------------------------------------------ asymmetric variant

def _asym_numpy(xf):
    """scale = (max - min) / 255, offset = 127 - max / scale, y = rint(x / scale + offset) in numpy float32, one
    operation at a time (numpy rounds every float32 operation separately; rint is half-even)."""
    xf = xf.astype(np.float32)
    mx, mn = xf.max(axis=-1, keepdims=True), xf.min(axis=-1, keepdims=True)
    scale = ((mx - mn) / np.float32(255.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        offset = (np.float32(127.0) - (mx / scale).astype(np.float32)).astype(np.float32)
        q = np.rint(((xf / scale).astype(np.float32) + offset).astype(np.float32))
    y = np.clip(q, -128, 127)
    flat = ~(mx > mn)
    y = np.where(flat, 0, y).astype(np.int8)
    scale, offset = np.where(flat, 0, scale), np.where(flat, 0, offset)
    return y, scale[..., 0].astype(np.float32), offset[..., 0].astype(np.float32)


@pytest.mark.parametrize("dtype", ["bf16", "fp16"])
def test_asymmetric_vs_numpy_float32(golden, dtype):
    g = torch.Generator().manual_seed(7)
    tdt = torch.bfloat16 if dtype == "bf16" else torch.float16
    for rows, cols, mul, shift in [(33, 1000, 1.0, 0.0), (8, 4096, 30.0, 5.0), (5, 24, 0.25, -2.0), (3, 1, 1.0, 0.0)]:
        x = (torch.randn(rows, cols, generator=g) * mul + shift).to(tdt)
        bits = x.view(torch.int16).numpy().view(np.uint16)
        y, s, o = golden.dynamic_quant_asymmetric(bits, dtype)
        wy, ws, wo = _asym_numpy(x.float().numpy())
        assert np.array_equal(s.view(np.uint32), ws.view(np.uint32)) and np.array_equal(o.view(np.uint32), wo.view(np.uint32))
        assert np.array_equal(y, wy)
        if cols > 1:                                     # the extremes of a row land on the ends of the int8 range
            xf = x.float().numpy()
            assert (y[np.arange(rows), xf.argmax(axis=1)] == 127).all() and (y[np.arange(rows), xf.argmin(axis=1)] == -128).all()
    sm = (torch.rand(1000, generator=g) + 0.5).to(tdt)
    x = torch.randn(7, 1000, generator=g).to(tdt)
    y, s, o = golden.dynamic_quant_asymmetric(x.view(torch.int16).numpy().view(np.uint16), dtype, sm.view(torch.int16).numpy().view(np.uint16))
    wy, ws, wo = _asym_numpy((x.float() * sm.float()).numpy())
    assert np.array_equal(y, wy) and np.array_equal(s, ws) and np.array_equal(o, wo)


def test_asymmetric_hand_computed_rows(golden):
    """Rows whose answers can be written down: [0 .. 255] has scale 1 and offset -128 (y = x - 128); [-1, 0, 1] has
    scale 2/255; [-255, 0, 255, ...] has scale 2 and offset -0.5 exactly, so 0, 1 and -2 land on ties and round to
    even; a constant row gives zeros."""
    x = torch.arange(256, dtype=torch.float32).to(torch.bfloat16).reshape(1, 256)
    assert torch.equal(x.float(), torch.arange(256, dtype=torch.float32).reshape(1, 256))     # exact in bf16
    y, s, o = golden.dynamic_quant_asymmetric(x.view(torch.int16).numpy().view(np.uint16))
    assert s[0] == 1.0 and o[0] == -128.0 and np.array_equal(y[0].astype(np.int32), np.arange(256) - 128)
    x = torch.tensor([[-1.0, 0.0, 1.0, 0.5]], dtype=torch.float16)
    y, s, o = golden.dynamic_quant_asymmetric(x.view(torch.int16).numpy().view(np.uint16), "fp16")
    assert s[0] == np.float32(2.0) / np.float32(255.0) and abs(o[0] + 0.5) < 1e-4     # 1 / fl(2/255) is not exactly 127.5
    assert y[0].tolist() == [-128, 0, 127, 63]           # 0 -> -0.49999 -> 0;  0.5 / scale + offset = 63.25
    x = torch.tensor([[-255.0, 0.0, 255.0, 1.0, 3.0, -2.0]], dtype=torch.bfloat16)   # scale 2, offset -0.5 exactly
    y, s, o = golden.dynamic_quant_asymmetric(x.view(torch.int16).numpy().view(np.uint16))
    assert s[0] == 2.0 and o[0] == -0.5
    assert y[0].tolist() == [-128, 0, 127, 0, 1, -2]     # ties -0.5 -> -0, 0.0 -> 0, 1.0, -1.5 -> -2: half to even
    x = torch.full((2, 16), 3.5, dtype=torch.bfloat16)
    y, s, o = golden.dynamic_quant_asymmetric(x.view(torch.int16).numpy().view(np.uint16))
    assert not y.any() and not s.any() and not o.any()
