"""Oracle of npu_quantize against what the mathematics fixes (CPU only)."""
import numpy as np
import torch

from oracle import golden


def test_matches_torch_quantize_per_channel_for_power_of_two_scales():
    # torch evaluates nearbyint(x * (1 / scale)) + zero_point; with power-of-two scales the reciprocal is exact and
    # with integer zero points nearbyint(v) + z == nearbyint(v + z) unless v + z rounds in float32 (|v| < 2^15 here)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 16, 5, generator=g) * 40
    scales = torch.tensor([2.0 ** (i % 5 - 3) for i in range(16)])
    zps = torch.arange(16, dtype=torch.int32) - 8
    zps = zps - zps % 2                                    # even: adding them keeps ties on ties to even
    q = torch.quantize_per_channel(x, scales, zps, axis=1, dtype=torch.qint8).int_repr().numpy()
    got = golden.quantize(x.numpy(), scales.numpy(), zps.float().numpy(), "int8", axis=1)
    assert np.array_equal(got, q)
    qu = torch.quantize_per_tensor(x, 0.25, 128, torch.quint8).int_repr().numpy()
    gotu = golden.quantize(x.numpy(), np.float32([0.25]), np.float32([128]), "uint8", axis=-1)
    assert np.array_equal(gotu, qu)


def test_hand_computed_values():
    x = np.float32([[0.5, 1.5, 2.5, -0.5, -1.5, 300.0, -300.0, np.nan]])
    one = np.float32([1.0])
    assert golden.quantize(x, one, None, "int8").tolist() == [[0, 2, 2, 0, -2, 127, -128, 0]]      # ties to even, clamp
    assert golden.quantize(x, one, None, "uint8").tolist() == [[0, 2, 2, 0, 0, 255, 0, 0]]
    assert golden.quantize(x, one, np.float32([1.0]), "int8").tolist() == [[2, 2, 4, 0, 0, 127, -128, 0]]  # rint(x + 1)
    # multiply mode and a per-channel axis in the middle
    y = np.float32([[[1.0, 2.0], [3.0, 4.0]]])                       # [1, 2, 2], axis 1
    got = golden.quantize(y, np.float32([2.0, 0.5]), np.float32([0.0, 10.0]), "int32", axis=1, div_mode=False)
    assert got.tolist() == [[[2, 4], [12, 12]]]                      # 3 * 0.5 + 10 = 11.5 -> 12, 4 * 0.5 + 10 = 12
    big = np.float32([[3e9, -3e9]])
    assert golden.quantize(big, one, None, "int32").tolist() == [[2 ** 31 - 1, -2 ** 31]]


def test_division_is_float32_division():
    # x / s in float32 differs from x * (1 / s) for some operands; the oracle divides
    x = np.float32([[5.0, 7.0, 9.0, 11.0]]) * np.float32(1.7)
    s = np.float32([3.0])
    got = golden.quantize(x * 1000, s, None, "int32")
    want = np.rint((x * 1000 / s).astype(np.float32)).astype(np.int32)
    assert np.array_equal(got, want)
