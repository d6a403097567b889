"""Pins oracle.int8_gemm / quant_matmul_epilogue: library routine (torch._int_mm), float64
matmul (exact below 2^53), closed forms, and elementwise float32 evaluation in torch."""
import numpy as np
import pytest
import torch

from pytorch_amd.testing import workloads


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("weight_nk", [False, True])
def test_accumulator_vs_int_mm_and_float64(golden, weight_nk):
    d = workloads.quant_matmul_inputs(seed=1, M=48, K=512, N=96, weight_nk=weight_nk)
    a, b = d["x1"], d["x2"]
    acc = golden.int8_gemm(a.numpy(), b.numpy())
    ref64 = a.double().numpy() @ b.double().numpy()
    assert np.array_equal(acc.astype(np.float64), ref64)
    im = torch._int_mm(torch.cat([a, a[:16]]).contiguous()[:64], b.contiguous()).numpy()[:48]
    assert np.array_equal(acc, im)


def test_accumulator_closed_forms(golden):
    K, M, N = 4096, 3, 5
    a = np.full((M, K), 127, np.int8)
    b = np.full((K, N), 127, np.int8)
    assert (golden.int8_gemm(a, b) == K * 16129).all()
    b2 = np.full((K, N), -127, np.int8)
    assert (golden.int8_gemm(a, b2) == -K * 16129).all()
    # K = 1: outer product
    u = np.arange(-4, 4, dtype=np.int8).reshape(8, 1)
    v = np.arange(-3, 5, dtype=np.int8).reshape(1, 8)
    assert np.array_equal(golden.int8_gemm(u, v), u.astype(np.int32) * v.astype(np.int32))
    # permutation matrix picks columns
    eye = np.eye(16, dtype=np.int8)[:, ::-1].copy()
    x = np.arange(-64, 64, dtype=np.int8).reshape(8, 16)
    assert np.array_equal(golden.int8_gemm(x, eye), x[:, ::-1].astype(np.int32))


def test_accumulator_triple_loop(golden):
    g = np.random.default_rng(0)
    a = g.integers(-127, 128, (5, 7), dtype=np.int8)
    b = g.integers(-127, 128, (7, 3), dtype=np.int8)
    want = [[sum(int(a[m, k]) * int(b[k, n]) for k in range(7)) for n in range(3)] for m in range(5)]
    assert golden.int8_gemm(a, b).tolist() == want


@pytest.mark.parametrize("bias", [False, True])
def test_epilogue_vs_torch_float32(golden, bias):
    d = workloads.quant_matmul_inputs(seed=2, M=32, K=256, N=64, bias=bias)
    out, acc = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(),
                                   d["pertoken_scale"].numpy(), None if not bias else _bits(d["bias"]))
    f = torch.from_numpy(acc).float() * d["pertoken_scale"][:, None]
    f = f * d["scale"][None, :]
    if bias:
        f = f + d["bias"].float()[None, :]
    assert np.array_equal(out, _bits(f.to(torch.bfloat16)))


def test_epilogue_special_cases(golden):
    # unit scales, no bias: out = bf16(float32(acc)); includes |acc| > 2^24 where int->float rounds
    acc = np.array([[0, 1, -1, 255, 256, 257, 16777217, -16777219, 66064384, 2 ** 31 - 1, -2 ** 31]], np.int32)
    out = golden.quant_matmul_epilogue(acc, np.ones(acc.shape[1], np.float32), np.ones(1, np.float32))
    want = torch.from_numpy(acc).to(torch.float32).to(torch.bfloat16)
    assert np.array_equal(out, _bits(want))
    assert golden.bf16_bits_to_f32(out)[0, :6].tolist() == [0.0, 1.0, -1.0, 255.0, 256.0, 256.0]
    # per-tensor scale broadcast and missing per-token scale
    out2 = golden.quant_matmul_epilogue(acc[:, :6], np.array([0.5], np.float32))
    assert golden.bf16_bits_to_f32(out2)[0].tolist() == [0.0, 0.5, -0.5, 127.5, 128.0, 128.0]  # 128.5 ties to even


def test_epilogue_operation_order_is_left_to_right(golden):
    # (f*ps)*s differs from f*(ps*s) for some inputs; the oracle must follow the former
    g = torch.Generator().manual_seed(7)
    acc = torch.randint(-2_000_000, 2_000_000, (64, 512), generator=g, dtype=torch.int32)
    ps = torch.rand(64, generator=g) * 9e-3 + 1e-3
    s = torch.rand(512, generator=g) * 9e-3 + 1e-3
    a = (acc.float() * ps[:, None]) * s[None, :]
    b = acc.float() * (ps[:, None] * s[None, :])
    assert (a != b).any()
    out = golden.quant_matmul_epilogue(acc.numpy(), s.numpy(), ps.numpy())
    assert np.array_equal(out, _bits(a.to(torch.bfloat16)))
