"""Pins oracle.unpack_int4 / antiquant / weight_quant_matmul / swiglu against the in-tree goldens
of the reference (test/custom_ops/test_npu_anti_quant.py:12-42,
test/contrib/test_linear_weight_quant.py:20-28) evaluated with torch / numpy, hand-typed
known answers and special cases that reduce to library routines."""
import numpy as np
import pytest
import torch

from pytorch_amd.testing import workloads, rtol_failures


def _bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_unpack_int4_known_answers(golden):
    words = np.array([0x76543210, np.int32(np.uint32(0xFEDCBA98).astype(np.int64) - 2 ** 32), 0x0000000F,
                      np.int32(-2 ** 31)], dtype=np.int32)
    got = golden.unpack_int4(words.reshape(1, 4))
    assert got.tolist() == [[0, 1, 2, 3, 4, 5, 6, 7, -8, -7, -6, -5, -4, -3, -2, -1,
                             -1, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, -8]]


def test_unpack_int4_byte_order_restatement(golden):
    """Same order as reading the int32 words as little-endian bytes and taking the low nibble
    of each byte first (test/custom_ops/test_npu_anti_quant.py:18-23)."""
    g = np.random.default_rng(0)
    words = g.integers(-2 ** 31, 2 ** 31, (6, 25), dtype=np.int64).astype(np.int32)
    by = np.frombuffer(words.tobytes(), dtype=np.uint8)
    nib = (by.reshape(-1, 1) >> np.array([0, 4], dtype=np.uint8)) & 0xF
    want = ((nib.astype(np.int16) ^ 8) - 8).astype(np.int8).reshape(6, 200)
    assert np.array_equal(golden.unpack_int4(words), want)
    assert np.array_equal(golden.pack_int4(want), words)
    w4 = torch.from_numpy(want)
    assert np.array_equal(workloads.pack_int4(w4).numpy(), words)


def test_antiquant_known_answers_and_torch(golden):
    w = np.array([[-128, -1, 0, 127]], np.int8)
    s = np.array([0.5, 2.0, 3.0, 0.25], np.float32)
    o = np.array([1.0, 1.0, -2.0, 1.0], np.float32)
    assert golden.antiquant(w, s, o).tolist() == [[-63.5, 0.0, -6.0, 32.0]]
    assert golden.antiquant(w, s).tolist() == [[-64.0, -2.0, 0.0, 31.75]]
    g = torch.Generator().manual_seed(0)
    wt = torch.randint(-127, 128, (10, 100), generator=g, dtype=torch.int8)
    st = torch.rand(100, generator=g) * 200 - 100
    ot = torch.rand(100, generator=g) * 200 - 100
    want = (wt.float() + ot) * st
    assert np.array_equal(golden.antiquant(wt.numpy(), st.numpy(), ot.numpy()), want.numpy())


def _torch_golden(x, w_f32, scale, offset, group_size):
    """cpu_linear_weight_quant of test/contrib/test_linear_weight_quant.py:20-28 in float32."""
    K, N = w_f32.shape
    if group_size:
        scale = scale.float().repeat_interleave(group_size, 0)
        offset = None if offset is None else offset.float().repeat_interleave(group_size, 0)
    else:
        scale = scale.float()[None, :]
        offset = None if offset is None else offset.float()[None, :]
    wf = w_f32 if offset is None else w_f32 + offset
    wf = wf * scale
    return x.float() @ wf, x.double() @ wf.double()


@pytest.mark.parametrize("weight_nk", [False, True])
def test_w8a16_vs_torch(golden, weight_nk):
    d = workloads.w8a16_inputs(seed=0, M=16, K=2048, N=256, weight_nk=weight_nk)
    out, outf = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                           _bits(d["antiquant_offset"]))
    t32, t64 = _torch_golden(d["x"], d["weight"].float(), d["antiquant_scale"], d["antiquant_offset"], 0)
    _, out64 = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                          _bits(d["antiquant_offset"]), accum="f64")
    # float64 accumulation over identical float32 weights: equal up to the final float32 rounding
    np.testing.assert_allclose(out64, t64.numpy(), rtol=2e-7, atol=1e-6)
    # float32 accumulation order differs between the oracle (k ascending) and torch's blocked GEMM
    np.testing.assert_allclose(outf, t32.numpy(), rtol=2e-5, atol=2e-3)
    dist = golden.bf16_ulp_distance(out, _bits(t32.to(torch.bfloat16)))
    assert dist.max() <= 1 and (dist == 0).mean() > 0.99


@pytest.mark.parametrize("M", [1, 8])
def test_w4a16_vs_torch(golden, M):
    d = workloads.w4a16_inputs(seed=1, M=M, K=1024, N=256, group_size=128)
    out, outf = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                           _bits(d["antiquant_offset"]), group_size=128)
    t32, t64 = _torch_golden(d["x"], d["weight_int4_values"].float(), d["antiquant_scale"],
                             d["antiquant_offset"], 128)
    np.testing.assert_allclose(outf, t32.numpy(), rtol=2e-5, atol=1e-3)
    _, out64 = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                          _bits(d["antiquant_offset"]), group_size=128, accum="f64")
    np.testing.assert_allclose(out64, t64.numpy(), rtol=2e-7, atol=1e-6)
    assert golden.bf16_ulp_distance(out, _bits(t32.to(torch.bfloat16))).max() <= 1


def test_special_cases(golden):
    g = torch.Generator().manual_seed(4)
    K, N, M = 256, 64, 4
    x = torch.randint(-8, 9, (M, K), generator=g).to(torch.bfloat16)      # small integers: sums are exact
    w = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8)
    one = torch.ones(N, dtype=torch.bfloat16)
    # offset absent, scale 1 -> plain integer matmul, exact in float32
    _, outf = golden.weight_quant_matmul(_bits(x), w.numpy(), _bits(one))
    assert np.array_equal(outf, (x.double() @ w.double()).float().numpy())
    # group_size = K equals per channel
    s = (torch.rand(N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
    o = (torch.rand(N, generator=g) * 8 - 4).to(torch.bfloat16)
    a = golden.weight_quant_matmul(_bits(x), w.numpy(), _bits(s), _bits(o))[1]
    b = golden.weight_quant_matmul(_bits(x), w.numpy(), _bits(s[None]), _bits(o[None]), group_size=K)[1]
    assert np.array_equal(a, b)
    # int4 path on the same values as an int8 weight restricted to [-8, 7]
    w4 = torch.randint(-8, 8, (K, N), generator=g, dtype=torch.int8)
    a = golden.weight_quant_matmul(_bits(x), w4.numpy(), _bits(s), _bits(o))[1]
    b = golden.weight_quant_matmul(_bits(x), workloads.pack_int4(w4).numpy(), _bits(s[None]), _bits(o[None]),
                                   group_size=K)[1]
    assert np.array_equal(a, b)
    # M = 1 row equals row 0 of the batched call
    c = golden.weight_quant_matmul(_bits(x[:1]), w4.numpy(), _bits(s), _bits(o))[1]
    assert np.array_equal(c[0], a[0])


def test_swiglu_vs_torch_cpu_bf16(golden):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(32, 512, generator=g) * 3).to(torch.bfloat16)
    a, b = x.chunk(2, -1)
    want = torch.nn.functional.silu(a) * b
    got = golden.swiglu(_bits(x))
    dist = golden.bf16_ulp_distance(got, _bits(want))
    # libm expf vs torch's vectorised exp may differ in the last float32 bit
    assert dist.max() <= 1 and (dist == 0).mean() > 0.995
    z = torch.tensor([[0.0, 1.0, -1.0, 2.0, 1.0, 1.0]], dtype=torch.bfloat16)
    out = golden.bf16_bits_to_f32(golden.swiglu(_bits(z)))[0]
    assert out[0] == 0.0 and abs(out[1] - 0.7311) < 4e-3 and abs(out[2] + 0.2689) < 2e-3


def test_float16_variant_follows_the_reference_test_recipe(golden):
    """The float16 statement of the golden against the recipe of test/contrib/test_linear_weight_quant.py:20-28 typed
    independently in torch: that recipe rounds (w + offset) and (. * scale) to float16 before the float32 matmul, the
    oracle keeps them in float32, and the reference accepts 1e-2 between the two."""
    g = torch.Generator().manual_seed(4)
    M, K, N = 24, 512, 96
    x = torch.randn(M, K, generator=g).to(torch.float16)
    w = torch.randn(N, K, generator=g).mul(40).to(torch.int8)                  # stored [N, K] like the module's weight
    scale = (torch.rand(N, generator=g) * 9e-3 + 1e-3).to(torch.float16)
    off = (torch.rand(N, generator=g) * 8 - 4).to(torch.float16)
    wt = w.to(torch.float16).t()                                               # [K, N] view, as the test passes it
    want = torch.matmul(x.float(), ((wt + off) * scale).float())               # the in-tree recipe, float16 intermediates
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)
    out, outf = golden.weight_quant_matmul(bits(x), w.t().numpy(), bits(scale), bits(off), dtype="fp16")
    got = torch.from_numpy(out.view(np.float16).astype(np.float32))
    assert rtol_failures(got, want.to(torch.float16).float(), 1e-2) == 0
    # and exactly the float32-intermediate evaluation, computed in float64
    ref = x.double() @ ((wt.double() + off.double()).float() * scale.float()).double()
    assert np.allclose(outf, ref.numpy(), rtol=2e-5, atol=1e-5)
    assert np.array_equal(out, torch.from_numpy(outf).to(torch.float16).view(torch.int16).numpy().view(np.uint16))


@pytest.mark.parametrize("dst", ["fp16", "bf16"])
def test_anti_quant_matches_the_in_tree_golden(golden, dst):
    """npu_anti_quant as the reference's own CPU golden evaluates it (test/custom_ops/test_npu_anti_quant.py:29-42,
    inputs of :49-66): x.to(float32) + offset, times scale, then .to(dst_dtype), with torch on the CPU; int32 inputs are
    unpacked with the numpy recipe of :12-24 first."""
    tdst = torch.float16 if dst == "fp16" else torch.bfloat16
    g = torch.Generator().manual_seed(0)
    for packed in (False, True):
        if packed:
            words = torch.randint(-2 ** 31, 2 ** 31 - 1, (10, 25), generator=g, dtype=torch.int64).to(torch.int32)
            by = np.frombuffer(words.numpy().tobytes(), dtype=np.uint8)
            nib = (by.reshape(-1, 1) >> np.array([0, 4], dtype=np.uint8)) & 0xF
            vals = torch.from_numpy(((nib.astype(np.int16) ^ 8) - 8).astype(np.int8).reshape(10, 200))
            x = words
        else:
            vals = torch.randint(-127, 128, (10, 100), generator=g, dtype=torch.int8)
            x = vals
        n = vals.shape[1]
        scale = (torch.rand(n, generator=g) * 200 - 100)
        offset = (torch.rand(n, generator=g) * 200 - 100)
        for off in (offset, None):
            want = ((vals.to(torch.float32) + (off if off is not None else 0.0)) * scale).to(tdst)
            got = golden.anti_quant(x.numpy(), scale.numpy(), None if off is None else off.numpy(), dst=dst)
            assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16))
    # a single scale / offset broadcasts
    vals = torch.randint(-127, 128, (3, 16), generator=g, dtype=torch.int8)
    want = ((vals.float() + 1.5) * 0.25).to(tdst)
    got = golden.anti_quant(vals.numpy(), np.array([0.25], np.float32), np.array([1.5], np.float32), dst=dst)
    assert np.array_equal(got, want.view(torch.int16).numpy().view(np.uint16))
