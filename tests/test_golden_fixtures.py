"""Golden fixtures of tests/golden: hand-typed known answers and frozen seeded problems.
CPU part: the oracle reproduces them.  GPU part: the HIP kernels, through the C ABI, reproduce them."""
import json
import os

import numpy as np
import pytest
import torch

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
KAT = json.load(open(os.path.join(HERE, "known_answers.json")))


def _npz(name):
    return np.load(os.path.join(HERE, name), allow_pickle=False)


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _bf16(u16):
    return torch.from_numpy(np.ascontiguousarray(u16).view(np.int16).copy()).view(torch.bfloat16)


# ------------------------------------------------------------------ CPU: oracle vs fixtures

def test_oracle_known_answers(golden):
    for case in KAT["dynamic_quant"]:
        x = torch.tensor([case["x"]], dtype=torch.bfloat16)
        assert x.float().tolist()[0] == case["x"]
        y, s = golden.dynamic_quant(_bits(x))
        assert y[0].tolist() == case["y"] and float(s[0]) == case["scale"]
    for case in KAT["unpack_int4"]:
        assert golden.unpack_int4(np.array([[case["word"]]], np.int32))[0].tolist() == case["values"]
    for case in KAT["quant_matmul"]:
        bias = torch.tensor(case["bias"], dtype=torch.bfloat16)
        out, acc = golden.quant_matmul(np.array(case["x1"], np.int8), np.array(case["x2"], np.int8),
                                       np.array(case["scale"], np.float32), np.array(case["pertoken_scale"], np.float32),
                                       _bits(bias))
        assert acc.tolist() == case["acc"] and golden.bf16_bits_to_f32(out).tolist() == case["out"]
    for case in KAT["weight_quant"]:
        x = torch.tensor(case["x"], dtype=torch.bfloat16)
        out, _ = golden.weight_quant_matmul(_bits(x), np.array(case["w"], np.int8),
                                            _bits(torch.tensor(case["scale"], dtype=torch.bfloat16)),
                                            _bits(torch.tensor(case["offset"], dtype=torch.bfloat16)))
        assert golden.bf16_bits_to_f32(out).tolist() == case["out"]


def test_oracle_reproduces_frozen_fixtures(golden):
    f = _npz("dynamic_quant.npz")
    y, s = golden.dynamic_quant(f["x"])
    assert np.array_equal(y, f["y"]) and np.array_equal(s, f["scale"])
    f = _npz("quant_matmul.npz")
    out, acc = golden.quant_matmul(f["x1"], f["x2"], f["scale"], f["pertoken_scale"], f["bias"])
    assert np.array_equal(acc, f["acc"]) and np.array_equal(out, f["out"])
    f = _npz("w8a16.npz")
    out, outf = golden.weight_quant_matmul(f["x"], f["weight"], f["scale"], f["offset"])
    assert np.array_equal(out, f["out"]) and np.array_equal(outf, f["out_f32"])
    f = _npz("w4a16.npz")
    out, outf = golden.weight_quant_matmul(f["x"], f["weight"], f["scale"], f["offset"], group_size=128)
    assert np.array_equal(out, f["out"]) and np.array_equal(outf, f["out_f32"])
    f = _npz("swiglu.npz")
    assert np.array_equal(golden.swiglu(f["x"]), f["out"])


# ------------------------------------------------------------------ GPU: kernels vs fixtures

@pytest.fixture(scope="module")
def capi():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pytorch_amd import _capi
    return _capi


@pytest.mark.gpu
def test_gpu_known_answers(capi):
    for case in KAT["dynamic_quant"]:
        x = torch.tensor([case["x"]], dtype=torch.bfloat16).cuda()
        y, s = capi.dynamic_quant(x)
        assert y[0].cpu().tolist() == case["y"] and float(s[0]) == case["scale"]
    for case in KAT["quant_matmul"]:
        x1 = torch.tensor(case["x1"], dtype=torch.int8).cuda()
        x2 = torch.tensor(case["x2"], dtype=torch.int8).cuda()
        acc = capi.quant_matmul(x1, x2, None, out_dtype=torch.int32)
        assert acc.cpu().tolist() == case["acc"]
        out = capi.quant_matmul(x1, x2, torch.tensor(case["scale"]).cuda(), torch.tensor(case["pertoken_scale"]).cuda(),
                                torch.tensor(case["bias"], dtype=torch.bfloat16).cuda())
        assert out.float().cpu().tolist() == case["out"]
    for case in KAT["weight_quant"]:
        out = capi.weight_quant_matmul(torch.tensor(case["x"], dtype=torch.bfloat16).cuda(),
                                       torch.tensor(case["w"], dtype=torch.int8).cuda(),
                                       torch.tensor(case["scale"], dtype=torch.bfloat16).cuda(),
                                       torch.tensor(case["offset"], dtype=torch.bfloat16).cuda())
        assert out.float().cpu().tolist() == case["out"]


@pytest.mark.gpu
def test_gpu_reproduces_frozen_fixtures(capi):
    from pytorch_amd.testing import bf16_gate
    f = _npz("dynamic_quant.npz")
    y, s = capi.dynamic_quant(_bf16(f["x"]).cuda())
    assert np.array_equal(y.cpu().numpy(), f["y"]) and np.array_equal(s.cpu().numpy(), f["scale"])
    f = _npz("quant_matmul.npz")
    x1, x2 = torch.from_numpy(f["x1"]).cuda(), torch.from_numpy(f["x2"]).cuda()
    assert np.array_equal(capi.quant_matmul(x1, x2, None, out_dtype=torch.int32).cpu().numpy(), f["acc"])
    out = capi.quant_matmul(x1, x2, torch.from_numpy(f["scale"]).cuda(), torch.from_numpy(f["pertoken_scale"]).cuda(),
                            _bf16(f["bias"]).cuda())
    assert np.array_equal(_bits(out), f["out"])
    for name, gs in (("w8a16.npz", 0), ("w4a16.npz", 128)):
        f = _npz(name)
        out = capi.weight_quant_matmul(_bf16(f["x"]).cuda(), torch.from_numpy(f["weight"]).cuda(), _bf16(f["scale"]).cuda(),
                                       _bf16(f["offset"]).cuda(), gs)
        bf16_gate(out, torch.from_numpy(f["out_f32"]))
    f = _npz("swiglu.npz")
    out = capi.swiglu(_bf16(f["x"]).cuda())
    d = np.abs(_bits(out).astype(np.int32) - f["out"].astype(np.int32))
    assert d.max() <= 1


def test_oracle_reproduces_later_fixtures(golden):
    f = _npz("anti_quant.npz")
    assert np.array_equal(golden.anti_quant(f["x"], f["scale"], f["offset"], dst="fp16"), f["out_fp16"])
    assert np.array_equal(golden.anti_quant(f["x"], f["scale"], f["offset"], dst="bf16"), f["out_bf16"])
    f = _npz("a4w4.npz")
    out, acc = golden.quant_matmul_a4w4(f["x1"], f["x2_n"], f["scale"], None, f["bias"], out="fp16")
    assert np.array_equal(out, f["out_n"]) and np.array_equal(acc, f["acc_n"])
    out, acc = golden.quant_matmul_a4w4(f["x1"], f["x2_k"].T, f["scale"], None, f["bias"], out="fp16")
    assert np.array_equal(out, f["out_k"]) and np.array_equal(acc, f["acc_k"])
    f = _npz("dynamic_quant_asymmetric.npz")
    y, s, o = golden.dynamic_quant_asymmetric(f["x"], "bf16", f["smooth"])
    assert np.array_equal(y, f["y"]) and np.array_equal(s, f["scale"]) and np.array_equal(o, f["offset"])


@pytest.mark.gpu
def test_gpu_reproduces_later_fixtures(capi):
    import pytorch_amd as pa
    f = _npz("anti_quant.npz")
    x, sc, of = (torch.from_numpy(f[k]).cuda() for k in ("x", "scale", "offset"))
    assert np.array_equal(capi.anti_quant(x, sc, of, dst_dtype=torch.float16).cpu().view(torch.int16).numpy().view(np.uint16), f["out_fp16"])
    assert np.array_equal(_bits(capi.anti_quant(x, sc, of, dst_dtype=torch.bfloat16)), f["out_bf16"])
    f = _npz("a4w4.npz")
    x1, scale, bias = (torch.from_numpy(f[k]).cuda() for k in ("x1", "scale", "bias"))
    for x2, tag in ((torch.from_numpy(f["x2_n"]).cuda(), "n"), (torch.from_numpy(f["x2_k"]).cuda().t(), "k")):
        out = pa.npu_quant_matmul(x1, x2, scale, bias=bias, output_dtype=torch.float16)
        assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), f["out_" + tag])
        assert np.array_equal(pa.npu_quant_matmul(x1, x2, scale, output_dtype=torch.int32).cpu().numpy(),
                              f["acc_" + tag])
    f = _npz("dynamic_quant_asymmetric.npz")
    y, s, o = capi.dynamic_quant_asymmetric(_bf16(f["x"]).cuda(), _bf16(f["smooth"]).cuda())
    assert np.array_equal(y.cpu().numpy(), f["y"]) and np.array_equal(s.cpu().numpy(), f["scale"])
    assert np.array_equal(o.cpu().numpy(), f["offset"])


def test_oracle_reproduces_quantize_fixtures(golden):
    f = _npz("quantize.npz")
    xf = _bf16(f["x"]).float().numpy()
    zp = f["zero_point"].astype(np.float32)
    assert np.array_equal(golden.quantize(xf, f["scale"], zp, "int8", 1, True), f["q_div_i8"])
    assert np.array_equal(golden.quantize(xf, f["scale"], zp, "uint8", 1, False), f["q_mul_u8"])
    f = _npz("quant_matmul_int8.npz")
    assert np.array_equal(golden.trans_quant_param(f["scale"], f["offset"]), f["qparam"])
    assert np.array_equal(golden.quant_matmul_requant(f["x1"], f["x2"], f["qparam"], f["bias"]), f["out"])


@pytest.mark.gpu
def test_gpu_reproduces_quantize_fixtures(capi):
    import pytorch_amd as pa
    f = _npz("quantize.npz")
    x, sc, zp = _bf16(f["x"]).cuda(), torch.from_numpy(f["scale"]).cuda(), torch.from_numpy(f["zero_point"]).cuda()
    assert np.array_equal(pa.npu_quantize(x, sc, zp, torch.qint8, 1).cpu().numpy(), f["q_div_i8"])
    assert np.array_equal(pa.npu_quantize(x, sc, zp, torch.quint8, 1, False).cpu().numpy(), f["q_mul_u8"])
    f = _npz("quant_matmul_int8.npz")
    x1, x2, scale, offset, bias = (torch.from_numpy(f[k]).cuda() for k in ("x1", "x2", "scale", "offset", "bias"))
    qp = pa.npu_trans_quant_param(scale, offset)
    assert np.array_equal(qp.cpu().numpy(), f["qparam"])
    assert np.array_equal(pa.npu_quant_matmul(x1, x2, qp, bias=bias, output_dtype=torch.int8).cpu().numpy(), f["out"])
    assert np.array_equal(pa.npu_quant_matmul(x1, x2, scale, offset=offset, bias=bias).cpu().numpy(), f["out"])


# The one part of npu_trans_quant_param's result that the reference tree does hold: the offset is a signed 9-bit
# integer obtained by rounding (ties to even, numpy's round) and clipping to [-256, 255] -- the helper f32_2_s9 of
# test/contrib/test_linear_weight_quant.py:13-16.  Inputs and the values that helper yields, typed by hand:
_S9_IN = [0.0, 0.4, 0.5, 0.6, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49, -3.51, 127.0, 128.0, 254.5, 255.0, 255.4, 255.5, 256.0, 300.0,
          1e9, -255.5, -256.0, -256.5, -257.0, -300.0, -1e9, 7.0, -8.0]
_S9_OUT = [0, 0, 0, 1, 2, 2, 0, -2, -2, 3, -4, 127, 128, 254, 255, 255, 255, 255, 255,
           255, -256, -256, -256, -256, -256, -256, 7, -8]


def test_trans_quant_param_offset_field_follows_f32_2_s9(golden):
    """Pins the offset field of the packed parameter (rounding and range; the bit positions stay unpinned): decoding the
    oracle's words gives f32_2_s9 of the offsets, and the field occupies nine bits."""
    off = np.array(_S9_IN, dtype=np.float32)
    want = np.array(_S9_OUT, dtype=np.float32)
    q = golden.trans_quant_param(np.full(off.size, 0.5, dtype=np.float32), off)
    scale, got = golden.quant_param_decode(q)
    assert np.array_equal(got, want)
    assert np.array_equal(scale, np.full(off.size, 0.5, dtype=np.float32))
    # a second scale does not disturb the field, and without an offset the field is zero
    assert np.array_equal(golden.quant_param_decode(golden.trans_quant_param(np.full(off.size, 3e-4, dtype=np.float32), off))[1], want)
    assert np.array_equal(golden.quant_param_decode(golden.trans_quant_param(np.float32([0.5, 2.0])))[1], np.float32([0, 0]))
    # nine bits: the extremes differ from each other only inside a 9-bit window
    lo, hi = golden.trans_quant_param(np.float32([1.0]), np.float32([-256.0])), golden.trans_quant_param(np.float32([1.0]), np.float32([255.0]))
    diff = int(lo.view(np.uint64)[0] ^ hi.view(np.uint64)[0])
    assert diff != 0 and (diff >> (diff.bit_length() - 9)) == 0x1FF and diff.bit_length() - 9 == (diff & -diff).bit_length() - 1


def test_weight_quant_requant_hand_computed(golden):
    """The int8 output of npu_weight_quant_batchmatmul with quant_scale / quant_offset as the oracle states it, on values
    typed by hand: the offset goes through f32_2_s9 (0.4 -> 0, 300 -> 255, -300 -> -256, 2.5 -> 2), products and sums are
    rounded to float32, ties go to even, the result saturates at the int8 range."""
    import torch
    out = torch.tensor([[1.5, 2.5, -3.0, 100.0, -0.5, 7.0]], dtype=torch.bfloat16)
    bits = out.view(torch.int16).numpy().view(np.uint16)
    scale = np.float32([1.0, 1.0, 2.0, 1.0, 1.0, 0.5])
    off = np.float32([0.4, 300.0, -300.0, 2.5, 0.0, 0.0])
    #            1.5+0 -> 2   2.5+255 -> 127   -6-256 -> -128   100+2 -> 102   -0.5 -> -0   3.5 -> 4
    assert golden.weight_quant_requant(bits, scale, off).tolist() == [[2, 127, -128, 102, 0, 4]]
    assert golden.weight_quant_requant(bits, scale, None).tolist() == [[2, 2, -6, 100, 0, 4]]
    h = out.to(torch.float16).view(torch.int16).numpy().view(np.uint16)
    assert golden.weight_quant_requant(h, scale, off, dtype="fp16").tolist() == [[2, 127, -128, 102, 0, 4]]


@pytest.mark.gpu
def test_gpu_trans_quant_param_offset_field_follows_f32_2_s9(capi, golden):
    off = torch.tensor(_S9_IN, dtype=torch.float32)
    qp = capi.trans_quant_param(torch.full((off.numel(),), 0.5).cuda(), off.cuda()).cpu().numpy()
    assert np.array_equal(golden.quant_param_decode(qp)[1], np.array(_S9_OUT, dtype=np.float32))
