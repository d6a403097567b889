"""Host-side tests that need no GPU: the C ABI library loads and exports what the header
declares, the torch operators are registered under torch_npu's names with its argument
layout, Meta (FakeTensor) shape inference matches the expectations of the reference's
test/test_fake_tensor.py:1670-1687,1883-1925, unsupported arguments raise instead of being
ignored, and the contrib modules marshal their arguments as the reference's do."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_abi_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "mi355_quant.h")).read()
    declared = set(re.findall(r"\b(mi355_[a-z0-9_]+)\s*\(", header))
    assert {"mi355_dynamic_quant", "mi355_quant_matmul", "mi355_weight_quant_matmul", "mi355_swiglu", "mi355_swiglu_quant", "mi355_anti_quant",
            "mi355_unpack_int4", "mi355_dynamic_quant_asymmetric", "mi355_quantize", "mi355_trans_quant_param", "mi355_workspace_status", "mi355_workspace_zero_bytes",
            "mi355_quant_matmul_qparam", "mi355_swiglu_quant_smooth"} <= declared
    lib = ctypes.CDLL(os.path.join(ROOT, "pytorch_amd", "csrc", "libmi355_quant.so"))
    for name in declared:
        assert hasattr(lib, name), name
    lib.mi355_status_string.restype = ctypes.c_char_p
    assert lib.mi355_status_string(0) == b"ok"
    assert lib.mi355_quant_abi_version() >= 2000
    from pytorch_amd import _capi
    assert set(_capi.EXPORTS) == declared


@pytest.fixture(scope="module")
def pa():
    import pytorch_amd
    return pytorch_amd


def test_operator_names_and_schemas(pa):
    assert set(pa.__all__) >= {"npu_dynamic_quant", "npu_quant_matmul", "npu_weight_quant_batchmatmul", "npu_swiglu",
                                "npu_swiglu_quant"}
    assert pa.npu_quant_matmul is torch.ops.npu.npu_quant_matmul
    s = str(torch.ops.npu.npu_dynamic_quant.default._schema)
    assert s.startswith("npu::npu_dynamic_quant(Tensor input, *, Tensor? smooth_scales=None, Tensor? group_index=None")
    s = str(torch.ops.npu.npu_quant_matmul.default._schema)
    assert "Tensor x1, Tensor x2, Tensor scale, *, Tensor? offset=None, Tensor? pertoken_scale=None, Tensor? bias=None" in s
    s = str(torch.ops.npu.npu_weight_quant_batchmatmul.default._schema)
    assert ("Tensor x, Tensor weight, Tensor antiquant_scale, Tensor? antiquant_offset=None, Tensor? quant_scale=None, "
            "Tensor? quant_offset=None, Tensor? bias=None, int antiquant_group_size=0, int inner_precise=0, *, "
            "ScalarType? weight_dtype=None") in s


def test_no_cpu_implementation(pa):
    with pytest.raises(NotImplementedError, match="CPU"):
        pa.npu_dynamic_quant(torch.zeros(4, 8, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError, match="CPU"):
        pa.npu_swiglu(torch.zeros(4, 8, dtype=torch.bfloat16))


def _m(*shape, dtype):
    return torch.empty(*shape, dtype=dtype, device="meta")


def test_meta_dynamic_quant(pa):
    # test/test_fake_tensor.py:1670-1687
    x = _m(4, 2048, 1024, dtype=torch.float16)
    sm = _m(1024, dtype=torch.float16)
    y, s = pa.npu_dynamic_quant(x, smooth_scales=sm)
    assert y.shape == (4, 2048, 1024) and y.dtype == torch.int8 and y.device == x.device
    assert s.shape == (4, 2048) and s.dtype == torch.float32
    y, s = pa.npu_dynamic_quant(_m(7, 64, dtype=torch.bfloat16), dst_type=torch.int8)
    assert y.shape == (7, 64) and s.shape == (7,)
    # per-expert smooth scales: smooth_scales [E, H] with group_index [E]
    y, s = pa.npu_dynamic_quant(x, smooth_scales=_m(4, 1024, dtype=torch.float16), group_index=_m(4, dtype=torch.int32))
    assert y.shape == (4, 2048, 1024) and s.shape == (4, 2048)
    with pytest.raises(RuntimeError, match="group_index needs smooth_scales"):
        pa.npu_dynamic_quant(x, group_index=_m(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="with group_index, smooth_scales must have shape"):
        pa.npu_dynamic_quant(x, smooth_scales=sm, group_index=_m(4, dtype=torch.int32))
    with pytest.raises(RuntimeError, match="group_index must be int32 or int64"):
        pa.npu_dynamic_quant(x, smooth_scales=_m(4, 1024, dtype=torch.float16), group_index=_m(4, dtype=torch.float32))
    # int4 codes: eight to an int32 word
    y, s = pa.npu_dynamic_quant(x, dst_type=torch.quint4x2)
    assert y.shape == (4, 2048, 128) and y.dtype == torch.int32 and s.shape == (4, 2048)
    with pytest.raises(RuntimeError, match="multiple of 8"):
        pa.npu_dynamic_quant(_m(4, 12, dtype=torch.float16), dst_type=torch.quint4x2)
    with pytest.raises(RuntimeError, match="dst_type must be"):
        pa.npu_dynamic_quant(x, dst_type=torch.uint8)
    with pytest.raises(RuntimeError, match="bfloat16 or float16"):
        pa.npu_dynamic_quant(_m(4, 8, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="smooth_scales"):
        pa.npu_dynamic_quant(x, smooth_scales=_m(8, dtype=torch.float16))


def test_meta_dynamic_quant_asymmetric(pa):
    # test/test_fake_tensor.py:1689-1709
    y, s, o = pa.npu_dynamic_quant_asymmetric(_m(4, 2048, 1024, dtype=torch.float16), smooth_scales=_m(1024, dtype=torch.float16))
    assert y.shape == (4, 2048, 1024) and y.dtype == torch.int8
    assert s.shape == (4, 2048) and s.dtype == torch.float32 and o.shape == (4, 2048) and o.dtype == torch.float32
    y, s, o = pa.npu_dynamic_quant_asymmetric(_m(64, 1024, dtype=torch.float16), smooth_scales=_m(3, 1024, dtype=torch.float16),
                                              group_index=_m(3, dtype=torch.int64))
    assert y.shape == (64, 1024) and s.shape == (64,) and o.shape == (64,)
    with pytest.raises(RuntimeError, match="dst_type must be torch.int8, got"):
        pa.npu_dynamic_quant_asymmetric(_m(64, 1024, dtype=torch.float16), dst_type=torch.quint4x2)


def test_meta_quant_matmul(pa):
    # shapes of test/test_fake_tensor.py:1883-1915 for the output types this build supports
    x1 = _m(1, 1, 1024, dtype=torch.int8)
    x2 = _m(1, 1024, 100, dtype=torch.int8)
    r = pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.bfloat16), offset=None, bias=_m(1, 1, 100, dtype=torch.bfloat16),
                            output_dtype=torch.bfloat16)
    assert r.shape == (1, 1, 100) and r.dtype == torch.bfloat16
    r = pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), output_dtype=torch.int32)
    assert r.shape == (1, 1, 100) and r.dtype == torch.int32
    r = pa.npu_quant_matmul(_m(5, 3, 16, 64, dtype=torch.int8), _m(3, 64, 32, dtype=torch.int8), _m(32, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    assert r.shape == (5, 3, 16, 32)
    r = pa.npu_quant_matmul(_m(16, 64, dtype=torch.int8), _m(32, 64, dtype=torch.int8).t(), _m(32, dtype=torch.float32),
                            pertoken_scale=_m(16, dtype=torch.float32), output_dtype=torch.bfloat16)
    assert r.shape == (16, 32)
    # unsupported variants raise, never silently ignored
    # output_dtype None is the re-quantised int8 output (test_fake_tensor.py:1886-1895), with a float32 or int64 scale
    r = pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), offset=_m(1, dtype=torch.float32))
    assert r.shape == (1, 1, 100) and r.dtype == torch.int8
    r = pa.npu_quant_matmul(x1, x2, _m(100, dtype=torch.int64), bias=_m(100, dtype=torch.int32), output_dtype=torch.int8)
    assert r.dtype == torch.int8
    r = pa.npu_quant_matmul(x1, x2, _m(100, dtype=torch.int64), output_dtype=torch.float16)
    assert r.dtype == torch.float16
    with pytest.raises(RuntimeError, match="pertoken_scale is not applicable to int8"):
        pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), pertoken_scale=_m(1, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="offset"):
        pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), offset=_m(1, dtype=torch.float32), output_dtype=torch.bfloat16)
    r = pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), bias=_m(100, dtype=torch.int32), output_dtype=torch.float16)
    assert r.shape == (1, 1, 100) and r.dtype == torch.float16          # test_fake_tensor.py:1903-1906
    with pytest.raises(RuntimeError, match="output_dtype must be"):
        pa.npu_quant_matmul(x1, x2, _m(1, dtype=torch.float32), output_dtype=torch.float32)
    # both operands packed int4: last dimension of x2 times 8 (test_fake_tensor.py:1917-1923), or the transposed
    # [N, K/8] weight of the module example (linear_quant.py:40-50)
    r = pa.npu_quant_matmul(_m(16, 8, dtype=torch.int32), _m(64, 5, dtype=torch.int32), _m(1, dtype=torch.float32),
                            offset=None, bias=_m(40, dtype=torch.int32), output_dtype=torch.float16)
    assert r.shape == (16, 40) and r.dtype == torch.float16
    r = pa.npu_quant_matmul(_m(1, 2, dtype=torch.int32), _m(128, 2, dtype=torch.int32).t(), _m(1, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    assert r.shape == (1, 128)
    with pytest.raises(RuntimeError, match="both be int8, or both int32"):
        pa.npu_quant_matmul(_m(16, 8, dtype=torch.int32), _m(64, 40, dtype=torch.int8), _m(1, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="int4 inner dimensions differ"):
        pa.npu_quant_matmul(_m(16, 8, dtype=torch.int32), _m(60, 5, dtype=torch.int32), _m(1, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="inner dimensions"):
        pa.npu_quant_matmul(_m(4, 8, dtype=torch.int8), _m(16, 4, dtype=torch.int8), _m(4, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="pertoken_scale must have shape"):
        pa.npu_quant_matmul(_m(4, 8, dtype=torch.int8), _m(8, 4, dtype=torch.int8), _m(4, dtype=torch.float32),
                            pertoken_scale=_m(3, dtype=torch.float32), output_dtype=torch.bfloat16)
    r = pa.npu_quant_matmul(_m(4, 8, dtype=torch.int8), _m(8, 4, dtype=torch.int8), _m(4, dtype=torch.float32),
                            bias=_m(4, dtype=torch.int32), output_dtype=torch.bfloat16)      # LinearQuant's bias dtype
    assert r.shape == (4, 4)
    with pytest.raises(RuntimeError, match="bias must be"):
        pa.npu_quant_matmul(_m(4, 8, dtype=torch.int8), _m(8, 4, dtype=torch.int8), _m(4, dtype=torch.float32),
                            bias=_m(4, dtype=torch.bfloat16), output_dtype=torch.float16)
    with pytest.raises(RuntimeError, match="bias must be int32"):
        pa.npu_quant_matmul(_m(4, 8, dtype=torch.int8), _m(8, 4, dtype=torch.int8), _m(4, dtype=torch.float32),
                            bias=_m(4, dtype=torch.float32), output_dtype=torch.int32)


def test_meta_weight_quant_batchmatmul(pa):
    x = _m(16, 8192, dtype=torch.bfloat16)
    w = _m(28672, 8192, dtype=torch.int8).t()
    s, o = _m(28672, dtype=torch.bfloat16), _m(28672, dtype=torch.bfloat16)
    assert pa.npu_weight_quant_batchmatmul(x, w, s, o).shape == (16, 28672)
    # int4: last dimension x 8 (test/test_fake_tensor.py:1917-1923 states the same rule for packed int32)
    w4 = _m(4096, 1792, dtype=torch.int32)
    sg, og = _m(32, 14336, dtype=torch.bfloat16), _m(32, 14336, dtype=torch.bfloat16)
    r = pa.npu_weight_quant_batchmatmul(_m(2, 4, 4096, dtype=torch.bfloat16), w4, sg, og, None, None, None, 128)
    assert r.shape == (2, 4, 14336) and r.dtype == torch.bfloat16
    # the module's int4 weight [N, K/8] arrives as the transposed view [K/8, N]: words along K (linear_weight_quant.py:71,106)
    w4k = _m(14336, 512, dtype=torch.int32).t()
    r = pa.npu_weight_quant_batchmatmul(_m(3, 4096, dtype=torch.bfloat16), w4k, _m(14336, 32, dtype=torch.bfloat16).t(),
                                        _m(14336, 32, dtype=torch.bfloat16).t(), None, None, None, 128)
    assert r.shape == (3, 14336)
    with pytest.raises(RuntimeError, match="inner dimensions differ"):
        pa.npu_weight_quant_batchmatmul(_m(3, 4096, dtype=torch.bfloat16), _m(500, 14336, dtype=torch.int32), sg, og, None, None,
                                        None, 128)
    xs = _m(1, 4096, dtype=torch.bfloat16)
    # quant_scale turns the output into int8 (float32 values, or the int64 words of npu_trans_quant_param)
    for qs in (_m(14336, dtype=torch.float32), _m(1, 14336, dtype=torch.int64), _m(1, dtype=torch.float32)):
        r = pa.npu_weight_quant_batchmatmul(xs, w4, sg, og, qs, None, None, 128)
        assert r.dtype == torch.int8 and r.shape == (1, 14336)
    r = pa.npu_weight_quant_batchmatmul(xs, w4, sg, og, _m(14336, dtype=torch.float32), _m(14336, dtype=torch.float32), None, 128)
    assert r.dtype == torch.int8
    r = pa.npu_weight_quant_batchmatmul(xs, w4, sg, og, antiquant_group_size=128, inner_precise=1)
    assert r.dtype == torch.bfloat16 and r.shape == (1, 14336)
    for kwargs, pat in [(dict(quant_offset=_m(14336, dtype=torch.float32)), "quant_offset needs quant_scale"),
                        (dict(quant_scale=_m(14336, dtype=torch.bfloat16)), "quant_scale must be float32"),
                        (dict(quant_scale=_m(100, dtype=torch.float32)), "quant_scale must have shape"),
                        (dict(quant_scale=_m(14336, dtype=torch.int64), quant_offset=_m(14336, dtype=torch.float32)),
                         "already holds the offset"),
                        (dict(bias=_m(14336, dtype=torch.float16)), "bias must have the dtype of x"),
                        (dict(inner_precise=2), "inner_precise must be 0 or 1"),
                        (dict(weight_dtype=torch.int8), "weight_dtype")]:
        with pytest.raises(RuntimeError, match=pat):
            pa.npu_weight_quant_batchmatmul(xs, w4, sg, og, antiquant_group_size=128, **kwargs)
    with pytest.raises(RuntimeError, match="antiquant_scale must have shape"):
        pa.npu_weight_quant_batchmatmul(xs, w4, _m(14336, dtype=torch.bfloat16), None, antiquant_group_size=128)
    with pytest.raises(RuntimeError, match="multiple of 32"):
        pa.npu_weight_quant_batchmatmul(xs, w4, sg, og, antiquant_group_size=100)
    with pytest.raises(RuntimeError, match="must have the dtype of x"):
        pa.npu_weight_quant_batchmatmul(_m(1, 4096, dtype=torch.float16), w4, sg, og, antiquant_group_size=128)
    r = pa.npu_weight_quant_batchmatmul(_m(1, 4096, dtype=torch.float16), w4, sg.to(torch.float16), og.to(torch.float16),
                                        antiquant_group_size=128)
    assert r.dtype == torch.float16 and r.shape == (1, 14336)          # float16 as in test_linear_weight_quant.py:57-62
    with pytest.raises(RuntimeError, match="x must be bfloat16 or float16"):
        pa.npu_weight_quant_batchmatmul(_m(1, 4096, dtype=torch.float32), w4, sg, og, antiquant_group_size=128)


def test_meta_swiglu_quant(pa):
    y, s = pa.npu_swiglu_quant(_m(64, 28672, dtype=torch.bfloat16), quant_mode=1)
    assert y.shape == (64, 14336) and y.dtype == torch.int8 and s.shape == (64,) and s.dtype == torch.float32
    y, s = pa.npu_swiglu_quant(_m(2, 3, 8, dtype=torch.bfloat16), activate_left=True, quant_mode=1)
    assert y.shape == (2, 3, 4) and s.shape == (2, 3)
    with pytest.raises(RuntimeError, match="quant_mode"):
        pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16))                      # static quantisation is not built
    y, s = pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), smooth_scales=_m(4, dtype=torch.bfloat16), quant_mode=1)
    assert y.shape == (4, 4) and s.shape == (4,)
    with pytest.raises(RuntimeError, match="smooth_scales must have shape"):       # per-expert scales need group_index
        pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), smooth_scales=_m(2, 4, dtype=torch.bfloat16), quant_mode=1)
    y, s = pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), smooth_scales=_m(2, 4, dtype=torch.bfloat16),
                               group_index=_m(2, dtype=torch.int64), quant_mode=1, group_list_type=1)
    assert y.shape == (4, 4) and s.shape == (4,)
    with pytest.raises(RuntimeError, match="group_index needs smooth_scales"):
        pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), group_index=_m(2, dtype=torch.int64), quant_mode=1)
    with pytest.raises(RuntimeError, match="group_list_type"):
        pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), quant_mode=1, group_list_type=2)
    with pytest.raises(RuntimeError, match="smooth_scales must be bfloat16"):
        pa.npu_swiglu_quant(_m(4, 8, dtype=torch.bfloat16), smooth_scales=_m(4, dtype=torch.float32), quant_mode=1)


def test_meta_anti_quant(pa):
    """Shapes and dtypes of test/test_fake_tensor.py:1949-1959 (same shape, float16) plus the int4 widening."""
    res = pa.npu_anti_quant(_m(20, 100, dtype=torch.int8), _m(100, dtype=torch.float32), offset=_m(100, dtype=torch.float32),
                            dst_dtype=torch.float16)
    assert res.shape == (20, 100) and res.dtype == torch.float16
    res = pa.npu_anti_quant(_m(10, 25, dtype=torch.int32), _m(200, dtype=torch.float32), dst_dtype=torch.bfloat16)
    assert res.shape == (10, 200) and res.dtype == torch.bfloat16
    assert pa.npu_anti_quant(_m(4, 8, dtype=torch.int8), _m(1, dtype=torch.float32)).dtype == torch.float16
    with pytest.raises(RuntimeError, match="scale must have"):
        pa.npu_anti_quant(_m(4, 8, dtype=torch.int8), _m(7, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="int8 or int32"):
        pa.npu_anti_quant(_m(4, 8, dtype=torch.int16), _m(8, dtype=torch.float32))


def test_meta_trans_quant_param(pa):
    """test/test_fake_tensor.py:1929-1943: int64, the shape of the larger argument."""
    res = pa.npu_trans_quant_param(_m(1, dtype=torch.float32), _m(4, dtype=torch.float32))
    assert res.shape == (4,) and res.dtype == torch.int64
    res = pa.npu_trans_quant_param(_m(1, 4, dtype=torch.float32), _m(1, 4, dtype=torch.float32))
    assert res.shape == (1, 4) and res.dtype == torch.int64
    assert pa.npu_trans_quant_param(_m(7, dtype=torch.float32)).shape == (7,)
    with pytest.raises(RuntimeError, match="scale must be float32"):
        pa.npu_trans_quant_param(_m(4, dtype=torch.float16))
    with pytest.raises(RuntimeError, match="same number of elements"):
        pa.npu_trans_quant_param(_m(3, dtype=torch.float32), _m(4, dtype=torch.float32))


def test_meta_npu_quantize(pa):
    """Shapes and output types of npu_quantize (signature test/torch_npu_schema.json:2273-2275; dtype codes
    torch_npu/onnx/wrapper_onnx_ops.py:869-877) without a GPU."""
    x = _m(5, 16, 8, dtype=torch.float32)
    res = pa.npu_quantize(x, _m(8, dtype=torch.float32), _m(8, dtype=torch.int32), torch.quint8, 2)
    assert res.shape == (5, 16, 8) and res.dtype == torch.uint8
    res = pa.npu_quantize(_m(4, 6, dtype=torch.bfloat16), _m(1, dtype=torch.float32), None, torch.qint8, -1, False)
    assert res.dtype == torch.int8
    assert pa.npu_quantize(_m(4, 6, dtype=torch.float16), _m(4, dtype=torch.float32), None, torch.qint32, 0).dtype == torch.int32
    s = str(torch.ops.npu.npu_quantize.default._schema)
    assert "Tensor inputs, Tensor scales, Tensor? zero_points, ScalarType dtype, int axis=1, bool div_mode=True" in s
    with pytest.raises(RuntimeError, match="scales must have one element or one per element"):
        pa.npu_quantize(x, _m(7, dtype=torch.float32), None, torch.qint8, 2)
    with pytest.raises(RuntimeError, match="dtype must be"):
        pa.npu_quantize(x, _m(8, dtype=torch.float32), None, torch.float16, 2)
    with pytest.raises(RuntimeError, match="axis"):
        pa.npu_quantize(x, _m(8, dtype=torch.float32), None, torch.qint8, 3)
    with pytest.raises(RuntimeError, match="inputs must be"):
        pa.npu_quantize(_m(4, 4, dtype=torch.int32), _m(4, dtype=torch.float32), None, torch.qint8, 1)


def test_meta_swiglu(pa):
    assert pa.npu_swiglu(_m(64, 28672, dtype=torch.bfloat16)).shape == (64, 14336)
    assert pa.npu_swiglu(_m(2, 3, 8, dtype=torch.bfloat16), -1).shape == (2, 3, 4)
    with pytest.raises(RuntimeError, match="last dimension"):
        pa.npu_swiglu(_m(4, 8, dtype=torch.bfloat16), 0)


def test_fake_tensor_mode(pa):
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(4, 2048, 1024, dtype=torch.float16, device="cuda")
        y, s = pa.npu_dynamic_quant(x)
        assert y.shape == x.shape and y.dtype == torch.int8 and y.device == x.device
        assert s.shape == (4, 2048) and s.dtype == torch.float32 and s.device == x.device


# ---------------------------------------------------------------- contrib modules (argument marshalling)

class _Recorder:
    def __init__(self, monkeypatch, name):
        self.calls = []
        real = getattr(torch.ops.npu, name)

        def fake(*args, **kwargs):
            self.calls.append((args, kwargs))
            return real(*args, **kwargs)
        monkeypatch.setattr(torch.ops.npu, name, fake, raising=False)


def test_linear_quant_marshalling(pa, monkeypatch):
    from pytorch_amd.contrib.module import LinearQuant, LinearA8W8Quant
    rec = _Recorder(monkeypatch, "npu_quant_matmul")
    m = LinearQuant(64, 32, bias=False, pertoken_scale=True, output_dtype=torch.bfloat16)
    assert m.weight.shape == (32, 64) and m.scale.shape == (32,) and m.bias is None and m.offset is None
    assert not m.weight.requires_grad
    m = m.to("meta")
    m.weight.data = _m(32, 64, dtype=torch.int8)
    m.pertoken_scale.data = _m(16, dtype=torch.float32)
    out = m(_m(16, 64, dtype=torch.int8))
    assert out.shape == (16, 32) and out.dtype == torch.bfloat16
    (args, kwargs), = rec.calls
    assert args[1].shape == (64, 32) and args[1].stride() == (1, 64)          # transposed view, K-contiguous
    assert set(kwargs) == {"offset", "pertoken_scale", "bias", "output_dtype"}
    with pytest.raises(ValueError, match="both torch.int32 or both torch.int8"):
        m(_m(16, 64, dtype=torch.float16))
    # float32 scale without pertoken_scale and without bf16/int32 output goes through npu_trans_quant_param
    # (linear_quant.py:104-108) and yields the re-quantised int8 output
    rec2 = _Recorder(monkeypatch, "npu_trans_quant_param")
    m2 = LinearQuant(64, 32, bias=False, offset=True).to("meta")
    m2.weight.data = _m(32, 64, dtype=torch.int8)
    out = m2(_m(16, 64, dtype=torch.int8))
    assert out.dtype == torch.int8 and out.shape == (16, 32)
    assert len(rec2.calls) == 1 and rec.calls[-1][0][2].dtype == torch.int64
    with pytest.warns(FutureWarning):
        a = LinearA8W8Quant(64, 32, bias=True, output_dtype=torch.bfloat16)
    assert a.bias.dtype == torch.int32
    a = a.to("meta")
    a.weight.data = _m(32, 64, dtype=torch.int8)
    a.scale.data = _m(32, dtype=torch.float16)
    with pytest.raises(ValueError, match="scale should be torch.int64, torch.float32 or torch.bfloat16"):
        a(_m(16, 64, dtype=torch.int8))
    a.scale.data = _m(32, dtype=torch.float32)
    a.output_dtype = torch.int32
    with pytest.raises(ValueError, match="output_dtype should be"):
        a(_m(16, 64, dtype=torch.int8))


def test_linear_weight_quant_marshalling(pa, monkeypatch):
    from pytorch_amd.contrib.module import LinearWeightQuant
    rec = _Recorder(monkeypatch, "npu_weight_quant_batchmatmul")
    m = LinearWeightQuant(256, 64, bias=False, antiquant_offset=True, antiquant_group_size=128).to("meta")
    assert m.weight.shape == (64, 256) and m.quant_scale is None and m.bias is None
    m.weight.data = _m(64, 256, dtype=torch.int8)
    m.antiquant_scale.data = _m(64, 2, dtype=torch.bfloat16)      # stored [N, G]
    m.antiquant_offset.data = _m(64, 2, dtype=torch.bfloat16)
    out = m(_m(3, 256, dtype=torch.bfloat16))
    assert out.shape == (3, 64)
    (args, kwargs), = rec.calls
    assert args[1].shape == (256, 64) and args[1].stride() == (1, 256)
    assert args[2].shape == (2, 64) and args[3].shape == (2, 64)   # handed over as [G, N] views
    assert args[7] == 128 and args[8] == 0 and kwargs == {"weight_dtype": None}


def test_prepared_copies_are_dropped_when_the_module_moves_or_reloads(pa):
    """prepare_() keeps derived weight copies in plain attributes; .to()/.half()/load_state_dict must drop them so that a
    stale or wrong-device copy can never be used (no kernel runs here: the copies are set by hand)."""
    from pytorch_amd.contrib.module import LinearQuant, LinearWeightQuant
    m = LinearQuant(64, 32, bias=False)
    m._prepared_i8 = torch.zeros(32, 64, dtype=torch.int8)
    m.to("meta")
    assert m._prepared_i8 is None
    m = LinearQuant(64, 32, bias=False)
    m._prepared_i8 = torch.zeros(32, 64, dtype=torch.int8)
    m.load_state_dict(LinearQuant(64, 32, bias=False).state_dict())
    assert m._prepared_i8 is None
    w = LinearWeightQuant(256, 64, bias=False)
    w._prepared = (torch.zeros(1), None, None)
    w.to(torch.device("cpu"), torch.float64)
    assert w._prepared is None
    w._prepared = (torch.zeros(1), None, None)
    w.load_state_dict(LinearWeightQuant(256, 64, bias=False).state_dict())
    assert w._prepared is None


def test_flop_counter_formulas(pa):
    """2*M*K*N for the quantised matmuls, as torch_npu/profiler/_flops_formulas.py:319-329 counts a matmul; counted on
    meta tensors, so no kernel runs."""
    from torch.utils.flop_counter import FlopCounterMode
    with FlopCounterMode(display=False) as fc:
        pa.npu_quant_matmul(_m(1024, 4096, dtype=torch.int8), _m(4096, 11008, dtype=torch.int8), _m(11008, dtype=torch.float32),
                            pertoken_scale=_m(1024, dtype=torch.float32), output_dtype=torch.bfloat16)
    assert fc.get_total_flops() == 2 * 1024 * 4096 * 11008
    with FlopCounterMode(display=False) as fc:
        pa.npu_weight_quant_batchmatmul(_m(2, 64, 4096, dtype=torch.bfloat16), _m(4096, 1792, dtype=torch.int32),
                                        _m(32, 14336, dtype=torch.bfloat16), _m(32, 14336, dtype=torch.bfloat16), None, None,
                                        None, 128)
    assert fc.get_total_flops() == 2 * 128 * 4096 * 14336
    with FlopCounterMode(display=False) as fc:
        pa.npu_quant_matmul(_m(3, 16, 256, dtype=torch.int8), _m(256, 64, dtype=torch.int8), _m(64, dtype=torch.float32),
                            output_dtype=torch.bfloat16)
    assert fc.get_total_flops() == 2 * 3 * 16 * 256 * 64


def test_weight_quant_workspace_query_follows_the_preferred_kernel():
    """Host logic of mi355_weight_quant_matmul_workspace (no GPU needed): the request is that of the kernel a launch with
    aligned pointers takes, not of a kernel further down the order.  int4 with K split between workgroups asks for the
    zero area; int4 at prefill sizes asks for the zero area plus the rewritten weight and parameters (words along K are
    rewritten per call from 256 rows up) and no longer for S x M x N x 4 bytes of partial sums; per-channel int4 splits
    K like the grouped case."""
    from pytorch_amd import _capi
    L = _capi.lib()
    zero_area = 16 * 1024 * 1024 + 16384
    q = L.mi355_weight_quant_matmul_workspace
    assert q(1, 14336, 4096, 4, 128) == zero_area            # decode kernel, four chunks of K
    # 128 rows: the register-expanding GEMM (words along N, two chunks of K) needs the zero area alone; with the words along
    # K the launch takes workgroups of eight wavefronts with K split two ways, so the request covers its partial sums
    two_chunks = zero_area + 2 * 128 * 14336 * 4
    assert q(128, 14336, 4096, 4, 128) == two_chunks
    assert q(128, 14336, 4096, 4, 0) == two_chunks           # per channel: the same split
    repack = zero_area + 4096 * (14336 // 8) * 4 + 2 * (4096 // 128) * 14336 * 2
    for rows in (256, 2048, 8192):
        assert q(rows, 14336, 4096, 4, 128) == repack
        assert q(rows, 14336, 4096, 8, 0) == 0                # int8 tiled GEMM with enough tiles: no split, no workspace
    assert q(0, 14336, 4096, 4, 128) == 0 and q(16, 14336, 4096, 5, 128) == 0
