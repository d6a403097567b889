"""ctypes/numpy front end of the CPU oracle (``oracle/golden.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by
the ``cpu_baseline`` leg of ``bench.py`` as the checker.  The shipped package never
imports it.

bfloat16 / float16 data cross this boundary as ``numpy.uint16`` bit patterns; the
helpers at the bottom convert from and to torch tensors.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle_golden.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile ``golden.c`` with the committed Makefile and return the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "liboracle_golden.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.orc_set_threads.argtypes = [i32]
        L.orc_get_threads.restype = i32
        L.orc_dynamic_quant.argtypes = [vp, i32, vp, i64, i64, i64, vp, vp]
        L.orc_dynamic_quant_asymmetric.argtypes = [vp, i32, vp, i64, i64, i64, vp, vp, vp]
        L.orc_int8_gemm.argtypes = [vp, i64, vp, i64, i64, i64, i64, i64, vp]
        L.orc_quant_matmul_epilogue.argtypes = [vp, vp, vp, i64, vp, i64, i64, vp]
        L.orc_quant_matmul_epilogue_ex.argtypes = [vp, vp, vp, i64, vp, i32, i32, i64, i64, vp]
        L.orc_unpack_int4.argtypes = [vp, i64, vp]
        L.orc_pack_int4.argtypes = [vp, i64, vp]
        L.orc_antiquant.argtypes = [vp, vp, vp, i64, i64, vp]
        L.orc_weight_quant_matmul.argtypes = [vp, i64, vp, i32, i64, i64, vp, vp,
                                              i64, i64, i64, i64, i32, vp, vp]
        L.orc_weight_quant_matmul_f16.argtypes = L.orc_weight_quant_matmul.argtypes
        L.orc_weight_quant_matmul_bias.argtypes = [vp, i64, vp, i32, i64, i64, vp, vp, vp, i32, i64, i64, i64, i64, i32, vp, vp]
        L.orc_swiglu.argtypes = [vp, i64, i64, vp]
        L.orc_bf16_to_f32.argtypes = [vp, vp, i64]
        L.orc_f32_to_bf16.argtypes = [vp, vp, i64]
        _lib = L
    return _lib


def set_threads(n: int) -> None:
    lib().orc_set_threads(int(n))


def get_threads() -> int:
    return int(lib().orc_get_threads())


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


# ------------------------------------------------------------------ operators

def dynamic_quant(x_u16: np.ndarray, in_dtype: str = "bf16", smooth_u16: np.ndarray | None = None):
    """x: uint16 bit patterns [..., cols] -> (y int8 same shape, scale float32 [...])."""
    x = _c(x_u16, np.uint16)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    y = np.empty(x.shape, dtype=np.int8)
    scale = np.empty(x.shape[:-1], dtype=np.float32)
    sm = None if smooth_u16 is None else _c(smooth_u16, np.uint16)
    if rows and cols:
        lib().orc_dynamic_quant(_p(x), 0 if in_dtype == "bf16" else 1, _p(sm), rows, cols, cols,
                                _p(y), _p(scale))
    elif rows:
        scale[...] = 0.0
    return y, scale


def dynamic_quant_grouped(x_u16: np.ndarray, smooth_u16: np.ndarray, group_index, in_dtype: str = "bf16"):
    """npu_dynamic_quant with per-expert smooth scales (``group_index`` of the operator's signature,
    test/test_fake_tensor.py:1670-1687; no call in the reference tree passes it): ``smooth_u16`` [E, cols],
    ``group_index`` [E] the running totals of the rows of each expert; rows group_index[e-1] .. group_index[e]-1 are
    quantised as dynamic_quant does with smooth_u16[e], rows past the last total with the last expert's scales.
    PARITY UNPINNED for the meaning of group_index (the operator's published description); the arithmetic is
    dynamic_quant's."""
    x = _c(x_u16, np.uint16)
    x2 = x.reshape(-1, x.shape[-1])
    sm = _c(smooth_u16, np.uint16)
    gi = [int(v) for v in np.asarray(group_index).reshape(-1)]
    assert sm.ndim == 2 and sm.shape[0] == len(gi) and sm.shape[1] == x.shape[-1]
    y = np.empty(x2.shape, dtype=np.int8)
    scale = np.empty(x2.shape[0], dtype=np.float32)
    lo = 0
    for e, hi in enumerate(gi):
        hi = x2.shape[0] if e == len(gi) - 1 else min(max(hi, lo), x2.shape[0])
        if hi > lo:
            y[lo:hi], scale[lo:hi] = dynamic_quant(x2[lo:hi], in_dtype, sm[e])
        lo = max(lo, hi)
    return y.reshape(x.shape), scale.reshape(x.shape[:-1])


def dynamic_quant_int4(x_u16: np.ndarray, in_dtype: str = "bf16", smooth_u16: np.ndarray | None = None):
    """npu_dynamic_quant with dst_type=torch.quint4x2 (the argument is in the operator's signature,
    test/test_fake_tensor.py:1670-1687; no call or golden in the reference tree): per row scale = max|x| / 7 and codes
    rint(x / scale) in [-7, 7] (float32 operations, ties to even, a zero row gives scale 0 and codes 0), packed eight to
    an int32 word, first column in the low nibble (the order pinned by test/custom_ops/test_npu_anti_quant.py:12-24).
    Returns (int32 [..., cols / 8], scale float32 [...]).  PARITY UNPINNED: the operator's published description."""
    u = _c(x_u16, np.uint16)
    x = u.view(np.float16).astype(np.float32) if in_dtype == "fp16" else bf16_bits_to_f32(u)
    if smooth_u16 is not None:
        sm = _c(smooth_u16, np.uint16)
        x = (x * (sm.view(np.float16).astype(np.float32) if in_dtype == "fp16" else bf16_bits_to_f32(sm))).astype(np.float32)
    amax = np.abs(x).max(axis=-1, keepdims=True).astype(np.float32)
    scale = (amax / np.float32(7.0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint((x / scale).astype(np.float32))
    q = np.where(amax > 0, np.clip(np.nan_to_num(q, nan=0.0), -7, 7), 0).astype(np.int8)
    return pack_int4(q), scale[..., 0]


def dynamic_quant_asymmetric(x_u16: np.ndarray, in_dtype: str = "bf16", smooth_u16: np.ndarray | None = None):
    """x: uint16 bit patterns [..., cols] -> (y int8 same shape, scale float32 [...], offset float32 [...])."""
    x = _c(x_u16, np.uint16)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    y = np.empty(x.shape, dtype=np.int8)
    scale = np.zeros(x.shape[:-1], dtype=np.float32)
    offset = np.zeros(x.shape[:-1], dtype=np.float32)
    sm = None if smooth_u16 is None else _c(smooth_u16, np.uint16)
    if rows and cols:
        lib().orc_dynamic_quant_asymmetric(_p(x), 0 if in_dtype == "bf16" else 1, _p(sm), rows, cols, cols,
                                           _p(y), _p(scale), _p(offset))
    return y, scale, offset


def dynamic_quant_asymmetric_grouped(x_u16: np.ndarray, smooth_u16: np.ndarray, group_index, in_dtype: str = "bf16"):
    """npu_dynamic_quant_asymmetric with per-expert smooth scales: dynamic_quant_asymmetric applied to every expert's rows
    with that expert's scales (group_index as in dynamic_quant_grouped; PARITY UNPINNED likewise)."""
    x = _c(x_u16, np.uint16)
    x2 = x.reshape(-1, x.shape[-1])
    sm = _c(smooth_u16, np.uint16)
    gi = [int(v) for v in np.asarray(group_index).reshape(-1)]
    y = np.empty(x2.shape, dtype=np.int8)
    scale = np.empty(x2.shape[0], dtype=np.float32)
    offset = np.empty(x2.shape[0], dtype=np.float32)
    lo = 0
    for e, hi in enumerate(gi):
        hi = x2.shape[0] if e == len(gi) - 1 else min(max(hi, lo), x2.shape[0])
        if hi > lo:
            y[lo:hi], scale[lo:hi], offset[lo:hi] = dynamic_quant_asymmetric(x2[lo:hi], in_dtype, sm[e])
        lo = max(lo, hi)
    return y.reshape(x.shape), scale.reshape(x.shape[:-1]), offset.reshape(x.shape[:-1])


def int8_gemm(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """a int8 [M,K] (row-major), b int8 [K,N] with arbitrary numpy strides -> int32 [M,N]."""
    a = _c(a, np.int8)
    assert b.dtype == np.int8 and a.shape[1] == b.shape[0]
    M, K = a.shape
    N = b.shape[1]
    acc = np.empty((M, N), dtype=np.int32)
    if M and N:
        lib().orc_int8_gemm(_p(a), K, _p(b), b.strides[0], b.strides[1], M, N, K, _p(acc))
    return acc


def quant_matmul_epilogue(acc, scale, pertoken_scale=None, bias_u16=None) -> np.ndarray:
    acc = _c(acc, np.int32)
    M, N = acc.shape
    scale = _c(scale, np.float32).reshape(-1)
    assert scale.size in (1, N)
    ps = None if pertoken_scale is None else _c(pertoken_scale, np.float32).reshape(-1)
    if ps is not None:
        assert ps.size == M
    bias = None if bias_u16 is None else _c(bias_u16, np.uint16).reshape(-1)
    out = np.empty((M, N), dtype=np.uint16)
    if M and N:
        lib().orc_quant_matmul_epilogue(_p(acc), _p(ps), _p(scale), scale.size, _p(bias), M, N, _p(out))
    return out


def quant_matmul_epilogue_ex(acc, scale, pertoken_scale=None, bias=None, out: str = "bf16") -> np.ndarray:
    """bias: None, uint16 (bf16 bit patterns), int32 or float32 array [N]; out: "bf16" / "fp16" (uint16 bit patterns)
    or "int32"."""
    acc = _c(acc, np.int32)
    M, N = acc.shape
    ps = None if pertoken_scale is None else _c(pertoken_scale, np.float32).reshape(-1)
    sc = None if scale is None else _c(scale, np.float32).reshape(-1)
    kind = 0
    if bias is not None:
        kind = {np.dtype(np.uint16): 1, np.dtype(np.int32): 2, np.dtype(np.float32): 3}[np.asarray(bias).dtype]
        bias = np.ascontiguousarray(np.asarray(bias).reshape(-1))
        assert bias.size == N
    out_kind = {"bf16": 0, "fp16": 1, "int32": 2}[out]
    res = np.empty((M, N), dtype=np.int32 if out_kind == 2 else np.uint16)
    if M and N:
        lib().orc_quant_matmul_epilogue_ex(_p(acc), _p(ps), _p(sc), 0 if sc is None else sc.size, _p(bias), kind,
                                           out_kind, M, N, _p(res))
    return res


def quant_matmul(a, b, scale, pertoken_scale=None, bias_u16=None):
    """Full W8A8 path -> (out bf16 bit patterns [M,N], acc int32 [M,N])."""
    acc = int8_gemm(a, b)
    return quant_matmul_epilogue(acc, scale, pertoken_scale, bias_u16), acc


def unpack_int4(packed: np.ndarray) -> np.ndarray:
    p = _c(packed, np.int32)
    out = np.empty(p.shape[:-1] + (p.shape[-1] * 8,), dtype=np.int8)
    lib().orc_unpack_int4(_p(p), p.size, _p(out))
    return out


def pack_int4(vals: np.ndarray) -> np.ndarray:
    v = _c(vals, np.int8)
    assert v.shape[-1] % 8 == 0
    out = np.empty(v.shape[:-1] + (v.shape[-1] // 8,), dtype=np.int32)
    lib().orc_pack_int4(_p(v), out.size, _p(out))
    return out


def quant_matmul_a4w4(x1_words, x2_words, scale, pertoken_scale=None, bias=None, out: str = "bf16"):
    """npu_quant_matmul with both operands packed int4 (test/test_fake_tensor.py:1917-1923,
    torch_npu/contrib/module/linear_quant.py:40-50): x1 int32 [M, K/8]; x2 int32 [K, N/8] (words along N) or
    [K/8, N] (words along K, the transposed view of a weight stored [N, K/8]), told apart by the row count.
    The nibbles are widened (order pinned by test/custom_ops/test_npu_anti_quant.py:12-24) and the int8 path
    runs on them -> (out [M, N], acc int32 [M, N])."""
    a = unpack_int4(x1_words)
    x2w = np.asarray(x2_words)
    if x2w.shape[0] == a.shape[1]:
        b = unpack_int4(x2w)
    else:
        assert x2w.shape[0] * 8 == a.shape[1], (x2w.shape, a.shape)
        b = np.ascontiguousarray(unpack_int4(np.ascontiguousarray(x2w.T)).T)
    acc = int8_gemm(a, b)
    return quant_matmul_epilogue_ex(acc, scale, pertoken_scale, bias, out), acc


def antiquant(w_i8, scale_f32, offset_f32=None) -> np.ndarray:
    w = _c(w_i8, np.int8)
    rows, cols = w.shape
    s = _c(scale_f32, np.float32)
    o = None if offset_f32 is None else _c(offset_f32, np.float32)
    out = np.empty((rows, cols), dtype=np.float32)
    lib().orc_antiquant(_p(w), _p(s), _p(o), rows, cols, _p(out))
    return out


def anti_quant(x, scale_f32, offset_f32=None, dst: str = "fp16") -> np.ndarray:
    """npu_anti_quant: x int8 [rows, cols] or int32 [rows, cols/8] (packed int4); scale / offset float32 with cols
    elements or one.  Returns the bit patterns of the float16 / bfloat16 result.  A composition of the restatements
    above (unpack, (x + offset) * scale in float32) and one IEEE rounding to the output type."""
    xa = np.asarray(x)
    vals = unpack_int4(xa) if xa.dtype == np.int32 else _c(xa, np.int8)
    vals = vals.reshape(-1, vals.shape[-1])
    cols = vals.shape[1]
    s = np.broadcast_to(_c(scale_f32, np.float32).reshape(-1), (cols,))
    o = None if offset_f32 is None else np.broadcast_to(_c(offset_f32, np.float32).reshape(-1), (cols,))
    f = antiquant(vals, s, o)
    if dst == "bf16":
        return f32_to_bf16_bits(f)
    assert dst == "fp16"
    return f.astype(np.float16).view(np.uint16)          # IEEE round to nearest even


def quantize(x_f32, scale_f32, zero_point_f32=None, out: str = "int8", axis: int = -1, div_mode: bool = True) -> np.ndarray:
    """npu_quantize (signature test/torch_npu_schema.json:2273-2275; output types
    torch_npu/onnx/wrapper_onnx_ops.py:869-877): q = clamp(rint(x / scale + zero_point)) along ``axis`` (x * scale
    with div_mode False), every operation rounded to float32, ties to even, NaN -> 0.  ``x_f32`` holds the input
    values as float32 (bf16 / fp16 inputs converted exactly).  PARITY UNPINNED for the general formula: the reference
    tree holds no golden or test vector for this operator; the formula is the vendor's published one.  Pinned by the
    tests where the mathematics fixes it: against torch.quantize_per_channel / quantize_per_tensor for power-of-two
    scales (where x / scale and x * (1 / scale) agree exactly) and against hand-computed ties."""
    x = _c(x_f32, np.float32)
    axis = axis % x.ndim
    shape = [1] * x.ndim
    shape[axis] = -1
    s = _c(scale_f32, np.float32).reshape(-1)
    s = s.reshape(shape) if s.size > 1 else s.reshape([1] * x.ndim)
    v = (x / s).astype(np.float32) if div_mode else (x * s).astype(np.float32)
    if zero_point_f32 is not None:
        z = _c(zero_point_f32, np.float32).reshape(-1)
        z = z.reshape(shape) if z.size > 1 else z.reshape([1] * x.ndim)
        v = (v + z).astype(np.float32)
    v = np.rint(v)
    v = np.where(np.isnan(v), np.float32(0), v)
    lo, hi, dt = {"int8": (-128, 127, np.int8), "uint8": (0, 255, np.uint8), "int32": (-2 ** 31, 2 ** 31 - 1, np.int32)}[out]
    return np.clip(v.astype(np.float64), lo, hi).astype(dt)


def weight_quant_requant(out_u16, quant_scale_f32, quant_offset_f32=None, dtype: str = "bf16") -> np.ndarray:
    """int8 output of npu_weight_quant_batchmatmul with quant_scale / quant_offset (the arguments
    torch_npu/contrib/module/linear_weight_quant.py:79-87,106-109 constructs and passes): the product rounded to the
    dtype of x (``out_u16``: its bit patterns), times quant_scale[n], plus the offset brought to the 9-bit integer range
    of the packed parameter words (round, clip to [-256, 255]: f32_2_s9, test/contrib/test_linear_weight_quant.py:13-16),
    rounded half to even and clamped to int8; every operation rounded to float32.  PARITY UNPINNED: the reference tree
    holds no golden or test vector for this output (its test builds the module with quant_scale=False); this is the
    re-quantisation of npu_quant_matmul's int8 output applied to the rounded product."""
    u = np.ascontiguousarray(out_u16, dtype=np.uint16)
    x = u.view(np.float16).astype(np.float32) if dtype == "fp16" else bf16_bits_to_f32(u)
    off = None
    if quant_offset_f32 is not None:
        off = np.clip(np.rint(_c(quant_offset_f32, np.float32)), -256, 255).astype(np.float32)
    return quantize(x, quant_scale_f32, off, out="int8", axis=-1, div_mode=False)


def trans_quant_param(scale_f32, offset_f32=None) -> np.ndarray:
    """npu_trans_quant_param (caller torch_npu/contrib/module/linear_quant.py:104-108, result type and shapes
    test/test_fake_tensor.py:1929-1943): int64 words with the float32 bit pattern of the scale in bits 0-31,
    clamp(rint(offset), -256, 255) as a 9-bit two's-complement field in bits 37-45 and bit 46 set.  PARITY UNPINNED:
    the bit layout is not in the reference tree (the operator's published description); the tests pin this function
    by hand-assembled words and by the decode round trip only."""
    sc = _c(scale_f32, np.float32).reshape(-1)
    n = sc.size if offset_f32 is None else max(sc.size, np.asarray(offset_f32).size)
    q = np.broadcast_to(sc.view(np.uint32).astype(np.uint64), (n,)).copy() | np.uint64(1 << 46)
    if offset_f32 is not None:
        o = np.clip(np.rint(_c(offset_f32, np.float32).reshape(-1)), -256, 255).astype(np.int64)
        q |= (np.broadcast_to(o, (n,)) & 0x1FF).astype(np.uint64) << np.uint64(37)
    return q.view(np.int64)


def quant_param_decode(q):
    """(scale float32, offset float32) carried by the words of trans_quant_param."""
    u = _c(q, np.int64).reshape(-1).view(np.uint64)
    scale = (u & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.float32)
    field = ((u >> np.uint64(37)) & np.uint64(0x1FF)).astype(np.int64)
    offset = np.where(field >= 256, field - 512, field).astype(np.float32)
    return scale, offset


def quant_matmul_requant(a, b, qparam, bias_i32=None) -> np.ndarray:
    """npu_quant_matmul with int8 output: clamp(rint(float32(acc + bias) * scale + offset), -128, 127), scale and offset
    decoded from the packed words, every operation rounded to float32, ties to even.  The int32 product is int8_gemm
    (pinned); the formula out = (x1 @ x2 + bias) * scale + offset is the operator's published one: PARITY UNPINNED."""
    acc = int8_gemm(a, b)
    if bias_i32 is not None:
        acc = (acc.astype(np.int64) + _c(bias_i32, np.int32).reshape(1, -1)).astype(np.int32)   # wraps like the accumulator
    scale, offset = quant_param_decode(qparam)
    v = (acc.astype(np.float32) * scale.reshape(1, -1)).astype(np.float32)
    v = (v + offset.reshape(1, -1)).astype(np.float32)
    return np.clip(np.rint(v), -128, 127).astype(np.int8)


def weight_quant_matmul(x_u16, w, scale_u16, off_u16=None, group_size: int = 0, accum: str = "f32", dtype: str = "bf16",
                        bias_u16=None):
    """x bf16 (or, with dtype="fp16", float16) bits [M,K]; w int8 [K,N] (any strides) or int32 [K,N/8] (packed int4);
    scale/off bits of the same type [N] or [G,N].  Returns (out bits [M,N], unrounded float32 [M,N])."""
    x = _c(x_u16, np.uint16)
    M, K = x.shape
    if w.dtype == np.int8:
        bits, N = 8, w.shape[1]
        ldk, ldn = w.strides
        wbuf = w
    else:
        wbuf = _c(w, np.int32)
        bits, N = 4, wbuf.shape[1] * 8
        ldk, ldn = 0, 0
    assert w.shape[0] == K
    s = _c(scale_u16, np.uint16).reshape(-1, N)
    o = None if off_u16 is None else _c(off_u16, np.uint16).reshape(-1, N)
    G = 1 if group_size <= 0 else (K + group_size - 1) // group_size
    assert s.shape[0] == G, (s.shape, G)
    out = np.empty((M, N), dtype=np.uint16)
    outf = np.empty((M, N), dtype=np.float32)
    if M and N:
        if bias_u16 is not None:
            b = _c(bias_u16, np.uint16).reshape(-1)
            assert b.size == N
            lib().orc_weight_quant_matmul_bias(_p(x), K, _p(wbuf), bits, ldk, ldn, _p(s), _p(o), _p(b), 0 if dtype == "bf16" else 1,
                                               M, N, K, group_size, 0 if accum == "f32" else 1, _p(out), _p(outf))
        else:
            fn = lib().orc_weight_quant_matmul if dtype == "bf16" else lib().orc_weight_quant_matmul_f16
            fn(_p(x), K, _p(wbuf), bits, ldk, ldn, _p(s), _p(o), M, N, K, group_size, 0 if accum == "f32" else 1,
               _p(out), _p(outf))
    return out, outf


def swiglu(x_u16: np.ndarray) -> np.ndarray:
    x = _c(x_u16, np.uint16)
    rows, two_half = x.shape
    assert two_half % 2 == 0
    out = np.empty((rows, two_half // 2), dtype=np.uint16)
    if out.size:
        lib().orc_swiglu(_p(x), rows, two_half // 2, _p(out))
    return out


def swiglu_quant(x_u16: np.ndarray, activate_left: bool = True, smooth_u16: np.ndarray | None = None):
    """dynamic_quant(swiglu(x), smooth): the composition of the two restatements above (no arithmetic of its own).
    activate_left=False activates the right half: silu(x[:, half:]) * x[:, :half]."""
    x = _c(x_u16, np.uint16)
    half = x.shape[1] // 2
    if not activate_left:
        x = np.concatenate([x[:, half:], x[:, :half]], axis=1)
    return dynamic_quant(swiglu(x), "bf16", smooth_u16)


# ------------------------------------------------------ bit-pattern helpers

def bf16_bits_to_f32(u16: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(u16, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_bf16_bits(f32: np.ndarray) -> np.ndarray:
    f = _c(f32, np.float32)
    out = np.empty(f.shape, dtype=np.uint16)
    lib().orc_f32_to_bf16(_p(f), _p(out), f.size)
    return out


def bits_of(t) -> np.ndarray:
    """torch bf16/fp16 tensor (any device) -> numpy uint16 bit patterns."""
    import torch
    assert t.dtype in (torch.bfloat16, torch.float16)
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_tensor(u16: np.ndarray):
    """numpy uint16 bit patterns -> torch bf16 CPU tensor."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(u16).view(np.int16).copy()).view(torch.bfloat16)


def bf16_ulp_distance(a_u16: np.ndarray, b_u16: np.ndarray) -> np.ndarray:
    """Distance in bf16 units-in-the-last-place between two bit-pattern arrays
    (sign-magnitude patterns mapped onto a monotone integer line)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7fff), u & 0x7fff)
    return np.abs(key(np.asarray(a_u16)) - key(np.asarray(b_u16)))
