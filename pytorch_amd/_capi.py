"""ctypes binding of the C ABI (``include/mi355_quant.h``) for torch tensors on the GPU.

This is the thinnest possible host side: it validates nothing beyond what is needed to
form the pointer/size arguments, so tests that call it exercise the C entry points
themselves.  The torch operators (``torch.ops.npu.*``) reach the same entry points from C++.
"""
from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libmi355_quant.so")

EXPORTS = ("mi355_status_string", "mi355_quant_abi_version", "mi355_dynamic_quant", "mi355_dynamic_quant_grouped", "mi355_dynamic_quant_int4", "mi355_dynamic_quant_asymmetric_grouped", "mi355_swiglu_quant_grouped",
           "mi355_quant_matmul_workspace", "mi355_quant_matmul",
           "mi355_weight_quant_matmul_workspace", "mi355_weight_quant_matmul", "mi355_swiglu", "mi355_swiglu_quant",
           "mi355_anti_quant", "mi355_unpack_int4", "mi355_dynamic_quant_asymmetric", "mi355_quantize",
           "mi355_trans_quant_param", "mi355_quant_matmul_qparam", "mi355_swiglu_quant_smooth", "mi355_set_tuning",
           "mi355_quant_matmul_noalloc", "mi355_stream_capture_id", "mi355_probe_clock", "mi355_device_info", "mi355_transpose_int8", "mi355_probe_empty_launch",
           "mi355_workspace_status", "mi355_workspace_zero_bytes")

_lib = None


class Mi355Error(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is missing: run `python pytorch_amd/build.py` (hipcc, gfx950) first")
        L = ctypes.CDLL(LIB_PATH)
        vp, i64, i32, sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_size_t
        L.mi355_status_string.restype = ctypes.c_char_p
        L.mi355_status_string.argtypes = [i32]
        L.mi355_quant_abi_version.restype = i32
        L.mi355_dynamic_quant.argtypes = [vp, i32, vp, vp, vp, i64, i64, i64, vp]
        L.mi355_dynamic_quant_grouped.argtypes = [vp, i32, vp, vp, i64, vp, vp, i64, i64, i64, vp]
        L.mi355_dynamic_quant_int4.argtypes = [vp, i32, vp, vp, i64, vp, vp, i64, i64, i64, vp]
        L.mi355_quant_matmul_workspace.restype = sz
        L.mi355_quant_matmul_workspace.argtypes = [i64, i64, i64, i64, i64]
        L.mi355_quant_matmul.argtypes = [vp, vp, vp, vp, i64, vp, i32, vp, i32, i64, i64, i64, i64, i64, i64, i64, vp, sz, vp]
        L.mi355_weight_quant_matmul_workspace.restype = sz
        L.mi355_weight_quant_matmul_workspace.argtypes = [i64, i64, i64, i32, i64]
        L.mi355_weight_quant_matmul.argtypes = [vp, i32, vp, i32, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64,
                                                i64, i64, vp, sz, vp]
        L.mi355_swiglu.argtypes = [vp, vp, i64, i64, i64, vp]
        L.mi355_swiglu_quant.argtypes = [vp, i32, vp, vp, i64, i64, i64, vp]
        L.mi355_swiglu_quant_smooth.argtypes = [vp, i32, vp, vp, vp, i64, i64, i64, vp]
        L.mi355_swiglu_quant_grouped.argtypes = [vp, i32, vp, vp, i64, vp, vp, i64, i64, i64, vp]
        L.mi355_anti_quant.argtypes = [vp, i32, vp, i64, vp, i64, vp, i32, i64, i64, i64, i64, vp]
        L.mi355_unpack_int4.argtypes = [vp, vp, i64, i64, i64, i64, vp]
        L.mi355_dynamic_quant_asymmetric.argtypes = [vp, i32, vp, vp, vp, vp, i64, i64, i64, vp]
        L.mi355_dynamic_quant_asymmetric_grouped.argtypes = [vp, i32, vp, vp, i64, vp, vp, vp, i64, i64, i64, vp]
        L.mi355_trans_quant_param.argtypes = [vp, i64, vp, i64, vp, i64, vp]
        L.mi355_quant_matmul_qparam.argtypes = [vp, vp, vp, i64, vp, i32, vp, i32, i64, i64, i64, i64, i64, i64, i64, vp, sz, vp]
        L.mi355_quantize.argtypes = [vp, i32, vp, i64, vp, i32, i64, vp, i32, i64, i64, i64, i32, vp]
        L.mi355_set_tuning.argtypes = [ctypes.c_char_p, i32]
        L.mi355_probe_clock.argtypes = [vp, i32, i32, vp]
        L.mi355_probe_empty_launch.argtypes = [i32, vp]
        L.mi355_transpose_int8.argtypes = [vp, vp, i64, i64, i64, vp]
        L.mi355_device_info.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.mi355_stream_capture_id.argtypes = [vp, ctypes.POINTER(ctypes.c_ulonglong)]
        L.mi355_quant_matmul_noalloc.argtypes = [vp, vp, vp, vp, i64, vp, i32, vp, i32, i64, i64, i64, i64, i64, i64, i64, vp]
        L.mi355_workspace_status.argtypes = [vp, sz, i32, vp]
        L.mi355_workspace_zero_bytes.restype = sz
        _lib = L
    return _lib


def empty_launch(workgroups: int = 2048) -> None:
    _check(lib().mi355_probe_empty_launch(workgroups, _stream()), "mi355_probe_empty_launch")


def device_info():
    """(peak engine clock in MHz, compute units) of the current device."""
    khz, cus = ctypes.c_int(0), ctypes.c_int(0)
    _check(lib().mi355_device_info(ctypes.byref(khz), ctypes.byref(cus)), "mi355_device_info")
    return khz.value // 1000, cus.value


def sustained_mfma_clock_mhz(workgroups: int = 256, iters: int = 20000) -> float:
    """Shader clock (MHz) the GPU holds while every SIMD issues int8 MFMAs back to back (median over the workgroups)."""
    out = torch.zeros((workgroups, 2), dtype=torch.int64, device="cuda")
    _check(lib().mi355_probe_clock(_ptr(out), workgroups, iters, _stream()), "mi355_probe_clock")
    torch.cuda.synchronize()
    o = out.cpu().double()
    return float((o[:, 0] / o[:, 1].clamp(min=1) * 100.0).median())


def set_tuning(name: str, value: int) -> None:
    """Set a planner knob (0 = automatic); the knob names are those of ``csrc/tuning.hip``."""
    _check(lib().mi355_set_tuning(name.encode(), int(value)), "mi355_set_tuning")


def _check(status: int, what: str) -> None:
    if status != 0:
        raise Mi355Error(f"{what}: {lib().mi355_status_string(status).decode()} (status {status})")


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _need_gpu(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise Mi355Error("the C ABI takes device pointers: tensors must live on the GPU")


def dynamic_quant(x: torch.Tensor, smooth: torch.Tensor | None = None, group_index: torch.Tensor | None = None):
    """smooth [cols], or with group_index (int32 [E], running row totals per expert) [E, cols]."""
    _need_gpu(x, smooth)
    assert x.dtype in (torch.bfloat16, torch.float16)
    assert group_index is None or (group_index.dtype == torch.int32 and group_index.is_cuda and smooth.is_contiguous())
    if x.numel() and x.stride(-1) != 1:
        x = x.contiguous()
    cols = x.shape[-1]
    x2 = x.reshape(-1, cols) if x.dim() != 2 else x
    if x2.dim() == 2 and x2.shape[0] > 1 and x2.stride(0) < cols:
        x2 = x2.contiguous()
    rows = x2.shape[0]
    y = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    scale = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    if group_index is not None:
        st = lib().mi355_dynamic_quant_grouped(_ptr(x2), 0 if x.dtype == torch.bfloat16 else 1, _ptr(smooth), _ptr(group_index),
                                               group_index.numel(), _ptr(y), _ptr(scale), rows, cols,
                                               x2.stride(0) if rows > 1 else max(cols, 1), _stream())
        _check(st, "mi355_dynamic_quant_grouped")
        return y, scale
    st = lib().mi355_dynamic_quant(_ptr(x2), 0 if x.dtype == torch.bfloat16 else 1, _ptr(smooth), _ptr(y), _ptr(scale),
                                   rows, cols, x2.stride(0) if rows > 1 else max(cols, 1), _stream())
    _check(st, "mi355_dynamic_quant")
    return y, scale


def quant_matmul(x1, x2, scale, pertoken_scale=None, bias=None, out_dtype=torch.bfloat16, workspace=None):
    """x1 int8 [M,K]; x2 int8 [K,N] with strides (N,1) or (1,K)."""
    _need_gpu(x1, x2, scale, pertoken_scale, bias)
    M, K = x1.shape
    N = x2.shape[1]
    out = torch.empty((M, N), dtype=out_dtype, device=x1.device)
    need = lib().mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
    if workspace is None and need:
        workspace = _wq_workspace(x1.device, need)      # its leading counters must start at zero
    bias_dtype = 0 if bias is None else {torch.bfloat16: 1, torch.int32: 2, torch.float32: 3}[bias.dtype]
    out_code = {torch.bfloat16: 0, torch.int32: 1, torch.float16: 2}[out_dtype]
    st = lib().mi355_quant_matmul(_ptr(x1), _ptr(x2), _ptr(pertoken_scale), _ptr(scale),
                                  0 if scale is None else scale.numel(), _ptr(bias), bias_dtype, _ptr(out), out_code,
                                  M, N, K, x1.stride(0), x2.stride(0), x2.stride(1), out.stride(0), _ptr(workspace),
                                  0 if workspace is None else workspace.numel(), _stream())
    _check(st, "mi355_quant_matmul")
    return out


def transpose_int8(w: torch.Tensor) -> torch.Tensor:
    """w int8 [K, N] with unit column stride -> new int8 [N, K] contiguous (one transposing pass on the GPU)."""
    _need_gpu(w)
    assert w.dtype == torch.int8 and w.dim() == 2 and (w.numel() == 0 or w.stride(1) == 1)
    K, N = w.shape
    out = torch.empty((N, K), dtype=torch.int8, device=w.device)
    _check(lib().mi355_transpose_int8(_ptr(w), _ptr(out), K, N, w.stride(0) if K > 1 else max(N, 1), _stream()), "mi355_transpose_int8")
    return out


def trans_quant_param(scale, offset=None):
    """float32 scale [n] or [1] (and offset likewise) -> int64 [n] packed quantisation parameters."""
    _need_gpu(scale, offset)
    n = max(scale.numel(), 1 if offset is None else offset.numel())
    out = torch.empty((n,), dtype=torch.int64, device=scale.device)
    _check(lib().mi355_trans_quant_param(_ptr(scale), scale.numel(), _ptr(offset), 0 if offset is None else offset.numel(),
                                         _ptr(out), n, _stream()), "mi355_trans_quant_param")
    return out


def quant_matmul_qparam(x1, x2, qparam, bias=None, out_dtype=torch.int8, workspace=None):
    """x1 int8 [M,K]; x2 int8 [K,N] with strides (N,1) or (1,K); qparam int64 [N] or [1] from trans_quant_param."""
    _need_gpu(x1, x2, qparam, bias)
    M, K = x1.shape
    N = x2.shape[1]
    out = torch.empty((M, N), dtype=out_dtype, device=x1.device)
    need = lib().mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
    if workspace is None and need:
        workspace = _wq_workspace(x1.device, need)
    bias_dtype = 0 if bias is None else {torch.bfloat16: 1, torch.int32: 2, torch.float32: 3}[bias.dtype]
    out_code = {torch.bfloat16: 0, torch.float16: 2, torch.int8: 3}[out_dtype]
    st = lib().mi355_quant_matmul_qparam(_ptr(x1), _ptr(x2), _ptr(qparam), qparam.numel(), _ptr(bias), bias_dtype, _ptr(out),
                                         out_code, M, N, K, x1.stride(0), x2.stride(0), x2.stride(1), out.stride(0),
                                         _ptr(workspace), 0 if workspace is None else workspace.numel(), _stream())
    _check(st, "mi355_quant_matmul_qparam")
    return out


_wq_workspaces = {}
_wq_capture_workspaces = {}
_wq_retired = []        # superseded workspaces stay alive: a captured graph may still hold their address
ZERO_AREA_BYTES = (16 << 20) + 16384     # MI355_WORKSPACE_ZERO_BYTES (checked against the library when it loads a workspace)


def workspace_status(ws, reset: bool = True) -> None:
    """Waits for the current stream and raises Mi355Error if a kernel reported a failure through the sticky status word
    of workspace `ws` (a bounded wait for split-K partial sums ran out; the affected outputs hold NaN).  With `reset` the
    workspace's zero area is cleared so that it can be used again."""
    _check(lib().mi355_workspace_status(_ptr(ws), ws.numel(), 1 if reset else 0, _stream()), "mi355_workspace_status")


def check_workspaces(reset: bool = True) -> None:
    """workspace_status() for every workspace this module keeps for eager calls (one per device and stream)."""
    for ws in list(_wq_workspaces.values()) + list(_wq_retired):
        with torch.cuda.device(ws.device):
            workspace_status(ws, reset)


def _wq_workspace(device, nbytes: int):
    """Zero-initialised workspace reused across calls on one stream: the kernels need its leading zero area to start
    at zero and leave it zero.  A call made while the stream is capturing uses the stream's eager workspace when one
    exists (the operator ran on this stream before the capture); otherwise the capture gets a workspace of its own
    (allocated from the graph's pool, its zero fill recorded into the graph), which eager calls never see."""
    stream = torch.cuda.current_stream().cuda_stream
    key = (device.index, stream)
    want = max(nbytes, ZERO_AREA_BYTES + (1 << 20))
    cid = ctypes.c_ulonglong(0)
    _check(lib().mi355_stream_capture_id(ctypes.c_void_p(stream), ctypes.byref(cid)), "mi355_stream_capture_id")
    if cid.value:
        ws = _wq_workspaces.get(key)
        if ws is not None and ws.numel() >= nbytes:
            return ws
        ent = _wq_capture_workspaces.get(key)
        if ent is None or ent[0] != cid.value or ent[1].numel() < nbytes:
            ent = (cid.value, torch.zeros(want, dtype=torch.int8, device=device))
            _wq_capture_workspaces[key] = ent
        return ent[1]
    _wq_capture_workspaces.pop(key, None)
    ws = _wq_workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            workspace_status(ws)                   # a failure reported into the outgrown buffer must not be lost
            _wq_retired.append(ws)
            want = max(want, 2 * ws.numel())       # geometric growth: a stream retires a bounded number of buffers
        assert lib().mi355_workspace_zero_bytes() == ZERO_AREA_BYTES
        ws = torch.zeros(want, dtype=torch.int8, device=device)
        _wq_workspaces[key] = ws
    return ws


def weight_quant_matmul(x, weight, scale, offset=None, group_size: int = 0, bias=None):
    """x bf16/fp16 [M,K]; weight int8 [K,N] (strides (N,1) or (1,K)), int32 [K,N/8] (words along N) or int32 [K/8,N] with
    strides (1, K/8) (words along K: the transposed view of an [N,K/8] tensor); scale/offset of x's dtype, [N] or [G,N]
    with any strides (only the words-along-K kernel reads non-contiguous ones at full speed)."""
    _need_gpu(x, weight, scale, offset)
    M, K = x.shape
    if weight.dtype == torch.int32 and weight.shape[0] == K:
        bits, N = 4, weight.shape[1] * 8
        ldk, ldn = weight.stride(0), 1
    elif weight.dtype == torch.int32:
        assert weight.shape[0] * 8 == K and weight.stride(0) == 1, "words along K: pass the transposed view of [N, K/8]"
        bits, N = 4, weight.shape[1]
        ldk, ldn = 1, weight.stride(1)
    else:
        bits, N = 8, weight.shape[1]
        ldk, ldn = weight.stride(0), weight.stride(1)
    if offset is not None:
        assert offset.stride() == scale.stride()
    ldg, ldp = (0, scale.stride(0)) if scale.dim() == 1 else (scale.stride(0), scale.stride(1))
    out = torch.empty((M, N), dtype=x.dtype, device=x.device)
    need = lib().mi355_weight_quant_matmul_workspace(M, N, K, bits, group_size)
    ws = _wq_workspace(x.device, need) if need else None
    st = lib().mi355_weight_quant_matmul(_ptr(x), 1 if x.dtype == torch.float16 else 0, _ptr(weight), bits, _ptr(scale),
                                         _ptr(offset), _ptr(bias), _ptr(out),
                                         M, N, K, group_size, ldg, ldp, x.stride(0), ldk, ldn, out.stride(0), _ptr(ws),
                                         0 if ws is None else ws.numel(), _stream())
    _check(st, "mi355_weight_quant_matmul")
    return out


def swiglu(x):
    _need_gpu(x)
    rows, two = x.shape
    out = torch.empty((rows, two // 2), dtype=torch.bfloat16, device=x.device)
    _check(lib().mi355_swiglu(_ptr(x), _ptr(out), rows, two // 2, x.stride(0), _stream()), "mi355_swiglu")
    return out


def swiglu_quant(x, activate_left: bool = True, smooth=None, group_index=None):
    """x bf16 [rows, 2*half] -> (int8 [rows, half], float32 [rows]) = dynamic_quant(swiglu(x), smooth)."""
    _need_gpu(x, smooth)
    rows, two = x.shape
    y = torch.empty((rows, two // 2), dtype=torch.int8, device=x.device)
    scale = torch.empty((rows,), dtype=torch.float32, device=x.device)
    if group_index is not None:
        _check(lib().mi355_swiglu_quant_grouped(_ptr(x), 1 if activate_left else 0, _ptr(smooth), _ptr(group_index), group_index.numel(),
                                                _ptr(y), _ptr(scale), rows, two // 2, x.stride(0), _stream()), "mi355_swiglu_quant_grouped")
        return y, scale
    if smooth is not None:
        _check(lib().mi355_swiglu_quant_smooth(_ptr(x), 1 if activate_left else 0, _ptr(smooth), _ptr(y), _ptr(scale), rows,
                                               two // 2, x.stride(0), _stream()), "mi355_swiglu_quant_smooth")
        return y, scale
    _check(lib().mi355_swiglu_quant(_ptr(x), 1 if activate_left else 0, _ptr(y), _ptr(scale), rows, two // 2, x.stride(0),
                                    _stream()), "mi355_swiglu_quant")
    return y, scale


def anti_quant(x, scale, offset=None, dst_dtype=torch.float16):
    """x int8 [rows, cols] or int32 [rows, cols/8] (packed int4), scale / offset float32 [cols] or [1] ->
    dst_dtype [rows, cols] = (float(x) + offset) * scale."""
    assert x.dim() == 2 and x.stride(1) == 1
    bits = 4 if x.dtype == torch.int32 else 8
    rows, cols = x.shape[0], x.shape[1] * (8 if bits == 4 else 1)
    out = torch.empty((rows, cols), dtype=dst_dtype, device=x.device)
    _check(lib().mi355_anti_quant(_ptr(x), bits, _ptr(scale), scale.numel(), _ptr(offset), 0 if offset is None else offset.numel(),
                                  _ptr(out), 1 if dst_dtype == torch.float16 else 0, rows, cols, x.stride(0), cols, _stream()),
           "mi355_anti_quant")
    return out


_IN_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
_Q_CODE = {torch.int8: 0, torch.uint8: 1, torch.int32: 2}


def quantize(x, scale, zero_point=None, out_dtype=torch.int8, axis=-1, div_mode=True):
    """x bf16/fp16/fp32 (contiguous, any rank), scale float32, zero_point float32 or int32, [x.shape[axis]] or [1] ->
    out_dtype tensor of the same shape: clamp(rint(x / scale + zero_point)) (x * scale with div_mode False)."""
    _need_gpu(x, scale, zero_point)
    assert x.is_contiguous()
    axis = axis % x.dim()
    outer = 1
    for d in x.shape[:axis]:
        outer *= d
    inner = 1
    for d in x.shape[axis + 1:]:
        inner *= d
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    zp_code = 3 if zero_point is not None and zero_point.dtype == torch.int32 else 2
    _check(lib().mi355_quantize(_ptr(x), _IN_CODE[x.dtype], _ptr(scale), scale.numel(), _ptr(zero_point), zp_code,
                                0 if zero_point is None else zero_point.numel(), _ptr(out), _Q_CODE[out_dtype], outer,
                                x.shape[axis], inner, 1 if div_mode else 0, _stream()), "mi355_quantize")
    return out


def unpack_int4(x, out=None):
    """x int32 [rows, cols/8] (row pitch x.stride(0) words) -> int8 [rows, cols]; `out` may be a wider int8
    matrix whose rows receive the result."""
    _need_gpu(x, out)
    rows, words = x.shape
    if out is None:
        out = torch.empty((rows, words * 8), dtype=torch.int8, device=x.device)
    _check(lib().mi355_unpack_int4(_ptr(x), _ptr(out), rows, words * 8, x.stride(0), out.stride(0), _stream()),
           "mi355_unpack_int4")
    return out


def dynamic_quant_int4(x: torch.Tensor, smooth: torch.Tensor | None = None, group_index: torch.Tensor | None = None):
    """x bf16/fp16 [rows, cols] (cols % 8 == 0) -> (int32 [rows, cols / 8] of eight int4 codes each, scale float32 [rows])."""
    _need_gpu(x, smooth)
    assert x.dim() == 2 and (x.numel() == 0 or x.stride(1) == 1) and x.shape[1] % 8 == 0
    rows, cols = x.shape
    y = torch.empty((rows, cols // 8), dtype=torch.int32, device=x.device)
    scale = torch.zeros((rows,), dtype=torch.float32, device=x.device)
    _check(lib().mi355_dynamic_quant_int4(_ptr(x), 1 if x.dtype == torch.float16 else 0, _ptr(smooth), _ptr(group_index),
                                          0 if group_index is None else group_index.numel(), _ptr(y), _ptr(scale), rows, cols,
                                          x.stride(0) if rows > 1 else max(cols, 1), _stream()),
           "mi355_dynamic_quant_int4")
    return y, scale


def dynamic_quant_asymmetric(x: torch.Tensor, smooth: torch.Tensor | None = None, group_index: torch.Tensor | None = None):
    """x bf16/fp16 [rows, cols] (row pitch x.stride(0)) -> (int8 [rows, cols], scale float32 [rows], offset float32 [rows]).
    With group_index (int32 [E], running row totals per expert) smooth is [E, cols]."""
    _need_gpu(x, smooth)
    assert x.dim() == 2 and (x.numel() == 0 or x.stride(1) == 1)
    rows, cols = x.shape
    y = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    scale = torch.zeros((rows,), dtype=torch.float32, device=x.device)
    offset = torch.zeros((rows,), dtype=torch.float32, device=x.device)
    if group_index is not None:
        _check(lib().mi355_dynamic_quant_asymmetric_grouped(_ptr(x), 1 if x.dtype == torch.float16 else 0, _ptr(smooth),
                                                            _ptr(group_index), group_index.numel(), _ptr(y), _ptr(scale), _ptr(offset),
                                                            rows, cols, x.stride(0) if rows > 1 else max(cols, 1), _stream()),
               "mi355_dynamic_quant_asymmetric_grouped")
        return y, scale, offset
    _check(lib().mi355_dynamic_quant_asymmetric(_ptr(x), 1 if x.dtype == torch.float16 else 0, _ptr(smooth), _ptr(y), _ptr(scale),
                                                _ptr(offset), rows, cols, x.stride(0) if rows > 1 else max(cols, 1), _stream()),
           "mi355_dynamic_quant_asymmetric")
    return y, scale, offset
