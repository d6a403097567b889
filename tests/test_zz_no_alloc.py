"""The allocation-free entry point of quant_matmul against the ordinary one (GPU)."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _call(L, fn_noalloc, x1, x2, scale, ps, bias, out, workspace=None):
    M, K = x1.shape
    N = x2.shape[1]
    p = lambda t: None if t is None else ctypes.c_void_p(t.data_ptr())  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = (p(x1), p(x2), p(ps), p(scale), scale.numel(), p(bias), 0 if bias is None else 1, p(out), 0, M, N, K,
              x1.stride(0), x2.stride(0), x2.stride(1), out.stride(0))
    if fn_noalloc:
        return L.mi355_quant_matmul_noalloc(*common, stream)
    return L.mi355_quant_matmul(*common, p(workspace), 0 if workspace is None else workspace.numel(), stream)


def test_quant_matmul_noalloc_matches_workspace_entry_point():
    """Two calls in a row through the C ABI, the second with a smaller input (and the other weight layout, whose
    transposed copy also lives in the fixed scratch): bit-identical to mi355_quant_matmul with a caller workspace.
    Both shapes split K, so counters and partial sums of the scratch array are in use; the device allocator's
    counters must not move across the calls."""
    from pytorch_amd import _capi
    L = _capi.lib()
    g = torch.Generator().manual_seed(5)
    cases = [(64, 14336, 4096, True), (24, 4096, 1024, False)]
    prepared = []
    for (M, K, N, weight_nk) in cases:
        x1 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
        w = torch.randint(-127, 128, (N, K) if weight_nk else (K, N), generator=g, dtype=torch.int8).cuda()
        x2 = w.t() if weight_nk else w
        scale = (torch.rand(N, generator=g) * 9e-3 + 1e-3).cuda()
        ps = (torch.rand(M, generator=g) * 9e-3 + 1e-3).cuda()
        bias = (torch.randn(N, generator=g) * 0.02).to(torch.bfloat16).cuda()
        need = L.mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
        zone = 16 << 20                                  # exchange zone of the shared workspaces, absent from the private scratch
        assert 16384 + zone < need <= (16 << 20) + 16384 + zone, need
        ws = torch.zeros(need, dtype=torch.int8, device="cuda")
        want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        assert _call(L, False, x1, x2, scale, ps, bias, want, ws) == 0
        got = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
        prepared.append((x1, x2, scale, ps, bias, want, got))
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
    for (x1, x2, scale, ps, bias, want, got) in prepared:
        assert _call(L, True, x1, x2, scale, ps, bias, got) == 0
    torch.cuda.synchronize()
    after = torch.cuda.memory_stats()["allocation.all.allocated"], torch.cuda.mem_get_info()[0]
    assert before == after, (before, after)
    for (_, _, _, _, _, want, got) in prepared:
        assert torch.equal(got, want)
    # and once more in the opposite order: the scratch keeps the last call's contents, counters are back at zero
    for (x1, x2, scale, ps, bias, want, got) in reversed(prepared):
        got.fill_(3.0)
        assert _call(L, True, x1, x2, scale, ps, bias, got) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want)
    # a shape whose preferred plan (large tiles, K split four ways: 64 MiB of partial sums) does not fit the scratch: the
    # entry point plans within its scratch instead of refusing, and integer sums make the result the same bit for bit
    M, K, N = 1024, 14336, 4096
    x1 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    x2 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda().t()
    scale = (torch.rand(N, generator=g) * 9e-3 + 1e-3).cuda()
    ps = (torch.rand(M, generator=g) * 9e-3 + 1e-3).cuda()
    bias = (torch.randn(N, generator=g) * 0.02).to(torch.bfloat16).cuda()
    need = L.mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
    assert need > (32 << 20) + 16384, need
    ws = torch.zeros(need, dtype=torch.int8, device="cuda")
    want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    got = torch.full((M, N), 3.0, dtype=torch.bfloat16, device="cuda")
    assert _call(L, False, x1, x2, scale, ps, bias, want, ws) == 0
    assert _call(L, True, x1, x2, scale, ps, bias, got) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # a request beyond the fixed scratch is refused with the workspace status, nothing is launched
    M, K, N = 16, 8192, 8192                          # [K,N] weight: 64 MiB transposed copy
    x1 = torch.zeros((M, K), dtype=torch.int8, device="cuda")
    x2 = torch.zeros((K, N), dtype=torch.int8, device="cuda")
    out = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    sc = torch.ones(N, device="cuda")
    assert _call(L, True, x1, x2, sc, None, None, out) == -4


def test_quant_matmul_noalloc_under_graph_capture():
    """The entry point exists for callers that cannot allocate, graph capture among them: two calls (a split-K shape and
    a smaller one) are captured on a fresh stream and replayed three times with eager work and synchronisations between
    the replays; every replay reproduces the bits of mi355_quant_matmul with a caller workspace."""
    from pytorch_amd import _capi
    L = _capi.lib()
    g = torch.Generator().manual_seed(9)
    cases = []
    for (M, K, N) in [(64, 14336, 4096), (40, 4096, 512)]:
        x1 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
        x2 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda().t()
        scale = (torch.rand(N, generator=g) * 9e-3 + 1e-3).cuda()
        ps = (torch.rand(M, generator=g) * 9e-3 + 1e-3).cuda()
        bias = (torch.randn(N, generator=g) * 0.02).to(torch.bfloat16).cuda()
        need = L.mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
        ws = torch.zeros(max(need, 16), dtype=torch.int8, device="cuda")
        want = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        assert _call(L, False, x1, x2, scale, ps, bias, want, ws if need else None) == 0
        got = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        cases.append((x1, x2, scale, ps, bias, want, got))
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        for (x1, x2, scale, ps, bias, want, got) in cases:
            assert _call(L, True, x1, x2, scale, ps, bias, got) == 0
    for it in range(3):
        for c in cases:
            c[6].fill_(1.0)
        graph.replay()
        torch.cuda.synchronize()
        for c in cases:
            assert torch.equal(c[6], c[5]), f"replay {it}"
        # eager work of the same entry point between the replays
        x1, x2, scale, ps, bias, want, got = cases[it % 2]
        eager = torch.zeros_like(want)
        assert _call(L, True, x1, x2, scale, ps, bias, eager) == 0
        torch.cuda.synchronize()
        assert torch.equal(eager, want)


def test_quant_matmul_noalloc_int32_output_and_forced_split():
    """An int32 output (raw accumulators) through the scratch array, and a split of K forced through the tuning knob: the
    forced split is held to the scratch's capacity like a planned one (here it fits), results equal to the ordinary entry
    point's."""
    from pytorch_amd import _capi
    L = _capi.lib()
    g = torch.Generator().manual_seed(11)
    M, K, N = 96, 8192, 1024
    x1 = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    x2 = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda().t()
    p = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    ref = torch.empty((M, N), dtype=torch.int32, device="cuda")
    need = L.mi355_quant_matmul_workspace(M, N, K, x2.stride(0), x2.stride(1))
    ws = torch.zeros(max(need, 16), dtype=torch.int8, device="cuda")
    args = (p(x1), p(x2), None, None, 0, None, 0)
    tail = (1, M, N, K, x1.stride(0), x2.stride(0), x2.stride(1), N)
    assert L.mi355_quant_matmul(*args, p(ref), *tail, p(ws), ws.numel(), stream) == 0
    for split in (0, 4):
        _capi.set_tuning("MI355_QMM_SPLIT", split)
        try:
            got = torch.full((M, N), 7, dtype=torch.int32, device="cuda")
            assert L.mi355_quant_matmul_noalloc(*args, p(got), *tail, stream) == 0
            torch.cuda.synchronize()
            assert torch.equal(got, ref), split
        finally:
            _capi.set_tuning("MI355_QMM_SPLIT", 0)
    import numpy as np
    from oracle import golden
    assert np.array_equal(ref.cpu().numpy(), golden.int8_gemm(x1.cpu().numpy(), x2.cpu().numpy()))
