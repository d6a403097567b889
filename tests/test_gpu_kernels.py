"""GPU parity tests: the HIP kernels, called through the C ABI, against the CPU oracle on
the same seeded inputs.  int8 codes, float32 row scales and int32 accumulators must be
bit-exact; bf16 outputs must pass the bf16 gate (>= 99.9 % within one bf16 ulp of the
float32 golden, no element outside 1e-2 abs-or-rel)."""
import numpy as np
import pytest
import torch

from pytorch_amd.testing import workloads, bf16_gate

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from pytorch_amd import _capi
    _capi.lib()
    return _capi


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


# ------------------------------------------------------------------ dynamic_quant

@pytest.mark.parametrize("rows,cols", [(2048, 4096), (64, 14336), (7, 512), (33, 1024), (5, 8), (3, 40), (2, 16384),
                                       (2, 20000), (9, 100), (1, 1), (5, 28672), (3, 32776), (2, 65536), (2, 65544),
                                       (3, 16388)])
def test_dynamic_quant_bit_exact(capi, golden, rows, cols):
    x = workloads.dynamic_quant_input(seed=rows + cols, rows=rows, cols=cols)
    y, s = capi.dynamic_quant(x.cuda())
    yg, sg = golden.dynamic_quant(_bits(x))
    assert np.array_equal(s.cpu().numpy(), sg)
    assert np.array_equal(y.cpu().numpy(), yg)


def test_dynamic_quant_fp16_and_strided(capi, golden):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(40, 2048, generator=g) * 5).to(torch.float16)
    y, s = capi.dynamic_quant(x.cuda())
    yg, sg = golden.dynamic_quant(_bits(x), in_dtype="fp16")
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)
    xb = workloads.dynamic_quant_input(seed=1, rows=16, cols=4096)
    view = xb.cuda()[:, :1024]                      # row stride 4096, 1024 columns
    y, s = capi.dynamic_quant(view)
    yg, sg = golden.dynamic_quant(_bits(xb[:, :1024]))
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)


def test_dynamic_quant_exhaustive_significands(capi, golden):
    """Every bf16 significand of the row maximum x every bf16 value that can round to a non-zero
    code, at several exponents including ones outside the fast-path range."""
    rows = []
    for e in (-100, -62, -30, -1, 0, 7, 40, 63, 100):
        for ma in range(128):
            amax = np.float32((1 + ma / 128.0) * 2.0 ** e)
            vals = [amax]
            for de in range(0, 10):
                for mx in range(128):
                    v = np.float32((1 + mx / 128.0) * 2.0 ** (e - de))
                    if v <= amax:
                        vals.append(v)
            rows.append(np.array(vals, np.float32))
    width = max(len(r) for r in rows)
    width = (width + 7) // 8 * 8
    mat = np.zeros((len(rows), width), np.float32)
    for i, r in enumerate(rows):
        mat[i, :len(r)] = r
        mat[i, 1:len(r):2] *= -1
    x = torch.from_numpy(mat).to(torch.bfloat16)
    assert torch.equal(x.float(), torch.from_numpy(mat))
    y, s = capi.dynamic_quant(x.cuda())
    yg, sg = golden.dynamic_quant(_bits(x))
    assert np.array_equal(s.cpu().numpy(), sg)
    assert np.array_equal(y.cpu().numpy(), yg)


def test_dynamic_quant_edge_cases(capi, golden):
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    x[1, 3] = -3.0
    x[2] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.5] * 8)
    y, s = capi.dynamic_quant(x.cuda())
    assert s.cpu().tolist()[0] == 0.0 and not y[0].any()
    assert y[1, 3].item() == -127
    assert y[2, :8].cpu().tolist() == [127, 0, 2, 2, 0, -2, -2, 4]
    yg, sg = golden.dynamic_quant(_bits(x))
    assert np.array_equal(y.cpu().numpy(), yg) and np.array_equal(s.cpu().numpy(), sg)
    e = torch.empty(0, 128, dtype=torch.bfloat16, device="cuda")
    y, s = capi.dynamic_quant(e)
    assert y.shape == (0, 128) and s.shape == (0,)
    x3 = workloads.dynamic_quant_input(seed=3, rows=24, cols=256).reshape(2, 12, 256)
    y, s = capi.dynamic_quant(x3.cuda())
    assert y.shape == (2, 12, 256) and s.shape == (2, 12)


def test_dynamic_quant_smooth(capi, golden):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(8, 512, generator=g).to(torch.bfloat16)
    sm = (torch.rand(512, generator=g) + 0.5).to(torch.bfloat16)
    y, s = capi.dynamic_quant(x.cuda(), sm.cuda())
    yg, sg = golden.dynamic_quant(_bits(x), smooth_u16=_bits(sm))
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (33, 8192), (7, 24), (64, 14336), (5, 1000), (3, 8200), (5, 28672),
                                       (3, 65536), (3, 65544)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_dynamic_quant_smooth_shapes(capi, golden, rows, cols, dt):
    """Smooth scales through the register-resident kernels (cols % 8 == 0, up to 65536) and the two-pass one (wider or odd
    rows), both input types, with rows that hold zeros, a zero row, tiny and huge values (both division paths of the
    kernel), bit-exact against the oracle."""
    g = torch.Generator().manual_seed(rows + cols)
    x = torch.randn(rows, cols, generator=g) * 3
    x[0] = 0
    if rows > 2:
        x[1, :8] = torch.tensor([1e-30, -1e-30, 0.0, 6e4, -6e4, 1e-7, 0.5, -0.5])     # tiny numerators next to a large maximum
        x[2] = x[2] * 1e-6
    x = x.to(dt)
    sm = (torch.rand(cols, generator=g) * 4 + 0.01).to(dt)
    y, s = capi.dynamic_quant(x.cuda(), sm.cuda())
    yg, sg = golden.dynamic_quant(_bits(x), "fp16" if dt == torch.float16 else "bf16", _bits(sm))
    assert np.array_equal(s.cpu().numpy(), sg)
    assert np.array_equal(y.cpu().numpy(), yg)


@pytest.mark.parametrize("rows,cols,totals", [(64, 4096, [10, 10, 37, 64]), (33, 1000, [0, 33]), (20, 8200, [5, 9, 12]),
                                              (128, 14336, [1, 2, 3, 4, 100, 128]), (7, 512, [7])])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_dynamic_quant_per_expert_smooth_scales(capi, golden, rows, cols, totals, dt):
    """group_index of npu_dynamic_quant (signature test/test_fake_tensor.py:1670-1687): smooth_scales [E, cols], the
    running row totals per expert select a row's scales.  Empty experts, totals short of the row count (the rest takes the
    last expert) and a single expert; register-resident and two-pass kernels; bit-exact against the oracle, which
    quantises every expert's rows separately with dynamic_quant."""
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * 3).to(dt)
    sm = (torch.rand(len(totals), cols, generator=g) * 4 + 0.01).to(dt)
    gi = torch.tensor(totals, dtype=torch.int32)
    y, s = capi.dynamic_quant(x.cuda(), sm.cuda(), gi.cuda())
    yg, sg = golden.dynamic_quant_grouped(_bits(x), _bits(sm), totals, "fp16" if dt == torch.float16 else "bf16")
    assert np.array_equal(s.cpu().numpy(), sg)
    assert np.array_equal(y.cpu().numpy(), yg)
    # one expert = the plain smooth-scale call
    y1, s1 = capi.dynamic_quant(x.cuda(), sm[:1].contiguous().cuda(), torch.tensor([rows], dtype=torch.int32).cuda())
    y0, s0 = capi.dynamic_quant(x.cuda(), sm[0].contiguous().cuda())
    assert torch.equal(y1, y0) and torch.equal(s1, s0)


@pytest.mark.parametrize("rows,cols", [(64, 4096), (5, 1000), (3, 24), (33, 14336)])
@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float16])
def test_dynamic_quant_int4_output(capi, golden, rows, cols, dt):
    """dst_type=torch.quint4x2 through the C ABI: packed int4 codes and scales bit-exact against the oracle, plain, with
    smooth scales and with per-expert smooth scales; a zero row, tiny values, rows that use every code."""
    name = "fp16" if dt == torch.float16 else "bf16"
    g = torch.Generator().manual_seed(rows * 7 + cols)
    x = torch.randn(rows, cols, generator=g) * 3
    x[0] = 0
    x[1] = x[1] * 1e-6
    x = x.to(dt)
    y, s = capi.dynamic_quant_int4(x.cuda())
    yg, sg = golden.dynamic_quant_int4(_bits(x), name)
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)
    codes = golden.unpack_int4(yg)
    assert codes.min() == -7 and codes.max() == 7
    sm = (torch.rand(2, cols, generator=g) * 4 + 0.01).to(dt)
    y, s = capi.dynamic_quant_int4(x.cuda(), sm[0].contiguous().cuda())
    yg, sg = golden.dynamic_quant_int4(_bits(x), name, _bits(sm[0]))
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)
    cut = rows // 2
    y, s = capi.dynamic_quant_int4(x.cuda(), sm.cuda(), torch.tensor([cut, rows], dtype=torch.int32).cuda())
    for lo, hi, e in ((0, cut, 0), (cut, rows, 1)):
        yg, sg = golden.dynamic_quant_int4(_bits(x[lo:hi]), name, _bits(sm[e]))
        assert np.array_equal(s[lo:hi].cpu().numpy(), sg) and np.array_equal(y[lo:hi].cpu().numpy(), yg)


@pytest.mark.parametrize("rows,cols,totals", [(64, 4096, [10, 10, 37, 64]), (20, 8200, [5, 9, 12]), (9, 1000, [9])])
def test_dynamic_quant_asymmetric_per_expert_smooth_scales(capi, golden, rows, cols, totals):
    """group_index of npu_dynamic_quant_asymmetric: as for the symmetric operator, bit-exact against the oracle applied per
    expert (register-resident, vector and scalar kernels)."""
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn(rows, cols, generator=g) * 3 + 0.5).to(torch.bfloat16)
    sm = (torch.rand(len(totals), cols, generator=g) * 4 + 0.01).to(torch.bfloat16)
    y, s, o = capi.dynamic_quant_asymmetric(x.cuda(), sm.cuda(), torch.tensor(totals, dtype=torch.int32).cuda())
    yg, sg, og = golden.dynamic_quant_asymmetric_grouped(_bits(x), _bits(sm), totals)
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(o.cpu().numpy(), og)
    assert np.array_equal(y.cpu().numpy(), yg)


@pytest.mark.parametrize("rows,half,totals", [(48, 2048, [10, 10, 30, 48]), (20, 8200, [4, 20]), (9, 500, [2, 5, 9])])
def test_swiglu_quant_per_expert_smooth_scales(capi, golden, rows, half, totals):
    """group_index of npu_swiglu_quant: the SwiGLU of a row is multiplied by its expert's smooth scales before the row is
    quantised; bit-exact against dynamic_quant_grouped(swiglu(x)) of the oracle (vector and scalar kernels)."""
    g = torch.Generator().manual_seed(rows + half)
    x = (torch.randn(rows, 2 * half, generator=g) * 2).to(torch.bfloat16)
    sm = (torch.rand(len(totals), half, generator=g) * 4 + 0.01).to(torch.bfloat16)
    y, s = capi.swiglu_quant(x.cuda(), True, sm.cuda(), torch.tensor(totals, dtype=torch.int32).cuda())
    yg, sg = golden.dynamic_quant_grouped(golden.swiglu(_bits(x)), _bits(sm), totals)
    assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)


# ------------------------------------------------------------------ quant_matmul

QMM_SHAPES = [(1024, 4096, 1024), (256, 512, 352), (64, 4096, 512), (100, 256, 200), (1, 128, 16), (300, 1024, 1000),
              (17, 96, 33), (2048, 256, 4096)]


@pytest.mark.parametrize("M,K,N", QMM_SHAPES)
@pytest.mark.parametrize("weight_nk", [True, False])
def test_quant_matmul_accumulators_bit_exact(capi, golden, M, K, N, weight_nk):
    d = workloads.quant_matmul_inputs(seed=M + N, M=M, K=K, N=N, weight_nk=weight_nk)
    acc = capi.quant_matmul(d["x1"].cuda(), d["x2"].cuda(), None, out_dtype=torch.int32)
    want = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    assert np.array_equal(acc.cpu().numpy(), want)


@pytest.mark.parametrize("M,K,N", QMM_SHAPES[:6])
@pytest.mark.parametrize("bias", [True, False])
def test_quant_matmul_bf16(capi, golden, M, K, N, bias):
    d = workloads.quant_matmul_inputs(seed=7 + M, M=M, K=K, N=N, weight_nk=True, bias=bias)
    out = capi.quant_matmul(d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), d["pertoken_scale"].cuda(),
                            None if not bias else d["bias"].cuda())
    want, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(),
                                  None if not bias else _bits(d["bias"]))
    assert np.array_equal(_bits(out), want)      # same operation order => bit-identical bf16


REQUANT_SHAPES = [(1024, 4096, 11008), (64, 4096, 1024), (48, 256, 192), (130, 384, 1000), (17, 100, 37), (256, 1024, 320),
                  (1, 4096, 4096), (16, 1152, 2056), (33, 2048, 4104), (5, 14336, 4096)]


@pytest.mark.parametrize("M,K,N", REQUANT_SHAPES)
@pytest.mark.parametrize("weight_nk", [True, False])
def test_quant_matmul_int8_output(capi, golden, M, K, N, weight_nk):
    """The re-quantised int8 output through mi355_trans_quant_param + mi355_quant_matmul_qparam, bit-exact against the
    oracle: tiled kernel (every tile shape these sizes select, split K at M=64), the generic kernel (K=100), the decode
    kernel (the last four shapes with the weight stored [N, K]), with and without an int32 bias, per-channel and single
    parameters, offsets that clamp and .5 ties."""
    d = workloads.quant_matmul_inputs(seed=M + N, M=M, K=K, N=N, weight_nk=weight_nk)
    g = torch.Generator().manual_seed(K)
    acc_scale = 40.0 / (K ** 0.5 * 74 * 74)                       # spreads the results over the int8 range
    scale = (torch.rand(N, generator=g) + 0.5) * acc_scale
    scale[: min(4, N)] = 0.5                                       # exact halves: ties to even
    offset = torch.randint(-30, 30, (N,), generator=g).float() + torch.rand(N, generator=g)
    bias = torch.randint(-5000, 5000, (N,), generator=g, dtype=torch.int32)
    x1, x2 = d["x1"].cuda(), d["x2"].cuda()
    for sc, of, b in ((scale, offset, bias), (scale, None, None), (scale[:1].clone(), offset[:1].clone(), bias)):
        qp = capi.trans_quant_param(sc.cuda(), None if of is None else of.cuda())
        want_q = golden.trans_quant_param(sc.numpy(), None if of is None else of.numpy())
        assert np.array_equal(qp.cpu().numpy(), want_q)
        got = capi.quant_matmul_qparam(x1, x2, qp, None if b is None else b.cuda(), torch.int8)
        qfull = np.repeat(want_q, N) if want_q.size == 1 else want_q
        want = golden.quant_matmul_requant(d["x1"].numpy(), d["x2"].numpy(), qfull, None if b is None else b.numpy())
        assert got.dtype == torch.int8
        assert np.array_equal(got.cpu().numpy(), want)
        assert np.abs(want.astype(np.int32)).max() > 20           # not everything collapsed to zero


def test_quant_matmul_packed_scale_float_outputs(capi, golden):
    """A packed scale with fp16 / bf16 output equals the float32-scale path bit for bit (the offset field is ignored)."""
    d = workloads.quant_matmul_inputs(seed=11, M=96, K=512, N=384, weight_nk=True)
    off = torch.full((384,), 7.0)
    qp = capi.trans_quant_param(d["scale"].cuda(), off.cuda())
    for dt in (torch.float16, torch.bfloat16):
        a = capi.quant_matmul_qparam(d["x1"].cuda(), d["x2"].cuda(), qp, None, dt)
        b = capi.quant_matmul(d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), None, None, dt)
        assert torch.equal(a, b)
    L = capi.lib()
    import ctypes
    vp = ctypes.c_void_p
    x1, x2 = d["x1"].cuda(), d["x2"].cuda()
    out = torch.empty(96, 384, dtype=torch.int8, device="cuda")
    # int8 output without packed parameters, and an int32 output through the packed entry point, are refused
    assert L.mi355_quant_matmul(vp(x1.data_ptr()), vp(x2.data_ptr()), None, vp(d["scale"].cuda().data_ptr()), 384, None, 0,
                                vp(out.data_ptr()), 3, 96, 384, 512, 512, 1, 512, 384, None, 0, None) == -1
    assert L.mi355_quant_matmul_qparam(vp(x1.data_ptr()), vp(x2.data_ptr()), vp(qp.data_ptr()), 384, None, 0,
                                       vp(out.data_ptr()), 1, 96, 384, 512, 512, 1, 512, 384, None, 0, None) == -1


def test_quant_matmul_random_shapes(capi, golden):
    """Seeded sweep over shapes (tiled, split over K, generic), weight layouts, bias kinds and output types: int32
    accumulators and rounded outputs bit-identical to the oracle."""
    import os
    rng = np.random.default_rng(7)
    for case in range(int(os.environ.get("MI355_SWEEP_CASES", "64"))):
        M = int(rng.choice([1, 7, 16, 33, 64, 100, 128, 200, 256, 300, 513]))
        K = int(rng.choice([16, 100, 128, 256, 384, 1024, 2048, 4096]))
        N = int(rng.choice([8, 33, 64, 128, 200, 256, 352, 512, 1000, 1536]))
        nk = bool(rng.random() < 0.6)
        kind = str(rng.choice(["none", "bf16", "i32", "f32"]))
        out_name = str(rng.choice(["bf16", "fp16", "int32"]))
        if out_name == "int32" and kind in ("bf16", "f32"):
            kind = "none"
        if out_name == "fp16" and kind == "bf16":
            kind = "f32"
        d = workloads.quant_matmul_inputs(seed=case, M=M, K=K, N=N, weight_nk=nk, bias=True)
        g = torch.Generator().manual_seed(case)
        bias = {"none": None, "bf16": d["bias"], "i32": torch.randint(-(1 << 20), 1 << 20, (N,), generator=g, dtype=torch.int32),
                "f32": torch.randn(N, generator=g)}[kind]
        dt = {"bf16": torch.bfloat16, "fp16": torch.float16, "int32": torch.int32}[out_name]
        tag = f"case {case}: M={M} K={K} N={N} nk={nk} bias={kind} out={out_name}"
        acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
        try:
            if out_name == "int32":
                out = capi.quant_matmul(d["x1"].cuda(), d["x2"].cuda(), None, None, None if bias is None else bias.cuda(),
                                        out_dtype=dt)
                want = acc if bias is None else (acc.astype(np.int64) + bias.numpy().astype(np.int64)).astype(np.int32)
                assert np.array_equal(out.cpu().numpy(), want), tag
            else:
                out = capi.quant_matmul(d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), d["pertoken_scale"].cuda(),
                                        None if bias is None else bias.cuda(), out_dtype=dt)
                b = None if bias is None else (_bits(bias) if kind == "bf16" else bias.numpy())
                want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy(), b, out=out_name)
                got = out.cpu().view(torch.int16).numpy().view(np.uint16)
                assert np.array_equal(got, want), tag
        except capi.Mi355Error as e:
            raise AssertionError(f"{tag}: {e}")


def test_quant_matmul_extreme_accumulators(capi, golden):
    M, K, N = 64, 4096, 64
    a = torch.full((M, K), 127, dtype=torch.int8)
    b = torch.full((N, K), -127, dtype=torch.int8).t()
    acc = capi.quant_matmul(a.cuda(), b.cuda(), None, out_dtype=torch.int32)
    assert (acc == -K * 16129).all()
    one = torch.ones(N, device="cuda")
    out = capi.quant_matmul(a.cuda(), b.cuda(), one, None, None)
    assert (out.float() == torch.tensor(float(-K * 16129)).to(torch.bfloat16).float()).all()
    half = capi.quant_matmul(a.cuda(), b.cuda(), torch.tensor([0.5], device="cuda"), None, None)
    want, _ = golden.quant_matmul(a.numpy(), b.numpy(), np.array([0.5], np.float32))
    assert np.array_equal(_bits(half), want)


@pytest.mark.parametrize("M,K,N", [(256, 512, 352), (64, 4096, 512), (100, 256, 200), (17, 96, 33)])
def test_quant_matmul_bias_kinds_and_fp16_output(capi, golden, M, K, N):
    """int32 bias (LinearQuant's default, added to the accumulator), float32 bias, fp16 output, int32 output with bias:
    bit-identical to the oracle's statement of the same formula."""
    d = workloads.quant_matmul_inputs(seed=11 + M, M=M, K=K, N=N, weight_nk=True, bias=True)
    g = torch.Generator().manual_seed(M)
    bias_i32 = torch.randint(-(1 << 20), 1 << 20, (N,), generator=g, dtype=torch.int32)
    bias_f32 = torch.randn(N, generator=g)
    x1, x2, sc, ps = d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), d["pertoken_scale"].cuda()
    acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    cases = [(bias_i32, torch.bfloat16, "bf16"), (bias_f32, torch.bfloat16, "bf16"), (bias_i32, torch.float16, "fp16"),
             (None, torch.float16, "fp16"), (bias_f32, torch.float16, "fp16")]
    for bias, dt, name in cases:
        out = capi.quant_matmul(x1, x2, sc, ps, None if bias is None else bias.cuda(), out_dtype=dt)
        want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy(),
                                               None if bias is None else bias.numpy(), out=name)
        assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), want), (name, None if bias is None else bias.dtype)
    out = capi.quant_matmul(x1, x2, None, None, bias_i32.cuda(), out_dtype=torch.int32)
    assert np.array_equal(out.cpu().numpy(), golden.quant_matmul_epilogue_ex(acc, None, None, bias_i32.numpy(), out="int32"))


@pytest.mark.parametrize("tile", [64128, 64256])
@pytest.mark.parametrize("M,K,N", [(64, 128, 1000), (33, 384, 520), (64, 4096, 2048), (16, 2048, 8200)])
def test_quant_matmul_deep_ring_small_tiles(capi, golden, tile, M, K, N):
    """Launches with at most one 64-row tile per CU do not rely on a second resident workgroup: the 64x128 tile streams its
    weight rows straight into registers (no workgroup ring), the 64x256 tile uses a ring of whole stages several steps
    ahead.  Fewer K steps than ring slots / register steps, ragged columns and rows, with and without a K split;
    accumulators bit-identical to the oracle and outputs to the shallow-ring kernel."""
    d = workloads.quant_matmul_inputs(seed=M + N, M=M, K=K, N=N, weight_nk=True, bias=True)
    x1, x2 = d["x1"].cuda(), d["x2"].cuda()
    want = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    capi.set_tuning("MI355_QMM_TILE", tile)
    try:
        for split in (0, 2):
            if split and K // 128 < split:
                continue
            capi.set_tuning("MI355_QMM_SPLIT", split)
            outs = []
            for deep_off in (0, 1, 2):      # streaming loop (64x128) / deep ring (64x256); two resident workgroups; deep ring
                capi.set_tuning("MI355_QMM_DEEP_OFF", deep_off)
                acc = capi.quant_matmul(x1, x2, None, out_dtype=torch.int32)
                assert np.array_equal(acc.cpu().numpy(), want), (tile, split, deep_off)
                outs.append(capi.quant_matmul(x1, x2, d["scale"].cuda(), d["pertoken_scale"].cuda(), d["bias"].cuda()))
            assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    finally:
        for k in ("MI355_QMM_TILE", "MI355_QMM_SPLIT", "MI355_QMM_DEEP_OFF"):
            capi.set_tuning(k, 0)


@pytest.mark.parametrize("tile", [256192, 256224, 256256, 128128, 128192])
@pytest.mark.parametrize("M,K,N", [(256, 128, 192), (300, 640, 500), (512, 4224, 1000), (1024, 1152, 2300), (255, 2048, 8 * 97),
                                   (520, 1152, 16 * 129)])
def test_quant_matmul_wide_loop_tiles(capi, golden, tile, M, K, N):
    """The 256-row tiles run the K loop with loader roles (activation slots released by an LDS flag between the two
    wavefronts that read them).  One K step, odd and even step counts, ragged rows and columns, with and without a split of
    K, both instruction orders: int32 accumulators bit-identical to the oracle, every epilogue (the LDS-parameter one for
    per-token scale + bf16 bias / no bias in bf16 and fp16, the LDS-parameter one for the re-quantised int8 output when the
    output rows are 16-byte aligned, and the general one for the other bias kinds, a single scale, no per-token scale, int32
    and unaligned int8 outputs) bit-identical to the generic loop and to the oracle.  (The
    256x256 tile, which only has the generic loop, runs through the same cases against the oracle; the 128x128 and 128x192
    tiles run their variant with three whole stages, MI355_QMM_LOOP = 4, against their usual rings.)"""
    d = workloads.quant_matmul_inputs(seed=M + N + K, M=M, K=K, N=N, weight_nk=True, bias=True)
    g = torch.Generator().manual_seed(M + K)
    x1, x2, sc, ps, bias = (d[k].cuda() for k in ("x1", "x2", "scale", "pertoken_scale", "bias"))
    bias_i32 = torch.randint(-(1 << 20), 1 << 20, (N,), generator=g, dtype=torch.int32).cuda()
    bias_f32 = torch.randn(N, generator=g).cuda()
    one = torch.tensor([3e-3], device="cuda")
    off = torch.randint(-20, 20, (N,), generator=g).float()
    qp = capi.trans_quant_param((d["scale"] * 1e-2).cuda(), off.cuda())
    acc_want = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    want_bf16, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(), _bits(d["bias"]))
    want_i8 = golden.quant_matmul_requant(d["x1"].numpy(), d["x2"].numpy(), golden.trans_quant_param((d["scale"] * 1e-2).numpy(), off.numpy()),
                                          bias_i32.cpu().numpy())

    def run_all():
        return [capi.quant_matmul(x1, x2, None, out_dtype=torch.int32),
                capi.quant_matmul(x1, x2, sc, ps, bias),
                capi.quant_matmul(x1, x2, sc, ps, None),
                capi.quant_matmul(x1, x2, sc, ps, bias, out_dtype=torch.float16),
                capi.quant_matmul(x1, x2, sc, ps, None, out_dtype=torch.float16),
                capi.quant_matmul(x1, x2, sc, ps, bias_f32),
                capi.quant_matmul(x1, x2, sc, ps, bias_i32),
                capi.quant_matmul(x1, x2, sc, None, bias),
                capi.quant_matmul(x1, x2, one, ps, bias),
                capi.quant_matmul(x1, x2, None, None, bias_i32, out_dtype=torch.int32),
                capi.quant_matmul_qparam(x1, x2, qp, bias_i32),
                capi.quant_matmul_qparam(x1, x2, qp, None, out_dtype=torch.bfloat16),
                capi.quant_matmul_qparam(x1, x2, qp, None),
                capi.quant_matmul_qparam(x1, x2, qp, bias_i32, out_dtype=torch.float16),
                capi.quant_matmul(x1, x2, one, None, bias_f32)]

    capi.set_tuning("MI355_QMM_TILE", tile)
    try:
        for split in (0, 2, 3):
            if split and K // 128 < split:
                continue
            capi.set_tuning("MI355_QMM_SPLIT", split)
            capi.set_tuning("MI355_QMM_LOOP", 1)            # the generic loop on the same tile
            ref = run_all()
            assert np.array_equal(ref[0].cpu().numpy(), acc_want), (tile, split)
            assert np.array_equal(_bits(ref[1]), want_bf16), (tile, split)
            assert np.array_equal(ref[10].cpu().numpy(), want_i8), (tile, split)
            for order in ((2, 3) if tile >= 256000 else (4,)):
                capi.set_tuning("MI355_QMM_LOOP", order)
                for stream_out in (1, 2):                   # ordinary / non-temporal row stores of the 16-bit epilogue
                    capi.set_tuning("MI355_QMM_STREAM_OUT", stream_out)
                    got = run_all()
                    for i, (a, b) in enumerate(zip(got, ref)):
                        assert torch.equal(a, b), (tile, split, order, stream_out, i)
                capi.set_tuning("MI355_QMM_STREAM_OUT", 0)
    finally:
        for k in ("MI355_QMM_TILE", "MI355_QMM_SPLIT", "MI355_QMM_LOOP", "MI355_QMM_STREAM_OUT"):
            capi.set_tuning(k, 0)


def test_quant_matmul_wide_loop_strided_operands(capi, golden):
    """Row pitches larger than the rows (views into wider buffers) and an output view whose rows are not 16-byte aligned
    (the general epilogue): the wide loop addresses rows through the pitches only."""
    M, K, N = 512, 1024, 384
    d = workloads.quant_matmul_inputs(seed=5, M=M, K=K, N=N, weight_nk=True, bias=True)
    xa = torch.zeros((M, K + 256), dtype=torch.int8, device="cuda")
    xa[:, :K] = d["x1"].cuda()
    wb = torch.zeros((N, K + 128), dtype=torch.int8, device="cuda")
    wb[:, :K] = d["x2"].t().cuda()
    want, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(), _bits(d["bias"]))
    capi.set_tuning("MI355_QMM_TILE", 256192)
    try:
        out = capi.quant_matmul(xa[:, :K], wb[:, :K].t(), d["scale"].cuda(), d["pertoken_scale"].cuda(), d["bias"].cuda())
        assert np.array_equal(_bits(out), want)
    finally:
        capi.set_tuning("MI355_QMM_TILE", 0)


def test_quant_matmul_split_k_repeated_launches(capi, golden):
    """A narrow output with a long K is split over K (workgroups meet at counters in the shared workspace): the
    down-projection shape of the MLP configuration, launched repeatedly on the same zero-initialised workspace."""
    M, K, N = 64, 14336, 4096
    assert capi.lib().mi355_quant_matmul_workspace(M, N, K, 1, K) > 0        # this shape does split
    for seed in (1, 2, 3):
        d = workloads.quant_matmul_inputs(seed=seed, M=M, K=K, N=N, weight_nk=True, bias=True)
        x1, x2 = d["x1"].cuda(), d["x2"].cuda()
        acc = capi.quant_matmul(x1, x2, None, out_dtype=torch.int32)
        assert np.array_equal(acc.cpu().numpy(), golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy()))
        out = capi.quant_matmul(x1, x2, d["scale"].cuda(), d["pertoken_scale"].cuda(), d["bias"].cuda())
        want, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(),
                                      _bits(d["bias"]))
        assert np.array_equal(_bits(out), want)


@pytest.mark.parametrize("M,K,N", [(512, 14336, 4096), (1024, 14336, 4096), (256, 8192, 8192), (128, 4096, 28672), (304, 5120, 1000)])
def test_quant_matmul_long_k_plans(capi, M, K, N):
    """Shapes on which the planner picks large tiles with a split of K (256x256 four ways, 128x256 four ways and two ways):
    accumulators against an exact float64 evaluation on the GPU (products and partial sums of 4096 terms are exact in
    float64), outputs against the same formula in separately rounded float32 tensor operations."""
    g = torch.Generator(device="cuda").manual_seed(M + K + N)
    x = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8, device="cuda")
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8, device="cuda")
    ps = torch.rand(M, device="cuda", generator=g) * 1e-2
    sc = torch.rand(N, device="cuda", generator=g) * 1e-2
    bias = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16)
    acc = torch.zeros(M, N, dtype=torch.float64, device="cuda")
    for k0 in range(0, K, 4096):
        acc += x[:, k0:k0 + 4096].double() @ w[:, k0:k0 + 4096].double().t()
    acc = acc.to(torch.int64).to(torch.int32)
    assert torch.equal(capi.quant_matmul(x, w.t(), None, out_dtype=torch.int32), acc)
    want = (((acc.float() * ps[:, None]) * sc[None, :]) + bias.float()[None, :]).to(torch.bfloat16)
    assert torch.equal(capi.quant_matmul(x, w.t(), sc, ps, bias).view(torch.int16), want.view(torch.int16))


QMM_DECODE_CASES = [(1, 4096, 4096), (7, 1024, 2048), (16, 1152, 2056), (5, 14336, 4096), (3, 11008, 2048), (16, 16384, 2048),
                    (1, 1024, 8200), (17, 4096, 6144), (32, 8192, 2048), (30, 2176, 4100), (33, 4096, 4104), (64, 2048, 5120),
                    (48, 1024, 16384)]


@pytest.mark.parametrize("M,K,N", QMM_DECODE_CASES)
def test_quant_matmul_decode_kernel(capi, golden, M, K, N):
    """At most 64 rows and a weight stored [N, K]: the kernel that splits K over the wavefronts of a workgroup and walks
    over strips of 16 columns (one, two and four tiles of 16 rows; 1 to 16 steps per wavefront, even and uneven; strips
    that end past N; more strips than workgroups).  Outputs bit-identical to the oracle for every bias kind, both output
    types, with and without per-token scales, a single scale, pitched activations; and to the tiled kernel."""
    d = workloads.quant_matmul_inputs(seed=M + K + N, M=M, K=K, N=N, weight_nk=True, bias=True)
    g = torch.Generator().manual_seed(M + N)
    bias_i32 = torch.randint(-(1 << 20), 1 << 20, (N,), generator=g, dtype=torch.int32)
    bias_f32 = torch.randn(N, generator=g)
    x1, x2, sc, ps = d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), d["pertoken_scale"].cuda()
    assert capi.lib().mi355_quant_matmul_workspace(M, N, K, 1, K) == 0          # no split of K over workgroups
    acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    cases = [(d["bias"], torch.bfloat16, "bf16", True), (bias_i32, torch.bfloat16, "bf16", True), (bias_f32, torch.float16, "fp16", True),
             (None, torch.float16, "fp16", True), (None, torch.bfloat16, "bf16", False), (bias_f32, torch.bfloat16, "bf16", False)]
    for bias, dt, name, with_ps in cases:
        out = capi.quant_matmul(x1, x2, sc, ps if with_ps else None, None if bias is None else bias.cuda(), out_dtype=dt)
        bias_np = None if bias is None else (_bits(bias) if bias.dtype == torch.bfloat16 else bias.numpy())
        want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy() if with_ps else None, bias_np, out=name)
        assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), want), (name, with_ps, None if bias is None else bias.dtype)
    # one scale for all columns; activations that are a view of a wider matrix
    one = capi.quant_matmul(x1, x2, sc[:1].contiguous(), ps, d["bias"].cuda())
    want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy()[:1], d["pertoken_scale"].numpy(), _bits(d["bias"]), out="bf16")
    assert np.array_equal(_bits(one), want)
    wide = torch.zeros(M, K + 64, dtype=torch.int8, device="cuda")
    wide[:, :K] = x1
    ref = capi.quant_matmul(x1, x2, sc, ps, d["bias"].cuda())
    assert torch.equal(capi.quant_matmul(wide[:, :K], x2, sc, ps, d["bias"].cuda()), ref)
    # the scale as packed 64-bit parameters (what LinearQuant hands over for a float16 output, linear_quant.py:104-108):
    # the same bits as with the float32 scale, per channel and single
    for scale in (sc, sc[:1].contiguous()):
        qp = capi.trans_quant_param(scale)
        for dt, name in ((torch.float16, "fp16"), (torch.bfloat16, "bf16")):
            got = capi.quant_matmul_qparam(x1, x2, qp, bias_i32.cuda(), out_dtype=dt)
            want = golden.quant_matmul_epilogue_ex(acc, scale.cpu().numpy(), None, bias_i32.numpy(), out=name)
            assert np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), want), (name, scale.numel())
    # the int32 accumulator itself (LinearQuant with output_dtype=torch.int32), with and without the int32 bias; a scale
    # passed along is ignored
    assert np.array_equal(capi.quant_matmul(x1, x2, None, out_dtype=torch.int32).cpu().numpy(), acc)
    got = capi.quant_matmul(x1, x2, sc, ps, bias_i32.cuda(), out_dtype=torch.int32)
    assert np.array_equal(got.cpu().numpy(), (acc.astype(np.int64) + bias_i32.numpy().astype(np.int64)).astype(np.int32))
    capi.set_tuning("MI355_QMM_DECODE_OFF", 1)
    try:
        assert torch.equal(capi.quant_matmul(x1, x2, sc, ps, d["bias"].cuda()), ref)
        assert torch.equal(capi.quant_matmul(x1, x2, sc, ps, bias_i32.cuda(), out_dtype=torch.int32), got)
    finally:
        capi.set_tuning("MI355_QMM_DECODE_OFF", 0)


QMM_MID_ROWS = [33, 64, 65, 128, 192, 256]
QMM_MID_PROJECTIONS = [(4096, 6144), (4096, 11008), (11008, 4096)]


@pytest.mark.parametrize("K,N", QMM_MID_PROJECTIONS)
@pytest.mark.parametrize("M", QMM_MID_ROWS)
def test_quant_matmul_mid_rows(capi, golden, M, K, N):
    """33 to 256 rows on the projections of a transformer layer, with whatever kernel, tile and split of K the planner
    picks for them (the decode kernel up to 64 rows where the activations fit its registers, the streaming loop of the
    64x128 tile, larger tiles with K split over workgroups): accumulators, the bf16 and fp16 epilogues with every bias
    kind, and the re-quantised int8 output, bit-identical to the oracle."""
    d = workloads.quant_matmul_inputs(seed=3 * M + K + N, M=M, K=K, N=N, weight_nk=True, bias=True)
    g = torch.Generator().manual_seed(M + K)
    bias_i32 = torch.randint(-(1 << 20), 1 << 20, (N,), generator=g, dtype=torch.int32)
    bias_f32 = torch.randn(N, generator=g)
    offset = torch.randint(-40, 40, (N,), generator=g).float()
    x1, x2, sc, ps = d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(), d["pertoken_scale"].cuda()
    acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    assert np.array_equal(capi.quant_matmul(x1, x2, None, out_dtype=torch.int32).cpu().numpy(), acc)
    for bias, dt, name, with_ps in [(d["bias"], torch.bfloat16, "bf16", True), (bias_i32, torch.bfloat16, "bf16", True),
                                    (bias_f32, torch.float16, "fp16", True), (None, torch.bfloat16, "bf16", False)]:
        out = capi.quant_matmul(x1, x2, sc, ps if with_ps else None, None if bias is None else bias.cuda(), out_dtype=dt)
        bias_np = None if bias is None else (_bits(bias) if bias.dtype == torch.bfloat16 else bias.numpy())
        want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy() if with_ps else None, bias_np, out=name)
        assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), want), (name, with_ps)
    rq_scale = (torch.rand(N, generator=g) + 0.5) * (40.0 / (K ** 0.5 * 74 * 74))     # spreads the results over the int8 range
    qp = capi.trans_quant_param(rq_scale.cuda(), offset.cuda())
    got = capi.quant_matmul_qparam(x1, x2, qp, bias_i32.cuda())
    want = golden.quant_matmul_requant(d["x1"].numpy(), d["x2"].numpy(), golden.trans_quant_param(rq_scale.numpy(), offset.numpy()),
                                       bias_i32.numpy())
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.abs(want.astype(np.int32)).max() > 20 and (np.abs(want.astype(np.int32)) < 127).mean() > 0.5
    # a second launch on the same workspace (the first must have left its counters and exchange area clean)
    again = capi.quant_matmul(x1, x2, sc, ps, d["bias"].cuda())
    want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy(), _bits(d["bias"]), out="bf16")
    assert np.array_equal(_bits(again), want)


@pytest.mark.parametrize("M,K,N,pad", [(8, 1024, 2049, 0), (16, 4096, 2054, 0), (5, 2048, 4096, 8), (64, 4096, 2049, 0)])
def test_quant_matmul_decode_shapes_that_fall_back(capi, M, K, N, pad):
    """Decode-sized problems the decode kernel declines (N not a multiple of 4, activation rows whose pitch is not a
    multiple of 16, a scale pointer that is not 16-byte aligned): the planner has already dropped the K split for them,
    and the kernels behind give the same bits as the formula in float32 tensor operations."""
    g = torch.Generator(device="cuda").manual_seed(M + N)
    xw = torch.randint(-128, 128, (M, K + pad), generator=g, dtype=torch.int8, device="cuda")
    x = xw[:, :K]
    w = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8, device="cuda")
    ps = torch.rand(M, device="cuda", generator=g) * 1e-2
    sc = torch.rand(N + 1, device="cuda", generator=g) * 1e-2
    bias = torch.randn(N, device="cuda", generator=g).to(torch.bfloat16)
    acc = (x.double() @ w.double().t()).to(torch.int64).to(torch.int32)
    for scale in (sc[:N], sc[1:]):
        want = (((acc.float() * ps[:, None]) * scale[None, :]) + bias.float()[None, :]).to(torch.bfloat16)
        out = capi.quant_matmul(x, w.t(), scale, ps, bias)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))


# ------------------------------------------------------------------ weight-quant matmul

def _wq_golden(golden, d, group):
    out, outf = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                           None if d.get("antiquant_offset") is None else _bits(d["antiquant_offset"]),
                                           group_size=group)
    return torch.from_numpy(outf)


@pytest.mark.parametrize("M,K,N", [(16, 8192, 512), (1, 1024, 256), (5, 512, 100), (40, 2048, 320), (16, 96, 64)])
def test_w8a16(capi, golden, M, K, N):
    d = workloads.w8a16_inputs(seed=M, M=M, K=K, N=N)
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                   d["antiquant_offset"].cuda())
    stats = bf16_gate(out, _wq_golden(golden, d, 0))
    print("w8a16", M, K, N, stats)


def test_w8a16_kmajor_and_no_offset(capi, golden):
    d = workloads.w8a16_inputs(seed=3, M=8, K=1024, N=192, weight_nk=True)
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                   d["antiquant_offset"].cuda())
    bf16_gate(out, _wq_golden(golden, d, 0))
    d2 = workloads.w8a16_inputs(seed=4, M=8, K=1024, N=192)
    d2["antiquant_offset"] = None
    out = capi.weight_quant_matmul(d2["x"].cuda(), d2["weight"].cuda(), d2["antiquant_scale"].cuda(), None)
    bf16_gate(out, _wq_golden(golden, d2, 0))


@pytest.mark.parametrize("M,K,N,f16", [(1, 4096, 4096, False), (16, 8192, 2048, False), (7, 1152, 2052, True), (16, 2176, 4104, False),
                                       (17, 4096, 2048, False), (32, 3072, 6144, True), (3, 1024, 8200, False)])
def test_w8a16_kmajor_decode_kernel(capi, golden, M, K, N, f16):
    """int8 weight stored [N, K], one scale per column, at most 32 rows: the kernel that splits K over the wavefronts of a
    workgroup and walks over strips of 16 columns (one and two tiles of 16 rows, 1 to 8 steps per wavefront, even and
    uneven, strips that end past N, more strips than workgroups; both activation types; with and without offset and bias;
    pitched activations).  No workspace; within the gate of the oracle, and of the tiled K-major kernel's own result."""
    d = workloads.w8a16_inputs(seed=M + K + N, M=M, K=K, N=N, weight_nk=True)
    g = torch.Generator().manual_seed(N)
    dt = torch.float16 if f16 else torch.bfloat16
    bits = _f16_bits if f16 else _bits
    x, sc, of = d["x"].to(dt), d["antiquant_scale"].to(dt), d["antiquant_offset"].to(dt)
    bias = torch.randn(N, generator=g).to(dt)
    w = d["weight"]
    assert capi.lib().mi355_weight_quant_matmul_workspace(M, N, K, 8, 0) >= 0
    for use_of, use_bias in ((True, True), (False, False), (True, False)):
        out = capi.weight_quant_matmul(x.cuda(), w.cuda(), sc.cuda(), of.cuda() if use_of else None, 0, bias.cuda() if use_bias else None)
        _, want = golden.weight_quant_matmul(bits(x), w.numpy(), bits(sc), bits(of) if use_of else None, group_size=0,
                                             bias_u16=bits(bias) if use_bias else None, dtype="fp16" if f16 else "bf16")
        bf16_gate(out, torch.from_numpy(want), floor=out.numel() < 8192)
    wide = torch.zeros(M, K + 64, dtype=dt, device="cuda")
    wide[:, :K] = x.cuda()
    ref = capi.weight_quant_matmul(x.cuda(), w.cuda(), sc.cuda(), of.cuda(), 0, bias.cuda())
    assert torch.equal(capi.weight_quant_matmul(wide[:, :K], w.cuda(), sc.cuda(), of.cuda(), 0, bias.cuda()), ref)
    capi.set_tuning("MI355_WQ_DECODE_OFF", 1)
    try:
        tiled = capi.weight_quant_matmul(x.cuda(), w.cuda(), sc.cuda(), of.cuda(), 0, bias.cuda())
    finally:
        capi.set_tuning("MI355_WQ_DECODE_OFF", 0)
    bf16_gate(ref, tiled.float().cpu(), floor=ref.numel() < 8192)


@pytest.mark.parametrize("M,K,N", [(5, 256, 130), (5, 256, 132), (32, 512, 6), (3, 128, 1)])
def test_w8a16_kmajor_ragged_columns(capi, golden, M, K, N):
    """int8 weight stored [N, K] with N not a multiple of 4 (or of 8): the K-major streaming kernel stores quads of
    columns, so such widths must take a path that writes exactly N columns; the row after the last column and the
    guard bytes behind the output must stay untouched."""
    d = workloads.w8a16_inputs(seed=N, M=M, K=K, N=N, weight_nk=True)
    x, w, sc, of = (d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset"))
    want = _wq_golden(golden, d, 0)
    for _ in range(3):                                   # a race between tiles would not repeat
        out = capi.weight_quant_matmul(x, w, sc, of)
        bf16_gate(out, want, floor=True)
    # output rows inside a wider, pre-filled buffer: nothing outside [M, N] may change
    wide = torch.full((M + 1, N + 8), 7.0, dtype=torch.bfloat16, device="cuda")
    view = wide[:M, :N]
    need = capi.lib().mi355_weight_quant_matmul_workspace(M, N, K, 8, 0)
    ws = capi._wq_workspace(x.device, need) if need else None
    st = capi.lib().mi355_weight_quant_matmul(x.data_ptr(), 0, w.data_ptr(), 8, sc.data_ptr(), of.data_ptr(), None, view.data_ptr(),
                                              M, N, K, 0, 0, 1, x.stride(0), w.stride(0), w.stride(1), wide.stride(0),
                                              None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(),
                                              torch.cuda.current_stream().cuda_stream)
    assert st == 0
    torch.cuda.synchronize()
    assert torch.equal(view, out)
    assert (wide[:, N:] == 7.0).all() and (wide[M] == 7.0).all()


@pytest.mark.parametrize("M", [1, 8, 32, 128])
def test_w4a16_grouped(capi, golden, M):
    d = workloads.w4a16_inputs(seed=M, M=M, K=4096, N=1024, group_size=128)
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                   d["antiquant_offset"].cuda(), group_size=128)
    stats = bf16_gate(out, _wq_golden(golden, d, 128))
    print("w4a16", M, stats)


def test_w4a16_other_groups_and_edges(capi, golden):
    # (31, 1536, 512, 128): twelve groups over four wavefronts in three K chunks - one group per wavefront, on the kernel
    # that only exists with the running total
    for (M, K, N, gs) in [(3, 512, 136, 64), (16, 256, 128, 256), (2, 1024, 8, 32), (20, 2048, 2056, 128), (31, 1536, 512, 128)]:
        d = workloads.w4a16_inputs(seed=K + N, M=M, K=K, N=N, group_size=gs)
        out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                       d["antiquant_offset"].cuda(), group_size=gs)
        bf16_gate(out, _wq_golden(golden, d, gs))


def _to_f16(d):
    """The same seeded problem with float16 activations and parameters (values re-rounded to float16)."""
    return {k: (v.to(torch.float16) if torch.is_tensor(v) and v.dtype == torch.bfloat16 else v) for k, v in d.items()}


def _f16_bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("M,K,N,nk", [(16, 2048, 512, False), (16, 2048, 512, True), (1, 1024, 256, True), (40, 2048, 320, False),
                                      (33, 1024, 384, True)])
def test_w8a16_float16(capi, golden, M, K, N, nk):
    """float16 activations (the dtype of the reference's own test, test/contrib/test_linear_weight_quant.py:57-62), both
    weight layouts."""
    d = _to_f16(workloads.w8a16_inputs(seed=M + N, M=M, K=K, N=N, weight_nk=nk))
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(), d["antiquant_offset"].cuda())
    assert out.dtype == torch.float16
    _, gold = golden.weight_quant_matmul(_f16_bits(d["x"]), d["weight"].numpy(), _f16_bits(d["antiquant_scale"]),
                                         _f16_bits(d["antiquant_offset"]), dtype="fp16")
    print("w8a16 fp16", M, K, N, nk, bf16_gate(out, torch.from_numpy(gold)))


@pytest.mark.parametrize("M", [1, 8, 32, 100])
def test_w4a16_float16(capi, golden, M):
    d = _to_f16(workloads.w4a16_inputs(seed=M, M=M, K=2048, N=1024, group_size=128))
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(), d["antiquant_offset"].cuda(),
                                   group_size=128)
    _, gold = golden.weight_quant_matmul(_f16_bits(d["x"]), d["weight"].numpy(), _f16_bits(d["antiquant_scale"]),
                                         _f16_bits(d["antiquant_offset"]), group_size=128, dtype="fp16")
    print("w4a16 fp16", M, bf16_gate(out, torch.from_numpy(gold)))


@pytest.mark.parametrize("bits,nk,M", [(8, False, 16), (8, True, 5), (4, False, 1), (4, False, 40)])
def test_weight_quant_bias(capi, golden, bits, nk, M):
    """The module's optional bias (linear_weight_quant.py:89-92): added to the float32 sum before the final rounding, on
    every kernel (N-major, K-major, int4, with and without a split over K)."""
    if bits == 8:
        d = workloads.w8a16_inputs(seed=M, M=M, K=2048, N=640, weight_nk=nk)
        gs = 0
    else:
        d = workloads.w4a16_inputs(seed=M, M=M, K=2048, N=1024, group_size=128)
        gs = 128
    N = d["antiquant_scale"].shape[-1]
    bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(), d["antiquant_offset"].cuda(),
                                   group_size=gs, bias=bias.cuda())
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]), group_size=gs, bias_u16=_bits(bias))
    bf16_gate(out, torch.from_numpy(gold))
    nobias = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                      d["antiquant_offset"].cuda(), group_size=gs)
    assert not torch.equal(out, nobias)


TILED_CASES = [  # bits, M, K, N, group, float16, bias
    (8, 33, 1024, 384, 0, False, False),      # 64-row tile, ragged rows
    (8, 128, 2048, 1000, 0, False, True),     # 128-row tile, last strip partly valid
    (8, 200, 1024, 256, 0, False, False),     # two row tiles, the second ragged
    (8, 64, 8192, 256, 0, True, False),       # few tiles: K split eight ways, per channel
    (8, 96, 1024, 512, 256, False, False),    # int8 with scale groups
    (4, 128, 4096, 1024, 128, False, False),  # several groups per workgroup and a K split
    (4, 40, 2048, 264, 128, False, True),     # second strip holds 8 columns
    (4, 100, 1024, 512, 256, True, False),
    (4, 130, 512, 2048, 512, False, False),   # one group = per channel
    (4, 320, 1024, 768, 128, False, False),   # three row tiles
    (4, 33, 128, 8, 128, False, False),       # one stage, one dword column, one group = per channel
    (4, 64, 1536, 520, 384, False, True),     # groups of three stages, last strip holds 8 columns
    (4, 256, 8192, 256, 8192, True, False),   # one strip, four row blocks, per channel with a K split
    (4, 384, 1024, 512, 128, False, False),
    (4, 400, 1024, 512, 128, False, False),   # ragged seventh row block
    # int8 weights stored [N, K] (the transposed view that LinearWeightQuant passes, linear_weight_quant.py:106)
    (8, 40, 1024, 384, 0, False, False, True),
    (8, 128, 2048, 1000, 0, False, True, True),
    (8, 200, 1024, 256, 256, False, False, True),
    (8, 64, 8192, 256, 0, True, False, True),
]


PAIRED_CASES = [  # M, K, N, group (0: per channel), float16, forced split
    (64, 128, 256, 128, False, 0),        # one stage: the second set of wavefronts has nothing to compute
    (64, 640, 512, 128, False, 0),        # five stages: the sets get three and two
    (128, 640, 520, 128, True, 2),        # chunks of two and three stages, last strip holds 8 columns
    (96, 1152, 768, 0, False, 0),         # per channel, nine stages
    (96, 1152, 768, 0, True, 3),          # per channel, chunks of three stages
    (384, 2048, 1024, 128, False, 4),
    (200, 4096, 3584, 128, False, 0),     # ragged last row block, several strips per XCD
    (128, 1536, 512, 256, False, 3),      # groups of two stages, chunks of two groups: each set has one stage per group
    (72, 2304, 264, 384, True, 2),        # groups of three stages: the sets alternate two and one
    (1100, 512, 1024, 128, False, 0),     # many row blocks per strip
]


@pytest.mark.parametrize("case", PAIRED_CASES, ids=lambda c: "-".join(str(v) for v in c))
def test_weight_quant_int4_register_kernel_variants(capi, golden, case):
    """The register-expanding int4 kernel (a scale group per stage, groups of several stages, or one group), with its
    K-split exchange through the L2 and through memory: both must meet the gate, and each must repeat its own result bit
    for bit (the sets of wavefronts and the chunks add in a fixed order)."""
    M, K, N, gs, f16, split = case
    d = workloads.w4a16_inputs(seed=M + N + K, M=M, K=K, N=N, group_size=gs if gs else K)
    bits_of = _bits
    if f16:
        d = _to_f16(d)
        bits_of = _f16_bits
    args = [d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")]
    _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(d["antiquant_scale"]),
                                         bits_of(d["antiquant_offset"]), group_size=gs if gs else K,
                                         dtype="fp16" if f16 else "bf16")
    capi.set_tuning("MI355_WQG_SPLIT", split)
    try:
        for variant in (0, 2):             # exchange through the L2 where the XCD allows; through memory
            capi.set_tuning("MI355_WQ_GEMM4_OFF", variant)
            out = capi.weight_quant_matmul(*args, group_size=gs if gs else K)
            bf16_gate(out, torch.from_numpy(gold))
            for _ in range(2):
                assert torch.equal(out, capi.weight_quant_matmul(*args, group_size=gs if gs else K))
    finally:
        capi.set_tuning("MI355_WQ_GEMM4_OFF", 0)
        capi.set_tuning("MI355_WQG_SPLIT", 0)


INT8_REGISTER_CASES = [  # M, K, N, group (0: per channel), float16, forced split
    (64, 128, 256, 0, False, 0),          # two stages of 64 rows: one per set of wavefronts
    (100, 640, 1000, 64, False, 0),       # a scale group per stage, ragged rows, last strip holds 232 columns
    (128, 768, 516, 192, True, 2),        # groups of three stages, two chunks of two groups, last strip holds 4 columns
    (256, 4096, 512, 0, False, 4),        # per channel, four chunks of K
    (72, 1024, 260, 128, False, 3),       # groups of two stages, uneven chunks
]


@pytest.mark.parametrize("case", INT8_REGISTER_CASES, ids=lambda c: "-".join(str(v) for v in c))
def test_weight_quant_int8_register_kernel_variants(capi, golden, case):
    """int8 weights [K, N] with more than 32 rows take the register-expanding kernel too (64-row stages, 256-byte
    strips): group sizes of one, two and three stages and per channel, K splits, exchange through the L2 and through
    memory; each variant repeats its own result bit for bit."""
    M, K, N, gs, f16, split = case
    d = workloads.w8a16_inputs(seed=M + N + K, M=M, K=K, N=N)
    if gs:
        g = torch.Generator().manual_seed(7)
        d["antiquant_scale"] = (torch.rand(K // gs, N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
        d["antiquant_offset"] = (torch.rand(K // gs, N, generator=g) * 8 - 4).to(torch.bfloat16)
    bits_of = _bits
    if f16:
        d = _to_f16(d)
        bits_of = _f16_bits
    args = [d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")]
    _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(d["antiquant_scale"]),
                                         bits_of(d["antiquant_offset"]), group_size=gs, dtype="fp16" if f16 else "bf16")
    capi.set_tuning("MI355_WQG_SPLIT", split)
    try:
        for variant in (0, 2):             # exchange through the L2 where the XCD allows; through memory
            capi.set_tuning("MI355_WQ_GEMM4_OFF", variant)
            out = capi.weight_quant_matmul(*args, group_size=gs)
            bf16_gate(out, torch.from_numpy(gold))
            for _ in range(2):
                assert torch.equal(out, capi.weight_quant_matmul(*args, group_size=gs))
    finally:
        capi.set_tuning("MI355_WQ_GEMM4_OFF", 0)
        capi.set_tuning("MI355_WQG_SPLIT", 0)


@pytest.mark.parametrize("case", TILED_CASES, ids=lambda c: "-".join(str(v) for v in c))
def test_weight_quant_tiled_kernel(capi, golden, case):
    bits, M, K, N, gs, f16, with_bias = case[:7]
    nk = len(case) > 7 and case[7]
    _tiled_case(capi, golden, bits, M, K, N, gs, f16, with_bias, nk)


def _tiled_case(capi, golden, bits, M, K, N, gs, f16, with_bias, nk):
    """More than 32 activation rows take the tiled kernel (weights decoded once per 64/128 rows): every tile shape,
    ragged rows and strips, grouped and per-channel parameters, both activation dtypes, with and without a K split."""
    if bits == 8:
        d = workloads.w8a16_inputs(seed=M + N, M=M, K=K, N=N, weight_nk=nk)
        if gs:
            g = torch.Generator().manual_seed(5)
            d["antiquant_scale"] = (torch.rand(K // gs, N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
            d["antiquant_offset"] = (torch.rand(K // gs, N, generator=g) * 8 - 4).to(torch.bfloat16)
    else:
        d = workloads.w4a16_inputs(seed=M + N, M=M, K=K, N=N, group_size=gs)
    bits_of = _bits
    if f16:
        d = _to_f16(d)
        bits_of = _f16_bits
    bias = None
    if with_bias:
        bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(d["x"].dtype)
    group = gs
    args = [d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")]
    out = capi.weight_quant_matmul(*args, group_size=group, bias=None if bias is None else bias.cuda())
    _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(d["antiquant_scale"]),
                                         bits_of(d["antiquant_offset"]), group_size=group, dtype="fp16" if f16 else "bf16",
                                         bias_u16=None if bias is None else bits_of(bias))
    print("tiled", bits, M, K, N, gs, bf16_gate(out, torch.from_numpy(gold)))
    # the split over K must not change a bit of the result, whatever the number of chunks, and repeated launches
    # (which reuse the workspace and its arrival counters) must repeat the result
    for split in (1, 2):
        capi.set_tuning("MI355_WQG_SPLIT", split)
        try:
            again = capi.weight_quant_matmul(*args, group_size=group, bias=None if bias is None else bias.cuda())
        finally:
            capi.set_tuning("MI355_WQG_SPLIT", 0)
        bf16_gate(again, torch.from_numpy(gold))
    for _ in range(5):
        assert torch.equal(capi.weight_quant_matmul(*args, group_size=group, bias=None if bias is None else bias.cuda()), out)
    # no offsets: the image bias alone is removed through the row sums
    out0 = capi.weight_quant_matmul(args[0], args[1], args[2], None, group_size=group)
    _, gold0 = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(d["antiquant_scale"]), None,
                                          group_size=group, dtype="fp16" if f16 else "bf16")
    bf16_gate(out0, torch.from_numpy(gold0))


KPACKED_CASES = [
    # M, K, N, group_size, float16, parameters stored [N, G] (passed as the transposed view), bias
    (1, 4096, 14336, 128, False, True, False),      # decode shape of the W4A16 configuration, module layout
    (8, 4096, 14336, 128, False, False, False),
    (32, 4096, 14336, 128, True, True, True),
    (128, 4096, 14336, 128, False, True, False),    # four m tiles, two chunks of rows
    (5, 512, 72, 128, False, True, True),           # ragged columns (N % 16 != 0, one partial workgroup)
    (17, 1024, 200, 256, True, False, False),       # group of two sub-steps
    (40, 768, 64, 384, False, True, False),         # group of three sub-steps: folds in the middle of a step
    (3, 2048, 4096, 0, False, False, True),         # per channel, 1-D parameters
    (70, 14336, 4096, 128, False, True, False),     # long K: K is split between workgroups, 112 groups
    (16, 256, 16, 128, True, True, False),          # a single step, a single wavefront's worth of columns
    # at most 32 rows, groups of 128, at least 2048 columns and k: the decode kernel (weight_quant_kpacked_decode.hip), as
    # are the first two cases above
    (16, 2048, 2048, 128, True, True, True),        # one step per wavefront of the two the kernel is built for
    (3, 4096, 4088, 128, False, False, True),       # at most 4096 columns: strips of 16 columns, the last partly valid
    (9, 5120, 2056, 128, False, False, True),       # two or three steps per wavefront, a strip that ends past N
    (4, 8192, 4096, 128, False, True, False),       # four steps per wavefront, one column tile per strip
    (16, 3072, 8224, 128, True, True, True),        # more strips than workgroups, uneven steps, fp16
    (17, 4096, 2048, 128, False, True, True),       # two tiles of rows (at most two steps per wavefront)
    (32, 3072, 4104, 128, True, False, False),      # the same, uneven steps, a strip that ends past N, fp16
    # from 256 rows up the weight is rewritten per call with its words along N (weight_quant_repack.hip)
    (256, 512, 1000, 128, False, True, True),       # ragged columns: 125 words per row, the last tile partly valid
    (300, 1024, 520, 256, True, True, False),       # ragged rows, groups of two stages, fp16
    (257, 640, 264, 0, False, False, False),        # per channel, K / 8 = 80 words: a partly valid tile along K
    (512, 4096, 14336, 128, False, True, False),    # the W4A16 configuration at prefill size, module layout
]


@pytest.mark.parametrize("M,K,N,gs,f16,params_ng,with_bias", KPACKED_CASES)
def test_weight_quant_int4_words_along_k(capi, golden, M, K, N, gs, f16, params_ng, with_bias):
    """int4 weights stored [N, K/8] (words along K) and passed as the transposed view, the way the contrib module
    passes its weight (linear_weight_quant.py:71,106): same values, same golden result as the [K, N/8] layout.
    Parameters row-major [G, N] or the module's transposed [N, G]; both activation types; repeated launches and a
    forced split of K must not change a bit."""
    d = workloads.w4a16_inputs(seed=M + N + K, M=M, K=K, N=N, group_size=gs if gs else K)
    if not gs:
        d["antiquant_scale"], d["antiquant_offset"] = d["antiquant_scale"][0].clone(), d["antiquant_offset"][0].clone()
    bits_of = _bits
    if f16:
        d = _to_f16(d)
        bits_of = _f16_bits
    w_nk = torch.from_numpy(golden.pack_int4(np.ascontiguousarray(d["weight_int4_values"].numpy().T)))   # [N, K/8]
    assert w_nk.shape == (N, K // 8)
    bias = torch.randn(N, generator=torch.Generator().manual_seed(1)).to(d["x"].dtype) if with_bias else None
    sc, of = d["antiquant_scale"], d["antiquant_offset"]
    if params_ng and gs:
        sc_dev, of_dev = sc.t().contiguous().cuda().t(), of.t().contiguous().cuda().t()
        assert sc_dev.stride() == (1, K // gs)
    else:
        sc_dev, of_dev = sc.cuda(), of.cuda()
    x, w = d["x"].cuda(), w_nk.cuda().t()
    call = lambda off=of_dev: capi.weight_quant_matmul(x, w, sc_dev, off, group_size=gs, bias=None if bias is None else bias.cuda())
    out = call()
    kw = dict(group_size=gs, dtype="fp16" if f16 else "bf16")
    _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(sc), bits_of(of),
                                         bias_u16=None if bias is None else bits_of(bias), **kw)
    print("kpacked", M, K, N, gs, bf16_gate(out, torch.from_numpy(gold)))
    for _ in range(3):
        assert torch.equal(call(), out)
    for split in (1, 2, 3):
        capi.set_tuning("MI355_WQ_SPLIT", split)
        try:
            bf16_gate(call(), torch.from_numpy(gold))
        finally:
            capi.set_tuning("MI355_WQ_SPLIT", 0)
    assert torch.equal(call(), out)
    out0 = call(None)
    _, gold0 = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(sc), None,
                                          bias_u16=None if bias is None else bits_of(bias), **kw)
    bf16_gate(out0, torch.from_numpy(gold0))


def test_weight_quant_int4_words_along_k_generic_fallback(capi, golden):
    """Shapes the fast kernel does not take (K not a multiple of 256, a group of 32) go to the one-thread-per-output
    kernel, which reads the same layout and strided parameters."""
    for (M, K, N, gs) in [(3, 128, 24, 32), (2, 384, 40, 128)]:
        d = workloads.w4a16_inputs(seed=K, M=M, K=K, N=N, group_size=gs)
        w_nk = torch.from_numpy(golden.pack_int4(np.ascontiguousarray(d["weight_int4_values"].numpy().T)))
        sc, of = d["antiquant_scale"], d["antiquant_offset"]
        out = capi.weight_quant_matmul(d["x"].cuda(), w_nk.cuda().t(), sc.t().contiguous().cuda().t(),
                                       of.t().contiguous().cuda().t(), group_size=gs)
        _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(sc), _bits(of), group_size=gs)
        bf16_gate(out, torch.from_numpy(gold))


def test_weight_quant_random_shapes(capi, golden):
    """Seeded sweep over shapes, layouts, group sizes and dtypes: whichever kernel the library picks (streaming, K-major,
    tiled, generic) must pass the gate against the oracle."""
    import os
    rng = np.random.default_rng(2024)
    for case in range(int(os.environ.get("MI355_SWEEP_CASES", "96"))):
        bits = int(rng.choice([8, 4]))
        M = int(rng.choice([1, 3, 16, 17, 31, 32, 33, 48, 64, 65, 100, 129, 160, 257]))
        K = int(rng.choice([32, 96, 128, 256, 384, 512, 1024, 1536]))
        N = int(rng.choice([8, 24, 64, 128, 136, 256, 264, 512, 520, 1000, 1024]))
        gs = 0
        if rng.random() < 0.6 or bits == 4:
            cands = [g for g in (32, 64, 128, 256, 512) if K % g == 0]
            gs = int(rng.choice(cands))
        nk = bool(bits == 8 and rng.random() < 0.4)
        f16 = bool(rng.random() < 0.3)
        with_off = bool(rng.random() < 0.8)
        if bits == 8:
            d = workloads.w8a16_inputs(seed=case, M=M, K=K, N=N, weight_nk=nk)
            if gs:
                g = torch.Generator().manual_seed(case)
                d["antiquant_scale"] = (torch.rand(K // gs, N, generator=g) * 9e-3 + 1e-3).to(torch.bfloat16)
                d["antiquant_offset"] = (torch.rand(K // gs, N, generator=g) * 8 - 4).to(torch.bfloat16)
        else:
            d = workloads.w4a16_inputs(seed=case, M=M, K=K, N=N, group_size=gs)
        bits_of = _bits
        if f16:
            d = _to_f16(d)
            bits_of = _f16_bits
        off = d["antiquant_offset"] if with_off else None
        _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(d["antiquant_scale"]),
                                             None if off is None else bits_of(off), group_size=gs,
                                             dtype="fp16" if f16 else "bf16")
        try:
            out = capi.weight_quant_matmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                           None if off is None else off.cuda(), group_size=gs)
            # outputs of a few hundred elements: one element that cancels to almost nothing is already more than
            # 0.1 % of them, so those are counted with the cancellation floor; larger ones strictly
            bf16_gate(out, torch.from_numpy(gold), floor=out.numel() < 8192)
        except (AssertionError, capi.Mi355Error) as e:
            raise AssertionError(f"case {case}: bits={bits} M={M} K={K} N={N} gs={gs} nk={nk} f16={f16} offset={with_off}: {e}")


def test_weight_quant_int4_words_along_k_random_shapes(capi, golden):
    """Seeded sweep for int4 weights stored [N, K/8]: shapes that take the fast kernel (K a multiple of 256, groups of
    whole sub-steps; every m-tile count, ragged columns, one or two K slices, K split between workgroups) and shapes
    that fall back to the generic kernel, parameters in either layout, both activation types."""
    import os
    rng = np.random.default_rng(4242)
    for case in range(int(os.environ.get("MI355_SWEEP_CASES", "64"))):
        M = int(rng.choice([1, 2, 15, 16, 17, 32, 33, 63, 64, 65, 100, 130, 256, 300]))
        K = int(rng.choice([128, 256, 512, 768, 1024, 1280, 2048, 3072]))
        N = int(rng.choice([8, 16, 24, 64, 72, 128, 136, 200, 256, 1000, 2048]))
        gs = int(rng.choice([g for g in (0, 32, 64, 128, 256, 384, 512, 1024) if g == 0 or K % g == 0]))
        f16 = bool(rng.random() < 0.3)
        with_off = bool(rng.random() < 0.8)
        params_ng = bool(rng.random() < 0.5)
        d = workloads.w4a16_inputs(seed=case, M=M, K=K, N=N, group_size=gs if gs else K)
        if not gs:
            d["antiquant_scale"], d["antiquant_offset"] = d["antiquant_scale"][0].clone(), d["antiquant_offset"][0].clone()
        bits_of = _bits
        if f16:
            d = _to_f16(d)
            bits_of = _f16_bits
        sc, of = d["antiquant_scale"], (d["antiquant_offset"] if with_off else None)
        _, gold = golden.weight_quant_matmul(bits_of(d["x"]), d["weight"].numpy(), bits_of(sc), None if of is None else bits_of(of),
                                             group_size=gs, dtype="fp16" if f16 else "bf16")
        w_nk = torch.from_numpy(golden.pack_int4(np.ascontiguousarray(d["weight_int4_values"].numpy().T)))
        dev = lambda t: None if t is None else (t.t().contiguous().cuda().t() if params_ng and t.dim() == 2 else t.cuda())  # noqa: E731
        try:
            out = capi.weight_quant_matmul(d["x"].cuda(), w_nk.cuda().t(), dev(sc), dev(of), group_size=gs)
            # small outputs are counted with the cancellation floor, as in the sweep above
            bf16_gate(out, torch.from_numpy(gold), floor=out.numel() < 8192)
        except (AssertionError, capi.Mi355Error) as e:
            raise AssertionError(f"case {case}: M={M} K={K} N={N} gs={gs} f16={f16} offset={with_off} params_ng={params_ng}: {e}")


def test_weight_quant_exact_special_case(capi):
    # small-integer activations, unit scale, zero offset: every partial sum is exact in float32
    g = torch.Generator().manual_seed(0)
    x = torch.randint(-8, 9, (16, 1024), generator=g).to(torch.bfloat16)
    w = torch.randint(-127, 128, (1024, 256), generator=g, dtype=torch.int8)
    one = torch.ones(256, dtype=torch.bfloat16)
    out = capi.weight_quant_matmul(x.cuda(), w.cuda(), one.cuda(), None)
    want = (x.double() @ w.double()).to(torch.bfloat16)
    assert torch.equal(out.cpu(), want)
    w4 = torch.randint(-8, 8, (1024, 256), generator=g, dtype=torch.int8)
    out = capi.weight_quant_matmul(x.cuda(), workloads.pack_int4(w4).cuda(), torch.ones(8, 256, dtype=torch.bfloat16).cuda(),
                                   None, group_size=128)
    assert torch.equal(out.cpu(), (x.double() @ w4.double()).to(torch.bfloat16))


# ------------------------------------------------------------------ swiglu

def test_swiglu(capi, golden):
    g = torch.Generator().manual_seed(0)
    for rows, half in [(64, 14336), (3, 24), (5, 7)]:
        x = (torch.randn(rows, 2 * half, generator=g) * 3).to(torch.bfloat16)
        out = capi.swiglu(x.cuda())
        want = golden.swiglu(_bits(x))
        dist = golden.bf16_ulp_distance(_bits(out), want)
        assert dist.max() <= 1 and (dist == 0).mean() > 0.995   # device expf vs libm expf


def test_swiglu_every_bf16_argument(capi, golden):
    """silu is evaluated on bf16 arguments and rounded to bf16, so there are 65536 cases: all of them (every bit pattern
    as the activated half, multiplied by 1 and by 3), through the vector kernel, the scalar kernel (odd width) and the
    fused SwiGLU + quantisation.  The kernels take hardware exp2 / reciprocal and fall back to the exact formula next to
    bf16 rounding boundaries; the results must be those of the exact formula as the oracle evaluates it (libm expf and
    IEEE division) wherever that is a number."""
    a = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    for mul in (1.0, 3.0):
        x = torch.cat([a.view(256, 256), torch.full((256, 256), mul, dtype=torch.bfloat16)], dim=1).contiguous()
        want = golden.swiglu(_bits(x))
        nan = np.isnan(golden.bf16_bits_to_f32(want))
        got = _bits(capi.swiglu(x.cuda()))
        assert np.array_equal(got[~nan], want[~nan]), int((got[~nan] != want[~nan]).sum())
        assert np.isnan(golden.bf16_bits_to_f32(got[nan])).all()
        # odd width: the scalar kernel
        xo = torch.cat([a.view(256, 256)[:, :255], torch.full((256, 255), mul, dtype=torch.bfloat16)], dim=1).contiguous()
        wo = golden.swiglu(_bits(xo))
        go = _bits(capi.swiglu(xo.cuda()))
        ok = ~np.isnan(golden.bf16_bits_to_f32(wo))
        assert np.array_equal(go[ok], wo[ok])
    # fused with the quantisation: rows of finite arguments only (a NaN or an infinity would own its row's scale)
    fin = a[torch.isfinite(a.float())]
    fin = fin[: fin.numel() // 256 * 256].view(-1, 256)
    xf = torch.cat([fin, torch.full(fin.shape, 1.0, dtype=torch.bfloat16)], dim=1).contiguous()
    y, s = capi.swiglu_quant(xf.cuda(), activate_left=True)
    wy, ws = golden.swiglu_quant(_bits(xf), activate_left=True)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32)) and np.array_equal(y.cpu().numpy(), wy)


# ------------------------------------------------------------------ anti_quant

@pytest.mark.parametrize("rows,cols,packed", [(10, 100, False), (10, 200, True), (4096, 14336, False), (512, 4096, True),
                                              (7, 24, False), (3, 8, True), (33, 1000, False)])
@pytest.mark.parametrize("dst", [torch.float16, torch.bfloat16])
def test_anti_quant(capi, golden, rows, cols, packed, dst):
    """Bit-exact against the oracle: int8 and packed-int4 inputs (the shapes of test/custom_ops/test_npu_anti_quant.py:49-58
    and large ones), per-column, single and absent parameters, both output types."""
    g = torch.Generator().manual_seed(rows + cols)
    if packed:
        x = torch.randint(-2 ** 31, 2 ** 31 - 1, (rows, cols // 8), generator=g, dtype=torch.int64).to(torch.int32)
    else:
        x = torch.randint(-128, 128, (rows, cols), generator=g, dtype=torch.int8)
    scale = torch.rand(cols, generator=g) * 200 - 100
    offset = torch.rand(cols, generator=g) * 200 - 100
    name = "fp16" if dst == torch.float16 else "bf16"
    for sc, of in [(scale, offset), (scale, None), (scale[:1].clone(), offset[:1].clone())]:
        out = capi.anti_quant(x.cuda(), sc.cuda(), None if of is None else of.cuda(), dst_dtype=dst)
        want = golden.anti_quant(x.numpy(), sc.numpy(), None if of is None else of.numpy(), dst=name)
        got = out.cpu().view(torch.int16).numpy().view(np.uint16)
        assert np.array_equal(got, want)


QUANTIZE_CASES = [  # shape, axis, number of scales ("c" = one per channel, 1 = single)
    ((2048, 4096), -1, "c"), ((5, 16, 8), 2, "c"), ((5, 16, 8), 1, "c"), ((3, 7, 5), 0, "c"), ((64, 24), -1, 1),
    ((33, 1000), -1, "c"), ((4, 12, 16), 1, "c"), ((1, 9), -1, "c"), ((128, 14336), -1, 1)]


@pytest.mark.parametrize("shape,axis,nscale", QUANTIZE_CASES)
@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_quantize(capi, golden, shape, axis, nscale, in_dtype):
    """npu_quantize through the C ABI, bit-exact against the oracle: every input and output type, division and
    multiplication mode, with and without zero points, the vector paths (shared channel / consecutive channels) and the
    element-wise fallback, values that clamp and exact .5 ties."""
    g = torch.Generator().manual_seed(sum(shape) + axis)
    x = (torch.randn(shape, generator=g) * 60).to(in_dtype)
    flat = x.view(-1)
    flat[: min(8, flat.numel())] = torch.tensor([0.5, 1.5, 2.5, -0.5, -2.5, 1000.0, -1000.0, 3.5])[: min(8, flat.numel())].to(in_dtype)
    ch = shape[axis] if nscale == "c" else 1
    scale = torch.rand(ch, generator=g) * 1.5 + 0.25
    scale[0] = 1.0
    zp = torch.randint(-20, 20, (ch,), generator=g).float()
    xf = x.float().numpy()
    for out_dtype, name in [(torch.int8, "int8"), (torch.uint8, "uint8"), (torch.int32, "int32")]:
        for div in (True, False):
            for z in (zp, None):
                zc = None if z is None else (z.cuda().to(torch.int32) if div else z.cuda())    # both zero-point types
                got = capi.quantize(x.cuda(), scale.cuda(), zc, out_dtype, axis, div)
                want = golden.quantize(xf, scale.numpy(), None if z is None else z.numpy(), name, axis, div)
                assert got.dtype == out_dtype and got.shape == x.shape
                assert np.array_equal(got.cpu().numpy(), want), (name, div, z is None)


def test_quantize_matches_torch_per_channel(capi):
    """Independent pin: torch.quantize_per_channel on the CPU for power-of-two scales and even zero points (where its
    nearbyint(x * (1 / scale)) + zero_point equals rint(x / scale + zero_point))."""
    g = torch.Generator().manual_seed(9)
    x = torch.randn(6, 32, 10, generator=g) * 50
    scales = torch.tensor([2.0 ** (i % 6 - 3) for i in range(32)])
    zps = (torch.arange(32, dtype=torch.int32) - 16) // 2 * 2
    want = torch.quantize_per_channel(x, scales, zps, axis=1, dtype=torch.qint8).int_repr()
    got = capi.quantize(x.cuda(), scales.cuda(), zps.float().cuda(), torch.int8, 1, True)
    assert torch.equal(got.cpu(), want)


def test_quantize_extreme_operands(capi, golden):
    """Operands outside the range where the kernel divides through the channel's reciprocal (tiny, huge, infinite,
    NaN, denormal numerators; tiny and huge scales): the ordinary division takes over for the whole wavefront, and
    results stay equal to the oracle element by element."""
    g = torch.Generator().manual_seed(77)
    x = torch.randn(64, 256, generator=g) * 50
    special = torch.tensor([1e-30, -1e-30, 1e30, -1e30, float("inf"), float("-inf"), float("nan"), 1e-42, 0.0, -0.0, 3e-20, 7e19])
    x[::3, :12] = special                                        # some wavefronts see them, others do not
    scale = torch.rand(256, generator=g) + 0.5
    scale[5], scale[9], scale[200] = 1e-25, 1e25, 3e-39          # channels with scales outside the range (one denormal)
    zp = torch.randint(-5, 5, (256,), generator=g).float()
    with np.errstate(all="ignore"):
        for name, dt in (("int8", torch.int8), ("int32", torch.int32)):
            want = golden.quantize(x.numpy(), scale.numpy(), zp.numpy(), name, -1, True)
            got = capi.quantize(x.cuda(), scale.cuda(), zp.cuda(), dt, -1, True)
            assert np.array_equal(got.cpu().numpy(), want), name
        want = golden.quantize(x.numpy(), scale[:1].numpy(), None, "int8", -1, True)
        assert np.array_equal(capi.quantize(x.cuda(), scale[:1].cuda(), None, torch.int8, -1, True).cpu().numpy(), want)


def test_quantize_bad_arguments(capi):
    import ctypes
    L = capi.lib()
    x = torch.zeros(16, device="cuda")
    o = torch.zeros(16, dtype=torch.int8, device="cuda")
    sc = torch.ones(4, device="cuda")
    call = lambda *a: L.mi355_quantize(*a)
    vp = ctypes.c_void_p
    assert call(vp(x.data_ptr()), 2, vp(sc.data_ptr()), 3, None, 2, 0, vp(o.data_ptr()), 0, 1, 4, 4, 1, None) == -1   # scale_len
    assert call(vp(x.data_ptr()), 7, vp(sc.data_ptr()), 4, None, 2, 0, vp(o.data_ptr()), 0, 1, 4, 4, 1, None) == -1   # in_dtype
    assert call(vp(x.data_ptr()), 2, vp(sc.data_ptr()), 4, None, 2, 0, vp(o.data_ptr()), 5, 1, 4, 4, 1, None) == -1   # out_dtype
    assert call(None, 2, vp(sc.data_ptr()), 4, None, 2, 0, vp(o.data_ptr()), 0, 1, 4, 4, 1, None) == -1
    assert call(None, 2, None, 4, None, 2, 0, None, 0, 0, 4, 4, 1, None) == 0                                        # empty


@pytest.mark.parametrize("rows,words,in_pad,out_pad,out_shift", [
    (16, 8, 0, 0, 0), (64, 5, 0, 0, 0), (1024, 512, 0, 0, 0), (4096, 1376, 0, 0, 0),   # 16-byte stores / one odd word count
    (33, 6, 1, 0, 0), (7, 3, 0, 8, 0), (9, 4, 2, 3, 0), (5, 2, 0, 0, 1), (1, 1, 0, 0, 0)])  # pitched and unaligned rows
def test_unpack_int4(capi, golden, rows, words, in_pad, out_pad, out_shift):
    """Packed int4 -> int8 bit-exact against the oracle's unpacking (nibble order of
    test/custom_ops/test_npu_anti_quant.py:12-24) on random words, with pitched inputs and outputs and an output
    that starts on an odd byte (every store width of the kernel); bytes between the rows stay untouched."""
    g = torch.Generator().manual_seed(rows * 131 + words)
    wide = torch.randint(-2 ** 31, 2 ** 31 - 1, (rows, words + in_pad), generator=g, dtype=torch.int64).to(torch.int32)
    x = wide.cuda()[:, :words]
    cols = words * 8
    buf = torch.full((rows * (cols + out_pad) + out_shift + 16,), 99, dtype=torch.int8, device="cuda")
    out = buf[out_shift:out_shift + rows * (cols + out_pad)].view(rows, cols + out_pad)
    capi.unpack_int4(x, out)
    want = golden.unpack_int4(wide[:, :words].contiguous().numpy())
    assert want.min() >= -8 and want.max() <= 7
    got = out.cpu().numpy()
    assert np.array_equal(got[:, :cols], want)
    assert (got[:, cols:] == 99).all() and (buf[:out_shift].cpu() == 99).all() and (buf[-16:].cpu() == 99).all()


def test_rowwise_kernels_random_shapes(capi, golden):
    """Seeded sweep over row counts and widths (every kernel variant: one wavefront per row, one block per row, the
    two-pass kernel, odd widths, strided rows) for dynamic_quant with and without smooth scales, both input types, and
    for the fused SwiGLU quantisation: codes and scales bit-identical to the oracle."""
    import os
    rng = np.random.default_rng(99)
    for case in range(int(os.environ.get("MI355_SWEEP_CASES", "60"))):
        rows = int(rng.choice([1, 2, 7, 33, 64, 129, 500]))
        cols = int(rng.choice([1, 8, 24, 100, 512, 1000, 2048, 4096, 4104, 8192, 14336, 16384, 16392, 20000]))
        f16 = bool(rng.random() < 0.3)
        smooth = bool(rng.random() < 0.3)
        strided = bool(rng.random() < 0.3)
        g = torch.Generator().manual_seed(case)
        dt = torch.float16 if f16 else torch.bfloat16
        wide = (torch.randn(rows, cols + (16 if strided else 0), generator=g) * float(rng.choice([1e-3, 1.0, 30.0]))).to(dt)
        x = wide[:, :cols]
        sm = (torch.rand(cols, generator=g) + 0.5).to(dt) if smooth else None
        bits = _f16_bits if f16 else _bits
        tag = f"case {case}: rows={rows} cols={cols} f16={f16} smooth={smooth} strided={strided}"
        y, sc = capi.dynamic_quant(x.cuda(), None if sm is None else sm.cuda())
        wy, ws = golden.dynamic_quant(bits(x), "fp16" if f16 else "bf16", None if sm is None else bits(sm))
        assert np.array_equal(y.cpu().numpy(), wy), tag
        assert np.array_equal(sc.cpu().numpy().view(np.uint32), ws.view(np.uint32)), tag
        if not f16 and not smooth and cols % 2 == 0:
            left = bool(rng.random() < 0.5)
            y, sc = capi.swiglu_quant(x.cuda(), activate_left=left)
            wy, ws = golden.swiglu_quant(_bits(x), activate_left=left)
            assert np.array_equal(sc.cpu().numpy().view(np.uint32), ws.view(np.uint32)), tag + " (swiglu_quant)"
            assert np.array_equal(y.cpu().numpy(), wy), tag + " (swiglu_quant)"


@pytest.mark.parametrize("rows,cols", [(2048, 4096), (33, 1000), (7, 24), (5, 1), (3, 20000), (64, 14336), (1, 8)])
@pytest.mark.parametrize("f16", [False, True])
def test_dynamic_quant_asymmetric(capi, golden, rows, cols, f16):
    """Codes, scales and offsets bit-identical to the oracle (every operation a separate float32 operation): aligned
    and odd widths, pitched rows, smooth scales, a constant row."""
    g = torch.Generator().manual_seed(rows + cols)
    dt = torch.float16 if f16 else torch.bfloat16
    bits = _f16_bits if f16 else _bits
    wide = (torch.randn(rows, cols + 8, generator=g) * 3 + 1).to(dt)
    wide[0, :] = 2.5                                                # a constant row: scale 0, offset 0, codes 0
    for x in (wide[:, :cols].contiguous(), wide[:, :cols]):
        for sm in (None, (torch.rand(cols, generator=g) + 0.5).to(dt)):
            y, s, o = capi.dynamic_quant_asymmetric(x.cuda(), None if sm is None else sm.cuda())
            wy, ws, wo = golden.dynamic_quant_asymmetric(bits(x), "fp16" if f16 else "bf16", None if sm is None else bits(sm))
            assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
            assert np.array_equal(o.cpu().numpy().view(np.uint32), wo.view(np.uint32))
            assert np.array_equal(y.cpu().numpy(), wy)
    assert not y[0].any() or sm is not None


def test_dynamic_quant_asymmetric_extreme_rows(capi, golden):
    """Rows that leave the range where the kernel divides through the row's reciprocal (huge elements, a tiny spread, tiny
    elements next to a normal spread) and rows inside it: bit-identical to the oracle either way."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(12, 512, generator=g) * 2
    x[1] = x[1] * 1e30                                              # elements above 2^60
    x[2] = x[2] * 1e-30                                             # scale below 2^-60
    x[3, :6] = torch.tensor([1e-30, -1e-30, 1e-38, 0.0, -0.0, 3e-20])   # tiny numerators, ordinary scale
    x[4] = 1000.0 + x[4] * 1e-3                                     # small spread around a large value
    x[5, 0] = 3e38
    x[6, 10] = float("nan")                                         # a NaN is skipped by the extremes and becomes code 0;
    x[7, ::67] = float("nan")                                       # its wavefront rounds the ordinary way, the others do not
    x = x.to(torch.bfloat16)
    with np.errstate(all="ignore"):
        wy, ws, wo = golden.dynamic_quant_asymmetric(_bits(x), "bf16", None)
    y, s, o = capi.dynamic_quant_asymmetric(x.cuda(), None)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(o.cpu().numpy().view(np.uint32), wo.view(np.uint32))
    assert np.array_equal(y.cpu().numpy(), wy)
    assert y[6, 10] == 0 and not y[7, ::67].any() and y[6].any() and y[7].any()
    # a wide row with one NaN: only the wavefront that holds it leaves the integer-clamp path
    xw = (torch.randn(3, 4096, generator=g) * 3 + 1).to(torch.bfloat16)
    xw[1, 1234] = float("nan")
    wy, ws, wo = golden.dynamic_quant_asymmetric(_bits(xw), "bf16", None)
    y, s, o = capi.dynamic_quant_asymmetric(xw.cuda(), None)
    assert np.array_equal(y.cpu().numpy(), wy) and y[1, 1234] == 0
    assert np.array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(o.cpu().numpy().view(np.uint32), wo.view(np.uint32))


# ------------------------------------------------------------------ error paths (host side, no kernel runs)

@pytest.mark.parametrize("rows,half", [(64, 14336), (512, 4096), (33, 512), (5, 100), (3, 16384 + 8), (7, 24), (5, 28672),
                                       (2, 65536), (2, 65536 + 8)])
@pytest.mark.parametrize("left", [True, False])
def test_swiglu_quant_with_smooth_scales(capi, golden, rows, half, left):
    """Fused SwiGLU + smooth scales + dynamic quantisation equals the oracle's composition bit for bit: the
    register-resident kernel (four and eight vectors per thread), the two-pass kernel (odd or very wide rows), both
    orientations, and through the operator."""
    import pytorch_amd as pa
    g = torch.Generator().manual_seed(rows + half)
    x = (torch.randn(rows, 2 * half, generator=g) * 2).to(torch.bfloat16)
    x[0] = 0
    sm = (torch.rand(half, generator=g) * 3 + 0.05).to(torch.bfloat16)
    wy, ws = golden.swiglu_quant(_bits(x), left, _bits(sm))
    y, s = capi.swiglu_quant(x.cuda(), left, sm.cuda())
    assert np.array_equal(s.cpu().numpy(), ws) and np.array_equal(y.cpu().numpy(), wy)
    y2, s2 = pa.npu_swiglu_quant(x.cuda(), smooth_scales=sm.cuda(), activate_left=left, quant_mode=1)
    assert torch.equal(y2, y) and torch.equal(s2, s)


@pytest.mark.parametrize("rows,half", [(64, 14336), (2048, 14336), (33, 512), (5, 100), (3, 16384 + 8), (7, 24), (5, 28672),
                                       (2, 65536), (2, 65536 + 8)])
@pytest.mark.parametrize("left", [True, False])
def test_swiglu_quant_equals_composition(capi, golden, rows, half, left):
    g = torch.Generator().manual_seed(rows + half)
    x = (torch.randn(rows, 2 * half, generator=g) * 2).to(torch.bfloat16)
    x[0, :] = 0                                                     # a zero row: scale 0, codes 0
    y, s = capi.swiglu_quant(x.cuda(), activate_left=left)
    want_y, want_s = golden.swiglu_quant(_bits(x), activate_left=left)
    assert np.array_equal(s.cpu().numpy().view(np.uint32), want_s.view(np.uint32))
    assert np.array_equal(y.cpu().numpy(), want_y)
    if left:                                                        # and the two separate kernels give the same bits
        y2, s2 = capi.dynamic_quant(capi.swiglu(x.cuda()))
        assert torch.equal(y, y2) and torch.equal(s, s2)


def test_c_abi_rejects_bad_arguments(capi):
    L = capi.lib()
    assert L.mi355_dynamic_quant(None, 0, None, None, None, -1, 8, 8, None) == -1
    assert L.mi355_dynamic_quant(None, 7, None, None, None, 1, 8, 8, None) == -1
    assert L.mi355_quant_matmul(None, None, None, None, 0, None, 0, None, 0, 4, 4, 4, 4, 4, 1, 4, None, 0, None) == -1
    assert L.mi355_weight_quant_matmul(None, 0, None, 5, None, None, None, None, 1, 8, 32, 0, 8, 1, 32, 8, 1, 8, None, 0, None) == -1
    assert L.mi355_weight_quant_matmul(None, 9, None, 8, None, None, None, None, 1, 8, 32, 0, 8, 1, 32, 8, 1, 8, None, 0, None) == -1
    assert L.mi355_anti_quant(None, 5, None, 1, None, 0, None, 0, 1, 8, 8, 8, None) == -1
    assert L.mi355_anti_quant(None, 4, None, 1, None, 0, None, 7, 1, 8, 1, 8, None) == -1
    assert b"workspace" in L.mi355_status_string(-4)
    x1 = torch.zeros(128, 128, dtype=torch.int8, device="cuda")
    x2 = torch.zeros(128, 128, dtype=torch.int8, device="cuda")
    with pytest.raises(capi.Mi355Error, match="workspace"):
        capi.quant_matmul(x1, x2, None, out_dtype=torch.int32, workspace=torch.empty(16, dtype=torch.int8, device="cuda"))


@pytest.mark.parametrize("bits,N", [(8, 100), (4, 104)])
def test_weight_quant_padded_rows_get_their_workspace(capi, golden, bits, N):
    """The workspace query knows no strides: a weight whose rows are padded to 128 bytes is accepted by kernels (with a K
    split) that the dense row length rules out, so the query must cover that plan as well."""
    M, K = 8, 4096
    if bits == 8:
        d = workloads.w8a16_inputs(seed=N, M=M, K=K, N=N)
        gs, cols, pitch = 0, N, 128
    else:
        d = workloads.w4a16_inputs(seed=N, M=M, K=K, N=N, group_size=128)
        gs, cols, pitch = 128, N // 8, 32
    wide = torch.zeros(K, pitch, dtype=d["weight"].dtype)
    wide[:, :cols] = d["weight"]
    w = wide.cuda()[:, :cols]
    assert w.stride(0) == pitch
    out = capi.weight_quant_matmul(d["x"].cuda(), w, d["antiquant_scale"].cuda(), d["antiquant_offset"].cuda(), group_size=gs)
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]), group_size=gs)
    bf16_gate(out, torch.from_numpy(gold), floor=True)


def test_w4a16_repeated_launches_reuse_workspace(capi, golden):
    """The split-K exchange reuses one workspace and its arrival counters across launches: alternate two
    problems many times and check every result (a stale partial sum or counter would show up here)."""
    cases = []
    for seed in (11, 12):
        d = workloads.w4a16_inputs(seed=seed, M=8, K=4096, N=2048, group_size=128)
        _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                             _bits(d["antiquant_offset"]), group_size=128)
        cases.append(([d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")], torch.from_numpy(gold)))
    first = [None, None]
    for it in range(40):
        args, gold = cases[it % 2]
        out = capi.weight_quant_matmul(*args, group_size=128)
        if first[it % 2] is None:
            bf16_gate(out, gold)
            first[it % 2] = out.clone()
        else:
            assert torch.equal(out, first[it % 2]), f"launch {it} differs from the first launch of the same problem"


@pytest.mark.parametrize("M", [8, 128])
def test_weight_quant_exchange_timeout_is_reported(capi, golden, M):
    """The int4 kernels' collecting workgroup waits a bounded number of polls for the other K chunks' partial sums.  The
    give-up path is driven from the host so that every kernel still ends normally: a knob lets only the collecting chunk
    run and shortens the bound to four polls.  The launch then reports MI355_OK (it was enqueued), its outputs hold NaN
    instead of a wrong sum, the workspace's sticky status word makes mi355_workspace_status fail once and clears the
    zero area, and the next ordinary launch on the same workspace is right again (M = 8: the decode kernel, M = 128: the
    register-expanding tiled kernel)."""
    d = workloads.w4a16_inputs(seed=3, M=M)
    x, w, sc, of = (d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset"))
    need = capi.lib().mi355_weight_quant_matmul_workspace(M, 14336, 4096, 4, 128)
    assert need > 0
    ws = capi._wq_workspace(x.device, need)
    good = capi.weight_quant_matmul(x, w, sc, of, group_size=128)
    capi.workspace_status(ws)                                   # nothing to report
    capi.set_tuning("MI355_WQ_MAX_POLLS", 4)
    capi.set_tuning("MI355_WQ_ONLY_CHUNK", -1)
    try:
        bad = capi.weight_quant_matmul(x, w, sc, of, group_size=128)
    finally:
        capi.set_tuning("MI355_WQ_MAX_POLLS", 0)
        capi.set_tuning("MI355_WQ_ONLY_CHUNK", 0)
    torch.cuda.synchronize()
    assert torch.isnan(bad.float()).all(), "the collector must mark what it could not sum"
    with pytest.raises(capi.Mi355Error, match="status word"):
        capi.workspace_status(ws)
    capi.workspace_status(ws)                                   # reported once, then cleared
    assert int(ws[:capi.ZERO_AREA_BYTES].count_nonzero()) == 0
    again = capi.weight_quant_matmul(x, w, sc, of, group_size=128)
    assert torch.equal(again, good)
