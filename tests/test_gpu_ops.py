"""GPU tests of the torch operators (torch.ops.npu.*) and the contrib modules at the benchmark
shapes: full-size parity against the CPU oracle where the oracle finishes in seconds, row
samples plus exact checksums where it does not, module-versus-operator equality as in the
reference's test/contrib/test_linear_{quant,a8w8_quant,weight_quant}.py, and the
Llama-3-8B-shaped W8A8 MLP chain checked stage by stage."""
import numpy as np
import pytest
import torch

from pytorch_amd.testing import workloads, bf16_gate, assert_rtol_equal

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pa():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    import pytorch_amd
    return pytorch_amd


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def test_c1_dynamic_quant_full_size(pa, golden):
    for seed in (0, 1):
        x = workloads.dynamic_quant_input(seed=seed)
        y, s = pa.npu_dynamic_quant(x.cuda())
        yg, sg = golden.dynamic_quant(_bits(x))
        assert np.array_equal(s.cpu().numpy(), sg) and np.array_equal(y.cpu().numpy(), yg)
        assert (y.abs().amax(-1) == 127).all()


@pytest.mark.parametrize("weight_nk", [True, False])
def test_c2_quant_matmul_full_size(pa, golden, weight_nk):
    d = workloads.quant_matmul_inputs(seed=0, weight_nk=weight_nk)
    x1, x2 = d["x1"].cuda(), d["x2"].cuda()
    acc = pa.npu_quant_matmul(x1, x2, d["scale"].cuda(), output_dtype=torch.int32).cpu()
    # exact checksum of every output row: sum_n acc[m,n] == x1[m,:] . (sum_n x2[:,n])
    colsum = d["x2"].to(torch.int64).sum(1)
    assert torch.equal(acc.to(torch.int64).sum(1), d["x1"].to(torch.int64) @ colsum)
    # ... and of every output column
    rowsum = d["x1"].to(torch.int64).sum(0)
    assert torch.equal(acc.to(torch.int64).sum(0), rowsum @ d["x2"].to(torch.int64))
    # every accumulator against the oracle's own integer product (about a second on the host cores)
    want_acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    assert np.array_equal(acc.numpy(), want_acc)
    for bias in (d["bias"], None):
        out = pa.npu_quant_matmul(x1, x2, d["scale"].cuda(), pertoken_scale=d["pertoken_scale"].cuda(),
                                  bias=None if bias is None else bias.cuda(), output_dtype=torch.bfloat16)
        want = golden.quant_matmul_epilogue(want_acc, d["scale"].numpy(), d["pertoken_scale"].numpy(),
                                            None if bias is None else _bits(bias))
        assert np.array_equal(_bits(out), want)


@pytest.mark.parametrize("weight_nk", [False, True])
def test_c3_w8a16_full_size(pa, golden, weight_nk):
    d = workloads.w8a16_inputs(seed=0, weight_nk=weight_nk)
    out = pa.npu_weight_quant_batchmatmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                          d["antiquant_offset"].cuda())
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]))
    print("C3", weight_nk, bf16_gate(out, torch.from_numpy(gold)))


@pytest.mark.parametrize("M", [1, 8, 32, 128])
def test_c4_w4a16_full_size(pa, golden, M):
    d = workloads.w4a16_inputs(seed=0, M=M)
    out = pa.npu_weight_quant_batchmatmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                          d["antiquant_offset"].cuda(), None, None, None, 128)
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]), group_size=128)
    print("C4", M, bf16_gate(out, torch.from_numpy(gold)))
    # inner_precise=1 (the vendor's faster accumulation mode) is accepted and gives the high-precision result
    fast = pa.npu_weight_quant_batchmatmul(d["x"].cuda(), d["weight"].cuda(), d["antiquant_scale"].cuda(),
                                           d["antiquant_offset"].cuda(), None, None, None, 128, 1)
    assert torch.equal(fast, out)


def test_quant_matmul_batched_and_scale_variants(pa, golden):
    g = torch.Generator().manual_seed(0)
    x1 = torch.randint(-127, 128, (2, 3, 16, 256), generator=g, dtype=torch.int8)
    x2 = torch.randint(-127, 128, (3, 256, 48), generator=g, dtype=torch.int8)
    s = torch.rand(48, generator=g) * 1e-2
    out = pa.npu_quant_matmul(x1.cuda(), x2.cuda(), s.cuda(), output_dtype=torch.bfloat16).cpu()
    assert out.shape == (2, 3, 16, 48)
    for b0 in range(2):
        for b1 in range(3):
            want, _ = golden.quant_matmul(x1[b0, b1].numpy(), x2[b1].numpy(), s.numpy())
            assert np.array_equal(_bits(out[b0, b1]), want)
    # per-token scales [M] with batches: they apply to every matrix of the batch (one weight, and a batch of weights)
    ps = torch.rand(16, generator=g) + 0.5
    bias16 = (torch.randn(48, generator=g) * 0.05).to(torch.bfloat16)
    out = pa.npu_quant_matmul(x1.cuda(), x2[1].cuda(), s.cuda(), pertoken_scale=ps.cuda(), bias=bias16.cuda(),
                              output_dtype=torch.bfloat16).cpu()
    outb = pa.npu_quant_matmul(x1.cuda(), x2.cuda(), s.cuda(), pertoken_scale=ps.cuda(), bias=bias16.cuda(),
                               output_dtype=torch.bfloat16).cpu()
    assert out.shape == (2, 3, 16, 48) and outb.shape == (2, 3, 16, 48)
    for b0 in range(2):
        for b1 in range(3):
            want, _ = golden.quant_matmul(x1[b0, b1].numpy(), x2[1].numpy(), s.numpy(), ps.numpy(), _bits(bias16))
            assert np.array_equal(_bits(out[b0, b1]), want)
            want, _ = golden.quant_matmul(x1[b0, b1].numpy(), x2[b1].numpy(), s.numpy(), ps.numpy(), _bits(bias16))
            assert np.array_equal(_bits(outb[b0, b1]), want)
    # leading batch of x1 against one weight (shapes of test/test_fake_tensor.py:1886-1894), per-tensor bf16 scale
    x1 = torch.randint(-127, 128, (1, 1, 1024), generator=g, dtype=torch.int8)
    x2 = torch.randint(-127, 128, (1, 1024, 100), generator=g, dtype=torch.int8)
    sb = torch.tensor([0.0078125], dtype=torch.bfloat16)
    bias = (torch.randn(1, 1, 100, generator=g)).to(torch.bfloat16)
    out = pa.npu_quant_matmul(x1.cuda(), x2.cuda(), sb.cuda(), bias=bias.cuda(), output_dtype=torch.bfloat16).cpu()
    want, _ = golden.quant_matmul(x1[0].numpy(), x2[0].numpy(), sb.float().numpy(), None, _bits(bias.reshape(-1)))
    assert out.shape == (1, 1, 100) and np.array_equal(_bits(out[0]), want)


def test_linear_quant_module_equals_operator(pa):
    """Module output == direct operator output (test/contrib/test_linear_quant.py:24-63)."""
    from pytorch_amd.contrib.module import LinearQuant, LinearA8W8Quant
    d = workloads.quant_matmul_inputs(seed=3, M=96, K=512, N=384, weight_nk=True)
    w_nk = d["x2"].t()                               # stored [N, K], contiguous
    assert w_nk.is_contiguous()
    for cls in (LinearQuant, LinearA8W8Quant):
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            m = cls(512, 384, bias=True, pertoken_scale=True, output_dtype=torch.bfloat16).cuda()
        m.weight.data = w_nk.cuda()
        m.scale.data = d["scale"].cuda()
        m.pertoken_scale.data = d["pertoken_scale"].cuda()
        m.bias.data = d["bias"].cuda()
        got = m(d["x1"].cuda())
        want = pa.npu_quant_matmul(d["x1"].cuda(), d["x2"].cuda(), d["scale"].cuda(),
                                   pertoken_scale=d["pertoken_scale"].cuda(), bias=d["bias"].cuda(),
                                   output_dtype=torch.bfloat16)
        assert_rtol_equal(got, want, 0.001)
        assert torch.equal(got, want)


def test_linear_quant_a4w4_prepare(pa):
    """LinearQuant with an int4 weight (int32 words, linear_quant.py:40-50): prepare_() widens the weight once; the
    forward pass then gives the same bits as the unprepared module, for 2-D and batched int32 activations."""
    from pytorch_amd.contrib.module import LinearQuant
    g = torch.Generator().manual_seed(8)
    rnd = lambda *sh: torch.randint(-2 ** 31, 2 ** 31 - 1, sh, generator=g, dtype=torch.int64).to(torch.int32)  # noqa: E731
    m = LinearQuant(512, 256, bias=True, pertoken_scale=True, output_dtype=torch.bfloat16).cuda()
    m.weight.data = rnd(256, 64).cuda()
    m.scale.data = (torch.rand(256, generator=g) * 1e-2).cuda()
    m.bias.data = torch.randint(-100, 100, (256,), generator=g, dtype=torch.int32).cuda()
    x = rnd(48, 64).cuda()
    m.pertoken_scale.data = (torch.rand(48, generator=g) * 1e-2).cuda()
    want = m(x)
    m.prepare_()
    assert m._prepared_i8.dtype == torch.int8 and m._prepared_i8.shape == (256, 512)
    assert torch.equal(m(x), want)
    m2 = LinearQuant(512, 256, bias=False, output_dtype=torch.float16).cuda()
    m2.weight.data, m2.scale.data = m.weight.data, m.scale.data
    xb = rnd(2, 3, 64).cuda()
    want = m2(xb)
    assert torch.equal(m2.prepare_()(xb), want) and want.shape == (2, 3, 256)


def test_quant_matmul_int8_output_operator_and_module(pa, golden):
    """npu_quant_matmul with output_dtype None / int8 (test/test_fake_tensor.py:1886-1895): a float32 scale is packed
    like npu_trans_quant_param packs it, an int64 scale is taken as packed; LinearQuant's default configuration
    (float32 scale, no pertoken_scale, output_dtype None) goes through npu_trans_quant_param like the reference's
    forward (linear_quant.py:104-112) and equals the direct call."""
    from pytorch_amd.contrib.module import LinearQuant
    d = workloads.quant_matmul_inputs(seed=21, M=48, K=256, N=192, weight_nk=True)
    g = torch.Generator().manual_seed(2)
    scale = (torch.rand(192, generator=g) + 0.5) * 4e-4
    offset = torch.randint(-20, 20, (192,), generator=g).float()
    bias = torch.randint(-3000, 3000, (192,), generator=g, dtype=torch.int32)
    want = golden.quant_matmul_requant(d["x1"].numpy(), d["x2"].numpy(), golden.trans_quant_param(scale.numpy(), offset.numpy()),
                                       bias.numpy())
    x1, x2 = d["x1"].cuda(), d["x2"].cuda()
    out = pa.npu_quant_matmul(x1, x2, scale.cuda(), offset=offset.cuda(), bias=bias.cuda())
    assert out.dtype == torch.int8 and np.array_equal(out.cpu().numpy(), want)
    qp = pa.npu_trans_quant_param(scale.cuda(), offset.cuda())
    assert qp.dtype == torch.int64 and np.array_equal(qp.cpu().numpy(), golden.trans_quant_param(scale.numpy(), offset.numpy()))
    out2 = pa.npu_quant_matmul(x1, x2, qp, offset=offset.cuda(), bias=bias.cuda(), output_dtype=torch.int8)
    assert torch.equal(out, out2)
    # batched x1 against one weight
    xb = torch.stack([d["x1"], d["x1"].flip(0)]).cuda()
    ob = pa.npu_quant_matmul(xb, x2, qp, bias=bias.cuda(), output_dtype=torch.int8)
    assert ob.shape == (2, 48, 192) and torch.equal(ob[0], out) and torch.equal(ob[1], out.flip(0))
    m = LinearQuant(256, 192, bias=True, offset=True).cuda()
    m.weight.data = d["x2"].t().contiguous().cuda()
    m.scale.data, m.offset.data, m.bias.data = scale.cuda(), offset.cuda(), bias.cuda()
    assert torch.equal(m(x1), out)
    # float16 output of the module: packed scale, same numbers as the float32 scale
    m16 = LinearQuant(256, 192, bias=False, output_dtype=torch.float16).cuda()
    m16.weight.data = d["x2"].t().contiguous().cuda()
    m16.scale.data = scale.cuda()
    assert torch.equal(m16(x1), pa.npu_quant_matmul(x1, x2, scale.cuda(), output_dtype=torch.float16))


def test_linear_quant_module_default_int32_bias_and_fp16(pa, golden):
    """LinearQuant as its constructor builds it (int32 bias, linear_quant.py:92) with float16 and bfloat16 outputs,
    against the oracle's statement of the formula."""
    from pytorch_amd.contrib.module import LinearQuant
    d = workloads.quant_matmul_inputs(seed=5, M=48, K=256, N=192, weight_nk=True)
    g = torch.Generator().manual_seed(9)
    bias = torch.randint(-50000, 50000, (192,), generator=g, dtype=torch.int32)
    acc = golden.int8_gemm(d["x1"].numpy(), d["x2"].numpy())
    for dt, name, pertoken in ((torch.float16, "fp16", False), (torch.bfloat16, "bf16", True), (torch.float16, "fp16", True)):
        m = LinearQuant(256, 192, bias=True, pertoken_scale=pertoken, output_dtype=dt).cuda()
        assert m.bias.dtype == torch.int32
        m.weight.data = d["x2"].t().contiguous().cuda()
        m.scale.data = d["scale"].cuda()
        m.bias.data = bias.cuda()
        if pertoken:
            m.pertoken_scale.data = d["pertoken_scale"].cuda()
        got = m(d["x1"].cuda())
        want = golden.quant_matmul_epilogue_ex(acc, d["scale"].numpy(), d["pertoken_scale"].numpy() if pertoken else None,
                                               bias.numpy(), out=name)
        assert got.dtype == dt
        assert np.array_equal(got.cpu().view(torch.int16).numpy().view(np.uint16), want)


def test_linear_weight_quant_module_equals_operator(pa, golden):
    """test/contrib/test_linear_weight_quant.py:53-73 with bf16 parameters, plus the per-group int4 case."""
    from pytorch_amd.contrib.module import LinearWeightQuant
    d = workloads.w8a16_inputs(seed=5, M=32, K=1024, N=256, weight_nk=True)
    m = LinearWeightQuant(1024, 256, bias=False, antiquant_offset=True).cuda()
    m.weight.data = d["weight"].t().cuda()           # [N, K]
    m.antiquant_scale.data = d["antiquant_scale"].cuda()
    m.antiquant_offset.data = d["antiquant_offset"].cuda()
    got = m(d["x"].cuda())
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]))
    bf16_gate(got, torch.from_numpy(gold))
    assert_rtol_equal(got.float().cpu().numpy(), gold, 0.01)
    # per-group parameters stored [N, G] and passed transposed
    d4 = workloads.w4a16_inputs(seed=6, M=4, K=512, N=128, group_size=128)
    m4 = LinearWeightQuant(512, 128, bias=False, antiquant_offset=True, antiquant_group_size=128).cuda()
    m4.antiquant_scale.data = d4["antiquant_scale"].t().contiguous().cuda()
    m4.antiquant_offset.data = d4["antiquant_offset"].t().contiguous().cuda()
    direct = pa.npu_weight_quant_batchmatmul(d4["x"].cuda(), d4["weight"].cuda(), d4["antiquant_scale"].cuda(),
                                             d4["antiquant_offset"].cuda(), None, None, None, 128)
    via = pa.npu_weight_quant_batchmatmul(d4["x"].cuda(), d4["weight"].cuda(), m4.antiquant_scale.t(),
                                          m4.antiquant_offset.t(), None, None, None, 128)
    assert torch.equal(direct, via)
    # a prefill-sized batch (3-D input, bias) through the module: the [N, K] weight takes the tiled kernel's K-major loader
    d = workloads.w8a16_inputs(seed=7, M=96, K=1024, N=384, weight_nk=True)
    mb = LinearWeightQuant(1024, 384, bias=True, antiquant_offset=True).cuda()
    mb.weight.data = d["weight"].t().cuda()
    mb.antiquant_scale.data = d["antiquant_scale"].cuda()
    mb.antiquant_offset.data = d["antiquant_offset"].cuda()
    bias = torch.randn(384, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    mb.bias.data = bias.cuda()
    got = mb(d["x"].cuda().view(2, 48, 1024))
    assert got.shape == (2, 48, 384)
    _, gold = golden.weight_quant_matmul(_bits(d["x"]), d["weight"].numpy(), _bits(d["antiquant_scale"]),
                                         _bits(d["antiquant_offset"]), bias_u16=_bits(bias))
    bf16_gate(got.view(96, 384), torch.from_numpy(gold))


def test_linear_weight_quant_module_int4(pa, golden):
    """The module with an int4 weight stored [out_features, in_features / 8] int32 and per-group parameters stored
    [N, G] (linear_weight_quant.py:71,98-109): its transposed views reach the kernel for words along K without a copy;
    after prepare_() the same module runs on the repacked copy (words along N).  Both against the oracle."""
    from pytorch_amd.contrib.module import LinearWeightQuant
    for (M, K, N, f16) in [(4, 512, 128, False), (48, 1024, 384, True), (8, 4096, 2048, False)]:
        d = workloads.w4a16_inputs(seed=M + N, M=M, K=K, N=N, group_size=128)
        dt = torch.float16 if f16 else torch.bfloat16
        m = LinearWeightQuant(K, N, bias=True, antiquant_offset=True, antiquant_group_size=128).cuda()
        w_nk = torch.from_numpy(golden.pack_int4(np.ascontiguousarray(d["weight_int4_values"].numpy().T)))
        sc, of = d["antiquant_scale"].to(dt), d["antiquant_offset"].to(dt)
        bias = torch.randn(N, generator=torch.Generator().manual_seed(2)).to(dt)
        m.weight.data = w_nk.cuda()
        m.antiquant_scale.data, m.antiquant_offset.data = sc.t().contiguous().cuda(), of.t().contiguous().cuda()
        m.bias.data = bias.cuda()
        x = d["x"].to(dt)
        bits = (lambda t: t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16))
        _, gold = golden.weight_quant_matmul(bits(x), d["weight"].numpy(), bits(sc), bits(of), group_size=128,
                                             dtype="fp16" if f16 else "bf16", bias_u16=bits(bias))
        got = m(x.cuda())
        assert got.shape == (M, N) and got.dtype == dt
        bf16_gate(got, torch.from_numpy(gold))
        m.prepare_()
        assert m._prepared[0].shape == (K, N // 8) and torch.equal(m._prepared[0].cpu(), d["weight"])
        assert m.weight.shape == (N, K // 8)                       # the parameter itself is untouched
        bf16_gate(m(x.cuda()), torch.from_numpy(gold))
    with pytest.raises(RuntimeError, match="inner dimensions differ"):
        pa.npu_weight_quant_batchmatmul(x.cuda(), w_nk.cuda()[:, :-1].t(), sc.cuda(), of.cuda(), None, None, None, 128)


def _mlp_gpu(pa, d):
    x = d["x"].cuda()
    xq, xs = pa.npu_dynamic_quant(x)
    gu = pa.npu_quant_matmul(xq, d["w_gate_up"].cuda().t(), d["scale_gate_up"].cuda(), pertoken_scale=xs,
                             output_dtype=torch.bfloat16)
    act = pa.npu_swiglu(gu)
    aq, as_ = pa.npu_dynamic_quant(act)
    out = pa.npu_quant_matmul(aq, d["w_down"].cuda().t(), d["scale_down"].cuda(), pertoken_scale=as_,
                              output_dtype=torch.bfloat16)
    return xq, xs, gu, act, aq, as_, out


def test_c5_mlp_chain_stagewise(pa, golden):
    """Each GPU stage against the oracle applied to that stage's actual GPU input."""
    d = workloads.mlp_inputs(seed=0, M=64)
    xq, xs, gu, act, aq, as_, out = _mlp_gpu(pa, d)
    yg, sg = golden.dynamic_quant(_bits(d["x"]))
    assert np.array_equal(xq.cpu().numpy(), yg) and np.array_equal(xs.cpu().numpy(), sg)
    want, _ = golden.quant_matmul(xq.cpu().numpy(), d["w_gate_up"].t().numpy(), d["scale_gate_up"].numpy(), xs.cpu().numpy())
    assert np.array_equal(_bits(gu), want)
    dist = golden.bf16_ulp_distance(_bits(act), golden.swiglu(_bits(gu)))
    assert dist.max() <= 1 and (dist == 0).mean() > 0.995
    yg, sg = golden.dynamic_quant(_bits(act))
    assert np.array_equal(aq.cpu().numpy(), yg) and np.array_equal(as_.cpu().numpy(), sg)
    want, _ = golden.quant_matmul(aq.cpu().numpy(), d["w_down"].t().numpy(), d["scale_down"].numpy(), as_.cpu().numpy())
    assert np.array_equal(_bits(out), want)
    assert torch.isfinite(out.float()).all()


def test_swiglu_quant_operator(pa, golden):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 40, 1024, generator=g).to(torch.bfloat16)
    for left in (True, False):
        y, s = pa.npu_swiglu_quant(x.cuda(), activate_left=left, quant_mode=1)
        wy, ws = golden.swiglu_quant(_bits(x).reshape(120, 1024), activate_left=left)
        assert y.shape == (3, 40, 512) and s.shape == (3, 40)
        assert np.array_equal(y.cpu().numpy().reshape(120, 512), wy)
        assert np.array_equal(s.cpu().numpy().reshape(120).view(np.uint32), ws.view(np.uint32))
    # the default orientation of the vendor signature activates the right half
    y0, _ = pa.npu_swiglu_quant(x.cuda(), quant_mode=1)
    assert torch.equal(y0, pa.npu_swiglu_quant(x.cuda(), activate_left=False, quant_mode=1)[0])
    with pytest.raises(RuntimeError, match="quant_mode"):
        pa.npu_swiglu_quant(x.cuda())
    # a strided 2-D view (the columns of a wider buffer) is read in place
    wide = torch.randn(16, 3000, generator=g).to(torch.bfloat16).cuda()
    view = wide[:, :2048]
    y1, s1 = pa.npu_swiglu_quant(view, activate_left=True, quant_mode=1)
    y2, s2 = pa.npu_dynamic_quant(pa.npu_swiglu(view.contiguous()))
    assert torch.equal(y1, y2) and torch.equal(s1, s2)


def test_dynamic_quant_asymmetric_operator(pa, golden):
    """torch_npu.npu_dynamic_quant_asymmetric(input, smooth_scales=...) as test/test_fake_tensor.py:1689-1709 calls it:
    three outputs, scale and offset shaped like the input without its last dimension."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(4, 64, 1024, generator=g).to(torch.float16)
    sm = (torch.rand(1024, generator=g) + 0.5).to(torch.float16)
    y, s, o = pa.npu_dynamic_quant_asymmetric(x.cuda(), smooth_scales=sm.cuda())
    assert y.shape == (4, 64, 1024) and y.dtype == torch.int8
    assert s.shape == (4, 64) and s.dtype == torch.float32 and o.shape == (4, 64) and o.dtype == torch.float32
    bits = lambda t: t.contiguous().view(torch.int16).numpy().view(np.uint16)  # noqa: E731
    wy, ws, wo = golden.dynamic_quant_asymmetric(bits(x), "fp16", bits(sm))
    assert np.array_equal(y.cpu().numpy(), wy) and np.array_equal(s.cpu().numpy(), ws) and np.array_equal(o.cpu().numpy(), wo)
    # what the quantisation means: (y - offset) * scale reproduces x * smooth to half a step
    back = (y.float().cpu() - o.cpu().unsqueeze(-1)) * s.cpu().unsqueeze(-1)
    assert ((back - x.float() * sm.float()).abs() <= 0.5001 * s.cpu().unsqueeze(-1) + 1e-6).all()
    with pytest.raises(RuntimeError, match="group_index"):
        pa.npu_dynamic_quant_asymmetric(x.cuda(), group_index=torch.zeros(1, dtype=torch.int32, device="cuda"))


def test_anti_quant_operator(pa, golden):
    """torch_npu.npu_anti_quant(x, scale, offset=..., dst_dtype=..., src_dtype=...) as test/custom_ops/test_npu_anti_quant.py
    calls it: default float16 output, leading batch dimensions, packed int4 widening the last dimension by 8, and the
    same-device error message of :86-88."""
    g = torch.Generator().manual_seed(2)
    x = torch.randint(-127, 128, (2, 10, 100), generator=g, dtype=torch.int8)
    scale, offset = torch.rand(100, generator=g) * 200 - 100, torch.rand(100, generator=g) * 200 - 100
    out = pa.npu_anti_quant(x.cuda(), scale.cuda(), offset=offset.cuda())
    assert out.dtype == torch.float16 and out.shape == (2, 10, 100)
    want = golden.anti_quant(x.numpy().reshape(20, 100), scale.numpy(), offset.numpy(), dst="fp16")
    assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16).reshape(20, 100), want)
    out = pa.npu_anti_quant(x.cuda(), scale.cuda(), dst_dtype=torch.bfloat16, src_dtype=torch.int8)
    want = golden.anti_quant(x.numpy().reshape(20, 100), scale.numpy(), None, dst="bf16")
    assert np.array_equal(_bits(out).reshape(20, 100), want)
    x4 = torch.randint(-2 ** 31, 2 ** 31 - 1, (10, 25), generator=g, dtype=torch.int64).to(torch.int32)
    s4, o4 = torch.rand(200, generator=g) * 2 - 1, torch.rand(200, generator=g) * 16 - 8
    out = pa.npu_anti_quant(x4.cuda(), s4.cuda(), offset=o4.cuda(), dst_dtype=torch.bfloat16)
    assert out.shape == (10, 200)
    assert np.array_equal(_bits(out), golden.anti_quant(x4.numpy(), s4.numpy(), o4.numpy(), dst="bf16"))
    with pytest.raises(RuntimeError, match="Expected all tensors to be on the same device"):
        pa.npu_anti_quant(x.cuda(), scale.cuda(), offset=offset)
    with pytest.raises(RuntimeError, match="dst_dtype"):
        pa.npu_anti_quant(x.cuda(), scale.cuda(), dst_dtype=torch.float32)


def test_npu_quantize_operator(pa, golden):
    """torch_npu.npu_quantize(inputs, scales, zero_points, dtype, axis, div_mode=True) as the reference's wrapper test
    calls it (test/onnx/test_wrapper_onnx_ops.py:1444-1452: float32 [5,16,8], eight scales of 0.1, int32 zero points,
    torch.quint8, axis 2), plus the other output types, a bf16 input with bf16 scales and the multiply mode."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(5, 16, 8, generator=g)
    scales = torch.tensor([0.1] * 8)
    zps = torch.tensor([0] * 8, dtype=torch.int32)
    out = pa.npu_quantize(x.cuda(), scales.cuda(), zps.cuda(), dtype=torch.quint8, axis=2)
    assert out.dtype == torch.uint8 and out.shape == (5, 16, 8)
    assert np.array_equal(out.cpu().numpy(), golden.quantize(x.numpy(), scales.numpy(), zps.float().numpy(), "uint8", 2))
    zps = torch.randint(-5, 5, (16,), generator=g, dtype=torch.int32)
    sc16 = (torch.rand(16, generator=g) + 0.5).to(torch.bfloat16)
    xb = (x * 30).to(torch.bfloat16)
    out = pa.npu_quantize(xb.cuda(), sc16.cuda(), zps.cuda(), torch.qint8, 1)
    assert out.dtype == torch.int8
    assert np.array_equal(out.cpu().numpy(), golden.quantize(xb.float().numpy(), sc16.float().numpy(), zps.float().numpy(), "int8", 1))
    out = pa.npu_quantize(xb.cuda(), sc16.cuda(), None, torch.qint32, 1, False)
    assert out.dtype == torch.int32
    assert np.array_equal(out.cpu().numpy(), golden.quantize(xb.float().numpy(), sc16.float().numpy(), None, "int32", 1, False))
    # a non-contiguous input is quantised by value
    xt = xb.cuda().transpose(0, 2)
    out = pa.npu_quantize(xt, sc16.cuda(), None, torch.qint8, 1)
    assert np.array_equal(out.cpu().numpy(), golden.quantize(xb.float().numpy().transpose(2, 1, 0), sc16.float().numpy(), None, "int8", 1))
    with pytest.raises(RuntimeError, match="Expected all tensors to be on the same device"):
        pa.npu_quantize(x.cuda(), scales, None, torch.qint8, 2)


def _rand_words(g, *shape):
    return torch.randint(-2 ** 31, 2 ** 31 - 1, shape, generator=g, dtype=torch.int64).to(torch.int32)


def test_quant_matmul_a4w4_operator(pa, golden):
    """Both operands int32 words of eight int4 values: the reference's own shapes (16,8) x (64,5) -> (16,40) float16
    with a single scale and an int32 bias (test/test_fake_tensor.py:1917-1923) and the transposed [N, K/8] weight of
    the module example (linear_quant.py:40-50), then a larger case with every output type, a pertoken scale and a
    batch of activations.  Accumulators bit-exact, floating outputs bit-identical to the oracle (same float32
    operation order)."""
    g = torch.Generator().manual_seed(5)
    x1, x2 = _rand_words(g, 16, 8), _rand_words(g, 64, 5)
    scale, bias = torch.rand(1, generator=g) * 0.01, torch.randint(-1000, 1000, (40,), generator=g, dtype=torch.int32)
    out = pa.npu_quant_matmul(x1.cuda(), x2.cuda(), scale.cuda(), offset=None, bias=bias.cuda(), output_dtype=torch.float16)
    assert out.shape == (16, 40) and out.dtype == torch.float16
    want, acc = golden.quant_matmul_a4w4(x1.numpy(), x2.numpy(), scale.numpy(), None, bias.numpy(), out="fp16")
    assert np.array_equal(out.cpu().view(torch.int16).numpy().view(np.uint16), want)
    got_acc = pa.npu_quant_matmul(x1.cuda(), x2.cuda(), scale.cuda(), output_dtype=torch.int32)
    assert np.array_equal(got_acc.cpu().numpy(), acc)

    w = _rand_words(g, 128, 2)                                   # weight [N, K/8]; the module passes weight.T
    xa = _rand_words(g, 1, 2)
    out = pa.npu_quant_matmul(xa.cuda(), w.cuda().t(), scale.cuda(), output_dtype=torch.bfloat16)
    assert out.shape == (1, 128)
    want, _ = golden.quant_matmul_a4w4(xa.numpy(), w.numpy().T, scale.numpy(), out="bf16")
    assert np.array_equal(_bits(out), want)

    M, K, N = 200, 1024, 1536
    x1, wn, wk = _rand_words(g, 3, M, K // 8), _rand_words(g, K, N // 8), _rand_words(g, N, K // 8)
    sc, ps = torch.rand(N, generator=g) * 0.02 + 1e-3, torch.rand(M, generator=g) * 0.1 + 1e-3
    for x2, x2_np in ((wn.cuda(), wn.numpy()), (wk.cuda().t(), wk.numpy().T)):
        want, acc = golden.quant_matmul_a4w4(x1[1].numpy(), x2_np, sc.numpy(), ps.numpy(), None, out="bf16")
        out = pa.npu_quant_matmul(x1[1].cuda(), x2, sc.cuda(), pertoken_scale=ps.cuda(), output_dtype=torch.bfloat16)
        assert np.array_equal(_bits(out), want)
        accs = pa.npu_quant_matmul(x1.cuda(), x2, sc.cuda(), output_dtype=torch.int32)      # batched activations
        assert accs.shape == (3, M, N) and np.array_equal(accs[1].cpu().numpy(), acc)
        assert np.array_equal(accs[2].cpu().numpy(), golden.quant_matmul_a4w4(x1[2].numpy(), x2_np, None, out="int32")[1])
    # the module with an int32 weight [N, K/8] (linear_quant.py:40-50): same bits as the operator and the oracle
    from pytorch_amd.contrib.module import LinearQuant
    m = LinearQuant(K, N, bias=False, pertoken_scale=True, output_dtype=torch.bfloat16).cuda()
    m.weight.data, m.scale.data, m.pertoken_scale.data = wk.cuda(), sc.cuda(), ps.cuda()
    got = m(x1[1].cuda())
    assert np.array_equal(_bits(got), golden.quant_matmul_a4w4(x1[1].numpy(), wk.numpy().T, sc.numpy(), ps.numpy(), out="bf16")[0])
    with pytest.raises(RuntimeError, match="both be int8, or both int32"):
        pa.npu_quant_matmul(x1[0].cuda(), torch.zeros(K, N, dtype=torch.int8, device="cuda"), sc.cuda(), output_dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="int4 inner dimensions differ"):
        pa.npu_quant_matmul(x1[0].cuda(), wn.cuda()[:K - 8], sc.cuda(), output_dtype=torch.bfloat16)


def test_graph_replays_match_eager(pa):
    """The operators launched from a captured HIP graph: every replay (with eager launches of the same operators in
    between, which share the per-stream workspaces and their arrival counters) must reproduce the eager bits.  Covers
    the K-split exchanges of both matmuls (bf16 and re-quantised int8 output), the per-call weight transpose, the tiled
    weight-only kernel with its row-sum pre-kernel, the fused SwiGLU quantisation, smooth scales and npu_quantize."""
    g = torch.Generator().manual_seed(11)
    d = workloads.mlp_inputs(seed=3, M=64, hidden=1024, inter=4096)
    x = d["x"].cuda()
    wd, sd = d["w_down"].cuda().t(), d["scale_down"].cuda()
    d4 = workloads.w4a16_inputs(seed=4, M=8, K=4096, N=1024, group_size=128)
    d4b = workloads.w4a16_inputs(seed=5, M=96, K=2048, N=1024, group_size=128)
    a4 = [d4[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")]
    a4b = [d4b[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")]
    act = torch.randn(64, 8192, generator=g).to(torch.bfloat16).cuda()
    qp = pa.npu_trans_quant_param((torch.rand(1024, generator=g) * 1e-4 + 1e-4).cuda(), torch.randint(-8, 8, (1024,), generator=g).float().cuda())
    bi = torch.randint(-1000, 1000, (1024,), generator=g, dtype=torch.int32).cuda()
    wkn = wd.contiguous()                                                          # the same weight stored [K, N]
    sm = (torch.rand(1024, generator=g) + 0.5).to(torch.bfloat16).cuda()
    zs, zz = (torch.rand(1024, generator=g) * 0.05 + 0.01).cuda(), torch.randint(-8, 8, (1024,), generator=g, dtype=torch.int32).cuda()

    def run():
        q, s = pa.npu_swiglu_quant(act, activate_left=True, quant_mode=1)          # [64, 4096] int8
        o1 = pa.npu_quant_matmul(q, wd, sd, pertoken_scale=s, output_dtype=torch.bfloat16)   # narrow output: K split
        o2 = pa.npu_weight_quant_batchmatmul(*a4, None, None, None, 128)            # streaming kernel, K split
        o3 = pa.npu_weight_quant_batchmatmul(*a4b, None, None, None, 128)           # row sums + tiled kernel, K split
        q1, s1 = pa.npu_dynamic_quant(x)
        o4 = pa.npu_quant_matmul(q, wd, qp, bias=bi, output_dtype=torch.int8)      # re-quantised output, K split
        o5 = pa.npu_quant_matmul(q, wkn, sd, pertoken_scale=s, output_dtype=torch.bfloat16)   # [K,N] weight: transposed per call
        q2, s2 = pa.npu_dynamic_quant(x, smooth_scales=sm)
        q3 = pa.npu_quantize(x, zs, zz, torch.qint8, -1)
        return q, s, o1, o2, o3, q1, s1, o4, o5, q2, s2, q3

    want = [t.clone() for t in run()]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        run()                                                                      # warm-up on the capture stream
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            outs = run()
    torch.cuda.current_stream().wait_stream(stream)
    for it in range(4):
        for t in outs:
            t.zero_() if t.dtype != torch.int8 else t.fill_(7)
        graph.replay()
        torch.cuda.synchronize()
        for got, exp in zip(outs, want):
            assert torch.equal(got, exp), f"replay {it} differs from the eager result"
        eager = run()                                                              # eager work between the replays
        torch.cuda.synchronize()
        for got, exp in zip(eager, want):
            assert torch.equal(got, exp)


def test_prepared_quant_matmul_weight(pa, golden):
    """prepare_quant_matmul_weight stores a [K,N] weight K-major once: the prepared tensor equals the original, has the
    strides the GEMM reads directly (no per-call transpose, hence no workspace for it) and gives the same bits."""
    from pytorch_amd import _capi
    d = workloads.quant_matmul_inputs(seed=5, M=96, K=512, N=384, weight_nk=False, bias=True)
    x1, w = d["x1"].cuda(), d["x2"].cuda()
    assert w.stride() == (384, 1)
    wp = pa.prepare_quant_matmul_weight(w)
    assert wp.shape == w.shape and wp.stride() == (1, 512) and torch.equal(wp, w)
    assert pa.prepare_quant_matmul_weight(wp) is wp                      # already K-major: unchanged
    L = _capi.lib()
    assert L.mi355_quant_matmul_workspace(96, 384, 512, *w.stride()) > L.mi355_quant_matmul_workspace(96, 384, 512, *wp.stride())
    kw = dict(pertoken_scale=d["pertoken_scale"].cuda(), bias=d["bias"].cuda(), output_dtype=torch.bfloat16)
    a, b = pa.npu_quant_matmul(x1, w, d["scale"].cuda(), **kw), pa.npu_quant_matmul(x1, wp, d["scale"].cuda(), **kw)
    want, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(), _bits(d["bias"]))
    assert torch.equal(a, b) and np.array_equal(_bits(b), want)
    # ragged sizes take the byte-wise transposing kernel; a batch of weights keeps its leading dimension
    wr = torch.randint(-127, 128, (3, 40, 24), dtype=torch.int8, generator=torch.Generator().manual_seed(1)).cuda()
    wrp = pa.prepare_quant_matmul_weight(wr)
    assert torch.equal(wrp, wr) and wrp.stride()[-2:] == (1, 40)


@pytest.mark.parametrize("M", [1, 16, 64, 128, 1024])
def test_prepared_weights_with_padded_row_pitch(pa, golden, M):
    """Weights whose rows are 4096 bytes are prepared with a row pitch of 4224: every kernel that a row count selects
    (decode, streaming loop, 256-row tiles) reads them through the pitch and returns the bits of the unprepared call,
    which equal the oracle's; the modules keep such a copy after prepare_()."""
    from pytorch_amd.contrib.module import LinearQuant, LinearWeightQuant
    from pytorch_amd.testing import workloads
    K, N = 4096, 1536
    d = workloads.quant_matmul_inputs(seed=M, M=M, K=K, N=N, weight_nk=True, bias=True)
    x1, w = d["x1"].cuda(), d["x2"].cuda()
    wp = pa.prepare_quant_matmul_weight(w)
    assert wp.stride() == (1, 4224) and torch.equal(wp, w) and pa.prepare_quant_matmul_weight(wp) is wp
    assert pa.prepare_quant_matmul_weight(w, row_pad=False) is w
    kw = dict(pertoken_scale=d["pertoken_scale"].cuda(), bias=d["bias"].cuda(), output_dtype=torch.bfloat16)
    out = pa.npu_quant_matmul(x1, wp, d["scale"].cuda(), **kw)
    want, _ = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(), _bits(d["bias"]))
    assert np.array_equal(_bits(out), want)
    assert torch.equal(pa.npu_quant_matmul(x1, wp, None, output_dtype=torch.int32), pa.npu_quant_matmul(x1, w, None, output_dtype=torch.int32))
    # a contiguous [K, N] weight: transposed and padded in one preparation
    wkn = w.contiguous()
    wkp = pa.prepare_quant_matmul_weight(wkn)
    assert wkp.stride() == (1, 4224) and torch.equal(wkp, wkn)
    assert torch.equal(pa.npu_quant_matmul(x1, wkp, d["scale"].cuda(), **kw), out)
    # the module keeps the padded copy and gives the same result with and without it
    m = LinearQuant(K, N, bias=True, pertoken_scale=True, output_dtype=torch.bfloat16).cuda()
    m.weight.data = w.t().contiguous()
    m.scale.data = d["scale"].cuda()
    m.pertoken_scale.data = d["pertoken_scale"].cuda()
    m.bias.data = d["bias"].cuda()
    ref = m(x1)
    assert torch.equal(ref, out)
    m.prepare_()
    assert m._prepared_i8 is not None and m._prepared_i8.stride() == (4224, 1)
    assert torch.equal(m(x1), ref)
    if M <= 64:
        dw = workloads.w8a16_inputs(seed=M, M=M, K=K, N=N)
        lw = LinearWeightQuant(K, N, bias=False, antiquant_offset=True)
        lw.weight.data = dw["weight"].t().contiguous()
        lw.antiquant_scale.data, lw.antiquant_offset.data = dw["antiquant_scale"], dw["antiquant_offset"]
        lw = lw.cuda()
        ref = lw(dw["x"].cuda())
        lw.prepare_()
        assert lw._prepared is not None and lw._prepared[0].stride() == (1, 4224)
        assert torch.equal(lw(dw["x"].cuda()), ref)


def test_workspace_outlives_growth_after_capture(pa):
    """A graph captured with a small split-K workspace must replay correctly after an eager call on the same stream
    needed a larger one: the superseded buffer is kept alive (and zeroed at rest), never handed back to the allocator."""
    from pytorch_amd import _capi
    g = torch.Generator().manual_seed(21)
    M, K, N = 64, 4096, 256
    q = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda().t()
    sc, ps = (torch.rand(N, generator=g) * 1e-2).cuda(), (torch.rand(M, generator=g) * 1e-2).cuda()
    Kb, Nb = 14336, 4096
    qb = torch.randint(-127, 128, (M, Kb), generator=g, dtype=torch.int8).cuda()
    wb = torch.randint(-127, 128, (Nb, Kb), generator=g, dtype=torch.int8).cuda().t()
    scb = (torch.rand(Nb, generator=g) * 1e-2).cuda()
    small_ws = _capi.lib().mi355_quant_matmul_workspace(M, N, K, 1, K)
    big_ws = _capi.lib().mi355_quant_matmul_workspace(M, Nb, Kb, 1, Kb)
    floor = _capi.ZERO_AREA_BYTES + (1 << 20)          # the smallest buffer the operator layer allocates
    assert 0 < small_ws <= floor < big_ws, (small_ws, big_ws)          # the second call must outgrow the first buffer
    small = lambda: pa.npu_quant_matmul(q, w, sc, pertoken_scale=ps, output_dtype=torch.bfloat16)
    big = lambda: pa.npu_quant_matmul(qb, wb, scb, pertoken_scale=ps, output_dtype=torch.bfloat16)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        want = small().clone()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = small()
        want_big = big().clone()                       # eager, same stream: allocates the larger workspace
        stream.synchronize()
        for it in range(3):
            out.zero_()
            graph.replay()
            stream.synchronize()
            assert torch.equal(out, want), f"replay {it} after the workspace grew differs"
            assert torch.equal(big(), want_big)
            assert torch.equal(small(), want)
    torch.cuda.synchronize()


def test_captures_without_warmup_on_their_stream(pa):
    """The usual capture idiom warms up on one stream and captures on another (torch.cuda.graph picks its own): a
    split-K operator then meets a stream without a workspace while capturing.  Every capture gets a workspace of its
    own from the graph's memory pool, zeroed by a node of that graph; two graphs captured one after the other on the
    same stream, replayed alternately with eager calls in between, must all reproduce the eager bits."""
    g = torch.Generator().manual_seed(22)
    M, K = 64, 4096
    q = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8).cuda()
    ops, wants = [], []
    for N in (256, 1024):
        w = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8).cuda().t()
        sc = (torch.rand(N, generator=g) * 1e-2).cuda()
        ops.append(lambda w=w, sc=sc: pa.npu_quant_matmul(q, w, sc, output_dtype=torch.bfloat16))
        wants.append(ops[-1]().clone())                # eager, default stream: also the one-time kernel set-up
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()                       # fresh stream: no workspace is cached for it
    graphs, outs = [], []
    for op in ops:
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=stream):
            outs.append(op())
        graphs.append(gr)
    for it in range(3):
        for gr, out, want, op in zip(graphs, outs, wants, ops):
            out.zero_()
            gr.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want), f"replay {it} differs"
            with torch.cuda.stream(stream):
                assert torch.equal(op(), want)         # eager call on the capture stream: its own workspace
            torch.cuda.synchronize()


def test_c5_mlp_prefill_properties(pa, golden):
    """M = 2048: rows are independent, so any subset of rows run alone must reproduce the same bits."""
    d = workloads.mlp_inputs(seed=1, M=2048)
    full = _mlp_gpu(pa, d)[-1]
    rows = torch.tensor([0, 5, 777, 2047])
    sub = dict(d)
    sub["x"] = d["x"][rows]
    part = _mlp_gpu(pa, sub)[-1]
    assert torch.equal(full[rows.cuda()], part)


def test_c5_mlp_prefill_stagewise_oracle(pa, golden):
    """M = 2048 against the oracle: every stage works row by row, so the oracle is applied, stage by stage, to a sample of
    128 rows of the GPU's own stage inputs that touches every 256-row tile (the plans this size selects: the 256x224 tile
    for gate|up, a 256x256 tile with K split in two for the down projection).  Quantisations and both GEMMs bit-exact,
    SwiGLU within one bf16 ulp."""
    d = workloads.mlp_inputs(seed=1, M=2048)
    rows = torch.cat([torch.arange(0, 2048, 32) + 3, torch.arange(0, 2048, 32) + 29]).sort().values
    xq, xs, gu, act, aq, as_, out = (t.cpu()[rows] for t in _mlp_gpu(pa, d))
    yg, sg = golden.dynamic_quant(_bits(d["x"][rows]))
    assert np.array_equal(xq.numpy(), yg) and np.array_equal(xs.numpy(), sg)
    want, _ = golden.quant_matmul(xq.numpy(), d["w_gate_up"].t().numpy(), d["scale_gate_up"].numpy(), xs.numpy())
    assert np.array_equal(_bits(gu), want)
    dist = golden.bf16_ulp_distance(_bits(act), golden.swiglu(_bits(gu)))
    assert dist.max() <= 1 and (dist == 0).mean() > 0.995
    yg, sg = golden.dynamic_quant(_bits(act))
    assert np.array_equal(aq.numpy(), yg) and np.array_equal(as_.numpy(), sg)
    want, _ = golden.quant_matmul(aq.numpy(), d["w_down"].t().numpy(), d["scale_down"].numpy(), as_.numpy())
    assert np.array_equal(_bits(out), want)


def test_prepare_weight_quant_weight(pa):
    """An int8 weight contiguous along N is rewritten once into the contrib module's storage ([N, K], passed as its
    transposed view): equal values, strides (1, K), the operator's result within the gate of the unprepared call's;
    weights already stored that way and int4 words come back unchanged."""
    from pytorch_amd.testing import workloads, bf16_gate
    d = workloads.w8a16_inputs(seed=5, M=16, K=4096, N=2304)
    w = d["weight"].cuda()
    wp = pa.prepare_weight_quant_weight(w, row_pad=False)
    assert wp.shape == w.shape and wp.stride() == (1, 4096) and torch.equal(wp, w)
    assert pa.prepare_weight_quant_weight(wp, row_pad=False) is wp
    wpp = pa.prepare_weight_quant_weight(w)                              # rows of 4096 bytes: padded pitch by default
    assert wpp.stride() == (1, 4224) and torch.equal(wpp, w) and pa.prepare_weight_quant_weight(wpp) is wpp
    assert torch.equal(pa.prepare_weight_quant_weight(wp), w) and pa.prepare_weight_quant_weight(wp).stride() == (1, 4224)
    words = torch.zeros(64, 8, dtype=torch.int32, device="cuda")
    assert pa.prepare_weight_quant_weight(words) is words
    x, sc, of = d["x"].cuda(), d["antiquant_scale"].cuda(), d["antiquant_offset"].cuda()
    ref = pa.npu_weight_quant_batchmatmul(x, w, sc, of)
    out = pa.npu_weight_quant_batchmatmul(x, wp, sc, of)
    bf16_gate(out, ref.float().cpu())
    assert torch.equal(pa.npu_weight_quant_batchmatmul(x, wpp, sc, of), out)     # the pitch changes no bit


def test_linear_weight_quant_reference_test_shape(pa):
    """test/contrib/test_linear_weight_quant.py:53-73 as it stands: m, k, n = 1024, 11264, 1664, float16 activations,
    an int8 weight drawn as randn().to(int8) and kept [n, k] by the module, per-channel float16 scale and offset drawn
    from randn().  Two goldens: the formula with float32 arithmetic for (w + offset) * scale, which is this build's
    contract (compared the way assertRtolEqual compares float16 arrays, testcase.py:158-227: at most 0.1 % of the
    elements off by more than 1e-3), and the test's own CPU formula (:20-28), which rounds the sum and the product to
    float16 before the float32 matmul.  Against the latter the exact antiquantisation differs by a few 1e-4 of a
    column's typical magnitude, which is more than 1e-3 of the smaller outputs: the comparison holds at the 0.01 the
    reference's call names, not at the 1e-3 that assertRtolEqual applies to float16 arrays."""
    from pytorch_amd.contrib.module import LinearWeightQuant
    from pytorch_amd.testing.compare import rtol_failures
    m, k, n = 1024, 11264, 1664
    g = torch.Generator().manual_seed(0)
    x_cpu = torch.randn((m, k), generator=g, dtype=torch.float32).to(torch.float16)
    weight_cpu = torch.randn((n, k), generator=g, dtype=torch.float32).to(torch.float16).to(torch.int8).to(torch.float16)
    scale_cpu = torch.randn((n,), generator=g, dtype=torch.float32).to(torch.float16)
    offset_cpu = torch.randn((n,), generator=g, dtype=torch.float32).to(torch.float16)
    model = LinearWeightQuant(k, n, bias=False, dtype=torch.float16, antiquant_offset=True, quant_scale=False, quant_offset=False,
                              antiquant_group_size=0).cuda()
    model.weight.data = weight_cpu.to(torch.int8).cuda()
    model.antiquant_scale.data = scale_cpu.cuda()
    model.antiquant_offset.data = offset_cpu.cuda()
    out = model(x_cpu.cuda()).cpu()
    assert out.dtype == torch.float16 and out.shape == (m, n)
    w = weight_cpu.transpose(0, 1)
    x32 = x_cpu.to(torch.float32)
    exact = torch.matmul(x32, (w.float() + offset_cpu.float()) * scale_cpu.float()).numpy().astype("float16")
    assert_rtol_equal(exact, out.numpy(), 0.01)                                  # float16 arrays: 1e-3, 0.1 % of the elements
    rounded = torch.matmul(x32, ((w + offset_cpu) * scale_cpu).to(torch.float32)).numpy().astype("float16")
    assert_rtol_equal(rounded, out.numpy(), 0.01, prec16=0.01)
    frac = rtol_failures(rounded, out.numpy(), 1e-3) / out.numel()
    print("reference shape: fraction beyond 1e-3 of the float16-rounded golden", round(frac, 4))
    assert frac < 0.25


def test_device_failure_report_reaches_the_operator_layer(pa):
    """torch.ops.npu path of the same report: after a launch whose collector gave up (driven from the host, every kernel
    ends normally), pytorch_amd.check_device_status() raises once, clears the workspace, and the operator works again."""
    from pytorch_amd import _capi
    d = workloads.w4a16_inputs(seed=4, M=8)
    args = [d[k].cuda() for k in ("x", "weight", "antiquant_scale", "antiquant_offset")] + [None, None, None, 128]
    good = pa.npu_weight_quant_batchmatmul(*args)
    pa.check_device_status()
    _capi.set_tuning("MI355_WQ_MAX_POLLS", 4)
    _capi.set_tuning("MI355_WQ_ONLY_CHUNK", -1)
    try:
        bad = pa.npu_weight_quant_batchmatmul(*args)
    finally:
        _capi.set_tuning("MI355_WQ_MAX_POLLS", 0)
        _capi.set_tuning("MI355_WQ_ONLY_CHUNK", 0)
    torch.cuda.synchronize()
    assert torch.isnan(bad.float()).all()
    with pytest.raises(RuntimeError, match="device-side failure"):
        pa.check_device_status()
    pa.check_device_status()
    assert torch.equal(pa.npu_weight_quant_batchmatmul(*args), good)


@pytest.mark.gpu
def test_weight_quant_batchmatmul_int8_output(pa, golden):
    """quant_scale / quant_offset of npu_weight_quant_batchmatmul (what LinearWeightQuant constructs and passes,
    torch_npu/contrib/module/linear_weight_quant.py:79-87,106-109): int8 = clamp(rint(out * quant_scale + s9(quant_offset))).
    Against the oracle applied to the operator's own 16-bit result (which other tests compare with the oracle), for
    float32 parameters, for the packed int64 words of npu_trans_quant_param, through the module, and for float16.
    The formula itself has no pin in the reference tree (parity unpinned); the offset's 9-bit range is the reference's
    f32_2_s9 helper (test/contrib/test_linear_weight_quant.py:13-16)."""
    from pytorch_amd.contrib.module import LinearWeightQuant
    g = torch.Generator().manual_seed(11)
    for (dt, name, M, K, N, bits) in [(torch.bfloat16, "bf16", 32, 1024, 256, 8), (torch.float16, "fp16", 5, 512, 384, 8),
                                      (torch.bfloat16, "bf16", 8, 1024, 512, 4)]:
        if bits == 8:
            d = workloads.w8a16_inputs(seed=M, M=M, K=K, N=N, weight_nk=True)
            gs = 0
        else:
            d = workloads.w4a16_inputs(seed=M, M=M, K=K, N=N, group_size=128)
            gs = 128
        x, sc, of = d["x"].to(dt).cuda(), d["antiquant_scale"].to(dt).cuda(), d["antiquant_offset"].to(dt).cuda()
        w = d["weight"].cuda()
        plain = pa.npu_weight_quant_batchmatmul(x, w, sc, of, None, None, None, gs)
        # scales that spread the results over the int8 range and beyond it, offsets beyond the 9-bit range
        qs = (torch.rand(N, generator=g) * 0.5 + 0.05) * (100.0 / max(float(plain.float().abs().max()), 1e-6))
        qo = torch.randn(N, generator=g) * 40.0
        qo[:4] = torch.tensor([300.0, -300.0, 0.5, 1.5])
        want = golden.weight_quant_requant(golden.bits_of(plain), qs.numpy(), qo.numpy(), dtype=name)
        got = pa.npu_weight_quant_batchmatmul(x, w, sc, of, qs.cuda(), qo.cuda(), None, gs)
        assert got.dtype == torch.int8 and got.shape == plain.shape
        assert np.array_equal(got.cpu().numpy(), want)
        assert len(np.unique(want)) > 100 and want.min() == -128 and want.max() == 127
        # no offset, and [1, N] parameters
        want0 = golden.weight_quant_requant(golden.bits_of(plain), qs.numpy(), None, dtype=name)
        got0 = pa.npu_weight_quant_batchmatmul(x, w, sc, of, qs.cuda().view(1, N), None, None, gs)
        assert np.array_equal(got0.cpu().numpy(), want0)
        # the packed words hold the same scale and the same 9-bit offset
        packed = pa.npu_trans_quant_param(qs.cuda(), qo.cuda())
        assert packed.dtype == torch.int64
        gotp = pa.npu_weight_quant_batchmatmul(x, w, sc, of, packed, None, None, gs)
        assert torch.equal(gotp, got)
        if bits == 8:
            m = LinearWeightQuant(K, N, bias=False, antiquant_offset=True, quant_scale=True, quant_offset=True, dtype=dt).cuda()
            m.weight.data = d["weight"].t().contiguous().cuda()
            m.antiquant_scale.data, m.antiquant_offset.data = sc, of
            m.quant_scale.data, m.quant_offset.data = qs.cuda(), qo.cuda()
            assert torch.equal(m(x), got)
    with pytest.raises(RuntimeError, match="quant_offset needs quant_scale"):
        pa.npu_weight_quant_batchmatmul(x, w, sc, of, None, qo.cuda(), None, gs)
    with pytest.raises(RuntimeError, match="already holds the offset"):
        pa.npu_weight_quant_batchmatmul(x, w, sc, of, packed, qo.cuda(), None, gs)
    with pytest.raises(RuntimeError, match="quant_scale must be float32"):
        pa.npu_weight_quant_batchmatmul(x, w, sc, of, qs.to(torch.bfloat16).cuda(), None, None, gs)


@pytest.mark.gpu
def test_npu_dynamic_quant_group_index_operator(pa, golden):
    """torch.ops.npu.npu_dynamic_quant with per-expert smooth scales: 3-D input, int64 totals."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 24, 1024, generator=g).to(torch.bfloat16)
    sm = (torch.rand(3, 1024, generator=g) + 0.5).to(torch.bfloat16)
    totals = [16, 16, 48]
    y, s = pa.npu_dynamic_quant(x.cuda(), smooth_scales=sm.cuda(), group_index=torch.tensor(totals).cuda())
    yg, sg = golden.dynamic_quant_grouped(golden.bits_of(x), golden.bits_of(sm), totals)
    assert y.shape == x.shape and s.shape == x.shape[:-1]
    assert np.array_equal(y.cpu().numpy(), yg) and np.array_equal(s.cpu().numpy(), sg)


@pytest.mark.gpu
def test_npu_dynamic_quant_int4_operator(pa, golden):
    """torch.ops.npu.npu_dynamic_quant(dst_type=torch.quint4x2): int32 words, last dimension an eighth; the words feed
    npu_anti_quant (int4 source) back to values within half a scale step of the input."""
    g = torch.Generator().manual_seed(5)
    x = torch.randn(3, 10, 512, generator=g).to(torch.bfloat16)
    y, s = pa.npu_dynamic_quant(x.cuda(), dst_type=torch.quint4x2)
    yg, sg = golden.dynamic_quant_int4(golden.bits_of(x))
    assert y.dtype == torch.int32 and y.shape == (3, 10, 64) and s.shape == (3, 10)
    assert np.array_equal(y.cpu().numpy(), yg) and np.array_equal(s.cpu().numpy(), sg)
    codes = torch.from_numpy(golden.unpack_int4(yg)).float()
    assert float(((codes * torch.from_numpy(sg)[..., None]) - x.float()).abs().max()) <= 0.5 * float(sg.max()) * 1.001


@pytest.mark.gpu
def test_npu_swiglu_quant_group_index_operator(pa, golden):
    """torch.ops.npu.npu_swiglu_quant with per-expert smooth scales, group_index as running totals (group_list_type 0) and
    as counts (1)."""
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(40, 2048, generator=g) * 2).to(torch.bfloat16)
    sm = (torch.rand(3, 1024, generator=g) + 0.5).to(torch.bfloat16)
    yg, sg = golden.dynamic_quant_grouped(golden.swiglu(golden.bits_of(x)), golden.bits_of(sm), [8, 30, 40])
    for gi, kind in ((torch.tensor([8, 30, 40]), 0), (torch.tensor([8, 22, 10]), 1)):
        y, s = pa.npu_swiglu_quant(x.cuda(), smooth_scales=sm.cuda(), group_index=gi.cuda(), activate_left=True, quant_mode=1,
                                   group_list_type=kind)
        assert np.array_equal(y.cpu().numpy(), yg) and np.array_equal(s.cpu().numpy(), sg)
