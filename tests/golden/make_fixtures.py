"""Writes the committed golden fixtures of this directory.

The reference tree holds no stored vectors for these operators (its op-level tests live in the
un-vendored op-plugin submodule), so the fixtures are (a) hand-typed known answers
(`known_answers.json`, written by hand, NOT by this script) and (b) small seeded problems with
the outputs of the CPU oracle (`*.npz`, written here).  (b) freezes the oracle: a later change
to oracle/golden.c that alters any output bit fails tests/test_golden_fixtures.py.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import golden  # noqa: E402
from pytorch_amd.testing import workloads  # noqa: E402


def bits(t):
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    x = workloads.dynamic_quant_input(seed=21, rows=24, cols=512)
    y, s = golden.dynamic_quant(bits(x))
    np.savez_compressed(os.path.join(HERE, "dynamic_quant.npz"), x=bits(x), y=y, scale=s)

    d = workloads.quant_matmul_inputs(seed=22, M=40, K=256, N=72, weight_nk=True, bias=True)
    out, acc = golden.quant_matmul(d["x1"].numpy(), d["x2"].numpy(), d["scale"].numpy(), d["pertoken_scale"].numpy(),
                                   bits(d["bias"]))
    np.savez_compressed(os.path.join(HERE, "quant_matmul.npz"), x1=d["x1"].numpy(), x2=np.ascontiguousarray(d["x2"].numpy()),
                        scale=d["scale"].numpy(), pertoken_scale=d["pertoken_scale"].numpy(), bias=bits(d["bias"]),
                        acc=acc, out=out)

    d = workloads.w8a16_inputs(seed=23, M=5, K=256, N=64)
    out, outf = golden.weight_quant_matmul(bits(d["x"]), d["weight"].numpy(), bits(d["antiquant_scale"]),
                                           bits(d["antiquant_offset"]))
    np.savez_compressed(os.path.join(HERE, "w8a16.npz"), x=bits(d["x"]), weight=d["weight"].numpy(),
                        scale=bits(d["antiquant_scale"]), offset=bits(d["antiquant_offset"]), out=out, out_f32=outf)

    d = workloads.w4a16_inputs(seed=24, M=3, K=256, N=64, group_size=128)
    out, outf = golden.weight_quant_matmul(bits(d["x"]), d["weight"].numpy(), bits(d["antiquant_scale"]),
                                           bits(d["antiquant_offset"]), group_size=128)
    np.savez_compressed(os.path.join(HERE, "w4a16.npz"), x=bits(d["x"]), weight=d["weight"].numpy(),
                        scale=bits(d["antiquant_scale"]), offset=bits(d["antiquant_offset"]), out=out, out_f32=outf)

    g = torch.Generator().manual_seed(25)
    xs = (torch.randn(6, 64, generator=g) * 3).to(torch.bfloat16)
    np.savez_compressed(os.path.join(HERE, "swiglu.npz"), x=bits(xs), out=golden.swiglu(bits(xs)))
    write_later_fixtures()
    print("fixtures written to", HERE)


def write_later_fixtures():
    """Fixtures of the operators added after the first set (kept in files of their own so that the first set's
    bytes never change): standalone antiquantisation, A4W4 quant_matmul, asymmetric dynamic quantisation."""
    g = torch.Generator().manual_seed(26)
    rnd = lambda *sh: torch.randint(-2 ** 31, 2 ** 31 - 1, sh, generator=g, dtype=torch.int64).to(torch.int32).numpy()  # noqa: E731
    xq = rnd(6, 5)                                                   # packed int4 [6, 40]
    sc, of = (torch.rand(40, generator=g) * 4 - 2).numpy(), (torch.rand(40, generator=g) * 16 - 8).numpy()
    np.savez_compressed(os.path.join(HERE, "anti_quant.npz"), x=xq, scale=sc, offset=of,
                        out_fp16=golden.anti_quant(xq, sc, of, dst="fp16"), out_bf16=golden.anti_quant(xq, sc, of, dst="bf16"))

    x1, x2n, x2k = rnd(16, 8), rnd(64, 5), rnd(40, 8)                # [16,64] x [64,40], words along N / along K
    scale = (torch.rand(1, generator=g) * 0.02).numpy()
    bias = torch.randint(-1000, 1000, (40,), generator=g, dtype=torch.int32).numpy()
    out_n, acc_n = golden.quant_matmul_a4w4(x1, x2n, scale, None, bias, out="fp16")
    out_k, acc_k = golden.quant_matmul_a4w4(x1, x2k.T, scale, None, bias, out="fp16")
    np.savez_compressed(os.path.join(HERE, "a4w4.npz"), x1=x1, x2_n=x2n, x2_k=x2k, scale=scale, bias=bias,
                        out_n=out_n, acc_n=acc_n, out_k=out_k, acc_k=acc_k)

    x = (torch.randn(12, 264, generator=g) * 2 + 0.5).to(torch.bfloat16)
    sm = (torch.rand(264, generator=g) + 0.5).to(torch.bfloat16)
    y, s, o = golden.dynamic_quant_asymmetric(bits(x), "bf16", bits(sm))
    np.savez_compressed(os.path.join(HERE, "dynamic_quant_asymmetric.npz"), x=bits(x), smooth=bits(sm), y=y, scale=s, offset=o)


def write_quantize_fixtures():
    """Static quantisation and the re-quantised int8 output of quant_matmul (files of their own, see above)."""
    g = torch.Generator().manual_seed(31)
    x = (torch.randn(6, 24, 4, generator=g) * 40).to(torch.bfloat16)
    sc = (torch.rand(24, generator=g) + 0.25).numpy()
    zp = torch.randint(-10, 10, (24,), generator=g, dtype=torch.int32).numpy()
    xf = x.float().numpy()
    np.savez_compressed(os.path.join(HERE, "quantize.npz"), x=bits(x), scale=sc, zero_point=zp,
                        q_div_i8=golden.quantize(xf, sc, zp.astype(np.float32), "int8", 1, True),
                        q_mul_u8=golden.quantize(xf, sc, zp.astype(np.float32), "uint8", 1, False))
    x1 = torch.randint(-128, 128, (20, 256), generator=g, dtype=torch.int8).numpy()
    x2 = torch.randint(-128, 128, (256, 48), generator=g, dtype=torch.int8).numpy()
    scale = ((torch.rand(48, generator=g) + 0.5) * 4e-4).numpy()
    offset = torch.randint(-20, 20, (48,), generator=g).float().numpy()
    bias = torch.randint(-3000, 3000, (48,), generator=g, dtype=torch.int32).numpy()
    qp = golden.trans_quant_param(scale, offset)
    np.savez_compressed(os.path.join(HERE, "quant_matmul_int8.npz"), x1=x1, x2=x2, scale=scale, offset=offset, bias=bias,
                        qparam=qp, out=golden.quant_matmul_requant(x1, x2, qp, bias))


if __name__ == "__main__":
    if "--quantize-only" in sys.argv:
        write_quantize_fixtures()
    elif "--later-only" in sys.argv:
        write_later_fixtures()
    else:
        main()
