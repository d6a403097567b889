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
    print("fixtures written to", HERE)


if __name__ == "__main__":
    main()
