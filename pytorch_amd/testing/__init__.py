"""Test helpers that mirror the part of ``torch_npu.testing`` the quantized-operator
tests rely on: the tolerance semantics of ``TestCase.assertRtolEqual``
(torch_npu/testing/testcase.py:158-227) and seeded synthetic workloads."""
from .compare import assert_rtol_equal, bf16_gate, rtol_failures  # noqa: F401
from . import workloads  # noqa: F401
