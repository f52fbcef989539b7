"""Runs the C++ adapter self-test (tests/cpp/adapter_test.cpp) on the GPU: the reference-shaped C++ surface
(ops::flash_attention, KVCache::update, GroupedQueryAttention core, scaled_dot_product_attention) against the oracle."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_adapter_suite():
    exe = os.path.join(ROOT, "tests", "cpp", "adapter_test")
    assert os.path.exists(exe), "tests/cpp/adapter_test not built: run __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=170)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "all adapter tests passed" in r.stdout
