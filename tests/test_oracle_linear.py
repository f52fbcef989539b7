"""The oracle's restatement of the attention modules' output projection (Linear::forward on a 3-D activation,
src/nn/linear.cpp:41-49 over the batched GEMM loop src/ops/gemm.cpp:254-279): bit-exact against the compiled reference
where that is built, and pinned by what the mathematics fixes (float64 product, identity weight, linearity, bias)."""
import numpy as np
import pytest

import _inputs as I
import _oracle as O


@pytest.mark.parametrize("B,T,K,N,bias", [(2, 1, 64, 48, True), (1, 3, 200, 33, False), (3, 2, 130, 130, True), (1, 1, 1, 1, True)])
def test_bit_exact_against_the_compiled_reference(B, T, K, N, bias):
    if O.ref is None or not hasattr(O.ref, "vref_linear"):
        pytest.skip("oracle/_ref not built here")
    x, w = I.normal(70, (B, T, K)), I.normal(71, (N, K), scale=0.1)
    b = I.normal(72, (N,)) if bias else None
    want = O.ref_linear(x, w, b)
    got = O.linear(x, w, b)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_against_float64_and_special_cases():
    x, w, b = I.normal(73, (4, 2, 300)), I.normal(74, (50, 300), scale=0.1), I.normal(75, (50,))
    y = O.linear(x, w, b)
    want = x.astype(np.float64) @ w.astype(np.float64).T + b
    assert np.abs(y - want).max() <= 2e-5 * np.abs(want).max()
    # a transposed operand or a dropped bias would show here
    assert np.abs(y - (x.astype(np.float64) @ w.astype(np.float64).T)).max() > 0.1
    eye = np.eye(300, dtype=np.float32)
    assert np.array_equal(O.linear(x, eye), x)                      # identity weight
    sel = np.zeros((2, 300), np.float32)
    sel[0, 7] = 1.0
    sel[1, 299] = -2.0
    out = O.linear(x, sel)
    assert np.array_equal(out[..., 0], x[..., 7]) and np.array_equal(out[..., 1], -2.0 * x[..., 299])   # rows of w pick inputs
    # the sum runs in index order in fp32: 1 + 2^-24 + 2^-24 stays 1 in that order, whereas summing the small terms first gives 1 + 2^-23
    xs = np.array([[1.0, 2.0**-24, 2.0**-24]], np.float32)
    assert O.linear(xs, np.ones((1, 3), np.float32))[0, 0] == np.float32(1.0)
