"""Pins of the oracle's attention backward (orc_flash_attention_backward_f32): the compiled reference, the fixture
written from it, float64 closed-form gradients, and central finite differences of the forward (the reference's own
gradient check, tests/test_flash_attention.cpp:342-405)."""
import os

import numpy as np
import pytest

import _inputs as I
import _oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(O.ref is None or not hasattr(O.ref, "vref_flash_attention_backward"),
                               reason="compiled reference not present")


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def closed_form_grads(dout, q, k, v, scale, causal):
    """float64: P = softmax(scale q k^T + mask); dV = P^T dO; dP = dO V^T; dS = P*(dP - rowsum(P*dP)); dQ = scale dS K;
    dK = scale dS^T Q.  Independent of the oracle's algebra (it uses rowsum(P*dP), not rowsum(dO*O))."""
    q, k, v, dout = [x.astype(np.float64) for x in (q, k, v, dout)]
    s = np.einsum("bhid,bhjd->bhij", q, k) * scale
    if causal:
        n = s.shape[-1]
        s = np.where(np.tril(np.ones((n, n), bool)), s, -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    dv = np.einsum("bhij,bhid->bhjd", p, dout)
    dp = np.einsum("bhid,bhjd->bhij", dout, v)
    ds = p * (dp - (p * dp).sum(-1, keepdims=True))
    return scale * np.einsum("bhij,bhjd->bhid", ds, k), scale * np.einsum("bhij,bhid->bhjd", ds, q), dv


def _case(B, H, N, D, causal, seed):
    q, k, v = I.qkv(seed, B, H, H, N, N, D)
    dout = I.normal(seed + 5, (B, H, N, D))
    scale = float(np.float32(1.0 / np.sqrt(D)))
    out, lse = O.flash_attention(q, k, v, scale, causal, return_lse=True)
    return q, k, v, dout, scale, out, lse


@needs_ref
@pytest.mark.parametrize("B,H,N,D,causal", [(1, 2, 16, 32, True), (2, 2, 45, 64, True), (1, 3, 64, 16, False),
                                            (1, 1, 97, 128, True)])
def test_bit_exact_vs_compiled_reference(B, H, N, D, causal):
    q, k, v, dout, scale, out, lse = _case(B, H, N, D, causal, 300 + N)
    a = O.flash_attention_backward(dout, q, k, v, out, lse, scale, causal)
    b = O.ref_flash_attention_backward(dout, q, k, v, out, lse, scale, causal)
    for x, y in zip(a, b):
        assert np.array_equal(_bits(x), _bits(y))


def test_fixture_written_from_the_reference():
    z = np.load(os.path.join(GOLD, "flash_backward.npz"), allow_pickle=False)
    for tag in ("t16", "r70", "nc33", "d128"):
        B, H, N, D, causal, seed = [int(x) for x in z[tag + "_meta"]]
        q, k, v, dout, scale, out, lse = _case(B, H, N, D, bool(causal), seed)
        dq, dk, dv = O.flash_attention_backward(dout, q, k, v, out, lse, scale, bool(causal))
        assert np.array_equal(_bits(dq), _bits(z[tag + "_dq"])), tag
        assert np.array_equal(_bits(dk), _bits(z[tag + "_dk"])), tag
        assert np.array_equal(_bits(dv), _bits(z[tag + "_dv"])), tag


@pytest.mark.parametrize("causal", [True, False])
def test_closed_form_float64(causal):
    q, k, v, dout, scale, out, lse = _case(2, 2, 40, 32, causal, 400)
    got = O.flash_attention_backward(dout, q, k, v, out, lse, scale, causal)
    want = closed_form_grads(dout, q, k, v, scale, causal)
    for g, w, name in zip(got, want, "qkv"):
        assert np.abs(g - w).max() <= 2e-5 * max(1.0, np.abs(w).max()), name


def test_central_finite_differences_of_the_forward():
    # loss = sum(out * dout); d loss / d x against (f(x+e) - f(x-e)) / 2e in float64 arithmetic of the closed form
    B, H, N, D, causal = 1, 1, 8, 16, True
    q, k, v, dout, scale, out, lse = _case(B, H, N, D, causal, 500)
    dq, dk, dv = O.flash_attention_backward(dout, q, k, v, out, lse, scale, causal)

    def loss(q_, k_, v_):
        s = np.einsum("bhid,bhjd->bhij", q_, k_) * scale
        s = np.where(np.tril(np.ones((N, N), bool)), s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        return float((np.einsum("bhij,bhjd->bhid", p, v_) * dout).sum())
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    rng = np.random.default_rng(3)
    for which, (arr, grad) in enumerate(((q64, dq), (k64, dk), (v64, dv))):
        for _ in range(10):
            idx = tuple(rng.integers(0, s_) for s_ in arr.shape)
            e = 1e-4
            orig = arr[idx]
            arr[idx] = orig + e
            lp = loss(q64, k64, v64)
            arr[idx] = orig - e
            lm = loss(q64, k64, v64)
            arr[idx] = orig
            num = (lp - lm) / (2 * e)
            assert abs(num - grad[idx]) <= 1e-4 * max(1.0, abs(num)), (which, idx, num, grad[idx])
