"""Pins of the oracle's rotary-embedding functions (orc_rope_angles, orc_rope_apply_f32) and of the product's
host-side table helper: against the compiled reference, against the fixture written from it, against the
values the reference's own tests assert, and against what the mathematics fixes."""
import ctypes as C
import os

import numpy as np
import pytest

import _inputs as I
import _oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
needs_ref = pytest.mark.skipif(O.ref is None or not hasattr(O.ref, "vref_rope_frequencies"),
                               reason="compiled reference not present")


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@needs_ref
@pytest.mark.parametrize("S,D,sp,theta", [(4, 4, 0, 1e4), (64, 64, 0, 1e4), (17, 128, 4090, 1e4), (9, 128, 65530, 5e5),
                                          (1, 2, 7, 1e4), (3, 96, 100, 1234.5)])
def test_angles_and_rotation_bit_exact_vs_compiled_reference(S, D, sp, theta):
    ang = O.rope_angles(S, D, sp, theta)
    assert np.array_equal(_bits(ang), _bits(O.ref_rope_angles(S, D, sp, theta)))
    x = I.normal(S * 1000 + D, (2, 3, S, D))
    assert np.array_equal(_bits(O.rope_apply(x, ang)), _bits(O.ref_rope_apply(x, ang)))


def test_fixture_written_from_the_reference():
    z = np.load(os.path.join(GOLD, "rope.npz"), allow_pickle=False)
    for ci, (S, D, sp, th) in enumerate(z["cfgs"]):
        S, D, sp = int(S), int(D), int(sp)
        ang = O.rope_angles(S, D, sp, float(th))
        assert np.array_equal(_bits(ang), _bits(z[f"c{ci}_angles"])), ci
        x = I.normal(8000 + ci, (2, 3, S, D))
        assert bytes(z[f"c{ci}_x_sha"]).hex() == I.sha(x)
        assert np.array_equal(_bits(O.rope_apply(x, ang)), _bits(z[f"c{ci}_out"])), ci


def test_known_answers_of_the_reference_tests():
    # tests/test_rope.cpp:11-39: head_dim 4 -> theta_0 = 1, theta_1 = 0.01; pos m -> [m, 0.01 m]
    ang = O.rope_angles(4, 4, 0)
    assert abs(ang[0, 0]) < 1e-5 and abs(ang[0, 1]) < 1e-5
    assert abs(ang[1, 0] - 1.0) < 1e-5 and abs(ang[1, 1] - 0.01) < 1e-5
    # tests/test_rope.cpp:41-73: ones rotated by angle 0 stay ones; by pi/2 become [-1, 1, -1, 1]
    x = np.ones((1, 1, 1, 4), np.float32)
    assert np.allclose(O.rope_apply(x, O.rope_angles(1, 4, 0)), 1.0, atol=1e-5)
    out = O.rope_apply(x, np.full((1, 2), np.float32(np.pi / 2), np.float32))
    assert np.allclose(out.reshape(-1), [-1, 1, -1, 1], atol=1e-5)
    # tests/test_rope_chapter33.cpp:71-108: position 0 -> cos 1, sin 0; frequencies fall with the pair index
    a = O.rope_angles(2, 64, 0)
    assert np.all(a[0] == 0) and a[1, 0] > 0 and a[1, 0] > a[1, 31]


def test_rotation_is_the_complex_product_and_preserves_norms():
    # closed form: (x0 + i x1) * exp(i a), in float64; a sign slip, swapped pair or adjacent-vs-half split fails
    S, D = 6, 32
    ang = O.rope_angles(S, D, 50)
    x = I.normal(77, (2, 2, S, D))
    out = O.rope_apply(x, ang).astype(np.float64)
    z = (x[..., 0::2].astype(np.float64) + 1j * x[..., 1::2]) * np.exp(1j * ang.astype(np.float64))[None, None]
    assert np.allclose(out[..., 0::2], z.real, atol=2e-6) and np.allclose(out[..., 1::2], z.imag, atol=2e-6)
    # tests/test_rope_chapter33.cpp:112-150
    assert np.allclose(np.linalg.norm(out, axis=-1), np.linalg.norm(x.astype(np.float64), axis=-1), rtol=1e-5)


def test_relative_position_property():
    # tests/test_rope_chapter33.cpp:155-195: <R_m q, R_n k> depends on m - n only
    D = 64
    q, k = I.normal(1, (1, 1, 1, D)), I.normal(2, (1, 1, 1, D))
    def score(m, n):
        qm = O.rope_apply(q, O.rope_angles(1, D, m))
        kn = O.rope_apply(k, O.rope_angles(1, D, n))
        return float(np.sum(qm.astype(np.float64) * kn))
    assert abs(score(5, 2) - score(103, 100)) < 1e-3 * max(1.0, abs(score(5, 2)))
    assert abs(score(5, 2) - score(2, 5)) > 1e-3  # and it is not symmetric


def test_angle_formula_against_float64():
    # dropped factor 2, wrong sign of the exponent or i/D vs 2i/D all fail this
    S, D, sp, th = 5, 128, 300, 10000.0
    ang = O.rope_angles(S, D, sp, th).astype(np.float64)
    i = np.arange(D // 2)
    want = (sp + np.arange(S))[:, None] * th ** (-2.0 * i / D)[None]
    assert np.allclose(ang, want, rtol=3e-6)


def test_product_host_table_matches_oracle_bitwise():
    from vesper_amd import _ffi
    for (n, D, sp, th) in [(40, 128, 0, 1e4), (7, 64, 32760, 5e5)]:
        tab = np.empty((n, D // 2, 2), np.float32)
        _ffi.lib.vsp_rope_fill_table(tab.ctypes.data_as(C.c_void_p), sp, n, D, th)
        # the oracle rotating the unit vector (1, 0) of every pair returns exactly (cos, sin) of the pair's angle
        x = np.zeros((1, 1, n, D), np.float32)
        x[..., 0::2] = 1.0
        cs = O.rope_apply(x, O.rope_angles(n, D, sp, th))[0, 0]
        assert np.array_equal(_bits(tab[..., 0]), _bits(cs[:, 0::2]))
        assert np.array_equal(_bits(tab[..., 1]), _bits(cs[:, 1::2]))
