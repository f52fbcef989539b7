"""Randomised bit-exact comparison of the oracle with the compiled reference (oracle/_ref).
Skipped where the reference binary is absent; tests/test_oracle_golden.py covers that case."""
import numpy as np
import pytest

import _inputs as I
import _oracle as O

pytestmark = pytest.mark.skipif(O.ref is None, reason="oracle/_ref/libvesper_ref.so not built")


@pytest.mark.parametrize("B,H,N,D", [(1, 1, 1, 8), (1, 2, 31, 16), (2, 1, 33, 64), (1, 1, 96, 128), (1, 2, 65, 40)])
@pytest.mark.parametrize("causal", [False, True])
def test_flash_bit_exact(B, H, N, D, causal):
    q, k, v = I.qkv(N * 7 + D, B, H, H, N, N, D)
    scale = float(np.float32(1.0 / np.sqrt(D)))
    a, la = O.flash_attention(q, k, v, scale, causal, return_lse=True)
    b, lb = O.ref_flash_attention(q, k, v, scale, causal)
    assert np.array_equal(a, b) and np.array_equal(la, lb)


@pytest.mark.parametrize("B,H,T,L,D,causal", [(1, 2, 5, 5, 8, True), (2, 2, 7, 19, 16, False), (1, 3, 1, 257, 64, False),
                                               (1, 1, 1, 64, 128, True), (1, 1, 513, 513, 16, True)])
def test_sdpa_bit_exact(B, H, T, L, D, causal):
    q, k, v = I.qkv(T * 3 + L, B, H, H, T, L, D)
    assert np.array_equal(O.sdpa(q, k, v, causal), O.ref_sdpa(q, k, v, causal))


def test_sdpa_causal_rectangular_rejected_like_the_reference():
    q, k, v = I.qkv(9, 1, 1, 1, 4, 6, 8)
    with pytest.raises(O.RefError):
        O.ref_sdpa(q, k, v, True)
    with pytest.raises(O.OracleError):
        O.sdpa(q, k, v, True)


def test_repeat_kv_bit_exact():
    x = I.normal(3, (2, 3, 5, 8))
    for n_rep in (1, 2, 4):
        want = O.ref_repeat_kv(x, n_rep) if n_rep > 1 else x
        assert np.array_equal(O.repeat_kv(x, n_rep), want)


def test_flash_validation_matches_reference_messages():
    cases = [([2, 2, 4], [2, 2, 4], [2, 2, 4], 0.0), ([1, 2, 4, 8], [1, 2, 5, 8], [1, 2, 4, 8], 0.0),
             ([1, 2, 4, 8], [1, 2, 4, 8], [1, 1, 4, 8], 0.0), ([1, 2, 4, 8], [1, 2, 4, 8], [1, 2, 4, 8], 1.0),
             ([1, 2, 4, 8], [1, 2, 4, 8], [1, 2, 4, 8], -0.1)]
    for qs, ks, vs, p in cases:
        with pytest.raises(O.RefError) as er:
            O.ref_flash_attention_shapes(qs, ks, vs, p)
        a = [np.asarray(s, np.int64) for s in (qs, ks, vs)]
        code = O.orc.orc_flash_attention_check(len(qs), O._p(a[0], O.i64p), len(ks), O._p(a[1], O.i64p),
                                               len(vs), O._p(a[2], O.i64p), 0, 0, 0, p)
        assert code != 0 and O.orc.orc_strerror(code).decode() == str(er.value)


@pytest.mark.parametrize("gqa", [False, True])
def test_kv_cache_random_walk(gqa):
    rng = np.random.default_rng(77)
    B, H, S_max, D = 2, 2, 24, 4
    a, b = O.KVCache(B, H, S_max, D), O.RefKVCache(B, H, S_max, D, gqa=gqa)
    for step in range(60):
        if rng.random() < 0.05:
            a.reset(), b.reset()
            assert a.current_seq_len() == b.current_seq_len() == 0
            continue
        T = int(rng.integers(0, 6))
        pos = int(rng.integers(-3, S_max + 3))
        nk, nv = I.normal(step, (B, H, T, D)), I.normal(1000 + step, (B, H, T, D))
        try:
            rk, rv = b.update(nk, nv, pos)
            ok = True
        except O.RefError as e:
            ok, msg = False, str(e)
        if ok:
            ak, av = a.update(nk, nv, pos)
            assert np.array_equal(ak, rk) and np.array_equal(av, rv), (step, T, pos)
        else:
            with pytest.raises(O.OracleError) as e2:
                a.update(nk, nv, pos)
            assert str(e2.value) == msg
        assert a.current_seq_len() == b.current_seq_len(), (step, T, pos)


def test_gqa_ctor_validation():
    assert O.gqa_config(64, 8, 2) == O.ref_gqa_ctor(64, 8, 2) == (8, 4)
    for bad in [(64, 8, 3), (60, 8, 2)]:
        with pytest.raises(O.RefError):
            O.ref_gqa_ctor(*bad)
        with pytest.raises(O.OracleError):
            O.gqa_config(*bad)


def test_bf16_bit_exact_sweep():
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[~np.isnan(f)]
    got = O.f32_to_bf16(f)
    want = np.array([O.ref.vref_f32_to_bf16(float(x)) for x in f[:3000]], np.uint16)
    assert np.array_equal(got[:3000], want)
    back = np.array([O.ref.vref_bf16_to_f32(int(x)) for x in got[:500]], np.float32)
    assert np.array_equal(O.bf16_to_f32(got[:500]).view(np.uint32), back.view(np.uint32))
