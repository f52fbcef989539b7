"""Pins of the oracle that do not need the reference at all: the known answers the reference's
own tests state (cited per test, paths relative to the reference tree), a float64 closed form,
and invariants chosen so that a dropped term, a wrong sign/index or a transposed operand fails."""
import numpy as np
import pytest

import _inputs as I
import _oracle as O


def closed_form(q, k, v, scale, causal):
    """softmax(q k^T * scale + mask) v in float64, GQA by head index division, causal aligned to the END
    of the context (query t sees keys <= L - T + t)."""
    q, k, v = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    B, Hq, T, D = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    n_rep = Hq // Hkv
    out = np.zeros((B, Hq, T, D))
    for b in range(B):
        for h in range(Hq):
            s = q[b, h] @ k[b, h // n_rep].T * scale
            if causal:
                i, j = np.arange(T)[:, None], np.arange(L)[None, :]
                s = np.where(j > i + (L - T), -np.inf, s)
            p = np.exp(s - s.max(-1, keepdims=True))
            p /= p.sum(-1, keepdims=True)
            out[b, h] = p @ v[b, h // n_rep]
    return out


@pytest.mark.parametrize("B,Hq,Hkv,N,D", [(1, 8, 2, 256, 64), (2, 4, 4, 50, 32), (1, 6, 1, 33, 128)])
@pytest.mark.parametrize("causal", [False, True])
def test_closed_form_float64(B, Hq, Hkv, N, D, causal):
    q, k, v = I.qkv(11, B, Hq, Hkv, N, N, D)
    scale = 1.0 / np.sqrt(D)
    want = closed_form(q, k, v, scale, causal)
    n_rep = Hq // Hkv
    flash = O.flash_attention(q, O.repeat_kv(k, n_rep), O.repeat_kv(v, n_rep), float(np.float32(scale)), causal)
    sdpa = O.gqa_attention(q, k, v, causal)
    assert np.abs(flash - want).max() < 2e-6
    assert np.abs(sdpa - want).max() < 2e-6


def test_lse_is_log_sum_exp():
    q, k, v = I.qkv(12, 1, 2, 2, 40, 40, 16)
    _, lse = O.flash_attention(q, k, v, 0.25, True, return_lse=True)
    s = np.einsum("bhnd,bhmd->bhnm", q.astype(np.float64), k.astype(np.float64)) * 0.25
    s[..., np.triu(np.ones((40, 40), bool), 1)] = -np.inf
    want = np.log(np.exp(s - s.max(-1, keepdims=True)).sum(-1)) + s.max(-1)
    assert np.abs(lse - want).max() < 1e-5


def test_hand_computed_2x2():
    # tests/test_attention_chapter32.cpp:279-338: Q=K=I2, V=[[1,2],[3,4]], D=2, non-causal
    q = np.eye(2, dtype=np.float32).reshape(1, 1, 2, 2)
    v = np.array([[1, 2], [3, 4]], np.float32).reshape(1, 1, 2, 2)
    e = np.exp(1 / np.sqrt(2))
    ph, pl = e / (1 + e), 1 / (1 + e)
    want = np.array([ph + 3 * pl, 2 * ph + 4 * pl, pl + 3 * ph, 2 * pl + 4 * ph])
    for out in (O.sdpa(q, q, v, False), O.flash_attention(q, q, v, float(np.float32(1 / np.sqrt(2))), False)):
        assert np.abs(out.reshape(-1) - want).max() < 1e-4


def test_causal_mask_structure():
    # tests/test_attention_chapter32.cpp:168-203: Q=K=1, V[i]=[i,0,0,0], S=4, causal -> 0, .5, 1, 1.5
    q = np.ones((1, 1, 4, 4), np.float32)
    v = np.zeros((1, 1, 4, 4), np.float32)
    v[0, 0, :, 0] = np.arange(4)
    for out in (O.sdpa(q, q, v, True), O.flash_attention(q, q, v, 0.5, True)):
        assert np.abs(out[0, 0, :, 0] - [0, 0.5, 1.0, 1.5]).max() < 1e-5


def test_constant_v_returns_v():
    # tests/test_attention_chapter32.cpp:209-239
    q, k, _ = I.qkv(13, 2, 2, 2, 9, 9, 8)
    v = np.full((2, 2, 9, 8), 3.25, np.float32)
    for causal in (False, True):
        assert np.abs(O.sdpa(q, k, v, causal) - 3.25).max() < 1e-5
        assert np.abs(O.flash_attention(q, k, v, 0.3, causal) - 3.25).max() < 1e-5


def test_single_token_returns_v():
    # tests/test_attention_comprehensive.cpp:112-135
    q, k, v = I.qkv(14, 2, 3, 3, 1, 1, 16)
    assert np.array_equal(O.sdpa(q, k, v, False), v)
    assert np.array_equal(O.flash_attention(q, k, v, 0.25, True), v)


def test_uniform_attention():
    # tests/test_attention_comprehensive.cpp:234-266: Q=K=1, V=I4 -> every output 0.25
    q = np.ones((1, 1, 4, 4), np.float32)
    v = np.eye(4, dtype=np.float32).reshape(1, 1, 4, 4)
    assert np.abs(O.sdpa(q, q, v, False) - 0.25).max() < 1e-6


def test_causal_first_and_last_token():
    # tests/test_attention_comprehensive.cpp:272-357: uniform scores, V[i] = i+1 -> first row 1, last row 2.5
    q = np.ones((1, 1, 4, 2), np.float32)
    v = np.repeat(np.arange(1, 5, dtype=np.float32)[:, None], 2, 1).reshape(1, 1, 4, 2)
    out = O.sdpa(q, q, v, True)
    assert abs(out[0, 0, 0, 0] - 1.0) < 1e-6 and abs(out[0, 0, 3, 0] - 2.5) < 1e-6


def test_causality_future_key_does_not_matter():
    # tests/test_attention.cpp:44-103
    q, k, v = I.qkv(15, 1, 2, 2, 12, 12, 8)
    a = O.flash_attention(q, k, v, 0.35, True)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, -1] += 5.0
    v2[:, :, -1] -= 3.0
    b = O.flash_attention(q, k2, v2, 0.35, True)
    assert np.array_equal(a[:, :, :-1], b[:, :, :-1]) and not np.array_equal(a[:, :, -1], b[:, :, -1])


def test_repeat_kv_iota_head_map():
    # tests/test_gqa_chapter33.cpp:76-118: q heads 0-3 <- kv head 0, 4-7 <- kv head 1
    x = np.zeros((1, 2, 1, 2), np.float32)
    x[0, 0], x[0, 1] = [1, 2], [3, 4]
    r = O.repeat_kv(x, 4)
    assert r.shape == (1, 8, 1, 2)
    assert all(np.array_equal(r[0, h, 0], [1, 2]) for h in range(4))
    assert all(np.array_equal(r[0, h, 0], [3, 4]) for h in range(4, 8))
    assert O.repeat_kv(x, 1) is x  # n_rep == 1 returns its input (src/ops/attention_ops.cpp:93-95)


def test_gqa_fused_equals_repeat_then_mha_bitwise():
    for (B, Hq, Hkv, T, L, D, causal) in [(2, 8, 2, 6, 6, 16, True), (1, 4, 1, 1, 37, 32, False), (1, 6, 3, 9, 9, 8, False)]:
        q, k, v = I.qkv(16, B, Hq, Hkv, T, L, D)
        n = Hq // Hkv
        assert np.array_equal(O.gqa_attention(q, k, v, causal), O.sdpa(q, O.repeat_kv(k, n), O.repeat_kv(v, n), causal))


def test_decode_equals_last_row_of_causal_prefill():
    # the equivalence tests/test_kv_cache_chapter33.cpp:66-188 checks at module level
    q, k, v = I.qkv(17, 1, 4, 2, 20, 20, 16)
    full = O.gqa_attention(q, k, v, True)
    last = O.gqa_attention(q[:, :, -1:], k, v, False)
    assert np.abs(full[:, :, -1:] - last).max() < 1e-6


def test_batch_and_head_permutation():
    q, k, v = I.qkv(18, 3, 4, 4, 10, 10, 8)
    a = O.flash_attention(q, k, v, 0.3, True)
    pb, ph = [2, 0, 1], [3, 1, 0, 2]
    b = O.flash_attention(q[pb][:, ph], k[pb][:, ph], v[pb][:, ph], 0.3, True)
    assert np.array_equal(a[pb][:, ph], b)


# ---- KV cache --------------------------------------------------------------------------------

def test_kv_cache_basic_append_values():
    # tests/test_kv_cache.cpp:8-43: ones at pos 0-1, 3.0 at pos 2 -> k_out[2*D] == 3.0, lengths 2 -> 3
    B, H, S, D = 1, 1, 10, 4
    c = O.KVCache(B, H, S, D)
    k1, v1 = c.update(np.ones((B, H, 2, D), np.float32), np.ones((B, H, 2, D), np.float32), 0)
    assert c.current_seq_len() == 2 and k1.shape == (1, 1, 2, 4)
    k2, v2 = c.update(np.full((B, H, 1, D), 3.0, np.float32), np.full((B, H, 1, D), 3.0, np.float32), 2)
    assert c.current_seq_len() == 3 and k2.shape[2] == 3
    assert k2.reshape(-1)[2 * D] == 3.0 and v2[0, 0, 2, 0] == 3.0 and k2[0, 0, 1, 0] == 1.0
    assert c.get_max_seq_len() == 10


def test_kv_cache_state_bookkeeping():
    # tests/test_kv_cache_chapter33.cpp:194-236: prefill 10 + 5 decodes, reset -> 0
    c = O.KVCache(2, 2, 32, 4)
    c.update(I.normal(1, (2, 2, 10, 4)), I.normal(2, (2, 2, 10, 4)), 0)
    assert c.current_seq_len() == 10
    for i in range(5):
        c.update(I.normal(3 + i, (2, 2, 1, 4)), I.normal(9 + i, (2, 2, 1, 4)), 10 + i)
        assert c.current_seq_len() == 11 + i
    c.reset()
    assert c.current_seq_len() == 0 and not c.planes()[0].any()


def test_kv_cache_against_plain_array_model():
    rng = np.random.default_rng(3)
    B, H, S, D = 2, 3, 20, 4
    c = O.KVCache(B, H, S, D)
    mk, mv, mlen = np.zeros((B, H, S, D), np.float32), np.zeros((B, H, S, D), np.float32), 0
    for step in range(40):
        T, pos = int(rng.integers(1, 5)), int(rng.integers(0, S))
        nk, nv = I.normal(step, (B, H, T, D)), I.normal(99 + step, (B, H, T, D))
        if pos + T > S:
            with pytest.raises(O.OracleError):
                c.update(nk, nv, pos)
            continue
        mk[:, :, pos:pos + T], mv[:, :, pos:pos + T] = nk, nv
        mlen = max(mlen, pos + T)
        kview, vview = c.update(nk, nv, pos)
        assert c.current_seq_len() == mlen
        assert np.array_equal(kview, mk[:, :, :mlen]) and np.array_equal(vview, mv[:, :, :mlen])
        # flat offset ((b*H+h)*S_max+s)*D+d
        flat = c.planes()[0].reshape(-1)
        b, h, s, d = 1, 2, pos, 3
        assert flat[((b * H + h) * S + s) * D + d] == nk[b, h, 0, d]
        assert list(c.last_view_meta) == [B, H, mlen, D, H * S * D, S * D, D, 1, 0]


def test_slice_bounds_python_semantics():
    for dim in (0, 1, 7):
        for start in [None, -9, -1, 0, 3, 7, 12]:
            for stop in [None, -8, -1, 0, 4, 7, 15]:
                for step in [None, 1, 2, -1, -3]:
                    idx = range(dim)[slice(start, stop, step)]
                    s, n = O.slice_bounds(dim, start, stop, step)
                    # the reference deviates from Python only for negative-step corner cases with
                    # explicit negative stops; restrict the check to what KVCache uses (positive step).
                    if step is None or step > 0:
                        assert n == len(idx), (dim, start, stop, step)
                        if n:
                            assert s == idx[0]
    with pytest.raises(O.OracleError):
        O.slice_bounds(5, 0, 3, 0)
