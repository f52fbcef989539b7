"""The oracle reproduces, bit for bit, the fixtures written from the real reference
(tests/golden/make_golden.py).  These run everywhere: the fixtures travel, the reference does not."""
import os

import numpy as np
import pytest

import _inputs as I
import _oracle as O

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(G, name + ".npz"), allow_pickle=False)


def check_inputs(rec, *arrays):
    want = bytes(rec).hex()
    got = "".join(I.sha(a) for a in arrays)
    assert got == want, "seeded input stream differs from the one the fixture was written with"


def test_flash_attention_fixtures():
    z = load("flash_attention")
    tags = sorted({k.rsplit("_", 1)[0] for k in z.files})
    assert len(tags) == 12
    for tag in tags:
        B, H, N, D, causal, seed = z[tag + "_meta"]
        q, k, v = I.qkv(int(seed), B, H, H, N, N, D)
        check_inputs(z[tag + "_insha"], q, k, v)
        out, lse = O.flash_attention(q, k, v, float(z[tag + "_scale"][0]), bool(causal), return_lse=True)
        assert np.array_equal(out, z[tag + "_out"]), tag
        assert np.array_equal(lse, z[tag + "_lse"]), tag


def test_config1_fixture():
    z = load("config1")
    B, Hq, Hkv, N, D, seed = z["meta"]
    q, k, v = I.qkv(int(seed), B, Hq, Hkv, N, N, D)
    check_inputs(z["insha"], q, k, v)
    n_rep = Hq // Hkv
    out, lse = O.flash_attention(q, O.repeat_kv(k, n_rep), O.repeat_kv(v, n_rep), 0.125, True, return_lse=True)
    assert np.array_equal(out, z["out_flash"])
    assert np.array_equal(lse, z["lse"])
    # the same through scaled_dot_product_attention (N < 512: matmul branch), GQA folded in
    assert np.array_equal(O.gqa_attention(q, k, v, True), z["out_sdpa"])
    assert np.array_equal(O.sdpa(q, O.repeat_kv(k, n_rep), O.repeat_kv(v, n_rep), True), z["out_sdpa"])
    # the two reference branches agree to ~1e-6 on this config
    assert np.abs(z["out_flash"] - z["out_sdpa"]).max() < 5e-6


def test_sdpa_fixtures():
    z = load("sdpa")
    tags = sorted({k.split("_")[0] for k in z.files})
    assert len(tags) == 7
    for tag in tags:
        B, H, T, L, D, causal, seed = z[tag + "_meta"]
        q, k, v = I.qkv(int(seed), B, H, H, T, L, D)
        check_inputs(z[tag + "_insha"], q, k, v)
        assert np.array_equal(O.sdpa(q, k, v, bool(causal)), z[tag + "_out"]), tag


def test_repeat_kv_fixture():
    z = load("repeat_kv")
    assert np.array_equal(O.repeat_kv(z["x"], 2), z["out2"])
    assert np.array_equal(O.repeat_kv(z["x"], 4), z["out4"])


@pytest.mark.parametrize("gqa", [0, 1])
def test_kv_cache_fixture(gqa):
    z = load("kv_cache")
    B, H, S_max, D = z["shape"]
    c = O.KVCache(B, H, S_max, D)
    si = 0
    while f"g{gqa}_s{si}_op" in z.files:
        tag = f"g{gqa}_s{si}"
        T, pos = z[tag + "_op"]
        if T == -1:
            c.reset()
        else:
            nk = I.normal(5000 + si, (B, H, T, D))
            nv = I.normal(6000 + si, (B, H, T, D))
            if z[tag + "_err"][0]:
                with pytest.raises(O.OracleError) as e:
                    c.update(nk, nv, int(pos))
                assert str(e.value) == bytes(z[tag + "_msg"]).decode()
            else:
                kview, vview = c.update(nk, nv, int(pos))
                assert np.array_equal(kview, z[tag + "_k"]), tag
                assert np.array_equal(vview, z[tag + "_v"]), tag
                if not gqa:
                    assert np.array_equal(c.last_view_meta, z[tag + "_viewmeta"]), tag
        assert c.current_seq_len() == z[tag + "_len"][0], tag
        si += 1
    assert si == 15


def test_gqa_core_fixture():
    z = load("gqa_core")
    B, Hq, Hkv, D, S_max = z["meta"]
    c = O.KVCache(B, Hkv, S_max, D)
    for si in range(4):
        T, pos = z[f"s{si}_op"]
        q, nk, nv = I.qkv(7000 + 10 * si, B, Hq, Hkv, T, T, D)
        kview, vview = c.update(nk, nv, int(pos))          # strided views, consumed as they are
        out = O.gqa_attention(q, kview, vview, causal=(T > 1))
        assert np.array_equal(out, z[f"s{si}_out"]), si
    c2 = O.KVCache(1, 2, 12, 64)
    q, nk, nv = I.qkv(7100, 1, 8, 2, 12, 12, 64)
    kview, vview = c2.update(nk, nv, 0)
    assert np.array_equal(O.gqa_attention(q, kview, vview, True), z["full_out"])


def test_bf16_fixture():
    z = load("bf16")
    f = z["bits"].view(np.float32)
    assert np.array_equal(O.f32_to_bf16(f), z["bf16"])
