"""Seeded sweep over random shapes through the C ABI against the oracle: prefill (fp32, bf16), decode over the three
cache formats with ragged lengths, and the backward (fp32, bf16).  The parametrised tests elsewhere pick the shapes
that the kernels' tilings make interesting; this file draws them blindly (tile-unaligned lengths, odd head groupings,
lengths of 1) so that an indexing mistake that those miss still has a chance to show."""
import math

import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I
import _oracle as O
from test_gpu_decode import fill_cache, oracle_decode

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def draw(seed, n_max):
    r = np.random.default_rng(seed)
    Hkv = int(r.choice([1, 2, 3, 4]))
    n_rep = int(r.choice([1, 2, 4, 8]))
    return dict(B=int(r.integers(1, 4)), Hq=Hkv * n_rep, Hkv=Hkv, n_rep=n_rep, N=int(r.integers(1, n_max + 1)),
                D=int(r.choice([64, 128])), causal=bool(r.integers(0, 2)))


@pytest.mark.parametrize("seed", range(12))
def test_prefill_random_shapes(va, seed):
    c = draw(1000 + seed, 300)
    B, Hq, Hkv, N, D, causal = c["B"], c["Hq"], c["Hkv"], c["N"], c["D"], c["causal"]
    q, k, v = [O.bf16_round(x) for x in I.qkv(2000 + seed, B, Hq, Hkv, N, N, D)]
    scale = float(np.float32(1.0 / math.sqrt(D)))
    want, want_lse = O.flash_attention(q, O.repeat_kv(k, c["n_rep"]), O.repeat_kv(v, c["n_rep"]), scale, causal, return_lse=True)
    out, lse = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), scale, causal, return_lse=True)
    G.assert_f32_close(out.cpu().numpy(), want, f"f32 {c}")
    G.assert_f32_close(lse.cpu().numpy(), want_lse, f"f32 lse {c}")
    out, lse = va.flash_attention(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), scale, causal, return_lse=True)
    G.assert_bf16_close(G.bf16_to_np(out), want, f"bf16 {c}")
    assert np.abs(lse.cpu().numpy() - want_lse).max() <= 2e-2, c


@pytest.mark.parametrize("seed", range(12))
def test_decode_random_shapes(va, seed):
    c = draw(3000 + seed, 700)
    B, Hq, Hkv, S, D = c["B"], c["Hq"], c["Hkv"], c["N"], c["D"]
    r = np.random.default_rng(3500 + seed)
    lens = [int(x) for x in r.integers(0, S + 1, size=B)]
    lens[int(r.integers(0, B))] = S
    q, k, v = I.qkv(4000 + seed, B, Hq, Hkv, 1, S, D)
    q, kb, vb = O.bf16_round(q), O.bf16_round(k), O.bf16_round(v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    out = va.decode_attention(G.to_bf16_dev(q), fill_cache(va, "bf16", kb, vb), seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kb, vb, lens), f"bf16 {c} {lens}")
    kd, vd = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    out = va.decode_attention(G.to_bf16_dev(q), fill_cache(va, "q8_0", k, v), seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kd, vd, lens), f"q8_0 {c} {lens}")
    out = va.decode_attention(G.f32_dev(q), fill_cache(va, "f32", k, v), seq_lens=sl)
    G.assert_f32_close(out.cpu().numpy(), oracle_decode(q, k, v, lens), f"f32 {c} {lens}")


@pytest.mark.parametrize("seed", range(8))
def test_decode_random_shapes_with_many_query_heads_per_kv_head(va, seed):
    # more than 16 query heads per kv head are served in column groups of 16 (bf16 / Q8_0 caches); 16 itself and the
    # counts around a group boundary are the interesting ones
    r = np.random.default_rng(7000 + seed)
    Hkv, n_rep = int(r.choice([1, 2, 3])), int(r.choice([15, 16, 17, 24, 31, 32, 33, 40]))
    B, S, D = int(r.integers(1, 4)), int(r.integers(1, 600)), int(r.choice([64, 128]))
    Hq = Hkv * n_rep
    lens = [int(x) for x in r.integers(0, S + 1, size=B)]
    lens[int(r.integers(0, B))] = S
    q, k, v = I.qkv(7500 + seed, B, Hq, Hkv, 1, S, D)
    q, kb, vb = O.bf16_round(q), O.bf16_round(k), O.bf16_round(v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    tag = f"B{B} Hq{Hq} Hkv{Hkv} S{S} D{D} {lens}"
    out = va.decode_attention(G.to_bf16_dev(q), fill_cache(va, "bf16", kb, vb), seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kb, vb, lens), "bf16 " + tag)
    kd, vd = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    out = va.decode_attention(G.to_bf16_dev(q), fill_cache(va, "q8_0", k, v), seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kd, vd, lens), "q8_0 " + tag)
    out = va.decode_attention(G.f32_dev(q), fill_cache(va, "f32", k, v), seq_lens=sl)
    G.assert_f32_close(out.cpu().numpy(), oracle_decode(q, k, v, lens), "f32 " + tag)


@pytest.mark.parametrize("seed", range(12))
def test_backward_random_shapes(va, seed):
    c = draw(5000 + seed, 200)
    B, Hq, Hkv, N, D, causal, n = c["B"], c["Hq"], c["Hkv"], c["N"], c["D"], c["causal"], c["n_rep"]
    q, k, v = [O.bf16_round(x) for x in I.qkv(6000 + seed, B, Hq, Hkv, N, N, D)]
    dout = O.bf16_round(I.normal(6500 + seed, (B, Hq, N, D)))
    scale = float(np.float32(1.0 / math.sqrt(D)))
    kr, vr = O.repeat_kv(k, n), O.repeat_kv(v, n)
    out, lse = O.flash_attention(q, kr, vr, scale, causal, return_lse=True)
    wq, wk, wv = O.flash_attention_backward(dout, q, kr, vr, out, lse, scale, causal)
    wk, wv = wk.reshape(B, Hkv, n, N, D).sum(2), wv.reshape(B, Hkv, n, N, D).sum(2)
    for bf16, fast in ((False, False), (True, False), (True, True)):   # fast: the workspace that keeps dS (bf16 only)
        cv = G.to_bf16_dev if bf16 else G.f32_dev
        tq, tk, tv, td = cv(q), cv(k), cv(v), cv(dout)
        o, l = va.flash_attention(tq, tk, tv, scale, causal, return_lse=True)
        got = va.flash_attention_backward(td, tq, tk, tv, o, l, scale, causal, workspace=va.backward_workspace(tq, fast=fast))
        for g, w, name in zip(got, (wq, wk, wv), ("dq", "dk", "dv")):
            if bf16:
                err = np.abs(G.bf16_to_np(g) - w)
                ref = max(1.0, float(np.abs(w).max()))
                assert err.max() <= 2e-2 * ref and err.mean() <= 2e-3 * ref, (name, c, fast, err.max(), ref)
            else:   # 1e-4 of the gradient's scale; a gradient that is exactly zero (N = 1: dS = P (dP - Di) with
                    # dP = Di up to rounding) has no scale of its own and gets 1e-5 absolute
                err = np.abs(g.cpu().numpy() - w)
                assert err.max() <= 1e-4 * max(float(np.abs(w).max()), 0.1), (name, c, err.max())
