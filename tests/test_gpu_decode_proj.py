"""Decode step with the attention module's output projection behind it (vsp_attn_decode_proj) against the oracle:
the reference's chain for T == 1 -- SDPA over the cache, heads merged by transpose(1,2).reshape({B,T,C}), then
wo_ / out_proj (src/nn/gqa_attention.cpp:140-152, src/nn/transformer.cpp:200-215, Linear::forward src/nn/linear.cpp:41-49)."""
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


def merged(o):
    """[B,Hq,1,D] -> [B,1,Hq*D]: transpose(1,2).reshape of the reference."""
    B, Hq, T, D = o.shape
    return np.ascontiguousarray(o.transpose(0, 2, 1, 3)).reshape(B, T, Hq * D)


def weights(seed, N, K, bias):
    w = O.bf16_round(I.normal(seed, (N, K), scale=1.0 / np.sqrt(K)))
    b = O.bf16_round(I.normal(seed + 1, (N,), scale=0.5)) if bias else None
    return w, b


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
@pytest.mark.parametrize("B,Hq,Hkv,S,D,N,lens,bias", [
    (2, 8, 2, 300, 128, 1024, [300, 77], True),        # the module's shape: N == Hq * D
    (1, 4, 4, 130, 64, 256, [129], False),             # one batch row
    (17, 4, 2, 96, 64, 40, None, True),                # two row tiles, N not a multiple of 16
    (40, 2, 1, 70, 128, 272, None, True),              # three row tiles through the four-tile kernel
    (70, 2, 2, 64, 64, 128, None, False),              # more rows than one pass holds
    (3, 6, 6, 70, 128, 768, [0, 70, 33], True)])       # an empty row projects zeros: y == bias
def test_bf16_decode_proj_against_oracle(va, fmt, B, Hq, Hkv, S, D, N, lens, bias):
    q, k, v = I.qkv(61, B, Hq, Hkv, 1, S, D)
    q = O.bf16_round(q)
    if fmt == "bf16":
        k, v = O.bf16_round(k), O.bf16_round(v)
        kd, vd = k, v
    else:
        kd, vd = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    if lens is None:
        lens = [1 + (7 * b * b + 11) % S for b in range(B)]
    c = fill_cache(va, fmt, k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    w, b = weights(62, N, Hq * D, bias)
    dq, dw = G.to_bf16_dev(q), G.to_bf16_dev(w)
    db = G.to_bf16_dev(b) if bias else None
    y = va.decode_attention_proj(dq, c, dw, db, seq_lens=sl)
    assert y.shape == (B, 1, N) and y.dtype == torch.bfloat16
    got = G.bf16_to_np(y)
    # end to end against the oracle's chain, at the attention tolerance (y is of the attention output's magnitude)
    want = O.linear(merged(O.bf16_round(oracle_decode(q, kd, vd, lens))), w, b)
    G.assert_bf16_close(got, want, f"decode + projection, {fmt}, lens={lens[:4]}")
    # the projection alone, over the very activations the attention step produced (vsp_attn_decode's output,
    # which the fused call leaves in its workspace bit for bit): only the order of the fp32 sums and the final
    # rounding to bf16 separate it from the oracle
    x = G.bf16_to_np(va.decode_attention(dq, c, seq_lens=sl))
    ref = O.linear(merged(x), w, b)
    assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0**-8 + 2e-5), float(np.abs(got - ref).max())
    for e, L in enumerate(lens):
        if L == 0:
            assert np.array_equal(got[e, 0], b if bias else np.zeros(N, np.float32))
    # deterministic run to run
    assert torch.equal(y, va.decode_attention_proj(dq, c, dw, db, seq_lens=sl))


@pytest.mark.parametrize("B,Hq,Hkv,S,D,N,lens,bias", [
    (2, 8, 2, 300, 64, 512, [300, 41], True), (9, 2, 1, 40, 32, 70, None, False), (1, 4, 4, 1200, 128, 33, [1111], True)])
def test_f32_decode_proj_against_oracle(va, B, Hq, Hkv, S, D, N, lens, bias):
    q, k, v = I.qkv(63, B, Hq, Hkv, 1, S, D)
    if lens is None:
        lens = [1 + (5 * b + 3) % S for b in range(B)]
    c = fill_cache(va, "f32", k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    w = I.normal(64, (N, Hq * D), scale=1.0 / np.sqrt(Hq * D))
    b = I.normal(65, (N,), scale=0.5) if bias else None
    y = va.decode_attention_proj(G.f32_dev(q), c, G.f32_dev(w), G.f32_dev(b) if bias else None, seq_lens=sl)
    want = O.linear(merged(oracle_decode(q, k, v, lens)), w, b)
    G.assert_f32_close(y.cpu().numpy(), want, "f32 decode + projection")


def test_single_length_cache_and_reference_module_shape(va):
    # GroupedQueryAttention(embed_dim 512, 8 heads, 2 kv heads) at T == 1 over a cache of 200 tokens: wo_ is [C, C], no bias
    # (src/nn/gqa_attention.cpp:71: Linear(embed_dim, embed_dim, false))
    B, Hq, Hkv, S, D = 2, 8, 2, 200, 64
    q, k, v = [O.bf16_round(x) for x in I.qkv(66, B, Hq, Hkv, 1, S, D)]
    c = fill_cache(va, "bf16", k, v)
    w, _ = weights(67, Hq * D, Hq * D, False)
    y = va.decode_attention_proj(G.to_bf16_dev(q), c, G.to_bf16_dev(w))
    want = O.linear(merged(O.bf16_round(oracle_decode(q, k, v, [S, S]))), w)
    G.assert_bf16_close(G.bf16_to_np(y), want, "module shape")


def test_argument_errors(va):
    from vesper_amd import _ffi
    B, Hq, Hkv, S, D, N = 2, 4, 2, 64, 64, 64
    q, k, v = [O.bf16_round(x) for x in I.qkv(68, B, Hq, Hkv, 1, S, D)]
    c = fill_cache(va, "bf16", k, v)
    dq = G.to_bf16_dev(q)
    w = torch.zeros(N, Hq * D, dtype=torch.bfloat16, device=G.dev())

    def code(**kw):
        args = dict(q=dq, cache=c, wo=w)
        args.update(kw)
        with pytest.raises(va.VspError) as e:
            va.decode_attention_proj(**args)
        return e.value.status

    assert code(wo=w[:, :-8]) == _ffi.ERR_SHAPE                       # K != Hq * D
    assert code(wo=w.float()) == _ffi.ERR_DTYPE
    assert code(bias=torch.zeros(N + 1, dtype=torch.bfloat16, device=G.dev())) == _ffi.ERR_SHAPE
    assert code(bias=torch.zeros(N, dtype=torch.float32, device=G.dev())) == _ffi.ERR_DTYPE
    assert code(out=torch.zeros(B, 1, N + 16, dtype=torch.bfloat16, device=G.dev())) == _ffi.ERR_SHAPE
    assert code(wo=w.t().contiguous().t()) == _ffi.ERR_STRIDE          # column-major weight
    wide = torch.zeros(N, Hq * D + 4, dtype=torch.bfloat16, device=G.dev())
    assert code(wo=wide[:, :Hq * D]) == _ffi.ERR_ALIGN                # row pitch not a multiple of 16 bytes
    assert code(workspace=torch.zeros(256, dtype=torch.uint8, device=G.dev())) == _ffi.ERR_WORKSPACE


def test_config4_shape_against_an_independent_gemm_and_linearity(va):
    # config 4's heads and width (32 / 8 heads, D 128, C 4096, B 32) over a shorter context: the projection of the very
    # activations vsp_attn_decode produced, against torch's fp32 matmul, and linearity in the weight
    B, Hq, Hkv, S, D = 32, 32, 8, 1024, 128
    C_ = Hq * D
    g = torch.Generator(device="cuda").manual_seed(71)
    dev = G.dev()
    cache = va.KVCache(B, Hkv, S, D, fmt="bf16")
    cache.update(torch.randn(B, Hkv, S, D, device=dev, generator=g).to(torch.bfloat16),
                 torch.randn(B, Hkv, S, D, device=dev, generator=g).to(torch.bfloat16), 0, return_views=False)
    lens = torch.randint(1, S + 1, (B,), device=dev, generator=g, dtype=torch.int32)
    q = torch.randn(B, Hq, 1, D, device=dev, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(C_, C_, device=dev, generator=g) / 64).to(torch.bfloat16)
    w2 = (torch.randn(C_, C_, device=dev, generator=g) / 64).to(torch.bfloat16)
    x = va.decode_attention(q, cache, seq_lens=lens).transpose(1, 2).reshape(B, 1, C_).float()
    y1 = va.decode_attention_proj(q, cache, w1, seq_lens=lens).float()
    y2 = va.decode_attention_proj(q, cache, w2, seq_lens=lens).float()
    ref1 = x @ w1.float().t()
    err = (y1 - ref1).abs()
    assert float(err.max()) <= 2.0**-8 * float(ref1.abs().max()) + 1e-3, float(err.max())
    # w1 + w2 is not a bf16 tensor in general, so compare in fp32: y(w1) + y(w2) against x (w1 + w2)^T
    ref12 = x @ (w1.float() + w2.float()).t()
    assert float((y1 + y2 - ref12).abs().max()) <= 2.0**-7 * float(ref12.abs().max()) + 2e-3
    assert torch.equal(va.decode_attention_proj(q, cache, w1, seq_lens=lens).float(), y1)  # bitwise run to run
