"""vsp_attn_decode_multi on the GPU: the last T tokens of each sequence attending to the cache through the decode kernels
(tokens and the query heads of a kv head share the 16 matrix-instruction columns).  The reference throws for T > 1 at
start_pos > 0 (its [T,T] mask does not broadcast onto [T,L] scores, src/nn/functional.cpp:397-421); the expected values
are rows [L-T, L) of its full causal forward over L tokens (the oracle's flash_attention, bit-exact to the compiled
reference), on the values the cache holds — the same rows vsp_attn_prefill_cached returns."""
import math

import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I
import _oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def _expected_rows(q_full, k, v, L, T):
    """Rows [L-T, L) of causal attention over the first L tokens, fp32 oracle; q_full holds all L query rows."""
    n = q_full.shape[1] // k.shape[1]
    scale = float(np.float32(1.0 / math.sqrt(q_full.shape[-1])))
    return O.flash_attention(q_full[:, :, :L], O.repeat_kv(k[:, :, :L], n), O.repeat_kv(v[:, :, :L], n), scale, True)[:, :, L - T:]


# small batches get 256-token splits: L = 513 / 514 put the last one or two keys alone in a split that the earlier tokens
# of the call must not see at all; L = T is the whole context in one call; (Hq, Hkv, T) fill the 16 columns in three ways
@pytest.mark.parametrize("fmt", ["bf16", "q8_0", "f32"])
@pytest.mark.parametrize("B,Hq,Hkv,T,D,L,S", [(2, 8, 2, 4, 128, 513, 600), (1, 16, 2, 2, 128, 514, 640), (2, 4, 4, 16, 64, 300, 320),
                                              (1, 8, 2, 3, 64, 3, 64), (3, 6, 2, 5, 128, 1000, 1024), (1, 4, 1, 4, 128, 70, 128)])
def test_against_oracle_rows(va, fmt, B, Hq, Hkv, T, D, L, S):
    q, k, v = I.qkv(5000 + L + T, B, Hq, Hkv, L, L, D)
    if fmt != "f32":
        q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in (q, k, v)]
    cv = G.f32_dev if fmt == "f32" else G.to_bf16_dev
    c = va.KVCache(B, Hkv, S, D, fmt=fmt)
    c.update(cv(k), cv(v), 0, return_views=False)
    kc, vc = k, v
    if fmt == "q8_0":
        kc, vc = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    want = _expected_rows(q, kc, vc, L, T)
    out = va.decode_attention_multi(cv(q[:, :, L - T:]), c)
    if fmt == "f32":
        G.assert_f32_close(out.cpu().numpy(), want, "rows")
    else:
        G.assert_bf16_close(G.bf16_to_np(out), want, "rows")
    assert torch.equal(out, va.decode_attention_multi(cv(q[:, :, L - T:]), c))   # fixed split order
    if fmt != "f32" or D in (64, 128):
        # the same rows through the chunked prefill over the planes (a different kernel family)
        ref = c.prefill(cv(q[:, :, L - T:]))
        tol = 1e-4 if fmt == "f32" else 2e-2
        assert (ref.float() - out.float()).abs().max().item() <= tol * max(1.0, float(np.abs(want).max()))


def test_one_token_is_the_decode_step_bit_for_bit(va):
    B, Hq, Hkv, D, L = 3, 8, 2, 128, 777
    q, k, v = [O.bf16_round(x) for x in I.qkv(5100, B, Hq, Hkv, 1, L, D)]
    for fmt in ("bf16", "q8_0"):
        c = va.KVCache(B, Hkv, 1024, D, fmt=fmt)
        c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
        tq = G.to_bf16_dev(q)
        assert torch.equal(va.decode_attention_multi(tq, c), va.decode_attention(tq, c))


def test_ragged_lengths_and_strided_queries(va):
    # per-row lengths on the device; q is a [B, T, Hq, D] buffer viewed as [B, Hq, T, D], as a fused projection hands it over
    B, Hq, Hkv, T, D, S = 4, 8, 2, 4, 128, 2048
    lens = np.array([2048, 4, 1300, 517], dtype=np.int32)
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(5200, B, Hq, Hkv, S, S, D)]
    c = va.KVCache(B, Hkv, S, D, fmt="bf16")
    c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
    sl = torch.from_numpy(lens).to(G.dev())
    qs = np.stack([q[b, :, lens[b] - T:lens[b]] for b in range(B)])          # [B, Hq, T, D]
    tq = G.to_bf16_dev(qs).transpose(1, 2).contiguous().transpose(1, 2)
    assert not tq.is_contiguous()
    out = va.decode_attention_multi(tq, c, seq_lens=sl)
    for b in range(B):
        L = int(lens[b])
        want = _expected_rows(q[b:b + 1], k[b:b + 1], v[b:b + 1], L, T)
        G.assert_bf16_close(G.bf16_to_np(out[b:b + 1]), want, f"row {b} (L={L})")
    # stale rows past a length never reach a result
    kk, vv = G.to_bf16_dev(k).clone(), G.to_bf16_dev(v).clone()
    for b in range(B):
        kk[b, :, lens[b]:] = float("nan")
        vv[b, :, lens[b]:] = float("inf")
    poisoned = va.KVCache(B, Hkv, S, D, fmt="bf16")
    poisoned.update(kk, vv, 0, return_views=False)
    assert torch.equal(out, va.decode_attention_multi(tq, poisoned, seq_lens=sl))


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
def test_small_chunks_of_a_continuous_batch_over_pages(va, fmt):
    # RaggedKVCache.prefill_chunk sends a full chunk of a few tokens through the decode kernels; over a paged cache
    # (shuffled page table, chunks that cross pages) the results are those of the contiguous cache, bit for bit
    B, Hq, Hkv, D, S_max, P, T = 3, 8, 2, 128, 640, 128, 4
    n_pages = B * (S_max // P) + 2
    flat = va.RaggedKVCache(B, Hkv, S_max, D, fmt=fmt)
    paged = va.RaggedKVCache(B, Hkv, S_max, D, fmt=fmt, paging=(P, n_pages))
    perm = np.random.default_rng(5).permutation(n_pages)[:B * (S_max // P)].astype(np.int32).reshape(B, S_max // P)
    paged.page_table.copy_(torch.from_numpy(perm))
    lens = [386, 130, 259]          # each chunk of 4 straddles a page boundary or a 256-token split
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(5300, B, Hq, Hkv, 400, 400, D)]
    n0 = torch.tensor([l - T for l in lens], dtype=torch.int32, device=G.dev())
    outs = []
    for c in (flat, paged):
        c.append(G.to_bf16_dev(k[:, :, :390]), G.to_bf16_dev(v[:, :, :390]), n_new=n0)
        ck = np.stack([k[b, :, lens[b] - T:lens[b]] for b in range(B)])
        cvv = np.stack([v[b, :, lens[b] - T:lens[b]] for b in range(B)])
        c.append(G.to_bf16_dev(ck), G.to_bf16_dev(cvv))
        cq = np.stack([q[b, :, lens[b] - T:lens[b]] for b in range(B)])
        outs.append(c.prefill_chunk(G.to_bf16_dev(cq)))
    assert paged.seq_lens.cpu().tolist() == lens
    assert torch.equal(outs[0], outs[1])
    kk, vv = (k, v) if fmt == "bf16" else (O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v)))
    for b in range(B):
        want = _expected_rows(q[b:b + 1], kk[b:b + 1], vv[b:b + 1], lens[b], T)
        G.assert_bf16_close(G.bf16_to_np(outs[1][b:b + 1]), want, f"row {b}")


def test_config4_shape_four_tokens(va):
    # benchmark config 4's shape (B32, 32/8 heads, D128, lengths U[1024, 32768]) with four tokens per sequence: sampled
    # sequences against the chunked prefill over the same planes
    B, Hq, Hkv, S, D, T = 32, 32, 8, 32768, 128, 4
    lens = I.seq_lens(4004, B, 1024, S)
    c = va.KVCache(B, Hkv, S, D, fmt="bf16")
    g = torch.Generator(device="cuda").manual_seed(31)
    c.update(torch.randn(B, Hkv, S, D, device=G.dev(), generator=g).to(torch.bfloat16),
             torch.randn(B, Hkv, S, D, device=G.dev(), generator=g).to(torch.bfloat16), 0, return_views=False)
    q = torch.randn(B, Hq, T, D, device=G.dev(), generator=g).to(torch.bfloat16)
    sl = torch.from_numpy(lens).to(G.dev())
    out = va.decode_attention_multi(q, c, seq_lens=sl)
    assert torch.isfinite(out.float()).all()
    ref = c.prefill(q, seq_lens=sl)
    assert (ref.float() - out.float()).abs().max().item() <= 1e-2


def test_argument_errors(va):
    from vesper_amd import _ffi
    d = G.dev()

    def code(fn):
        with pytest.raises(va.VspError) as e:
            fn()
        return e.value.status

    c = va.KVCache(1, 2, 64, 128, fmt="bf16")
    c.set_len(32)
    z = lambda hq, t, dd=128: torch.zeros(1, hq, t, dd, device=d, dtype=torch.bfloat16)
    assert code(lambda: va.decode_attention_multi(z(8, 5), c)) == _ffi.ERR_UNSUPPORTED      # 4 heads per kv head x 5 tokens > 16
    assert code(lambda: va.decode_attention(z(8, 2), c)) == _ffi.ERR_SHAPE                  # the plain step takes one token
    assert code(lambda: va.decode_attention_multi(z(3, 2), c)) == _ffi.ERR_GQA_HEADS
    c32 = va.KVCache(1, 2, 64, 32, fmt="f32")
    c32.set_len(8)
    assert code(lambda: va.decode_attention_multi(torch.zeros(1, 4, 2, 32, device=d), c32)) == _ffi.ERR_UNSUPPORTED
    out = va.decode_attention_multi(z(8, 4), c)
    assert out.shape == (1, 8, 4, 128) and not out.any()
