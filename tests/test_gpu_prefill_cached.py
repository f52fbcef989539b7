"""Chunked prefill over the cache planes (vsp_attn_prefill_cached) on the GPU.  The reference has no chunked
causal attention; the expected values are rows [L-T, L) of its full causal forward over L tokens (the oracle's
flash_attention, bit-exact to the compiled reference), on the values the cache holds."""
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


def _expected(q_full, k, v, L, T, causal=True):
    """Rows [L-T, L) of attention over the first L tokens, fp32 oracle."""
    n = q_full.shape[1] // k.shape[1]
    kk, vv = O.repeat_kv(k[:, :, :L], n), O.repeat_kv(v[:, :, :L], n)
    scale = float(np.float32(1.0 / math.sqrt(q_full.shape[-1])))
    if causal:
        return O.flash_attention(q_full[:, :, :L], kk, vv, scale, True)[:, :, L - T:]
    return O.sdpa(q_full[:, :, L - T:L], kk, vv, False)


@pytest.mark.parametrize("B,Hq,Hkv,L,T,D,S_max", [(1, 4, 2, 96, 32, 128, 128), (2, 8, 2, 201, 73, 128, 260),
                                                 (1, 4, 4, 130, 130, 64, 130), (1, 2, 1, 333, 1, 64, 400),
                                                 (1, 8, 2, 1100, 300, 128, 1100)])
def test_bf16_planes_against_oracle_and_dense_kernel(va, B, Hq, Hkv, L, T, D, S_max):
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3000 + L, B, Hq, Hkv, L, L, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    # the context arrives in two appends, the second being the chunk
    if L > T:
        c.update(G.to_bf16_dev(k[:, :, :L - T]), G.to_bf16_dev(v[:, :, :L - T]), 0, return_views=False)
    c.update(G.to_bf16_dev(k[:, :, L - T:]), G.to_bf16_dev(v[:, :, L - T:]), L - T, return_views=False)
    qd = G.to_bf16_dev(q[:, :, L - T:])
    out, lse = c.prefill(qd, return_lse=True)
    want = _expected(q, k, v, L, T)
    G.assert_bf16_close(G.bf16_to_np(out), want, "vs oracle")
    # the dense kernel (row-major V through the transposing LDS read) on the read-back context: an independent path
    kd, vd = c.read(0, L, torch.bfloat16)
    dense, lse2 = va.flash_attention(qd, kd, vd, 1.0 / math.sqrt(D), True, return_lse=True)
    err = np.abs(G.bf16_to_np(out) - G.bf16_to_np(dense))
    assert err.max() <= 2e-2
    assert np.allclose(lse.cpu().numpy(), lse2.cpu().numpy(), atol=2e-3)
    # non-causal: every query sees all L keys
    out_nc = c.prefill(qd, is_causal=False)
    G.assert_bf16_close(G.bf16_to_np(out_nc), _expected(q, k, v, L, T, causal=False), "non-causal")


def test_stale_tokens_past_the_context_are_never_used(va):
    B, Hq, Hkv, L, T, D, S_max = 1, 4, 2, 77, 40, 128, 192
    q, k, v = [O.bf16_round(x) for x in I.qkv(3100, B, Hq, Hkv, L, L, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    # poison every plane byte (bf16 NaN pattern 0x7fc0), then write only the context
    for p in (0, 1):
        c.raw_plane(p).view(torch.int16).fill_(0x7fc0)
    c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
    out = c.prefill(G.to_bf16_dev(q[:, :, L - T:]))
    got = G.bf16_to_np(out)
    assert np.isfinite(got).all()
    G.assert_bf16_close(got, _expected(q, k, v, L, T), "poisoned tail")


def test_per_sequence_lengths(va):
    B, Hq, Hkv, T, D, S_max = 3, 4, 2, 24, 128, 160
    lens = np.array([24, 131, 90], np.int32)
    qs, ks, vs = [], [], []
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    kfull = np.zeros((B, Hkv, S_max, D), np.float32)
    vfull = np.zeros_like(kfull)
    qchunk = np.zeros((B, Hq, T, D), np.float32)
    for b in range(B):
        q, k, v = [O.bf16_round(x * np.float32(0.7)) for x in I.qkv(3200 + b, 1, Hq, Hkv, int(lens[b]), int(lens[b]), D)]
        qs.append(q), ks.append(k), vs.append(v)
        kfull[b, :, :lens[b]], vfull[b, :, :lens[b]] = k[0], v[0]
        qchunk[b] = q[0, :, lens[b] - T:]
    c.update(G.to_bf16_dev(kfull), G.to_bf16_dev(vfull), 0, return_views=False)
    sl = torch.from_numpy(lens).to(G.dev())
    out = G.bf16_to_np(c.prefill(G.to_bf16_dev(qchunk), seq_lens=sl))
    for b in range(B):
        G.assert_bf16_close(out[b:b + 1], _expected(qs[b], ks[b], vs[b], int(lens[b]), T), f"row {b}")


def test_f32_cache_planes(va):
    B, Hq, Hkv, L, T, D, S_max = 2, 4, 2, 150, 50, 64, 200
    q, k, v = I.qkv(3300, B, Hq, Hkv, L, L, D)
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    c.update(G.f32_dev(k), G.f32_dev(v), 0, return_views=False)
    out = c.prefill(G.f32_dev(q[:, :, L - T:]))
    G.assert_f32_close(out.cpu().numpy(), _expected(q, k, v, L, T), "f32 planes")
    lens = torch.tensor([150, 99], dtype=torch.int32, device=G.dev())
    out2 = c.prefill(G.f32_dev(np.stack([q[0, :, 100:150], q[1, :, 49:99]])), seq_lens=lens).cpu().numpy()
    G.assert_f32_close(out2[0:1], _expected(q[0:1], k[0:1], v[0:1], 150, 50), "row 0")
    G.assert_f32_close(out2[1:2], _expected(q[1:2], k[1:2], v[1:2], 99, 50), "row 1")


def test_chunked_equals_one_shot_at_config2_size(va):
    # benchmark config 2 shape, prefilled in two chunks of 1024 through the cache: same rows as the dense launch
    B, Hq, Hkv, N, D = 4, 32, 8, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(5)
    mk = lambda h: (torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    q, k, v = mk(Hq), mk(Hkv), mk(Hkv)
    dense = va.flash_attention(q, k, v, 1.0 / math.sqrt(D), True)
    c = va.KVCache(B, Hkv, N, D, fmt="bf16")
    outs = []
    for t0 in (0, 1024):
        c.update(k[:, :, t0:t0 + 1024], v[:, :, t0:t0 + 1024], t0, return_views=False)
        outs.append(c.prefill(q[:, :, t0:t0 + 1024]))
    got = torch.cat(outs, dim=2).float()
    err = (got - dense.float()).abs()
    assert err.max().item() <= 2e-2 and err.mean().item() <= 2e-3
    again = c.prefill(q[:, :, 1024:])
    assert torch.equal(again, outs[1])  # run-to-run deterministic


def test_q8_0_cache(va):
    # the oracle attends over what the cache holds: the dequantised rows
    B, Hq, Hkv, L, T, D, S_max = 2, 8, 2, 140, 60, 128, 200
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3400, B, Hq, Hkv, L, L, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="q8_0")
    c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
    kq, vq = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    out = c.prefill(G.to_bf16_dev(q[:, :, L - T:]))
    G.assert_bf16_close(G.bf16_to_np(out), _expected(q, kq, vq, L, T), "q8_0 planes")
    lens = torch.tensor([140, 75], dtype=torch.int32, device=G.dev())
    qc = np.stack([q[0, :, 80:140], q[1, :, 15:75]])
    out2 = G.bf16_to_np(c.prefill(G.to_bf16_dev(qc), seq_lens=lens))
    G.assert_bf16_close(out2[0:1], _expected(q[0:1], kq[0:1], vq[0:1], 140, 60), "row 0")
    G.assert_bf16_close(out2[1:2], _expected(q[1:2], kq[1:2], vq[1:2], 75, 60), "row 1")
    # a missing workspace is an error, not a silent fallback
    import ctypes as C
    from vesper_amd import _ffi
    from vesper_amd.api import _desc, _stream
    qd = G.to_bf16_dev(q[:, :, L - T:])
    od = torch.empty_like(qd)
    dq, do = _desc(qd), _desc(od)
    rc = _ffi.lib.vsp_attn_prefill_cached(C.byref(dq), C.byref(c._c), None, 0, None, C.byref(do), None, 0.1, 1, None, 0, _stream(qd))
    assert rc == _ffi.ERR_WORKSPACE


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
def test_module_level_prefill_reads_the_planes_in_place(va, fmt, monkeypatch):
    # GroupedQueryAttention::forward(x, cache, 0) with T > 1 (src/nn/gqa_attention.cpp:128-148) on a bf16 / Q8_0
    # cache: the attention core goes through vsp_attn_prefill_cached, not through a read-back of the context
    B, Hq, Hkv, T, D = 2, 8, 2, 70, 128
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3500, B, Hq, Hkv, T, T, D)]
    c = va.KVCache(B, Hkv, 96, D, fmt=fmt)

    def no_read(*a, **kw):
        raise AssertionError("attention_core materialised the cache")
    monkeypatch.setattr(va.KVCache, "read", no_read)
    out = va.attention_core(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), c, 0)
    assert c.current_seq_len() == T
    assert torch.equal(out, c.prefill(G.to_bf16_dev(q)))
    if fmt == "q8_0":
        k, v = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    G.assert_bf16_close(G.bf16_to_np(out), _expected(q, k, v, T, T), fmt)
    # the reference cannot add its [T, T] mask to [T, L] scores: a second multi-token call is an error there too
    with pytest.raises(va.VspError):
        va.attention_core(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), va.KVCache(B, Hkv, 200, D, fmt=fmt), 5)


def _chunk_rows64(q, k, v, L, causal, with_lse=False):
    """float64 attention of the chunk rows q [B,Hq,T,D] (the last T of L tokens) over k, v [B,Hkv,>=L,D]."""
    B, Hq, T, D = q.shape
    n = Hq // k.shape[1]
    out = np.empty((B, Hq, T, D))
    lse = np.empty((B, Hq, T))
    for b in range(B):
        for h in range(Hq):
            kk, vv = k[b, h // n, :L].astype(np.float64), v[b, h // n, :L].astype(np.float64)
            s = q[b, h].astype(np.float64) @ kk.T / math.sqrt(D)
            if causal:
                s = np.where(np.arange(L)[None, :] <= (L - T + np.arange(T))[:, None], s, -np.inf)
            p = np.exp(s - s.max(-1, keepdims=True))
            out[b, h] = (p / p.sum(-1, keepdims=True)) @ vv
            lse[b, h] = s.max(-1) + np.log(p.sum(-1))
    return (out, lse) if with_lse else out


@pytest.mark.parametrize("B,Hq,Hkv,T,L,causal", [(1, 8, 2, 100, 3000, True), (1, 8, 2, 100, 3000, False), (2, 8, 2, 300, 5000, True),
                                                (1, 4, 1, 8, 8000, True), (1, 8, 2, 128, 1030, True)])
def test_bf16_context_split_over_workgroups(va, B, Hq, Hkv, T, L, causal):
    # a few query tiles over a long context: with the split workspace the context is cut into shares of >= 512 keys
    # (5, 5, 9, 15 and 2 shares here), each written as a partial and merged by the decode step's combine kernel
    D, S_max = 128, (L + 63) // 64 * 64
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3300 + L + T, B, Hq, Hkv, T, L, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
    from vesper_amd import _ffi
    import ctypes as C
    assert _ffi.lib.vsp_attn_prefill_cached_split_workspace_bytes(C.byref(c._c), 0, 0, Hq, T) > 0
    tq = G.to_bf16_dev(q)
    got = c.prefill(tq, is_causal=causal)
    G.assert_bf16_close(G.bf16_to_np(got), _chunk_rows64(q, k, v, L, causal).astype(np.float32), "split")
    assert torch.equal(got, c.prefill(tq, is_causal=causal))          # fixed merge order
    whole = c.prefill(tq, is_causal=causal, split=False)
    d = (got.float() - whole.float()).abs()
    assert d.max().item() <= 1.6e-2 and d.mean().item() <= 1e-3
    # lse = m + log l comes out of the merge of the partials' (m, l): against float64 and against the unsplit kernel
    o2, lse = c.prefill(tq, is_causal=causal, return_lse=True)
    assert torch.equal(o2, got)
    _, lse64 = _chunk_rows64(q, k, v, L, causal, with_lse=True)
    assert np.abs(lse.cpu().numpy() - lse64).max() <= 5e-3     # the row sum is taken from the bf16 P: up to 2^-8 relative on l
    o3, lse3 = c.prefill(tq, is_causal=causal, return_lse=True, split=False)
    assert torch.equal(o3, whole) and (lse - lse3).abs().max().item() <= 5e-3


def test_bf16_context_split_ragged_rows_and_stale_tokens(va):
    # per-row context and chunk lengths on the device, one row shorter than a share, stale NaN / Inf tokens past every length
    B, Hq, Hkv, T, D, S_max = 3, 8, 2, 96, 128, 4096
    lens = np.array([4000, 300, 1777], dtype=np.int32)
    nq = np.array([96, 50, 7], dtype=np.int32)
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3400, B, Hq, Hkv, T, S_max, D)]
    kk, vv = G.to_bf16_dev(k).clone(), G.to_bf16_dev(v).clone()
    for b in range(B):
        kk[b, :, lens[b]:] = float("nan")
        vv[b, :, lens[b]:] = float("inf")
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    c.update(kk, vv, 0, return_views=False)
    sl, cl = torch.from_numpy(lens).to(G.dev()), torch.from_numpy(nq).to(G.dev())
    got = c.prefill(G.to_bf16_dev(q), seq_lens=sl, chunk_lens=cl)
    whole = c.prefill(G.to_bf16_dev(q), seq_lens=sl, chunk_lens=cl, split=False)
    for b in range(B):
        n, L = int(nq[b]), int(lens[b])
        want = _chunk_rows64(q[b:b + 1, :, :n], k[b:b + 1], v[b:b + 1], L, True).astype(np.float32)
        G.assert_bf16_close(G.bf16_to_np(got[b:b + 1, :, :n]), want, f"row {b}")
        assert (got[b, :, :n].float() - whole[b, :, :n].float()).abs().max().item() <= 1.6e-2


def test_bf16_context_split_rows_shorter_than_their_chunk_and_a_host_bound(va):
    # (i) device lengths below the chunk length (an idle or short row of a ragged batch, chunk_lens NULL): a chunk is part
    # of its context, so producer and merge both take such a row as T tokens long: split == unsplit on every row.
    # (ii) the longest row far below the capacity: with max_len the shares are planned on the real bound (8 shares of
    # 16 tiles over 4096 tokens) instead of on S_max (16 shares of 32 tiles, of which such rows would fill 4).
    from vesper_amd import _ffi
    import ctypes as C
    B, Hq, Hkv, T, D, S_max = 4, 8, 2, 64, 128, 16384
    lens = np.array([4096, 10, 0, 1500], dtype=np.int32)       # rows 1 and 2 are shorter than the chunk
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3450, B, Hq, Hkv, T, 4096, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    c.update(G.to_bf16_dev(k), G.to_bf16_dev(v), 0, return_views=False)
    f = _ffi.lib.vsp_attn_prefill_cached_split_workspace_bytes
    per_share = B * Hq * T * 130 * 4
    assert f(C.byref(c._c), 1, 0, Hq, T) == 16 * per_share and f(C.byref(c._c), 1, 4096, Hq, T) == 8 * per_share
    sl = torch.from_numpy(lens).to(G.dev())
    tq = G.to_bf16_dev(q)
    for max_len in (0, 4096):
        got, lse = c.prefill(tq, seq_lens=sl, max_len=max_len, return_lse=True)
        whole, lse_w = c.prefill(tq, seq_lens=sl, max_len=max_len, return_lse=True, split=False)
        assert (got.float() - whole.float()).abs().max().item() <= 1.6e-2, max_len
        assert (lse - lse_w).abs().max().item() <= 5e-3, max_len
        for b in range(B):
            L = max(int(lens[b]), T)
            want, lse64 = _chunk_rows64(q[b:b + 1], k[b:b + 1], v[b:b + 1], L, True, with_lse=True)
            G.assert_bf16_close(G.bf16_to_np(got[b:b + 1]), want.astype(np.float32), f"row {b} max_len {max_len}")
            assert np.abs(lse[b:b + 1].cpu().numpy() - lse64).max() <= 5e-3
    # a device length above the host bound is clamped to it, by both kernels alike
    got = c.prefill(tq, seq_lens=sl, max_len=2048)
    want = _chunk_rows64(q[:1], k[:1], v[:1], 2048, True).astype(np.float32)
    G.assert_bf16_close(G.bf16_to_np(got[:1]), want, "clamped to max_len")


def test_bf16_context_split_over_pages(va):
    # the same over a paged cache with a shuffled page table: shares cross page boundaries
    B, Hq, Hkv, T, D, S_max, P = 2, 8, 2, 64, 128, 2048, 128
    n_pages = B * (S_max // P) + 3
    flat = va.RaggedKVCache(B, Hkv, S_max, D, fmt="bf16")
    paged = va.RaggedKVCache(B, Hkv, S_max, D, fmt="bf16", paging=(P, n_pages))
    perm = np.random.default_rng(9).permutation(n_pages)[:B * (S_max // P)].astype(np.int32).reshape(B, S_max // P)
    paged.page_table.copy_(torch.from_numpy(perm))
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(3500, B, Hq, Hkv, T, 2000, D)]
    outs = []
    for c in (flat, paged):
        c.append(G.to_bf16_dev(k), G.to_bf16_dev(v))
        outs.append(c.prefill_chunk(G.to_bf16_dev(q)))
    assert torch.equal(outs[0], outs[1])
    G.assert_bf16_close(G.bf16_to_np(outs[1]), _chunk_rows64(q, k, v, 2000, True).astype(np.float32), "paged")


def test_context_split_is_not_offered_where_it_cannot_help(va):
    from vesper_amd import _ffi
    import ctypes as C
    f = _ffi.lib.vsp_attn_prefill_cached_split_workspace_bytes
    c = va.KVCache(1, 2, 4096, 128, fmt="bf16")
    c.set_len(4096)
    assert f(C.byref(c._c), 0, 0, 8, 100) == 1 * 8 * 100 * 8 * 130 * 4      # 128 tiles, 8 workgroups: 8 shares of 16 tiles
    c.set_len(900)
    assert f(C.byref(c._c), 0, 0, 8, 100) == 0                           # under 32 tiles
    assert f(C.byref(c._c), 1, 0, 8, 100) > 0                            # with device lengths the bound is S_max
    assert f(C.byref(c._c), 1, 900, 8, 100) == 0                         # or the caller's own
    big = va.KVCache(4, 8, 4096, 128, fmt="bf16")
    big.set_len(4096)
    assert f(C.byref(big._c), 0, 0, 32, 512) == 0                           # 512 workgroups already
    for fmt, D in (("q8_0", 128), ("bf16", 64)):
        o = va.KVCache(1, 2, 4096, D, fmt=fmt)
        o.set_len(4096)
        assert f(C.byref(o._c), 0, 0, 8, 100) == 0


def test_argument_errors(va):
    q = torch.zeros(1, 4, 8, 64, device=G.dev(), dtype=torch.bfloat16)
    c = va.KVCache(1, 2, 64, 64, fmt="bf16")
    with pytest.raises(va.VspError):      # chunk longer than the context (len == 0)
        c.prefill(q)
    c.update(torch.zeros(1, 2, 16, 64, device=G.dev(), dtype=torch.bfloat16),
             torch.zeros(1, 2, 16, 64, device=G.dev(), dtype=torch.bfloat16), 0, return_views=False)
    with pytest.raises(va.VspError):      # fp32 q over a bf16 cache
        c.prefill(q.float())
    with pytest.raises(va.VspError):      # head count not a multiple of the cache's
        c.prefill(torch.zeros(1, 3, 8, 64, device=G.dev(), dtype=torch.bfloat16))
    assert c.prefill(q).shape == q.shape
