"""Single-token decode over the KV cache on the GPU (vsp_kv_append + vsp_attn_decode) against the oracle:
per sequence, repeat_kv -> matmul/softmax/matmul branch of the reference's SDPA, over the values the cache holds."""
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


def oracle_decode(q, k, v, lens):
    """q [B,Hq,1,D]; k,v [B,Hkv,S,D] fp32 (values as the cache holds them); per-sequence lengths."""
    out = np.zeros_like(q)
    for b, L in enumerate(lens):
        if L > 0:
            out[b:b + 1] = O.gqa_attention(q[b:b + 1], k[b:b + 1, :, :L], v[b:b + 1, :, :L], causal=False)
    return out


def fill_cache(va, fmt, k, v):
    B, H, S, D = k.shape
    c = va.KVCache(B, H, S, D, fmt=fmt)
    c.update(G.f32_dev(k), G.f32_dev(v), 0, return_views=False)
    return c


@pytest.mark.parametrize("B,Hq,Hkv,S,D,lens", [
    (2, 8, 2, 300, 128, [300, 77]), (3, 4, 4, 130, 64, [1, 64, 129]), (1, 32, 8, 1500, 128, [1411]),
    (2, 16, 2, 640, 128, [640, 63]), (2, 6, 6, 70, 128, [0, 70]), (1, 16, 1, 257, 64, [257])])
def test_bf16_decode_against_oracle(va, B, Hq, Hkv, S, D, lens):
    q, k, v = I.qkv(41, B, Hq, Hkv, 1, S, D)
    q, k, v = O.bf16_round(q), O.bf16_round(k), O.bf16_round(v)
    c = fill_cache(va, "bf16", k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    out = va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, k, v, lens), f"lens={lens}")
    if len(set(lens)) == 1 and lens[0] == S:  # reference-style single length (cache.len == S here)
        out2 = va.decode_attention(G.to_bf16_dev(q), c)
        assert torch.equal(out, out2)
    # a tighter max_len bound changes the launch shape, not the result beyond rounding of the split order
    out3 = va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl, max_len=max(max(lens), 1))
    G.assert_bf16_close(G.bf16_to_np(out3), oracle_decode(q, k, v, lens), "max_len bound")


@pytest.mark.parametrize("B,Hq,Hkv,S,D,lens", [
    (2, 16, 2, 300, 128, [300, 45]), (1, 64, 8, 1100, 128, [1100]), (2, 4, 2, 200, 64, [17, 200]), (1, 8, 8, 64, 128, [64])])
def test_q8_0_decode_against_oracle_over_dequantised_cache(va, B, Hq, Hkv, S, D, lens):
    q, k, v = I.qkv(42, B, Hq, Hkv, 1, S, D)
    q = O.bf16_round(q)
    c = fill_cache(va, "q8_0", k, v)
    kd, vd = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    out = va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kd, vd, lens), f"q8_0 lens={lens}")


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
@pytest.mark.parametrize("B,Hq,Hkv,S,D,lens", [
    (2, 32, 1, 700, 128, [700, 129]),        # multi-query attention: 32 query heads on one kv head (two groups of 16)
    (1, 128, 2, 1300, 128, [1211]),          # 64 per kv head (four groups)
    (3, 40, 2, 300, 64, [300, 0, 65]),       # 20 per kv head: a full group and one of four heads
    (9, 17, 1, 130, 128, [130, 1, 64, 65, 2, 130, 99, 17, 33])])   # nine (item, kv head) pairs: the grid is padded to 16
def test_more_than_16_query_heads_per_kv_head(va, fmt, B, Hq, Hkv, S, D, lens):
    # ops::repeat_kv takes any n_rep (src/ops/attention_ops.cpp:92-155): beyond the 16 columns of the matrix
    # instructions the heads of a kv head are served in groups of 16, one workgroup per group
    q, k, v = I.qkv(48, B, Hq, Hkv, 1, S, D)
    q = O.bf16_round(q)
    if fmt == "bf16":
        k, v = O.bf16_round(k), O.bf16_round(v)
        kd, vd = k, v
    else:
        kd, vd = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    c = fill_cache(va, fmt, k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    out = va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl)
    G.assert_bf16_close(G.bf16_to_np(out), oracle_decode(q, kd, vd, lens), f"{fmt} lens={lens}")
    assert torch.equal(out, va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl))   # fixed merge order
    # the same heads 16 at a time through the one-group path give the same bits: a group is a pure partition of the work
    n = Hq // Hkv
    if n % 16 == 0:
        qd = G.to_bf16_dev(q).view(B, Hkv, n // 16, 16, 1, D)
        for gi in range(n // 16):
            part = va.decode_attention(qd[:, :, gi].reshape(B, Hkv * 16, 1, D).contiguous(), c, seq_lens=sl)
            assert torch.equal(part.view(B, Hkv, 16, 1, D), out.view(B, Hkv, n // 16, 16, 1, D)[:, :, gi])


# D 64 / 128 with up to 16 query heads per kv head run on the fp32 matrix instructions, everything else (D 32: the
# reference's own test shapes; 32 query heads on one kv head) on the plain-FMA kernel
@pytest.mark.parametrize("B,Hq,Hkv,S,D,lens", [
    (2, 8, 2, 300, 64, [300, 41]), (1, 4, 4, 1200, 128, [1111]), (1, 2, 1, 40, 32, [40]),
    (3, 16, 1, 2500, 128, [2500, 1, 1025]), (2, 6, 2, 777, 64, [0, 777]), (2, 12, 4, 130, 128, [31, 33]),
    (1, 32, 1, 200, 64, [200]), (4, 8, 8, 96, 128, [16, 17, 32, 96])])
def test_f32_decode_against_oracle(va, B, Hq, Hkv, S, D, lens):
    q, k, v = I.qkv(43, B, Hq, Hkv, 1, S, D)
    c = fill_cache(va, "f32", k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    out = va.decode_attention(G.f32_dev(q), c, seq_lens=sl)
    G.assert_f32_close(out.cpu().numpy(), oracle_decode(q, k, v, lens), "f32 decode")
    assert torch.equal(out, va.decode_attention(G.f32_dev(q), c, seq_lens=sl))  # fixed split order


@pytest.mark.parametrize("D", [64, 128])
def test_f32_decode_ignores_rows_past_the_length(va, D):
    # the fp32 planes are the reference's layout, unpadded: rows past a sequence's length may hold anything (here NaN
    # and infinities), and the last row of the last head is the end of the allocation
    B, Hq, Hkv, S = 2, 8, 2, 300
    lens = [173, 300]
    q, k, v = I.qkv(47, B, Hq, Hkv, 1, S, D)
    c = fill_cache(va, "f32", k, v)
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    a = va.decode_attention(G.f32_dev(q), c, seq_lens=sl)
    G.assert_f32_close(a.cpu().numpy(), oracle_decode(q, k, v, lens), "before poisoning")
    kp = c.raw_plane(0).view(torch.float32).view(B, Hkv, S, D)
    vp = c.raw_plane(1).view(torch.float32).view(B, Hkv, S, D)
    kp[0, :, lens[0]:] = float("nan")
    vp[0, :, lens[0]:] = float("inf")
    assert torch.equal(a, va.decode_attention(G.f32_dev(q), c, seq_lens=sl))


def test_decode_after_token_by_token_appends_matches_causal_prefill(va):
    # the equivalence the reference checks in tests/test_kv_cache_chapter33.cpp:66-188, at kernel level:
    # prefill T tokens through the cache, then decode token by token; each decode == last row of causal attention
    B, Hq, Hkv, D, T0, steps = 2, 8, 2, 128, 37, 6
    N = T0 + steps
    q, k, v = [O.bf16_round(x) for x in I.qkv(44, B, Hq, Hkv, N, N, D, scale=0.5)]
    full, _ = O.flash_attention(q, O.repeat_kv(k, 4), O.repeat_kv(v, 4), float(np.float32(1 / math.sqrt(D))), True, return_lse=True)
    c = va.KVCache(B, Hkv, 64, D, fmt="bf16")
    dq, dk, dv = G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v)
    out0 = va.attention_core(dq[:, :, :T0].contiguous(), dk[:, :, :T0].contiguous(), dv[:, :, :T0].contiguous(), c, 0)
    G.assert_bf16_close(G.bf16_to_np(out0), full[:, :, :T0], "prefill through the cache")
    for t in range(T0, N):
        o = va.attention_core(dq[:, :, t:t + 1].contiguous(), dk[:, :, t:t + 1].contiguous(), dv[:, :, t:t + 1].contiguous(), c, t)
        assert c.current_seq_len() == t + 1
        G.assert_bf16_close(G.bf16_to_np(o), full[:, :, t:t + 1], f"decode step {t}")


def test_gqa_core_fixture_from_reference(va):
    # tests/golden/gqa_core.npz: cache->update -> repeat_kv -> SDPA run by the real reference (fp32)
    import os
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gqa_core.npz"), allow_pickle=False)
    B, Hq, Hkv, D, S_max = [int(x) for x in z["meta"]]
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    for si in range(4):
        T, pos = [int(x) for x in z[f"s{si}_op"]]
        q, nk, nv = I.qkv(7000 + 10 * si, B, Hq, Hkv, T, T, D)
        out = va.attention_core(G.f32_dev(q), G.f32_dev(nk), G.f32_dev(nv), c, pos)
        G.assert_f32_close(out.cpu().numpy(), z[f"s{si}_out"], f"step {si}")


def test_decode_is_deterministic_and_ignores_stale_tail(va):
    B, Hq, Hkv, S, D = 2, 8, 2, 512, 128
    q, k, v = [O.bf16_round(x) for x in I.qkv(45, B, Hq, Hkv, 1, S, D)]
    c = fill_cache(va, "bf16", k, v)
    sl = torch.tensor([200, 333], dtype=torch.int32, device=G.dev())
    a = va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl)
    assert torch.equal(a, va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl))
    # poison everything beyond the valid lengths with NaN bit patterns: the result must not change
    kp = c.raw_plane(0).cpu().numpy().view(np.uint16).reshape(B, Hkv, S, D).copy()
    vp = c.raw_plane(1).cpu().numpy().view(np.uint16).reshape(B, Hkv, S // 8, D, 8).copy()
    vl = vp.transpose(0, 1, 2, 4, 3).reshape(B, Hkv, S, D).copy()  # logical [s][d] order of the blocked plane
    for b, L in enumerate([200, 333]):
        kp[b, :, L:] = 0x7FC0
        vl[b, :, L:] = 0x7FC0
    vp = vl.reshape(B, Hkv, S // 8, 8, D).transpose(0, 1, 2, 4, 3).copy()
    c.raw_plane(0).copy_(torch.from_numpy(kp.view(np.uint8).reshape(-1)).to(G.dev()))
    c.raw_plane(1).copy_(torch.from_numpy(vp.view(np.uint8).reshape(-1)).to(G.dev()))
    assert torch.equal(a, va.decode_attention(G.to_bf16_dev(q), c, seq_lens=sl))


def test_decode_config4_shape_properties(va):
    # benchmark config 4 at full size (B32, 32/8 heads, D128, S_max 32768, lengths U[1024, 32768]):
    # two sequences against the oracle, all of them against the prefill kernel's last row (an independent kernel).
    B, Hq, Hkv, S, D = 32, 32, 8, 32768, 128
    lens = I.seq_lens(4004, B, 1024, S)
    c = va.KVCache(B, Hkv, S, D, fmt="bf16")
    g = torch.Generator(device="cuda").manual_seed(11)
    kfull = torch.randn(B, Hkv, S, D, device=G.dev(), generator=g).to(torch.bfloat16)
    vfull = torch.randn(B, Hkv, S, D, device=G.dev(), generator=g).to(torch.bfloat16)
    q = torch.randn(B, Hq, 1, D, device=G.dev(), generator=g).to(torch.bfloat16)
    c.update(kfull, vfull, 0, return_views=False)
    sl = torch.from_numpy(lens).to(G.dev())
    out = va.decode_attention(q, c, seq_lens=sl)
    assert torch.isfinite(out.float()).all()
    scale = 1.0 / math.sqrt(D)
    for b in (int(np.argmin(lens)), 17):
        L = int(lens[b])
        want = O.gqa_attention(G.bf16_to_np(q[b:b + 1]), G.bf16_to_np(kfull[b:b + 1, :, :L]), G.bf16_to_np(vfull[b:b + 1, :, :L]), False)
        G.assert_bf16_close(G.bf16_to_np(out[b:b + 1]), want, f"config-4 sequence {b} (L={L})")
    for b in range(0, B, 5):
        L = int(lens[b])
        ref = va.flash_attention(q[b:b + 1], kfull[b:b + 1, :, :L], vfull[b:b + 1, :, :L], scale, False)
        assert (ref.float() - out[b:b + 1].float()).abs().max().item() <= 1e-2


def test_decode_config5_shape_properties(va):
    # benchmark config 5 at full size (B16, 64/8 heads, D128, Q8_0 cache, L = 65536)
    B, Hq, Hkv, S, D = 16, 64, 8, 65536, 128
    c = va.KVCache(B, Hkv, S, D, fmt="q8_0")
    g = torch.Generator(device="cuda").manual_seed(13)
    for t0 in range(0, S, 8192):  # fill through the append path in slices (bounded temporaries)
        kb = torch.randn(B, Hkv, 8192, D, device=G.dev(), generator=g).to(torch.bfloat16)
        vb = torch.randn(B, Hkv, 8192, D, device=G.dev(), generator=g).to(torch.bfloat16)
        c.update(kb, vb, t0, return_views=False)
        del kb, vb
    assert c.current_seq_len() == S
    q = torch.randn(B, Hq, 1, D, device=G.dev(), generator=g).to(torch.bfloat16)
    out = va.decode_attention(q, c)
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, va.decode_attention(q, c))  # fixed split order: run-to-run deterministic
    # two (sequence, kv head) slices against a float64 closed form over the dequantised rows the cache holds
    for b, kvh in ((0, 0), (11, 5)):
        import ctypes as C
        kq, vq = c.read(0, S, torch.float32)
        ks, vs = kq[b, kvh].cpu().numpy().astype(np.float64), vq[b, kvh].cpu().numpy().astype(np.float64)
        del kq, vq
        qs = G.bf16_to_np(q[b, kvh * 8:(kvh + 1) * 8, 0]).astype(np.float64)
        s = qs @ ks.T / math.sqrt(D)
        p = np.exp(s - s.max(axis=1, keepdims=True))
        want = (p / p.sum(axis=1, keepdims=True)) @ vs
        G.assert_bf16_close(G.bf16_to_np(out[b, kvh * 8:(kvh + 1) * 8, 0]), want.astype(np.float32), f"config-5 ({b},{kvh})")


def test_decode_argument_errors(va):
    c = va.KVCache(2, 2, 64, 128, fmt="bf16")
    q = torch.zeros(2, 4, 1, 128, dtype=torch.bfloat16, device=G.dev())
    with pytest.raises(va.VspError) as e:
        va.decode_attention(q[:, :3], c)  # 3 query heads over 2 kv heads
    assert e.value.status == 8
    with pytest.raises(va.VspError) as e:
        va.decode_attention(q.float(), c)
    assert e.value.status == 33
    with pytest.raises(va.VspError) as e:
        va.decode_attention(torch.zeros(2, 4, 2, 128, dtype=torch.bfloat16, device=G.dev()), c)
    assert e.value.status == 2
    out = va.decode_attention(q, c)  # empty cache: zeros, like an empty sum
    assert not out.float().any()


@pytest.mark.parametrize("fmt", ["bf16", "q8_0", "f32"])
def test_device_lengths_above_the_host_bound_are_clamped_inside_the_workspace(va, fmt):
    # max_len sizes the grid, the split count and the workspace; a device-side length above it must neither write
    # outside the partials' rows nor change another row's result: the row attends to its first max_len keys.
    B, Hq, Hkv, S, D, max_len = 2, 8, 2, 1024, 128 if fmt != "f32" else 64, 512
    lens = [300, 1024]  # the LAST row exceeds the bound: unclamped, its splits 2 and 3 would land past the buffer
    q, k, v = I.qkv(47, B, Hq, Hkv, 1, S, D)
    if fmt != "f32":
        q = O.bf16_round(q)
    c = fill_cache(va, fmt, k, v)
    if fmt == "bf16":
        kc, vc = O.bf16_round(k), O.bf16_round(v)
    elif fmt == "q8_0":
        kc, vc = O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v))
    else:
        kc, vc = k, v
    need = va._ffi.lib.vsp_attn_decode_workspace_bytes(B, Hq, D, max_len)
    assert need == B * Hq * (max_len // 256) * (D + 2) * 4  # 256-token splits here: the whole workspace is in use
    guard = 1 << 20
    ws = torch.full((need + guard,), 0x5A, dtype=torch.uint8, device=G.dev())
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    qd = G.f32_dev(q) if fmt == "f32" else G.to_bf16_dev(q)
    out = va.decode_attention(qd, c, seq_lens=sl, max_len=max_len, workspace=ws[:need])
    torch.cuda.synchronize()
    assert bool((ws[need:] == 0x5A).all()), "partials written past the workspace"
    want = oracle_decode(q, kc, vc, [300, max_len])
    if fmt == "f32":
        G.assert_f32_close(out.cpu().numpy(), want, "clamped decode")
    else:
        G.assert_bf16_close(G.bf16_to_np(out), want, "clamped decode")
    # host-side length above the bound: a caller error, reported before any launch
    with pytest.raises(va.VspError) as e:
        va.decode_attention(qd, c, max_len=max_len)  # cache.len == 1024
    assert e.value.status == va._ffi.ERR_ARG
