"""Prefill parity on the GPU through the C ABI (vsp_attn_prefill) against the oracle and the reference's fixtures."""
import math
import os

import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I
import _oracle as O

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def oracle_gqa_flash(q, k, v, scale, causal):
    """repeat_kv -> ops::flash_attention on the CPU oracle (fp32)."""
    n = q.shape[1] // k.shape[1]
    return O.flash_attention(q, O.repeat_kv(k, n), O.repeat_kv(v, n), scale, causal, return_lse=True)


def closed_form64(q, k, v, scale, causal):
    from test_oracle_known_answers import closed_form
    return closed_form(q, k, v, scale, causal)


# ---- fp32 -----------------------------------------------------------------------------------------

def test_f32_config1_against_reference_fixture(va):
    # benchmark config 1: B1, 8 q heads / 2 kv heads, D64, N256, scale 1/8, causal
    z = np.load(os.path.join(GOLD, "config1.npz"), allow_pickle=False)
    B, Hq, Hkv, N, D, seed = [int(x) for x in z["meta"]]
    q, k, v = I.qkv(seed, B, Hq, Hkv, N, N, D)
    out, lse = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), 0.125, True, return_lse=True)
    assert tuple(out.shape) == (1, 8, 256, 64)
    G.assert_f32_close(out.cpu().numpy(), z["out_flash"], "config1 vs reference flash")
    G.assert_f32_close(out.cpu().numpy(), z["out_sdpa"], "config1 vs reference sdpa")
    G.assert_f32_close(lse.cpu().numpy(), z["lse"], "config1 lse")
    out2 = va.scaled_dot_product_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), True)
    assert torch.equal(out, out2)


def test_f32_flash_fixtures(va):
    z = np.load(os.path.join(GOLD, "flash_attention.npz"), allow_pickle=False)
    for tag in sorted({k.rsplit("_", 1)[0] for k in z.files}):
        B, H, N, D, causal, seed = [int(x) for x in z[tag + "_meta"]]
        assert D in (32, 64, 128)  # every case the reference's own tests hold runs (head_dim 32 included)
        q, k, v = I.qkv(seed, B, H, H, N, N, D)
        out, lse = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), float(z[tag + "_scale"][0]), bool(causal),
                                      return_lse=True)
        G.assert_f32_close(out.cpu().numpy(), z[tag + "_out"], tag)
        G.assert_f32_close(lse.cpu().numpy(), z[tag + "_lse"], tag + " lse")


@pytest.mark.parametrize("B,Hq,Hkv,T,L,D,causal", [
    (1, 4, 1, 1, 1, 64, True), (2, 6, 2, 37, 37, 64, True), (1, 2, 2, 130, 130, 128, False),
    (1, 4, 2, 50, 200, 128, False), (1, 4, 2, 50, 200, 64, True), (1, 8, 8, 129, 129, 128, True),
    (1, 1, 1, 8, 8, 32, True), (2, 4, 2, 70, 70, 32, True), (1, 2, 1, 33, 100, 32, False)])
def test_f32_against_oracle_and_closed_form(va, B, Hq, Hkv, T, L, D, causal):
    q, k, v = I.qkv(21, B, Hq, Hkv, T, L, D)
    scale = 1.0 / math.sqrt(D)
    out = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), scale, causal).cpu().numpy()
    G.assert_f32_close(out, closed_form64(q, k, v, scale, causal).astype(np.float32), "closed form")
    if T == L:
        want, _ = oracle_gqa_flash(q, k, v, float(np.float32(scale)), causal)
        G.assert_f32_close(out, want, "oracle")


@pytest.mark.parametrize("B,Hq,Hkv,T,L,D,causal", [
    (1, 16, 4, 8, 8, 16, True), (1, 32, 8, 8, 8, 8, True),          # embed_dim 256 with 16 and 32 heads: the reference's
    (1, 8, 1, 8, 8, 32, True),                                      # own GQA configurations, tests/test_gqa_chapter33.cpp:600-627
    (2, 4, 2, 70, 70, 24, True), (1, 3, 1, 40, 90, 5, False), (1, 2, 2, 33, 33, 100, True), (1, 4, 2, 65, 65, 1, True),
    (1, 2, 1, 50, 50, 129, True), (1, 2, 2, 37, 80, 200, False), (1, 1, 1, 20, 20, 256, True)])
def test_f32_any_head_dim(va, B, Hq, Hkv, T, L, D, causal):
    # the reference's forward takes any head_dim (src/ops/flash_attention.cpp:235-238); here the fp32 kernel pads the
    # tile to the next of 32 / 64 / 128 / 256 inside the kernel, rows of any length are read element by element
    q, k, v = I.qkv(1200 + D, B, Hq, Hkv, T, L, D)
    scale = 1.0 / math.sqrt(D)
    out, lse = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), scale, causal, return_lse=True)
    out = out.cpu().numpy()
    G.assert_f32_close(out, closed_form64(q, k, v, scale, causal).astype(np.float32), "closed form")
    if T == L:
        want, want_lse = oracle_gqa_flash(q, k, v, float(np.float32(scale)), causal)
        G.assert_f32_close(out, want, "oracle")
        assert np.abs(lse.cpu().numpy() - want_lse).max() < 1e-4
    # a strided view (rows of a wider buffer): nothing about the row pitch is assumed
    wide = torch.zeros(B, Hkv, L, D + 3, device=G.dev())
    wide[..., :D] = G.f32_dev(k)
    out2 = va.flash_attention(G.f32_dev(q), wide[..., :D], G.f32_dev(v), scale, causal).cpu().numpy()
    assert np.array_equal(out, out2)


def test_head_dims_that_stay_unsupported(va):
    z = lambda *s: torch.zeros(*s, device=G.dev())
    with pytest.raises(va.VspError):      # fp32 beyond 256
        va.flash_attention(z(1, 1, 4, 257), z(1, 1, 4, 257), z(1, 1, 4, 257), 0.1, True)
    b = lambda *s: torch.zeros(*s, device=G.dev(), dtype=torch.bfloat16)
    with pytest.raises(va.VspError):      # bf16 keeps its two tile widths
        va.flash_attention(b(1, 1, 4, 32), b(1, 1, 4, 32), b(1, 1, 4, 32), 0.1, True)


def test_f32_known_answers_of_the_reference_tests(va):
    # causal structure, tests/test_attention_chapter32.cpp:168-203 (padded to D=64: extra dims are zero)
    q = np.ones((1, 1, 4, 64), np.float32)
    v = np.zeros((1, 1, 4, 64), np.float32)
    v[0, 0, :, 0] = np.arange(4)
    out = va.flash_attention(G.f32_dev(q), G.f32_dev(q), G.f32_dev(v), 0.5, True).cpu().numpy()
    assert np.abs(out[0, 0, :, 0] - [0, 0.5, 1.0, 1.5]).max() < 1e-5
    # constant V -> V, tests/test_attention_chapter32.cpp:209-239
    q, k, _ = I.qkv(5, 2, 2, 2, 9, 9, 64)
    vv = np.full((2, 2, 9, 64), 3.25, np.float32)
    out = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(vv), 0.3, True).cpu().numpy()
    assert np.abs(out - 3.25).max() < 1e-5
    # single token -> V, tests/test_attention_comprehensive.cpp:112-135
    q, k, v = I.qkv(6, 2, 3, 3, 1, 1, 64)
    out = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), 0.25, True).cpu().numpy()
    assert np.abs(out - v).max() < 1e-6
    # negative scale is legal mathematics
    q, k, v = I.qkv(7, 1, 2, 2, 20, 20, 64)
    out = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), -0.2, True).cpu().numpy()
    G.assert_f32_close(out, closed_form64(q, k, v, -0.2, True).astype(np.float32), "negative scale")


# ---- bf16 -----------------------------------------------------------------------------------------

def run_bf16(va, q, k, v, scale, causal, **kw):
    """q,k,v fp32 numpy already rounded to bf16 values."""
    return va.flash_attention(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), scale, causal, **kw)


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", [
    (1, 4, 2, 64, 128, True), (2, 4, 1, 200, 128, True), (1, 2, 2, 333, 128, False), (1, 8, 2, 257, 64, True),
    (1, 1, 1, 1, 128, True), (1, 4, 4, 127, 64, False), (1, 2, 1, 1024, 128, True)])
def test_bf16_against_oracle(va, B, Hq, Hkv, N, D, causal):
    # inputs N(0,1)*0.5 rounded to bf16 (the reference's RNE); the oracle consumes the rounded values in fp32
    q, k, v = [O.bf16_round(x) for x in I.qkv(31, B, Hq, Hkv, N, N, D, scale=0.5)]
    scale = 1.0 / math.sqrt(D)
    out, lse = run_bf16(va, q, k, v, scale, causal, return_lse=True)
    want, want_lse = oracle_gqa_flash(q, k, v, float(np.float32(scale)), causal)
    G.assert_bf16_close(G.bf16_to_np(out), want, f"N={N}")
    assert np.abs(lse.cpu().numpy() - want_lse).max() < 2e-2


def test_bf16_unit_variance_inputs(va):
    # harder numerically than the benchmark distribution: N(0,1) inputs, peaked softmax
    q, k, v = [O.bf16_round(x) for x in I.qkv(32, 1, 4, 2, 512, 512, 128)]
    scale = 1.0 / math.sqrt(128)
    out = run_bf16(va, q, k, v, scale, True)
    want, _ = oracle_gqa_flash(q, k, v, float(np.float32(scale)), True)
    G.assert_bf16_close(G.bf16_to_np(out), want, "N(0,1)")


def test_bf16_gqa_head_map(va):
    # every kv head holds a distinct constant V: output of q head h must be the constant of kv head h // n_rep
    B, Hq, Hkv, N, D = 1, 8, 2, 70, 128
    q, k, _ = [O.bf16_round(x) for x in I.qkv(33, B, Hq, Hkv, N, N, D)]
    v = np.zeros((B, Hkv, N, D), np.float32)
    v[:, 0], v[:, 1] = 1.0, -2.0
    out = G.bf16_to_np(run_bf16(va, q, k, v, 0.1, True))
    assert np.abs(out[:, :4] - 1.0).max() < 1e-2 and np.abs(out[:, 4:] + 2.0).max() < 2e-2


def test_bf16_chunk_appended_to_longer_context(va):
    # T < L, causal aligned to the end of the context (what a chunked prefill over a cache needs)
    B, Hq, Hkv, T, L, D = 1, 4, 2, 100, 300, 128
    q, k, v = [O.bf16_round(x) for x in I.qkv(34, B, Hq, Hkv, T, L, D, scale=0.5)]
    scale = 1.0 / math.sqrt(D)
    out = G.bf16_to_np(run_bf16(va, q, k, v, scale, True))
    G.assert_bf16_close(out, closed_form64(q, k, v, scale, True).astype(np.float32), "T<L causal")
    out = G.bf16_to_np(run_bf16(va, q, k, v, scale, False))
    G.assert_bf16_close(out, closed_form64(q, k, v, scale, False).astype(np.float32), "T<L full")


def test_bf16_strided_views(va):
    # k, v given as [:, :, 0:L, :] views of a larger [B,H,S_max,D] buffer, q/out as transposed [B,T,H,D] storage
    B, Hq, Hkv, N, S_max, D = 2, 4, 2, 96, 160, 128
    q, k, v = [O.bf16_round(x) for x in I.qkv(35, B, Hq, Hkv, N, N, D, scale=0.5)]
    kb = torch.zeros(B, Hkv, S_max, D, dtype=torch.bfloat16, device=G.dev())
    vb = torch.full((B, Hkv, S_max, D), float("nan"), dtype=torch.bfloat16, device=G.dev())
    kb[:, :, :N], vb[:, :, :N] = G.to_bf16_dev(k), G.to_bf16_dev(v)
    qt = G.to_bf16_dev(q).permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    assert not qt.is_contiguous()
    scale = 1.0 / math.sqrt(D)
    out = va.flash_attention(qt, kb[:, :, :N], vb[:, :, :N], scale, True)
    want, _ = oracle_gqa_flash(q, k, v, float(np.float32(scale)), True)
    G.assert_bf16_close(G.bf16_to_np(out), want, "strided")


def test_bf16_negative_scale_and_large_logits(va):
    q, k, v = [O.bf16_round(x) for x in I.qkv(36, 1, 2, 2, 150, 150, 64)]
    out = G.bf16_to_np(run_bf16(va, q, k, v, -0.3, True))
    G.assert_bf16_close(out, closed_form64(q, k, v, -0.3, True).astype(np.float32), "negative scale")
    # logits growing along the sequence force the reference maximum to be raised many times
    k2 = k * np.linspace(0.1, 6.0, 150, dtype=np.float32)[None, None, :, None]
    k2 = O.bf16_round(k2)
    out = G.bf16_to_np(run_bf16(va, q, k2, v, 1.0, False))
    G.assert_bf16_close(out, closed_form64(q, k2, v, 1.0, False).astype(np.float32), "growing logits")


@pytest.mark.parametrize("D", [128, 64])
@pytest.mark.parametrize("N", [160, 300, 1111])
@pytest.mark.parametrize("kind", ["growing", "spike_first", "spike_mid", "spike_last", "alternating_tiles", "negative_scale"])
def test_bf16_logits_in_the_tens_and_hundreds(va, N, kind, D):
    # head_dim 128 (the pipelined kernel, and the same kernel over a cache's planes) and 64 (the general kernel) with
    # scale 1 on unit-variance operands: logits of standard deviation 11 (8 at head_dim 64), up to several hundred in the
    # scaled cases.  Both kernels raise a row's reference maximum only when the row sum shows it has fallen behind: here
    # that happens many times, by single keys hundreds above the rest in the spike cases (the exp2 of a tile overflows
    # before the raise), and a score that carried a rounding of 2^-9 (Q multiplied by the scale in bf16) would miss the
    # bar by an order of magnitude.
    q, k, v = [O.bf16_round(x) for x in I.qkv(70 + N, 1, 4, 2, N, N, D)]
    scale = 1.0
    if kind in ("growing", "negative_scale"):
        k = O.bf16_round(k * np.linspace(0.1, 6.0, N, dtype=np.float32)[None, None, :, None])
        scale = -1.0 if kind == "negative_scale" else 1.0
    elif kind == "alternating_tiles":
        k = O.bf16_round(k * np.where(np.arange(N) % 64 < 32, 0.05, 5.0).astype(np.float32)[None, None, :, None])
    else:  # one key aligned with the last query of each head pair: its score is about 4 |q|^2 = 512
        pos = {"spike_first": 0, "spike_mid": N // 2, "spike_last": N - 1}[kind]
        k = k.copy()
        k[:, :, pos] = O.bf16_round(q[:, ::2, N - 1] * 4.0)
    tq, tk, tv = G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v)
    for causal in (True, False):
        want = closed_form64(q, k, v, scale, causal).astype(np.float32)
        # outputs reach |v| ~ 4, where one bf16 step is 0.0156 - 0.031: the bar is the usual one plus that rounding
        got = G.bf16_to_np(va.flash_attention(tq, tk, tv, scale, causal))
        G.assert_bf16_close_wide_range(got, want, f"{kind} N={N} causal={causal}")
    c = va.KVCache(1, 2, (N + 63) // 64 * 64, D, fmt="bf16")
    c.update(tk, tv, 0, return_views=False)
    want = closed_form64(q, k, v, scale, True).astype(np.float32)
    got = G.bf16_to_np(c.prefill(tq, scale=scale))
    G.assert_bf16_close_wide_range(got, want, f"planes {kind} N={N}")


@pytest.mark.parametrize("kind", ["growing", "spike_mid"])
def test_bf16_d128_general_kernel_logits_in_the_tens_and_hundreds(va, kind):
    # the same inputs on a grid large enough (3 x 32 heads x 9 query tiles = 864 workgroups, context <= 2560) that
    # head_dim 128 goes to the general kernel
    B, Hq, Hkv, N, D = 3, 32, 8, 1111, 128
    q, k, v = [O.bf16_round(x) for x in I.qkv(77, B, Hq, Hkv, N, N, D)]
    if kind == "growing":
        k = O.bf16_round(k * np.linspace(0.1, 6.0, N, dtype=np.float32)[None, None, :, None])
    else:
        k = k.copy()
        k[:, :, N // 2] = O.bf16_round(q[:, ::4, N - 1] * 4.0)
    got = G.bf16_to_np(va.flash_attention(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), 1.0, True))
    want = closed_form64(q, k, v, 1.0, True).astype(np.float32)
    G.assert_bf16_close_wide_range(got, want, kind)


@pytest.mark.parametrize("causal", [True, False])
def test_bf16_d128_general_kernel_chunk_over_longer_context(va, causal):
    # T < L on a grid of 8 x 32 heads x 3 query tiles = 768 workgroups: head_dim 128 through the general kernel, causal
    # mask aligned to the end of the context, a context that ends inside a key tile, strided K/V views of a larger buffer
    B, Hq, Hkv, T, L, D, S_max = 8, 32, 8, 384, 700, 128, 768
    q, k, v = [O.bf16_round(x) for x in I.qkv(78, B, Hq, Hkv, T, L, D, scale=0.5)]
    kb = torch.zeros(B, Hkv, S_max, D, dtype=torch.bfloat16, device=G.dev())
    vb = torch.full((B, Hkv, S_max, D), float("nan"), dtype=torch.bfloat16, device=G.dev())
    kb[:, :, :L], vb[:, :, :L] = G.to_bf16_dev(k), G.to_bf16_dev(v)
    scale = 1.0 / math.sqrt(D)
    out, lse = va.flash_attention(G.to_bf16_dev(q), kb[:, :, :L], vb[:, :, :L], scale, causal, return_lse=True)
    G.assert_bf16_close(G.bf16_to_np(out), closed_form64(q, k, v, scale, causal).astype(np.float32), f"T<L causal={causal}")
    # lse of a few rows against the definition
    n = Hq // Hkv
    for (b, h, t) in ((0, 0, 0), (3, 17, 200), (7, 31, 383)):
        s = (k[b, h // n, :L].astype(np.float64) @ q[b, h, t].astype(np.float64)) * scale
        if causal:
            s = s[:L - T + t + 1]
        want = np.log(np.exp(s - s.max()).sum()) + s.max()
        assert abs(lse[b, h, t].item() - want) < 2e-2


def test_bf16_d128_the_two_kernels_agree(va):
    # head_dim 128 is served by two kernels: short contexts on a grid that fills the chip (here B2 x 32 heads x 2048:
    # 1024 workgroups) go to the general kernel, the same rows one batch row at a time (512 workgroups) and longer
    # contexts to the software-pipelined one.  Same inputs, same rows: the results differ by bf16 roundings only, and
    # the sampled rows match the oracle.
    B, Hq, Hkv, N, D = 2, 32, 8, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(11)
    mk = lambda h: (torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    q, k, v = mk(Hq), mk(Hkv), mk(Hkv)
    scale = 1.0 / math.sqrt(D)
    both = va.flash_attention(q, k, v, scale, True)
    for b in range(B):
        one = va.flash_attention(q[b:b + 1], k[b:b + 1], v[b:b + 1], scale, True)
        d = (both[b:b + 1].float() - one.float()).abs()
        assert d.max().item() <= 1.6e-2 and d.mean().item() <= 1e-3, (b, d.max().item(), d.mean().item())
    # oracle on one (batch row, kv head): 4 query heads, all 2048 rows
    qn = q[1:2, 4:8].float().cpu().numpy()
    kn, vn = k[1:2, 1:2].float().cpu().numpy(), v[1:2, 1:2].float().cpu().numpy()
    want, _ = oracle_gqa_flash(qn, kn, vn, float(np.float32(scale)), True)
    G.assert_bf16_close(G.bf16_to_np(both[1:2, 4:8]), want, "general kernel, head_dim 128, N 2048")


def test_bf16_full_size_properties(va):
    # benchmark config 2 shape (B4, 32/8 heads, D128, N2048): properties that need no oracle at this size
    B, Hq, Hkv, N, D = 4, 32, 8, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(7)
    q = (torch.randn(B, Hq, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    k = (torch.randn(B, Hkv, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(B, Hkv, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    out, lse = va.flash_attention(q, k, v, scale, True, return_lse=True)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    # run-to-run determinism (tests/test_attention_chapter32.cpp:376-411 of the reference)
    assert torch.equal(out, va.flash_attention(q, k, v, scale, True))
    # causal prefix independence: the first 512 rows do not depend on later tokens
    out_prefix = va.flash_attention(q[:, :, :512].contiguous(), k[:, :, :512].contiguous(), v[:, :, :512].contiguous(), scale, True)
    assert (out[:, :, :512].float() - out_prefix.float()).abs().max().item() <= 1e-2
    # constant V -> V
    vc = torch.full_like(v, 0.75)
    assert (va.flash_attention(q, k, vc, scale, True).float() - 0.75).abs().max().item() < 1e-2
    # one (batch, head) slice against the oracle at full length
    b, h = 3, 21
    qs, ks, vs = [G.bf16_to_np(t) for t in (q[b:b + 1, h:h + 1], k[b:b + 1, h // 4:h // 4 + 1], v[b:b + 1, h // 4:h // 4 + 1])]
    want, _ = O.flash_attention(qs, ks, vs, float(np.float32(scale)), True, return_lse=True)
    G.assert_bf16_close(G.bf16_to_np(out[b:b + 1, h:h + 1]), want, "config-2 slice")


def test_bf16_config3_size_properties(va):
    # benchmark config 3 shape (B1, 32/8 heads, D128, N8192)
    B, Hq, Hkv, N, D = 1, 32, 8, 8192, 128
    g = torch.Generator(device="cuda").manual_seed(9)
    q = (torch.randn(B, Hq, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    k = (torch.randn(B, Hkv, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    v = (torch.randn(B, Hkv, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    scale = 1.0 / math.sqrt(D)
    out, lse = va.flash_attention(q, k, v, scale, True, return_lse=True)
    assert torch.isfinite(out.float()).all() and torch.isfinite(lse).all()
    assert torch.equal(out, va.flash_attention(q, k, v, scale, True))
    # causal prefix: rows < 4096 see exactly the tiles a 4096-token launch sees, in the same order -> bit-identical
    half = va.flash_attention(q[:, :, :4096].contiguous(), k[:, :, :4096].contiguous(), v[:, :, :4096].contiguous(), scale, True)
    assert torch.equal(out[:, :, :4096], half)
    # the last 128 rows of two heads against a float64 closed form over all 8192 keys
    for h in (0, 29):
        qs = G.bf16_to_np(q[0, h, N - 128:]).astype(np.float64)
        ks, vs = G.bf16_to_np(k[0, h // 4]).astype(np.float64), G.bf16_to_np(v[0, h // 4]).astype(np.float64)
        s = qs @ ks.T * scale
        s[np.arange(N)[None, :] > (N - 128 + np.arange(128))[:, None]] = -np.inf
        p = np.exp(s - s.max(axis=1, keepdims=True))
        want = (p / p.sum(axis=1, keepdims=True)) @ vs
        G.assert_bf16_close(G.bf16_to_np(out[0, h, N - 128:]), want.astype(np.float32), f"config-3 head {h}")
        want_lse = s.max(axis=1) + np.log(p.sum(axis=1))
        assert np.abs(lse[0, h, N - 128:].cpu().numpy() - want_lse).max() < 2e-2


def test_validation_errors_follow_the_reference(va):
    d = G.dev()
    f = lambda *s, dt=torch.bfloat16: torch.zeros(*s, dtype=dt, device=d)
    with pytest.raises(va.VspError) as e:
        va.flash_attention(f(2, 4, 64), f(2, 4, 64), f(2, 4, 64), 1.0)
    assert str(e.value) == "flash_attention: inputs must be 4D [B, H, N, D]"
    with pytest.raises(va.VspError) as e:
        va.flash_attention(f(1, 2, 4, 64), f(1, 2, 5, 64), f(1, 2, 4, 64), 1.0)
    assert str(e.value) == "flash_attention: Q, K, V must have same shape"
    with pytest.raises(va.VspError) as e:
        va.flash_attention(f(1, 3, 4, 64), f(1, 2, 4, 64), f(1, 2, 4, 64), 1.0)  # 3 q heads over 2 kv heads
    assert e.value.status == 2
    with pytest.raises(va.VspError) as e:
        va.flash_attention(f(1, 2, 4, 64), f(1, 2, 4, 64), f(1, 2, 4, 64, dt=torch.float32), 1.0)
    assert str(e.value) == "flash_attention: Q, K, V must have same dtype"
    for p in (1.0, -0.1):
        with pytest.raises(va.VspError) as e:
            va.flash_attention(f(1, 2, 4, 64), f(1, 2, 4, 64), f(1, 2, 4, 64), 1.0, dropout_p=p)
        assert str(e.value) == "flash_attention: dropout_p must be in [0, 1)"
    # inference semantics: dropout_p > 0 with training == False is a no-op (src/ops/flash_attention.cpp:241)
    q = torch.randn(1, 2, 8, 64, device=d).to(torch.bfloat16)
    assert torch.equal(va.flash_attention(q, q, q, 0.3, True, dropout_p=0.5, training=False), va.flash_attention(q, q, q, 0.3, True))
    with pytest.raises(va.VspError) as e:
        va.flash_attention(f(1, 2, 4, 80), f(1, 2, 4, 80), f(1, 2, 4, 80), 1.0)
    assert e.value.status == 33
    with pytest.raises(va.VspError) as e:
        va.scaled_dot_product_attention(f(1, 2, 4, 64), f(1, 2, 6, 64), f(1, 2, 6, 64), True)
    assert e.value.status == 10
    # empty batch is a no-op
    assert va.flash_attention(f(0, 2, 4, 64), f(0, 2, 4, 64), f(0, 2, 4, 64), 1.0).numel() == 0
