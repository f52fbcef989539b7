"""Attention backward on the GPU through the C ABI (vsp_attn_prefill_backward) against the oracle (bit-exact to the
compiled reference), the reference-written fixture and a float64 closed form.  fp32: 1e-4 relative.  bf16 inputs run
on bf16 matrix cores (P and dS are rounded to bf16 between the products, accumulation is fp32): max-abs 2e-2 and
mean-abs 2e-3 relative to the gradient's scale, the bar of the bf16 forward."""
import math
import os

import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I
import _oracle as O
from test_oracle_backward import closed_form_grads

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def _forward_then_backward(va, q, k, v, dout, scale, causal, bf16=False, fast=False):
    # fast: the larger workspace, with which the bf16 path computes dS once (vsp_attn_backward_fast_workspace_bytes)
    cv = G.to_bf16_dev if bf16 else G.f32_dev
    dq_, dk_, dv_, dd_ = cv(q), cv(k), cv(v), cv(dout)
    out, lse = va.flash_attention(dq_, dk_, dv_, scale, causal, return_lse=True)
    return va.flash_attention_backward(dd_, dq_, dk_, dv_, out, lse, scale, causal, workspace=va.backward_workspace(dq_, fast=fast))


def test_fixture_written_from_the_reference(va):
    z = np.load(os.path.join(GOLD, "flash_backward.npz"), allow_pickle=False)
    for tag in ("r70", "nc33", "d128", "t16"):   # t16: the reference's own {1,1,8,32} shape
        B, H, N, D, causal, seed = [int(x) for x in z[tag + "_meta"]]
        q, k, v = I.qkv(seed, B, H, H, N, N, D)
        dout = I.normal(seed + 5, (B, H, N, D))
        scale = float(np.float32(1.0 / np.sqrt(D)))
        dq, dk, dv = _forward_then_backward(va, q, k, v, dout, scale, bool(causal))
        G.assert_f32_close(dq.cpu().numpy(), z[tag + "_dq"], tag + " dq")
        G.assert_f32_close(dk.cpu().numpy(), z[tag + "_dk"], tag + " dk")
        G.assert_f32_close(dv.cpu().numpy(), z[tag + "_dv"], tag + " dv")


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", [(1, 4, 2, 100, 64, True), (2, 8, 2, 257, 128, True), (1, 4, 4, 64, 128, False),
                                                 (1, 6, 1, 33, 64, True)])
def test_f32_gqa_against_oracle_through_repeat_kv(va, B, Hq, Hkv, N, D, causal):
    # GroupedQueryAttention trains through repeat_kv -> flash_attention: dk / dv of a kv head are the sums of the
    # repeated heads' gradients (the backward of ops::repeat_kv, src/ops/attention_ops.cpp:120-150)
    q, k, v = I.qkv(700 + N, B, Hq, Hkv, N, N, D)
    dout = I.normal(705 + N, (B, Hq, N, D))
    scale = float(np.float32(1.0 / np.sqrt(D)))
    n = Hq // Hkv
    kr, vr = O.repeat_kv(k, n), O.repeat_kv(v, n)
    out, lse = O.flash_attention(q, kr, vr, scale, causal, return_lse=True)
    wq, wk, wv = O.flash_attention_backward(dout, q, kr, vr, out, lse, scale, causal)
    wk = wk.reshape(B, Hkv, n, N, D).sum(2)
    wv = wv.reshape(B, Hkv, n, N, D).sum(2)
    dq, dk, dv = _forward_then_backward(va, q, k, v, dout, scale, causal)
    G.assert_f32_close(dq.cpu().numpy(), wq, "dq")
    G.assert_f32_close(dk.cpu().numpy(), wk, "dk")
    G.assert_f32_close(dv.cpu().numpy(), wv, "dv")
    # and the float64 closed form (independent algebra)
    cq, ck, cv = closed_form_grads(dout, q, kr, vr, scale, causal)
    G.assert_f32_close(dq.cpu().numpy(), cq.astype(np.float32), "dq closed form")
    G.assert_f32_close(dk.cpu().numpy(), ck.reshape(B, Hkv, n, N, D).sum(2).astype(np.float32), "dk closed form")


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", [(1, 16, 4, 8, 16, True), (1, 32, 8, 8, 8, True), (2, 4, 2, 70, 24, True),
                                                 (1, 3, 1, 45, 5, False), (1, 2, 2, 33, 100, True)])
def test_f32_any_head_dim(va, B, Hq, Hkv, N, D, causal):
    # the reference's backward takes any head_dim (src/ops/flash_attention.cpp:366-482); 16 and 8 are what its own GQA
    # configurations have at embed_dim 256 (tests/test_gqa_chapter33.cpp:600-627)
    q, k, v = I.qkv(800 + D, B, Hq, Hkv, N, N, D)
    dout = I.normal(805 + D, (B, Hq, N, D))
    scale = float(np.float32(1.0 / np.sqrt(D)))
    n = Hq // Hkv
    kr, vr = O.repeat_kv(k, n), O.repeat_kv(v, n)
    out, lse = O.flash_attention(q, kr, vr, scale, causal, return_lse=True)
    wq, wk, wv = O.flash_attention_backward(dout, q, kr, vr, out, lse, scale, causal)
    dq, dk, dv = _forward_then_backward(va, q, k, v, dout, scale, causal)
    G.assert_f32_close(dq.cpu().numpy(), wq, "dq")
    G.assert_f32_close(dk.cpu().numpy(), wk.reshape(B, Hkv, n, N, D).sum(2), "dk")
    G.assert_f32_close(dv.cpu().numpy(), wv.reshape(B, Hkv, n, N, D).sum(2), "dv")
    cq, ck, cv = closed_form_grads(dout, q, kr, vr, scale, causal)
    G.assert_f32_close(dq.cpu().numpy(), cq.astype(np.float32), "dq closed form")
    G.assert_f32_close(dv.cpu().numpy(), cv.reshape(B, Hkv, n, N, D).sum(2).astype(np.float32), "dv closed form")


def test_single_token(va):
    # N = 1: P = 1, so dS = dP - Di = 0 and dq = dk = 0 exactly in exact arithmetic, dv = dout
    q, k, v = I.qkv(750, 1, 2, 2, 1, 1, 64)
    dout = I.normal(755, (1, 2, 1, 64))
    dq, dk, dv = _forward_then_backward(va, q, k, v, dout, 0.125, True)
    assert np.abs(dq.cpu().numpy()).max() < 1e-5 and np.abs(dk.cpu().numpy()).max() < 1e-5
    G.assert_f32_close(dv.cpu().numpy(), dout, "dv")


@pytest.mark.parametrize("fast", [False, True])
def test_bf16_inputs_and_determinism(va, fast):
    B, Hq, Hkv, N, D = 2, 8, 2, 300, 128
    q, k, v = [O.bf16_round(x * np.float32(0.5)) for x in I.qkv(800, B, Hq, Hkv, N, N, D)]
    dout = O.bf16_round(I.normal(805, (B, Hq, N, D)))
    scale = 1.0 / math.sqrt(D)
    dq, dk, dv = _forward_then_backward(va, q, k, v, dout, scale, True, bf16=True, fast=fast)
    again = _forward_then_backward(va, q, k, v, dout, scale, True, bf16=True, fast=fast)
    for a, b in zip((dq, dk, dv), again):
        assert torch.equal(a, b)          # no atomics: bitwise reproducible
    kr, vr = O.repeat_kv(k, 4), O.repeat_kv(v, 4)
    cq, ck, cv = closed_form_grads(dout, q, kr, vr, float(np.float32(scale)), True)
    ck = ck.reshape(B, Hkv, 4, N, D).sum(2)
    cv = cv.reshape(B, Hkv, 4, N, D).sum(2)
    # the forward's bf16 output and fp32 lse feed the backward: tolerance of the bf16 path
    for got, want, name in ((dq, cq, "dq"), (dk, ck, "dk"), (dv, cv, "dv")):
        g = G.bf16_to_np(got)
        err = np.abs(g - want)
        assert np.isfinite(g).all() and err.max() <= 3e-2 * max(1.0, np.abs(want).max()), (name, err.max())
        assert err.mean() <= 2e-3 * max(1.0, np.abs(want).mean() * 10), (name, err.mean())


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", [(1, 4, 2, 100, 64, True), (2, 8, 2, 257, 128, True), (1, 4, 4, 64, 128, False),
                                                 (1, 6, 1, 33, 64, True), (1, 2, 1, 129, 128, False), (1, 8, 8, 1, 64, True),
                                                 (1, 4, 1, 512, 128, True), (1, 2, 2, 96, 64, True), (2, 4, 2, 200, 128, False)])
@pytest.mark.parametrize("fast", [False, True])
def test_bf16_against_oracle(va, B, Hq, Hkv, N, D, causal, fast):
    q, k, v = [O.bf16_round(x) for x in I.qkv(820 + N, B, Hq, Hkv, N, N, D)]
    dout = O.bf16_round(I.normal(825 + N, (B, Hq, N, D)))
    scale = float(np.float32(1.0 / np.sqrt(D)))
    n = Hq // Hkv
    kr, vr = O.repeat_kv(k, n), O.repeat_kv(v, n)
    out, lse = O.flash_attention(q, kr, vr, scale, causal, return_lse=True)
    wq, wk, wv = O.flash_attention_backward(dout, q, kr, vr, out, lse, scale, causal)
    wk = wk.reshape(B, Hkv, n, N, D).sum(2)
    wv = wv.reshape(B, Hkv, n, N, D).sum(2)
    dq, dk, dv = _forward_then_backward(va, q, k, v, dout, scale, causal, bf16=True, fast=fast)
    for got, want, name in ((dq, wq, "dq"), (dk, wk, "dk"), (dv, wv, "dv")):
        g = G.bf16_to_np(got)
        err = np.abs(g - want)
        ref = max(1.0, float(np.abs(want).max()))
        assert np.isfinite(g).all() and err.max() <= 2e-2 * ref, (name, err.max(), ref)
        assert err.mean() <= 2e-3 * ref, (name, err.mean(), ref)


def test_bf16_dS_once_against_dS_twice(va):
    # The two bf16 paths differ in where dQ's dS comes from: recomputed from the fp32 P in the dQ pass, or the tiles the
    # dK / dV pass left behind (P rounded to bf16 first: one more rounding of 2^-9 relative per element of dS), and in
    # the summation order of Di.  dK and dV go through the same arithmetic in both.
    B, Hq, Hkv, N, D = 2, 8, 2, 1000, 128
    g = torch.Generator(device="cuda").manual_seed(23)
    mk = lambda h: (torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.7).to(torch.bfloat16)
    q, k, v, dout = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    scale = 1.0 / math.sqrt(D)
    for causal in (True, False):
        out, lse = va.flash_attention(q, k, v, scale, causal, return_lse=True)
        two = va.flash_attention_backward(dout, q, k, v, out, lse, scale, causal)
        ws = va.backward_workspace(q, fast=True)
        ws.fill_(0xff)            # stale tiles would show as NaNs
        one = va.flash_attention_backward(dout, q, k, v, out, lse, scale, causal, workspace=ws)
        for a, b, name in zip(one, two, ("dq", "dk", "dv")):
            a, b = a.float(), b.float()
            assert torch.isfinite(a).all(), name
            ref = max(1.0, b.abs().max().item())
            assert (a - b).abs().max().item() <= (2e-2 if name == "dq" else 8e-3) * ref, (name, causal, (a - b).abs().max().item())
            assert (a - b).abs().mean().item() <= (1e-3 if name == "dq" else 1e-4) * ref, (name, causal, (a - b).abs().mean().item())


def test_the_workspace_size_selects_the_bf16_path(va):
    # one byte short of vsp_attn_backward_fast_workspace_bytes(): the recomputing path, bit for bit; fp32 tensors ignore
    # the extra room
    B, Hq, Hkv, N, D = 1, 4, 2, 300, 64
    g = torch.Generator(device="cuda").manual_seed(29)
    mk = lambda h, dt: (torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.7).to(dt)
    for dt in (torch.bfloat16, torch.float32):
        q, k, v, dout = mk(Hq, dt), mk(Hkv, dt), mk(Hkv, dt), mk(Hq, dt)
        out, lse = va.flash_attention(q, k, v, 0.125, True, return_lse=True)
        small = va.flash_attention_backward(dout, q, k, v, out, lse, 0.125, True)
        big = va.backward_workspace(q, fast=True)
        short = va.flash_attention_backward(dout, q, k, v, out, lse, 0.125, True, workspace=big[:big.numel() - 1])
        full = va.flash_attention_backward(dout, q, k, v, out, lse, 0.125, True, workspace=big)
        for a, b in zip(short, small):
            assert torch.equal(a, b)
        if dt == torch.float32:
            for a, b in zip(full, small):
                assert torch.equal(a, b)
        else:
            assert not torch.equal(full[0], small[0])      # dQ from the stored tiles: P rounded before the multiply
            assert (full[0].float() - small[0].float()).abs().max().item() <= 2e-2 * max(1.0, small[0].float().abs().max().item())


@pytest.mark.parametrize("bf16,fast", [(False, False), (True, False), (True, True)])
def test_strided_operands(va, bf16, fast):
    # [B, N, H, D] storage viewed as [B, H, N, D] (what a fused qkv projection hands over): the strides of every
    # operand and of every gradient are honoured
    B, Hq, Hkv, N, D = 2, 4, 2, 70, 64
    q, k, v = [O.bf16_round(x) for x in I.qkv(860, B, Hq, Hkv, N, N, D)]
    dout = O.bf16_round(I.normal(865, (B, Hq, N, D)))
    cv = G.to_bf16_dev if bf16 else G.f32_dev
    dense = [cv(x) for x in (dout, q, k, v)]
    strided = [t.transpose(1, 2).contiguous().transpose(1, 2) for t in dense]
    assert not strided[0].is_contiguous()
    out, lse = va.flash_attention(dense[1], dense[2], dense[3], 0.125, True, return_lse=True)
    ws = lambda: va.backward_workspace(dense[1], fast=fast)
    want = va.flash_attention_backward(*dense, out, lse, 0.125, True, workspace=ws())
    got = va.flash_attention_backward(*strided, out.transpose(1, 2).contiguous().transpose(1, 2), lse, 0.125, True, workspace=ws())
    for g, w in zip(got, want):
        assert g.stride() != w.stride() and torch.equal(g, w)


def test_bf16_rows_must_be_16_byte_aligned(va):
    d = G.dev()
    flat = torch.zeros(4 + 2 * 8 * 64, dtype=torch.bfloat16, device=d)
    off = flat[4:].view(1, 2, 8, 64)       # 8-byte aligned only
    ok = torch.zeros(1, 2, 8, 64, dtype=torch.bfloat16, device=d)
    with pytest.raises(va.VspError):
        va.flash_attention_backward(ok, off, ok, ok, ok, torch.zeros(1, 2, 8, device=d), 0.1)


@pytest.mark.parametrize("fast", [False, True])
def test_bf16_config3_shape_causal_truncation(va, fast):
    # benchmark config 3's shape (B1, 32/8 heads, D128, N8192).  With dO = 0 from row n on, causal attention makes the
    # first n rows of dq / dk / dv those of the n-token problem - bit for bit, because the later query tiles add exact
    # zeros (dP = 0, Di = 0, so dS = 0, and P * 0 = 0) in between the same partial sums - and the rest exactly zero.
    B, Hq, Hkv, N, D, n = 1, 32, 8, 8192, 128, 2048
    g = torch.Generator(device="cuda").manual_seed(19)
    mk = lambda h: (torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.5).to(torch.bfloat16)
    q, k, v, dout = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    dout[:, :, n:] = 0
    scale = 1.0 / math.sqrt(D)
    out, lse = va.flash_attention(q, k, v, scale, True, return_lse=True)
    dq, dk, dv = va.flash_attention_backward(dout, q, k, v, out, lse, scale, True, workspace=va.backward_workspace(q, fast=fast))
    cut = lambda t: t[:, :, :n].contiguous()
    sq, sk, sv = va.flash_attention_backward(cut(dout), cut(q), cut(k), cut(v), cut(out), lse[:, :, :n].contiguous(), scale, True,
                                             workspace=va.backward_workspace(cut(q), fast=fast))
    for big, small, name in ((dq, sq, "dq"), (dk, sk, "dk"), (dv, sv, "dv")):
        assert torch.isfinite(big.float()).all(), name
        assert torch.equal(big[:, :, :n], small), name
        assert not big[:, :, n:].any(), name
        assert small.float().abs().max() > 1e-3, name      # the comparison is not between zeros
    # dv of the last key of the sub-problem: only query n - 1 sees it, P = exp(s - lse) -> dv = P * dO[n - 1], summed
    # over the 4 query heads of the group (float64, from the kernel's own lse)
    qf, kf = G.bf16_to_np(q[0, :, n - 1]).astype(np.float64), G.bf16_to_np(k[0, :, n - 1]).astype(np.float64)
    dof = G.bf16_to_np(dout[0, :, n - 1]).astype(np.float64)
    l = lse[0, :, n - 1].cpu().numpy().astype(np.float64)
    for kvh in (0, 5):
        want = sum(np.exp(qf[h] @ kf[kvh] * scale - l[h]) * dof[h] for h in range(4 * kvh, 4 * kvh + 4))
        got = G.bf16_to_np(dv[0, kvh, n - 1]).astype(np.float64)
        assert np.abs(got - want).max() <= 2e-2 * max(1.0, np.abs(want).max())


def test_argument_errors(va):
    d = G.dev()
    q = torch.zeros(1, 4, 8, 64, device=d)
    k = torch.zeros(1, 2, 8, 64, device=d)
    lse = torch.zeros(1, 4, 8, device=d)
    with pytest.raises(va.VspError):   # bf16: head dim 64 or 128 only
        z = torch.zeros(1, 2, 8, 32, device=d, dtype=torch.bfloat16)
        va.flash_attention_backward(z, z, z, z, z, torch.zeros(1, 2, 8, device=d), 0.1)
    with pytest.raises(va.VspError):   # fp32: any head dim up to 128
        z = torch.zeros(1, 2, 8, 160, device=d)
        va.flash_attention_backward(z, z, z, z, z, torch.zeros(1, 2, 8, device=d), 0.1)
    with pytest.raises(va.VspError):   # 3 query heads over 2 kv heads
        q3 = torch.zeros(1, 3, 8, 64, device=d)
        va.flash_attention_backward(q3, q3, k, k, q3, torch.zeros(1, 3, 8, device=d), 0.1)
    with pytest.raises(va.VspError):   # mixed dtypes
        va.flash_attention_backward(q.to(torch.bfloat16), q, k, k, q, lse, 0.1)
    dq, dk, dv = va.flash_attention_backward(q, q, k, k, q, lse, 0.1)
    assert dq.shape == q.shape and dk.shape == k.shape and not dq.any() and not dv.any()
