"""fp32 tensors through the bf16 matrix cores (vsp_attn_prefill_split: operands as two bf16 terms, three MFMAs per
product) against the reference's fp32 results: the fixtures the compiled reference wrote, the oracle, a float64 closed
form.  The bar is the fp32 one, 1e-4 of the output's magnitude; the observed error is asserted a factor below it so that
a lost term (which costs 2^-9) cannot hide inside the bar."""
import math
import os

import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I
from test_gpu_prefill import GOLD, closed_form64, oracle_gqa_flash

pytestmark = pytest.mark.gpu

TIGHT = 3e-5   # a dropped hi*lo term shows as ~4e-3, a dropped lo split of P as ~2e-3


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def rel_err(got, want):
    return float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max() / max(float(np.abs(want).max()), 1e-30))


def test_config1_against_reference_fixture(va):
    z = np.load(os.path.join(GOLD, "config1.npz"), allow_pickle=False)
    B, Hq, Hkv, N, D, seed = [int(x) for x in z["meta"]]
    q, k, v = I.qkv(seed, B, Hq, Hkv, N, N, D)
    out, lse = va.flash_attention_split(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), 0.125, True, return_lse=True)
    G.assert_f32_close(out.cpu().numpy(), z["out_flash"], "config1 vs reference flash")
    G.assert_f32_close(lse.cpu().numpy(), z["lse"], "config1 lse")
    assert rel_err(out.cpu().numpy(), z["out_flash"]) < TIGHT


def test_flash_fixtures_of_the_reference(va):
    z = np.load(os.path.join(GOLD, "flash_attention.npz"), allow_pickle=False)
    ran = 0
    for tag in sorted({k.rsplit("_", 1)[0] for k in z.files}):
        B, H, N, D, causal, seed = [int(x) for x in z[tag + "_meta"]]
        if D == 32:
            continue  # head_dim 32 stays with the fp32-MFMA kernel (asserted below)
        q, k, v = I.qkv(seed, B, H, H, N, N, D)
        out, lse = va.flash_attention_split(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), float(z[tag + "_scale"][0]), bool(causal),
                                            return_lse=True)
        G.assert_f32_close(out.cpu().numpy(), z[tag + "_out"], tag)
        G.assert_f32_close(lse.cpu().numpy(), z[tag + "_lse"], tag + " lse")
        ran += 1
    assert ran >= 4


@pytest.mark.parametrize("B,Hq,Hkv,T,L,D,causal", [
    (1, 4, 1, 1, 1, 64, True), (2, 6, 2, 37, 37, 64, True), (1, 2, 2, 130, 130, 128, False),
    (1, 4, 2, 50, 200, 128, False), (1, 4, 2, 50, 200, 64, True), (1, 8, 8, 129, 129, 128, True),
    (2, 8, 2, 300, 300, 128, True), (1, 4, 4, 1000, 1000, 64, True)])
def test_against_oracle_and_closed_form(va, B, Hq, Hkv, T, L, D, causal):
    q, k, v = I.qkv(23, B, Hq, Hkv, T, L, D)
    scale = 1.0 / math.sqrt(D)
    out = va.flash_attention_split(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), scale, causal).cpu().numpy()
    want64 = closed_form64(q, k, v, scale, causal)
    assert rel_err(out, want64) < TIGHT, rel_err(out, want64)
    if T == L:
        want, _ = oracle_gqa_flash(q, k, v, float(np.float32(scale)), causal)
        G.assert_f32_close(out, want, "oracle")
    # and next to the fp32-MFMA kernel of the same library
    ref = va.flash_attention(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), scale, causal).cpu().numpy()
    assert rel_err(out, ref) < TIGHT


def test_large_values_negative_scale_and_strided_views(va):
    # scores of several units (sharp softmax), a negative scale, and q/k/v as [B,T,H,D] storage viewed as [B,H,T,D]
    B, Hq, Hkv, N, D = 2, 4, 2, 96, 64
    q, k, v = I.qkv(31, B, Hq, Hkv, N, N, D, scale=2.0)
    for scale in (0.125, -0.125):
        tq = G.f32_dev(q.transpose(0, 2, 1, 3).copy()).transpose(1, 2)
        tk = G.f32_dev(k.transpose(0, 2, 1, 3).copy()).transpose(1, 2)
        tv = G.f32_dev(v.transpose(0, 2, 1, 3).copy()).transpose(1, 2)
        assert not tq.is_contiguous()
        out = va.flash_attention_split(tq, tk, tv, scale, True).cpu().numpy()
        assert rel_err(out, closed_form64(q, k, v, scale, True)) < TIGHT
    # the known answers of the reference's tests that survive a 16-bit operand: constant V, causal structure
    qq, kk, _ = I.qkv(5, 2, 2, 2, 9, 9, 64)
    vv = np.full((2, 2, 9, 64), 3.25, np.float32)
    out = va.flash_attention_split(G.f32_dev(qq), G.f32_dev(kk), G.f32_dev(vv), 0.3, True).cpu().numpy()
    assert np.abs(out - 3.25).max() < 1e-5                          # tests/test_attention_chapter32.cpp:209-239
    q1 = np.ones((1, 1, 4, 64), np.float32)
    v1 = np.zeros((1, 1, 4, 64), np.float32)
    v1[0, 0, :, 0] = np.arange(4)
    out = va.flash_attention_split(G.f32_dev(q1), G.f32_dev(q1), G.f32_dev(v1), 0.5, True).cpu().numpy()
    assert np.abs(out[0, 0, :, 0] - [0, 0.5, 1.0, 1.5]).max() < 1e-5  # tests/test_attention_chapter32.cpp:168-203


def test_config2_shape_properties(va):
    # benchmark config 2's shape with fp32 tensors: deterministic run to run, causal prefix independence, and a slice
    # against the float64 closed form
    B, Hq, Hkv, N, D = 1, 8, 2, 2048, 128
    q, k, v = I.qkv(41, B, Hq, Hkv, N, N, D, scale=0.5)
    tq, tk, tv = G.f32_dev(q), G.f32_dev(k), G.f32_dev(v)
    scale = 1.0 / math.sqrt(D)
    out = va.flash_attention_split(tq, tk, tv, scale, True)
    assert torch.equal(out, va.flash_attention_split(tq, tk, tv, scale, True))
    half = va.flash_attention_split(tq[:, :, :1024].contiguous(), tk[:, :, :1024].contiguous(), tv[:, :, :1024].contiguous(), scale, True)
    assert torch.equal(out[:, :, :1024], half)
    sl = slice(2040, 2048)
    want = closed_form64(q[:, :1, sl], k[:, :1], v[:, :1], scale, True)    # the last 8 rows as a chunk at the end of the context
    assert rel_err(out[:, :1, sl].cpu().numpy(), want) < TIGHT


def test_argument_errors(va):
    from vesper_amd import _ffi
    q, k, v = I.qkv(7, 1, 2, 2, 16, 16, 64)

    def code(fn):
        with pytest.raises(va.VspError) as e:
            fn()
        return e.value.status

    tq, tk, tv = G.f32_dev(q), G.f32_dev(k), G.f32_dev(v)
    assert code(lambda: va.flash_attention_split(tq.bfloat16(), tk.bfloat16(), tv.bfloat16(), 0.1)) == _ffi.ERR_UNSUPPORTED
    q32, k32, v32 = [G.f32_dev(x) for x in I.qkv(7, 1, 2, 2, 16, 16, 32)]
    assert code(lambda: va.flash_attention_split(q32, k32, v32, 0.1)) == _ffi.ERR_UNSUPPORTED
    small = torch.zeros(64, dtype=torch.uint8, device=G.dev())
    assert code(lambda: va.flash_attention_split(tq, tk, tv, 0.1, workspace=small)) == _ffi.ERR_WORKSPACE
    assert code(lambda: va.flash_attention_split(tq, tk, tv[:, :, :8], 0.1)) == _ffi.ERR_SHAPE
    assert code(lambda: va.flash_attention_split(tq, tk, tv, 0.0)) == _ffi.ERR_ARG
