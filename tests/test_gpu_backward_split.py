"""fp32 attention backward through the bf16 matrix cores (vsp_attn_prefill_backward_split: operands as two bf16 terms,
three MFMAs per product, P and dS split after the fp32 algebra, fp32 gradients) on the GPU, against the oracle (bit-exact
to the compiled reference's flash_attention_backward), the reference-written fixture and the float64 closed form.  The
reference's bar is 1e-4 of the gradient's magnitude; the tests hold the path to TIGHT so that a lost term cannot hide
inside that bar (a dropped hi*lo term costs ~2^-9 of a product)."""
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
TIGHT = 4e-5


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


def _close(got, want, what, tol=TIGHT, floor=1e-30):
    got = got.cpu().numpy() if hasattr(got, "cpu") else got
    assert np.isfinite(got).all(), what
    rel = np.abs(got.astype(np.float64) - want.astype(np.float64)).max() / max(float(np.abs(want).max()), floor)
    assert rel <= tol, f"{what}: relative error {rel:.3g} > {tol}"


def _grads(va, q, k, v, dout, scale, causal):
    """Forward in exact fp32 (the fp32-MFMA kernel), backward through the split path."""
    tq, tk, tv, td = G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), G.f32_dev(dout)
    out, lse = va.flash_attention(tq, tk, tv, scale, causal, return_lse=True)
    return va.flash_attention_backward_split(td, tq, tk, tv, out, lse, scale, causal)


def test_fixture_written_from_the_reference(va):
    z = np.load(os.path.join(GOLD, "flash_backward.npz"), allow_pickle=False)
    for tag in ("r70", "nc33", "d128"):   # the fixture's head_dim 32 case belongs to the fp32-MFMA path
        B, H, N, D, causal, seed = [int(x) for x in z[tag + "_meta"]]
        q, k, v = I.qkv(seed, B, H, H, N, N, D)
        dout = I.normal(seed + 5, (B, H, N, D))
        dq, dk, dv = _grads(va, q, k, v, dout, float(np.float32(1.0 / np.sqrt(D))), bool(causal))
        _close(dq, z[tag + "_dq"], tag + " dq")
        _close(dk, z[tag + "_dk"], tag + " dk")
        _close(dv, z[tag + "_dv"], tag + " dv")


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", [(1, 4, 2, 100, 64, True), (2, 8, 2, 257, 128, True), (1, 4, 4, 64, 128, False),
                                                 (1, 6, 1, 33, 64, True), (1, 2, 1, 129, 128, False), (1, 8, 8, 1, 64, True),
                                                 (1, 4, 1, 512, 128, True), (1, 4, 2, 200, 64, False)])
def test_gqa_against_oracle_and_closed_form(va, B, Hq, Hkv, N, D, causal):
    q, k, v = I.qkv(900 + N, B, Hq, Hkv, N, N, D)
    dout = I.normal(905 + N, (B, Hq, N, D))
    scale = float(np.float32(1.0 / np.sqrt(D)))
    n = Hq // Hkv
    kr, vr = O.repeat_kv(k, n), O.repeat_kv(v, n)
    out, lse = O.flash_attention(q, kr, vr, scale, causal, return_lse=True)
    wq, wk, wv = O.flash_attention_backward(dout, q, kr, vr, out, lse, scale, causal)
    wk = wk.reshape(B, Hkv, n, N, D).sum(2)
    wv = wv.reshape(B, Hkv, n, N, D).sum(2)
    dq, dk, dv = _grads(va, q, k, v, dout, scale, causal)
    # a single token has dq = dk = 0 in exact arithmetic (P = 1, dP = Di): measured against the scale of dO V there
    floor = float(np.abs(np.einsum("bhnd,bhnd->bhn", dout, vr)).max()) if N == 1 else 1e-30
    _close(dq, wq, "dq", floor=floor)
    _close(dk, wk, "dk", floor=floor)
    _close(dv, wv, "dv")
    cq, ck, cv = closed_form_grads(dout, q, kr, vr, scale, causal)
    _close(dq, cq, "dq closed form", floor=floor)
    _close(dk, ck.reshape(B, Hkv, n, N, D).sum(2), "dk closed form", floor=floor)
    _close(dv, cv.reshape(B, Hkv, n, N, D).sum(2), "dv closed form")


def test_larger_magnitudes_and_scale(va):
    # scores of order 10: P spans many orders of magnitude and the split of Q and K carries the accuracy of the exponent
    B, Hq, Hkv, N, D = 1, 4, 2, 160, 128
    q, k, v = I.qkv(950, B, Hq, Hkv, N, N, D)
    q = q * np.float32(1.7)
    dout = I.normal(955, (B, Hq, N, D)) * np.float32(3.0)
    scale = 0.21
    kr, vr = O.repeat_kv(k, 2), O.repeat_kv(v, 2)
    cq, ck, cv = closed_form_grads(dout, q, kr, vr, scale, True)
    dq, dk, dv = _grads(va, q, k, v, dout, scale, True)
    _close(dq, cq, "dq", 1e-4)
    _close(dk, ck.reshape(B, Hkv, 2, N, D).sum(2), "dk", 1e-4)
    _close(dv, cv.reshape(B, Hkv, 2, N, D).sum(2), "dv", 1e-4)


def test_strided_operands_and_determinism(va):
    # [B, N, H, D] storage viewed as [B, H, N, D]: strides of every operand and of every gradient are honoured
    B, Hq, Hkv, N, D = 2, 4, 2, 70, 64
    q, k, v = I.qkv(960, B, Hq, Hkv, N, N, D)
    dout = I.normal(965, (B, Hq, N, D))
    dense = [G.f32_dev(x) for x in (dout, q, k, v)]
    strided = [t.transpose(1, 2).contiguous().transpose(1, 2) for t in dense]
    assert not strided[0].is_contiguous()
    out, lse = va.flash_attention(dense[1], dense[2], dense[3], 0.125, True, return_lse=True)
    want = va.flash_attention_backward_split(*dense, out, lse, 0.125, True)
    got = va.flash_attention_backward_split(*strided, out.transpose(1, 2).contiguous().transpose(1, 2), lse, 0.125, True)
    for g, w in zip(got, want):
        assert g.stride() != w.stride() and torch.equal(g, w)
    again = va.flash_attention_backward_split(*dense, out, lse, 0.125, True)
    for a, w in zip(again, want):
        assert torch.equal(a, w)          # no atomics: bitwise reproducible


def test_config2_shape_against_the_fp32_path(va):
    # benchmark config 2's shape (B4, 32/8 heads, D128, N2048) with fp32 tensors, one batch row: the split path against
    # the library's own fp32-MFMA backward (itself held to the oracle at 1e-4 on small shapes)
    B, Hq, Hkv, N, D = 1, 32, 8, 2048, 128
    g = torch.Generator(device="cuda").manual_seed(23)
    mk = lambda h: torch.randn(B, h, N, D, device=G.dev(), generator=g) * 0.5
    q, k, v, dout = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
    scale = 1.0 / np.sqrt(D)
    out, lse = va.flash_attention(q, k, v, scale, True, return_lse=True)
    want = va.flash_attention_backward(dout, q, k, v, out, lse, scale, True)
    got = va.flash_attention_backward_split(dout, q, k, v, out, lse, scale, True)
    for gt, w, name in zip(got, want, ("dq", "dk", "dv")):
        _close(gt, w.cpu().numpy(), name, 1e-4)


def test_argument_errors(va):
    from vesper_amd import _ffi
    d = G.dev()

    def code(fn):
        with pytest.raises(va.VspError) as e:
            fn()
        return e.value.status

    q = torch.zeros(1, 4, 8, 64, device=d)
    k = torch.zeros(1, 2, 8, 64, device=d)
    lse = torch.zeros(1, 4, 8, device=d)
    b = lambda t: t.to(torch.bfloat16)
    assert code(lambda: va.flash_attention_backward_split(b(q), b(q), b(k), b(k), b(q), lse, 0.1)) == _ffi.ERR_UNSUPPORTED
    z = torch.zeros(1, 2, 8, 32, device=d)   # head_dim 32: the fp32-MFMA path has it, this one does not
    assert code(lambda: va.flash_attention_backward_split(z, z, z, z, z, torch.zeros(1, 2, 8, device=d), 0.1)) == _ffi.ERR_UNSUPPORTED
    q3 = torch.zeros(1, 3, 8, 64, device=d)
    assert code(lambda: va.flash_attention_backward_split(q3, q3, k, k, q3, torch.zeros(1, 3, 8, device=d), 0.1)) == _ffi.ERR_SHAPE
    small = torch.zeros(64, dtype=torch.uint8, device=d)
    assert code(lambda: va.flash_attention_backward_split(q, q, k, k, q, lse, 0.1, workspace=small)) == _ffi.ERR_WORKSPACE
    need = _ffi.lib.vsp_attn_backward_split_workspace_bytes(1, 4, 2, 8, 64)
    assert need == 2 * 4 * 8 * 4 + 4 * (4 + 2) * 8 * 64 * 2
    dq, dk, dv = va.flash_attention_backward_split(q, q, k, k, q, lse, 0.1)
    assert dq.shape == q.shape and dk.shape == k.shape and not dq.any() and not dv.any()
