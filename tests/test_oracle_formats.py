"""bf16 / fp16 / Q8_0 restatements against independent implementations and closed forms."""
import numpy as np
import torch

import _oracle as O


def test_bf16_rne_against_torch_and_integer_model():
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[np.isfinite(f)]
    got = O.f32_to_bf16(f)
    # independent #1: torch's conversion
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    big = np.abs(f) > 3.38e38  # the reference has no overflow special-case, nor does RNE need one: carries to inf
    assert np.array_equal(got[~big], want[~big])
    # independent #2: exact integer arithmetic (ties to even on the dropped 16 bits)
    b = f.view(np.uint32).astype(np.uint64)
    lo, hi = b & 0xFFFF, b >> 16
    up = (lo > 0x8000) | ((lo == 0x8000) & ((hi & 1) == 1))
    assert np.array_equal(got, (hi + up).astype(np.uint16))
    assert np.array_equal(O.bf16_to_f32(got).view(np.uint32), got.astype(np.uint32) << 16)


def test_bf16_known_values():
    cases = {1.0: 0x3F80, -2.0: 0xC000, 0.0: 0x0000, 1.00390625: 0x3F80, 1.01171875: 0x3F82, 3.0e38: 0x7F62}
    for x, want in cases.items():
        assert O.orc.orc_f32_to_bf16(x) == want, x


def test_f16_against_numpy():
    rng = np.random.default_rng(1)
    bits = rng.integers(0, 2**32, size=100000, dtype=np.uint64).astype(np.uint32)
    f = np.concatenate([bits.view(np.float32), rng.standard_normal(50000).astype(np.float32) * 1e-5,
                        np.float32([0, -0.0, 65504, 65519.99, 65520, 1e-8, 6e-8, 5.96e-8, 2.98e-8, 6.1e-5, np.inf, -np.inf])])
    f = f[~np.isnan(f)]
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([O.orc.orc_f32_to_f16(float(x)) for x in f[:40000]], np.uint16)
    assert np.array_equal(got, want[:40000])
    allh = np.arange(65536, dtype=np.uint16)
    back = np.array([O.orc.orc_f16_to_f32(int(h)) for h in allh], np.float32)
    want_back = allh.view(np.float16).astype(np.float32)
    ok = ~np.isnan(want_back)
    assert np.array_equal(back[ok].view(np.uint32), want_back[ok].view(np.uint32))


def test_q8_0_closed_form_known_answers():
    # block of 32 with amax 127 -> d = 1, q_i = round(x_i)
    x = np.linspace(-127, 127, 32, dtype=np.float32)
    d, qs = O.q8_0_quantize(x[None])
    assert d[0, 0] == 0x3C00 and np.array_equal(qs[0], np.round(x).astype(np.int8))
    # all-zero block -> d = 0, qs = 0
    d, qs = O.q8_0_quantize(np.zeros((1, 32), np.float32))
    assert d[0, 0] == 0 and not qs.any()
    # roundf is half-away-from-zero: with amax = 127, +-0.5 -> +-1, 2.5 -> 3
    x = np.zeros(32, np.float32)
    x[:5] = [127, 0.5, -0.5, 2.5, -1.5]
    _, qs = O.q8_0_quantize(x[None])
    assert list(qs[0, :5]) == [127, 1, -1, 3, -2]
    # two blocks are independent; the max element always maps to +-127
    rng = np.random.default_rng(2)
    x = rng.standard_normal((50, 128)).astype(np.float32)
    d, qs = O.q8_0_quantize(x)
    blocks = x.reshape(50, 4, 32)
    amax = np.abs(blocks).max(-1)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16).view(np.uint16))
    assert np.array_equal(np.abs(qs.reshape(50, 4, 32)).max(-1), np.full((50, 4), 127))
    idv = np.float32(1) / (amax / np.float32(127))
    want = np.sign(blocks) * np.floor(np.abs(blocks * idv[..., None]) + np.float32(0.5))
    assert np.array_equal(qs.reshape(50, 4, 32), want.astype(np.int8))
    # dequant = q * f16(d); error bound half a step
    xd = O.q8_0_dequantize(d, qs)
    step = d.view(np.float16).astype(np.float32)
    assert np.array_equal(xd.reshape(50, 4, 32), qs.reshape(50, 4, 32).astype(np.float32) * step[..., None])
    assert (np.abs(xd - x).reshape(50, 4, 32) <= 0.51 * step[..., None] + 1e-3 * amax[..., None]).all()
