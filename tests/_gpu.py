"""Helpers shared by the GPU parity tests: bit-level conversions between torch device tensors and the
numpy arrays the oracle consumes, and the tolerances the benchmark definition states."""
import numpy as np
import torch

import _oracle as O

# benchmark tolerances: bf16 max-abs 2e-2 / mean-abs 2e-3; fp32 1e-4 relative
BF16_MAX_ABS = 2e-2
BF16_MEAN_ABS = 2e-3
F32_REL = 1e-4


def dev():
    return torch.device("cuda:0")


def to_bf16_dev(x_f32):
    """numpy fp32 -> torch bf16 on the GPU using the REFERENCE's rounding (via the oracle), bit-exactly."""
    bits = O.f32_to_bf16(x_f32)
    return torch.from_numpy(bits.view(np.int16).copy()).to(dev()).view(torch.bfloat16)


def bf16_bits(t):
    """torch bf16 tensor -> numpy uint16 bits."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def bf16_to_np(t):
    return O.bf16_to_f32(bf16_bits(t))


def f32_dev(x):
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev())


def assert_bf16_close(got_f32, want_f32, what=""):
    err = np.abs(got_f32.astype(np.float64) - want_f32.astype(np.float64))
    assert np.isfinite(got_f32).all(), what
    assert err.max() <= BF16_MAX_ABS, f"{what}: max-abs {err.max():.4g} > {BF16_MAX_ABS}"
    assert err.mean() <= BF16_MEAN_ABS, f"{what}: mean-abs {err.mean():.4g} > {BF16_MEAN_ABS}"


def assert_bf16_close_wide_range(got_f32, want_f32, what=""):
    """The bf16 bar for outputs that are not of order one: max-abs 2e-2 plus one bf16 step of the expected value itself
    (storing an exact result of magnitude 4 as bf16 already moves it by up to 0.0156), elementwise; mean-abs as usual."""
    assert np.isfinite(got_f32).all(), what
    want = want_f32.astype(np.float64)
    err = np.abs(got_f32.astype(np.float64) - want)
    ulp = np.exp2(np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -126))) - 7)   # spacing of bf16 numbers at |want|
    over = err - (BF16_MAX_ABS + ulp)
    assert over.max() <= 0, f"{what}: error {err.flat[over.argmax()]:.4g} where 2e-2 + one bf16 step is {BF16_MAX_ABS + ulp.flat[over.argmax()]:.4g}"
    assert err.mean() <= BF16_MEAN_ABS, f"{what}: mean-abs {err.mean():.4g} > {BF16_MEAN_ABS}"


def assert_f32_close(got, want, what=""):
    """1e-4 relative, measured against the magnitude of the reference output (elementwise relative error
    is meaningless where the output crosses zero)."""
    assert np.isfinite(got).all(), what
    denom = max(float(np.abs(want).max()), 1e-30)
    rel = np.abs(got.astype(np.float64) - want.astype(np.float64)).max() / denom
    assert rel <= F32_REL, f"{what}: relative error {rel:.3g} > {F32_REL}"
