"""CPU-side checks of the product: the C-ABI library loads and exports every symbol include/vsp_attn.h
declares, the host-side format helpers are bit-exact against the oracle, and argument validation that needs
no GPU behaves like the reference.  No compute kernel is launched here."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import _oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def ffi():
    from vesper_amd import _ffi
    return _ffi


def test_library_exports_every_declared_symbol(ffi):
    header = open(os.path.join(ROOT, "include", "vsp_attn.h")).read()
    declared = set(re.findall(r"\b(vsp_[a-z0-9_]+)\s*\(", header))
    declared -= {"vsp_tensor", "vsp_kv_cache"}
    assert declared == set(ffi.SYMBOLS), declared ^ set(ffi.SYMBOLS)
    for name in declared:
        assert hasattr(ffi.lib, name), name
    assert ffi.lib.vsp_attn_abi_version() == 2


def test_status_strings_are_the_reference_messages(ffi):
    assert ffi.lib.vsp_status_str(0) == b"ok"
    for code in (1, 2, 3, 4, 5):  # same numbering and text as the oracle's restatement of the reference throws
        assert ffi.lib.vsp_status_str(code) == O.orc.orc_strerror(code)
    assert ffi.lib.vsp_status_str(7) == O.orc.orc_strerror(7)


def test_host_bf16_f16_bit_exact(ffi):
    rng = np.random.default_rng(0)
    bits = rng.integers(0, 2**32, size=30000, dtype=np.uint64).astype(np.uint32)
    f = bits.view(np.float32)
    f = f[~np.isnan(f)]
    assert all(ffi.lib.vsp_f32_to_bf16(float(x)) == O.orc.orc_f32_to_bf16(float(x)) for x in f[:5000])
    with np.errstate(over="ignore"):
        want = f.astype(np.float16).view(np.uint16)
    got = np.array([ffi.lib.vsp_f32_to_f16(float(x)) for x in f[:20000]], np.uint16)
    assert np.array_equal(got, want[:20000])
    small = (rng.standard_normal(5000) * 1e-5).astype(np.float32)
    assert all(ffi.lib.vsp_f32_to_f16(float(x)) == int(np.float16(x).view(np.uint16)) for x in small)
    for h in list(range(0, 65536, 7)) + [0x0001, 0x03FF, 0x0400, 0x7BFF, 0x7C00, 0xFC00, 0x8001]:
        w = np.uint16(h).view(np.float16).astype(np.float32)
        if not np.isnan(w):
            assert np.float32(ffi.lib.vsp_f16_to_f32(h)).view(np.uint32) == w.view(np.uint32), hex(h)


def test_host_q8_0_matches_oracle(ffi):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal((40, 128)).astype(np.float32), np.zeros((2, 128), np.float32),
                        (rng.standard_normal((8, 128)) * 1e-6).astype(np.float32)])
    want_d, want_q = O.q8_0_quantize(x)
    d = np.empty_like(want_d)
    q = np.empty_like(want_q)
    ffi.lib.vsp_q8_0_quantize_row(x.ctypes.data, x.size, d.ctypes.data, q.ctypes.data)
    assert np.array_equal(d, want_d) and np.array_equal(q, want_q)
    back = np.empty_like(x)
    ffi.lib.vsp_q8_0_dequantize_row(d.ctypes.data, q.ctypes.data, x.size, back.ctypes.data)
    assert np.array_equal(back, O.q8_0_dequantize(want_d, want_q))


def test_slice_and_gqa_config_match_oracle(ffi):
    for dim in (0, 1, 16):
        for start in range(-20, 21):
            for T in (0, 1, 5):
                s, n = C.c_int64(), C.c_int64()
                ffi.lib.vsp_slice_bounds(dim, start, start + T, C.byref(s), C.byref(n))
                ws, wn = O.slice_bounds(dim, start, start + T, 1)
                assert (n.value, s.value if n.value else 0) == (wn, ws if wn else 0), (dim, start, T)
    hd, nr = C.c_int64(), C.c_int64()
    assert ffi.lib.vsp_gqa_config(64, 8, 2, C.byref(hd), C.byref(nr)) == 0 and (hd.value, nr.value) == (8, 4)
    assert ffi.lib.vsp_gqa_config(64, 8, 3, None, None) == ffi.ERR_GQA_HEADS
    assert ffi.lib.vsp_gqa_config(60, 8, 2, None, None) == ffi.ERR_GQA_EMBED


def test_plane_sizes_follow_the_documented_layouts(ffi):
    pb = ffi.lib.vsp_kv_plane_bytes
    assert pb(ffi.KV_F32, 2, 3, 100, 64, 0) == 2 * 3 * 100 * 64 * 4 and pb(ffi.KV_F32, 2, 3, 100, 64, 2) == 0
    assert pb(ffi.KV_BF16, 2, 3, 100, 64, 1) == 2 * 3 * 128 * 64 * 2  # S_pad = 128
    assert pb(ffi.KV_Q8_0, 1, 8, 65536, 128, 0) == 8 * 65536 * 128 and pb(ffi.KV_Q8_0, 1, 8, 65536, 128, 3) == 8 * 65536 * 4 * 2


def test_validation_that_needs_no_gpu(ffi):
    t = ffi.VspTensor()
    t.ndim, t.dtype = 3, ffi.BF16
    assert ffi.lib.vsp_attn_prefill(C.byref(t), C.byref(t), C.byref(t), C.byref(t), None, 1.0, 1, 0.0, 0, None) == ffi.ERR_NDIM
    assert ffi.lib.vsp_attn_prefill(None, None, None, None, None, 1.0, 1, 0.0, 0, None) == ffi.ERR_NULL
    q, k = ffi.VspTensor(), ffi.VspTensor()
    for d, shape in ((q, (1, 4, 8, 64)), (k, (1, 2, 9, 64))):
        d.ndim, d.dtype = 4, ffi.BF16
        for i, s in enumerate(shape):
            d.shape[i] = s
    assert ffi.lib.vsp_attn_prefill(C.byref(q), C.byref(k), C.byref(q), C.byref(q), None, 1.0, 1, 0.0, 0, None) == ffi.ERR_SHAPE
    assert ffi.lib.vsp_attn_prefill(C.byref(q), C.byref(k), C.byref(k), C.byref(q), None, 1.0, 1, 1.5, 0, None) == ffi.ERR_DROPOUT
    c = ffi.VspKVCache()
    c.format, c.B, c.Hkv, c.S_max, c.D = 7, 1, 1, 8, 64
    assert ffi.lib.vsp_kv_cache_reset(C.byref(c), None) == ffi.ERR_UNSUPPORTED
    c.format = ffi.KV_BF16
    assert ffi.lib.vsp_kv_cache_reset(C.byref(c), None) == ffi.ERR_NULL  # planes missing


def test_backward_validation_that_needs_no_gpu(ffi):
    # every rejection below is decided on the host before anything is launched (the pointers are never followed)
    def tens(shape, dtype, ptr=0x10000, strides=None):
        t = ffi.VspTensor()
        t.ndim, t.dtype, t.data = len(shape), dtype, ptr
        st = strides or [int(np.prod(shape[i + 1:])) for i in range(len(shape))]
        for i, (n, m) in enumerate(zip(shape, st)):
            t.shape[i], t.stride[i] = n, m
        return t

    def call(dout, q, k, v, out, lse, dq, dk, dv, ws=0x20000, ws_bytes=1 << 30):
        a = [C.byref(x) if x is not None else None for x in (dout, q, k, v, out, lse, dq, dk, dv)]
        return ffi.lib.vsp_attn_prefill_backward(*a, 0.125, 1, ws, ws_bytes, None)

    B, Hq, Hkv, N, D = 1, 4, 2, 8, 64
    q, k, lse = tens((B, Hq, N, D), ffi.BF16), tens((B, Hkv, N, D), ffi.BF16), tens((B, Hq, N), ffi.F32)
    assert ffi.lib.vsp_attn_backward_workspace_bytes(B, Hq, N) == 2 * B * Hq * N * 4
    assert ffi.lib.vsp_attn_backward_workspace_bytes(0, Hq, N) == 0
    assert call(q, None, k, k, q, lse, q, k, k) == ffi.ERR_NULL
    assert call(q, tens((B, Hq, N), ffi.BF16), k, k, q, lse, q, k, k) == ffi.ERR_NDIM
    k3 = tens((B, 3, N, D), ffi.BF16)
    assert call(q, q, k3, k3, q, lse, q, k3, k3) == ffi.ERR_SHAPE                       # 4 query heads over 3 kv heads
    assert call(q, q, k, tens((B, Hkv, N + 1, D), ffi.BF16), q, lse, q, k, k) == ffi.ERR_SHAPE
    assert call(q, q, k, tens((B, Hkv, N, D), ffi.F32), q, lse, q, k, k) == ffi.ERR_DTYPE  # one dtype for all
    assert call(q, q, k, k, q, tens((B, Hq, N), ffi.BF16), q, k, k) == ffi.ERR_DTYPE       # lse is fp32
    q32, k32 = tens((B, Hq, N, 32), ffi.BF16), tens((B, Hkv, N, 32), ffi.BF16)
    assert call(q32, q32, k32, k32, q32, lse, q32, k32, k32) == ffi.ERR_UNSUPPORTED        # head dim 32
    assert call(q, q, k, k, q, lse, q, k, k, ws=None) == ffi.ERR_WORKSPACE
    assert call(q, q, k, k, q, lse, q, k, k, ws_bytes=16) == ffi.ERR_WORKSPACE
    off = tens((B, Hq, N, D), ffi.BF16, ptr=0x10008)                                       # rows not 16-byte aligned
    assert call(q, off, k, k, q, lse, q, k, k) == ffi.ERR_ALIGN
    narrow = tens((B, Hq, N, D), ffi.BF16, strides=[Hq * N * 32, N * 32, 32, 1])           # rows overlap: stride < D
    assert call(q, narrow, k, k, q, lse, q, k, k) == ffi.ERR_STRIDE
    inner = tens((B, Hq, N, D), ffi.BF16, strides=[Hq * N * D * 2, N * D * 2, D * 2, 2])   # innermost stride != 1
    assert call(q, inner, k, k, q, lse, q, k, k) == ffi.ERR_STRIDE
    empty = tens((B, Hq, 0, D), ffi.BF16)
    ek, el = tens((B, Hkv, 0, D), ffi.BF16), tens((B, Hq, 0), ffi.F32)
    assert call(empty, empty, ek, ek, empty, el, empty, ek, ek) == 0                       # nothing to do


def test_cache_descriptor_validation_that_needs_no_gpu(ffi):
    # check_cache (behind every cache entry point) through vsp_kv_cache_reset, plus the argument checks of
    # vsp_kv_read and vsp_seq_lens_advance that come before any launch
    def cache(fmt=None, **kw):
        c = ffi.VspKVCache()
        c.format, c.B, c.Hkv, c.S_max, c.D = ffi.KV_BF16 if fmt is None else fmt, 2, 2, 256, 128
        c.k = c.v = c.k_scale = c.v_scale = 0x10000
        for key, val in kw.items():
            setattr(c, key, val)
        return c

    reset = lambda c: ffi.lib.vsp_kv_cache_reset(C.byref(c), None)
    assert reset(cache(len=257)) == ffi.ERR_ARG                      # length beyond the capacity
    assert reset(cache(D=96)) == ffi.ERR_UNSUPPORTED                 # bf16 / q8_0 planes exist for D 64 and 128
    assert reset(cache(fmt=ffi.KV_F32, D=6)) == ffi.ERR_UNSUPPORTED
    assert reset(cache(k=0x10008)) == ffi.ERR_ALIGN
    assert reset(cache(fmt=ffi.KV_Q8_0, k_scale=None)) == ffi.ERR_NULL
    paged = dict(page_table=0x30000, page_tokens=64, pages_per_seq=4, n_pages=10)
    assert reset(cache(fmt=ffi.KV_F32, **paged)) == ffi.ERR_UNSUPPORTED          # paging is for the compact formats
    assert reset(cache(**dict(paged, page_tokens=48))) == ffi.ERR_ARG            # pages are multiples of 64 tokens
    assert reset(cache(**dict(paged, pages_per_seq=3))) == ffi.ERR_ARG           # pages_per_seq * page_tokens == S_max
    assert reset(cache(page_tokens=64)) == ffi.ERR_ARG                           # paging fields without a table
    c = cache()
    assert ffi.lib.vsp_kv_read(C.byref(c), 200, 100, None, None, None) == ffi.ERR_ARG    # past the capacity
    assert ffi.lib.vsp_kv_read(C.byref(c), 0, 10, None, None, None) == ffi.ERR_NULL      # neither output given
    t = ffi.VspTensor()
    t.ndim, t.dtype = 4, ffi.BF16
    for i, n in enumerate((2, 2, 11, 128)):
        t.shape[i] = n
    assert ffi.lib.vsp_kv_read(C.byref(c), 0, 10, C.byref(t), None, None) == ffi.ERR_NUMEL
    assert ffi.lib.vsp_seq_lens_advance(None, None, 1, -1, 8, None) == ffi.ERR_ARG
    assert ffi.lib.vsp_seq_lens_advance(None, None, 1, 0, 8, None) == 0
    assert ffi.lib.vsp_seq_lens_advance(None, None, 1, 4, 8, None) == ffi.ERR_NULL


def test_adapter_host_side_checks():
    exe = os.path.join(ROOT, "tests", "cpp", "adapter_test")
    if not os.path.exists(exe):
        pytest.skip("tests/cpp/adapter_test not built (python -c 'import __graft_entry__ as g; g.build()')")
    r = subprocess.run([exe, "--cpu-only"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr


def test_product_never_touches_the_oracle():
    # the shipped package must not import, load or link anything under oracle/
    for dirpath, _, files in os.walk(os.path.join(ROOT, "vesper_amd")):
        if "build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".hpp", ".h")) or f == "Makefile":
                src = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "oracle" not in src.lower(), os.path.join(dirpath, f)
