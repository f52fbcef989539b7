"""ctypes bindings of the checker libraries (TEST INFRASTRUCTURE).

`orc`  : oracle/libvsp_oracle.so  - this repo's C restatement of the reference CPU path.
`ref`  : oracle/_ref/libvesper_ref.so - the real reference compiled CPU-only (optional:
         it is built in the authoring container and travels as a binary; tests that
         need it skip when it is absent).

Nothing under vesper_amd/ imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
_ORC_PATH = os.path.join(ORACLE_DIR, "libvsp_oracle.so")
_REF_PATH = os.path.join(ORACLE_DIR, "_ref", "libvesper_ref.so")

f32p = C.POINTER(C.c_float)
i64p = C.POINTER(C.c_int64)
u16p = C.POINTER(C.c_uint16)
i8p = C.POINTER(C.c_int8)
i64 = C.c_int64


def _p(a, t=f32p):
    return a.ctypes.data_as(t)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _load_oracle():
    src = os.path.join(ORACLE_DIR, "vsp_oracle.c")
    if (not os.path.exists(_ORC_PATH)) or os.path.getmtime(_ORC_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"], stdout=subprocess.DEVNULL)
    L = C.CDLL(_ORC_PATH)
    L.orc_strerror.restype = C.c_char_p
    L.orc_strerror.argtypes = [C.c_int]
    L.orc_flash_attention_check.argtypes = [C.c_int, i64p, C.c_int, i64p, C.c_int, i64p,
                                            C.c_int, C.c_int, C.c_int, C.c_float]
    L.orc_flash_attention_f32.argtypes = [f32p] * 5 + [i64] * 4 + [C.c_float, C.c_int]
    L.orc_flash_attention_f32.restype = None
    L.orc_repeat_kv_f32.argtypes = [f32p, f32p] + [i64] * 5
    L.orc_repeat_kv_f32.restype = None
    L.orc_sdpa_matmul_f32.argtypes = [f32p, f32p, i64p, f32p, i64p, f32p] + [i64] * 6 + [C.c_int]
    L.orc_sdpa_f32.argtypes = [f32p] * 4 + [i64] * 5 + [C.c_int]
    L.orc_gqa_attention_f32.argtypes = [f32p, f32p, i64p, f32p, i64p, f32p] + [i64] * 6 + [C.c_int]
    L.orc_gqa_config.argtypes = [i64, i64, i64, i64p, i64p]
    L.orc_slice_bounds.argtypes = [i64, C.c_int, i64, C.c_int, i64, C.c_int, i64, i64p, i64p]
    L.orc_kv_new.restype = C.c_void_p
    L.orc_kv_new.argtypes = [i64] * 4
    L.orc_kv_free.argtypes = [C.c_void_p]
    L.orc_kv_free.restype = None
    L.orc_kv_reset.argtypes = [C.c_void_p]
    L.orc_kv_reset.restype = None
    L.orc_kv_update.argtypes = [C.c_void_p, f32p, f32p] + [i64] * 5 + [i64p]
    L.orc_f32_to_bf16.argtypes = [C.c_float]
    L.orc_f32_to_bf16.restype = C.c_uint16
    L.orc_bf16_to_f32.argtypes = [C.c_uint16]
    L.orc_bf16_to_f32.restype = C.c_float
    L.orc_f32_to_bf16_array.argtypes = [f32p, u16p, i64]
    L.orc_f32_to_bf16_array.restype = None
    L.orc_bf16_to_f32_array.argtypes = [u16p, f32p, i64]
    L.orc_bf16_to_f32_array.restype = None
    L.orc_f32_to_f16.argtypes = [C.c_float]
    L.orc_f32_to_f16.restype = C.c_uint16
    L.orc_f16_to_f32.argtypes = [C.c_uint16]
    L.orc_f16_to_f32.restype = C.c_float
    L.orc_q8_0_quantize_row.argtypes = [f32p, i64, u16p, i8p]
    L.orc_q8_0_quantize_row.restype = None
    L.orc_q8_0_dequantize_row.argtypes = [u16p, i8p, i64, f32p]
    L.orc_q8_0_dequantize_row.restype = None
    L.orc_flash_attention_backward_f32.argtypes = [f32p] * 9 + [i64] * 4 + [C.c_float, C.c_int]
    L.orc_flash_attention_backward_f32.restype = None
    L.orc_rope_angles.argtypes = [C.c_int, C.c_int, C.c_int, C.c_float, f32p]
    L.orc_rope_angles.restype = None
    L.orc_rope_apply_f32.argtypes = [f32p] + [i64] * 4 + [f32p, f32p]
    L.orc_linear_f32.argtypes = [f32p, f32p, f32p, f32p, i64, i64, i64]
    L.orc_linear_f32.restype = None
    L.orc_rope_apply_f32.restype = None
    return L


orc = _load_oracle()


class OrcKVStruct(C.Structure):
    _fields_ = [("k", f32p), ("v", f32p), ("B", i64), ("H", i64), ("S_max", i64), ("D", i64),
                ("current_len", i64)]


class OracleError(RuntimeError):
    def __init__(self, code):
        self.code = code
        super().__init__(orc.orc_strerror(code).decode())


def _chk(code):
    if code != 0:
        raise OracleError(code)


# ---- attention ------------------------------------------------------------------------------

def flash_attention(q, k, v, scale, causal=True, return_lse=False):
    """ops::flash_attention on contiguous fp32 [B,H,N,D] (validation included)."""
    for t in (q, k, v):
        pass
    shp = [np.asarray(t.shape, dtype=np.int64) for t in (q, k, v)]
    _chk(orc.orc_flash_attention_check(q.ndim, _p(shp[0], i64p), k.ndim, _p(shp[1], i64p),
                                       v.ndim, _p(shp[2], i64p), 0, 0, 0, 0.0))
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, N, D = q.shape
    out = np.empty_like(q)
    lse = np.empty((B, H, N), np.float32)
    orc.orc_flash_attention_f32(_p(q), _p(k), _p(v), _p(out), _p(lse), B, H, N, D, scale, int(causal))
    return (out, lse) if return_lse else out


def repeat_kv(x, n_rep):
    if n_rep == 1:
        return x
    x = _f32(x)
    B, H, S, D = x.shape
    out = np.empty((B, H * n_rep, S, D), np.float32)
    orc.orc_repeat_kv_f32(_p(x), _p(out), B, H, S, D, n_rep)
    return out


def _strides_elems(a):
    return np.asarray([s // a.itemsize for s in a.strides], dtype=np.int64)


def sdpa(q, k, v, causal=False):
    """functional::scaled_dot_product_attention, contiguous MHA inputs."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, T, D = q.shape
    L = k.shape[2]
    out = np.empty_like(q)
    _chk(orc.orc_sdpa_f32(_p(q), _p(k), _p(v), _p(out), B, H, T, L, D, int(causal)))
    return out


def sdpa_matmul(q, k, v, causal=False, n_rep=1):
    """The non-flash branch regardless of T; k, v may be strided fp32 views [B,H/n_rep,L,D]."""
    q = _f32(q)
    assert k.dtype == np.float32 and v.dtype == np.float32
    B, H, T, D = q.shape
    L = k.shape[2]
    ks, vs = _strides_elems(k), _strides_elems(v)
    out = np.empty_like(q)
    _chk(orc.orc_sdpa_matmul_f32(_p(q), _p(k), _p(ks, i64p), _p(v), _p(vs, i64p), _p(out),
                                 B, H, T, L, D, n_rep, int(causal)))
    return out


def gqa_attention(q, k, v, causal):
    """repeat_kv(k), repeat_kv(v) -> scaled_dot_product_attention; k, v fp32 [B,Hkv,L,D], may be views."""
    q = _f32(q)
    assert k.dtype == np.float32 and v.dtype == np.float32
    B, Hq, T, D = q.shape
    Hkv, L = k.shape[1], k.shape[2]
    assert Hq % Hkv == 0
    ks, vs = _strides_elems(k), _strides_elems(v)
    out = np.empty_like(q)
    _chk(orc.orc_gqa_attention_f32(_p(q), _p(k), _p(ks, i64p), _p(v), _p(vs, i64p), _p(out),
                                   B, Hq, T, L, D, Hq // Hkv, int(causal)))
    return out


def gqa_config(embed_dim, num_heads, num_kv_heads):
    hd, nr = i64(0), i64(0)
    _chk(orc.orc_gqa_config(embed_dim, num_heads, num_kv_heads, C.byref(hd), C.byref(nr)))
    return hd.value, nr.value


def slice_bounds(dim, start=None, stop=None, step=None):
    s, n = i64(0), i64(0)
    _chk(orc.orc_slice_bounds(dim, start is not None, start or 0, stop is not None, stop or 0,
                              step is not None, step or 0, C.byref(s), C.byref(n)))
    return s.value, n.value


class KVCache:
    """nn::KVCache / nn::GQAKVCache model (fp32 [B,H,S_max,D], one length)."""

    def __init__(self, B, H, S_max, D):
        self._h = orc.orc_kv_new(B, H, S_max, D)
        self.shape = (B, H, S_max, D)

    def __del__(self):
        if getattr(self, "_h", None):
            orc.orc_kv_free(self._h)
            self._h = None

    def _st(self):
        return C.cast(self._h, C.POINTER(OrcKVStruct)).contents

    def current_seq_len(self):
        return int(self._st().current_len)

    def get_max_seq_len(self):
        return self.shape[2]

    def reset(self):
        orc.orc_kv_reset(self._h)

    def planes(self):
        n = int(np.prod(self.shape))
        st = self._st()
        k = np.ctypeslib.as_array(st.k, shape=(n,)).reshape(self.shape)
        v = np.ctypeslib.as_array(st.v, shape=(n,)).reshape(self.shape)
        return k, v

    def update(self, new_k, new_v, start_pos):
        new_k, new_v = _f32(new_k), _f32(new_v)
        nB, nH, T, nD = new_k.shape
        meta = np.zeros(9, np.int64)
        _chk(orc.orc_kv_update(self._h, _p(new_k), _p(new_v), nB, nH, T, nD, start_pos, _p(meta, i64p)))
        k, v = self.planes()
        L = int(meta[2])
        self.last_view_meta = meta
        return k[:, :, :L, :], v[:, :, :L, :]


# ---- formats --------------------------------------------------------------------------------

def f32_to_bf16(a):
    a = _f32(a)
    out = np.empty(a.shape, np.uint16)
    orc.orc_f32_to_bf16_array(_p(a), _p(out, u16p), a.size)
    return out


def bf16_to_f32(a):
    a = np.ascontiguousarray(a, dtype=np.uint16)
    out = np.empty(a.shape, np.float32)
    orc.orc_bf16_to_f32_array(_p(a, u16p), _p(out), a.size)
    return out


def bf16_round(a):
    """fp32 -> bf16 (reference RNE) -> fp32."""
    return bf16_to_f32(f32_to_bf16(a))


def q8_0_quantize(x):
    """x fp32 [..., D] with D % 32 == 0 -> (d uint16 [..., D/32], qs int8 [..., D])."""
    x = _f32(x)
    assert x.shape[-1] % 32 == 0
    d = np.empty(x.shape[:-1] + (x.shape[-1] // 32,), np.uint16)
    qs = np.empty(x.shape, np.int8)
    orc.orc_q8_0_quantize_row(_p(x), x.size, _p(d, u16p), _p(qs, i8p))
    return d, qs


def q8_0_dequantize(d, qs):
    d = np.ascontiguousarray(d, np.uint16)
    qs = np.ascontiguousarray(qs, np.int8)
    out = np.empty(qs.shape, np.float32)
    orc.orc_q8_0_dequantize_row(_p(d, u16p), _p(qs, i8p), qs.size, _p(out))
    return out


def flash_attention_backward(dout, q, k, v, out, lse, scale, causal=True):
    """Gradients (dq, dk, dv) of the reference's flash attention, all heads equal (no GQA: repeat first)."""
    dout, q, k, v, out, lse = [_f32(x) for x in (dout, q, k, v, out, lse)]
    B, H, N, D = q.shape
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    orc.orc_flash_attention_backward_f32(_p(dout), _p(q), _p(k), _p(v), _p(out), _p(lse), _p(dq), _p(dk), _p(dv),
                                         B, H, N, D, scale, int(causal))
    return dq, dk, dv


def rope_angles(seq_len, head_dim, start_pos=0, theta=10000.0):
    out = np.empty((seq_len, head_dim // 2), np.float32)
    orc.orc_rope_angles(seq_len, head_dim, start_pos, theta, _p(out))
    return out


def rope_apply(x, angles):
    x, angles = _f32(x), _f32(angles)
    B, H, S, D = x.shape
    assert angles.shape == (S, D // 2)
    out = np.empty_like(x)
    orc.orc_rope_apply_f32(_p(x), B, H, S, D, _p(angles), _p(out))
    return out


def linear(x, w, bias=None):
    """Linear::forward on a [..., K] activation: x w^T + bias, the modules' output projection."""
    x, w = _f32(x), _f32(w)
    K, N = x.shape[-1], w.shape[0]
    assert w.shape == (N, K)
    M = x.size // K
    y = np.empty(x.shape[:-1] + (N,), np.float32)
    b = _f32(bias) if bias is not None else None
    orc.orc_linear_f32(_p(x), _p(w), _p(b) if b is not None else None, _p(y), M, K, N)
    return y


# ---- the compiled reference (optional) ----------------------------------------------------

def _load_ref():
    if not os.path.exists(_REF_PATH):
        return None
    L = C.CDLL(_REF_PATH)
    L.vref_last_error.restype = C.c_char_p
    L.vref_flash_attention.argtypes = [f32p] * 5 + [i64] * 4 + [C.c_float, C.c_int]
    L.vref_flash_attention_shapes.argtypes = [i64p, i64p, i64p, C.c_int, C.c_int, C.c_int, C.c_float]
    L.vref_repeat_kv.argtypes = [f32p, f32p] + [i64] * 5
    L.vref_sdpa.argtypes = [f32p] * 4 + [i64] * 5 + [C.c_int]
    L.vref_kvcache_new.restype = C.c_void_p
    L.vref_kvcache_new.argtypes = [C.c_int] * 4
    L.vref_kvcache_free.argtypes = [C.c_void_p]
    L.vref_kvcache_free.restype = None
    L.vref_kvcache_len.argtypes = [C.c_void_p]
    L.vref_kvcache_max_len.argtypes = [C.c_void_p]
    L.vref_kvcache_reset.argtypes = [C.c_void_p]
    L.vref_kvcache_update.argtypes = [C.c_void_p, f32p, f32p] + [i64] * 4 + [C.c_int, f32p, f32p, i64p]
    L.vref_gqacache_new.restype = C.c_void_p
    L.vref_gqacache_new.argtypes = [i64] * 4
    L.vref_gqacache_free.argtypes = [C.c_void_p]
    L.vref_gqacache_free.restype = None
    L.vref_gqacache_len.argtypes = [C.c_void_p]
    L.vref_gqacache_len.restype = i64
    L.vref_gqacache_reset.argtypes = [C.c_void_p]
    L.vref_gqacache_update.argtypes = [C.c_void_p, f32p, f32p] + [i64] * 5 + [f32p, f32p]
    L.vref_gqa_core.argtypes = [C.c_void_p, f32p, f32p, f32p] + [i64] * 5 + [C.c_int, C.c_int, f32p]
    L.vref_gqa_ctor.argtypes = [i64, i64, i64, i64p, i64p]
    if hasattr(L, "vref_flash_attention_backward"):
        L.vref_flash_attention_backward.argtypes = [f32p] * 9 + [i64] * 4 + [C.c_float, C.c_int]
    if hasattr(L, "vref_rope_frequencies"):
        L.vref_rope_frequencies.argtypes = [C.c_int, C.c_int, C.c_int, C.c_float, f32p]
        L.vref_apply_rotary_emb.argtypes = [f32p] + [i64] * 4 + [f32p, f32p]
        L.vref_gqa_rope_core.argtypes = [C.c_void_p, f32p, f32p, f32p] + [i64] * 5 + [C.c_int, C.c_float, f32p, f32p]
    if hasattr(L, "vref_linear"):
        L.vref_linear.argtypes = [f32p, f32p, f32p, f32p] + [i64] * 4
    L.vref_f32_to_bf16.argtypes = [C.c_float]
    L.vref_f32_to_bf16.restype = C.c_uint16
    L.vref_bf16_to_f32.argtypes = [C.c_uint16]
    L.vref_bf16_to_f32.restype = C.c_float
    return L


ref = _load_ref()


class RefError(RuntimeError):
    pass


def _rchk(code):
    if code != 0:
        raise RefError(ref.vref_last_error().decode())


def ref_flash_attention(q, k, v, scale, causal=True):
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, N, D = q.shape
    out = np.empty_like(q)
    lse = np.empty((B, H, N), np.float32)
    _rchk(ref.vref_flash_attention(_p(q), _p(k), _p(v), _p(out), _p(lse), B, H, N, D, scale, int(causal)))
    return out, lse


def ref_flash_attention_shapes(qs, ks, vs, dropout_p=0.0):
    a = [np.asarray(s, dtype=np.int64) for s in (qs, ks, vs)]
    _rchk(ref.vref_flash_attention_shapes(_p(a[0], i64p), _p(a[1], i64p), _p(a[2], i64p),
                                          len(qs), len(ks), len(vs), dropout_p))


def ref_repeat_kv(x, n_rep):
    x = _f32(x)
    B, H, S, D = x.shape
    out = np.empty((B, H * n_rep, S, D), np.float32)
    _rchk(ref.vref_repeat_kv(_p(x), _p(out), B, H, S, D, n_rep))
    return out


def ref_sdpa(q, k, v, causal=False):
    q, k, v = _f32(q), _f32(k), _f32(v)
    B, H, T, D = q.shape
    L = k.shape[2]
    out = np.empty_like(q)
    _rchk(ref.vref_sdpa(_p(q), _p(k), _p(v), _p(out), B, H, T, L, D, int(causal)))
    return out


class RefKVCache:
    def __init__(self, B, H, S_max, D, gqa=False):
        self.gqa = gqa
        self.shape = (B, H, S_max, D)
        self._h = (ref.vref_gqacache_new if gqa else ref.vref_kvcache_new)(B, H, S_max, D)
        if not self._h:
            raise RefError(ref.vref_last_error().decode())

    def __del__(self):
        if getattr(self, "_h", None):
            (ref.vref_gqacache_free if self.gqa else ref.vref_kvcache_free)(self._h)
            self._h = None

    def current_seq_len(self):
        return int((ref.vref_gqacache_len if self.gqa else ref.vref_kvcache_len)(self._h))

    def reset(self):
        _rchk((ref.vref_gqacache_reset if self.gqa else ref.vref_kvcache_reset)(self._h))

    def update(self, new_k, new_v, start_pos):
        new_k, new_v = _f32(new_k), _f32(new_v)
        nB, nH, T, nD = new_k.shape
        B, H, S_max, D = self.shape
        kbuf = np.zeros((B, H, S_max, D), np.float32)
        vbuf = np.zeros((B, H, S_max, D), np.float32)
        meta = np.zeros(9, np.int64)
        if self.gqa:
            _rchk(ref.vref_gqacache_update(self._h, _p(new_k), _p(new_v), nB, nH, T, nD, start_pos,
                                           _p(kbuf), _p(vbuf)))
            L = self.current_seq_len()
        else:
            _rchk(ref.vref_kvcache_update(self._h, _p(new_k), _p(new_v), nB, nH, T, nD, start_pos,
                                          _p(kbuf), _p(vbuf), _p(meta, i64p)))
            L = int(meta[2])
            self.last_view_meta = meta
        n = B * H * L * D
        return (kbuf.reshape(-1)[:n].reshape(B, H, L, D).copy(),
                vbuf.reshape(-1)[:n].reshape(B, H, L, D).copy())

    def gqa_core(self, q, new_k, new_v, start_pos, make_contiguous=True):
        assert not self.gqa
        q, new_k, new_v = _f32(q), _f32(new_k), _f32(new_v)
        B, Hq, T, D = q.shape
        Hkv = new_k.shape[1]
        out = np.empty_like(q)
        _rchk(ref.vref_gqa_core(self._h, _p(q), _p(new_k), _p(new_v), B, Hq, Hkv, T, D, start_pos,
                                int(make_contiguous), _p(out)))
        return out


    def gqa_rope_core(self, q, new_k, new_v, start_pos, theta=10000.0):
        """RoPE(q, k) at start_pos -> update -> repeat_kv -> attention; returns (rotated q, output)."""
        assert not self.gqa
        q, new_k, new_v = _f32(q), _f32(new_k), _f32(new_v)
        B, Hq, T, D = q.shape
        Hkv = new_k.shape[1]
        q_rot, out = np.empty_like(q), np.empty_like(q)
        _rchk(ref.vref_gqa_rope_core(self._h, _p(q), _p(new_k), _p(new_v), B, Hq, Hkv, T, D, start_pos,
                                     theta, _p(q_rot), _p(out)))
        return q_rot, out


def ref_flash_attention_backward(dout, q, k, v, out, lse, scale, causal=True):
    dout, q, k, v, out, lse = [_f32(x) for x in (dout, q, k, v, out, lse)]
    B, H, N, D = q.shape
    dq, dk, dv = np.empty_like(q), np.empty_like(q), np.empty_like(q)
    _rchk(ref.vref_flash_attention_backward(_p(dout), _p(q), _p(k), _p(v), _p(out), _p(lse), _p(dq), _p(dk), _p(dv),
                                            B, H, N, D, scale, int(causal)))
    return dq, dk, dv


def ref_rope_angles(seq_len, head_dim, start_pos=0, theta=10000.0):
    out = np.empty((seq_len, head_dim // 2), np.float32)
    _rchk(ref.vref_rope_frequencies(seq_len, head_dim, start_pos, theta, _p(out)))
    return out


def ref_rope_apply(x, angles):
    x, angles = _f32(x), _f32(angles)
    B, H, S, D = x.shape
    out = np.empty_like(x)
    _rchk(ref.vref_apply_rotary_emb(_p(x), B, H, S, D, _p(angles), _p(out)))
    return out


def ref_linear(x, w, bias=None):
    """x [B, T, K] through the compiled reference's nn::Linear(K, N) with the given weight [N, K] and bias [N]."""
    x, w = _f32(x), _f32(w)
    B, T, K = x.shape
    N = w.shape[0]
    y = np.empty((B, T, N), np.float32)
    b = _f32(bias) if bias is not None else None
    _rchk(ref.vref_linear(_p(x), _p(w), _p(b) if b is not None else None, _p(y), B, T, K, N))
    return y


def ref_gqa_ctor(embed_dim, num_heads, num_kv_heads):
    hd, nr = i64(0), i64(0)
    _rchk(ref.vref_gqa_ctor(embed_dim, num_heads, num_kv_heads, C.byref(hd), C.byref(nr)))
    return hd.value, nr.value
