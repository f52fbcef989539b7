"""Python view of the reference's operator surface for the attention path, on torch device tensors.

torch is used for device memory and streams only; every computation is a call into libvsp_attn.so.
Names and argument meaning follow the reference (paths relative to its tree):
  flash_attention(q,k,v,scale,is_causal,dropout_p,training)  include/vesper/ops/flash_attention.h:34-41
  scaled_dot_product_attention(q,k,v,is_causal,dropout_p)     include/vesper/nn/functional.h:132-136
  KVCache / GQAKVCache .update/.reset/.current_seq_len         include/vesper/nn/transformer.h:21-39,
                                                               include/vesper/nn/gqa_attention.h:110-163
  attention_core(q,k,v,cache,start_pos)                        steps 4-6 of GroupedQueryAttention::forward,
                                                               src/nn/gqa_attention.cpp:128-148
"""
import ctypes as C
import math

import torch

from . import _ffi
from ._ffi import VspError, VspKVCache, VspTensor, check, lib

_DT = {torch.float32: _ffi.F32, torch.bfloat16: _ffi.BF16, torch.float16: _ffi.F16, torch.int8: _ffi.I8,
       torch.int32: _ffi.I32}


def _desc(t):
    d = VspTensor()
    d.data = t.data_ptr() if t.numel() > 0 else (t.data_ptr() or 0)
    if t.dtype not in _DT:
        raise VspError(_ffi.ERR_UNSUPPORTED)
    d.dtype = _DT[t.dtype]
    d.ndim = min(t.dim(), 4)
    for i in range(min(t.dim(), 4)):
        d.shape[i] = t.shape[i]
        d.stride[i] = t.stride(i)
    if t.dim() > 4:
        d.ndim = t.dim()  # rejected by the library with the reference's message
    return d


def _stream(t):
    return C.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def repeat_kv_is_fused():
    """ops::repeat_kv (src/ops/attention_ops.cpp:92-155) has no kernel here: query head h reads kv head
    h // n_rep inside the attention kernels."""
    return True


def flash_attention(q, k, v, scale, is_causal=True, dropout_p=0.0, training=False, return_lse=False):
    """ops::flash_attention; k, v may have fewer heads than q (GQA)."""
    if not (q.is_cuda and k.is_cuda and v.is_cuda):
        raise RuntimeError("flash_attention: unsupported device")  # src/ops/flash_attention.cpp:111-112
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=q.device) if (return_lse and q.dim() == 4) else None
    dq, dk, dv, do = _desc(q), _desc(k), _desc(v), _desc(out)
    dl = _desc(lse) if lse is not None else None
    check(lib.vsp_attn_prefill(C.byref(dq), C.byref(dk), C.byref(dv), C.byref(do),
                               C.byref(dl) if dl is not None else None, float(scale), int(bool(is_causal)),
                               float(dropout_p), int(bool(training)), _stream(q)))
    return (out, lse) if return_lse else out


def flash_attention_split(q, k, v, scale, is_causal=True, return_lse=False, workspace=None):
    """ops::flash_attention for fp32 tensors through the bf16 matrix cores (vsp_attn_prefill_split): every operand as two
    bf16 terms, three MFMAs per product, fp32 accumulation; within the reference's 1e-4 of its fp32 result."""
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    lse = torch.empty(q.shape[:3], dtype=torch.float32, device=q.device) if (return_lse and q.dim() == 4) else None
    if workspace is None:
        nws = lib.vsp_attn_prefill_split_workspace_bytes(q.shape[0], q.shape[1], k.shape[1], q.shape[2], k.shape[2], q.shape[3]) \
            if q.dim() == 4 and k.dim() == 4 else 0
        workspace = torch.empty(max(nws, 16), dtype=torch.uint8, device=q.device)
    dq, dk, dv, do = _desc(q), _desc(k), _desc(v), _desc(out)
    dl = _desc(lse) if lse is not None else None
    check(lib.vsp_attn_prefill_split(C.byref(dq), C.byref(dk), C.byref(dv), C.byref(do),
                                     C.byref(dl) if dl is not None else None, float(scale), int(bool(is_causal)),
                                     C.c_void_p(workspace.data_ptr()), workspace.numel(), _stream(q)))
    return (out, lse) if return_lse else out


def backward_workspace(q, fast=False):
    """Workspace of flash_attention_backward for tensors of q's shape; fast: the larger one that lets the bf16 path
    compute dS once (vsp_attn_backward_fast_workspace_bytes)."""
    f = lib.vsp_attn_backward_fast_workspace_bytes if fast else lib.vsp_attn_backward_workspace_bytes
    return torch.empty(max(f(q.shape[0], q.shape[1], q.shape[2]), 16), dtype=torch.uint8, device=q.device)


def flash_attention_backward(grad_output, q, k, v, output, lse, scale, is_causal=True, workspace=None):
    """ops::flash_attention_backward: (dq, dk, dv); k, v may have fewer heads than q (their gradients then sum over
    the query heads of each group).  workspace: from backward_workspace(); its size selects the bf16 path."""
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    descs = [_desc(t) for t in (grad_output, q, k, v, output, lse, dq, dk, dv)]
    ws = workspace if workspace is not None else backward_workspace(q)
    check(lib.vsp_attn_prefill_backward(*[C.byref(d) for d in descs], float(scale), int(bool(is_causal)),
                                        C.c_void_p(ws.data_ptr()), ws.numel(), _stream(q)))
    return dq, dk, dv


def flash_attention_backward_split(grad_output, q, k, v, output, lse, scale, is_causal=True, workspace=None):
    """ops::flash_attention_backward for fp32 tensors through the bf16 matrix cores (vsp_attn_prefill_backward_split):
    every operand as two bf16 terms, three MFMAs per product, fp32 accumulation and fp32 gradients."""
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    descs = [_desc(t) for t in (grad_output, q, k, v, output, lse, dq, dk, dv)]
    if workspace is None:
        nws = lib.vsp_attn_backward_split_workspace_bytes(q.shape[0], q.shape[1], k.shape[1], q.shape[2], q.shape[3]) \
            if q.dim() == 4 and k.dim() == 4 else 0
        workspace = torch.empty(max(nws, 16), dtype=torch.uint8, device=q.device)
    check(lib.vsp_attn_prefill_backward_split(*[C.byref(d) for d in descs], float(scale), int(bool(is_causal)),
                                              C.c_void_p(workspace.data_ptr()), workspace.numel(), _stream(q)))
    return dq, dk, dv


class RopeTable:
    """{cos, sin} of the angles of functional::compute_rope_frequencies (src/nn/functional.cpp:424-443) for
    absolute positions [0, length): computed once on the host by the library, kept on the device."""

    def __init__(self, length, head_dim, theta=10000.0, device="cuda"):
        host = torch.empty((length, head_dim // 2, 2), dtype=torch.float32)
        lib.vsp_rope_fill_table(C.c_void_p(host.data_ptr()), 0, int(length), int(head_dim), float(theta))
        self.length, self.head_dim, self.theta = int(length), int(head_dim), float(theta)
        self.host = host
        self.table = host.to(device)


class KVCache:
    """nn::KVCache with selectable storage: fmt 'f32' (the reference's layout), 'bf16' or 'q8_0'."""

    _FMT = {"f32": _ffi.KV_F32, "bf16": _ffi.KV_BF16, "q8_0": _ffi.KV_Q8_0}

    def __init__(self, batch_size, num_heads, max_seq_len, head_dim, device="cuda", fmt="f32", paging=None):
        """paging=(page_tokens, n_pages): the planes hold n_pages pages of page_tokens tokens and `page_table`
        (device int32 [batch, max_seq_len / page_tokens], set by the caller) says which page holds which tokens."""
        self.fmt = fmt
        self.device = torch.device(device)
        c = VspKVCache()
        c.format = self._FMT[fmt]
        c.B, c.Hkv, c.S_max, c.D = batch_size, num_heads, max_seq_len, head_dim
        self.page_table = None
        if paging is not None:
            page_tokens, n_pages = paging
            c.page_tokens, c.n_pages = int(page_tokens), int(n_pages)
            c.pages_per_seq = max_seq_len // max(int(page_tokens), 1)
            self.page_table = torch.zeros((batch_size, max(c.pages_per_seq, 1)), dtype=torch.int32, device=self.device)
            c.page_table = self.page_table.data_ptr()
        self._planes = []
        for plane in range(4):
            if paging is not None:
                n = lib.vsp_kv_plane_bytes(c.format, c.n_pages, c.Hkv, c.page_tokens, c.D, plane)
            else:
                n = lib.vsp_kv_plane_bytes(c.format, c.B, c.Hkv, c.S_max, c.D, plane)
            self._planes.append(torch.empty(n, dtype=torch.uint8, device=self.device) if n else None)
        c.k, c.v, c.k_scale, c.v_scale = [p.data_ptr() if p is not None else None for p in self._planes]
        c.len = 0
        self._c = c
        check(lib.vsp_kv_cache_reset(C.byref(c), _stream(self._planes[0])))  # vesper::zeros, transformer.cpp:40-41

    # -- reference interface
    def current_seq_len(self):
        return int(self._c.len)

    def get_max_seq_len(self):
        return int(self._c.S_max)

    max_seq_len = get_max_seq_len

    def reset(self):
        check(lib.vsp_kv_cache_reset(C.byref(self._c), _stream(self._planes[0])))

    def update(self, new_k, new_v, start_pos, return_views=True, start_pos_dev=None):
        dk, dv = _desc(new_k), _desc(new_v)
        sp = C.c_void_p(start_pos_dev.data_ptr()) if start_pos_dev is not None else None
        check(lib.vsp_kv_append(C.byref(self._c), C.byref(dk), C.byref(dv), int(start_pos), sp, _stream(new_k)))
        if not return_views:
            return None
        return self.views()

    def rope_update(self, q, new_k, new_v, start_pos, rope, out_dtype=None, start_pos_dev=None, return_views=False,
                    out=None):
        """Steps 3-4 of the attention modules' cached forward in one launch (src/nn/gqa_attention.cpp:124-130):
        q and k rotated by `rope` (a RopeTable) at positions start_pos.., k and v written to the cache.
        Returns the rotated q (and the cache views when asked)."""
        q_out = out if out is not None else torch.empty(q.shape, dtype=out_dtype or q.dtype, device=q.device)
        dq, dk, dv, do = _desc(q), _desc(new_k), _desc(new_v), _desc(q_out)
        sp = C.c_void_p(start_pos_dev.data_ptr()) if start_pos_dev is not None else None
        check(lib.vsp_rope_kv_append(C.byref(self._c), C.byref(dq), C.byref(dk), C.byref(dv), C.byref(do),
                                     C.c_void_p(rope.table.data_ptr()), rope.length, int(start_pos), sp, _stream(q)))
        return (q_out, self.views()) if return_views else q_out

    def prefill(self, q, seq_lens=None, is_causal=True, scale=None, return_lse=False, chunk_lens=None, split=True, max_len=0):
        """Attention of the last T tokens (q [B,Hq,T,D]) over the cached context, read in place from the planes:
        chunked prefill.  seq_lens: device int32[B] per-row context lengths (default: the cache's one length).
        split=False withholds the workspace that lets the library split a long context over workgroups.
        max_len: host-side bound of the device-side lengths (0: the cache's capacity), which the split is planned on."""
        out = torch.empty_like(q)
        lse = torch.empty(q.shape[:3], dtype=torch.float32, device=q.device) if return_lse else None
        dq, do = _desc(q), _desc(out)
        dl = _desc(lse) if lse is not None else None
        sl = C.c_void_p(seq_lens.data_ptr()) if seq_lens is not None else None
        cl = C.c_void_p(chunk_lens.data_ptr()) if chunk_lens is not None else None
        sc = float(scale) if scale is not None else 1.0 / math.sqrt(q.shape[-1])
        nws = lib.vsp_attn_prefill_cached_workspace_bytes(C.byref(self._c), int(seq_lens is not None), int(max_len))
        ws = torch.empty(nws, dtype=torch.uint8, device=q.device) if nws else None
        if not nws and split:  # a few query tiles over a long context: the context is split over workgroups
            nws = lib.vsp_attn_prefill_cached_split_workspace_bytes(C.byref(self._c), int(seq_lens is not None), int(max_len), q.shape[1], q.shape[2])
            ws = _workspace(q.device, nws) if nws else None   # the per-stream block the decode step uses (bounded: <= 70 MB)
        check(lib.vsp_attn_prefill_cached(C.byref(dq), C.byref(self._c), sl, int(max_len), cl, C.byref(do),
                                          C.byref(dl) if dl is not None else None, sc, int(bool(is_causal)),
                                          C.c_void_p(ws.data_ptr()) if ws is not None else None, nws, _stream(q)))
        return (out, lse) if return_lse else out

    # -- reads
    def views(self, dtype=None):
        """[:, :, 0:len, :] of K and V.  fp32 storage: true views (no copy), like the reference;
        other formats: materialised in `dtype` (default fp32)."""
        c = self._c
        if c.format == _ffi.KV_F32:
            shape = (c.B, c.Hkv, c.S_max, c.D)
            k = self._planes[0].view(torch.float32).view(shape)[:, :, :c.len, :]
            v = self._planes[1].view(torch.float32).view(shape)[:, :, :c.len, :]
            return k, v
        return self.read(0, c.len, dtype or torch.float32)

    def read(self, start, count, dtype=torch.float32):
        c = self._c
        k = torch.empty((c.B, c.Hkv, count, c.D), dtype=dtype, device=self.device)
        v = torch.empty_like(k)
        dk, dv = _desc(k), _desc(v)
        check(lib.vsp_kv_read(C.byref(c), int(start), int(count), C.byref(dk), C.byref(dv), _stream(k)))
        return k, v

    def read_q8_0(self, plane, start, count):
        c = self._c
        qs = torch.empty((c.B, c.Hkv, count, c.D), dtype=torch.int8, device=self.device)
        sc = torch.empty((c.B, c.Hkv, count, c.D // 32), dtype=torch.int16, device=self.device)
        check(lib.vsp_kv_read_q8_0(C.byref(c), plane, int(start), int(count), qs.data_ptr(), sc.data_ptr(), _stream(qs)))
        return qs, sc

    def raw_plane(self, plane):
        return self._planes[plane]

    def set_len(self, n):
        """Bench/test helper: declare `n` tokens valid without appending (planes filled directly)."""
        self._c.len = int(n)


class GQAKVCache(KVCache):
    """nn::GQAKVCache: same semantics, int64 bookkeeping in the reference."""


class RaggedKVCache(KVCache):
    """A cache whose rows have their own lengths, kept in a device int32[B] array (the reference's caches have
    one host-side length for the batch).  Every step is asynchronous: nothing is read back to the host.
    `upper` is a host-side upper bound of the longest row, used only to size work (grids, workspaces)."""

    def __init__(self, batch_size, num_heads, max_seq_len, head_dim, device="cuda", fmt="bf16", paging=None):
        super().__init__(batch_size, num_heads, max_seq_len, head_dim, device=device, fmt=fmt, paging=paging)
        self.seq_lens = torch.zeros(batch_size, dtype=torch.int32, device=self.device)
        self.upper = 0

    def reset_rows(self, rows):
        """Forget the given rows (a finished request leaves the batch); their tokens become stale, not zero."""
        self.seq_lens[torch.as_tensor(rows, device=self.device, dtype=torch.long)] = 0

    def _advance(self, n_new, T, ref):
        nn_ = C.c_void_p(n_new.data_ptr()) if n_new is not None else None
        check(lib.vsp_seq_lens_advance(C.c_void_p(self.seq_lens.data_ptr()), nn_, int(T), self._c.B, self._c.S_max,
                                       _stream(ref)))
        self.upper = min(self.upper + int(T), self._c.S_max)

    def append(self, new_k, new_v, n_new=None, q=None, rope=None, q_dtype=None):
        """Row b's first n_new[b] (default: all T) tokens go to positions seq_lens[b]..; with `rope`, q and k are
        rotated at those positions in the same launch and the rotated q is returned."""
        T = new_k.shape[2]
        if rope is not None:
            out = self.rope_update(q, new_k, new_v, 0, rope, out_dtype=q_dtype, start_pos_dev=self.seq_lens)
        else:
            self.update(new_k, new_v, 0, return_views=False, start_pos_dev=self.seq_lens)
            out = None
        self._advance(n_new, T, new_k)
        return out

    def decode(self, q, scale=None, out=None):
        return decode_attention(q, self, seq_lens=self.seq_lens, max_len=max(self.upper, 1), scale=scale, out=out)

    def prefill_chunk(self, q, n_new=None, scale=None):
        """Attention of the chunk just appended (q [B,Hq,T,D], row b valid for n_new[b] rows) over each row's context.
        A full chunk of a few tokens (T * query heads per kv head <= 16) goes through the decode kernels."""
        T, D = q.shape[2], q.shape[3]
        if n_new is None and T > 1 and T * (q.shape[1] // self._c.Hkv) <= 16 and D in (64, 128):
            return decode_attention_multi(q, self, seq_lens=self.seq_lens, max_len=max(self.upper, 1), scale=scale)
        return self.prefill(q, seq_lens=self.seq_lens, chunk_lens=n_new, scale=scale, max_len=max(self.upper, 1))


_WS = {}


def _workspace(device, nbytes):
    """Grow-only split-K workspace, one per (device, stream): calls on different streams never share partials.
    A buffer that a captured graph may hold must not be replaced, so growth during stream capture is refused:
    size it with one eager call (or pass `workspace=`) before capturing."""
    key = (device.type, device.index, torch.cuda.current_stream(device).cuda_stream)
    ws = _WS.get(key)
    if ws is None or ws.numel() < nbytes:
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("decode_attention: the workspace would have to grow during stream capture; "
                               "run one eager call of this size first, or pass workspace=")
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=device)
        _WS[key] = ws
    return ws


def decode_attention(q, cache, seq_lens=None, max_len=0, scale=None, out=None, workspace=None):
    """One new token per sequence attending to the cache: q [B,Hq,1,D] -> [B,Hq,1,D].
    workspace: a caller-owned uint8 device tensor for the split-K partials (default: a cached one per stream)."""
    c = cache._c
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])  # src/nn/functional.cpp:403
    if out is None:
        out = torch.empty_like(q)
    if workspace is None:
        bound = max_len or (c.S_max if seq_lens is not None else c.len)
        nbytes = lib.vsp_attn_decode_workspace_bytes(q.shape[0], q.shape[1], q.shape[3], max(int(bound), 1))
        workspace = _workspace(q.device, nbytes)
    dq, do = _desc(q), _desc(out)
    sl = C.c_void_p(seq_lens.data_ptr()) if seq_lens is not None else None
    check(lib.vsp_attn_decode(C.byref(dq), C.byref(c), sl, int(max_len), C.byref(do), float(scale),
                              C.c_void_p(workspace.data_ptr()), workspace.numel(), _stream(q)))
    return out


def decode_attention_multi(q, cache, seq_lens=None, max_len=0, scale=None, out=None, workspace=None):
    """The last T tokens of each sequence (already appended) attending to the cache at the decode kernels' rate:
    q [B,Hq,T,D] -> [B,Hq,T,D], token t sees keys [0, L_b - T + t]; T * Hq/Hkv <= 16 (vsp_attn_decode_multi)."""
    c = cache._c
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    if out is None:
        out = torch.empty_like(q)
    if workspace is None:
        bound = max_len or (c.S_max if seq_lens is not None else c.len)
        nbytes = lib.vsp_attn_decode_workspace_bytes(q.shape[0] * q.shape[2], q.shape[1], q.shape[3], max(int(bound), 1))
        workspace = _workspace(q.device, nbytes)
    dq, do = _desc(q), _desc(out)
    sl = C.c_void_p(seq_lens.data_ptr()) if seq_lens is not None else None
    check(lib.vsp_attn_decode_multi(C.byref(dq), C.byref(c), sl, int(max_len), C.byref(do), float(scale),
                                    C.c_void_p(workspace.data_ptr()), workspace.numel(), _stream(q)))
    return out


def decode_attention_proj(q, cache, wo, bias=None, seq_lens=None, max_len=0, scale=None, out=None, workspace=None):
    """decode_attention followed by the module's output projection (src/nn/gqa_attention.cpp:151-152, Linear::forward
    src/nn/linear.cpp:41-49) in one call: q [B,Hq,1,D], wo [N, Hq*D], bias [N] or None -> y [B,1,N]."""
    c = cache._c
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    if out is None:
        out = torch.empty((q.shape[0], 1, wo.shape[0]), dtype=q.dtype, device=q.device)
    if workspace is None:
        bound = max_len or (c.S_max if seq_lens is not None else c.len)
        nbytes = lib.vsp_attn_decode_proj_workspace_bytes(q.shape[0], q.shape[1], q.shape[3], max(int(bound), 1), wo.shape[0])
        workspace = _workspace(q.device, nbytes)
    dq, dw, dy = _desc(q), _desc(wo), _desc(out)
    db = _desc(bias) if bias is not None else None
    sl = C.c_void_p(seq_lens.data_ptr()) if seq_lens is not None else None
    check(lib.vsp_attn_decode_proj(C.byref(dq), C.byref(c), sl, int(max_len), C.byref(dw), C.byref(db) if db is not None else None,
                                   C.byref(dy), float(scale), C.c_void_p(workspace.data_ptr()), workspace.numel(), _stream(q)))
    return out


def decode_attention_noalloc(q, cache, out, seq_lens=None, max_len=0, scale=None):
    """decode_attention through vsp_attn_decode_noalloc: the partials go to the library's fixed per-GPU array
    and the call allocates nothing (`out` is the caller's).  Calls overlapping on one GPU race."""
    if scale is None:
        scale = 1.0 / math.sqrt(q.shape[-1])
    dq, do = _desc(q), _desc(out)
    sl = C.c_void_p(seq_lens.data_ptr()) if seq_lens is not None else None
    check(lib.vsp_attn_decode_noalloc(C.byref(dq), C.byref(cache._c), sl, int(max_len), C.byref(do), float(scale),
                                      _stream(q)))
    return out


def scaled_dot_product_attention(q, k, v, is_causal=False, dropout_p=0.0):
    """functional::scaled_dot_product_attention (src/nn/functional.cpp:370-422) on explicit tensors.
    The reference switches algorithm at T >= 512 for speed; here one kernel serves every T.
    Like the reference, a causal mask needs T == L (its [T,T] mask does not broadcast otherwise)
    unless T == 1."""
    if dropout_p > 0.0:
        raise VspError(_ffi.ERR_UNSUPPORTED)
    T, L = q.shape[2], k.shape[2]
    if is_causal and T != L and T != 1:
        raise VspError(_ffi.ERR_BROADCAST)
    scale = 1.0 / math.sqrt(q.shape[-1])
    return flash_attention(q, k, v, scale, is_causal=bool(is_causal) and T > 1)


def attention_core(q, new_k, new_v, cache=None, start_pos=0, rope=None, q_dtype=None):
    """Steps 4-6 of GroupedQueryAttention::forward(x, cache, start_pos), src/nn/gqa_attention.cpp:128-148
    (== MultiHeadAttention::forward, src/nn/transformer.cpp:190-205, with n_rep = 1):
    cache.update(k, v, start_pos); repeat_kv (fused); SDPA with use_causal = (T > 1).
    With `rope` (a RopeTable) step 3 (:124-127) is included: q and k are rotated at start_pos in the same
    launch that writes the cache; q continues in `q_dtype` (default: its own)."""
    T = q.shape[2]
    if cache is None:
        return scaled_dot_product_attention(q, new_k, new_v, is_causal=(T > 1))
    if rope is not None:
        q = cache.rope_update(q, new_k, new_v, start_pos, rope, out_dtype=q_dtype)
    else:
        cache.update(new_k, new_v, start_pos, return_views=False)
    if T == 1:
        return decode_attention(q, cache)
    if cache.current_seq_len() != T:
        raise VspError(_ffi.ERR_BROADCAST)  # the reference's [T,T] mask cannot be added to [T,L] scores
    if cache.fmt == "f32":
        k, v = cache.views()  # true views of the fp32 planes, as in the reference
        return flash_attention(q, k, v, 1.0 / math.sqrt(q.shape[-1]), is_causal=True)
    if q.dtype == torch.bfloat16:
        return cache.prefill(q, is_causal=True)  # bf16 / Q8_0 planes are read in place, nothing is materialised
    k, v = cache.views(dtype=q.dtype)  # fp32 queries over a narrower cache: the context is widened once
    return flash_attention(q, k, v, 1.0 / math.sqrt(q.shape[-1]), is_causal=True)
