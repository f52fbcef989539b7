"""A ragged batch end to end on the GPU: prompts of different lengths prefilled in one call, then token-by-token
decode with one row leaving and a new request taking its place, all lengths kept on the device.  Every row is checked
against the oracle's full causal attention over that row's own tokens (RoPE included), on the values the cache holds."""
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


class RowModel:
    """CPU model of one request: all of its q, k, v so far (already rotated, bf16-rounded as the cache holds them)."""

    def __init__(self, Hq, Hkv, D):
        self.q = np.zeros((1, Hq, 0, D), np.float32)
        self.k = np.zeros((1, Hkv, 0, D), np.float32)
        self.v = np.zeros((1, Hkv, 0, D), np.float32)

    def push(self, q, k, v):
        start = self.k.shape[2]
        ang = O.rope_angles(q.shape[2], q.shape[3], start)
        self.q = np.concatenate([self.q, O.bf16_round(O.rope_apply(q, ang))], axis=2)
        self.k = np.concatenate([self.k, O.bf16_round(O.rope_apply(k, ang))], axis=2)
        self.v = np.concatenate([self.v, O.bf16_round(v)], axis=2)

    def expect_last(self, n):
        L, D = self.k.shape[2], self.k.shape[3]
        rep = self.q.shape[1] // self.k.shape[1]
        out = O.flash_attention(self.q, O.repeat_kv(self.k, rep), O.repeat_kv(self.v, rep),
                                float(np.float32(1.0 / math.sqrt(D))), True)
        return out[:, :, L - n:]


def test_continuous_batching_scenario(va):
    B, Hq, Hkv, D, S_max = 3, 8, 2, 128, 192
    rope = va.RopeTable(S_max, D)
    cache = va.RaggedKVCache(B, Hkv, S_max, D, fmt="bf16")
    models = [RowModel(Hq, Hkv, D) for _ in range(B)]
    seed = [4000]

    def fresh(T):
        seed[0] += 3
        return I.qkv(seed[0], 1, Hq, Hkv, T, T, D, scale=0.6)

    def step(n_new, T):
        """Every row b receives n_new[b] new tokens (padded to T rows); returns device output [B,Hq,T,D]."""
        q = np.zeros((B, Hq, T, D), np.float32)
        k = np.zeros((B, Hkv, T, D), np.float32)
        v = np.zeros((B, Hkv, T, D), np.float32)
        for b in range(B):
            if n_new[b]:
                qb, kb, vb = fresh(n_new[b])
                q[b, :, :n_new[b]], k[b, :, :n_new[b]], v[b, :, :n_new[b]] = qb[0], kb[0], vb[0]
                models[b].push(qb, kb, vb)
        nn = torch.tensor(n_new, dtype=torch.int32, device=G.dev())
        q_rot = cache.append(G.f32_dev(k), G.f32_dev(v), n_new=nn, q=G.f32_dev(q), rope=rope, q_dtype=torch.bfloat16)
        if T == 1:
            return cache.decode(q_rot)
        return cache.prefill_chunk(q_rot, n_new=nn)

    def check(out, n_new, what):
        got = G.bf16_to_np(out)
        for b in range(B):
            if n_new[b]:
                G.assert_bf16_close(got[b:b + 1, :, :n_new[b]], models[b].expect_last(n_new[b]), f"{what} row {b}")

    prompts = [37, 5, 64]
    check(step(prompts, 64), prompts, "ragged prompt prefill")
    assert cache.seq_lens.cpu().tolist() == prompts
    for i in range(3):
        check(step([1, 1, 1], 1), [1, 1, 1], f"decode {i}")
    # row 1 finishes; a new request with a 20-token prompt takes its slot while rows 0 and 2 idle this step
    cache.reset_rows([1])
    models[1] = RowModel(Hq, Hkv, D)
    check(step([0, 20, 0], 32), [0, 20, 0], "late joiner prefill")
    assert cache.seq_lens.cpu().tolist() == [40, 20, 67]
    for i in range(2):
        check(step([1, 1, 1], 1), [1, 1, 1], f"decode after join {i}")
    # a second chunk for row 2 only (chunked prefill of a long prompt), others decode-idle
    check(step([0, 0, 33], 64), [0, 0, 33], "second chunk")
    assert cache.seq_lens.cpu().tolist() == [42, 22, 102]


def test_advance_clamps_and_validates(va):
    import ctypes as C
    from vesper_amd import _ffi
    lens = torch.tensor([0, 10, 60], dtype=torch.int32, device=G.dev())
    nn = torch.tensor([-3, 9, 2], dtype=torch.int32, device=G.dev())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert _ffi.lib.vsp_seq_lens_advance(C.c_void_p(lens.data_ptr()), C.c_void_p(nn.data_ptr()), 4, 3, 64, st) == 0
    assert lens.cpu().tolist() == [0, 14, 62]
    assert _ffi.lib.vsp_seq_lens_advance(C.c_void_p(lens.data_ptr()), None, 4, 3, 64, st) == 0
    assert lens.cpu().tolist() == [4, 18, 64]
    assert _ffi.lib.vsp_seq_lens_advance(None, None, 4, 3, 64, st) == _ffi.ERR_NULL
