"""Fused RoPE + KV append on the GPU, through the C ABI.  The rotation is fp32 with separately rounded products
and sums and a host-computed table, so fp32 results, bf16 roundings and Q8_0 blocks are all bit-exact against
the oracle (which is bit-exact against the compiled reference)."""
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


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _oracle_rot(x, start, theta=10000.0):
    return O.rope_apply(x, O.rope_angles(x.shape[2], x.shape[3], start, theta))


@pytest.mark.parametrize("B,Hq,Hkv,T,D,start", [(2, 8, 2, 8, 64, 0), (1, 4, 4, 1, 128, 37), (2, 6, 3, 19, 128, 70),
                                                (1, 2, 1, 5, 32, 3)])
def test_f32_cache_bit_exact(va, B, Hq, Hkv, T, D, start):
    S_max = 96
    rope = va.RopeTable(S_max, D)
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    q, k, v = I.qkv(900 + T, B, Hq, Hkv, T, T, D)
    q_out, (ck, cv) = c.rope_update(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), start, rope, return_views=True)
    assert c.current_seq_len() == start + T
    assert np.array_equal(_bits(q_out.cpu().numpy()), _bits(_oracle_rot(q, start)))
    assert np.array_equal(_bits(ck[:, :, start:].cpu().numpy()), _bits(_oracle_rot(k, start)))
    assert np.array_equal(cv[:, :, start:].cpu().numpy(), v)          # V is not rotated
    assert not ck[:, :, :start].any() and not cv[:, :, :start].any()  # nothing else touched


@pytest.mark.parametrize("D", [64, 128])
def test_bf16_and_q8_0_caches_bit_exact(va, D):
    B, Hq, Hkv, T, S_max, start = 2, 8, 2, 21, 90, 40
    rope = va.RopeTable(S_max, D, theta=500000.0)
    q, k, v = I.qkv(950, B, Hq, Hkv, T, T, D)
    k_rot, q_rot = _oracle_rot(k, start, 500000.0), _oracle_rot(q, start, 500000.0)
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    q_out = c.rope_update(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), start, rope, out_dtype=torch.bfloat16)
    assert np.array_equal(G.bf16_bits(q_out), O.f32_to_bf16(q_rot))
    ck, cv = c.read(start, T, torch.bfloat16)
    assert np.array_equal(G.bf16_bits(ck), O.f32_to_bf16(k_rot))
    assert np.array_equal(G.bf16_bits(cv), O.f32_to_bf16(v))
    c8 = va.KVCache(B, Hkv, S_max, D, fmt="q8_0")
    c8.rope_update(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), start, rope)
    for plane, m in ((0, k_rot), (1, v)):
        want_d, want_q = O.q8_0_quantize(m)
        qs, sc = c8.read_q8_0(plane, start, T)
        assert np.array_equal(qs.cpu().numpy(), want_q), plane
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_d), plane


def test_bf16_inputs_are_widened_exactly(va):
    B, Hq, Hkv, T, D, S_max = 1, 4, 2, 9, 64, 64
    rope = va.RopeTable(S_max, D)
    q, k, v = [O.bf16_round(x) for x in I.qkv(960, B, Hq, Hkv, T, T, D)]
    c = va.KVCache(B, Hkv, S_max, D, fmt="bf16")
    q_out = c.rope_update(G.to_bf16_dev(q), G.to_bf16_dev(k), G.to_bf16_dev(v), 5, rope)
    assert q_out.dtype == torch.bfloat16
    assert np.array_equal(G.bf16_bits(q_out), O.f32_to_bf16(_oracle_rot(q, 5)))
    ck, cv = c.read(5, T, torch.bfloat16)
    assert np.array_equal(G.bf16_bits(ck), O.f32_to_bf16(_oracle_rot(k, 5)))
    assert np.array_equal(G.bf16_bits(cv), O.f32_to_bf16(v))


def test_strided_views_of_a_fused_projection_and_in_place_q(va):
    # q, k, v as views of one [B, T, (Hq + 2 Hkv) D] buffer: the layout the projections produce before the
    # reference's view + transpose copies (src/nn/gqa_attention.cpp:114-122)
    B, Hq, Hkv, T, D, S_max = 2, 4, 2, 7, 64, 32
    rope = va.RopeTable(S_max, D)
    fused = I.normal(970, (B, T, (Hq + 2 * Hkv) * D))
    fd = G.f32_dev(fused)
    qv = fd[:, :, :Hq * D].view(B, T, Hq, D).transpose(1, 2)
    kv = fd[:, :, Hq * D:(Hq + Hkv) * D].view(B, T, Hkv, D).transpose(1, 2)
    vv = fd[:, :, (Hq + Hkv) * D:].view(B, T, Hkv, D).transpose(1, 2)
    assert not qv.is_contiguous()
    qn = fused[:, :, :Hq * D].reshape(B, T, Hq, D).transpose(0, 2, 1, 3)
    kn = fused[:, :, Hq * D:(Hq + Hkv) * D].reshape(B, T, Hkv, D).transpose(0, 2, 1, 3)
    vn = fused[:, :, (Hq + Hkv) * D:].reshape(B, T, Hkv, D).transpose(0, 2, 1, 3)
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    q_out, (ck, cv) = c.rope_update(qv, kv, vv, 2, rope, return_views=True)
    assert np.array_equal(_bits(q_out.cpu().numpy()), _bits(_oracle_rot(qn, 2)))
    assert np.array_equal(_bits(ck[:, :, 2:].cpu().numpy()), _bits(_oracle_rot(kn, 2)))
    assert np.array_equal(cv[:, :, 2:].cpu().numpy(), np.ascontiguousarray(vn))
    # in place: q_out aliasing q
    import ctypes as C
    from vesper_amd import _ffi
    from vesper_amd.api import _desc, _stream
    c2 = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    dq, dk, dv = _desc(qv), _desc(kv), _desc(vv)
    _ffi.check(_ffi.lib.vsp_rope_kv_append(C.byref(c2._c), C.byref(dq), C.byref(dk), C.byref(dv), C.byref(dq),
                                           C.c_void_p(rope.table.data_ptr()), rope.length, 2, None, _stream(qv)))
    assert np.array_equal(_bits(qv.cpu().numpy()), _bits(_oracle_rot(qn, 2)))


def test_per_sequence_positions(va):
    B, Hq, Hkv, T, D, S_max = 3, 4, 2, 1, 128, 64
    rope = va.RopeTable(S_max, D)
    starts = np.array([5, 0, 41], np.int32)
    q, k, v = I.qkv(980, B, Hq, Hkv, T, T, D)
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    sp = torch.from_numpy(starts).to(G.dev())
    q_out = c.rope_update(G.f32_dev(q), G.f32_dev(k), G.f32_dev(v), 0, rope, start_pos_dev=sp)
    c.set_len(S_max)
    ck, cv = c.views()
    for b in range(B):
        s = int(starts[b])
        assert np.array_equal(_bits(q_out[b:b + 1].cpu().numpy()), _bits(_oracle_rot(q[b:b + 1], s)))
        assert np.array_equal(_bits(ck[b:b + 1, :, s:s + T].cpu().numpy()), _bits(_oracle_rot(k[b:b + 1], s)))
        assert np.array_equal(cv[b, :, s:s + T].cpu().numpy(), v[b])


def test_cached_attention_with_rope_replays_the_reference_fixture(va):
    # GroupedQueryAttention::forward(x, cache, start_pos) steps 3-6 (src/nn/gqa_attention.cpp:124-148)
    z = np.load(os.path.join(GOLD, "rope.npz"), allow_pickle=False)
    B, Hq, Hkv, D, S_max = [int(x) for x in z["meta"]]
    rope = va.RopeTable(S_max, D)
    for fmt in ("f32", "bf16"):
        c = va.KVCache(B, Hkv, S_max, D, fmt=fmt)
        si = 0
        while f"s{si}_op" in z.files:
            T, pos = [int(x) for x in z[f"s{si}_op"]]
            q, nk, nv = I.qkv(8100 + 10 * si, B, Hq, Hkv, T, T, D)
            if fmt == "f32":
                out = va.attention_core(G.f32_dev(q), G.f32_dev(nk), G.f32_dev(nv), c, pos, rope=rope)
                G.assert_f32_close(out.cpu().numpy(), z[f"s{si}_out"], f"step {si}")
            else:
                out = va.attention_core(G.f32_dev(q), G.f32_dev(nk), G.f32_dev(nv), c, pos, rope=rope,
                                        q_dtype=torch.bfloat16)
                G.assert_bf16_close(G.bf16_to_np(out), z[f"s{si}_out"], f"step {si}")
            assert c.current_seq_len() == pos + T
            si += 1
        assert si == 4
    # the rotated q itself, bit for bit
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    q, nk, nv = I.qkv(8100, B, Hq, Hkv, 8, 8, D)
    q_rot = c.rope_update(G.f32_dev(q), G.f32_dev(nk), G.f32_dev(nv), 0, rope)
    assert np.array_equal(_bits(q_rot.cpu().numpy()), _bits(z["s0_qrot"]))


def test_argument_errors(va):
    B, Hq, Hkv, T, D, S_max = 1, 4, 2, 4, 64, 16
    rope = va.RopeTable(8, D)
    c = va.KVCache(B, Hkv, S_max, D, fmt="f32")
    q, k, v = [G.f32_dev(x) for x in I.qkv(990, B, Hq, Hkv, T, T, D)]
    with pytest.raises(va.VspError):   # positions 6..9 leave the 8-row table
        c.rope_update(q, k, v, 6, rope)
    big = va.RopeTable(64, D)
    with pytest.raises(va.VspError) as e:  # slot leaves the cache: the reference's copy_from error
        c.rope_update(q, k, v, 14, big)
    assert "element count mismatch" in str(e.value)
    with pytest.raises(va.VspError):   # q of another dtype than k
        c.rope_update(q.to(torch.bfloat16), k, v, 0, big)
    with pytest.raises(va.VspError):   # k with the wrong head count
        c.rope_update(q, k[:, :1], v[:, :1], 0, big)
    assert c.current_seq_len() == 0
