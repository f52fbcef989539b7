"""KV-cache append / read parity on the GPU, through the C ABI: indexing and block packing are bit-exact."""
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


@pytest.mark.parametrize("gqa", [0, 1])
def test_f32_cache_replays_reference_fixture(va, gqa):
    z = np.load(os.path.join(GOLD, "kv_cache.npz"), allow_pickle=False)
    B, H, S_max, D = [int(x) for x in z["shape"]]
    c = (va.GQAKVCache if gqa else va.KVCache)(B, H, S_max, D, fmt="f32")
    si = 0
    while f"g{gqa}_s{si}_op" in z.files:
        tag = f"g{gqa}_s{si}"
        T, pos = [int(x) for x in z[tag + "_op"]]
        if T == -1:
            c.reset()
        else:
            nk, nv = I.normal(5000 + si, (B, H, T, D)), I.normal(6000 + si, (B, H, T, D))
            if z[tag + "_err"][0]:
                with pytest.raises(va.VspError) as e:
                    c.update(G.f32_dev(nk), G.f32_dev(nv), pos)
                assert str(e.value) == bytes(z[tag + "_msg"]).decode()
            else:
                k, v = c.update(G.f32_dev(nk), G.f32_dev(nv), pos)
                assert np.array_equal(k.cpu().numpy(), z[tag + "_k"]), tag
                assert np.array_equal(v.cpu().numpy(), z[tag + "_v"]), tag
                if not gqa:
                    meta = list(k.shape) + list(k.stride()) + [k.storage_offset()]
                    assert meta == list(z[tag + "_viewmeta"]), tag
        assert c.current_seq_len() == int(z[tag + "_len"][0]), tag
        si += 1
    assert si == 15 and c.get_max_seq_len() == S_max


def test_f32_cache_basic_values_from_reference_test(va):
    # tests/test_kv_cache.cpp:8-43 of the reference
    c = va.KVCache(1, 1, 10, 4, fmt="f32")
    ones = torch.ones(1, 1, 2, 4, device=G.dev())
    k1, _ = c.update(ones, ones, 0)
    assert c.current_seq_len() == 2 and tuple(k1.shape) == (1, 1, 2, 4)
    three = torch.full((1, 1, 1, 4), 3.0, device=G.dev())
    k2, v2 = c.update(three, three, 2)
    assert c.current_seq_len() == 3 and k2.shape[2] == 3
    assert k2.reshape(-1)[2 * 4].item() == 3.0 and v2[0, 0, 2, 0].item() == 3.0 and k2[0, 0, 1, 0].item() == 1.0


def _random_walk(va, fmt, D, src_dtype):
    rng = np.random.default_rng(11)
    B, H, S_max = 2, 3, 90  # not a multiple of 64: exercises S_pad
    c = va.KVCache(B, H, S_max, D, fmt=fmt)
    model = O.KVCache(B, H, S_max, D)
    for step in range(25):
        if step == 12:
            c.reset(), model.reset()
        T, pos = int(rng.integers(0, 20)), int(rng.integers(-2, S_max + 2))
        nk, nv = I.normal(step, (B, H, T, D)), I.normal(500 + step, (B, H, T, D))
        if src_dtype == "bf16":
            nk, nv = O.bf16_round(nk), O.bf16_round(nv)
            dk, dv = G.to_bf16_dev(nk), G.to_bf16_dev(nv)
        else:
            dk, dv = G.f32_dev(nk), G.f32_dev(nv)
        try:
            model.update(nk, nv, pos)
            ok = True
        except O.OracleError as e:
            ok, msg = False, str(e)
        if ok:
            c.update(dk, dv, pos, return_views=False)
        else:
            with pytest.raises(va.VspError) as e2:
                c.update(dk, dv, pos, return_views=False)
            assert str(e2.value) == msg
        assert c.current_seq_len() == model.current_seq_len()
    return c, model


@pytest.mark.parametrize("src_dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D", [64, 128])
def test_bf16_cache_random_walk_bit_exact(va, D, src_dtype):
    c, model = _random_walk(va, "bf16", D, src_dtype)
    mk, mv = model.planes()
    B, H, S_max, _ = mk.shape
    # logical read-back of the WHOLE capacity (zeros where nothing was written) == RNE of the model
    k, v = c.read(0, S_max, torch.bfloat16)
    assert np.array_equal(G.bf16_bits(k), O.f32_to_bf16(mk))
    assert np.array_equal(G.bf16_bits(v), O.f32_to_bf16(mv))
    k32, v32 = c.read(0, S_max, torch.float32)
    assert np.array_equal(k32.cpu().numpy(), O.bf16_round(mk))
    # physical layout as documented in include/vsp_attn.h, computed independently here
    S_pad = (S_max + 63) // 64 * 64
    kp = c.raw_plane(0).cpu().numpy().view(np.uint16).reshape(B, H, S_pad, D)
    assert np.array_equal(kp[:, :, :S_max], O.f32_to_bf16(mk)) and not kp[:, :, S_max:].any()
    vp = c.raw_plane(1).cpu().numpy().view(np.uint16).reshape(B, H, S_pad // 8, D, 8)
    want_v = np.zeros((B, H, S_pad, D), np.uint16)
    want_v[:, :, :S_max] = O.f32_to_bf16(mv)
    assert np.array_equal(vp, want_v.reshape(B, H, S_pad // 8, 8, D).transpose(0, 1, 2, 4, 3))


@pytest.mark.parametrize("src_dtype", ["f32", "bf16"])
@pytest.mark.parametrize("D", [64, 128])
def test_q8_0_cache_block_packing_bit_exact(va, D, src_dtype):
    c, model = _random_walk(va, "q8_0", D, src_dtype)
    mk, mv = model.planes()
    B, H, S_max, _ = mk.shape
    for plane, m in ((0, mk), (1, mv)):
        want_d, want_q = O.q8_0_quantize(m)
        qs, sc = c.read_q8_0(plane, 0, S_max)
        assert np.array_equal(qs.cpu().numpy(), want_q), f"plane {plane} qs"
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_d), f"plane {plane} scales"
    k32, v32 = c.read(0, S_max, torch.float32)
    assert np.array_equal(k32.cpu().numpy(), O.q8_0_dequantize(*O.q8_0_quantize(mk)))
    assert np.array_equal(v32.cpu().numpy(), O.q8_0_dequantize(*O.q8_0_quantize(mv)))
    # physical layout
    S_pad = (S_max + 63) // 64 * 64
    dq, qq = O.q8_0_quantize(mv)
    vq = np.zeros((B, H, S_pad, D), np.int8)
    vq[:, :, :S_max] = qq
    vs = np.zeros((B, H, S_pad, D // 32), np.uint16)
    vs[:, :, :S_max] = dq
    got_vq = c.raw_plane(1).cpu().numpy().view(np.int8).reshape(B, H, S_pad // 16, D, 16)
    got_vs = c.raw_plane(3).cpu().numpy().view(np.uint16).reshape(B, H, S_pad // 16, D // 32, 16)
    assert np.array_equal(got_vq, vq.reshape(B, H, S_pad // 16, 16, D).transpose(0, 1, 2, 4, 3))
    assert np.array_equal(got_vs, vs.reshape(B, H, S_pad // 16, 16, D // 32).transpose(0, 1, 2, 4, 3))
    kq = c.raw_plane(0).cpu().numpy().view(np.int8).reshape(B, H, S_pad, D)
    assert np.array_equal(kq[:, :, :S_max], O.q8_0_quantize(mk)[1])


def test_q8_0_quantiser_edge_values(va):
    # zero blocks, a subnormal-scale block, exact halves (roundf is half-away-from-zero), huge values
    D = 64
    x = np.zeros((1, 1, 6, D), np.float32)
    x[0, 0, 1, :32] = 1e-7
    x[0, 0, 2, :5] = [127, 0.5, -0.5, 2.5, -1.5]
    x[0, 0, 3] = np.linspace(-3e4, 3e4, D)
    x[0, 0, 4, 32:] = -1.0
    x[0, 0, 5] = I.normal(1, (D,)) * 1e-3
    c = va.KVCache(1, 1, 8, D, fmt="q8_0")
    c.update(G.f32_dev(x), G.f32_dev(x[..., ::-1].copy()), 0, return_views=False)
    for plane, m in ((0, x), (1, x[..., ::-1].copy())):
        want_d, want_q = O.q8_0_quantize(m)
        qs, sc = c.read_q8_0(plane, 0, 6)
        assert np.array_equal(qs.cpu().numpy(), want_q)
        assert np.array_equal(sc.cpu().numpy().view(np.uint16), want_d)


def test_strided_source_and_per_sequence_positions(va):
    B, H, S_max, D, T = 3, 2, 64, 64, 5
    c = va.KVCache(B, H, S_max, D, fmt="bf16")
    base = I.normal(3, (B, T, H, 2 * D))  # [B,T,H,2D] -> take a [B,H,T,D] strided view of the first half
    src = G.f32_dev(base)
    view = src[..., :D].permute(0, 2, 1, 3)
    assert not view.is_contiguous()
    pos = torch.tensor([0, 7, 40], dtype=torch.int32, device=G.dev())
    c.update(view, view, 0, return_views=False, start_pos_dev=pos)
    assert c.current_seq_len() == 0  # ragged appends leave the single batch-wide length alone
    k, v = c.read(0, S_max, torch.float32)
    want = np.zeros((B, H, S_max, D), np.float32)
    for b, p in enumerate([0, 7, 40]):
        want[b, :, p:p + T] = O.bf16_round(base[b, :, :, :D].transpose(1, 0, 2))
    assert np.array_equal(k.cpu().numpy(), want) and np.array_equal(v.cpu().numpy(), want)


def test_argument_errors(va):
    c = va.KVCache(1, 2, 16, 64, fmt="bf16")
    k = torch.zeros(1, 2, 3, 64, device=G.dev())
    with pytest.raises(va.VspError) as e:
        c.update(k[0], k[0], 0)  # 3-D
    assert e.value.status == 1
    with pytest.raises(va.VspError) as e:
        c.update(k, k.to(torch.bfloat16), 0)
    assert str(e.value) == "copy_from: dtype mismatch."
    with pytest.raises(va.VspError) as e:
        c.update(k, k, 14)  # runs past S_max: the reference clamps the slot and then copy_from throws
    assert str(e.value) == "copy_from: element count mismatch."
    assert c.current_seq_len() == 0
    with pytest.raises(va.VspError):
        va.KVCache(1, 1, 8, 80, fmt="bf16")  # head_dim the MFMA layouts do not cover
