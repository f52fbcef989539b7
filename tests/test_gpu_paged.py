"""Paged KV cache on the GPU: a paged cache with any page table must behave exactly like a contiguous cache holding
the same tokens -- the kernels do the same arithmetic in the same order, only the addresses differ -- so appends read
back bit-identically and decode outputs are torch.equal to the contiguous cache's (which the other tests pin to the
oracle)."""
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


def _pair(va, fmt, B, Hkv, S_max, D, P, seed, extra_pages=3):
    pps = S_max // P
    n_pages = B * pps + extra_pages
    flat = va.RaggedKVCache(B, Hkv, S_max, D, fmt=fmt)
    paged = va.RaggedKVCache(B, Hkv, S_max, D, fmt=fmt, paging=(P, n_pages))
    perm = np.random.default_rng(seed).permutation(n_pages)[:B * pps].astype(np.int32).reshape(B, pps)
    paged.page_table.copy_(torch.from_numpy(perm))
    return flat, paged


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
@pytest.mark.parametrize("D", [64, 128])
def test_append_read_decode_match_the_contiguous_cache(va, fmt, D):
    B, Hq, Hkv, S_max, P = 3, 8, 2, 512, 128
    flat, paged = _pair(va, fmt, B, Hkv, S_max, D, P, seed=D)
    rope = va.RopeTable(S_max, D)
    prompts = torch.tensor([300, 17, 129], dtype=torch.int32, device=G.dev())
    T = 300
    q, k, v = I.qkv(6000 + D, B, Hq, Hkv, T, T, D, scale=0.5)
    for c in (flat, paged):
        c.append(G.f32_dev(k), G.f32_dev(v), n_new=prompts, q=G.f32_dev(q), rope=rope, q_dtype=torch.bfloat16)
    assert flat.seq_lens.cpu().tolist() == paged.seq_lens.cpu().tolist() == [300, 17, 129]
    # logical read-back over the whole capacity: identical, including the garbage rows past each length
    kf, vf = flat.read(0, 320, torch.bfloat16)
    kp, vp = paged.read(0, 320, torch.bfloat16)
    lens = [300, 17, 129]
    for b in range(B):
        assert torch.equal(kf[b, :, :lens[b]], kp[b, :, :lens[b]]) and torch.equal(vf[b, :, :lens[b]], vp[b, :, :lens[b]])
    if fmt == "q8_0":
        for plane in (0, 1):
            qf_, sf_ = flat.read_q8_0(plane, 0, 128)
            qp_, sp_ = paged.read_q8_0(plane, 0, 128)
            assert torch.equal(qf_[1, :, :17], qp_[1, :, :17]) and torch.equal(sf_[1, :, :17], sp_[1, :, :17])
    # token-by-token decode with appends crossing page boundaries (129 -> 130, ...)
    for step in range(4):
        qd, kd, vd = I.qkv(6100 + step, B, Hq, Hkv, 1, 1, D, scale=0.5)
        outs = []
        for c in (flat, paged):
            qr = c.append(G.f32_dev(kd), G.f32_dev(vd), q=G.f32_dev(qd), rope=rope, q_dtype=torch.bfloat16)
            outs.append(c.decode(qr))
        assert torch.equal(outs[0], outs[1]), f"decode step {step}"
        assert torch.isfinite(outs[1].float()).all()


def test_decode_against_the_oracle_and_shared_prefix_pages(va):
    # two sequences share their first page (a common prompt prefix stored once); each decodes as if it owned a copy
    B, Hq, Hkv, D, P, S_max = 2, 8, 2, 128, 64, 256
    c = va.RaggedKVCache(B, Hkv, S_max, D, fmt="bf16", paging=(P, 8))
    c.page_table.copy_(torch.tensor([[5, 2, 7, 0], [5, 3, 1, 4]], dtype=torch.int32))
    q, k, v = [O.bf16_round(x) for x in I.qkv(6200, B, Hq, Hkv, 100, 100, D, scale=0.5)]
    k[1, :, :P], v[1, :, :P] = k[0, :, :P], v[0, :, :P]  # the shared prefix
    c.append(G.to_bf16_dev(k), G.to_bf16_dev(v))
    assert c.seq_lens.cpu().tolist() == [100, 100]
    qd = O.bf16_round(I.normal(6201, (B, Hq, 1, D), 0.5))
    out = G.bf16_to_np(c.decode(G.to_bf16_dev(qd)))
    for b in range(B):
        want = O.gqa_attention(qd[b:b + 1], k[b:b + 1], v[b:b + 1], causal=False)
        G.assert_bf16_close(out[b:b + 1], want, f"row {b}")


def test_validation(va):
    with pytest.raises(va.VspError):   # page size not a multiple of 64
        va.KVCache(1, 2, 96, 64, fmt="bf16", paging=(48, 4))
    with pytest.raises(va.VspError):   # fp32 caches are not paged
        va.KVCache(1, 2, 128, 64, fmt="f32", paging=(64, 4))
    with pytest.raises(va.VspError):   # capacity not a whole number of pages
        va.KVCache(1, 2, 100, 64, fmt="bf16", paging=(64, 4))
    c = va.RaggedKVCache(1, 2, 128, 64, fmt="bf16", paging=(64, 4))
    c.page_table.copy_(torch.tensor([[1, 3]], dtype=torch.int32))


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
def test_chunked_prefill_over_pages_matches_the_contiguous_cache(va, fmt):
    B, Hq, Hkv, D, S_max, P = 3, 8, 2, 128, 640, 128
    flat, paged = _pair(va, fmt, B, Hkv, S_max, D, P, seed=11)
    lens = [500, 130, 333]
    T = 100
    q, k, v = [O.bf16_round(x) for x in I.qkv(6300, B, Hq, Hkv, 500, 500, D, scale=0.5)]
    n0 = torch.tensor([l - T for l in lens], dtype=torch.int32, device=G.dev())
    outs = []
    for c in (flat, paged):
        c.append(G.to_bf16_dev(k[:, :, :400]), G.to_bf16_dev(v[:, :, :400]), n_new=n0)      # the context
        chunk_k = np.stack([k[b, :, lens[b] - T:lens[b]] for b in range(B)])
        chunk_v = np.stack([v[b, :, lens[b] - T:lens[b]] for b in range(B)])
        c.append(G.to_bf16_dev(chunk_k), G.to_bf16_dev(chunk_v))                            # the chunk, crossing pages
        chunk_q = np.stack([q[b, :, lens[b] - T:lens[b]] for b in range(B)])
        outs.append(c.prefill_chunk(G.to_bf16_dev(chunk_q)))
    assert paged.seq_lens.cpu().tolist() == lens
    assert torch.equal(outs[0], outs[1])
    # and against the oracle, on what the cache holds
    kk, vv = (k, v) if fmt == "bf16" else (O.q8_0_dequantize(*O.q8_0_quantize(k)), O.q8_0_dequantize(*O.q8_0_quantize(v)))
    got = G.bf16_to_np(outs[1])
    for b in range(B):
        L = lens[b]
        want = O.flash_attention(q[b:b + 1, :, :L], O.repeat_kv(kk[b:b + 1, :, :L], 4), O.repeat_kv(vv[b:b + 1, :, :L], 4),
                                 float(np.float32(1.0 / np.sqrt(D))), True)[:, :, L - T:]
        G.assert_bf16_close(got[b:b + 1], want, f"row {b}")
