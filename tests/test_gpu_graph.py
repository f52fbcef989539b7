"""The decode step (RoPE + append at device-side positions, length advance, split-K decode, combine) recorded
into a HIP graph and replayed: every entry point is asynchronous, allocates nothing and records no memset node, so a
serving loop can replay one graph per token.  Each replay is checked against the same step run eagerly, with the
program's own eager work and synchronisations between replays.  The same for a training step's attention: prefill
forward and backward in one graph."""
import numpy as np
import pytest
import torch

import _gpu as G
import _inputs as I

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def va():
    import vesper_amd
    return vesper_amd


@pytest.mark.parametrize("fmt", ["bf16", "q8_0"])
def test_decode_step_replays_bit_identically(va, fmt):
    B, Hq, Hkv, D, S_max, steps = 4, 16, 4, 128, 512, 4
    rope = va.RopeTable(S_max, D)
    prompts = [100, 37, 250, 5]

    def make_cache():
        c = va.RaggedKVCache(B, Hkv, S_max, D, fmt=fmt)
        P = max(prompts)
        q, k, v = I.qkv(5000, B, Hq, Hkv, P, P, D, scale=0.5)
        c.append(G.f32_dev(k), G.f32_dev(v), n_new=torch.tensor(prompts, dtype=torch.int32, device=G.dev()),
                 q=G.f32_dev(q), rope=rope, q_dtype=torch.bfloat16)
        c.upper = P + steps  # host-side bound for the whole replayed range: the graph's grid must cover it
        return c

    toks = [I.qkv(5100 + 7 * i, B, Hq, Hkv, 1, 1, D, scale=0.5) for i in range(steps)]

    # eager run
    ce = make_cache()
    eager = []
    for q, k, v in toks:
        qr = ce.append(G.f32_dev(k), G.f32_dev(v), q=G.f32_dev(q), rope=rope, q_dtype=torch.bfloat16)
        eager.append(ce.decode(qr).clone())
    torch.cuda.synchronize()

    # graph run: static input/output buffers, one capture, one replay per token
    cg = make_cache()
    sq = torch.empty(B, Hq, 1, D, device=G.dev())
    sk = torch.empty(B, Hkv, 1, D, device=G.dev())
    sv = torch.empty(B, Hkv, 1, D, device=G.dev())
    q_rot = torch.empty(B, Hq, 1, D, device=G.dev(), dtype=torch.bfloat16)
    out = torch.empty_like(q_rot)
    # the graph keeps the workspace's address, so the test owns it (the per-stream default refuses to grow in capture)
    ws = torch.empty(va._ffi.lib.vsp_attn_decode_workspace_bytes(B, Hq, D, S_max), dtype=torch.uint8, device=G.dev())
    lens0 = cg.seq_lens.clone()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            cg.rope_update(sq, sk, sv, 0, rope, start_pos_dev=cg.seq_lens, out=q_rot)
            cg._advance(None, 1, sq)
            va.decode_attention(q_rot, cg, seq_lens=cg.seq_lens, max_len=cg.upper, out=out, workspace=ws)
    torch.cuda.synchronize()
    cg.seq_lens.copy_(lens0)  # capture does not execute; make sure the lengths are the prompt lengths
    for i, (q, k, v) in enumerate(toks):
        sq.copy_(G.f32_dev(q)), sk.copy_(G.f32_dev(k)), sv.copy_(G.f32_dev(v))  # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[i]), f"replay {i}"
    assert cg.seq_lens.cpu().tolist() == [p + steps for p in prompts]


def test_forward_backward_replays_bit_identically(va):
    # a training step's attention (prefill forward with lse, then dq / dk / dv) in one graph: three launches of the
    # backward share a workspace the caller owns, nothing is cleared by a memset node
    B, Hq, Hkv, N, D = 2, 8, 2, 200, 128
    mk = lambda seed, h: G.to_bf16_dev(I.normal(seed, (B, h, N, D), scale=0.5))
    sq, sk, sv, sd = mk(1, Hq), mk(2, Hkv), mk(3, Hkv), mk(4, Hq)
    inputs = [[mk(10 * i + j, h) for j, h in enumerate((Hq, Hkv, Hkv, Hq))] for i in range(1, 4)]
    eager = []
    for q, k, v, d in inputs:
        o, l = va.flash_attention(q, k, v, 0.1, True, return_lse=True)
        eager.append([o.clone()] + [t.clone() for t in va.flash_attention_backward(d, q, k, v, o, l, 0.1, True)])
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            o, l = va.flash_attention(sq, sk, sv, 0.1, True, return_lse=True)
            grads = va.flash_attention_backward(sd, sq, sk, sv, o, l, 0.1, True)
    torch.cuda.synchronize()
    for i, (q, k, v, d) in enumerate(inputs):
        sq.copy_(q), sk.copy_(k), sv.copy_(v), sd.copy_(d)   # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip([o] + list(grads), eager[i]):
            assert torch.equal(got, want), f"replay {i}"


def test_decode_through_the_output_projection_replays_bit_identically(va):
    # the four launches of vsp_attn_decode_proj (split-K decode, combine, projection partials, reduce) in one graph;
    # the workspace, which also carries the merged heads between the launches, belongs to the caller
    B, Hq, Hkv, D, S = 3, 8, 2, 128, 300
    C_ = Hq * D
    dev = G.dev()
    c = va.KVCache(B, Hkv, S, D, fmt="bf16")
    c.update(G.to_bf16_dev(I.normal(21, (B, Hkv, S, D))), G.to_bf16_dev(I.normal(22, (B, Hkv, S, D))), 0, return_views=False)
    lens = torch.tensor([300, 17, 128], dtype=torch.int32, device=dev)
    wo = G.to_bf16_dev(I.normal(23, (C_, C_), scale=1.0 / 32))
    bias = G.to_bf16_dev(I.normal(24, (C_,), scale=0.5))
    qs = [G.to_bf16_dev(I.normal(30 + i, (B, Hq, 1, D))) for i in range(3)]
    eager = [va.decode_attention_proj(q, c, wo, bias, seq_lens=lens).clone() for q in qs]
    torch.cuda.synchronize()
    sq = torch.empty_like(qs[0])
    y = torch.empty(B, 1, C_, dtype=torch.bfloat16, device=dev)
    ws = torch.empty(va._ffi.lib.vsp_attn_decode_proj_workspace_bytes(B, Hq, D, S, C_), dtype=torch.uint8, device=dev)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            va.decode_attention_proj(sq, c, wo, bias, seq_lens=lens, max_len=S, out=y, workspace=ws)
    torch.cuda.synchronize()
    for i, q in enumerate(qs):
        sq.copy_(q)          # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager[i]), f"replay {i}"
