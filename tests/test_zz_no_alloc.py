"""vsp_attn_decode_noalloc (the decode entry point that allocates nothing: split-K partials in the library's
fixed per-GPU array) against vsp_attn_decode with a caller workspace, bit for bit, on two calls in a row, the
second with a smaller input (so stale partials of the first call sit in the array while it runs)."""
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


def _case(va, fmt, seed, B, Hq, Hkv, S, D, lens):
    q, k, v = I.qkv(seed, B, Hq, Hkv, 1, S, D)
    c = va.KVCache(B, Hkv, S, D, fmt=fmt)
    c.update(G.f32_dev(k), G.f32_dev(v), 0, return_views=False)
    qd = G.f32_dev(q) if fmt == "f32" else G.to_bf16_dev(O.bf16_round(q))
    sl = torch.tensor(lens, dtype=torch.int32, device=G.dev())
    return c, qd, sl, (O.bf16_round(q) if fmt != "f32" else q, k, v)


@pytest.mark.parametrize("fmt", ["bf16", "q8_0", "f32"])
def test_noalloc_decode_matches_workspace_decode_twice(va, fmt):
    big = _case(va, fmt, 71, 3, 16, 4, 2304, 128, [2304, 1500, 9])
    small = _case(va, fmt, 75, 2, 8, 2, 320, 128 if fmt != "f32" else 64, [300, 41])
    for name, (c, qd, sl, host) in (("first (larger)", big), ("second (smaller)", small)):
        print(f"noalloc decode {fmt} {name}", flush=True)
        want = va.decode_attention(qd, c, seq_lens=sl)
        out = torch.full_like(qd, float("nan"))
        # the number of allocations torch's caching allocator has served must not move (frees by Python's garbage
        # collector may happen at any time and are not counted)
        before = torch.cuda.memory_stats().get("allocation.all.allocated", 0)
        va.decode_attention_noalloc(qd, c, out, seq_lens=sl)
        assert torch.cuda.memory_stats().get("allocation.all.allocated", 0) == before
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16 if fmt != "f32" else torch.int32),
                           want.view(torch.int16 if fmt != "f32" else torch.int32)), f"{fmt} {name}"
    # and the result is the oracle's (bf16 path; the others follow from bit-equality with the tested entry point)
    if fmt == "bf16":
        c, qd, sl, (q, k, v) = small
        k, v = O.bf16_round(k), O.bf16_round(v)
        ref = np.zeros_like(q)
        for b, L in enumerate([300, 41]):
            ref[b:b + 1] = O.gqa_attention(q[b:b + 1], k[b:b + 1, :, :L], v[b:b + 1, :, :L], causal=False)
        G.assert_bf16_close(G.bf16_to_np(out), ref, "noalloc decode vs oracle")


def test_noalloc_decode_rejects_oversized_requests(va):
    # partials of B*Hq*splits*(D+2)*4 bytes above the fixed 32 MiB: refused on the host before any launch.
    # (The planes are never touched, so a small dummy allocation stands in for them: the size check comes first.)
    import ctypes as C
    from vesper_amd import _ffi
    B, Hq, Hkv, S, D = 64, 128, 8, 65536, 128
    c = _ffi.VspKVCache()
    c.format, c.B, c.Hkv, c.S_max, c.D = _ffi.KV_BF16, B, Hkv, S, D
    dummy = torch.zeros(1024, dtype=torch.uint8, device=G.dev())
    c.k = c.v = dummy.data_ptr()
    c.len = S
    q = torch.zeros(B, Hq, 1, D, dtype=torch.bfloat16, device=G.dev())
    out = torch.empty_like(q)
    with pytest.raises(va.VspError) as e:
        va.api.check(_ffi.lib.vsp_attn_decode_noalloc(C.byref(va.api._desc(q)), C.byref(c), None, 0,
                                                      C.byref(va.api._desc(out)), 0.1, None))
    assert e.value.status == _ffi.ERR_WORKSPACE


def test_noalloc_decode_with_an_empty_context_skips_the_size_check(va):
    # nothing is attended to and no partial is written, so the 32 MiB bound does not apply: zeros, as vsp_attn_decode
    B, Hq, Hkv, S, D = 64, 128, 8, 65536, 128
    import ctypes as C
    from vesper_amd import _ffi
    c = _ffi.VspKVCache()
    c.format, c.B, c.Hkv, c.S_max, c.D = _ffi.KV_BF16, B, Hkv, S, D
    dummy = torch.zeros(1024, dtype=torch.uint8, device=G.dev())
    c.k = c.v = dummy.data_ptr()
    c.len = 0
    q = torch.ones(B, Hq, 1, D, dtype=torch.bfloat16, device=G.dev())
    out = torch.full_like(q, float("nan"))
    va.api.check(_ffi.lib.vsp_attn_decode_noalloc(C.byref(va.api._desc(q)), C.byref(c), None, 0,
                                                  C.byref(va.api._desc(out)), 0.1, None))
    torch.cuda.synchronize()
    assert torch.count_nonzero(out.float()).item() == 0


def test_noalloc_decode_replays_from_a_graph_after_one_eager_call(va):
    # the first call on a device looks the array up and must be eager; after it the entry point can be captured
    c, qd, sl, _ = _case(va, "bf16", 81, 3, 16, 4, 640, 128, [640, 200, 33])
    q2 = G.to_bf16_dev(O.bf16_round(I.normal(82, tuple(qd.shape))))
    eager = []
    for q in (qd, q2, qd):
        o = torch.empty_like(q)
        va.decode_attention_noalloc(q, c, o, seq_lens=sl, max_len=640)
        eager.append(o)
    torch.cuda.synchronize()
    sq, out = torch.empty_like(qd), torch.empty_like(qd)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            va.decode_attention_noalloc(sq, c, out, seq_lens=sl, max_len=640)
    torch.cuda.synchronize()
    for i, q in enumerate((qd, q2, qd)):
        sq.copy_(q)  # eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager[i]), f"replay {i}"
