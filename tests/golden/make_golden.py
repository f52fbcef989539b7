"""Writes tests/golden/*.npz from the REAL reference (oracle/_ref/libvesper_ref.so).

Run in the authoring container only (needs /root/reference to have been compiled by
`make -C oracle ref`):   python tests/golden/make_golden.py
The fixtures hold inputs (or their seed + SHA-256) and the reference's outputs; no
reference source travels.  tests/test_oracle_golden.py checks the oracle against them
bit-for-bit, so the oracle stays pinned on machines where the reference is absent.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import _inputs as I  # noqa: E402
import _oracle as O  # noqa: E402

assert O.ref is not None, "build oracle/_ref first: make -C oracle ref"


def save(name, **arrays):
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
    print("wrote", name, {k: getattr(v, "shape", None) for k, v in arrays.items()})


def flash_cases():
    # the four size tuples of the reference's tests/test_flash_attention.cpp:110-179, causal and not,
    # plus ragged N (not a multiple of the 32-row blocks) and D=128.
    out = {}
    cases = [(1, 1, 8, 32), (2, 4, 64, 64), (1, 8, 128, 64), (4, 2, 32, 128), (1, 2, 77, 64), (1, 1, 200, 128)]
    for ci, (B, H, N, D) in enumerate(cases):
        for causal in (0, 1):
            seed = 100 + 10 * ci
            q, k, v = I.qkv(seed, B, H, H, N, N, D)
            scale = np.float32(1.0 / np.sqrt(D))
            o, lse = O.ref_flash_attention(q, k, v, float(scale), bool(causal))
            tag = f"c{ci}_{causal}"
            out[tag + "_meta"] = np.array([B, H, N, D, causal, seed], np.int64)
            out[tag + "_scale"] = np.array([scale], np.float32)
            out[tag + "_insha"] = np.frombuffer(bytes.fromhex(I.sha(q) + I.sha(k) + I.sha(v)), np.uint8)
            out[tag + "_out"] = o
            out[tag + "_lse"] = lse
    save("flash_attention", **out)


def config1():
    # benchmark config 1: causal GQA fp32, B1, 8 q heads / 2 kv heads, D64, N256, scale 1/8:
    # repeat_kv -> flash_attention, and the same through scaled_dot_product_attention (N<512 => matmul branch).
    B, Hq, Hkv, N, D = 1, 8, 2, 256, 64
    q, k, v = I.qkv(1001, B, Hq, Hkv, N, N, D)
    kr, vr = O.ref_repeat_kv(k, Hq // Hkv), O.ref_repeat_kv(v, Hq // Hkv)
    o_flash, lse = O.ref_flash_attention(q, kr, vr, 0.125, True)
    o_sdpa = O.ref_sdpa(q, kr, vr, True)
    save("config1", meta=np.array([B, Hq, Hkv, N, D, 1001], np.int64),
         insha=np.frombuffer(bytes.fromhex(I.sha(q) + I.sha(k) + I.sha(v)), np.uint8),
         out_flash=o_flash, lse=lse, out_sdpa=o_sdpa)


def sdpa_cases():
    out = {}
    # (B,H,T,L,D,causal): square causal/non-causal, cross shapes (T != L), decode shapes (T=1), T>=512 flash route
    cases = [(2, 2, 16, 16, 32, 1), (2, 2, 16, 16, 32, 0), (1, 4, 64, 128, 64, 0), (2, 3, 1, 300, 64, 0),
             (1, 2, 1, 1, 128, 0), (1, 1, 512, 512, 64, 1), (1, 2, 4, 4, 2, 1)]
    for ci, (B, H, T, L, D, causal) in enumerate(cases):
        seed = 300 + 10 * ci
        q, k, v = I.qkv(seed, B, H, H, T, L, D)
        o = O.ref_sdpa(q, k, v, bool(causal))
        tag = f"s{ci}"
        out[tag + "_meta"] = np.array([B, H, T, L, D, causal, seed], np.int64)
        out[tag + "_insha"] = np.frombuffer(bytes.fromhex(I.sha(q) + I.sha(k) + I.sha(v)), np.uint8)
        out[tag + "_out"] = o
    save("sdpa", **out)


def repeat_kv_case():
    x = np.arange(2 * 2 * 3 * 4, dtype=np.float32).reshape(2, 2, 3, 4)
    save("repeat_kv", x=x, out2=O.ref_repeat_kv(x, 2), out4=O.ref_repeat_kv(x, 4))


def kv_cache_cases():
    # a scripted sequence of updates (prefill, appends, an overwrite in the middle, a reset),
    # recording after every step: the returned views, the length, and the error text if it threw.
    B, H, S_max, D = 2, 3, 16, 8
    steps = [(5, 0), (1, 5), (1, 6), (3, 2), (4, 7), (1, 11), ("reset", 0), (2, 0), (1, 2), (6, 10), (1, 15),
             (1, 16), (2, 15), (1, -1), (0, 3)]
    out = {"shape": np.array([B, H, S_max, D], np.int64)}
    for gqa in (0, 1):
        c = O.RefKVCache(B, H, S_max, D, gqa=bool(gqa))
        for si, (T, pos) in enumerate(steps):
            tag = f"g{gqa}_s{si}"
            if T == "reset":
                c.reset()
                out[tag + "_op"] = np.array([-1, 0], np.int64)
                out[tag + "_len"] = np.array([c.current_seq_len()], np.int64)
                continue
            nk = I.normal(5000 + si, (B, H, T, D))
            nv = I.normal(6000 + si, (B, H, T, D))
            out[tag + "_op"] = np.array([T, pos], np.int64)
            try:
                kview, vview = c.update(nk, nv, pos)
                out[tag + "_err"] = np.array([0], np.int64)
                out[tag + "_k"] = kview
                out[tag + "_v"] = vview
                if not gqa:
                    out[tag + "_viewmeta"] = c.last_view_meta.copy()
            except O.RefError as e:
                out[tag + "_err"] = np.array([1], np.int64)
                out[tag + "_msg"] = np.frombuffer(str(e).encode(), np.uint8)
            out[tag + "_len"] = np.array([c.current_seq_len()], np.int64)
    save("kv_cache", **out)


def gqa_core_cases():
    # cache->update -> repeat_kv -> SDPA as in GroupedQueryAttention::forward(x, cache, start_pos):
    # prefill 8 tokens then 3 single-token decodes (the intent of tests/test_gqa_chapter33.cpp:236-271),
    # B2, 8 q heads / 2 kv heads, D64, S_max 32 (partial-length views -> contiguous copies, see ref_shim).
    B, Hq, Hkv, D, S_max = 2, 8, 2, 64, 32
    c = O.RefKVCache(B, Hkv, S_max, D)
    out = {"meta": np.array([B, Hq, Hkv, D, S_max], np.int64)}
    pos = 0
    for si, T in enumerate([8, 1, 1, 1]):
        q, nk, nv = I.qkv(7000 + 10 * si, B, Hq, Hkv, T, T, D)
        out[f"s{si}_op"] = np.array([T, pos], np.int64)
        out[f"s{si}_out"] = c.gqa_core(q, nk, nv, pos, make_contiguous=True)
        pos += T
    # and one case where the view is full-length, calling the reference exactly as written
    c2 = O.RefKVCache(1, 2, 12, 64)
    q, nk, nv = I.qkv(7100, 1, 8, 2, 12, 12, 64)
    out["full_out"] = c2.gqa_core(q, nk, nv, 0, make_contiguous=False)
    save("gqa_core", **out)


def rope_cases():
    # functional::compute_rope_frequencies + apply_rotary_emb (src/nn/functional.cpp:424-494): angle tables
    # at several (seq_len, head_dim, start_pos, theta); rotations of seeded inputs; and the cached attention
    # sequence with RoPE as GroupedQueryAttention::forward(x, cache, start_pos) runs it
    # (src/nn/gqa_attention.cpp:124-148): prefill 8 tokens, then 3 single-token steps.
    out = {}
    cfgs = [(4, 4, 0, 10000.0), (16, 64, 0, 10000.0), (5, 128, 1000, 10000.0), (3, 128, 32765, 500000.0)]
    out["cfgs"] = np.array(cfgs, np.float64)
    for ci, (S, D, sp, th) in enumerate(cfgs):
        ang = O.ref_rope_angles(S, D, sp, th)
        x = I.normal(8000 + ci, (2, 3, S, D))
        out[f"c{ci}_angles"] = ang
        out[f"c{ci}_x_sha"] = np.frombuffer(bytes.fromhex(I.sha(x)), np.uint8)
        out[f"c{ci}_out"] = O.ref_rope_apply(x, ang)
    B, Hq, Hkv, D, S_max = 2, 8, 2, 64, 32
    c = O.RefKVCache(B, Hkv, S_max, D)
    out["meta"] = np.array([B, Hq, Hkv, D, S_max], np.int64)
    pos = 0
    for si, T in enumerate([8, 1, 1, 1]):
        q, nk, nv = I.qkv(8100 + 10 * si, B, Hq, Hkv, T, T, D)
        out[f"s{si}_op"] = np.array([T, pos], np.int64)
        out[f"s{si}_qrot"], out[f"s{si}_out"] = c.gqa_rope_core(q, nk, nv, pos)
        pos += T
    save("rope", **out)


def backward_cases():
    # ops::flash_attention_backward (src/ops/flash_attention.cpp:165-216, :366-482) on the forward's own out/lse:
    # the shape of the reference's own test (tests/test_flash_attention.cpp:292-340), a ragged causal one, a
    # non-causal one and D=128.
    out = {}
    for tag, (B, H, N, D, causal, seed) in {"t16": (1, 2, 16, 32, 1, 9000), "r70": (2, 3, 70, 64, 1, 9010),
                                            "nc33": (1, 2, 33, 64, 0, 9020), "d128": (1, 2, 130, 128, 1, 9030)}.items():
        q, k, v = I.qkv(seed, B, H, H, N, N, D)
        dout = I.normal(seed + 5, (B, H, N, D))
        scale = float(np.float32(1.0 / np.sqrt(D)))
        o, lse = O.ref_flash_attention(q, k, v, scale, bool(causal))
        dq, dk, dv = O.ref_flash_attention_backward(dout, q, k, v, o, lse, scale, bool(causal))
        out[tag + "_meta"] = np.array([B, H, N, D, causal, seed], np.int64)
        out[tag + "_dq"], out[tag + "_dk"], out[tag + "_dv"] = dq, dk, dv
    save("flash_backward", **out)


def bf16_vectors():
    rng = np.random.default_rng(42)
    bits = np.concatenate([
        rng.integers(0, 2**32, size=4096, dtype=np.uint64).astype(np.uint32),
        np.array([0, 0x80000000, 0x3F800000, 0x3F808000, 0x3F818000, 0x3F807FFF, 0x3F808001, 0x7F7FFFFF,
                  0x7F800000, 0xFF800000, 0x00000001, 0x00008000, 0x00018000, 0x7F7F8000, 0x7FC00000,
                  0x7F800001, 0x7FFFFFFF], np.uint32)])
    f = bits.view(np.float32)
    out = np.array([O.ref.vref_f32_to_bf16(float(x)) if not np.isnan(x) else 0 for x in f], np.uint16)
    # NaNs cannot be passed through a C float argument reliably bit-for-bit; keep non-NaN inputs only
    keep = ~np.isnan(f)
    save("bf16", bits=bits[keep], bf16=out[keep])


if __name__ == "__main__":
    flash_cases()
    config1()
    sdpa_cases()
    repeat_kv_case()
    kv_cache_cases()
    gqa_core_cases()
    rope_cases()
    backward_cases()
    bf16_vectors()
