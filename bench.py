#!/usr/bin/env python3
"""Benchmark of the attention hot path on ONE MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2|p4k|c3|c2f|c4|c5|c4f|c4p|c4w|c4m|c2c|c3c|k512|r2|b2|b3|b2s|b3r|b2f] [--no-cpu] [--no-extra]

A "step" is one pass of the hot path over one batch of synthetic input that is already resident in
HBM: one prefill launch (c2, p4k, c3) or one decode call = split-K kernel + combine kernel (c4, c5).
Prints ONE JSON line.  `value` is the primary workload's throughput (benchmark config 2 by default:
causal GQA prefill bf16, B4, 32/8 heads, D128, N2048, in TFLOP/s of algorithmic causal FLOPs
2*D*B*Hq*N*(N+1)); `other_workloads` carries the remaining benchmark configs (decode in GB/s of
algorithmic KV bytes).  `roofline` is for the primary workload's dominant kernel, timed with events
on the launch stream; `cpu_baseline` is the reference's own CPU path (oracle/_ref, else the oracle
port) timed on this host on a bounded sample of the same workload.  `yardsticks` (with the other workloads) says what
the same box sustains on the bf16 matrix cores outside this library: the vendor GEMM behind torch.matmul and torch's own
attention on config 2's tensors; context for the fractions, nothing else.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
HBM_PEAK_GBS = 8000.0

WORKLOADS = {
    "c2": dict(kind="prefill", B=4, Hq=32, Hkv=8, D=128, N=2048,
               name="BASELINE config 2: causal GQA prefill bf16, B4, 32 q / 8 kv heads, D128, N2048"),
    "p4k": dict(kind="prefill", B=2, Hq=32, Hkv=8, D=128, N=4096,
                name="4k-context point: causal GQA prefill bf16, B2, 32 q / 8 kv heads, D128, N4096"),
    "c3": dict(kind="prefill", B=1, Hq=32, Hkv=8, D=128, N=8192,
               name="BASELINE config 3: causal GQA prefill bf16, B1, 32 q / 8 kv heads, D128, N8192"),
    "c2f": dict(kind="prefill_split", B=4, Hq=32, Hkv=8, D=128, N=2048,
                name="config 2's shape with fp32 tensors through the bf16 matrix cores (operands as two bf16 terms, three MFMAs "
                     "per product, within the fp32 bar of 1e-4): causal GQA prefill, B4, 32 q / 8 kv heads, D128, N2048; "
                     "algorithmic FLOPs, against the bf16 MFMA peak"),
    "c4": dict(kind="decode", fmt="bf16", B=32, Hq=32, Hkv=8, D=128, S=32768, lens=(1024, 32768, 4004),
               name="BASELINE config 4: batched decode bf16 KV cache, B32, 32 q / 8 kv heads, D128, L~U[1024,32768]"),
    "c5": dict(kind="decode", fmt="q8_0", B=16, Hq=64, Hkv=8, D=128, S=65536, lens=None,
               name="BASELINE config 5: decode over Q8_0 KV cache, B16, 64 q / 8 kv heads, D128, L=65536"),
    "c4f": dict(kind="decode", fmt="f32", B=32, Hq=32, Hkv=8, D=128, S=32768, lens=(1024, 32768, 4004),
                name="config 4 with the reference's own fp32 cache layout (fp32 q, fp32 matrix instructions): B32, 32 q / 8 kv heads, "
                     "D128, L~U[1024,32768]; algorithmic bytes = the fp32 K and V rows"),
    "c4p": dict(kind="decode", fmt="bf16", B=32, Hq=32, Hkv=8, D=128, S=32768, lens=(1024, 32768, 4004), page=256,
                name="config 4 over a paged cache: pages of 256 tokens in a shuffled page table, otherwise as config 4"),
    "c4w": dict(kind="decode", fmt="bf16", B=32, Hq=32, Hkv=8, D=128, S=32768, lens=(1024, 32768, 4004), proj=True,
                name="config 4 through the module's output projection: decode as config 4, heads merged, y = x Wo^T with "
                     "Wo [4096, 4096] bf16 in the same call (algorithmic bytes: KV + Wo)"),
    "c4m": dict(kind="decode", fmt="bf16", B=32, Hq=32, Hkv=8, D=128, S=32768, lens=(1024, 32768, 4004), tokens=4,
                name="config 4 with four tokens per sequence in one decode step (speculative verification: the tokens and the query "
                     "heads of a kv head share the MFMA columns, K/V read once per kv head): otherwise as config 4; algorithmic "
                     "bytes = config 4's KV rows + the four tokens' q / out"),
    "c2c": dict(kind="prefill_cached", fmt="bf16", B=4, Hq=32, Hkv=8, D=128, N=2048,
                name="config 2 through the cache: causal GQA prefill bf16 reading K/V from the bf16 cache planes, "
                     "B4, 32 q / 8 kv heads, D128, N2048"),
    "c3c": dict(kind="prefill_cached", fmt="bf16", B=1, Hq=32, Hkv=8, D=128, N=8192,
                name="config 3 through the cache: causal GQA prefill bf16 reading K/V from the bf16 cache planes, "
                     "B1, 32 q / 8 kv heads, D128, N8192"),
    "k512": dict(kind="prefill_cached", fmt="bf16", B=1, Hq=32, Hkv=8, D=128, N=32768, T=512,
                 name="one chunk of a long prompt: the last 512 tokens of a 32768-token context read from the bf16 cache planes, "
                      "B1, 32 q / 8 kv heads, D128 (128 workgroups of queries: the context is split over workgroups and merged by "
                      "the decode step's combine kernel)"),
    "b2": dict(kind="backward", B=4, Hq=32, Hkv=8, D=128, N=2048, fast=False,
               name="attention backward at config 2's shape: causal GQA bf16 in/out, bf16 MFMA with fp32 accumulation, "
                    "B4, 32 q / 8 kv heads, D128, N2048 (dq, dk, dv; 2.5 x the forward's FLOPs); the small workspace: dS "
                    "recomputed in the dQ pass, which is the faster path at this context length"),
    "b3": dict(kind="backward", B=1, Hq=32, Hkv=8, D=128, N=8192, fast=True,
               name="attention backward at config 3's shape: causal GQA bf16 in/out, bf16 MFMA with fp32 accumulation, "
                    "B1, 32 q / 8 kv heads, D128, N8192 (dq, dk, dv; 2.5 x the forward's FLOPs); dS computed once and kept as "
                    "bf16 tiles in the workspace (vsp_attn_backward_fast_workspace_bytes), the faster path from 4096 tokens on"),
    "b2s": dict(kind="backward", B=4, Hq=32, Hkv=8, D=128, N=2048, fast=True,
                name="attention backward at config 2's shape with dS computed once and kept as bf16 tiles in the larger "
                     "workspace (five tile products for five)"),
    "b3r": dict(kind="backward", B=1, Hq=32, Hkv=8, D=128, N=8192, fast=False,
                name="attention backward at config 3's shape with the small workspace: dS recomputed in the dQ pass (seven tile "
                     "products for five)"),
    "b2f": dict(kind="backward_split", B=4, Hq=32, Hkv=8, D=128, N=2048,
                name="attention backward at config 2's shape with fp32 tensors through the bf16 matrix cores (operands as two "
                     "bf16 terms, three MFMAs per product, fp32 gradients, within the fp32 bar of 1e-4): causal GQA, B4, "
                     "32 q / 8 kv heads, D128, N2048; algorithmic FLOPs, against the bf16 MFMA peak"),
    "r2": dict(kind="rope", fmt="bf16", B=4, Hq=32, Hkv=8, D=128, N=2048,
               name="RoPE + KV append for config 2: q/k/v bf16 views of one fused projection buffer [B,T,(Hq+2Hkv)D], "
                    "rotated q out bf16, bf16 cache, B4, 32 q / 8 kv heads, D128, T2048"),
}


def rope_bytes(w):
    e = 2  # bf16 in, bf16 out
    return float(w["B"] * w["N"] * w["D"] * e * (2 * w["Hq"] + 4 * w["Hkv"]) + w["N"] * w["D"] * 4)


def prefill_flops(w):
    T = w.get("T", w["N"])  # the last T rows of the causal triangle over N keys
    return 4.0 * w["D"] * w["B"] * w["Hq"] * (T * (w["N"] - T) + T * (T + 1) / 2.0)


def decode_bytes(w, lens):
    esz = {"bf16": 2, "f32": 4}.get(w["fmt"])
    row = esz * w["D"] if esz else (w["D"] + 2 * (w["D"] // 32))  # bytes per (token, kv head) per plane
    return float(sum(2 * w["Hkv"] * int(L) * row for L in lens) + w["B"] * w["Hq"] * w.get("tokens", 1) * w["D"] * 2 * (esz or 2))


def prefill_kernel_name(torch, B, Hq, N, planes):
    """The library's own choice between its two head_dim-128 bf16 kernels (launch_prefill in csrc/prefill.hip): the general
    kernel for contexts up to 2560 tokens on a grid of at least 3 x CUs workgroups, the software-pipelined one otherwise."""
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    short = N <= 2560 and -(-N // 128) * B * Hq >= 3 * cus
    p = "true" if planes else "false"
    return f"prefill_bf16_kernel<128, {p}>" if short else f"prefill_bf16_pipe_kernel<{p}>"


class Runner:
    """Builds the device-resident inputs of one workload and exposes step()."""

    def __init__(self, key, torch, va):
        self.w = w = WORKLOADS[key]
        self.key, self.torch, self.va = key, torch, va
        dev = torch.device("cuda:0")
        g = torch.Generator(device="cuda").manual_seed(1000 + sum(map(ord, key)))
        if w["kind"] == "prefill":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            mk = lambda h: (torch.randn(B, h, N, D, device=dev, generator=g) * 0.5).to(torch.bfloat16)
            self.q, self.k, self.v = mk(Hq), mk(Hkv), mk(Hkv)
            self.scale = 1.0 / math.sqrt(D)
            self.work = prefill_flops(w)
            self.unit, self.peak, self.bound = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS, "mfma"
            self.kernel = prefill_kernel_name(torch, B, Hq, N, False)
        elif w["kind"] == "prefill_split":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            mk = lambda h: torch.randn(B, h, N, D, device=dev, generator=g) * 0.5
            self.q, self.k, self.v = mk(Hq), mk(Hkv), mk(Hkv)
            self.scale = 1.0 / math.sqrt(D)
            self.ws = torch.empty(va._ffi.lib.vsp_attn_prefill_split_workspace_bytes(B, Hq, Hkv, N, N, D), dtype=torch.uint8, device=dev)
            self.work = prefill_flops(w)
            self.unit, self.peak, self.bound = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS, "mfma"
            self.kernel = "split_f32_kernel + prefill_split_kernel<128>"
        elif w["kind"] == "prefill_cached":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            T = w.get("T", N)
            mk = lambda h, n=N: (torch.randn(B, h, n, D, device=dev, generator=g) * 0.5).to(torch.bfloat16)
            self.q = mk(Hq, T)
            self.cache = va.KVCache(B, Hkv, N, D, fmt=w["fmt"])
            self.cache.update(mk(Hkv), mk(Hkv), 0, return_views=False)
            self.work = prefill_flops(w)
            self.unit, self.peak, self.bound = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS, "mfma"
            self.kernel = (prefill_kernel_name(torch, B, Hq, N, True) if T == N else
                           "prefill_bf16_pipe_kernel<true> (context split) + decode_combine_kernel")
        elif w["kind"] == "backward":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            mk = lambda h: (torch.randn(B, h, N, D, device=dev, generator=g) * 0.5).to(torch.bfloat16)
            self.q, self.k, self.v, self.dout = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
            self.scale = 1.0 / math.sqrt(D)
            self.o, self.lse = va.flash_attention(self.q, self.k, self.v, self.scale, True, return_lse=True)
            self.ws = va.backward_workspace(self.q, fast=w["fast"])
            self.work = 2.5 * prefill_flops(w)
            self.unit, self.peak, self.bound = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS, "mfma"
            self.kernel = ("bwd_rowstats_bf16_kernel<128> + bwd_dkdv_bf16_kernel<128, false, true> + bwd_dq_stream_kernel<128> "
                           "(the three launches of one step)" if w["fast"] else
                           "bwd_dq_bf16_kernel<128> + bwd_dkdv_bf16_kernel<128> (the two launches of one step)")
        elif w["kind"] == "backward_split":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            mk = lambda h: torch.randn(B, h, N, D, device=dev, generator=g) * 0.5
            self.q, self.k, self.v, self.dout = mk(Hq), mk(Hkv), mk(Hkv), mk(Hq)
            self.scale = 1.0 / math.sqrt(D)
            ws = torch.empty(va._ffi.lib.vsp_attn_prefill_split_workspace_bytes(B, Hq, Hkv, N, N, D), dtype=torch.uint8, device=dev)
            self.o, self.lse = va.flash_attention_split(self.q, self.k, self.v, self.scale, True, return_lse=True, workspace=ws)
            self.ws = torch.empty(va._ffi.lib.vsp_attn_backward_split_workspace_bytes(B, Hq, Hkv, N, D), dtype=torch.uint8, device=dev)
            self.work = 2.5 * prefill_flops(w)
            self.unit, self.peak, self.bound = "TFLOP/s", MFMA_BF16_PEAK_TFLOPS, "mfma"
            self.kernel = "bwd_split_kernel + bwd_dq_bf16_kernel<128, true> + bwd_dkdv_bf16_kernel<128, true> (the three launches of one step)"
        elif w["kind"] == "rope":
            B, Hq, Hkv, D, N = w["B"], w["Hq"], w["Hkv"], w["D"], w["N"]
            fused = (torch.randn(B, N, (Hq + 2 * Hkv) * D, device=dev, generator=g) * 0.5).to(torch.bfloat16)
            self.q = fused[:, :, :Hq * D].view(B, N, Hq, D).transpose(1, 2)
            self.k = fused[:, :, Hq * D:(Hq + Hkv) * D].view(B, N, Hkv, D).transpose(1, 2)
            self.v = fused[:, :, (Hq + Hkv) * D:].view(B, N, Hkv, D).transpose(1, 2)
            self.cache = va.KVCache(B, Hkv, N, D, fmt=w["fmt"])
            self.rope = va.RopeTable(N, D)
            self.out = torch.empty(B, Hq, N, D, device=dev, dtype=torch.bfloat16)
            self.work = rope_bytes(w)
            self.unit, self.peak, self.bound = "GB/s", HBM_PEAK_GBS, "hbm"
            self.kernel = "append_bf16_tile_kernel<unsigned short, true, 128>"
        else:
            import numpy as np
            B, Hq, Hkv, D, S = w["B"], w["Hq"], w["Hkv"], w["D"], w["S"]
            if w["lens"]:
                lo, hi, seed = w["lens"]
                lens = np.random.default_rng(seed).integers(lo, hi + 1, size=B, dtype=np.int64).astype(np.int32)
            else:
                lens = np.full(B, S, np.int32)
            self.lens = lens
            if w.get("page"):
                P = w["page"]
                n_pages = B * (S // P)
                self.cache = va.KVCache(B, Hkv, S, D, fmt=w["fmt"], paging=(P, n_pages))
                perm = np.random.default_rng(7).permutation(n_pages).astype(np.int32).reshape(B, S // P)
                self.cache.page_table.copy_(torch.from_numpy(perm))
                for t0 in range(0, S, 2048):  # fill through the append path, 2048 tokens of every row at a time
                    kb = torch.randn(B, Hkv, 2048, D, device=dev, generator=g).to(torch.bfloat16)
                    vb = torch.randn(B, Hkv, 2048, D, device=dev, generator=g).to(torch.bfloat16)
                    self.cache.update(kb, vb, t0, return_views=False)
                    del kb, vb
            else:
                self.cache = va.KVCache(B, Hkv, S, D, fmt=w["fmt"])
                for b in range(B):  # fill through the append path, a batch row at a time (bounded fp32 temporaries)
                    kb = torch.randn(1, Hkv, S, D, device=dev, generator=g)
                    vb = torch.randn(1, Hkv, S, D, device=dev, generator=g)
                    self._append_row(b, kb, vb)
                    del kb, vb
            self.cache.set_len(S)
            self.seq_lens = torch.from_numpy(lens).to(dev)
            self.q = torch.randn(B, Hq, w.get("tokens", 1), D, device=dev, generator=g).to(torch.float32 if w["fmt"] == "f32" else torch.bfloat16)
            self.out = torch.empty_like(self.q)
            self.scale = 1.0 / math.sqrt(D)
            self.work = decode_bytes(w, lens)
            if w.get("proj"):
                C_ = Hq * D
                self.wo = (torch.randn(C_, C_, device=dev, generator=g) * (1.0 / math.sqrt(C_))).to(torch.bfloat16)
                self.y = torch.empty(B, 1, C_, device=dev, dtype=torch.bfloat16)
                self.work += C_ * C_ * 2
            self.unit, self.peak, self.bound = "GB/s", HBM_PEAK_GBS, "hbm"
            paged = "true" if w.get("page") else "false"
            self.kernel = {"bf16": f"decode_bf16_kernel<128, {paged}>", "q8_0": f"decode_q8_kernel<128, {paged}>",
                           "f32": "decode_f32_mfma_kernel<128>"}[w["fmt"]]
            self.max_len = int(lens.max())

    def _append_row(self, b, kb, vb):
        """Append one batch row's K/V [1,Hkv,S,D] at position 0 of row b via per-sequence start positions."""
        import ctypes as C
        from vesper_amd import _ffi
        from vesper_amd.api import _desc, _stream
        c = self.cache._c
        sub = _ffi.VspKVCache()
        for f, _ in _ffi.VspKVCache._fields_:
            setattr(sub, f, getattr(c, f))
        # window: same planes offset to row b, batch 1
        for plane, name in ((0, "k"), (1, "v"), (2, "k_scale"), (3, "v_scale")):
            nbytes = _ffi.lib.vsp_kv_plane_bytes(c.format, 1, c.Hkv, c.S_max, c.D, plane)
            base = getattr(c, name)
            setattr(sub, name, (base + b * nbytes) if base else None)
        sub.B = 1
        dk, dv = _desc(kb), _desc(vb)
        _ffi.check(_ffi.lib.vsp_kv_append(C.byref(sub), C.byref(dk), C.byref(dv), 0, None, _stream(kb)))

    def step(self):
        if self.w["kind"] == "prefill":
            return self.va.flash_attention(self.q, self.k, self.v, self.scale, True)
        if self.w["kind"] == "prefill_split":
            return self.va.flash_attention_split(self.q, self.k, self.v, self.scale, True, workspace=self.ws)
        if self.w["kind"] == "backward_split":
            return self.va.flash_attention_backward_split(self.dout, self.q, self.k, self.v, self.o, self.lse, self.scale, True,
                                                          workspace=self.ws)
        if self.w["kind"] == "backward":
            return self.va.flash_attention_backward(self.dout, self.q, self.k, self.v, self.o, self.lse, self.scale, True,
                                                    workspace=self.ws)
        if self.w["kind"] == "prefill_cached":
            return self.cache.prefill(self.q)
        if self.w["kind"] == "rope":
            return self.cache.rope_update(self.q, self.k, self.v, 0, self.rope, out=self.out)
        if self.w.get("proj"):
            return self.va.decode_attention_proj(self.q, self.cache, self.wo, None, seq_lens=self.seq_lens, max_len=self.max_len,
                                                 scale=self.scale, out=self.y)
        if self.w.get("tokens", 1) > 1:
            return self.va.decode_attention_multi(self.q, self.cache, seq_lens=self.seq_lens, max_len=self.max_len,
                                                  scale=self.scale, out=self.out)
        return self.va.decode_attention(self.q, self.cache, seq_lens=self.seq_lens, max_len=self.max_len,
                                        scale=self.scale, out=self.out)

    def rate(self, seconds_per_step):
        return self.work / seconds_per_step / (1e12 if self.unit == "TFLOP/s" else 1e9)


CONDITION_SECONDS = 0.3


def condition(torch, fn, seconds=CONDITION_SECONDS):
    """Untimed: keep the GPU busy with the workload for a fixed wall time before the warm-up steps.  The part
    raises its clocks over the first ~50 ms of sustained load (a 0.14 ms kernel takes 0.20 ms right after an
    idle period and settles after ~300 launches); a serving process is always in the settled state, and a
    warm-up counted in steps would measure the ramp for short kernels."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def time_steps(torch, fn, steps, warmup, conditioning=True):
    """clock conditioning and `warmup` steps untimed, then exactly `steps` steps: wall clock bracketed by
    synchronize, and device time from events recorded on the launch stream around the same region.  An event after
    every step gives the per-step durations (median and minimum) without touching the timed region's length."""
    if conditioning:
        condition(torch, fn)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    ev[0].record()
    for i in range(steps):
        fn()
        ev[i + 1].record()
    torch.cuda.synchronize()
    wall = (time.perf_counter() - t0) / steps
    dev = ev[0].elapsed_time(ev[steps]) * 1e-3 / steps
    per_step = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    stats = {"median_ms": round(per_step[len(per_step) // 2], 5), "min_ms": round(per_step[0], 5)}
    return wall, dev, stats


def cpu_baseline(key):
    """The reference's CPU path on a bounded sample of the primary workload, one thread (the path is
    single-threaded in the reference)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import numpy as np
    import _oracle as O
    w = WORKLOADS[key]
    use_ref = O.ref is not None
    kind = "reference" if use_ref else "port"
    rng = np.random.default_rng(1)
    if w["kind"] == "prefill":
        # sample: one full batch row (32 query heads, 8 kv groups) at full N: repeat_kv + flash_attention, fp32
        Hq_s, Hkv_s, N, D = 32, 8, w["N"], w["D"]
        q = O.bf16_round(rng.standard_normal((1, Hq_s, N, D), dtype=np.float32) * 0.5)
        k = O.bf16_round(rng.standard_normal((1, Hkv_s, N, D), dtype=np.float32) * 0.5)
        v = O.bf16_round(rng.standard_normal((1, Hkv_s, N, D), dtype=np.float32) * 0.5)
        scale = float(np.float32(1.0 / math.sqrt(D)))
        t0 = time.perf_counter()
        if use_ref:
            kr, vr = O.ref_repeat_kv(k, 4), O.ref_repeat_kv(v, 4)
            O.ref_flash_attention(q, kr, vr, scale, True)
        else:
            O.flash_attention(q, O.repeat_kv(k, 4), O.repeat_kv(v, 4), scale, True)
        dt = time.perf_counter() - t0
        flops = 2.0 * D * Hq_s * N * (N + 1)
        return dict(value=flops / dt / 1e12, unit="TFLOP/s", cores=1, kind=kind,
                    sample=f"1 batch row x {Hq_s} query heads ({Hkv_s} kv heads) of the workload at N={N}: "
                           f"repeat_kv + flash_attention fp32, {dt:.1f} s; whole workload = x{w['B'] * w['Hq'] // Hq_s}",
                    seconds=dt)
    # decode sample: one sequence, one kv group, fp32 cache: repeat_kv + matmul/softmax/matmul branch
    L, D, n_rep = 8192, w["D"], w["Hq"] // w["Hkv"]
    q = rng.standard_normal((1, n_rep, 1, D), dtype=np.float32)
    k = rng.standard_normal((1, 1, L, D), dtype=np.float32)
    v = rng.standard_normal((1, 1, L, D), dtype=np.float32)
    reps = 6
    t0 = time.perf_counter()
    for _ in range(reps):
        if use_ref:
            O.ref_sdpa(q, O.ref_repeat_kv(k, n_rep), O.ref_repeat_kv(v, n_rep), False)
        else:
            O.sdpa(q, O.repeat_kv(k, n_rep), O.repeat_kv(v, n_rep), False)
    dt = (time.perf_counter() - t0) / reps
    row = 2 * D if w["fmt"] == "bf16" else D + 2 * (D // 32)
    return dict(value=2 * L * row / dt / 1e9, unit="GB/s", cores=1, kind=kind,
                sample=f"one sequence x one kv head ({n_rep} query heads), L={L}, fp32 cache as in the reference: "
                       f"repeat_kv x2 + matmul/div/softmax/matmul, {dt * 1e3:.0f} ms per call x{reps}; "
                       f"rate in the workload's algorithmic KV bytes",
                seconds=dt * reps)


# HBM bytes per launch of the dominant kernel come from the rocprofv3 summaries committed under profiles/ (FETCH_SIZE and
# WRITE_SIZE runs of this script, see the command lines at the top of each file).  The raw counters are scaled by what
# they read for a 1 GiB read + 1 GiB write elementwise kernel launched by --copy-calibration in the same run.  Counters
# cannot be collected inside a timed run, so these are properties of the workload shapes, not live values.
PROFILE_OF = {
    # workload: (summary under profiles/, name fragments of the step's kernels (their counters are added up), algorithmic
    # bytes of a step: every input read once and every output written once)
    "c2": ("prefill_bf16_config2.txt", ("prefill_bf16",), 96 * 2**20 + 65 * 2**20),
    "p4k": ("prefill_bf16_4k.txt", ("prefill_bf16",), 96 * 2**20 + 65 * 2**20),
    "c3": ("prefill_bf16_config3.txt", ("prefill_bf16",), 96 * 2**20 + 65 * 2**20),
    "c2c": ("prefill_bf16_cache_planes_config2.txt", ("prefill_bf16",), 96 * 2**20 + 65 * 2**20),
    "c3c": ("prefill_bf16_cache_planes_config3.txt", ("prefill_bf16",), 96 * 2**20 + 65 * 2**20),
    "k512": ("prefill_bf16_chunk512_context32k.txt", ("prefill_bf16", "decode_combine_kernel"), 2 * 4194304 + 2 * 67108864),
    "c2f": ("prefill_split_f32_config2.txt", ("prefill_split_kernel", "split_f32_kernel"), 2 * 134217728 + 2 * 33554432),
    "r2": ("rope_append_bf16_config2.txt", ("append_bf16_tile_kernel<unsigned short, true",), 202375168),
    "c4": ("decode_bf16_config4.txt", ("decode_bf16_kernel", "decode_combine_kernel"), 2614935552),
    "c4m": ("decode_bf16_multi_config4.txt", ("decode_bf16_kernel", "decode_combine_kernel"), 2614935552 + 3 * 524288),
    "c4p": ("decode_bf16_paged_config4.txt", ("decode_bf16_kernel", "decode_combine_kernel"), 2614935552),
    "c4w": ("decode_bf16_proj_config4.txt", ("decode_bf16_kernel", "decode_combine_kernel", "proj_bf16_partial_kernel", "proj_reduce_kernel"),
            2614935552 + 33554432),
    "c5": ("decode_q8_0_config5.txt", ("decode_q8_kernel", "decode_combine_kernel"), 2282225664),
    "c4f": ("decode_f32_config4.txt", ("decode_f32_mfma_kernel", "decode_combine_kernel"), 5229871104),
    # backward: Q, dO, O, K, V, lse read; dQ, dK, dV written
    "b2": ("backward_bf16_config2.txt", ("bwd_dq_bf16_kernel", "bwd_dkdv_bf16_kernel"), 4 * 67108864 + 4 * 16777216 + 1048576),
    "b3r": ("backward_bf16_config3.txt", ("bwd_dq_bf16_kernel", "bwd_dkdv_bf16_kernel"), 4 * 67108864 + 4 * 16777216 + 1048576),
    # the same tensors in fp32: twice the bytes
    "b2f": ("backward_split_f32_config2.txt", ("bwd_split_kernel", "bwd_dq_bf16_kernel", "bwd_dkdv_bf16_kernel"),
            4 * 134217728 + 4 * 33554432 + 1048576),
    "b2s": ("backward_bf16_stored_ds_config2.txt", ("bwd_rowstats_bf16_kernel", "bwd_dkdv_bf16_kernel", "bwd_dq_stream_kernel"),
            4 * 67108864 + 4 * 16777216 + 1048576),
    "b3": ("backward_bf16_stored_ds_config3.txt", ("bwd_rowstats_bf16_kernel", "bwd_dkdv_bf16_kernel", "bwd_dq_stream_kernel"),
           4 * 67108864 + 4 * 16777216 + 1048576),
}
CALIBRATION_KERNEL, CALIBRATION_KIB = "CUDAFunctorOnSelf_add<int>", 1048576.0


def traffic_from_profile(key):
    """{"fetch_bytes", "write_bytes", "algorithmic_bytes", "source"} parsed from profiles/<file>, or None."""
    if key not in PROFILE_OF:
        return None
    fname, kernels, algorithmic = PROFILE_OF[key]
    path = os.path.join(ROOT, "profiles", fname)
    if not os.path.exists(path):
        return None
    out, section = {}, None
    raw = {"FETCH_SIZE": {}, "WRITE_SIZE": {}}
    for line in open(path):
        if line.startswith("## "):
            section = "FETCH_SIZE" if "FETCH_SIZE" in line else ("WRITE_SIZE" if "WRITE_SIZE" in line else None)
            continue
        if section and section in line:
            left, right = line.rsplit(section, 1)
            cols = right.split()
            if len(cols) >= 2:
                value = float(cols[1])  # columns after the counter name: n, avg, min, max
                if CALIBRATION_KERNEL in left:
                    raw[section].setdefault("calibration", value)
                elif any(k in left for k in kernels):
                    raw[section]["kernel"] = raw[section].get("kernel", 0.0) + value  # one line per kernel and counter
    try:
        for section, field in (("FETCH_SIZE", "fetch_bytes"), ("WRITE_SIZE", "write_bytes")):
            scale = CALIBRATION_KIB / raw[section]["calibration"]
            out[field] = int(raw[section]["kernel"] * scale * 1024)
    except KeyError:
        return None
    out["algorithmic_bytes"] = algorithmic
    out["source"] = "profiles/" + fname
    return out


def yardsticks(torch):
    """What the same box sustains on the bf16 matrix cores outside this library, for scale next to the roofline fractions
    (not a baseline and not part of any figure above): the vendor GEMM behind torch.matmul on 8192^3 bf16 operands, and
    torch's own scaled_dot_product_attention on config 2's tensors."""
    import time as _t

    def rate(fn, flops, n):
        t0 = _t.time()
        while _t.time() - t0 < CONDITION_SECONDS:
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return round(flops / (e0.elapsed_time(e1) / n * 1e-3) / 1e12, 1)

    out = {"note": "same box, same process; outside this library (torch.matmul -> vendor GEMM, torch SDPA); TFLOP/s"}
    g = torch.Generator(device="cuda").manual_seed(5)
    mk = lambda *shape: (torch.randn(*shape, device="cuda:0", generator=g) * 0.5).to(torch.bfloat16)
    try:
        a, b = mk(8192, 8192), mk(8192, 8192)
        out["bf16_gemm_8192_nt"] = rate(lambda: torch.matmul(a, b.t()), 2 * 8192 ** 3, 20)
        out["bf16_gemm_8192_nn"] = rate(lambda: torch.matmul(a, b), 2 * 8192 ** 3, 20)
        del a, b
    except Exception as e:  # a yardstick, never a reason to fail the run
        out["bf16_gemm_error"] = repr(e)[:200]
    try:
        import torch.nn.functional as F
        q, k, v = mk(4, 32, 2048, 128), mk(4, 8, 2048, 128), mk(4, 8, 2048, 128)
        out["torch_sdpa_config2"] = rate(lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True, enable_gqa=True),
                                         2 * 128 * 4 * 32 * 2048 * 2049, 10)
    except Exception as e:
        out["torch_sdpa_error"] = repr(e)[:200]
    torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="only the primary workload")
    ap.add_argument("--no-conditioning", action="store_true",
                    help="skip the fixed 0.3 s of untimed load that lets the clocks settle before the warm-up steps")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one 1 GiB read + 1 GiB write elementwise kernel (counter calibration for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path shards without communication over "
              "batch and kv heads; no multi-GPU figure is produced). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import torch
    import vesper_amd as va  # raises if the HIP library is missing: no fallback

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    props = torch.cuda.get_device_properties(0)

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.int32, device="cuda:0")
        dst = torch.empty_like(src)
        torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst

    primary = Runner(args.workload, torch, va)
    wall, dev, stats = time_steps(torch, primary.step, args.steps, args.warmup, not args.no_conditioning)
    value = primary.rate(wall)
    achieved = primary.rate(dev)
    result = {
        "metric": "prefill attn TFLOP/s (% MFMA peak); decode attn HBM GB/s (% of 8 TB/s)",
        "value": round(value, 3),
        "unit": primary.unit,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3, 5),
        "median_ms": stats["median_ms"],
        "min_ms": stats["min_ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": ("f32 operands as two bf16 terms (bf16 MFMA, fp32 accumulation)" if primary.w["kind"] in ("prefill_split", "backward_split")
                  else {"bf16": "bf16", "f32": "f32", "q8_0": "q8_0 (int8 payload, fp16 MFMA)"}[primary.w.get("fmt", "bf16")]),
        "data": "synthetic",
        "config": {"workload": primary.w["name"], "key": args.workload,
                   "algorithmic_work_per_step": primary.work,
                   "work_unit": "FLOP" if primary.bound == "mfma" else "bytes"},
        "roofline": {"bound": primary.bound, "achieved": round(achieved, 3), "peak": primary.peak,
                     "unit": primary.unit, "frac": round(achieved / primary.peak, 4),
                     "traffic": traffic_from_profile(args.workload),
                     "kernel": primary.kernel, "kernel_ms": round(dev * 1e3, 5),
                     "timing": "HIP events on the launch stream around the timed steps / steps"},
        "clock_state": ("cold start" if args.no_conditioning else
                        f"steady state: {CONDITION_SECONDS} s of untimed load before the warm-up steps (clocks settled)"),
        "clock_conditioning_s": 0.0 if args.no_conditioning else CONDITION_SECONDS,
        "device": {"name": props.name, "cus": props.multi_processor_count,
                   "peak_used": f"{primary.peak} {primary.unit}"},
    }
    del primary
    torch.cuda.empty_cache()

    if not args.no_extra:
        others = {}
        for key in ("c2", "p4k", "c3", "c2f", "c4", "c5", "c4f", "c4p", "c4w", "c4m", "c2c", "c3c", "k512", "r2", "b2", "b3", "b2s", "b3r", "b2f"):
            if key == args.workload:
                continue
            r = Runner(key, torch, va)
            steps = max(50, args.steps)
            w_, d_, st_ = time_steps(torch, r.step, steps, max(3, args.warmup // 2), not args.no_conditioning)
            others[key] = {"workload": r.w["name"], "value": round(r.rate(w_), 3), "unit": r.unit,
                           "ms_per_step": round(w_ * 1e3, 5), "kernel_ms": round(d_ * 1e3, 5),
                           "median_ms": st_["median_ms"], "min_ms": st_["min_ms"],
                           "roofline_frac": round(r.rate(d_) / r.peak, 4), "bound": r.bound, "steps": steps}
            if traffic_from_profile(key):
                others[key]["traffic"] = traffic_from_profile(key)
            del r
            torch.cuda.empty_cache()
        result["other_workloads"] = others
        result["yardsticks"] = yardsticks(torch)

    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(args.workload)
        result["cpu_baseline"]["host_cores_available"] = os.cpu_count()
        # the decode configs get their own CPU figure (a one-sequence slice, about a second each)
        for key in ("c4", "c5"):
            if key in result.get("other_workloads", {}):
                result["other_workloads"][key]["cpu_baseline"] = cpu_baseline(key)

    print(json.dumps(result))


if __name__ == "__main__":
    main()
