#!/usr/bin/env python3
"""Headline benchmark: SQAttn prefill attention at 128K (Qwen2.5-7B layer shape, FP8-e4m3 P) on one MI355X,
with the 1M-token split-KV decode as the second half of the metric, a roofline object for the dominant
kernel and the reference's fake-quant + SDPA path timed on the host cores.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--seq-len N] [--no-cpu-baseline] [--no-decode]

Prints ONE JSON line on stdout.  A "step" is one full prefill attention call (V pre-pass + main kernel) on
inputs already resident in HBM.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "prefill attn TFLOP/s @128K + decode HBM GB/s @1M, Qwen2.5-7B GQA 28/4 heads"
PEAK_MFMA_BF16_TFLOPS = 2500.0   # MI355X dense bf16/fp16 MFMA
PEAK_MFMA_FP8_TFLOPS = 5000.0    # MI355X dense fp8 MFMA
# Q.K^T (half of the FLOPs) runs on the bf16 pipe, P.V (the other half) on the fp8 pipe in the default mode
PEAK_MFMA_BLEND_TFLOPS = 1.0 / (0.5 / PEAK_MFMA_BF16_TFLOPS + 0.5 / PEAK_MFMA_FP8_TFLOPS)
PEAK_HBM_GBS = 8000.0            # MI355X HBM3E


def prefill_traffic_bytes(N, p_quant):
    """L2<->fabric bytes of one prefill_kernel launch, from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary of this
    shape (profiles/prefill_kernel_128k.traffic.json: counters in KiB, each scaled by what the same counter read for a
    1 GiB copy); None for shapes and P modes the summary does not cover."""
    if N != 131072 or p_quant != 5:
        return None
    try:
        with open(os.path.join(ROOT, "profiles", "prefill_kernel_128k.traffic.json")) as f:
            t = json.load(f)
        return (t["fetch_size_kib"] * t["fetch_scale"] + t["write_size_kib"] * t["write_scale"]) * 1024.0
    except (OSError, KeyError, ValueError):
        return None


P_MODE_NOTE = {
    0: "no P quantisation",
    4: "e4m3 P with the static scale 448 and e4m3 V, fp8 MFMA P.V",
    5: "e4m3 P with a power-of-two block scale per query row and 64-key tile and e4m3 V, block-scaled fp8 MFMA P.V",
}


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def prefill_inputs(torch, N):
    """BASELINE config 2's seeded inputs (CPU generator), uploaded once: q [1,28,N,128], k/v [1,4,N,128]."""
    from longcontext_sqattn_paddle_amd import workloads

    dev = torch.device("cuda:0")
    t0 = time.time()
    q, k, v = workloads.prefill_inputs(1, 28, 4, N, 128, seed=2)
    q, k, v = q.to(dev), k.to(dev), v.to(dev)
    log(f"[bench] prefill inputs N={N} generated and uploaded in {time.time() - t0:.1f}s")
    return q, k, v


def time_prefill(torch, qkv, steps, warmup, p_quant):
    from longcontext_sqattn_paddle_amd.sqattn._prefill import prefill_workspace
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

    q, k, v = qkv
    dev = q.device
    Hq, Hkv, N, D = q.shape[1], k.shape[1], q.shape[2], q.shape[3]
    ws = prefill_workspace(1, Hkv, N, dev)
    out = torch.empty_like(q)
    stream = torch.cuda.current_stream(dev)

    def step():
        attn_causal(q, k, v, "HND", torch.bfloat16, p_quant=p_quant, workspace=ws, out=out)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(stream)
    for _ in range(steps):
        step()
    e1.record(stream)
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / steps
    flops = 4.0 * N * N * D * Hq / 2   # causal half, FlashAttention convention
    # a finite, non-trivial output guards against timing a launch that did nothing
    chk = out[0, :, -1, :].float()
    assert bool(torch.isfinite(chk).all()) and float(chk.abs().sum()) > 0
    return ms, flops


def time_mfma_only(torch, qkv):
    """What the matrix cores sustain when a kernel issues nothing but MFMAs (`sq_probe_mfma_rate`: one workgroup of
    eight waves per CU, operands loaded once): with constant operands, and with operand registers that hold values like
    this workload's -- bf16 words of the benchmark's own K tensor; e4m3 codes of uniform probabilities x 448 and of V.  The
    published peaks are reached on constant operands only: on random ones the chip lowers its clock under the matrix
    cores' switching power.  The last figure is the harmonic blend for half the FLOPs on each pipe, as in P mode 5."""
    from longcontext_sqattn_paddle_amd import _native as NV

    dev = qkv[1].device
    lib = NV.probe_lib()
    nbytes = int(lib.sq_probe_mfma_operand_bytes())
    sink = torch.empty(131072, dtype=torch.float32, device=dev)
    k_words = qkv[1].reshape(-1)[:nbytes // 2].contiguous()
    g = torch.Generator(device=dev).manual_seed(12)
    p8 = (torch.rand(nbytes // 2, device=dev, generator=g) * 448.0).to(torch.float8_e4m3fn)
    v8 = (qkv[2].reshape(-1)[:nbytes // 2].float() * 2.0 ** 12).to(torch.float8_e4m3fn)   # N(0,1)/sqrt(128) scaled into e4m3's range
    f8 = torch.cat([p8.view(torch.uint8), v8.view(torch.uint8)]).contiguous()
    sets = {"bf16_constant": (0, torch.ones(nbytes // 2, dtype=torch.bfloat16, device=dev)), "bf16_workload_values": (0, k_words),
            "e4m3_constant": (1, torch.full((nbytes,), 0x38, dtype=torch.uint8, device=dev)), "e4m3_workload_values": (1, f8)}
    out = {}
    stream = torch.cuda.current_stream(dev)
    for name, (kind, ops) in sets.items():
        iters = 20000 if kind == 0 else 10000
        b = [NV.dl(ops), NV.dl(sink)]
        times = []
        for rep in range(4):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(stream)
            NV.check(lib.sq_probe_mfma_rate(kind, NV.ptr(b[0]), NV.ptr(b[1]), iters, NV.current_stream(dev)), lib)
            e1.record(stream)
            torch.cuda.synchronize()
            times.append(e0.elapsed_time(e1))
        ms = sorted(times[1:])[1]
        out[name] = round(int(lib.sq_probe_mfma_flops(kind, iters)) / ms / 1e9, 1)
    out["blend_workload_values"] = round(1.0 / (0.5 / out["bf16_workload_values"] + 0.5 / out["e4m3_workload_values"]), 1)
    out["unit"] = "TFLOP/s"
    out["note"] = ("a loop of nothing but MFMAs, two waves per SIMD on all 256 CUs, about 10 ms per launch: the published peaks hold for "
                   "constant operands; the figures on workload values are what this GPU sustains on operands like the benchmark's, "
                   "before any load, LDS or vector instruction shares the power budget")
    return out


def time_plugin(torch, qkv, steps=3):
    """The path `ATTN_TYPE=SQAttn` dispatches to (sqattn/attn_replacer.py:423-448): the closure of `mp_triton_wrapper`
    = operand pre-pass (key centring, int8 fake quantisation) + sink/window kernel with relative windows, at the prefill
    benchmark shape in the plugin's [B,N,H,D] layout.  Window settings: the reference's shipped default (ratio 0.1 for
    both windows, sink 256: sqattn/window_search.py:102-104, attn_replacer.py:24) and a wide one (0.25 / 0.5).  For each:
    the whole closure call and the attention kernel alone on operands quantised beforehand."""
    import types

    from longcontext_sqattn_paddle_amd import workloads
    from longcontext_sqattn_paddle_amd.sqattn._prefill import prefill_workspace
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import mp_triton_wrapper
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window, window_tokens
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    q, k, v = (t.permute(0, 2, 1, 3).contiguous() for t in qkv)   # the plugin boundary's layout
    dev = q.device
    N, Hq, D = q.shape[1], q.shape[2], q.shape[3]
    layer = types.SimpleNamespace(num_key_value_groups=Hq // k.shape[2])
    args = types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=True)
    ws = prefill_workspace(1, k.shape[2], N, dev)
    out = {}

    def timed(fn):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    for name, r8, r4, sink in (("default_ratio_0.1_sink_256", 0.1, 0.1, 256), ("ratio_0.25_0.5_sink_256", 0.25, 0.5, 256)):
        closure = mp_triton_wrapper(1, r8, r4, sink, args)
        call_ms = timed(lambda: closure(layer, q, k, v, None))
        q8, _, k8, _, v8 = fused_int_prepass(q, k, v, want_4bit=False, tensor_layout="NHD")
        o = torch.empty_like(q8)
        kern_ms = timed(lambda: attn_hierarchical_relative_window(q8, k8, q8, k8, v8, r8, r4, sink, "NHD", torch.bfloat16, workspace=ws, out=o))
        assert bool(torch.isfinite(o[0, -1].float()).all()) and float(o[0, -1].float().abs().sum()) > 0
        flops = workloads.window_flops(N, D, sink, [window_tokens(r8, N)] * Hq, [window_tokens(r4, N)] * Hq, 64)
        tf = flops / kern_ms / 1e9
        out[name] = {"window_tokens": [window_tokens(r8, N), window_tokens(r4, N)], "flops": flops,
                     "fraction_of_full_causal_flops": round(flops / (4.0 * N * N * D * Hq / 2), 4),
                     "plugin_call_ms": round(call_ms, 3), "kernel_ms": round(kern_ms, 3),
                     "roofline": {"bound": "mfma", "kernel": "prefill_kernel (sink + windows, fp16 P.V)", "achieved": round(tf, 1),
                                  "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_MFMA_BF16_TFLOPS, 4)}}
        # the same call with Q.K^T as a real integer product (args.int8_qk): blended peak = half the FLOPs on the int8 pipe
        # (5.0 POP/s), half on the 16-bit pipe (2.5 PFLOP/s)
        from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int8qk_prepass

        args8 = types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=True, int8_qk=True)
        closure8 = mp_triton_wrapper(1, r8, r4, sink, args8)
        call8_ms = timed(lambda: closure8(layer, q, k, v, None))
        kc, ks, v8b = fused_int8qk_prepass(q, k, v, "NHD")
        kern8_ms = timed(lambda: attn_hierarchical_relative_window(q, kc, q, kc, v8b, r8, r4, sink, "NHD", torch.bfloat16, workspace=ws, out=o,
                                                                   k_scale=ks))
        tf8 = flops / kern8_ms / 1e9
        out[name]["int8_qk"] = {"plugin_call_ms": round(call8_ms, 3), "kernel_ms": round(kern8_ms, 3),
                                "roofline": {"bound": "mfma", "kernel": "prefill_kernel (int8 Q.K^T, fp16 P.V, compiler-scheduled step)",
                                             "achieved": round(tf8, 1), "peak": round(PEAK_MFMA_BLEND_TFLOPS, 1), "unit": "TFLOP/s",
                                             "frac": round(tf8 / PEAK_MFMA_BLEND_TFLOPS, 4)},
                                "note": "build-defined option, off by default: same visited keys and P.V, scores from the int8 MFMA"}
        del q8, k8, v8, o, kc, ks, v8b
        torch.cuda.empty_cache()
    # the absolute-window launch (sqattn/attn_triton_mix_bad.py:285-426, args.use_relative_distance false): 128-row query
    # blocks, the 4-bit window range on its own 4-bit fake-quantised operands (two query blocks per workgroup, the tiles on
    # which they want different operand sets walked twice)
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_bad import attn_hierarchical_window

    w8, w4, sink = 8192, 32768, 256
    args_abs = types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=False)
    closure = mp_triton_wrapper(1, w8, w4, sink, args_abs)
    call_ms = timed(lambda: closure(layer, q, k, v, None))
    q8, q4, k8, k4, v8 = fused_int_prepass(q, k, v, want_4bit=True, tensor_layout="NHD")
    o = torch.empty_like(q8)
    kern_ms = timed(lambda: attn_hierarchical_window(q8, k8, q4, k4, v8, w8, w4, sink, "NHD", torch.bfloat16, workspace=ws, out=o))
    assert bool(torch.isfinite(o[0, -1].float()).all()) and float(o[0, -1].float().abs().sum()) > 0
    flops = workloads.window_flops(N, D, sink, [w8] * Hq, [w4] * Hq, 128)
    tf = flops / kern_ms / 1e9
    out["absolute_w8_8192_w4_32768_sink_256"] = {
        "window_tokens": [w8, w4], "flops": flops, "fraction_of_full_causal_flops": round(flops / (4.0 * N * N * D * Hq / 2), 4),
        "plugin_call_ms": round(call_ms, 3), "kernel_ms": round(kern_ms, 3),
        "roofline": {"bound": "mfma", "kernel": "prefill_kernel (sink + absolute windows, separate 4-bit operands: two 128-row query blocks per 8-wave workgroup, fp16 P.V)",
                     "achieved": round(tf, 1), "peak": PEAK_MFMA_BF16_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / PEAK_MFMA_BF16_TFLOPS, 4)}}
    del q8, q4, k8, k4, v8, o
    torch.cuda.empty_cache()
    return out


def time_decode(torch, B, L, iters=10, warmup=5, rounds=7, preheat=None):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import DecodePlan

    dev = torch.device("cuda:0")
    Hq, Hkv, D = 28, 4, 128
    g = torch.Generator(device=dev).manual_seed(3)
    nset = 2   # rotate buffer sets so that the 256 MB Infinity Cache cannot serve a re-read
    plans, total = [], 0
    for _ in range(nset):
        q = torch.randn(B, 1, Hq, D, device=dev, generator=g).bfloat16()
        kc = torch.randn(B, L, Hkv, D, device=dev, generator=g, dtype=torch.bfloat16)
        vc = torch.randn(B, L, Hkv, D, device=dev, generator=g, dtype=torch.bfloat16)
        lens = torch.randint((3 * L) // 4, L + 1, (B,), device=dev, generator=g, dtype=torch.int32) if B > 1 else \
            torch.full((B,), L, device=dev, dtype=torch.int32)
        plans.append(DecodePlan(q, kc, vc, "NHD", torch.bfloat16, seqlens=lens))
        total = int(lens.sum().item())
    stream = torch.cuda.current_stream(dev)
    for i in range(warmup):
        plans[i % nset].run()
    torch.cuda.synchronize()
    samples = []
    for _ in range(rounds):   # median over rounds of `iters` back-to-back calls (HIP events on the launch stream)
        if preheat is not None:   # queued on the same stream right in front of the timed calls
            preheat()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for i in range(iters):
            plans[i % nset].run()
        e1.record(stream)
        torch.cuda.synchronize()
        samples.append(e0.elapsed_time(e1) / iters * 1e3)
    us = sorted(samples)[len(samples) // 2]
    nbytes = 2048.0 * total   # K+V bf16, 4 kv heads x 128, read once for all 7 q-heads of a group
    return us, nbytes


def time_decode_selected(torch, B, L, k, iters=20, rounds=5, run=1):
    """Decode attention over k selected tokens per (sequence, kv head) of an L-token cache: the consumer of the
    k-means top-k selection.  With run == 1 the ids are random and distinct per head, so every row is a separate
    256-byte read; with run > 1 they are runs of `run` neighbouring rows at random places, which is what a selection
    of whole clusters reads from a cache kept in cluster order (sq_kv_cache_reorder)."""
    from longcontext_sqattn_paddle_amd import _native as Nn

    dev = torch.device("cuda:0")
    Hq, Hkv, D = 28, 4, 128
    g = torch.Generator(device=dev).manual_seed(6)
    q = torch.randn(B, 1, Hq, D, device=dev, generator=g).bfloat16()
    kc = torch.randn(B, L, Hkv, D, device=dev, generator=g, dtype=torch.bfloat16)
    vc = torch.randn(B, L, Hkv, D, device=dev, generator=g, dtype=torch.bfloat16)
    if run == 1:
        ids = torch.stack([torch.randperm(L, device=dev, generator=g)[:k] for _ in range(B * Hkv)]).to(torch.int32)
    else:
        starts = torch.stack([torch.randperm(L // run, device=dev, generator=g)[:k // run] for _ in range(B * Hkv)]) * run
        ids = (starts[:, :, None] + torch.arange(run, device=dev)).reshape(B * Hkv, k).to(torch.int32)
    lib = Nn.lib()
    S = lib.sq_decode_num_splits(B, Hkv, k)
    ws = torch.empty(lib.sq_decode_workspace_bytes(B, Hq, 128, S) // 4, dtype=torch.float32, device=dev)
    out = torch.empty_like(q)
    params = Nn.DecodeParams(Nn.LAYOUT["NHD"], Nn.P_NONE, S, 128)
    b = [Nn.dl(t) for t in (q, kc, vc, ids, None, out, None, ws)]
    ptrs = [Nn.ptr(x) for x in b]
    st = Nn.current_stream(dev)
    for _ in range(5):
        Nn.check(lib.sq_decode_selected_fwd(*ptrs, params, st))
    torch.cuda.synchronize()
    samples = []
    for _ in range(rounds):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            Nn.check(lib.sq_decode_selected_fwd(*ptrs, params, st))
        e1.record()
        torch.cuda.synchronize()
        samples.append(e0.elapsed_time(e1) / iters * 1e3)
    assert bool(torch.isfinite(out.float()).all()) and float(out.float().abs().sum()) > 0
    return sorted(samples)[len(samples) // 2], 2.0 * B * Hkv * k * D * 2


def time_layer_kernels(torch, N, iters=10):
    """The element-wise passes around the attention call at Qwen2.5-7B's sizes (hidden 3584, intermediate 18944,
    28/4 heads of 128): RMSNorm and RoPE over the N-token prompt, SiLU*mul over one 8192-token chunk of the MLP
    (the reference's chunk, model_hub/LLM.py:72-81)."""
    from longcontext_sqattn_paddle_amd.model_hub import utils as U

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(7)
    out = {}

    def timed(fn):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters * 1e3

    x = torch.randn(N, 3584, device=dev, generator=g).bfloat16()
    w = torch.ones(3584, device=dev, dtype=torch.bfloat16)
    y = torch.empty_like(x)
    us = timed(lambda: U.rmsnorm(x, w, 1e-6, out=y))
    out["rmsnorm"] = (us, 2.0 * x.numel() * 2)
    del x, y
    h = torch.randn(8192, 2 * 18944, device=dev, generator=g).bfloat16()
    o = torch.empty(8192, 18944, device=dev, dtype=torch.bfloat16)
    us = timed(lambda: U.silu_and_mul(h, out=o))
    out["silu_and_mul"] = (us, 1.5 * h.numel() * 2)
    del h, o
    q = torch.randn(N, 28 * 128, device=dev, generator=g).bfloat16()
    k = torch.randn(N, 4 * 128, device=dev, generator=g).bfloat16()
    table = U.yarn_cos_sin_cache(128, 1000000.0, 32768, N, dev)
    pos = torch.arange(N, device=dev)[None]
    us = timed(lambda: U.apply_rope_with_cos_sin_cache_inplace(pos, q, k, 128, table))
    out["rope"] = (us, 2.0 * (q.numel() + k.numel()) * 2 + table.numel() * 4 + N * 8)
    torch.cuda.empty_cache()
    return out


def time_decode_projections(torch, rows=1, iters=40, rounds=5):
    """The matmuls of one decode step at Qwen2.5-7B's sizes through `sq_linear_rows` (one activation row: batch 1),
    each with the BLAS library's time for the same product beside it.  Every call reads another copy of the weight
    (about 1.2 GB of copies per shape), so the weights stream from HBM as they do across the 28 layers of a step."""
    from longcontext_sqattn_paddle_amd.model_hub import utils as U

    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(9)
    shapes = [("wqkv", 4608, 3584, True, False), ("wo", 3584, 3584, False, True), ("gate_up_proj", 37888, 3584, False, False),
              ("down_proj", 3584, 18944, False, True), ("lm_head", 152064, 3584, False, False)]
    out = {}
    for name, n, k, has_bias, has_res in shapes:
        copies = max(2, min(12, int(1.2e9 // (n * k * 2))))
        ws = [(torch.randn(n, k, device=dev, generator=g) * k ** -0.5).bfloat16() for _ in range(copies)]
        x = torch.randn(rows, k, device=dev, generator=g).bfloat16()
        bias = torch.randn(n, device=dev, generator=g).bfloat16() if has_bias else None
        res = torch.randn(rows, n, device=dev, generator=g).bfloat16() if has_res else None

        def blas(w):
            y = torch.nn.functional.linear(x, w, bias)
            return y if res is None else res + y

        def timed(fn):
            """`iters` calls captured into one HIP graph and replayed: kernel time without the host's launch cost,
            as in the graph-replayed decode step."""
            for i in range(3):
                fn(ws[i % copies])
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for i in range(iters):
                    fn(ws[i % copies])
            graph.replay()
            torch.cuda.synchronize()
            samples = []
            for _ in range(rounds):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                graph.replay()
                e1.record()
                torch.cuda.synchronize()
                samples.append(e0.elapsed_time(e1) / iters * 1e3)
            del graph
            return sorted(samples)[len(samples) // 2]

        y = U.linear(x, ws[0], bias, res)
        ref = blas(ws[0])
        assert float((y.float() - ref.float()).abs().max()) <= 2.0 ** -5 * float(ref.float().abs().max())
        out[name] = (timed(lambda w: U.linear(x, w, bias, res)), timed(blas), float(n) * k * 2)
        del ws
        torch.cuda.empty_cache()
    return out


def time_model_layers(torch, N):
    """Two decoder layers of Qwen2.5-7B's shapes (random weights) through the runtime mirror: prompt of N tokens
    (embedding, 2 x layer_prefill, final norm, lm head), then decode steps against the N-token cache."""
    from longcontext_sqattn_paddle_amd.model_hub.qwen import QwenConfig, QwenModel

    dev = "cuda:0"
    cfg = QwenConfig(num_hidden_layers=2)
    model = QwenModel("Qwen2.5-7B-shaped", N + 16, torch.bfloat16, dev, "SDPA", config=cfg, seed=1)
    ids = torch.randint(0, cfg.vocab_size, (1, N), device=dev, generator=torch.Generator(device=dev).manual_seed(2))
    out = {}
    for name, pq in (("exact_attention", None), ("fp8_pv_attention", 5)):
        for layer in model.layers:
            layer.p_quant = pq
        ms = []
        for _ in range(3):
            model.batch_size, model.max_new_length = 1, 16
            model.init_kv_cache(N, [0])
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            logits = model.prefill_forward(ids)
            e1.record()
            torch.cuda.synchronize()
            ms.append(e0.elapsed_time(e1))
        assert bool(torch.isfinite(logits).all())
        out["prefill_ms_per_layer_" + name] = sorted(ms)[1] / cfg.num_hidden_layers
    tok = logits.argmax(dim=-1)
    for _ in range(3):
        model.decode_forward(tok)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(8):
        model.decode_forward(tok)
    e1.record()
    torch.cuda.synchronize()
    out["decode_ms_per_layer"] = e0.elapsed_time(e1) / 8 / cfg.num_hidden_layers
    del model
    torch.cuda.empty_cache()
    return out


def time_e2e(torch, N, new_tokens=17, sqattn=False, kv_selection=False, graph=False):
    """The whole 28-layer decoder of Qwen2.5-7B's shapes (random weights) through `generate`: prefill of one N-token
    prompt and greedy decoding, as the reference's latency logs measure them (model_hub/LLM.py:167-203).  With
    `sqattn`, layers 1..26 run the quantised sink/window closure of `process_model` with relative windows 0.25 / 0.5
    (the reference keeps exact attention in the first and last layer).  With `kv_selection` the prompt's keys are
    clustered after the prefill (1024 clusters per kv head, 10 Lloyd iterations) and every decode step attends to the
    4096 tokens of the best-scoring clusters plus the generated tokens (the benchmark's end-to-end configuration)."""
    import types

    from longcontext_sqattn_paddle_amd.model_hub.qwen import QwenConfig, QwenModel
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    dev = "cuda:0"
    cfg = QwenConfig()
    model = QwenModel("Qwen2.5-7B-shaped", N + new_tokens + 32, torch.bfloat16, dev, "SQAttn" if sqattn else "FlashAttn", config=cfg, seed=1)
    if sqattn:
        ws = {i: {"bit8": 0.25, "bit4": 0.5, "sink": 256} for i in range(1, cfg.num_hidden_layers - 1)}
        process_model(model, "SQAttn", ws, types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=True))
    ids = torch.randint(0, cfg.vocab_size, (1, N), device=dev, generator=torch.Generator(device=dev).manual_seed(2))
    if N > 262144:   # minutes per prefill: say where it is
        inner = model.layer_prefill

        def layer_prefill(layer_idx, start_bdx, hidden_states):
            out = inner(layer_idx, start_bdx, hidden_states)
            if hidden_states.shape[1] == N and layer_idx % 4 == 3:
                torch.cuda.synchronize()
                log(f"[bench] e2e ({'SQAttn' if sqattn else 'exact'}): layer {layer_idx + 1} of {cfg.num_hidden_layers} prefilled")
            return out

        model.layer_prefill = layer_prefill
    if kv_selection:
        model.enable_kv_selection(num_centroids=1024, topk=4096, num_iters=10)
    model.generate(model.attention_type, ids[:, :4096], None, 3, verbose=False)    # warm-up: library handles, GEMM heuristics
    eager = model.generate(model.attention_type, ids, None, new_tokens, verbose=False, use_graph=graph)
    res = {"prefill_s": round(model.prefill_latency, 3), "decode_ms_per_step": round(model.decode_latency * 1e3, 3),
           "tokens": N, "layers": cfg.num_hidden_layers, "attention": "SQAttn windows 0.25/0.5, sink 256" if sqattn else "exact causal"}
    if graph:
        res["decode_loop"] = "steps after the second replayed from a HIP graph"
    if kv_selection:
        res["decode"] = "k-means KV selection: 1024 clusters per kv head, 10 iterations, 4096 tokens per kv head and step"
        res["clustering_s"] = round(model.cluster_latency, 3)
    if (not sqattn or kv_selection) and N <= 262144 and not graph:   # (a second prefill of a longer prompt only for this check would take minutes)
        # the same generation with the decode step replayed from a HIP graph: must produce the same tokens
        graphed = model.generate(model.attention_type, ids, None, new_tokens + 32, verbose=False, use_graph=True)
        assert graphed[0][:new_tokens] == eager[0], "graph-replayed decode diverged from the eager decode"
        res["decode_ms_per_step_hip_graph"] = round(model.decode_latency * 1e3, 3)
    del model
    torch.cuda.empty_cache()
    return res


def time_config5(torch, new_tokens=128):
    """The benchmark's end-to-end configuration as written: the 28-layer Qwen2.5-7B-shaped decoder (random weights,
    bf16), one prompt of 1 048 576 seeded random tokens prefilled through `generate` (MLP in 8192-token chunks; exact
    attention in the first and last layer, the SQAttn closure of `process_model` with the reference's shipped windows --
    ratio 0.1 / 0.1, sink 256 -- in layers 1..26), the whole KV cache resident in HBM, k-means clustering of the prompt's
    keys (1024 clusters per kv head, 10 iterations), then `new_tokens` greedy tokens with the decode step replayed from a
    HIP graph over the 4096-token selection (model_hub/LLM.py:40-116, 167-203).  Beside it: where the prefill's time goes
    (HIP events around the attention slot and around the projections / MLP), and the dense decode step over the same
    cache."""
    import types

    from longcontext_sqattn_paddle_amd import workloads
    from longcontext_sqattn_paddle_amd.model_hub.qwen import QwenConfig, QwenModel
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import window_tokens

    dev, N = "cuda:0", 1 << 20
    free_gib = torch.cuda.mem_get_info()[0] / 2.0 ** 30
    if free_gib < 150.0:
        return {"skipped": f"needs 150 GiB of free HBM (60 GiB cache x 1.3 headroom, weights, a layer's activations); {free_gib:.0f} GiB free"}
    cfg = QwenConfig()
    model = QwenModel("Qwen2.5-7B-shaped", N + new_tokens + 32, torch.bfloat16, dev, "SQAttn", config=cfg, seed=1)
    ratio, sink = 0.1, 256
    process_model(model, "SQAttn", {i: {"bit8": ratio, "bit4": ratio, "sink": sink} for i in range(1, cfg.num_hidden_layers - 1)},
                  types.SimpleNamespace(qk_qtype="int", v_qtype="int", use_relative_distance=True))
    model.enable_kv_selection(num_centroids=1024, topk=4096, num_iters=10)
    spans = {"attention": [], "projections_and_mlp": []}

    def timed(kind, fn, is_prefill):
        def wrapper(*a, **kw):
            if not is_prefill(*a, **kw):
                return fn(*a, **kw)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            out = fn(*a, **kw)
            e1.record()
            spans[kind].append((e0, e1))
            return out
        return wrapper

    for layer in model.layers:   # the slots process_model bound (layers 1..26) and the exact ones (0, 27)
        layer.prefill_attention = timed("attention", layer.prefill_attention, lambda *a, **kw: True)
    model.wqkv = timed("projections_and_mlp", model.wqkv, lambda h, layer: h.shape[1] > 1)
    model.wo = timed("projections_and_mlp", model.wo, lambda h, layer, bsz, seq_len, dim, residual=None: seq_len > 1)
    model.mlp = timed("projections_and_mlp", model.mlp, lambda h, layer, residual=None, norm=None: h.shape[1] > 1)
    inner = model.layer_prefill

    def layer_prefill(layer_idx, start_bdx, hidden_states):
        out = inner(layer_idx, start_bdx, hidden_states)
        if hidden_states.shape[1] == N and layer_idx % 4 == 3:
            torch.cuda.synchronize()
            log(f"[bench] config 5: layer {layer_idx + 1} of {cfg.num_hidden_layers} prefilled")
        return out

    model.layer_prefill = layer_prefill
    ids = torch.randint(0, cfg.vocab_size, (1, N), device=dev, generator=torch.Generator(device=dev).manual_seed(5))
    model.generate("SQAttn", ids[:, :4096], None, 3, verbose=False)    # warm-up: library handles, GEMM heuristics
    for v in spans.values():
        v.clear()
    out = model.generate("SQAttn", ids, None, new_tokens, verbose=False, use_graph=True)
    torch.cuda.synchronize()
    assert len(out[0]) == new_tokens and model.kv_cache.valid_length.cpu().tolist() == [N + new_tokens - 1]
    share = {k: sum(e0.elapsed_time(e1) for e0, e1 in v) / 1e3 for k, v in spans.items()}
    w = window_tokens(ratio, N)
    attn_flops = 2 * (4.0 * N * N * 128 * 28 / 2) + (cfg.num_hidden_layers - 2) * workloads.window_flops(N, 128, sink, [w] * 28, [w] * 28, 64)
    res = {"config": f"{cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, 28/4 heads of 128, bf16 random weights; prompt {N} tokens, "
                     f"{new_tokens} greedy tokens; SQAttn closure (ratio {ratio}/{ratio}, sink {sink}) in layers 1..{cfg.num_hidden_layers - 2}, exact "
                     "attention in the first and last; 1024 clusters per kv head, 10 Lloyd iterations, 4096 selected tokens per kv head and step",
           "prefill_s": round(model.prefill_latency, 2), "clustering_s": round(model.cluster_latency, 3),
           "decode_ms_per_step_selection_hip_graph": round(model.decode_latency * 1e3, 3),
           "prefill_seconds_by_part": {"attention_calls": round(share["attention"], 2), "projections_and_mlp": round(share["projections_and_mlp"], 2),
                                       "other": round(model.prefill_latency - share["attention"] - share["projections_and_mlp"], 2),
                                       "note": "HIP events around the attention slot of every layer (pre-pass + kernel) and around wqkv, wo and "
                                               "the chunked MLP (hipBLASLt GEMMs + SiLU*mul); other = norms, rotary embedding, cache rows, embedding, host"},
           "prefill_attention_TFLOP_per_s": round(attn_flops / share["attention"] / 1e12, 1),
           "kv_cache_GB": round(2 * cfg.num_hidden_layers * N * 4 * 128 * 2 / 1e9, 1)}
    # the dense decode step over the same cache, replayed from a graph as well.  The cache holds exactly prompt + new
    # tokens, so it is rewound to the prompt first: the steps rewrite rows that are already there.
    model.disable_kv_selection()
    cache = model.kv_cache
    cache.valid_length.fill_(N)
    cache._host_valid, cache.context = [N], N
    tok = torch.tensor([[out[0][0]]], device=dev)
    tok = model.decode_forward(tok).argmax(dim=-1)
    tok = model.capture_decode_step(tok).argmax(dim=-1)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(8):
        tok = model.replay_decode_step(tok).argmax(dim=-1)
    e1.record()
    torch.cuda.synchronize()
    model.release_decode_graph()
    res["decode_ms_per_step_dense_hip_graph"] = round(e0.elapsed_time(e1) / 8, 3)
    del model
    torch.cuda.empty_cache()
    return res


def time_kv_cache(torch, N, iters=10):
    """The KV cache's two row movements at the benchmark shape (4 kv heads x 128, bf16): the store of an N-token
    prompt (K and V, each read once and written once) and the append of one token per sequence at batch 8."""
    from longcontext_sqattn_paddle_amd import _native as Nn

    dev = torch.device("cuda:0")
    Hkv, D = 4, 128
    g = torch.Generator(device=dev).manual_seed(5)
    lib = Nn.lib()
    st = Nn.current_stream(dev)
    nset = 2   # alternate source/destination sets: the 256 MB Infinity Cache must not serve the re-read
    sets = []
    for _ in range(nset):
        ks = torch.randn(1, N, Hkv, D, device=dev, generator=g).bfloat16()
        vs = torch.randn(1, N, Hkv, D, device=dev, generator=g).bfloat16()
        kc = torch.empty(1, N, Hkv, D, device=dev, dtype=torch.bfloat16)
        vc = torch.empty(1, N, Hkv, D, device=dev, dtype=torch.bfloat16)
        sets.append([Nn.dl(t) for t in (ks, vs, kc, vc)])
    def store(i):
        Nn.check(lib.sq_kv_cache_store(*[Nn.ptr(x) for x in sets[i % nset]], 0, 0, st))
    for i in range(2):
        store(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        store(i)
    e1.record()
    torch.cuda.synchronize()
    store_us = e0.elapsed_time(e1) / iters * 1e3
    assert torch.equal(sets[0][2].tensor[0, -1], sets[0][0].tensor[0, -1])
    store_bytes = 2.0 * 2 * N * Hkv * D * 2   # K and V, read + written
    B, L = 8, 131072
    kc = torch.empty(B, L, Hkv, D, device=dev, dtype=torch.bfloat16)
    vc = torch.empty(B, L, Hkv, D, device=dev, dtype=torch.bfloat16)
    kn = torch.randn(B, 1, Hkv, D, device=dev, generator=g).bfloat16()
    vn = torch.randn(B, 1, Hkv, D, device=dev, generator=g).bfloat16()
    lens = torch.full((B,), 1000, device=dev, dtype=torch.int32)
    att = torch.zeros(B, device=dev, dtype=torch.int32)
    b = [Nn.dl(t) for t in (kn, vn, kc, vc, lens, att)]
    ptrs = [Nn.ptr(x) for x in b]
    for _ in range(5):
        Nn.check(lib.sq_kv_cache_append(*ptrs, 1, st))
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(100):
        Nn.check(lib.sq_kv_cache_append(*ptrs, 1, st))
    e1.record()
    torch.cuda.synchronize()
    append_us = e0.elapsed_time(e1) / 100 * 1e3
    assert int(lens[0].item()) == 1105 and torch.equal(kc[:, 1104], kn[:, 0])
    return store_us, store_bytes, append_us


def time_calibration(torch, N, iters=3):
    """The window search's histogram kernel at the benchmark's head shape (28 q heads / 4 kv heads / 128) on an
    N-token sample, both binning rules the calibration drivers use.  Work: Q.K^T over the causal half twice (once for
    the row normalisers, once for the probabilities) = 4 N^2 D Hq / 2 FLOP, i.e. what the prefill kernel does."""
    from longcontext_sqattn_paddle_amd.sqattn.window_search import ABSOLUTE, RELATIVE_SINK, attention_histograms

    dev = torch.device("cuda:0")
    Hq, Hkv, D = 28, 4, 128
    g = torch.Generator(device=dev).manual_seed(6)
    q = (torch.randn(1, N, Hq, D, device=dev, generator=g) * 1.5).bfloat16()
    k = torch.randn(1, N, Hkv, D, device=dev, generator=g).bfloat16()
    out = {}
    for name, kind, bins, sink in (("absolute", ABSOLUTE, N, 0), ("relative_sink", RELATIVE_SINK, 200, 256)):
        hist = torch.zeros(1, Hq, bins, dtype=torch.float64, device=dev)
        attention_histograms(q, k, kind, bins, sink, out=hist)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            attention_histograms(q, k, kind, bins, sink, out=hist)
        e1.record()
        torch.cuda.synchronize()
        out[name] = e0.elapsed_time(e1) / iters
    return out, 4.0 * N * N * D * Hq / 2


def time_kmeans(torch, iters=10):
    """BASELINE config 4 at its shape (4 kv heads x 131072 tokens x 128, 1024 centroids): one Lloyd iteration (assign +
    counting sort + exact cluster sums + centroid update), the whole `segment_k_means` of 10 iterations with its value sums
    and reverse index, and the top-k selection behind it.  Two key sets alternate, so that a 134 MB key tensor does not
    simply stay in the 256 MB Infinity Cache between iterations."""
    from longcontext_sqattn_paddle_amd import workloads
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _triton_k_means_train, _workspace, segment_k_means, topk_select

    dev = torch.device("cuda:0")
    G, N, C, D = 4, 131072, 1024, 128
    idx0 = (torch.arange(C, dtype=torch.float32) * (N / C) + N / C / 2).to(torch.int64).to(dev)
    sets = []
    for seed in (4, 5):
        key, value = workloads.kmeans_inputs(G, N, D, seed=seed)
        key, value = key.to(dev), value.to(dev)
        sets.append((key, value, key.index_select(1, idx0).contiguous()))
    ws = _workspace(G, N, C, dev)
    idx = torch.empty(G, N, dtype=torch.int32, device=dev)
    for i in range(4):
        _triton_k_means_train(sets[i % 2][0], sets[i % 2][2], max_idx=idx, workspace=ws)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        _triton_k_means_train(sets[i % 2][0], sets[i % 2][2], max_idx=idx, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / iters * 1e3
    flops = 2.0 * N * C * D * G
    nbytes = G * (N * D * 2 + N * 4 + C * D * 2 * 2 + C * 4)   # keys read once, assignment written, centroids read and written, counts
    # the iteration loop as segment_k_means runs it: three steps that re-sum every row, the third leaving the exact sums
    # in the workspace, then steps that only apply the tokens that changed cluster (sq_kmeans_train_stateful).  Each key
    # set has its own assignment and workspace (the carried state), and the two alternate as above.
    from longcontext_sqattn_paddle_amd import _native as NV

    state = [(torch.empty(G, N, dtype=torch.int32, device=dev), _workspace(G, N, C, dev)) for _ in sets]
    run10, carried = [], []
    for rep in range(3):
        cents = [s_[0].index_select(1, idx0).contiguous() for s_ in sets]
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        ev[0].record()
        for it in range(10):
            if it == 3:
                ev[1].record()
            st = NV.KMEANS_STATELESS if it < 2 else (NV.KMEANS_KEEP_SUMS if it == 2 else NV.KMEANS_APPLY_CHANGES)
            for k in range(2):
                _triton_k_means_train(sets[k][0], cents[k], max_idx=state[k][0], workspace=state[k][1], state=st)
        ev[2].record()
        torch.cuda.synchronize()
        run10.append(ev[0].elapsed_time(ev[2]) / 20 * 1e3)
        carried.append(ev[1].elapsed_time(ev[2]) / 14 * 1e3)
    us_run10, us_carried = sorted(run10)[1], sorted(carried)[1]
    del state
    # the configuration as written: 10 Lloyd iterations (9 normalised + the final one), value sums, reverse index, then top-k
    full = []
    for i in range(4):
        key, value, _ = sets[i % 2]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cent, _, clusters, size = segment_k_means(key, value, C, num_iters=10)
        torch.cuda.synchronize()
        full.append((time.perf_counter() - t0) * 1e3)
    assert int(size.sum()) == G * N
    q = torch.randn(1, 28, D, device=dev, generator=torch.Generator(device=dev).manual_seed(9)).bfloat16()
    out = torch.empty(G, 4096, dtype=torch.int32, device=dev)
    for _ in range(3):
        topk_select(q, cent, clusters, size, 4096, 7, out=out, workspace=ws)
    torch.cuda.synchronize()
    e0.record()
    for _ in range(20):
        topk_select(q, cent, clusters, size, 4096, 7, out=out, workspace=ws)
    e1.record()
    torch.cuda.synchronize()
    assert int(out.min()) >= 0 and int(out.max()) < N
    return us, flops, nbytes, e0.elapsed_time(e1) / 20 * 1e3, sorted(full[1:])[1], us_run10, us_carried


def time_prepass(torch, N, want4, iters=10, skip_query=False):
    """The plugin closure's operand pre-pass (key centring + int8/int4 per-token + int8 per-channel fake quantisation)
    at the prefill benchmark shape, tensors in the plugin's NHD layout.  `skip_query`: what the closure runs with relative
    windows, where the attention kernel quantises the query rows as it loads them."""
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    dev = torch.device("cuda:0")
    Hq, Hkv, D = 28, 4, 128
    g = torch.Generator(device=dev).manual_seed(2)
    q = torch.randn(1, N, Hq, D, device=dev, generator=g).bfloat16()
    k = torch.randn(1, N, Hkv, D, device=dev, generator=g).bfloat16()
    v = torch.randn(1, N, Hkv, D, device=dev, generator=g).bfloat16()
    for _ in range(2):
        outs = fused_int_prepass(q, k, v, want_4bit=want4, skip_query=skip_query)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        outs = fused_int_prepass(q, k, v, want_4bit=want4, skip_query=skip_query)
    e1.record()
    torch.cuda.synchronize()
    assert bool(torch.isfinite(outs[2][0, -1].float()).all())
    us = e0.elapsed_time(e1) / iters * 1e3
    qb, kb = (0 if skip_query else N * Hq * D * 2), N * Hkv * D * 2
    nbytes = (qb + 2 * kb + kb) + (qb + kb + kb) + ((qb + kb) if want4 else 0)   # reads (K twice) + writes
    return us, float(nbytes)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--seq-len", type=int, default=131072)
    ap.add_argument("--settle", type=float, default=2.0,
                    help="seconds of idle time before each leg after the headline one (they follow seconds of work at the power limit)")
    ap.add_argument("--p-quant", type=int, default=5,
                    help="0 none, 1 e4m3 static 448 exactly as the reference rounds it, 2 e4m3 block absmax, "
                         "3 e4m3 static 448 with the scale folded into the exponent, "
                         "4 = 3 plus e4m3 V so that P.V runs on the fp8 matrix pipe, "
                         "5 (default) = 4 with one power-of-two block scale per query row and 64-key tile on P")
    ap.add_argument("--no-variants", action="store_true", help="skip the other P modes (0 - 4) of the prefill kernel")
    ap.add_argument("--no-mfma-probe", action="store_true", help="skip the MFMA-only loop (sustained matrix-core rate on constant / workload operands)")
    ap.add_argument("--no-plugin", action="store_true", help="skip the plugin closure (pre-pass + sink/window kernel)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="run one 1 GiB device-to-device copy first: a kernel of known traffic for scaling FETCH_SIZE/WRITE_SIZE")
    ap.add_argument("--no-kmeans", action="store_true")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true")
    ap.add_argument("--no-prepass", action="store_true")
    ap.add_argument("--no-kv-cache", action="store_true")
    ap.add_argument("--no-layer", action="store_true")
    ap.add_argument("--no-model", action="store_true")
    ap.add_argument("--no-calibration", action="store_true")
    ap.add_argument("--e2e-runs", default="exact,sqattn,selection",
                    help="which end-to-end runs --e2e makes: exact attention, the SQAttn closure, the SQAttn closure with "
                         "k-means KV selection in the decode steps")
    ap.add_argument("--e2e-new-tokens", type=int, default=17, help="tokens generated by each end-to-end run")
    ap.add_argument("--e2e-graph", action="store_true",
                    help="the end-to-end runs replay their decode steps from a HIP graph (for prompts too long to prefill twice)")
    ap.add_argument("--no-config5", action="store_true",
                    help="skip the end-to-end configuration as written (28 layers, 1 048 576-token prompt, 128 graph-replayed steps: about two minutes)")
    ap.add_argument("--e2e", action="store_true",
                    help="also run the whole 28-layer Qwen2.5-7B-shaped decoder (random weights): prefill latency and decode ms/step")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(3)
    N = args.seq_len
    if args.calibration_copy:
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device="cuda:0")   # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()
    qkv = prefill_inputs(torch, N)
    ms, flops = time_prefill(torch, qkv, args.steps, args.warmup, args.p_quant)
    tflops = flops / ms / 1e9
    log(f"[bench] prefill N={N}: {ms:.2f} ms/step, {tflops:.1f} TFLOP/s")
    if args.p_quant >= 4:
        peak, peak_note = PEAK_MFMA_BLEND_TFLOPS, "harmonic blend: Q.K^T on bf16 MFMA (2.5 PFLOP/s), P.V on fp8 MFMA (5.0 PFLOP/s)"
    else:
        peak, peak_note = PEAK_MFMA_BF16_TFLOPS, "both GEMMs on 16-bit MFMA"

    result = {
        "metric": METRIC,
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"prefill attention, batch 1, 28 q heads / 4 kv heads, head_dim 128, seq {N}, causal, "
                        f"bf16 N(0,1)/sqrt(128) with 2% K outlier channels x8, P quant mode {args.p_quant} "
                        f"({P_MODE_NOTE.get(args.p_quant, 'e4m3 P, fp16 MFMA P.V')}), fp32 accumulate",
            "flops_per_step": flops,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": "prefill_kernel",
            "achieved": round(tflops, 2),
            "peak": round(peak, 1),
            "peak_note": peak_note,
            "unit": "TFLOP/s",
            "frac": round(tflops / peak, 4),
            "frac_of_bf16_peak": round(tflops / PEAK_MFMA_BF16_TFLOPS, 4),
            "traffic": prefill_traffic_bytes(N, args.p_quant),
            "traffic_note": "bytes per launch through the L2/fabric interface, read from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE "
                            "summary of this shape (profiles/prefill_kernel_128k.traffic.json), not re-measured by this run; null for other shapes",
            "numerics": "P mode 5 is build-defined (the reference multiplies fp16 P by fp16 V): see `variants` for the reference's own modes",
        },
    }
    if not args.no_mfma_probe:
        probe = time_mfma_only(torch, qkv)
        ceiling = probe["blend_workload_values"] if args.p_quant >= 4 else probe["bf16_workload_values"]
        result["roofline"]["mfma_only_loop"] = probe
        result["roofline"]["frac_of_mfma_only_loop"] = round(tflops / ceiling, 4)
        log(f"[bench] MFMA-only loop: {probe}")
    if not args.no_variants:
        # the reference's own numerics (modes 0 and 1) and the other P modes, a few steps each: the kernel is the same,
        # only the quantisation of P (and of V in mode 4) differs.  Each entry is priced against the peak of the matrix
        # pipes it uses.
        result["variants"] = {}
        for mode, name, note in ((0, "no_P_quant_fp16_PV", "attn_triton.py:83, is_P_fp8_quant=False (the reference's default)"),
                                 (1, "e4m3_P_reference_rounding_fp16_PV", "attn_triton.py:81-82 op for op: fp16(fp16(e4m3(448 p)) / 448)"),
                                 (3, "e4m3_P_folded_scale_fp16_PV", "the same e4m3 grid, 448 folded into the exponent (build-defined)"),
                                 (2, "e4m3_P_block_absmax_fp16_PV", "per 64x64 block absmax scale on P (build-defined, BASELINE config 1)"),
                                 (4, "e4m3_P_static_scale_fp8_PV", "e4m3 V and fp8 MFMA P.V with the static scale 448 (build-defined)")):
            vms, _ = time_prefill(torch, qkv, 3, 1, mode)
            vpeak = PEAK_MFMA_BLEND_TFLOPS if mode >= 4 else PEAK_MFMA_BF16_TFLOPS
            vt = flops / vms / 1e9
            result["variants"][name] = {"p_quant": mode, "ms_per_step": round(vms, 3), "TFLOP_per_s": round(vt, 1),
                                        "peak": round(vpeak, 1), "frac": round(vt / vpeak, 4), "numerics": note}
            log(f"[bench] prefill variant {name}: {vms:.2f} ms = {vt:.0f} TFLOP/s = {vt / vpeak:.3f} of {vpeak:.0f}")
    if not args.no_plugin:
        result["plugin"] = time_plugin(torch, qkv)
        log(f"[bench] plugin closure: {result['plugin']}")
    def settle():
        # The prefill legs above run the matrix cores at the chip's power limit for several seconds; a leg measured
        # right behind them inherits that state (the 1M-token decode reads 322 us then and 307 - 312 us from an idle
        # chip).  Every leg below therefore starts after a short pause, like the headline leg, which starts the process.
        torch.cuda.synchronize()
        time.sleep(args.settle)

    result["settle_s"] = args.settle
    if not args.no_decode:
        # Every decode leg is timed under two conditions: from a chip that has idled for `settle` seconds, and "hot",
        # right behind half a second of prefill attention at the power limit (what a serving loop that interleaves
        # prefill and decode sees).
        ws_heat = None

        def heat():
            nonlocal ws_heat
            from longcontext_sqattn_paddle_amd.sqattn._prefill import prefill_workspace
            from longcontext_sqattn_paddle_amd.sqattn.attn_triton import attn_causal

            if ws_heat is None:
                ws_heat = (prefill_workspace(1, 4, N, qkv[0].device), torch.empty_like(qkv[0]))
            for _ in range(6):
                attn_causal(qkv[0], qkv[1], qkv[2], "HND", torch.bfloat16, p_quant=args.p_quant, workspace=ws_heat[0], out=ws_heat[1])

        dec = {}
        for name, B, L in (("1M_b1", 1, 1048576), ("128K_b1", 1, 131072), ("128K_b4", 4, 131072), ("128K_b8", 8, 131072)):
            settle()
            us, nbytes = time_decode(torch, B, L)
            us_hot, _ = time_decode(torch, B, L, preheat=heat)
            gbs = nbytes / us / 1e3
            dec[name] = {"us_per_call": round(us, 2), "GB_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / PEAK_HBM_GBS, 4),
                         "us_per_call_hot": round(us_hot, 2), "frac_of_hbm_peak_hot": round(nbytes / us_hot / 1e3 / PEAK_HBM_GBS, 4),
                         "bytes": nbytes}
            log(f"[bench] decode {name}: {us:.1f} us, {gbs:.0f} GB/s; right behind prefill work {us_hot:.1f} us")
            torch.cuda.empty_cache()
        dec["note"] = ("us_per_call: after settle_s seconds of idle time; us_per_call_hot: timed immediately behind six prefill attention "
                       "calls (0.45 s at the power limit)")
        result["decode"] = dec
        ws_heat = None
        sel = {}
        for name, B, L, k, run in (("4096_of_128K_b1", 1, 131072, 4096, 1), ("4096_of_128K_b8", 8, 131072, 4096, 1),
                                   ("65536_of_1M_b1", 1, 1048576, 65536, 1), ("65536_of_1M_b1_runs_of_64", 1, 1048576, 65536, 64),
                                   ("4096_of_128K_b8_runs_of_64", 8, 131072, 4096, 64)):
            us, nbytes = time_decode_selected(torch, B, L, k, run=run)
            sel[name] = {"us_per_call": round(us, 2), "GB_per_s": round(nbytes / us / 1e3, 1), "bytes": nbytes}
            log(f"[bench] decode over selected tokens {name}: {us:.1f} us, {nbytes / us / 1e3:.0f} GB/s")
            torch.cuda.empty_cache()
        result["decode_selected"] = sel
    del qkv
    torch.cuda.empty_cache()
    if not args.no_prepass:
        settle()
        pre = {}
        for name, want4, skip_q in (("int8", False, False), ("int8_int4", True, False), ("int8_key_and_value_only", False, True)):
            us, nbytes = time_prepass(torch, N, want4, skip_query=skip_q)
            pre[name] = {"us_per_call": round(us, 1), "GB_per_s": round(nbytes / us / 1e3, 1),
                         "frac_of_hbm_peak": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4), "bytes": nbytes}
            log(f"[bench] plugin pre-pass {name}: {us:.0f} us, {nbytes / us / 1e3:.0f} GB/s")
            torch.cuda.empty_cache()
        result["plugin_prepass"] = pre
    if not args.no_kv_cache:
        settle()
        sus, sbytes, aus = time_kv_cache(torch, N)
        result["kv_cache"] = {"store_us": round(sus, 1), "store_GB_per_s": round(sbytes / sus / 1e3, 1),
                              "store_frac_of_hbm_peak": round(sbytes / sus / 1e3 / PEAK_HBM_GBS, 4), "store_bytes": sbytes,
                              "append_us_batch8": round(aus, 2)}
        log(f"[bench] kv cache: store of {N} tokens {sus:.0f} us ({sbytes / sus / 1e3:.0f} GB/s), append (batch 8) {aus:.1f} us")
        torch.cuda.empty_cache()
    if not args.no_layer:
        settle()
        lay = {}
        for name, (us, nbytes) in time_layer_kernels(torch, N).items():
            lay[name] = {"us_per_call": round(us, 1), "GB_per_s": round(nbytes / us / 1e3, 1),
                         "frac_of_hbm_peak": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4), "bytes": nbytes}
            log(f"[bench] layer kernel {name}: {us:.0f} us, {nbytes / us / 1e3:.0f} GB/s")
        result["layer_kernels"] = lay
        proj = {}
        for name, (us, blas_us, nbytes) in time_decode_projections(torch).items():
            proj[name] = {"us_per_call": round(us, 1), "GB_per_s": round(nbytes / us / 1e3, 1),
                          "frac_of_hbm_peak": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4), "bytes": nbytes, "blas_us_per_call": round(blas_us, 1)}
            log(f"[bench] decode projection {name}: {us:.1f} us, {nbytes / us / 1e3:.0f} GB/s (BLAS library: {blas_us:.1f} us)")
        proj["note"] = ("one activation row (batch 1), bf16, bias / residual as in the decode step; 40 calls replayed from one HIP "
                        "graph, each on another copy of the weight")
        result["decode_projections"] = proj
    if not args.no_model:
        ml = time_model_layers(torch, N)
        result["model_layers"] = {k: round(v, 3) for k, v in ml.items()}
        result["model_layers"]["note"] = ("Qwen2.5-7B-shaped decoder layers with random weights, batch 1: per-layer time of a "
                                          f"{N}-token prefill (includes 1/2 of embedding + lm head) and of a decode step at that context")
        log(f"[bench] model layers: {ml}")
    if not args.no_calibration:
        n_cal = 32768
        cal, cflops = time_calibration(torch, n_cal)
        result["calibration"] = {name: {"ms_per_call": round(ms, 3), "TFLOP_per_s": round(cflops / ms / 1e9, 1)} for name, ms in cal.items()}
        result["calibration"]["shape"] = (f"one {n_cal}-token sample, 28 q heads / 4 kv heads / 128: energy histograms of all heads from "
                                          f"Q and K; the dense attention map the reference reduces would hold {28 * n_cal * n_cal * 2 / 1e9:.0f} GB")
        log(f"[bench] calibration histograms: {cal}")
        torch.cuda.empty_cache()
    if args.e2e:
        runs = {"exact": dict(sqattn=False), "sqattn": dict(sqattn=True), "selection": dict(sqattn=True, kv_selection=True)}
        result["e2e_runs"] = [time_e2e(torch, N, new_tokens=args.e2e_new_tokens, graph=args.e2e_graph, **runs[r]) for r in args.e2e_runs.split(",")]
        log(f"[bench] end to end: {result['e2e_runs']}")
    if not args.no_kmeans:
        settle()
        us, kflops, kbytes, topk_us, full_ms, us_run10, us_carried = time_kmeans(torch)
        t_mfma, t_hbm = kflops / PEAK_MFMA_BF16_TFLOPS / 1e6, kbytes / PEAK_HBM_GBS / 1e3
        result["kmeans"] = {"us_per_iteration": round(us, 1), "TFLOP_per_s": round(kflops / us / 1e6, 1),
                            "frac_of_bf16_mfma_peak": round(kflops / us / 1e6 / PEAK_MFMA_BF16_TFLOPS, 4),
                            "GB_per_s": round(kbytes / us / 1e3, 1), "frac_of_hbm_peak": round(kbytes / us / 1e3 / PEAK_HBM_GBS, 4),
                            "bound_us": round(max(t_mfma, t_hbm), 1), "frac_of_bound": round(max(t_mfma, t_hbm) / us, 4),
                            "bytes": kbytes, "flops": kflops,
                            "shape": "4 heads x 131072 tokens x 128, 1024 centroids, one Lloyd iteration that re-sums every row, two key sets alternating",
                            "us_per_iteration_carried_sums": round(us_carried, 1),
                            "frac_of_bound_carried_sums": round(max(t_mfma, t_hbm) / us_carried, 4),
                            "us_per_iteration_mean_of_the_10_iteration_run": round(us_run10, 1),
                            "carried_sums_note": "the loop of segment_k_means: iterations 1-3 re-sum every row, 4-10 apply only the tokens that changed "
                                                 "cluster to the exact sums kept in the workspace (same centroids bit for bit); iterations 4-10 alone, "
                                                 "and the mean over all ten",
                            "segment_k_means_10_iterations_ms": round(full_ms, 3),
                            "segment_k_means_note": "10 iterations + value sums + reverse index, host wall clock including its one host "
                                                    "synchronisation (the reference's Cnt.max().item(), cache_hub/kmeans.py:195)",
                            "topk_select_us": round(topk_us, 1),
                            "topk_shape": "4096 tokens per kv head for one 28-head query, 1024 clusters per kv head"}
        log(f"[bench] kmeans iteration: {us:.0f} us")
    if not args.no_config5:
        settle()
        try:
            result["e2e"] = time_config5(torch)
        except Exception as exc:   # the headline line must come out whatever happens to this leg
            result["e2e"] = {"error": f"{type(exc).__name__}: {exc}"[:500]}
            torch.cuda.empty_cache()
        log(f"[bench] config 5 end to end: {result['e2e']}")
    if not args.no_cpu_baseline:
        from oracle import cpu_baseline as CB   # the checker's CPU path, timed as the baseline only

        cpu_tflops, threads, dt, n = CB.time_cpu_baseline(budget_s=6.0)
        one_tflops, _, one_dt, one_n = CB.time_cpu_baseline(budget_s=4.0, threads=1)
        pts, extrap_s = CB.time_prefill_points()
        dec_gbs, dec_dt = CB.time_decode_cpu()
        km_dt, km_tflops = CB.time_kmeans_iteration_cpu()
        result["cpu_baseline"] = {
            "value": round(cpu_tflops, 4),
            "unit": "TFLOP/s",
            "cores": threads,
            "kind": "port",
            "cpu": f"{CB.cpu_model()}, {os.cpu_count()} logical CPUs visible, torch intra-op threads {threads}",
            "sample": f"config-1 shape (batch 1, 4 q heads on 1 kv head, head_dim 128, seq 4096, causal): GQA expand, K centring, "
                      f"int8/int4 fake-quant, torch CPU SDPA in bf16; {n} passes of {dt * 1e3:.1f} ms on {threads} threads "
                      f"({os.cpu_count()} logical CPUs)",
            "one_thread": {"value": round(one_tflops, 4), "unit": "TFLOP/s", "cores": 1, "sample": f"the same shape, {one_n} passes of {one_dt * 1e3:.1f} ms"},
            "config2_prefill_points": {"points": pts, "cores": threads,
                                       "extrapolated_seconds_at_131072_tokens_28_heads": round(extrap_s, 1),
                                       "note": "4 of the 28 query heads (one kv head) timed once per length, attention in 2048-row query chunks; "
                                               "the 131072-token figure is EXTRAPOLATED from the largest point by (N ratio)^2 x 7, not measured"},
            "config3_decode_128K_b1": {"value": round(dec_gbs, 2), "unit": "GB/s", "cores": threads, "seconds_per_call": round(dec_dt, 5),
                                       "sample": "one query token, 28/4 heads, full 131072-token bf16 cache, 5 calls"},
            "config4_kmeans_iteration": {"value": round(km_tflops, 4), "unit": "TFLOP/s", "cores": threads,
                                         "seconds_per_iteration_4_heads": round(4 * km_dt, 3),
                                         "sample": "one Lloyd iteration of one head (131072 x 128 keys, 1024 centroids, fp32), timed once, x 4 heads"},
        }
        log(f"[bench] cpu baseline: {cpu_tflops:.3f} TFLOP/s on {threads} threads, {one_tflops:.3f} on one; C2 points {pts}; "
            f"decode {dec_gbs:.1f} GB/s; k-means iteration {4 * km_dt:.2f} s")
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
