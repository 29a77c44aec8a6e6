#!/usr/bin/env python3
"""Headline benchmark: training tokens/s (forward + backward + AdamW) of the packed-batch
training step on ONE MI355X, with the dominant kernel's roofline fraction measured live and
the CPU oracle timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c4|c1] [--headline-only] [--pmc-calibration]

Workloads (BASELINE.json configs): c5 = Qwen3-1.7B-shape full-weight FP32 training,
4 x 4096 tokens (default); c4 = the same model, LoRA r16 on q/k/v/o, 1 x 2048; c1 = the
33M Seraph-native model, 8 x 256.  Synthetic data: uniform token ids, N(0, 0.02) weights,
norm gains 1, fixed seeds.  Prints ONE JSON line.  The headline keys (value, ms_per_step, roofline,
cpu_baseline ...) are the named workload's.  The default run (c5) then also measures the rest of the
metric and adds it under extra keys: `workloads` (c1 and c4 as whole steps, each with its own roofline),
`ops` (the single-op configurations alone: attention backward at B8 H16 S1024 D64, and cross entropy,
RMSNorm backward, SwiGLU backward, AdamW, RoPE, qk_norm and embedding backward at 16384 tokens), and
`drop_in_path` (the reference's unmodified step driver over this backend's vulkan_* symbols).

--pmc-calibration launches the library's in-place scale kernel three times over 1 GiB before
the steps (reads 1 GiB, writes 1 GiB per launch): under `rocprofv3 --pmc FETCH_SIZE` /
`--pmc WRITE_SIZE` its counter readings give the factor that turns the counter into bytes.
roofline.traffic is read from profiles/train_step_<workload>_hbm_traffic.txt when that file
holds a line `traffic_bytes_per_launch | <kernel> | N` (taken from such counter runs), else null.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3      # MI355X dense FP32 matrix peak
PEAK_HBM_GBS = 8000.0              # MI355X HBM3E peak

WORKLOADS = {
    "c5": dict(name="qwen3-1.7b-shape full-weight fp32, 4x4096 packed", hidden=2048, layers=28, heads=16, kv_heads=8,
               head_dim=128, ffn=6144, vocab=151936, rms_eps=1e-6, rope_theta=1e6, batch=4, seq=4096, lr=3.14e-4,
               clip=0.0, lora=None),
    "c4": dict(name="qwen3-1.7b-shape LoRA r16 a32 on q/k/v/o fp32, 1x2048", hidden=2048, layers=28, heads=16, kv_heads=8,
               head_dim=128, ffn=6144, vocab=151936, rms_eps=1e-6, rope_theta=1e6, batch=1, seq=2048, lr=3.14e-4,
               clip=0.0, lora=dict(rank=16, alpha=32.0, mask=0b1111)),
    "c1": dict(name="seraph-native 33M full-weight fp32, 8x256 packed", hidden=512, layers=8, heads=8, kv_heads=8,
               head_dim=64, ffn=1408, vocab=8192, rms_eps=1e-6, rope_theta=10000.0, batch=8, seq=256, lr=3.14e-4,
               clip=1.0, lora=None),
}


def norm_gain_slices(w):
    """(start, stop) of every RMSNorm gain inside the flat parameter arena."""
    h, qd, kv, f, V = w["hidden"], w["heads"] * w["head_dim"], w["kv_heads"] * w["head_dim"], w["ffn"], w["vocab"]
    out = [(V * h, V * h + h)]
    stride = h + qd * h + 2 * kv * h + h * qd + h + 3 * f * h
    for l in range(w["layers"]):
        base = V * h + h + l * stride
        out.append((base, base + h))
        pn = base + h + qd * h + 2 * kv * h + h * qd
        out.append((pn, pn + h))
    return out


def cpu_baseline(w, budget_tokens=192):
    """The CPU oracle's own step (same mathematics, OpenMP over rows/heads, double accumulation)
    on a bounded sample: the real widths and vocabulary, `budget_tokens` tokens in one sequence,
    with one and with three layers (best of two runs each, the first run also warms the
    allocator); the per-layer and the head costs are then scaled to the full depth."""
    from oracle import oracle as orc
    T = min(budget_tokens, w["seq"])
    tok = np.random.default_rng(0).integers(0, w["vocab"], T).astype(np.int32)
    best = {}
    for L in (1, 1, 3, 3):
        kw = dict(hidden=w["hidden"], layers=L, heads=w["heads"], kv_heads=w["kv_heads"], head_dim=w["head_dim"],
                  ffn=w["ffn"], vocab=w["vocab"], rms_eps=w["rms_eps"], rope_theta=w["rope_theta"])
        if w["lora"]:
            kw.update(lora_rank=w["lora"]["rank"], lora_alpha=w["lora"]["alpha"], lora_mask=w["lora"]["mask"])
        cfg = orc.make_config(**kw)
        p = np.full(orc.param_count(cfg), 0.01, np.float32)
        lo = np.full(max(orc.lora_param_count(cfg), 1), 0.01, np.float32)
        t0 = time.perf_counter()
        if w["lora"]:
            orc.step_lora(cfg, p, lo, tok)
        else:
            orc.step_full(cfg, p, tok)
        dt = time.perf_counter() - t0
        best[L] = min(best.get(L, dt), dt)
        del p
    per_layer = max((best[3] - best[1]) / 2.0, 1e-9)
    head = max(best[1] - per_layer, 0.0)
    full = head + per_layer * w["layers"]
    # AdamW as the step runs it: one pass over every trainable parameter (all weights, or the adapters), timed once in
    # place on the oracle's own loop; its cost does not depend on the number of tokens
    kw["layers"] = w["layers"]
    cfg = orc.make_config(**kw)
    n = orc.lora_param_count(cfg) if w["lora"] else orc.param_count(cfg)
    import ctypes as C
    arrs = [np.full(n, v, np.float32) for v in (0.01, 1e-3, 0.0, 0.0)]
    t0 = time.perf_counter()
    orc.lib().orc_adamw(*[a.ctypes.data_as(C.POINTER(C.c_float)) for a in arrs], C.c_int64(n), C.c_float(3.14e-6), C.c_float(0.9),
                        C.c_float(0.999), C.c_float(0.01), C.c_float(1e-8), C.c_int(1), C.c_float(w["clip"]))
    opt = time.perf_counter() - t0
    del arrs
    model, cpus = host_cpu()
    return dict(value=round(T / (full + opt), 3), unit="tok/s", cores=orc.num_threads(), kind="port", cpu_model=model, host_cpus=cpus,
                sample=(f"oracle step (fwd+loss+bwd) on {T} tokens in 1 sequence at full width and vocabulary, "
                        f"1 layer {best[1]:.2f}s and 3 layers {best[3]:.2f}s (best of 2); LM-head/embedding cost "
                        f"{head:.2f}s + {per_layer:.2f}s per layer scaled to {w['layers']} layers = {full:.1f}s, plus one "
                        f"AdamW pass over all {n} trainable parameters, {opt:.2f}s (timed once)"))


def host_cpu():
    """(model name, logical CPUs the process may run on) of the host."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        n = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        n = os.cpu_count() or 0
    return model, n


def cpu_ops():
    """The oracle's own loops for the single-op configurations, on the host cores, each on a bounded part of the
    configuration (fewer rows, heads or sequences: the ops are independent per row / head / sequence) and scaled to the whole:
    name -> dict(ms, sample).  Best of two runs each; a few seconds in all."""
    import ctypes as C
    from oracle import oracle as orc
    r = np.random.default_rng(3)
    out = {}

    def best_of_2(fn):
        b = 1e30
        for _ in range(2):
            t0 = time.perf_counter()
            fn()
            b = min(b, time.perf_counter() - t0)
        return b

    def put(name, seconds, factor, sample):
        out[name] = dict(ms=round(1e3 * seconds * factor, 2), unit="ms", cores=orc.num_threads(), kind="port",
                         sample=f"{sample}: {1e3 * seconds:.2f} ms, x {factor:g}")

    # attention at B8 H16 S1024 D64: one sequence, two heads of the sixteen
    S, H, D = 1024, 2, 64
    q, k, v, do = (r.standard_normal((S, H * D)).astype(np.float32) / 8 for _ in range(4))
    put("attention_backward_b8_h16_s1024_d64", best_of_2(lambda: orc.attention_backward(q, k, v, do, H, H, D)), 8 * 16 / H,
        "one sequence of 1024 tokens, 2 heads")
    put("attention_forward_b8_h16_s1024_d64", best_of_2(lambda: orc.attention_forward(q, k, v, H, H, D)), 8 * 16 / H,
        "one sequence of 1024 tokens, 2 heads")
    # the bandwidth-bound chain: half of the 16384 rows (1/64 for the cross entropy, 1/8 for SwiGLU, half of the AdamW elements)
    rows, cols, V = 16384, 2048, 151936
    x = 2 * r.standard_normal((rows // 64, V), dtype=np.float32)
    t = r.integers(0, V, rows // 64).astype(np.uint32)
    put("cross_entropy_grad_16384_x_151936", best_of_2(lambda: orc.cross_entropy_grad(x, t)), 64, "256 rows of 151936")
    del x
    n = rows // 2
    a, b = r.standard_normal((n, cols), dtype=np.float32), 1e-2 * r.standard_normal((n, cols), dtype=np.float32)
    gains = (1 + 0.02 * r.standard_normal(cols)).astype(np.float32)
    put("rmsnorm_backward_16384_x_2048", best_of_2(lambda: orc.rmsnorm_backward_batch(a, gains, b, 1e-6)), 2, "8192 rows of 2048")
    put("qk_norm_backward_16384_x_16_heads_128", best_of_2(lambda: orc.qk_norm_backward(a, b, 16, 128, 1e-6)), 2, "8192 tokens, 16 heads of 128")
    put("rope_backward_16384_x_16_heads_128", best_of_2(lambda: orc.rope(a, 16, 128, 1e6, backward=True)), 2, "8192 tokens, 16 heads of 128")
    table = np.zeros((V, cols), np.float32)
    tok = r.integers(0, V, n).astype(np.uint32)
    f32p = lambda arr: arr.ctypes.data_as(C.POINTER(C.c_float))
    put("embedding_backward_16384_x_2048_into_151936_rows",
        best_of_2(lambda: orc.lib().orc_embedding_backward(tok.ctypes.data_as(C.POINTER(C.c_uint32)), f32p(a), f32p(table), C.c_int64(n),
                                                           C.c_int64(cols), C.c_int64(V))), 2, "8192 tokens into the 151936-row table, in place")
    del table
    g3 = [r.standard_normal((rows // 8, 6144), dtype=np.float32) for _ in range(3)]
    put("swiglu_backward_16384_x_6144", best_of_2(lambda: orc.swiglu_backward(*g3)), 8, "2048 rows of 6144")
    del g3
    m = 25_000_000
    arrs = [np.full(m, val, np.float32) for val in (0.01, 1e-3, 0.0, 0.0)]
    for clip in (0.0, 1.0):
        put(f"adamw_50m_clip_{clip:g}",
            best_of_2(lambda: orc.lib().orc_adamw(*[f32p(z) for z in arrs], C.c_int64(m), C.c_float(3.14e-4), C.c_float(0.9), C.c_float(0.999),
                                                  C.c_float(0.01), C.c_float(1e-8), C.c_int(1), C.c_float(clip))), 2, "25 M elements, in place")
    return out


def measured_traffic(kernel, workload):
    """HBM bytes per launch of `kernel` from the committed counter summary, or None."""
    path = os.path.join(ROOT, "profiles", f"train_step_{workload}_hbm_traffic.txt")
    try:
        with open(path) as f:
            for line in f:
                part = [x.strip() for x in line.split("|")]
                if len(part) == 3 and part[0] == "traffic_bytes_per_launch" and part[1] == kernel:
                    return float(part[2])
    except OSError:
        pass
    return None


def gemm_table(w):
    """Every GEMM shape of one training step of workload `w`, timed alone through the C ABI and,
    beside it, torch.matmul (hipBLASLt) on the same operands; prints one line per shape."""
    import torch
    from seraph_amd import ops
    ops.init(0)

    def timeit(fn):
        # about 30 ms of untimed calls first (a row that follows allocations and host work would otherwise be timed on
        # clocks that have not come back up: the first row of either table read 6-10 % slow for both libraries), then
        # at least 5 calls and 50 ms under one event pair
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        once = max(time.perf_counter() - t0, 1e-5)
        for _ in range(min(200, max(2, int(0.03 / once)))):
            fn()
        iters = min(200, max(5, int(0.05 / once)))
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(iters):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    T, h, f, V = w["batch"] * w["seq"], w["hidden"], w["ffn"], w["vocab"]
    qd, kv, L = w["heads"] * w["head_dim"], w["kv_heads"] * w["head_dim"], w["layers"]
    tot = [0.0, 0.0]
    warm_a, warm_b = torch.randn(4096, 4096, device="cuda"), torch.randn(4096, 4096, device="cuda")
    for _ in range(60):                                        # the clocks settle before the first row is timed
        torch.matmul(warm_a, warm_b)
    torch.cuda.synchronize()
    del warm_a, warm_b
    for name, o, i, per_step in (("q", qd, h, L), ("k/v", kv, h, 2 * L), ("o", h, qd, L), ("gate/up", f, h, 2 * L),
                                 ("down", h, f, L), ("lm head", V, h, 1)):
        for form, M, N, K, tA, tB in ((f"fwd {name} NT", T, o, i, 0, 1), (f"dgrad {name} NN", T, i, o, 0, 0),
                                      (f"wgrad {name} TN", o, i, T, 1, 0)):
            A = torch.randn((K, M) if tA else (M, K), device="cuda")
            B = torch.randn((N, K) if tB else (K, N), device="cuda")
            C = torch.empty(M, N, device="cuda")
            ms = timeit(lambda: ops.gemm(A, B, M, N, K, tA, tB, out=C))
            ref = timeit(lambda: torch.matmul(A.T if tA else A, B.T if tB else B, out=C))
            tot[0] += per_step * ms
            tot[1] += per_step * ref
            print(f"{form:18s} {M:6d} x {N:6d} x {K:6d}: {ms:8.3f} ms {2 * M * N * K / ms / 1e9:6.1f} TFLOP/s | "
                  f"hipBLASLt {ref:8.3f} ms {2 * M * N * K / ref / 1e9:6.1f} TFLOP/s | x{per_step} per step", flush=True)
            del A, B, C
    print(f"GEMM time per step, one launch per product: this library {tot[0]:.1f} ms, hipBLASLt {tot[1]:.1f} ms")

    # The launches the step really makes for projections that share an operand: q/k/v and gate/up forward and their
    # weight gradients as one grouped launch each, their input gradients as one launch that sums the products.
    print("\nproducts the step joins in one launch (hipBLASLt column: the same products one call each, the sum with beta = 1):")
    R = lambda *sh: torch.randn(*sh, device="cuda")
    fused = [0.0, 0.0]
    for name, outs in (("q+k+v", (qd, kv, kv)), ("gate+up", (f, f))):
        x, ws = R(T, h), [R(o, h) for o in outs]
        ys, gs, dws = [torch.empty(T, o, device="cuda") for o in outs], [R(T, o) for o in outs], [torch.zeros(o, h, device="cuda") for o in outs]
        dx = torch.empty(T, h, device="cuda")
        flops = 2.0 * T * h * sum(outs)
        cases = (
            (f"fwd {name} grouped NT", lambda: ops.gemm_grouped([(x, w_, y, T, o) for w_, y, o in zip(ws, ys, outs)], h, 0, 1),
             lambda: [torch.matmul(x, w_.T, out=y) for w_, y in zip(ws, ys)]),
            (f"dgrad {name} summed NN", lambda: ops.gemm_chain([(g_, w_, o) for g_, w_, o in zip(gs, ws, outs)], T, h, 0, 0, out=dx),
             lambda: [torch.matmul(gs[0], ws[0], out=dx)] + [dx.addmm_(g_, w_) for g_, w_ in zip(gs[1:], ws[1:])]),
            (f"wgrad {name} grouped TN", lambda: ops.gemm_grouped([(g_, x, dw, o, h) for g_, dw, o in zip(gs, dws, outs)], T, 1, 0, accumulate=True),
             lambda: [dw.addmm_(g_.T, x) for g_, dw in zip(gs, dws)]),
        )
        for form, ours, theirs in cases:
            ms, ref = timeit(ours), timeit(theirs)
            fused[0] += L * ms
            fused[1] += L * ref
            print(f"{form:26s} {T} tokens, widths {h} <-> {'+'.join(str(o) for o in outs)}: {ms:8.3f} ms {flops / ms / 1e9:6.1f} TFLOP/s | "
                  f"hipBLASLt {ref:8.3f} ms {flops / ref / 1e9:6.1f} TFLOP/s | x{L} per step", flush=True)
        del x, ws, ys, gs, dws, dx
    print(f"these launches per step: this library {fused[0]:.1f} ms, hipBLASLt {fused[1]:.1f} ms")


def run_workload(w, key, steps, warmup, op_timing=True, pmc_calibration=False, wgrad_overlap=True):
    """`warmup` untimed steps, then `steps` timed ones of workload `w`; returns the fields of the bench line."""
    import torch
    from seraph_amd import trainer as tr

    T = w["batch"] * w["seq"]
    lora = w["lora"] or dict(rank=0, alpha=0.0, mask=0)
    cfg = tr.model_config(w["hidden"], w["layers"], w["heads"], w["kv_heads"], w["head_dim"], w["ffn"], w["vocab"],
                          w["rms_eps"], w["rope_theta"], lora["rank"], lora["alpha"], lora["mask"], 1 if w.get("qk_norm") else 0)
    opt = tr.optim_config(w["lr"], clip=w["clip"])
    n = tr.param_count(cfg)

    torch.manual_seed(1234)
    dev = torch.device("cuda:0")
    params = torch.empty(n, dtype=torch.float32, device=dev).normal_(0.0, 0.02)
    for a, b in norm_gain_slices(w):
        params[a:b] = 1.0
    if w["lora"]:
        ext = (params, None, None, None)
    else:
        ext = (params, torch.zeros(n, dtype=torch.float32, device=dev), torch.zeros(n, dtype=torch.float32, device=dev),
               torch.zeros(n, dtype=torch.float32, device=dev))
    torch.cuda.synchronize()
    t = tr.Trainer(cfg, opt, max_tokens=T, max_batch=w["batch"], device=0, ext=ext)
    if not wgrad_overlap:
        t.enable_wgrad_overlap(False)                     # else the trainer's own choice by step size
    if w["lora"]:
        nl = tr.lora_param_count(cfg)
        lo = (0.01 * np.random.default_rng(5).standard_normal(nl)).astype(np.float32)     # A ~ N(0, 0.01)
        h, qd, kv, r = w["hidden"], w["heads"] * w["head_dim"], w["kv_heads"] * w["head_dim"], lora["rank"]
        o = 0
        for _ in range(w["layers"]):                                                    # B = 0
            for i, oo in ((h, qd), (h, kv), (h, kv), (qd, h)):
                o += r * i
                lo[o:o + oo * r] = 0
                o += oo * r
        t.upload(tr.LORA_PARAMS, lo)

    if pmc_calibration:
        from seraph_amd import ops
        cal = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        for _ in range(3):
            ops.scale_(cal, 1.0)
        torch.cuda.synchronize()
        del cal

    rng = np.random.default_rng(99)
    starts = np.arange(0, T + 1, w["seq"], dtype=np.int32)
    batches = [rng.integers(0, w["vocab"], T).astype(np.int32) for _ in range(warmup + steps)]

    losses = []
    tw = time.perf_counter()
    for i in range(warmup):
        losses.append(t.step(batches[i], starts))
    torch.cuda.synchronize()
    warm_ms = 1000.0 * (time.perf_counter() - tw) / max(warmup, 1)

    # Per-kernel timing brackets every kernel-library call of the step with a HIP event pair on the step's
    # stream.  On a step of hundreds of milliseconds that costs well under 1 % and runs inside the timed
    # region.  On a step of a few milliseconds (c1) the ~1000 event records would take a third of the step, and
    # the ~12000 of the LoRA step (c4, 130 ms) a tenth of it, so there the timed region runs without them and the
    # same batches are replayed once more with them.
    in_region = op_timing and (warmup == 0 or warm_ms >= 400.0)
    t.enable_op_timing(in_region)
    t.reset_op_stats()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        losses.append(t.step(batches[warmup + i], starts))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timing = t.last_timing()
    roofline_from = "timed region"
    if not in_region and op_timing:
        t.enable_op_timing(True)
        t.reset_op_stats()
        for i in range(steps):
            t.step(batches[warmup + i], starts)
        torch.cuda.synchronize()
        roofline_from = ("second pass over the timed region's batches: per-kernel events inside a step this short "
                         "would dominate it")

    stats = t.op_stats()
    total_ms = sum(s["ms"] for s in stats) or 1.0
    kernels = {}
    for s in sorted(stats, key=lambda s: -s["ms"]):
        avg = s["ms"] / max(s["launches"], 1)
        e = dict(launches=s["launches"], avg_ms=round(avg, 4), share=round(s["ms"] / total_ms, 4))
        if s["flops"] > 0:
            e["tflops"] = round(s["flops"] / s["ms"] / 1e9, 2)
            e["frac_mfma_peak"] = round(s["flops"] / s["ms"] / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4)
        elif s["bytes"] > 0:
            e["gbs"] = round(s["bytes"] / s["ms"] / 1e6, 1)
            e["frac_hbm_peak"] = round(s["bytes"] / s["ms"] / 1e6 / PEAK_HBM_GBS, 4)
        kernels[s["name"]] = e
    dom = max(stats, key=lambda s: s["ms"]) if stats else None
    if dom is None:
        roofline = None
    elif dom["flops"] > 0:
        achieved = dom["flops"] / dom["ms"] / 1e9
        roofline = dict(bound="mfma", kernel=dom["name"], achieved=round(achieved, 2), peak=PEAK_FP32_MFMA_TFLOPS,
                        unit="TFLOP/s", frac=round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), traffic=None,
                        launches=dom["launches"], avg_launch_ms=round(dom["ms"] / dom["launches"], 4),
                        flops_per_launch=dom["flops"] / dom["launches"])
    else:
        achieved = dom["bytes"] / dom["ms"] / 1e6
        roofline = dict(bound="hbm", kernel=dom["name"], achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                        frac=round(achieved / PEAK_HBM_GBS, 4), traffic=None, launches=dom["launches"],
                        avg_launch_ms=round(dom["ms"] / dom["launches"], 4), bytes_per_launch=dom["bytes"] / dom["launches"])

    if roofline is not None:
        roofline["traffic"] = measured_traffic(dom["name"], key)
        roofline["measured_over"] = roofline_from

    out = {
        "value": round(steps * T / elapsed, 2), "unit": "tok/s", "steps": steps, "warmup": warmup,
        "ms_per_step": round(1000.0 * elapsed / steps, 3),
        "config": {"workload": w["name"], "tokens_per_step": T, "batch": w["batch"], "seq_len": w["seq"],
                   "params": n, "device_bytes": t.device_bytes + sum(x.numel() * 4 for x in ext if x is not None),
                   "rms_eps": w["rms_eps"], "adamw_clip": w["clip"], "qk_norm": bool(w.get("qk_norm")), "seed": 1234},
        "loss_first_last": [round(losses[0], 5), round(losses[-1], 5)],
        "phase_ms_last_step": {k: round(v, 3) for k, v in timing.items()},
        "roofline": roofline,
        "kernels": kernels,
    }
    t.close()
    del params, ext
    torch.cuda.empty_cache()
    return out


def time_op(fn, iters, warm=2, reps=1):
    """Mean device time of one fn() call in ms.  One event pair brackets `reps` back-to-back calls (a pair costs a few
    microseconds, which matters for ops of tens of microseconds); the events are recorded on the stream the op is
    launched on (the ops below run on torch's current stream, which is where torch records its events).  fn gets a
    running call index so that it can rotate between operand sets."""
    import torch
    ms = []
    call = 0
    # Untimed calls for about 40 ms first.  Two warm-up groups were not enough for the first op that runs on freshly
    # allocated operand sets: the RMSNorm backward read 77 us in a process's first pass and 72 us in every later one
    # (the other ops moved by under 1 %), so the figure depended on what had run before it.
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.04:
        for _ in range(reps):
            fn(call)
            call += 1
        torch.cuda.synchronize()
    for i in range(warm + iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(reps):
            fn(call)
            call += 1
        b.record()
        torch.cuda.synchronize()
        if i >= warm:
            ms.append(a.elapsed_time(b) / reps)
    return sum(ms) / len(ms), min(ms)


def isolated_ops():
    """The single-op configurations: causal attention backward at B8 H16 S1024 D64 and the bandwidth-bound backward
    chain over 16384 tokens (hidden 2048, FFN 6144, vocabulary 151936, AdamW over 50 M parameters), each op alone
    through the C ABI.  Bandwidth-bound ops run on operands too large for the caches or on rotating operand sets,
    so every call starts cold.  Algorithmic work: each input read once, each output written once."""
    import torch
    from seraph_amd import ops
    ops.init(0)
    out = {}
    dev = "cuda"

    # 24 calls per event pair: the pair's markers and the first launch's way to an idle queue (some 30 us together)
    # weigh a microsecond on each call instead of five
    def hbm(name, nbytes, fn, iters=6, reps=24, note=None):
        avg, best = time_op(fn, iters, reps=reps)
        e = dict(ms=round(avg, 4), min_ms=round(best, 4), bound="hbm", algorithmic_bytes=nbytes,
                 achieved=round(nbytes / avg / 1e6, 1), unit="GB/s", peak=PEAK_HBM_GBS, frac=round(nbytes / avg / 1e6 / PEAK_HBM_GBS, 4))
        if note:
            e["note"] = note
        out[name] = e

    # ---- attention backward, B8 H16 S1024 D64 (saved O and log-sum-exp from the forward, as the step has them)
    B, S, H, D = 8, 1024, 16, 64
    T = B * S
    g = torch.Generator(device=dev).manual_seed(7)
    mk = lambda w: torch.randn(T, w, device=dev, generator=g) / 8.0
    Q, K, V, dO = mk(H * D), mk(H * D), mk(H * D), mk(H * D)
    ss = torch.arange(0, T + 1, S, device=dev, dtype=torch.int32)
    O, L = ops.attention_forward(Q, K, V, H, H, D, ss)
    dQ, dK, dV = torch.empty_like(Q), torch.zeros_like(K), torch.zeros_like(V)
    flops = 10.0 * D * H * B * S * (S + 1) / 2
    # (16 calls per event pair, for the reason given at hbm() above)
    avg, best = time_op(lambda i: ops.attention_backward(Q, K, V, dO, H, H, D, ss, out=O, lse=L, dK=dK, dV=dV, dQ=dQ, max_seq_len=S), 6, reps=16)
    out["attention_backward_b8_h16_s1024_d64"] = dict(
        ms=round(avg, 4), min_ms=round(best, 4), bound="mfma", algorithmic_flops=flops, achieved=round(flops / avg / 1e9, 2),
        unit="TFLOP/s", peak=PEAK_FP32_MFMA_TFLOPS, frac=round(flops / avg / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4),
        note="delta + dK/dV (+ dS band) + dQ kernels; dK/dV accumulate into the caller's buffers")
    avg, best = time_op(lambda i: ops.attention_forward(Q, K, V, H, H, D, ss), 6, reps=16)
    out["attention_forward_b8_h16_s1024_d64"] = dict(
        ms=round(avg, 4), min_ms=round(best, 4), bound="mfma", algorithmic_flops=0.4 * flops, achieved=round(0.4 * flops / avg / 1e9, 2),
        unit="TFLOP/s", peak=PEAK_FP32_MFMA_TFLOPS, frac=round(0.4 * flops / avg / 1e9 / PEAK_FP32_MFMA_TFLOPS, 4))
    del Q, K, V, dO, O, L, dQ, dK, dV

    # ---- cross entropy 16384 x 151936, logits N(0, 2), gradient written over the logits as in the step
    rows, cols = 16384, 151936
    x = torch.randn(rows, cols, device=dev, generator=g) * 2.0
    tgt = torch.randint(0, cols, (rows,), device=dev, dtype=torch.int32)

    def ce(i):
        ops.cross_entropy_grad(x, tgt, rows, grad=x)
    # in place the second call would see gradients as logits: still 2 x rows x cols x 4 bytes of the same traffic
    hbm("cross_entropy_grad_16384_x_151936", 2 * rows * cols * 4 + 8 * rows, ce, iters=5, reps=1)
    del x

    # ---- RMSNorm backward 16384 x 2048 (x N(0,1), gains N(1, 0.02), dY N(0, 1e-2)); three operand sets in rotation
    rows, cols = 16384, 2048
    sets = [(torch.randn(rows, cols, device=dev, generator=g), torch.randn(rows, cols, device=dev, generator=g) * 1e-2,
             torch.empty(rows, cols, device=dev)) for _ in range(3)]
    gains = 1.0 + 0.02 * torch.randn(cols, device=dev, generator=g)
    gs = torch.zeros(cols, device=dev)
    hbm("rmsnorm_backward_16384_x_2048", 3 * rows * cols * 4 + 2 * cols * 4,
        lambda i: ops.rmsnorm_backward(sets[i % 3][0], gains, sets[i % 3][1], 1e-6, grad_scale=gs, out=sets[i % 3][2]),
        note="row kernel + column sum of the gain gradient")
    # qk_norm backward as the step runs it (from the normalised output and the saved rms), all 16 heads of a token together
    rms_tok = torch.rand(rows, device=dev, generator=g) + 0.5
    hbm("qk_norm_backward_16384_x_16_heads_128", 3 * rows * cols * 4 + 4 * rows,
        lambda i: ops.qk_norm_backward_saved(sets[i % 3][0], rms_tok, sets[i % 3][1], 16, 128, 1e-6, out=sets[i % 3][2]))
    # RoPE backward in place over 16 heads of 128
    hbm("rope_backward_16384_x_16_heads_128", 2 * rows * cols * 4,
        lambda i: ops.rope(sets[i % 3][0], 16, 128, 1e6, None, backward=True, out=sets[i % 3][0]))
    # embedding backward: 16384 rows of 2048 into a 151936-row table, uniform tokens
    # Eight token sets in rotation: every call touches other rows of the 1.24 GB table (8 x 127 MB of rows), so the rows,
    # like the gradients, come from HBM.  With one token set for every call the touched rows stay in the 256 MB
    # last-level cache between calls; that figure goes into the note.
    V = 151936
    toks = [torch.randint(0, V, (rows,), device=dev, dtype=torch.int32) for _ in range(8)]
    uniq = sum(int(torch.unique(t).numel()) for t in toks) / len(toks)
    table = torch.zeros(V, cols, device=dev)
    warm, _ = time_op(lambda i: ops.embedding_backward(toks[0], sets[i % 3][0], table), 4, reps=24)
    hbm("embedding_backward_16384_x_2048_into_151936_rows", int(rows * cols * 4 + 2 * uniq * cols * 4 + rows * 4),
        lambda i: ops.embedding_backward(toks[i % 8], sets[i % 3][0], table),
        note=f"{uniq:.0f} distinct tokens per call, eight token sets in rotation; two launches (chain links, row sums); "
             f"with the same tokens every call (touched rows still in the last-level cache) {1e3 * warm:.1f} us")
    del sets, table

    # ---- SwiGLU backward 16384 x 6144
    n = 16384 * 6144
    gate, up, dH = (torch.randn(n, device=dev, generator=g) for _ in range(3))
    outs = (torch.empty(n, device=dev), torch.empty(n, device=dev))
    hbm("swiglu_backward_16384_x_6144", 5 * n * 4, lambda i: ops.swiglu_backward(gate, up, dH, out=outs))
    del gate, up, dH, outs

    # ---- AdamW over 50 M parameters, gradients N(0, 1e-3) with 1 % entries of magnitude 10
    n = 50_000_000
    wts = [torch.randn(n, device=dev, generator=g) * 0.02 for _ in range(2)]
    grad = torch.randn(n, device=dev, generator=g) * 1e-3
    grad[torch.rand(n, device=dev, generator=g) < 0.01] = 10.0
    m, v = torch.zeros(n, device=dev), torch.zeros(n, device=dev)
    for clip in (0.0, 1.0):
        hbm(f"adamw_50m_clip_{clip:g}", 7 * n * 4,
            lambda i: ops.adamw_(wts[i % 2], grad, m, v, 3.14e-4, 0.9, 0.999, 0.01, 1e-8, 1 + i, clip),
            note="clip 0 is the reference's formula" if clip == 0.0 else "per-element clamp of the gradient first")
    del wts, grad, m, v
    torch.cuda.empty_cache()
    return out


def reference_cpu_step(w, tokens=64):
    """The reference's own CPU training step (its C code in src/train.c, compiled from the Seraph tree into
    oracle/_ref/ref_step_hip where that tree was present at build time), one sequence of `tokens` tokens,
    single-threaded as the reference runs it.  None when the binary is not there."""
    import struct
    import subprocess
    import tempfile
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_step_hip")
    if not os.path.exists(exe) or w["lora"]:
        return None
    from oracle import oracle as orc
    cfg = orc.make_config(hidden=w["hidden"], layers=w["layers"], heads=w["heads"], kv_heads=w["kv_heads"], head_dim=w["head_dim"],
                          ffn=w["ffn"], vocab=w["vocab"], rms_eps=w["rms_eps"], rope_theta=w["rope_theta"])
    n = orc.param_count(cfg)
    r = np.random.default_rng(3)
    with tempfile.TemporaryDirectory() as d:
        with open(os.path.join(d, "in.bin"), "wb") as f:
            f.write(struct.pack("11i", w["hidden"], w["layers"], w["heads"], w["kv_heads"], w["head_dim"], w["ffn"], w["vocab"], 1, tokens, 0, 0))
            f.write(struct.pack("3f", w["lr"], w["rope_theta"], 0.0))
            f.write((0.02 * r.standard_normal(n)).astype(np.float32).tobytes())
            f.write(r.integers(0, w["vocab"], tokens).astype(np.int32).tobytes())
        p = subprocess.run([exe, "--cpu", "--time", os.path.join(d, "in.bin"), os.path.join(d, "out.bin")],
                           capture_output=True, text=True, timeout=600)
    for line in p.stdout.splitlines():
        if line.startswith("seconds_per_step"):
            sec = float(line.split()[1])
            return dict(value=round(tokens / sec, 3), unit="tok/s", cores=1, kind="reference",
                        sample=(f"the reference's CPU training step (train_step with no backend: train_forward_fp32, loss, "
                                f"train_backward, AdamW; src/train.c) on one sequence of {tokens} tokens of this model, "
                                f"{sec:.1f} s, single-threaded as the reference runs it; its backward is the reference's "
                                f"approximate CPU gradient, timed only"))
    return None


def drop_in_step(w, seq, steps=6):
    """tok/s of the reference's own step driver (train_step -> train_step_gpu_full, unmodified, one sequence per step,
    its per-tensor AdamW and cache copies) running over this backend's vulkan_* symbols: what `make hip` gives a
    Seraph user without touching train.c.  None when oracle/_ref/ref_step_hip is not there."""
    import struct
    import subprocess
    import tempfile
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_step_hip")
    if not os.path.exists(exe) or w["lora"]:
        return None
    from oracle import oracle as orc
    cfg = orc.make_config(hidden=w["hidden"], layers=w["layers"], heads=w["heads"], kv_heads=w["kv_heads"], head_dim=w["head_dim"],
                          ffn=w["ffn"], vocab=w["vocab"])
    n = orc.param_count(cfg)
    r = np.random.default_rng(4)
    with tempfile.TemporaryDirectory() as d:
        with open(os.path.join(d, "in.bin"), "wb") as f:
            f.write(struct.pack("11i", w["hidden"], w["layers"], w["heads"], w["kv_heads"], w["head_dim"], w["ffn"], w["vocab"], steps, seq, 0, 0))
            f.write(struct.pack("3f", w["lr"], w["rope_theta"], 0.0))
            f.write((0.02 * r.standard_normal(n)).astype(np.float32).tobytes())
            f.write(r.integers(0, w["vocab"], steps * seq).astype(np.int32).tobytes())
        p = subprocess.run([exe, "--time", os.path.join(d, "in.bin"), os.path.join(d, "out.bin")], capture_output=True, text=True, timeout=600)
    for line in p.stdout.splitlines():
        if line.startswith("seconds_per_step"):
            sec = float(line.split()[1])
            return dict(value=round(seq / sec, 1), unit="tok/s", ms_per_step=round(1000 * sec, 3), tokens_per_step=seq,
                        what="reference train_step_gpu_full, unmodified, over this backend; one sequence per step")
    return None


def front_end_step(w, binary, steps=45, skip=8):
    """tok/s of the reference's own batched front end (tools/seraph_train_cuda.c, unmodified) training this model from a
    model directory and a .ttok file, `batch` packed sequences of `seq` tokens per step: the median of the rates it prints
    per step (its own clock around its step call), first `skip` steps left out.  `binary` is one of the two builds of
    that front end under oracle/_ref/ (where the Seraph tree was present at build time): over the cuda_train_* ops one
    by one, or with the fused step behind cuda_train_step_gpu_full_batch.  None when the binary is not there."""
    import re
    import subprocess
    import tempfile
    exe = os.path.join(ROOT, "oracle", "_ref", binary)
    if not os.path.exists(exe) or w["lora"]:
        return None
    from seraph_amd import io as sio
    from seraph_amd import trainer as tr
    shape = dict(hidden=w["hidden"], layers=w["layers"], heads=w["heads"], kv_heads=w["kv_heads"], head_dim=w["head_dim"],
                 ffn=w["ffn"], vocab=w["vocab"])
    cfg = tr.model_config(**shape, rms_eps=1e-5, rope_theta=w["rope_theta"])
    r = np.random.default_rng(5)
    arena = (0.02 * r.standard_normal(tr.param_count(cfg))).astype(np.float32)
    for a, b in norm_gain_slices(w):
        arena[a:b] = 1.0
    B, S = w["batch"], w["seq"]
    with tempfile.TemporaryDirectory() as d:
        sio.checkpoint_save(os.path.join(d, "model.safetensors"), cfg, arena)
        with open(os.path.join(d, "config.json"), "w") as f:
            json.dump({"model_type": "qwen2", "vocab_size": w["vocab"], "hidden_size": w["hidden"], "num_hidden_layers": w["layers"],
                       "intermediate_size": w["ffn"], "num_attention_heads": w["heads"], "num_key_value_heads": w["kv_heads"],
                       "head_dim": w["head_dim"], "rms_norm_eps": 1e-6, "rope_theta": w["rope_theta"]}, f)
        with open(os.path.join(d, "vocab.json"), "w") as f:        # the reference's train_init wants a tokenizer to be there
            json.dump({f"t{i}": i for i in range(w["vocab"])}, f)
        with open(os.path.join(d, "merges.txt"), "w") as f:
            f.write("t 0\n")
        n = steps * B
        sio.ttok_write(os.path.join(d, "train.ttok"), r.integers(0, w["vocab"], n * S).astype(np.int32),
                       np.arange(0, n * S + 1, S, dtype=np.int32), w["vocab"])
        p = subprocess.run([exe, d, os.path.join(d, "train.ttok"), "--full-training", "--batch", str(B), "--max-seq", str(S),
                            "--lr", str(w["lr"]), "--log-every", "1", "--save-every", "0", "--checkpoint", os.path.join(d, "ckpt")],
                           capture_output=True, text=True, timeout=900)
    rates = [float(x) for x in re.findall(r"Step \d+/\d+ \| Loss: [0-9.]+ .*? ([0-9]+) tok/s", p.stdout)]
    if p.returncode != 0 or len(rates) <= skip:
        return None
    rates = sorted(rates[skip:])
    med = rates[len(rates) // 2]
    return dict(value=med, unit="tok/s", ms_per_step=round(1e3 * B * S / med, 3), tokens_per_step=B * S,
                what=f"{binary}: the reference's tools/seraph_train_cuda.c, unmodified, {B} x {S} packed per step, median of "
                     f"the {len(rates)} per-step rates it printed after the first {skip}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="c5", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true")
    ap.add_argument("--no-op-timing", action="store_true",
                    help="do not bracket every kernel-library call with an event pair (no roofline / kernels objects)")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the headline workload: no other workloads, isolated ops or drop-in path in the line")
    ap.add_argument("--one-stream", action="store_true",
                    help="keep the weight gradients on the step's one stream (default: on a second stream beside the chain)")
    ap.add_argument("--gemm-table", action="store_true",
                    help="instead of the benchmark, time every GEMM shape of the workload's step beside hipBLASLt")
    args = ap.parse_args()
    if args.gemm_table:
        gemm_table(WORKLOADS[args.workload])
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
                 "(value is the one GPU's throughput)")

    w = WORKLOADS[args.workload]
    head = run_workload(w, args.workload, args.steps, args.warmup, op_timing=not args.no_op_timing, wgrad_overlap=not args.one_stream,
                        pmc_calibration=args.pmc_calibration)
    # Key order: the bulky per-kernel tables first, the contract's keys after them and a compact `summary` of every
    # headline number last, so that a reader who keeps only the end of the line still has all of them.
    out = {"kernels": head["kernels"]}
    contract = {
        "metric": "train tok/s (fwd+bwd+AdamW)", "value": head["value"], "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": head["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": head["config"], "loss_first_last": head["loss_first_last"], "phase_ms_last_step": head["phase_ms_last_step"],
        "roofline": head["roofline"],
    }
    full = args.workload == "c5" and not args.headline_only
    if full:
        # the rest of the metric: the 33M model and the LoRA configuration as whole steps, the single-op
        # configurations alone, and the unmodified reference step driver over the vulkan_* symbols
        others = {}
        # The two 1.7B configurations again with qk_norm on: the reference's text-mode step never applies it
        # (src/train.c:4687-4689 acts only with the video flag), so the headline leaves it off; these lines say what
        # the RMS over all heads after RoPE and its backward cost when the option is used.
        extra = {"c5_with_qk_norm": dict(WORKLOADS["c5"], qk_norm=1, name=WORKLOADS["c5"]["name"] + ", qk_norm on"),
                 "c4_with_qk_norm": dict(WORKLOADS["c4"], qk_norm=1, name=WORKLOADS["c4"]["name"] + ", qk_norm on")}
        for key, steps, warmup in (("c1", 30, 5), ("c4", 8, 2), ("c5_with_qk_norm", 2, 1), ("c4_with_qk_norm", 4, 1)):
            r = run_workload(WORKLOADS.get(key) or extra[key], key, steps, warmup, op_timing=not args.no_op_timing, wgrad_overlap=not args.one_stream)
            others[key] = {k: r[k] for k in ("value", "unit", "ms_per_step", "steps", "warmup", "config", "loss_first_last", "roofline")}
            top = sorted(r["kernels"].items(), key=lambda kv: -kv[1]["share"])[:6]
            others[key]["kernels"] = dict(top)
        out["workloads"] = others
        out["ops"] = isolated_ops()
        c1 = WORKLOADS["c1"]
        di = {f"c1_shape_1x{seq}": drop_in_step(c1, seq) for seq in (256, 2048)}
        di["c1_front_end_op_by_op_8x256"] = front_end_step(c1, "seraph-train-cuda-hip")
        di["c1_front_end_fused_8x256"] = front_end_step(c1, "seraph-train-cuda-hip-fused")
        if any(v is not None for v in di.values()):
            out["drop_in_path"] = di
    if not args.no_cpu_baseline:
        contract["cpu_baseline"] = cpu_baseline(w)
        if full:
            c1 = WORKLOADS["c1"]
            from oracle import oracle as orc
            tok = np.random.default_rng(0).integers(0, c1["vocab"], 2048).astype(np.int32)
            cfg = orc.make_config(hidden=c1["hidden"], layers=c1["layers"], heads=c1["heads"], kv_heads=c1["kv_heads"],
                                  head_dim=c1["head_dim"], ffn=c1["ffn"], vocab=c1["vocab"], rms_eps=c1["rms_eps"], rope_theta=c1["rope_theta"])
            p = np.full(orc.param_count(cfg), 0.01, np.float32)
            best = 1e9
            for _ in range(2):
                t0 = time.perf_counter()
                _, g = orc.step_full(cfg, p, tok, np.arange(0, 2049, 256, dtype=np.int32))
                z = np.zeros_like(p)
                orc.adamw(p, g, z, z, 3.14e-6, 0.9, 0.999, 0.01, 1e-8, 1, clip=1.0)
                best = min(best, time.perf_counter() - t0)
            out["workloads"]["c1"]["cpu_baseline"] = dict(
                value=round(2048 / best, 2), unit="tok/s", cores=orc.num_threads(), kind="port",
                sample=f"one full step of the 33M configuration (8 x 256 tokens: forward, loss, backward, AdamW) with the oracle, {best:.2f} s (best of 2)")
            ref = reference_cpu_step(c1)
            if ref is not None:
                out["workloads"]["c1"]["cpu_baseline_reference"] = ref
            for name, cpu in cpu_ops().items():
                if name in out["ops"]:
                    out["ops"][name]["cpu_baseline"] = cpu
    out.update(contract)
    summary = {args.workload: [head["value"], head["ms_per_step"]]}
    for key, r in out.get("workloads", {}).items():
        summary[key] = [r["value"], r["ms_per_step"]]
    if "ops" in out:
        summary["ops"] = {k: v["frac"] for k, v in out["ops"].items()}
    for key, r in (out.get("drop_in_path") or {}).items():
        if r is not None:
            summary["drop_in_" + key] = [r["value"], r["ms_per_step"]]
    summary["units"] = "workloads and drop-in paths: [tok/s, ms per step]; ops: fraction of the bounding peak (HBM 8 TB/s, FP32 MFMA 157.3 TFLOP/s)"
    out["summary"] = summary
    print(json.dumps(out))


if __name__ == "__main__":
    main()
