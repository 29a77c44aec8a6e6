#!/usr/bin/env python3
"""Headline benchmark: training tokens/s (forward + backward + AdamW) of the packed-batch
training step on ONE MI355X, with the dominant kernel's roofline fraction measured live and
the CPU oracle timed beside it.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c5|c4|c1] [--pmc-calibration]

Workloads (BASELINE.json configs): c5 = Qwen3-1.7B-shape full-weight FP32 training,
4 x 4096 tokens (default); c4 = the same model, LoRA r16 on q/k/v/o, 1 x 2048; c1 = the
33M Seraph-native model, 8 x 256.  Synthetic data: uniform token ids, N(0, 0.02) weights,
norm gains 1, fixed seeds.  Prints ONE JSON line.

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
    return dict(value=round(T / full, 3), unit="tok/s", cores=orc.num_threads(), kind="port",
                sample=(f"oracle step (fwd+loss+bwd, no AdamW) on {T} tokens in 1 sequence at full width and vocabulary, "
                        f"1 layer {best[1]:.2f}s and 3 layers {best[3]:.2f}s (best of 2); LM-head/embedding cost "
                        f"{head:.2f}s + {per_layer:.2f}s per layer scaled to {w['layers']} layers"))


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

    def timeit(fn, iters=5, warm=2):
        for _ in range(warm):
            fn()
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
    print(f"GEMM time per step: this library {tot[0]:.1f} ms, hipBLASLt {tot[1]:.1f} ms")


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
    ap.add_argument("--gemm-table", action="store_true",
                    help="instead of the benchmark, time every GEMM shape of the workload's step beside hipBLASLt")
    args = ap.parse_args()
    if args.gemm_table:
        gemm_table(WORKLOADS[args.workload])
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus N with N > 1 is not supported "
                 "(value is the one GPU's throughput)")

    import torch
    from seraph_amd import trainer as tr

    w = WORKLOADS[args.workload]
    T = w["batch"] * w["seq"]
    lora = w["lora"] or dict(rank=0, alpha=0.0, mask=0)
    cfg = tr.model_config(w["hidden"], w["layers"], w["heads"], w["kv_heads"], w["head_dim"], w["ffn"], w["vocab"],
                          w["rms_eps"], w["rope_theta"], lora["rank"], lora["alpha"], lora["mask"])
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

    if args.pmc_calibration:
        from seraph_amd import ops
        cal = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        for _ in range(3):
            ops.scale_(cal, 1.0)
        torch.cuda.synchronize()
        del cal

    rng = np.random.default_rng(99)
    starts = np.arange(0, T + 1, w["seq"], dtype=np.int32)
    batches = [rng.integers(0, w["vocab"], T).astype(np.int32) for _ in range(args.warmup + args.steps)]

    losses = []
    tw = time.perf_counter()
    for i in range(args.warmup):
        losses.append(t.step(batches[i], starts))
    torch.cuda.synchronize()
    warm_ms = 1000.0 * (time.perf_counter() - tw) / max(args.warmup, 1)

    # Per-kernel timing brackets every kernel-library call of the step with a HIP event pair on the step's
    # stream.  On a step of hundreds of milliseconds that costs well under 1 % and runs inside the timed
    # region.  On a step of a few milliseconds (c1) the ~1000 event records would take a third of the step,
    # so the timed region runs without them and the same batches are replayed once more with them.
    in_region = (not args.no_op_timing) and (args.warmup == 0 or warm_ms >= 100.0)
    t.enable_op_timing(in_region)
    t.reset_op_stats()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        losses.append(t.step(batches[args.warmup + i], starts))
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    timing = t.last_timing()
    roofline_from = "timed region"
    if not in_region and not args.no_op_timing:
        t.enable_op_timing(True)
        t.reset_op_stats()
        for i in range(args.steps):
            t.step(batches[args.warmup + i], starts)
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
        roofline["traffic"] = measured_traffic(dom["name"], args.workload)
        roofline["measured_over"] = roofline_from

    out = {
        "metric": "train tok/s (fwd+bwd+AdamW)", "value": round(args.steps * T / elapsed, 2), "unit": "tok/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(1000.0 * elapsed / args.steps, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": w["name"], "tokens_per_step": T, "batch": w["batch"], "seq_len": w["seq"],
                   "params": n, "device_bytes": t.device_bytes + sum(x.numel() * 4 for x in ext if x is not None),
                   "rms_eps": w["rms_eps"], "adamw_clip": w["clip"], "seed": 1234},
        "loss_first_last": [round(losses[0], 5), round(losses[-1], 5)],
        "phase_ms_last_step": {k: round(v, 3) for k, v in timing.items()},
        "roofline": roofline,
        "kernels": kernels,
    }
    t.close()
    del params, ext
    torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
