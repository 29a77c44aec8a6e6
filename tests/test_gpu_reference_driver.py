"""The reference's own step driver (train_step -> train_step_gpu_full, src/train.c:6808/:4365),
compiled unmodified from the Seraph tree and linked against this repository's vulkan_* backend
(oracle/_ref/ref_step_hip, built by `make -C oracle ref` where the tree is present), must agree
with the CPU oracle's step: same loss, same gradients, same weights after its AdamW schedule.

What this pins: the oracle's op ORDER, scaling factors, target shift, warm-up schedule and
optimizer constants against the reference's real driver code, and the backend's whole vulkan_*
surface under the call pattern the reference actually uses (command recording, buffer reuse,
fill ranges, accumulate flags).  The binary is skipped when it was not built."""
import os
import subprocess
import numpy as np
import pytest

from tests.test_gpu_step import init_params, tensor_slices, check_tensors

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "..", "oracle", "_ref", "ref_step_hip")

CASES = [
    dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101, T=48, steps=2),
    dict(hidden=128, layers=1, heads=2, kv_heads=1, head_dim=64, ffn=160, vocab=211, T=130, steps=3),
]


needs_bin = pytest.mark.skipif(not os.path.exists(BIN), reason="oracle/_ref/ref_step_hip not built (needs the Seraph tree)")


def run_driver(tmp_path, case, steps, T, lr0, theta, p, tok, rank=0, mask=0, alpha=0.0, lora=None, flags=(), stdout=None):
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        np.array([case["hidden"], case["layers"], case["heads"], case["kv_heads"], case["head_dim"], case["ffn"],
                  case["vocab"], steps, T, rank, mask], np.int32).tofile(f)
        np.array([lr0, theta, alpha], np.float32).tofile(f)
        p.tofile(f)
        if lora is not None:
            lora.tofile(f)
        tok.tofile(f)
    print(f"running {BIN} case={case} T={T} steps={steps} rank={rank} mask={mask:#b}", flush=True)
    r = subprocess.run([BIN, *flags, str(fin), str(fout)], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    if stdout is not None:
        stdout.append(r.stdout)
    return np.fromfile(fout, np.float32)


@needs_bin
@pytest.mark.parametrize("case", CASES)
def test_reference_driver_matches_oracle(orc, case, tmp_path):
    case = dict(case)
    T, steps = case.pop("T"), case.pop("steps")
    lr0, theta = 2e-3, 10000.0
    ocfg = orc.make_config(**case, rms_eps=1e-5, rope_theta=theta)
    p = init_params(orc, ocfg, 11)
    tok = np.random.default_rng(12).integers(0, case["vocab"], steps * T).astype(np.int32)
    out = run_driver(tmp_path, case, steps, T, lr0, theta, p, tok)
    n = p.size
    assert out.size == steps + 2 * n
    loss, g, w = out[:steps], out[steps:steps + n], out[steps + n:]

    # oracle: the same steps with the reference's schedule (src/train.c:5449-5466)
    rw, rm, rv = p.copy(), np.zeros_like(p), np.zeros_like(p)
    starts = np.array([0, T], np.int32)
    for s in range(steps):
        ref_loss, ref_g = orc.step_full(ocfg, rw, tok[s * T:(s + 1) * T], starts)
        assert abs(loss[s] - ref_loss) < 1e-5 * max(1.0, abs(ref_loss)), (s, loss[s], ref_loss)
        lr = orc.lr_schedule(lr0, s + 1, 1)
        rw, rm, rv = orc.adamw(rw, ref_g, rm, rv, lr, 0.9, 0.999, 0.01, 1e-8, s + 1)
    sl = tensor_slices(ocfg)
    check_tensors(g, ref_g, sl, "reference-driver grad")
    check_tensors(w, rw, sl, "reference-driver weight")


C1 = dict(hidden=512, layers=8, heads=8, kv_heads=8, head_dim=64, ffn=1408, vocab=8192)


@needs_bin
@pytest.mark.parametrize("T", [256, 2048])
def test_reference_driver_at_the_33m_shape(orc, T, tmp_path):
    """The 33M model exactly (512 wide, 8 layers, 8 heads of 64, FFN 1408, vocabulary 8192) through the reference's own
    train_step_gpu_full over the vulkan_* symbols, one sequence of 256 and of 2048 tokens, two optimizer steps: the
    op-by-op path at the sizes where it takes the banded attention backward, K runs in vulkan_matmul_transpose and
    the 512-fan-in vulkan_reduce_sum over more than one pass.  Loss per step, every gradient tensor of the last step
    and every weight tensor after it against the oracle's step + AdamW, element-wise 1e-5 + 1e-4 |ref|."""
    case, steps, lr0, theta = dict(C1), 2, 3.14e-4, 10000.0
    ocfg = orc.make_config(**case, rms_eps=1e-5, rope_theta=theta)
    r = np.random.default_rng(31)
    p = (0.02 * r.standard_normal(orc.param_count(ocfg))).astype(np.float32)
    sl = tensor_slices(ocfg)
    for name, a, b in sl:
        if name.endswith("norm"):
            p[a:b] = 1.0
    tok = r.integers(0, case["vocab"], steps * T).astype(np.int32)
    out = run_driver(tmp_path, case, steps, T, lr0, theta, p, tok)
    n = p.size
    assert out.size == steps + 2 * n
    loss, g, w = out[:steps], out[steps:steps + n], out[steps + n:]
    rw, rm, rv = p.copy(), np.zeros_like(p), np.zeros_like(p)
    starts = np.array([0, T], np.int32)
    for s in range(steps):
        ref_loss, ref_g = orc.step_full(ocfg, rw, tok[s * T:(s + 1) * T], starts)
        assert abs(loss[s] - ref_loss) < 1e-5 * max(1.0, abs(ref_loss)), (s, loss[s], ref_loss)
        rw, rm, rv = orc.adamw(rw, ref_g, rm, rv, orc.lr_schedule(lr0, s + 1, 1), 0.9, 0.999, 0.01, 1e-8, s + 1)
    check_tensors(g, ref_g, sl, "reference-driver grad")
    check_tensors(w, rw, sl, "reference-driver weight")
    rel = max(np.linalg.norm(g[a:b] - ref_g[a:b]) / (np.linalg.norm(ref_g[a:b]) + 1e-30) for _, a, b in sl)
    assert rel <= 1e-4, rel
    print(f"\n  T={T}: losses {loss.tolist()}, worst per-tensor rel-L2 of the gradients {rel:.2e}")


@needs_bin
@pytest.mark.parametrize("mask", [0b0000101, 0b0001111, 0b1111111])
def test_reference_lora_driver_matches_oracle(orc, mask, tmp_path):
    """train_step_gpu_lora (src/train.c:5846-6719) over this backend: adapters, Adam moments and loss
    after three steps against the oracle's LoRA step + AdamW.  The first moment after step 1 is
    0.1 * gradient, so the moments pin the gradients themselves; from step 2 on B != 0, which is
    where the reference's dropped adapter input-gradient term (grad_input = NULL) matters."""
    case = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101)
    T, steps, rank, alpha, lr0, theta = 57, 3, 8, 16.0, 5e-2, 10000.0
    ocfg = orc.make_config(**case, rms_eps=1e-5, rope_theta=theta, lora_rank=rank, lora_alpha=alpha, lora_mask=mask)
    p = init_params(orc, ocfg, 21)
    r = np.random.default_rng(22)
    n = orc.lora_param_count(ocfg)
    lo = (0.05 * r.standard_normal(n)).astype(np.float32)
    tok = r.integers(0, case["vocab"], steps * T).astype(np.int32)
    out = run_driver(tmp_path, case, steps, T, lr0, theta, p, tok, rank, mask, alpha, lo)
    assert out.size == steps + 3 * n
    loss, w, m, v = out[:steps], out[steps:steps + n], out[steps + n:steps + 2 * n], out[steps + 2 * n:]

    rw, rm, rv = lo.copy(), np.zeros_like(lo), np.zeros_like(lo)
    starts = np.array([0, T], np.int32)
    for s in range(steps):
        ref_loss, ref_g = orc.step_lora(ocfg, p, rw, tok[s * T:(s + 1) * T], starts)
        assert abs(loss[s] - ref_loss) < 1e-5 * max(1.0, abs(ref_loss)), (s, loss[s], ref_loss)
        rw, rm, rv = orc.adamw(rw, ref_g, rm, rv, orc.lr_schedule(lr0, s + 1, 1), 0.9, 0.999, 0.01, 1e-8, s + 1)
    for name, got, ref in (("adapter", w, rw), ("adam m", m, rm), ("adam v", v, rv)):
        bad = np.abs(got.astype(np.float64) - ref) > 1e-5 + 1e-4 * np.abs(ref)
        assert not bad.any(), f"{name}: {bad.sum()}/{bad.size} outside tolerance, max {np.abs(got - ref).max():.3e}"
    assert np.abs(w - lo).max() > 1e-5            # the adapters did move


@needs_bin
def test_profiler_report_has_the_reference_layout(orc, tmp_path):
    """vulkan_profiler_end_step prints what src/vulkan_backend.c:152-207 prints: the header, the nine categories in
    order, the per-operation table, with the ops under the reference's names (src/vulkan_backend.c:1674-3482,
    src/vulkan_backend_backward.c:164-1191), so that the substring roll-up fills the same rows: attention backward
    apart from forward, RMSNorm backward apart from forward, cross entropy, AdamW."""
    import re
    case = dict(CASES[0])
    T, steps = case.pop("T"), case.pop("steps")
    ocfg = orc.make_config(**case, rms_eps=1e-5, rope_theta=10000.0)
    p = init_params(orc, ocfg, 41)
    tok = np.random.default_rng(42).integers(0, case["vocab"], steps * T).astype(np.int32)
    text = []
    out = run_driver(tmp_path, case, steps, T, 1e-3, 10000.0, p, tok, flags=("--profile",), stdout=text)
    text = text[0]
    assert text.count("SERAPH VULKAN STEP PROFILER (step ") == steps
    m = re.search(r"SERAPH VULKAN STEP PROFILER \(step 2, seq=%d, loss=([0-9.]+)\)\n  (\d+) operations, ([0-9.]+) ms total" % T, text)
    assert m and abs(float(m.group(1)) - out[1]) < 1e-3 and int(m.group(2)) > 50
    report = text[text.rindex("SERAPH VULKAN STEP PROFILER"):]
    cats = re.findall(r"^  (matmul \(all\)|attention fwd|attention bwd|rmsnorm fwd|rmsnorm bwd|cross_entropy|adamw|copy/fill|other) +([0-9.]+) +([0-9.]+)%", report, re.M)
    assert [c[0] for c in cats] == ["matmul (all)", "attention fwd", "attention bwd", "rmsnorm fwd", "rmsnorm bwd", "cross_entropy",
                                    "adamw", "copy/fill", "other"]
    ms = {c[0]: float(c[1]) for c in cats}
    assert all(ms[k] > 0 for k in ("matmul (all)", "attention fwd", "attention bwd", "rmsnorm fwd", "rmsnorm bwd", "cross_entropy", "adamw", "copy/fill", "other"))
    assert abs(sum(ms.values()) - float(m.group(3))) < 0.05 * float(m.group(3)) + 0.01
    assert "── CATEGORY BREAKDOWN ──" in report and "── PER-OPERATION DETAIL ──" in report
    assert re.search(r"^     #  Operation +Time \(ms\) +%  Grid / Block", report, re.M)
    L, h, qd, kv, f, V = case["layers"], case["hidden"], case["heads"] * case["head_dim"], case["kv_heads"] * case["head_dim"], case["ffn"], case["vocab"]
    for needle in (f"matmul_t [{T}x{qd} K={h}]", f"matmul [{T}x{h} K={f}]", f"attn_fwd [seq={T} h={case['heads']} hd={case['head_dim']}]",
                   f"attn_bwd [seq={T} h={case['heads']} hd={case['head_dim']}]", f"rmsnorm [{T}x{h}] 256-thr", f"rmsnorm_bwd [{T}x{h}] 256-thr",
                   f"cross_entropy_grad [{T - 1}x{V}] 256-thr", f"adamw [{V * h}] 256-thr", "rope_fwd", "rope_bwd", "silu_bwd", "mul_bwd",
                   "embed_lookup", "embed_bwd", "reduce_sum"):
        assert needle in report, needle
    ops = re.findall(r"^ +(\d+)  (\S.*?) +([0-9.]+) +([0-9.]+)%", report[report.index("PER-OPERATION DETAIL"):], re.M)
    assert len(ops) == int(m.group(2)) and [int(o[0]) for o in ops] == list(range(len(ops)))
    assert sum(1 for o in ops if o[1].startswith("attn_bwd")) == L and sum(1 for o in ops if o[1].startswith("rmsnorm_bwd")) == 2 * L + 1
