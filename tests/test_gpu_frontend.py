"""The batched front end (seraph_amd/bin/seraph-train-hip) and the trainer features around the
step - evaluation, NaN flag lattice, checkpoints and exact resume - against the CPU oracle.

The front end is run as a user would run it: a model directory (config.json + BF16
safetensors), a .ttok file, the reference's options.  Its printed losses are compared with the
oracle stepping the same packed batches from the same BF16-rounded weights (printed with four
decimals: tolerance 1.5e-4), its exact-resume file with the oracle's weights and moments at
|got - ref| <= 1e-5 + 1e-4 |ref|, its BF16 checkpoint with the truncated oracle weights to one
BF16 ulp."""
import json
import os
import re
import struct
import subprocess

import numpy as np
import pytest
import torch

from tests.test_gpu_step import ATOL, RTOL, check_tensors, init_params, tensor_slices
from tests.test_io_formats import named_tensors, reference_pack, write_ttok

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "seraph_amd", "bin", "seraph-train-hip")
SHAPE = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=160)


@pytest.fixture(scope="module")
def tr():
    from seraph_amd import trainer
    return trainer


def make_model_dir(path, orc, shape, seed, std=0.05):
    from safetensors.torch import save_file
    from seraph_amd.trainer import model_config
    os.makedirs(path, exist_ok=True)
    ocfg = orc.make_config(**shape, rms_eps=1e-5, rope_theta=10000.0)
    cfg = model_config(**shape, rms_eps=1e-5, rope_theta=10000.0)
    p = init_params(orc, ocfg, seed, std)
    p = torch.from_numpy(p).to(torch.bfloat16).to(torch.float32).numpy()             # what a BF16 file can hold
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in named_tensors(cfg, p).items()},
              os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"model_type": "qwen2", "vocab_size": shape["vocab"], "hidden_size": shape["hidden"],
                   "num_hidden_layers": shape["layers"], "intermediate_size": shape["ffn"],
                   "num_attention_heads": shape["heads"], "num_key_value_heads": shape["kv_heads"],
                   "head_dim": shape["head_dim"], "rms_norm_eps": 1e-6, "rope_theta": 10000.0}, f)
    return ocfg, cfg, p


def make_samples(seed, n, vocab, lo=1, hi=30):
    r = np.random.default_rng(seed)
    return [r.integers(0, vocab, size=int(r.integers(lo, hi + 1))).astype(np.int32) for _ in range(n)]


def run_cli(args, timeout=170):
    print("seraph-train-hip", " ".join(map(str, args)), flush=True)
    p = subprocess.run([BIN] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)
    return p.returncode, p.stdout, p.stderr


def step_losses(stdout):
    return [(int(m.group(1)), float(m.group(2))) for m in re.finditer(r"Step (\d+)/\d+ \| Loss: ([0-9.]+|nan|-nan)", stdout)]


def oracle_run(orc, ocfg, p, batches, lr, accum=1):
    """Steps the oracle through packed batches with the reference's schedule; returns losses, weights, m, v."""
    m, v = np.zeros_like(p), np.zeros_like(p)
    losses, grads, opt_step, counter = [], None, 0, 0
    for tokens, starts in batches:
        loss, g = orc.step_full(ocfg, p, np.asarray(tokens, np.int32), np.asarray(starts, np.int32),
                                grads0=grads if counter else None)
        losses.append(loss)
        grads = g
        counter += 1
        if counter >= accum:
            opt_step += 1
            p, m, v = orc.adamw(p, g, m, v, orc.lr_schedule(lr, opt_step, accum), 0.9, 0.999, 0.01, 1e-8, opt_step)
            counter = 0
    return losses, p, m, v


def read_optim(path):
    from safetensors import safe_open
    with safe_open(path + ".optim", framework="np") as f:
        return f.get_tensor("params"), f.get_tensor("adam.m"), f.get_tensor("adam.v")


def test_front_end_full_training_matches_oracle(tmp_path, orc):
    assert os.path.exists(BIN), "seraph_amd/bin/seraph-train-hip is not built"
    mdir, ckpt = str(tmp_path / "model"), str(tmp_path / "ckpt")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=11)
    samples = make_samples(12, 17, SHAPE["vocab"])
    samples[4] = samples[4][:1]                                   # skipped: nothing to predict
    samples[7] = np.concatenate([samples[7]] * 3)[:50]            # truncated to --max-seq
    write_ttok(os.path.join(mdir, "train.ttok"), samples, vocab=SHAPE["vocab"])
    rc, out, err = run_cli([mdir, os.path.join(mdir, "train.ttok"), "--full-training", "--batch", 3, "--max-seq", 24,
                            "--lr", 2e-3, "--log-every", 1, "--save-every", 4, "--checkpoint", ckpt])
    assert rc == 0, err[-2000:]
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 3, 24)
    ref_losses, rp, rm, rv = oracle_run(orc, ocfg, p0.copy(), batches, 2e-3)
    got = step_losses(out)
    assert [s for s, _ in got] == list(range(1, len(batches) + 1))
    assert np.allclose([l for _, l in got], ref_losses, atol=1.5e-4), (got, ref_losses)
    assert f"batch={len(batches[0][1]) - 1}" in out

    final = os.path.join(ckpt, "checkpoint_final.safetensors")
    gp, gm, gv = read_optim(final)
    sl = tensor_slices(ocfg)
    check_tensors(gp, rp, sl, "weight")
    check_tensors(gm, rm, sl, "adam m")
    check_tensors(gv, rv, sl, "adam v")
    from seraph_amd import io as sio
    bf = sio.checkpoint_load(final, cfg)
    assert np.array_equal(bf.view(np.uint32), gp.view(np.uint32) & np.uint32(0xFFFF0000))     # truncation of what was trained
    st = sio.train_state_load(final)
    assert st["step"] == len(batches) and st["optimizer_step"] == len(batches) and st["epoch"] == 0
    assert abs(st["loss"] - ref_losses[-1]) < 1e-5 * max(1.0, ref_losses[-1])
    assert os.path.exists(os.path.join(ckpt, "checkpoint_4.safetensors.state"))
    log = open(os.path.join(ckpt, "train.log")).read()
    assert len(step_losses(log)) == len(batches)


def test_front_end_resume_continues_exactly(tmp_path, orc):
    mdir = str(tmp_path / "model")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=21)
    samples = make_samples(22, 12, SHAPE["vocab"], lo=8, hi=20)
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    common = [mdir, ttok, "--full-training", "--batch", 2, "--max-seq", 32, "--lr", 1e-3, "--log-every", 1, "--save-every", 0]
    rc, out_all, err = run_cli(common + ["--checkpoint", tmp_path / "a"])
    assert rc == 0, err[-2000:]
    rc, out_1, err = run_cli(common + ["--checkpoint", tmp_path / "b", "--max-steps", 3])
    assert rc == 0, err[-2000:]
    # second epoch from the three-step checkpoint: same schedule position, same moments
    rc, out_2, err = run_cli(common + ["--checkpoint", tmp_path / "c", "--epochs", 2, "--max-steps", 2,
                                       "--resume", tmp_path / "b" / "checkpoint_final.safetensors"])
    assert rc == 0, err[-2000:]
    assert "Loaded FP32 weights and Adam moments" in out_2 and "step 3" in out_2
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    ref_losses, rp, rm, rv = oracle_run(orc, ocfg, p0.copy(), batches[:3] + batches[:2], 1e-3)
    got = [l for _, l in step_losses(out_1)] + [l for _, l in step_losses(out_2)]
    assert np.allclose(got, ref_losses, atol=1.5e-4), (got, ref_losses)
    gp, gm, gv = read_optim(str(tmp_path / "c" / "checkpoint_final.safetensors"))
    sl = tensor_slices(ocfg)
    check_tensors(gp, rp, sl, "weight after resume")
    check_tensors(gv, rv, sl, "adam v after resume")


def test_front_end_lora_and_validation(tmp_path, orc):
    mdir = str(tmp_path / "model")
    ocfg0, cfg0, p0 = make_model_dir(mdir, orc, SHAPE, seed=31)
    samples = make_samples(32, 10, SHAPE["vocab"], lo=6, hi=24)
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    val = make_samples(33, 5, SHAPE["vocab"], lo=2, hi=24)
    vtok = os.path.join(mdir, "val.ttok")
    write_ttok(vtok, val, vocab=SHAPE["vocab"])
    ckpt = tmp_path / "l"
    rc, out, err = run_cli([mdir, ttok, "--batch", 2, "--max-seq", 32, "--lr", 1e-3, "--log-every", 1, "--lora-rank", 4,
                            "--lora-alpha", 8, "--seed", 77, "--val", vtok, "--eval-every", 2, 0, "--checkpoint", ckpt])
    assert rc == 0, err[-2000:]
    from seraph_amd import io as sio
    from seraph_amd.trainer import model_config
    shape = dict(SHAPE, lora_rank=4, lora_alpha=8.0, lora_mask=0b0000101)
    ocfg = orc.make_config(**shape, rms_eps=1e-5, rope_theta=10000.0)
    cfg = model_config(**shape, rms_eps=1e-5, rope_theta=10000.0)
    lp = sio.lora_init(cfg, 77)
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    m, v = np.zeros_like(lp), np.zeros_like(lp)
    ref_losses, val_losses = [], []
    for i, (tk, ss) in enumerate(batches, 1):
        loss, g = orc.step_lora(ocfg, p0, lp, np.asarray(tk, np.int32), np.asarray(ss, np.int32))
        ref_losses.append(loss)
        lp, m, v = orc.adamw(lp, g, m, v, orc.lr_schedule(1e-3, i, 1), 0.9, 0.999, 0.01, 1e-8, i)
        if i % 2 == 0:                                            # src/train_cuda.c:2812-2847: mean of per-sample losses
            per = [orc.step_lora(ocfg, p0, lp, s[:32], np.array([0, min(len(s), 32)], np.int32))[0] for s in val if len(s) >= 2]
            val_losses.append(float(np.mean(per)))
    got = [l for _, l in step_losses(out)]
    assert np.allclose(got, ref_losses, atol=1.5e-4), (got, ref_losses)
    got_val = [float(x) for x in re.findall(r"\[VAL\] Step \d+ \| Val Loss: ([0-9.]+)", out)]
    assert np.allclose(got_val, val_losses, atol=1.5e-4), (got_val, val_losses)
    saved = sio.lora_load(str(ckpt / "checkpoint_final.bin"), cfg)
    bad = np.abs(saved - lp) > ATOL + RTOL * np.abs(lp)
    assert not bad.any()
    raw = open(ckpt / "checkpoint_final.bin", "rb").read()
    assert struct.unpack_from("<IIiif", raw) == (0x4C4F5241, 2, SHAPE["layers"], 4, 8.0)


def test_eval_forward_changes_nothing_and_matches_the_step_loss(tr, orc):
    shape = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101)
    ocfg = orc.make_config(**shape)
    cfg = tr.model_config(**shape)
    p = init_params(orc, ocfg, 41)
    starts = np.array([0, 30, 31, 64], np.int32)
    tok = np.random.default_rng(42).integers(0, 101, 64).astype(np.int32)
    ref_loss, _ = orc.step_full(ocfg, p, tok, starts)
    t = tr.Trainer(cfg, tr.optim_config(1e-3, gradient_accumulation_steps=2), max_tokens=64, max_batch=3)
    t.upload(tr.PARAMS, p)
    t.step(tok, starts)                                           # first micro-step: gradients pending
    g_before = t.download(tr.GRADS)
    loss = t.eval_forward(tok, starts)
    assert abs(loss - ref_loss) < 1e-5 * max(1.0, abs(ref_loss))
    assert t.accumulation_counter == 1 and t.optimizer_step == 0
    assert np.array_equal(t.download(tr.GRADS), g_before) and np.array_equal(t.download(tr.PARAMS), p)
    # evaluate(): per-sample mean and perplexity, truncation and the <2 token skip
    offsets = np.array([0, 30, 31, 64], np.int32)
    per = [orc.step_full(ocfg, p, tok[a:min(b, a + 20)], np.array([0, min(b - a, 20)], np.int32))[0]
           for a, b in zip(offsets[:-1], offsets[1:]) if b - a >= 2]
    vl, ppl = t.evaluate(tok, offsets, max_seq_len=20)
    assert abs(vl - np.mean(per)) < 1e-5 * max(1.0, abs(vl)) and abs(ppl - np.exp(vl)) < 1e-3 * ppl
    t.close()


def test_nan_lattice_flags_the_first_poisoned_buffers_and_protects_the_weights(tr, orc):
    shape = dict(hidden=64, layers=3, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101)
    ocfg = orc.make_config(**shape)
    cfg = tr.model_config(**shape)
    p = init_params(orc, ocfg, 51)
    tok = np.random.default_rng(52).integers(0, 101, 48).astype(np.int32)
    starts = np.array([0, 20, 48], np.int32)
    L = tr.param_layout(cfg)
    NL = shape["layers"]
    fwd, bwd, gh, opt = 10, 10 + NL, 10 + 6 * NL, 10 + 7 * NL              # src/train.c:4525-4537

    t = tr.Trainer(cfg, tr.optim_config(1e-3), max_tokens=48, max_batch=2)
    t.enable_nan_check()
    t.upload(tr.PARAMS, p)
    loss = t.step(tok, starts)                                   # clean step: no flag, optimizer runs
    assert np.isfinite(loss) and not t.nan_detected and t.optimizer_step == 1
    flags = t.nan_flags()
    assert flags.size == 10 + 7 * NL + 5 and not flags.any()

    # poison the down projection of layer 1: hidden is clean after layer 0, not after layer 1
    before = t.download(tr.PARAMS)
    bad = before.copy()
    bad[L.layer0 + 1 * L.layer_stride + L.down + 5] = np.nan
    t.upload(tr.PARAMS, bad)
    loss = t.step(tok, starts)
    assert np.isnan(loss) and t.nan_detected
    flags = t.nan_flags()
    assert flags[7] == 0 and flags[fwd + 0] == 0 and flags[fwd + 1] == 1 and flags[fwd + 2] == 1
    assert flags[1] == 1 and flags[2] == 1 and flags[6] == 1 and flags[3] == 1 and flags[4] == 1
    assert flags[opt + 0] == 0                                   # the embedding itself was clean
    assert all(flags[bwd + 5 * l + 0] == 1 for l in range(NL)) and flags[gh + 0] == 1 and flags[8] == 1
    assert t.optimizer_step == 2                                 # counted (src/train.c:5452), but AdamW did not run:
    after = t.download(tr.PARAMS)
    assert np.array_equal(np.isnan(after), np.isnan(bad)) and np.array_equal(after[~np.isnan(bad)], bad[~np.isnan(bad)])
    m = t.download(tr.ADAM_M)
    assert np.isfinite(m).all()

    # an Inf in the embedding is caught by the very first check
    t.upload(tr.PARAMS, before)
    worse = before.copy()
    worse[L.embed + 3] = np.inf
    t.upload(tr.PARAMS, worse)
    t.step(tok, starts)
    assert t.nan_flags()[opt + 0] == 1 and t.nan_detected
    t.close()


# ------------------------------------------------------------------ the reference's own batched trainer
# oracle/_ref/seraph-train-cuda-hip is Seraph's tools/seraph_train_cuda.c + src/train_cuda.c + src/train.c,
# compiled unmodified where they lie and linked against seraph_amd/seraph_tree/hip_cuda_backend.c
# (`make -C oracle ref`, needs the Seraph tree; the binary travels to the GPU box prebuilt).
REF_BIN = os.path.join(ROOT, "oracle", "_ref", "seraph-train-cuda-hip")
needs_ref = pytest.mark.skipif(not os.path.exists(REF_BIN), reason="oracle/_ref/seraph-train-cuda-hip is not built (no Seraph tree)")


def add_tokenizer(mdir, vocab):
    """The reference's train_init insists on a tokenizer (src/train.c:7866-7881); a toy one satisfies it."""
    with open(os.path.join(mdir, "vocab.json"), "w") as f:
        json.dump({f"t{i}": i for i in range(vocab)}, f)
    with open(os.path.join(mdir, "merges.txt"), "w") as f:
        f.write("t 0\n")


# The same front end with seraph_amd/seraph_tree/hip_fused_step.c behind its step functions (the reference's
# src/train_cuda.c still compiled in, unmodified, as the op-by-op fallback).
FUSED_BIN = os.path.join(ROOT, "oracle", "_ref", "seraph-train-cuda-hip-fused")
BINARIES = [pytest.param(REF_BIN, id="op-by-op"),
            pytest.param(FUSED_BIN, id="fused", marks=pytest.mark.skipif(not os.path.exists(FUSED_BIN), reason="fused front end not built"))]


def run_ref(args, timeout=170, binary=REF_BIN, env=None):
    print(os.path.basename(binary), " ".join(map(str, args)), flush=True)
    p = subprocess.run([binary] + [str(a) for a in args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout,
                       env=dict(os.environ, **env) if env else None)
    return p.returncode, p.stdout, p.stderr


@needs_ref
@pytest.mark.parametrize("binary", BINARIES)
@pytest.mark.parametrize("flash", [False, True])
def test_reference_batched_trainer_runs_unmodified_and_matches_oracle(tmp_path, orc, flash, binary):
    mdir, ckpt = str(tmp_path / "model"), str(tmp_path / "ckpt")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=61)
    add_tokenizer(mdir, SHAPE["vocab"])
    samples = make_samples(62, 14, SHAPE["vocab"], lo=1, hi=30)
    samples[2] = samples[2][:1]
    samples[5] = np.concatenate([samples[5]] * 3)[:40]
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    args = [mdir, ttok, "--full-training", "--batch", 3, "--max-seq", 24, "--lr", 2e-3, "--log-every", 1,
            "--save-every", 0, "--checkpoint", ckpt] + (["--flash"] if flash else [])
    rc, out, err = run_ref(args, binary=binary)
    assert rc == 0, (out[-1500:], err[-1500:])
    assert ("[HIP] fused training step" in err) == (binary == FUSED_BIN)
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 3, 24)
    ref_losses, rp, _, _ = oracle_run(orc, ocfg, p0.copy(), batches, 2e-3)
    got = [l for _, l in step_losses(out)]
    assert len(got) == len(batches)
    assert np.allclose(got, ref_losses, atol=1.5e-4), (got, ref_losses)
    # the checkpoint the reference's writer produced, read by this repo's reader: BF16 truncation of the
    # trained weights, so one BF16 ulp (2^-7 relative) of the oracle's
    from seraph_amd import io as sio
    saved = sio.checkpoint_load(os.path.join(ckpt, "checkpoint_final.safetensors"), cfg)
    assert np.all(np.abs(saved - rp) <= 2.0 ** -7 * np.abs(rp) + 1e-6)
    # and this repo's front end on the same inputs prints the same losses
    rc, mine, err = run_cli(args[:-1] if flash else args)
    assert rc == 0, err[-1500:]
    assert np.allclose([l for _, l in step_losses(mine)], got, atol=1.1e-4)


C1_SHAPE = dict(hidden=512, layers=8, heads=8, kv_heads=8, head_dim=64, ffn=1408, vocab=8192)


@needs_ref
@pytest.mark.parametrize("binary", BINARIES)
def test_reference_batched_trainer_at_the_33m_shape_8_x_256(tmp_path, orc, binary):
    """The 33M model exactly, eight packed sequences of 256 tokens per step, three optimizer steps through the
    reference's own cuda_train_step_gpu_full_batch (src/train_cuda.c:1966-2326) over the cuda_train_* symbols:
    the printed losses step by step and the final checkpoint against the oracle's step + AdamW."""
    mdir, ckpt = str(tmp_path / "model"), str(tmp_path / "ckpt")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, C1_SHAPE, seed=81, std=0.02)
    add_tokenizer(mdir, C1_SHAPE["vocab"])
    r = np.random.default_rng(82)
    samples = [r.integers(0, C1_SHAPE["vocab"], 256).astype(np.int32) for _ in range(24)]
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=C1_SHAPE["vocab"])
    args = [mdir, ttok, "--full-training", "--batch", 8, "--max-seq", 256, "--lr", 3.14e-4, "--log-every", 1,
            "--save-every", 0, "--checkpoint", ckpt]
    rc, out, err = run_ref(args, binary=binary)
    assert rc == 0, (out[-1500:], err[-1500:])
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 8, 256)
    assert len(batches) == 3 and all(len(b[1]) == 9 and b[1][-1] == 2048 for b in batches)
    ref_losses, rp, _, _ = oracle_run(orc, ocfg, p0.copy(), batches, 3.14e-4)
    got = [l for _, l in step_losses(out)]
    assert len(got) == 3
    assert np.allclose(got, ref_losses, atol=1.5e-4), (got, ref_losses)
    from seraph_amd import io as sio
    saved = sio.checkpoint_load(os.path.join(ckpt, "checkpoint_final.safetensors"), cfg)
    assert np.all(np.abs(saved - rp) <= 2.0 ** -7 * np.abs(rp) + 1e-6)
    assert np.abs(rp - p0).max() > 1e-6                              # the weights moved, so the bound above says something
    # this repository's own front end (the fused step) on the same files
    rc, mine, err = run_cli(args)
    assert rc == 0, err[-1500:]
    assert np.allclose([l for _, l in step_losses(mine)], ref_losses, atol=1.5e-4)
    gp, gm, gv = read_optim(os.path.join(ckpt, "checkpoint_final.safetensors"))
    sl = tensor_slices(ocfg)
    check_tensors(gp, rp, sl, "weight (33M shape, fused front end)")


@needs_ref
@pytest.mark.parametrize("binary", BINARIES)
def test_reference_batched_trainer_profile_and_lora(tmp_path, orc, binary):
    mdir = str(tmp_path / "model")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=71)
    add_tokenizer(mdir, SHAPE["vocab"])
    samples = make_samples(72, 8, SHAPE["vocab"], lo=6, hi=24)
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    ckpt = tmp_path / "p"
    rc, out, err = run_ref([mdir, ttok, "--full-training", "--batch", 2, "--max-seq", 32, "--profile", 2, "--checkpoint", ckpt], binary=binary)
    assert rc == 0, (out[-1500:], err[-1500:])
    plog = open(ckpt / "profile.log").read()
    # the op-by-op step reports every op; the fused step one entry per kernel class, under names that land in the same categories
    ops = ("matmul_Bt [", "attn_bwd_packed", "adamw ") if binary == REF_BIN else ("matmul gemm_f32_mfma", "attn_bwd attention_backward x2", "adamw x1")
    for needle in ("SERAPH STEP PROFILER", "CATEGORY BREAKDOWN", "matmul (all)", "attention bwd", "PER-OPERATION DETAIL",
                   "PERFORMANCE METRICS", "TOP 20 SLOWEST OPERATIONS") + ops:
        assert needle in plog, needle
    cats = dict(re.findall(r"^  (matmul \(all\)|attention fwd|attention bwd|rmsnorm fwd|rmsnorm bwd|cross_entropy|adamw) +([0-9.]+) ", plog, re.M))
    assert len(cats) == 7 and all(float(v) > 0 for v in cats.values()), cats
    assert "PROFILE STEP 2 (batch=2" in out
    # LoRA through the reference's trainer: adapters start with B = 0, so the first loss is the base model's
    # (the adapter seed is the wall clock there, src/tools: srand(time(NULL)); later steps are not comparable)
    rc, out, err = run_ref([mdir, ttok, "--batch", 2, "--max-seq", 32, "--lr", 1e-3, "--log-every", 1, "--lora-rank", 4,
                            "--checkpoint", tmp_path / "q"], binary=binary)
    assert rc == 0, (out[-1500:], err[-1500:])
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    base_loss, _ = orc.step_full(ocfg, p0, np.asarray(batches[0][0], np.int32), np.asarray(batches[0][1], np.int32))
    got = [l for _, l in step_losses(out)]
    assert len(got) == len(batches) and abs(got[0] - base_loss) < 1.5e-4
    assert all(np.isfinite(got))
    assert os.path.exists(tmp_path / "q" / "checkpoint_final.bin")
    # The reference's batched LoRA backward gives every adapter the final hidden gradient as its output gradient
    # (src/train_cuda.c:2596-2644).  For the query adapter of this shape (q_dim 128, hidden 64) that product would read
    # past the end of the buffer: the backend refuses it with a message and leaves the adapter alone; the value adapter
    # (kv_dim 64) fits and runs.
    assert "lora_gB [128x4" in err and "skipped: operand 0" in err, err[-1500:]
    assert "lora_gB [64x4" not in err


def poison_first_query_projection(mdir):
    from safetensors.torch import load_file, save_file
    f = os.path.join(mdir, "model.safetensors")
    tensors = load_file(f)
    name = [k for k in tensors if "layers.0." in k and "q_proj" in k][0]
    tensors[name][0, 3] = float("nan")
    save_file(tensors, f)


@needs_ref
@pytest.mark.parametrize("binary", BINARIES)
def test_reference_front_end_with_debug_nan_check(tmp_path, orc, binary):
    """--debug-nan-check through the reference's front end.  Its single-sequence step checks its buffers
    (src/train_cuda.c:633-661, :1080-1187), its packed step does not; the fused step checks in both.  A clean model trains
    to the same losses with the checks on; a model with a NaN in its first query projection is stopped by the fused
    step at step 1 (report, dump files, the front end's [FATAL] lines, tools/seraph_train_cuda.c:472-476), with packed
    batches too."""
    import glob
    mdir = str(tmp_path / "model")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=85)
    add_tokenizer(mdir, SHAPE["vocab"])
    samples = make_samples(86, 7, SHAPE["vocab"], lo=6, hi=24)      # the seventh is a batch of its own: the single-sequence step
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    args = [mdir, ttok, "--full-training", "--batch", 2, "--max-seq", 32, "--lr", 2e-3, "--log-every", 1, "--save-every", 0,
            "--debug-nan-check"]
    rc, out, err = run_ref(args + ["--checkpoint", tmp_path / "clean"], binary=binary)
    assert rc == 0, (out[-1500:], err[-1500:])
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    ref_losses, _, _, _ = oracle_run(orc, ocfg, p0.copy(), batches, 2e-3)
    assert np.allclose([l for _, l in step_losses(out)], ref_losses, atol=1.5e-4)
    assert "[NAN]" not in err
    if binary != FUSED_BIN:
        return                                                   # the reference's packed step has no checks to trip
    poison_first_query_projection(mdir)
    before = set(glob.glob("/tmp/seraph_nan_step_1_*"))
    rc, out, err = run_ref(args + ["--checkpoint", tmp_path / "poisoned"], binary=binary)
    try:
        assert "[NAN] detected at step=1" in err and "(optimizer skipped)" in err, err[-1500:]
        assert "  - buffer: " in err and "[FATAL] NaN detected at step 1 - stopping training" in err
        dumps = set(glob.glob("/tmp/seraph_nan_step_1_*")) - before
        assert any(d.endswith("_meta.txt") for d in dumps), dumps
        assert not step_losses(out)
    finally:
        for dump in set(glob.glob("/tmp/seraph_nan_step_1_*")) - before:
            os.remove(dump)


def test_front_end_stops_on_a_nan_and_says_where(tmp_path, orc):
    """--debug-nan-check through the stand-alone front end, as tools/seraph_train_cuda.c:457-476 behaves: a model whose
    first query projection holds a NaN stops at step 1 with exit status 2, the optimizer is skipped, the report names the
    first poisoned buffers and no checkpoint of poisoned weights is left behind."""
    import glob
    mdir, ckpt = str(tmp_path / "model"), str(tmp_path / "ckpt")
    make_model_dir(mdir, orc, SHAPE, seed=81)
    poison_first_query_projection(mdir)
    write_ttok(os.path.join(mdir, "train.ttok"), make_samples(82, 6, SHAPE["vocab"], lo=5), vocab=SHAPE["vocab"])
    before = set(glob.glob("/tmp/seraph_nan_step_1_*"))
    rc, out, err = run_cli([mdir, os.path.join(mdir, "train.ttok"), "--full-training", "--batch", 2, "--max-seq", 24, "--log-every", 1,
                            "--debug-nan-check", "--checkpoint", ckpt])
    try:
        assert rc == 2, (out[-800:], err[-1500:])
        assert "[NAN] detected at step=1" in err and "(optimizer skipped)" in err
        assert "  - buffer: " in err and "[FATAL] NaN detected at step 1 - stopping training" in err
        assert not step_losses(out)                               # the step is not logged as a training step
        assert not os.path.exists(os.path.join(ckpt, "checkpoint_final.safetensors"))
    finally:
        for dump in set(glob.glob("/tmp/seraph_nan_step_1_*")) - before:
            os.remove(dump)


def test_nan_detection_writes_the_dump_files_the_reference_inspector_reads(tr, orc, tmp_path):
    """A step that detects a NaN writes the step's buffers as the reference does (src/train.c:5562-5653).  The files are
    read back with a restatement of what tools/nan_dump_inspect.c does with them (sizes from the token file and the model
    dimensions, NaN / Inf counts per file) and, where the reference tree was present at build time, by that tool itself."""
    import json
    import subprocess
    shape = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101)
    ocfg, cfg = orc.make_config(**shape), tr.model_config(**shape)
    p = init_params(orc, ocfg, 61)
    T = 40
    tok = np.random.default_rng(62).integers(0, 101, T).astype(np.int32)
    L = tr.param_layout(cfg)
    p[L.layer0 + 0 * L.layer_stride + L.q + 7] = np.nan              # layer 0's query projection: q is the first poisoned buffer
    t = tr.Trainer(cfg, tr.optim_config(1e-3), max_tokens=T, max_batch=1)
    t.enable_nan_check()
    t.set_nan_dump_prefix(str(tmp_path / "seraph_nan_step"))
    t.upload(tr.PARAMS, p)
    t.step(tok, None)                                                # step 1: detected at once
    assert t.nan_detected
    t.close()
    prefix = str(tmp_path / "seraph_nan_step_1")
    meta = dict(line.split("=") for line in open(prefix + "_meta.txt").read().split())
    assert meta["step"] == "1" and meta["seq"] == str(T) and meta["num_predictions"] == str(T - 1)
    assert meta["hidden_size"] == "64" and meta["q_dim"] == "128" and meta["kv_dim"] == "64" and meta["vocab_size"] == "101"
    toks = np.fromfile(prefix + "_tokens.u32", np.uint32)
    assert (toks == tok.astype(np.uint32)).all()
    assert (np.fromfile(prefix + "_targets.u32", np.uint32) == tok[1:].astype(np.uint32)).all()
    seq, npred, h, f, V, qd, kv = T, T - 1, 64, 96, 101, 128, 64
    items = [("hidden", seq * h, 1), ("hidden_norm", seq * h, 1), ("logits", seq * V, 1), ("grad_logits", npred * V, 1),
             ("grad_hidden", seq * h, 1), ("grad_tmp_hidden", seq * h, 0), ("grad_x_norm", seq * h, 0), ("grad_ffn", seq * f, 0),
             ("grad_gate", seq * f, 0), ("grad_up", seq * f, 0), ("L0_layer_in", seq * h, 0), ("L0_x_norm_attn", seq * h, 0),
             ("L0_post_attn_in", seq * h, 0), ("L0_x_norm_ffn", seq * h, 0), ("L0_ffn_gate", seq * f, 0), ("L0_ffn_up", seq * f, 0),
             ("L0_silu", seq * f, 0), ("L0_ffn_hidden", seq * f, 0), ("L0_q", seq * qd, 0), ("L0_k", seq * kv, 0), ("L0_v", seq * kv, 0),
             ("L0_attn_out", seq * qd, 0), ("grad_attn", seq * qd, 0), ("grad_q", seq * qd, 0), ("grad_k", seq * kv, 0), ("grad_v", seq * kv, 0)]
    nan_in = {}
    for name, count, _ in items:                                     # tools/nan_dump_inspect.c:189-246
        data = np.fromfile(f"{prefix}_{name}.f32", np.float32)
        assert data.size == count, (name, data.size, count)
        nan_in[name] = int(np.isnan(data).sum())
    assert nan_in["L0_layer_in"] == 0 and nan_in["L0_x_norm_attn"] == 0 and nan_in["L0_k"] == 0 and nan_in["L0_v"] == 0
    assert nan_in["L0_q"] == 2 * T                                   # one poisoned output feature per token, spread over its RoPE pair
    assert nan_in["logits"] > 0 and nan_in["hidden"] > 0
    inspector = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "_ref", "nan_dump_inspect")
    if os.path.exists(inspector):
        (tmp_path / "model").mkdir()
        json.dump(dict(vocab_size=101, hidden_size=64, num_hidden_layers=2, intermediate_size=96, num_attention_heads=4,
                       num_key_value_heads=2, head_dim=32, rms_norm_eps=1e-6, rope_theta=10000.0, model_type="llama"),
                  open(tmp_path / "model" / "config.json", "w"))
        out = subprocess.run([inspector, "--model-dir", str(tmp_path / "model"), "--prefix", prefix], capture_output=True, text=True)
        assert out.returncode == 0, out.stderr
        assert "MISSING" not in out.stderr and "WARN" not in out.stderr and "BAD SIZE" not in out.stderr, out.stderr
        line = next(l for l in out.stdout.splitlines() if l.startswith("L0_q "))
        assert f"n={seq * qd}" in line and f"nan={nan_in['L0_q']}" in line
        assert f"seq={T} hidden=64 inter=96 vocab=101 q_dim=128 kv_dim=64" in out.stdout


def test_bench_line_contract():
    """bench.py prints one JSON line with the agreed keys (33M workload, two steps)."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--workload", "c1", "--steps", "2", "--warmup", "1",
                        "--no-cpu-baseline"], capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
              "vs_baseline", "dtype", "data", "config", "roofline"):
        assert k in d, k
    assert d["n_gpus"] == 1 and d["steps"] == 2 and d["warmup"] == 1 and d["dtype"] == "f32" and d["vs_baseline"] is None
    assert d["value"] > 0 and abs(d["value"] - d["config"]["tokens_per_step"] / d["ms_per_step"] * 1e3) < 1e-3 * d["value"]
    rf = d["roofline"]
    assert rf["bound"] in ("hbm", "mfma") and abs(rf["frac"] - rf["achieved"] / rf["peak"]) < 1e-3


@pytest.mark.skipif(not os.path.exists(FUSED_BIN), reason="fused front end not built")
def test_fused_front_end_validation_accumulation_and_the_switch_back(tmp_path, orc):
    """The reference's front end over the fused step: validation losses (cuda_evaluate), gradient accumulation over two
    micro-steps (the state's counters travel through the fused step), and SERAPH_HIP_FUSED_STEP=0, which makes the same
    binary run the reference's op-by-op step: all three print the oracle's numbers."""
    mdir = str(tmp_path / "model")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=91)
    add_tokenizer(mdir, SHAPE["vocab"])
    samples = make_samples(92, 12, SHAPE["vocab"], lo=6, hi=24)
    val = make_samples(93, 5, SHAPE["vocab"], lo=2, hi=24)
    ttok, vtok = os.path.join(mdir, "train.ttok"), os.path.join(mdir, "val.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    write_ttok(vtok, val, vocab=SHAPE["vocab"])
    args = [mdir, ttok, "--full-training", "--batch", 2, "--max-seq", 32, "--lr", 2e-3, "--log-every", 1, "--save-every", 0,
            "--accum", 2, "--val", vtok, "--eval-every", 2, 0]
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    ref_losses, rp, _, _ = oracle_run(orc, ocfg, p0.copy(), batches, 2e-3, accum=2)
    outs = {}
    for name, env in (("fused", None), ("switched back", {"SERAPH_HIP_FUSED_STEP": "0"})):
        rc, out, err = run_ref(args + ["--checkpoint", tmp_path / name.replace(" ", "_")], binary=FUSED_BIN, env=env)
        assert rc == 0, (out[-1500:], err[-1500:])
        assert ("[HIP] fused training step" in err) == (env is None)
        got = [l for _, l in step_losses(out)]
        assert len(got) == len(batches) and np.allclose(got, ref_losses, atol=1.5e-4), (name, got, ref_losses)
        outs[name] = [float(x) for x in re.findall(r"Val Loss: ([0-9.]+)", out)]
        assert len(outs[name]) >= 1
    assert np.allclose(outs["fused"], outs["switched back"], atol=1.5e-4), outs
    from seraph_amd import io as sio
    saved = sio.checkpoint_load(str(tmp_path / "fused" / "checkpoint_final.safetensors"), cfg)
    assert np.all(np.abs(saved - rp) <= 2.0 ** -7 * np.abs(rp) + 1e-6)


@pytest.mark.skipif(not os.path.exists(FUSED_BIN), reason="fused front end not built")
def test_fused_front_end_grows_with_the_batches_and_takes_single_sequences(tmp_path, orc):
    """Two more ways into the fused step from the reference's front end.  (1) SERAPH_HIP_FUSED_TOKENS=1: the fused trainer
    starts with room for the first batch only; the samples get longer, so later batches make a larger trainer and the four
    arenas (weights, the gradients of an open accumulation window, both Adam moments) travel to it.  (2) A batch that
    holds a single sequence - the thirteenth sample is left over - goes through cuda_train_step_gpu_full
    (tools/seraph_train_cuda.c:431-435).  The losses and the final weights are the oracle's."""
    mdir = str(tmp_path / "model")
    ocfg, cfg, p0 = make_model_dir(mdir, orc, SHAPE, seed=95)
    add_tokenizer(mdir, SHAPE["vocab"])
    r = np.random.default_rng(96)
    samples = [r.integers(0, SHAPE["vocab"], n).astype(np.int32) for n in (5, 6, 8, 9, 12, 13, 17, 18, 24, 25, 31, 32, 20)]
    ttok = os.path.join(mdir, "train.ttok")
    write_ttok(ttok, samples, vocab=SHAPE["vocab"])
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    batches = reference_pack(tokens.tolist(), offsets, 2, 32)
    assert len(batches) == 7 and len(batches[-1][1]) == 2            # the last batch: one sequence
    args = [mdir, ttok, "--full-training", "--batch", 2, "--max-seq", 32, "--lr", 2e-3, "--log-every", 1, "--save-every", 0,
            "--accum", 2, "--checkpoint", tmp_path / "ckpt"]
    rc, out, err = run_ref(args, binary=FUSED_BIN, env={"SERAPH_HIP_FUSED_TOKENS": "1"})
    assert rc == 0, (out[-1500:], err[-1500:])
    assert "[HIP] fused training step" in err and err.count("room grown to") >= 3, err[-1500:]
    ref_losses, rp, _, _ = oracle_run(orc, ocfg, p0.copy(), batches, 2e-3, accum=2)
    got = [l for _, l in step_losses(out)]
    assert len(got) == len(batches) and np.allclose(got, ref_losses, atol=1.5e-4), (got, ref_losses)
    from seraph_amd import io as sio
    saved = sio.checkpoint_load(str(tmp_path / "ckpt" / "checkpoint_final.safetensors"), cfg)
    assert np.all(np.abs(saved - rp) <= 2.0 ** -7 * np.abs(rp) + 1e-6)
    assert np.abs(rp - p0).max() > 1e-6
