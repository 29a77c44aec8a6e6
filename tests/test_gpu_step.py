"""End-to-end parity of the packed training steps (forward + loss + backward + AdamW on the
GPU) against the CPU oracle's step on identical seeded weights and batches.  Gradients and
post-AdamW weights: |got - ref| <= 1e-5 + 1e-4 |ref| per tensor; loss to 1e-5."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def rng(seed):
    return np.random.default_rng(seed)


@pytest.fixture(scope="module")
def tr():
    from seraph_amd import trainer
    return trainer


def init_params(orc, ocfg, seed, std=0.05):
    r = rng(seed)
    p = (std * r.standard_normal(orc.param_count(ocfg))).astype(np.float32)
    h, L = ocfg.hidden, ocfg.layers
    qd, kv, f, V = ocfg.heads * ocfg.head_dim, ocfg.kv_heads * ocfg.head_dim, ocfg.ffn, ocfg.vocab
    o = V * h
    p[o:o + h] = 1.0
    stride = h + qd * h + 2 * kv * h + h * qd + h + 2 * f * h + h * f
    for l in range(L):
        base = V * h + h + l * stride
        p[base:base + h] = 1.0
        pn = base + h + qd * h + 2 * kv * h + h * qd
        p[pn:pn + h] = 1.0
    return p


def tensor_slices(ocfg):
    """(name, start, stop) of every tensor in the flat arena."""
    h, L = ocfg.hidden, ocfg.layers
    qd, kv, f, V = ocfg.heads * ocfg.head_dim, ocfg.kv_heads * ocfg.head_dim, ocfg.ffn, ocfg.vocab
    out, o = [], 0

    def take(name, n):
        nonlocal o
        out.append((name, o, o + n))
        o += n

    take("embed", V * h); take("final_norm", h)
    for l in range(L):
        for name, n in (("in_norm", h), ("q", qd * h), ("k", kv * h), ("v", kv * h), ("o", h * qd), ("post_norm", h),
                        ("gate", f * h), ("up", f * h), ("down", h * f)):
            take(f"layer{l}.{name}", n)
    return out


def check_tensors(got, ref, slices, what):
    for name, a, b in slices:
        g, r = got[a:b].astype(np.float64), ref[a:b].astype(np.float64)
        assert np.isfinite(g).all(), f"{what} {name}: non-finite"
        bad = np.abs(g - r) > ATOL + RTOL * np.abs(r)
        assert not bad.any(), (f"{what} {name}: {bad.sum()}/{bad.size} outside tolerance, max abs err "
                               f"{np.abs(g - r).max():.3e}, rel-L2 {np.linalg.norm(g - r) / (np.linalg.norm(r) + 1e-30):.3e}")


CASES = [
    dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101, starts=[0, 33, 34, 70]),
    dict(hidden=128, layers=1, heads=2, kv_heads=2, head_dim=64, ffn=256, vocab=300, starts=[0, 150]),
    dict(hidden=256, layers=2, heads=2, kv_heads=1, head_dim=128, ffn=128, vocab=64, starts=[0, 40, 100, 129]),
    # 512 tokens: the weight gradients are small outputs with a long K and run as sums over runs of K
    dict(hidden=128, layers=1, heads=2, kv_heads=2, head_dim=64, ffn=256, vocab=300, starts=[0, 200, 512]),
]


@pytest.mark.parametrize("case", CASES)
def test_full_step_gradients_and_adamw(tr, orc, case):
    case = dict(case)
    starts = np.array(case.pop("starts"), np.int32)
    ocfg = orc.make_config(**case, rms_eps=1e-5, rope_theta=10000.0)
    cfg = tr.model_config(**case, rms_eps=1e-5, rope_theta=10000.0)
    assert tr.param_count(cfg) == orc.param_count(ocfg)
    p = init_params(orc, ocfg, 1)
    T = int(starts[-1])
    tok = rng(2).integers(0, case["vocab"], T).astype(np.int32)
    tok[3] = tok[T - 2] = tok[5]                       # repeated ids exercise the scatter-add
    tok[7] = -4                                        # negative id -> 0 (src/train.c:4473)
    ref_loss, ref_g = orc.step_full(ocfg, p, tok, starts)

    t = tr.Trainer(cfg, tr.optim_config(3.14e-4), max_tokens=T, max_batch=len(starts) - 1)
    t.upload(tr.PARAMS, p)
    loss = t.step(tok, starts, run_optimizer=False)
    assert abs(loss - ref_loss) < 1e-5 * max(1.0, abs(ref_loss))
    sl = tensor_slices(ocfg)
    check_tensors(t.download(tr.GRADS), ref_g, sl, "grad")
    assert (t.download(tr.PARAMS) == p).all()          # run_optimizer=False leaves weights alone

    # second call: gradients are re-zeroed (accumulation count 1), then AdamW runs
    loss2 = t.step(tok, starts, run_optimizer=True)
    assert abs(loss2 - ref_loss) < 1e-5 * max(1.0, abs(ref_loss))
    assert t.optimizer_step == 1
    lr = orc.lr_schedule(3.14e-4, 1, 1)                # warm-up: step 1 runs at lr/100 (src/train.c:5456-5461)
    assert abs(t.last_lr - lr) < 1e-12
    z = np.zeros_like(p)
    rw, rm, rv = orc.adamw(p, ref_g, z, z, lr, 0.9, 0.999, 0.01, 1e-8, 1)
    check_tensors(t.download(tr.PARAMS), rw, sl, "weight")
    check_tensors(t.download(tr.ADAM_M), rm, sl, "adam m")
    t.close()


def test_full_step_gradient_accumulation(tr, orc):
    case = dict(CASES[0])
    starts = np.array(case.pop("starts"), np.int32)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    p = init_params(orc, ocfg, 3)
    T = int(starts[-1])
    tokA = rng(4).integers(0, case["vocab"], T).astype(np.int32)
    tokB = rng(5).integers(0, case["vocab"], T).astype(np.int32)
    _, gA = orc.step_full(ocfg, p, tokA, starts)
    _, gAB = orc.step_full(ocfg, p, tokB, starts, grads0=gA)
    t = tr.Trainer(cfg, tr.optim_config(1e-3, gradient_accumulation_steps=2), max_tokens=T, max_batch=3)
    t.upload(tr.PARAMS, p)
    t.step(tokA, starts)
    assert t.optimizer_step == 0                       # no update until the second micro-step
    t.step(tokB, starts)
    assert t.optimizer_step == 1
    check_tensors(t.download(tr.GRADS), gAB, tensor_slices(ocfg), "accumulated grad")
    lr = orc.lr_schedule(1e-3, 1, 2)                   # lr divided by the accumulation count (src/train.c:5461)
    z = np.zeros_like(p)
    rw, _, _ = orc.adamw(p, gAB, z, z, lr, 0.9, 0.999, 0.01, 1e-8, 1)
    check_tensors(t.download(tr.PARAMS), rw, tensor_slices(ocfg), "weight")
    t.close()


def test_twelve_optimizer_steps_follow_the_oracle(tr, orc):
    """A short training run: every step a new batch, the warm-up schedule moving, Adam's moments and bias corrections
    carried from step to step, clipping on.  Per-step loss, then weights and both moments at the end, against the
    oracle's step and AdamW applied in the same order."""
    case = dict(CASES[0])
    starts = np.array(case.pop("starts"), np.int32)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    p = init_params(orc, ocfg, 11)
    T, base_lr, clip = int(starts[-1]), 1e-2, 1.0
    t = tr.Trainer(cfg, tr.optim_config(base_lr, clip=clip), max_tokens=T, max_batch=len(starts) - 1)
    t.upload(tr.PARAMS, p)
    w, m, v = p.copy(), np.zeros_like(p), np.zeros_like(p)
    worst_loss = 0.0
    for step in range(1, 13):
        tok = rng(100 + step).integers(0, case["vocab"], T).astype(np.int32)
        ref_loss, g = orc.step_full(ocfg, w, tok, starts)
        lr = orc.lr_schedule(base_lr, step, 1)
        w, m, v = orc.adamw(w, g, m, v, lr, 0.9, 0.999, 0.01, 1e-8, step, clip)
        loss = t.step(tok, starts)
        assert t.optimizer_step == step and abs(t.last_lr - lr) < 1e-12
        worst_loss = max(worst_loss, abs(loss - ref_loss) / max(1.0, abs(ref_loss)))
    sl = tensor_slices(ocfg)
    check_tensors(t.download(tr.PARAMS), w, sl, "weight after 12 steps")
    check_tensors(t.download(tr.ADAM_M), m, sl, "adam m after 12 steps")
    got_v, ref_v = t.download(tr.ADAM_V), v
    check_tensors(got_v, ref_v, sl, "adam v after 12 steps")
    rel_v = max(np.linalg.norm(got_v[a:b] - ref_v[a:b]) / (np.linalg.norm(ref_v[a:b]) + 1e-30) for _, a, b in sl)
    print(f"\n  [margin] twelve steps: worst loss difference {worst_loss:.2e} (bar 1e-5), adam v worst rel-L2 {rel_v:.2e} (bar 1e-4)")
    assert worst_loss <= 1e-5 and rel_v <= 1e-4
    assert np.abs(w - p).max() > 1e-3                    # the run did move the weights
    t.close()


def test_weight_gradients_on_the_second_stream_change_no_bit(tr, orc):
    """Three optimizer steps with the weight gradients beside the input-gradient chain (default) and with everything on
    one stream: every product is one kernel either way, so weights, gradients and moments must be identical; a missing
    wait between the streams would show as a difference (and the step above already pins the default against the oracle)."""
    case = dict(hidden=256, layers=4, heads=4, kv_heads=2, head_dim=64, ffn=704, vocab=4096)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    p = init_params(orc, ocfg, 31)
    starts = np.array([0, 256, 300, 1024], np.int32)
    toks = [rng(40 + i).integers(0, case["vocab"], 1024).astype(np.int32) for i in range(3)]
    out = []
    for overlap in (True, False):
        t = tr.Trainer(cfg, tr.optim_config(1e-3, warmup_steps=1), max_tokens=1024, max_batch=3)
        t.enable_wgrad_overlap(overlap)
        t.upload(tr.PARAMS, p)
        losses = [t.step(tok, starts) for tok in toks]
        out.append((losses, t.download(tr.PARAMS), t.download(tr.GRADS), t.download(tr.ADAM_V)))
        t.close()
    assert out[0][0] == out[1][0]
    for a, b in zip(out[0][1:], out[1][1:]):
        assert np.array_equal(a, b)
    assert np.abs(out[0][1] - p).max() > 0


def test_adapter_gradients_on_the_second_stream_change_no_bit(tr, orc):
    """The LoRA step sends the rank-sized products of every adapter's gradients to the second stream (default); with
    everything on one stream the same kernels run in another order of launches: adapters, their gradients and moments
    must be identical over three optimizer steps, with all seven adapter kinds present."""
    case = dict(hidden=256, layers=3, heads=4, kv_heads=2, head_dim=64, ffn=704, vocab=4096, lora_rank=16,
                lora_alpha=32.0, lora_mask=0b1111111)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    p = init_params(orc, ocfg, 33)
    lo = (0.05 * rng(34).standard_normal(orc.lora_param_count(ocfg))).astype(np.float32)
    starts = np.array([0, 256, 300, 1024], np.int32)
    toks = [rng(50 + i).integers(0, case["vocab"], 1024).astype(np.int32) for i in range(3)]
    out = []
    for overlap in (True, False):
        t = tr.Trainer(cfg, tr.optim_config(1e-3, warmup_steps=1), max_tokens=1024, max_batch=3)
        t.enable_wgrad_overlap(overlap)
        t.upload(tr.PARAMS, p)
        t.upload(tr.LORA_PARAMS, lo)
        losses = [t.step(tok, starts) for tok in toks]
        out.append((losses, t.download(tr.LORA_PARAMS), t.download(tr.LORA_GRADS), t.download(tr.LORA_V)))
        t.close()
    assert out[0][0] == out[1][0]
    for a, b in zip(out[0][1:], out[1][1:]):
        assert np.array_equal(a, b)
    assert np.abs(out[0][1] - lo).max() > 0


@pytest.mark.parametrize("mask", [0b0001111, 0b1111111, 0b1010101])
@pytest.mark.parametrize("b_zero", [True, False])
def test_lora_step(tr, orc, b_zero, mask):
    case = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101, lora_rank=16,
                lora_alpha=32.0, lora_mask=mask)
    starts = np.array([0, 41, 90], np.int32)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    assert tr.lora_param_count(cfg) == orc.lora_param_count(ocfg)
    p = init_params(orc, ocfg, 6)
    r = rng(7)
    lo = (0.05 * r.standard_normal(orc.lora_param_count(ocfg))).astype(np.float32)
    if b_zero:                                         # the reference's initial state: B = 0 (src/lora.c:76-78)
        h, qd, kv, f, rk = 64, 128, 64, 96, 16
        o = 0
        for _ in range(2):
            for bit, (i, oo) in enumerate(((h, qd), (h, kv), (h, kv), (qd, h), (h, f), (h, f), (f, h))):
                if not (mask >> bit) & 1:
                    continue
                o += rk * i
                lo[o:o + oo * rk] = 0
                o += oo * rk
    tok = r.integers(0, 101, 90).astype(np.int32)
    ref_loss, ref_g = orc.step_lora(ocfg, p, lo, tok, starts)
    t = tr.Trainer(cfg, tr.optim_config(1e-3), max_tokens=90, max_batch=2)
    t.upload(tr.PARAMS, p)
    t.upload(tr.LORA_PARAMS, lo)
    loss = t.step(tok, starts, run_optimizer=True)
    assert abs(loss - ref_loss) < 1e-5 * max(1.0, abs(ref_loss))
    g = t.download(tr.LORA_GRADS).astype(np.float64)
    bad = np.abs(g - ref_g) > ATOL + RTOL * np.abs(ref_g)
    assert not bad.any(), f"{bad.sum()} lora grads outside tolerance, max {np.abs(g - ref_g).max():.3e}"
    z = np.zeros_like(lo)
    rw, _, _ = orc.adamw(lo, ref_g, z, z, orc.lr_schedule(1e-3, 1), 0.9, 0.999, 0.01, 1e-8, 1)
    w = t.download(tr.LORA_PARAMS).astype(np.float64)
    assert (np.abs(w - rw) <= ATOL + RTOL * np.abs(rw)).all()
    assert (t.download(tr.PARAMS) == p).all()          # base weights frozen
    t.close()


def test_eight_lora_steps_from_the_initial_state_follow_the_oracle(tr, orc):
    """From B = 0 (the adapters' initial state, src/lora.c:76-78): the first step moves only B, the later ones both
    factors, with the forward's kept x A^T feeding every backward.  Per-step loss, then the adapters and Adam's first
    moment after eight steps, against the oracle."""
    mask = 0b1111111
    case = dict(hidden=64, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=101, lora_rank=16,
                lora_alpha=32.0, lora_mask=mask)
    starts = np.array([0, 41, 90], np.int32)
    ocfg = orc.make_config(**case)
    cfg = tr.model_config(**case)
    p = init_params(orc, ocfg, 6)
    lo = (0.05 * rng(8).standard_normal(orc.lora_param_count(ocfg))).astype(np.float32)
    h, qd, kv, f, rk = 64, 128, 64, 96, 16
    o = 0
    for _ in range(2):
        for i, oo in ((h, qd), (h, kv), (h, kv), (qd, h), (h, f), (h, f), (f, h)):
            o += rk * i
            lo[o:o + oo * rk] = 0
            o += oo * rk
    base_lr = 2e-2
    t = tr.Trainer(cfg, tr.optim_config(base_lr), max_tokens=90, max_batch=2)
    t.upload(tr.PARAMS, p)
    t.upload(tr.LORA_PARAMS, lo)
    w, m, v = lo.copy(), np.zeros_like(lo), np.zeros_like(lo)
    worst_loss = 0.0
    for step in range(1, 9):
        tok = rng(200 + step).integers(0, 101, 90).astype(np.int32)
        ref_loss, g = orc.step_lora(ocfg, p, w, tok, starts)
        w, m, v = orc.adamw(w, g.astype(np.float32), m, v, orc.lr_schedule(base_lr, step), 0.9, 0.999, 0.01, 1e-8, step)
        loss = t.step(tok, starts)
        worst_loss = max(worst_loss, abs(loss - ref_loss) / max(1.0, abs(ref_loss)))
    print(f"\n  [margin] eight LoRA steps: worst loss difference {worst_loss:.2e} (bar 1e-5)")
    assert worst_loss <= 1e-5
    got = t.download(tr.LORA_PARAMS).astype(np.float64)
    assert (np.abs(got - w) <= ATOL + RTOL * np.abs(w)).all(), np.abs(got - w).max()
    gm = t.download(tr.LORA_M).astype(np.float64)
    assert (np.abs(gm - m) <= ATOL + RTOL * np.abs(m)).all(), np.abs(gm - m).max()
    assert np.abs(w - lo).max() > 1e-3 and (t.download(tr.PARAMS) == p).all()
    t.close()


@pytest.mark.parametrize("lora", [False, True])
def test_step_with_qk_norm(tr, orc, lora):
    """use_qk_norm = 1 in both step drivers: forward after RoPE, derivative before the RoPE backward (the reference's
    backward has no such term: parity unpinned by the reference; the oracle's is pinned by float64 autograd)."""
    case = dict(hidden=128, layers=2, heads=4, kv_heads=2, head_dim=32, ffn=192, vocab=211, rms_eps=1e-5, use_qk_norm=1)
    if lora:
        case.update(lora_rank=8, lora_alpha=16.0, lora_mask=0b1111)
    ocfg, cfg = orc.make_config(**case), tr.model_config(**case)
    p = init_params(orc, ocfg, 21)
    starts = np.array([0, 70, 71, 200], np.int32)
    tok = rng(22).integers(0, 211, 200).astype(np.int32)
    t = tr.Trainer(cfg, tr.optim_config(1e-3), max_tokens=200, max_batch=3)
    t.upload(tr.PARAMS, p)
    if lora:
        lo = (0.05 * rng(23).standard_normal(orc.lora_param_count(ocfg))).astype(np.float32)
        t.upload(tr.LORA_PARAMS, lo)
        ref_loss, ref_g = orc.step_lora(ocfg, p, lo, tok, starts)
    else:
        ref_loss, ref_g = orc.step_full(ocfg, p, tok, starts)
    loss = t.step(tok, starts, run_optimizer=False)
    assert abs(loss - ref_loss) < 1e-5 * max(1.0, abs(ref_loss))
    g = t.download(tr.LORA_GRADS if lora else tr.GRADS).astype(np.float64)
    bad = np.abs(g - ref_g) > ATOL + RTOL * np.abs(ref_g)
    assert not bad.any(), f"{bad.sum()} gradients outside tolerance, max {np.abs(g - ref_g).max():.3e}"
    assert np.linalg.norm(g - ref_g) <= 1e-4 * np.linalg.norm(ref_g)
    # the same model without the switch gives another gradient: the option is live
    off = dict(case, use_qk_norm=0)
    g_off = (orc.step_lora(orc.make_config(**off), p, lo, tok, starts) if lora else orc.step_full(orc.make_config(**off), p, tok, starts))[1]
    assert np.linalg.norm(g_off - ref_g) > 1e-2 * np.linalg.norm(ref_g)
    t.close()


def test_step_rejects_bad_batches(tr):
    from seraph_amd._lib import SeraphError
    cfg = tr.model_config(64, 1, 2, 2, 32, 64, 50)
    t = tr.Trainer(cfg, tr.optim_config(1e-3), max_tokens=32, max_batch=2)
    with pytest.raises(SeraphError):
        t.step(np.zeros(64, np.int32), np.array([0, 64], np.int32))          # more tokens than capacity
    with pytest.raises(SeraphError):
        t.step(np.zeros(16, np.int32), np.array([0, 8, 8, 16], np.int32))    # empty sequence / too many sequences
    t.close()
