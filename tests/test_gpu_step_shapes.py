"""Step-level parity at the benchmark configurations' shapes: the packed training step (forward + loss +
backward + AdamW on the GPU, through hip_train_step_full_batch / hip_train_step_lora_batch) against the CPU
oracle's step on identical seeded weights and batches.

  * the 33M model exactly (512 wide, 8 layers, 8 x 64 heads, FFN 1408, vocabulary 8192, 8 x 256 packed),
    with the reference's AdamW formula and with clipping;
  * a mid-size model whose vocabulary takes the in-place long-row cross entropy and whose batch takes the
    128 x 128 GEMM tiles with accumulation and the split dK/dV path;
  * the Qwen3-1.7B shape at full width and vocabulary with two layers: LoRA r16 on q/k/v/o over one
    2048-token sequence (with B = 0 and with B != 0), and full-weight training
    over 2 x 4096 packed tokens (logits beyond 4 GiB, the dS band of a 4096-token sequence);
  * the full 28-layer model through properties no oracle is needed for: bit-identical reruns, a packed
    batch equal to the weighted sum of its sequences run alone, accumulation equal to the sum.

Bar: loss to 1e-5 relative; every gradient tensor, post-AdamW weight and moment tensor element-wise within
1e-5 + 1e-4 |ref|.  Each case prints the worst rel-L2 over its tensors."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


@pytest.fixture(scope="module")
def tr():
    from seraph_amd import trainer
    return trainer


def tensor_slices(c):
    """(name, start, stop) of every tensor in the flat parameter arena."""
    h, qd, kv, f, V = c["hidden"], c["heads"] * c["head_dim"], c["kv_heads"] * c["head_dim"], c["ffn"], c["vocab"]
    out, o = [], 0
    for name, n in [("embed", V * h), ("final_norm", h)] + [
            (f"layer{l}.{nm}", n) for l in range(c["layers"]) for nm, n in
            (("in_norm", h), ("q", qd * h), ("k", kv * h), ("v", kv * h), ("o", h * qd), ("post_norm", h),
             ("gate", f * h), ("up", f * h), ("down", h * f))]:
        out.append((name, o, o + n))
        o += n
    return out


def seeded_params(c, n, seed):
    """N(0, 0.02) weights with unit norm gains, generated once (on the GPU) and shared with the oracle."""
    g = torch.Generator(device="cuda").manual_seed(seed)
    p = torch.empty(n, dtype=torch.float32, device="cuda").normal_(0.0, 0.02, generator=g)
    for name, a, b in tensor_slices(c):
        if name.endswith("norm"):
            p[a:b] = 1.0
    return p.cpu().numpy()


NORMWISE = 1e-4


def check(got, ref, slices, what, normwise=NORMWISE):
    """Per tensor: the element-wise bar, and rel-L2 <= `normwise` (the element-wise bar alone says little about
    tensors whose entries are no larger than its absolute term).  Returns the worst rel-L2 for the record."""
    worst = 0.0
    for name, a, b in slices:
        g, r = got[a:b].astype(np.float64), ref[a:b].astype(np.float64)
        assert np.isfinite(g).all(), f"{what} {name}: non-finite"
        err = np.abs(g - r)
        rel = float(np.linalg.norm(g - r) / (np.linalg.norm(r) + 1e-30))
        bad = err > ATOL + RTOL * np.abs(r)
        assert not bad.any(), (f"{what} {name}: {bad.sum()}/{bad.size} outside tolerance, max abs err {err.max():.3e}, "
                               f"rel-L2 {rel:.3e}")
        assert rel <= normwise, f"{what} {name}: rel-L2 {rel:.3e} above {normwise:.0e}"
        worst = max(worst, rel)
    return worst


def run_full_case(tr, orc, c, starts, lr, clip, seed):
    ocfg = orc.make_config(**c)
    cfg = tr.model_config(**c)
    n = tr.param_count(cfg)
    assert n == orc.param_count(ocfg)
    p = seeded_params(c, n, seed)
    T = int(starts[-1])
    tok = np.random.default_rng(seed + 1).integers(0, c["vocab"], T).astype(np.int32)
    ref_loss, ref_g = orc.step_full(ocfg, p, tok, starts)
    t = tr.Trainer(cfg, tr.optim_config(lr, clip=clip), max_tokens=T, max_batch=len(starts) - 1)
    try:
        t.upload(tr.PARAMS, p)
        loss = t.step(tok, starts, run_optimizer=True)
        assert abs(loss - ref_loss) <= 1e-5 * max(1.0, abs(ref_loss)), (loss, ref_loss)
        sl = tensor_slices(c)
        worst = {"grad": check(t.download(tr.GRADS), ref_g, sl, "grad")}
        step_lr = orc.lr_schedule(lr, 1, 1)               # warm-up: optimizer step 1 runs at lr/100 (src/train.c:5456-5461)
        assert abs(t.last_lr - step_lr) < 1e-12
        z = np.zeros_like(p)
        rw, rm, rv = orc.adamw(p, ref_g, z, z, step_lr, 0.9, 0.999, 0.01, 1e-8, 1, clip=clip)
        del z
        w = t.download(tr.PARAMS)
        worst["weight"] = check(w, rw, sl, "weight")
        # the update itself (a few 1e-6 per element at the warm-up learning rate: below the element-wise bar), normwise
        worst["update"] = check(w.astype(np.float64) - p, rw.astype(np.float64) - p, sl, "update", normwise=1e-2)
        worst["adam m"] = check(t.download(tr.ADAM_M), rm, sl, "adam m")
        worst["adam v"] = check(t.download(tr.ADAM_V), rv, sl, "adam v")
    finally:
        t.close()
    print(f"\n  loss {loss:.6f} (oracle {ref_loss:.6f}); worst rel-L2 per tensor: " +
          ", ".join(f"{k} {v:.2e}" for k, v in worst.items()))


C1 = dict(hidden=512, layers=8, heads=8, kv_heads=8, head_dim=64, ffn=1408, vocab=8192, rms_eps=1e-6, rope_theta=10000.0)


def test_33m_model_hundred_steps_identical_on_one_and_two_streams(tr):
    """The 33M model's step runs its weight gradients on a second stream, ordered by events that the producing
    kernels complete themselves.  A hundred optimizer steps with and without the second stream: every loss, the weights
    and the second moments agree to the bit (one ordering edge too few would let a product read or overwrite a buffer
    early, sooner or later), and the loss falls on the eight batches it keeps seeing."""
    cfg = tr.model_config(**C1)
    n = tr.param_count(cfg)
    p = seeded_params(C1, n, 3)
    starts = np.arange(0, 2049, 256, dtype=np.int32)
    toks = [np.random.default_rng(100 + i).integers(0, C1["vocab"], 2048).astype(np.int32) for i in range(8)]
    res = []
    for overlap in (True, False):
        t = tr.Trainer(cfg, tr.optim_config(3e-4, warmup_steps=1), max_tokens=2048, max_batch=8)
        try:
            t.enable_wgrad_overlap(overlap)
            t.upload(tr.PARAMS, p)
            losses = np.array([t.step(toks[i % 8], starts) for i in range(100)])
            res.append((losses, t.download(tr.PARAMS), t.download(tr.ADAM_V)))
        finally:
            t.close()
    for a, b in zip(res[0], res[1]):
        assert np.array_equal(a, b)
    assert np.isfinite(res[0][0]).all() and res[0][0][-1] < res[0][0][0] - 1.0


@pytest.mark.parametrize("clip", [0.0, 1.0])
def test_33m_model_step_8_x_256(tr, orc, clip):
    """The 33M configuration exactly; clip 0 is the reference's AdamW, clip 1.0 the configuration's clipped variant."""
    run_full_case(tr, orc, C1, np.arange(0, 2049, 256, dtype=np.int32), 3.14e-4, clip, seed=11)


def test_33m_model_step_with_large_gradients_clipped(tr, orc):
    """The same shape with weights large enough that gradient elements exceed the clip threshold."""
    c = dict(C1, layers=2)
    ocfg, cfg = orc.make_config(**c), tr.model_config(**c)
    n = tr.param_count(cfg)
    p = seeded_params(c, n, 12) * np.float32(4.0)
    for name, a, b in tensor_slices(c):
        if name.endswith("norm"):
            p[a:b] = 1.0
    starts = np.array([0, 100, 101, 356, 512], np.int32)
    tok = np.random.default_rng(13).integers(0, 8192, 512).astype(np.int32)
    tok[100] = tok[50]
    ref_loss, ref_g = orc.step_full(ocfg, p, tok, starts)
    clip = float(np.quantile(np.abs(ref_g[ref_g != 0]), 0.9))          # a tenth of the touched elements are clipped
    t = tr.Trainer(cfg, tr.optim_config(1e-3, clip=clip), max_tokens=512, max_batch=4)
    t.upload(tr.PARAMS, p)
    loss = t.step(tok, starts, run_optimizer=True)
    assert abs(loss - ref_loss) <= 1e-5 * max(1.0, abs(ref_loss))
    z = np.zeros_like(p)
    rw, rm, _ = orc.adamw(p, ref_g, z, z, orc.lr_schedule(1e-3, 1, 1), 0.9, 0.999, 0.01, 1e-8, 1, clip=clip)
    assert np.abs(rm).max() <= 0.1 * clip * (1 + 1e-6)                  # the clamp was active in the reference result
    sl = tensor_slices(c)
    check(t.download(tr.GRADS), ref_g, sl, "grad")
    check(t.download(tr.PARAMS), rw, sl, "weight")
    check(t.download(tr.ADAM_M), rm, sl, "adam m")
    t.close()


MID = dict(hidden=512, layers=2, heads=8, kv_heads=4, head_dim=64, ffn=1536, vocab=40960, rms_eps=1e-5, rope_theta=10000.0)


def test_mid_size_step_long_vocabulary_rows(tr, orc):
    """Vocabulary rows beyond 32768 columns (cross entropy in place over the logits, rows partly resident in LDS), 2 x 1024
    packed tokens (big GEMM tiles with accumulation, dK/dV items split between workgroups)."""
    run_full_case(tr, orc, MID, np.array([0, 1024, 2048], np.int32), 1e-3, 0.0, seed=21)


def lora_init(c, n, seed, b_zero=True):
    """A ~ N(0, 0.01), B = 0 (src/lora.c:76-78) for the adapters in the mask, layer by layer: A[r, in] then B[out, r]."""
    r = np.random.default_rng(seed)
    lo = (0.01 * r.standard_normal(n)).astype(np.float32)
    h, qd, kv, f, rk = c["hidden"], c["heads"] * c["head_dim"], c["kv_heads"] * c["head_dim"], c["ffn"], c["lora_rank"]
    o = 0
    for _ in range(c["layers"]):
        for bit, (i, oo) in enumerate(((h, qd), (h, kv), (h, kv), (qd, h), (h, f), (h, f), (f, h))):
            if not (c["lora_mask"] >> bit) & 1:
                continue
            o += rk * i
            if b_zero:
                lo[o:o + oo * rk] = 0
            o += oo * rk
    assert o == n
    return lo


def run_lora_case(tr, orc, c, starts, lr, seed, b_zero):
    ocfg, cfg = orc.make_config(**c), tr.model_config(**c)
    n, nl = tr.param_count(cfg), tr.lora_param_count(cfg)
    assert nl == orc.lora_param_count(ocfg)
    p = seeded_params(c, n, seed)
    lo = lora_init(c, nl, seed + 1, b_zero)
    T = int(starts[-1])
    tok = np.random.default_rng(seed + 2).integers(0, c["vocab"], T).astype(np.int32)
    ref_loss, ref_g = orc.step_lora(ocfg, p, lo, tok, starts)
    assert np.abs(ref_g).max() > 0
    t = tr.Trainer(cfg, tr.optim_config(lr), max_tokens=T, max_batch=len(starts) - 1)
    try:
        t.upload(tr.PARAMS, p)
        t.upload(tr.LORA_PARAMS, lo)
        loss = t.step(tok, starts, run_optimizer=True)
        assert abs(loss - ref_loss) <= 1e-5 * max(1.0, abs(ref_loss)), (loss, ref_loss)
        whole = [("lora", 0, nl)]
        rg = check(t.download(tr.LORA_GRADS), ref_g, whole, "lora grad")
        z = np.zeros_like(lo)
        rw, rm, rv = orc.adamw(lo, ref_g, z, z, orc.lr_schedule(lr, 1, 1), 0.9, 0.999, 0.01, 1e-8, 1)
        w = t.download(tr.LORA_PARAMS)
        check(w, rw, whole, "lora weight")
        ru = check(w.astype(np.float64) - lo, rw.astype(np.float64) - lo, whole, "lora update", normwise=1e-2)
        check(t.download(tr.LORA_M), rm, whole, "lora m")
        check(t.download(tr.LORA_V), rv, whole, "lora v")
        assert (t.download(tr.PARAMS) == p).all()          # base weights stay frozen
    finally:
        t.close()
    print(f"\n  B {'= 0' if b_zero else '!= 0'}: loss {loss:.6f} (oracle {ref_loss:.6f}); rel-L2 grad {rg:.2e}, update {ru:.2e}")


@pytest.mark.parametrize("b_zero", [True, False])
def test_mid_size_lora_step(tr, orc, b_zero):
    c = dict(MID, lora_rank=16, lora_alpha=32.0, lora_mask=0b1111111)
    run_lora_case(tr, orc, c, np.array([0, 1024, 2048], np.int32), 1e-3, seed=31, b_zero=b_zero)


QWEN = dict(hidden=2048, layers=2, heads=16, kv_heads=8, head_dim=128, ffn=6144, vocab=151936, rms_eps=1e-6, rope_theta=1e6)


@pytest.mark.parametrize("b_zero", [True, False])
def test_qwen3_shape_lora_step_1_x_2048_two_layers(tr, orc, b_zero):
    """The LoRA configuration at full width and vocabulary, depth 2: r16, alpha 32 on q/k/v/o over one 2048-token sequence,
    with B = 0 (the configuration's initial state: only B receives a gradient) and with B ~ N(0, 0.01) (any later step)."""
    c = dict(QWEN, lora_rank=16, lora_alpha=32.0, lora_mask=0b1111)
    run_lora_case(tr, orc, c, np.array([0, 2048], np.int32), 3.14e-4, seed=41, b_zero=b_zero)


def test_qwen3_shape_full_step_2_x_4096_two_layers(tr, orc):
    """Full-weight training at full width and vocabulary, depth 2, two packed sequences of 4096 tokens: 8192 x 151936 logits
    (4.98 GB: offsets beyond 32 bits), the 151936-row embedding scatter on top of the LM-head gradient, K runs, the dS band."""
    run_full_case(tr, orc, QWEN, np.array([0, 4096, 8192], np.int32), 3.14e-4, 0.0, seed=51)


def test_qwen3_shape_lora_step_with_qk_norm(tr, orc):
    """The LoRA configuration as it is worded ("with qk_norm"): use_qk_norm = 1 at head_dim 128 over 16 / 8 heads, B != 0
    so that both adapter matrices receive a gradient through the normalised queries and keys.  Forward after RoPE as
    src/train.c:4687-4689; the derivative (saved rms, before the RoPE backward) is this build's own, pinned by
    float64 autograd in the oracle's tests."""
    c = dict(QWEN, lora_rank=16, lora_alpha=32.0, lora_mask=0b1111, use_qk_norm=1)
    run_lora_case(tr, orc, c, np.array([0, 2048], np.int32), 3.14e-4, seed=43, b_zero=False)


def test_qwen3_shape_full_step_with_qk_norm(tr, orc):
    """Full-weight training at full width and vocabulary, depth 2, 2 x 4096 packed, use_qk_norm = 1."""
    run_full_case(tr, orc, dict(QWEN, use_qk_norm=1), np.array([0, 4096, 8192], np.int32), 3.14e-4, 0.0, seed=53)


# ------------------------------------------------------------------ the full 28-layer model, through properties
def test_qwen3_shape_full_depth_step_properties(tr):
    """28 layers, 4 x 4096 tokens, 1.72 G parameters.  (1) The step is deterministic: the same state and batch give
    bit-identical gradients.  (2) Packed sequences are independent: the gradient of the batch is the sum of the four
    sequences' own gradients weighted by their prediction counts (loss = mean over T - B predictions).  (3) Gradient
    accumulation over two micro-steps equals the sum of the two.  (4) AdamW on the arena: one embedding slice and one
    layer slice against the closed form on the host."""
    c = dict(QWEN, layers=28)
    cfg = tr.model_config(**c)
    n = tr.param_count(cfg)
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cuda").manual_seed(61)
    params = torch.empty(n, dtype=torch.float32, device=dev).normal_(0.0, 0.02, generator=g)
    for name, a, b in tensor_slices(c):
        if name.endswith("norm"):
            params[a:b] = 1.0
    p0 = params.clone()
    grads, m, v = (torch.zeros(n, dtype=torch.float32, device=dev) for _ in range(3))
    T, S = 16384, 4096
    starts = np.arange(0, T + 1, S, dtype=np.int32)
    tok = np.random.default_rng(62).integers(0, c["vocab"], T).astype(np.int32)
    lr = 3.14e-4
    t = tr.Trainer(cfg, tr.optim_config(lr, gradient_accumulation_steps=1), max_tokens=T, max_batch=4, ext=(params, grads, m, v))
    try:
        loss = t.step(tok, starts, run_optimizer=False)
        torch.cuda.synchronize()
        assert np.isfinite(loss) and abs(loss - np.log(c["vocab"])) < 1.0
        g_batch = grads.clone()
        assert torch.isfinite(g_batch).all()
        loss2 = t.step(tok, starts, run_optimizer=False)
        torch.cuda.synchronize()
        assert loss2 == loss and torch.equal(grads, g_batch), "rerun from the same state is not bit-identical"

        # (2) each sequence alone, weighted by its share of the predictions
        total = torch.zeros_like(g_batch)
        wl = 0.0
        for b in range(4):
            lb = t.step(tok[b * S:(b + 1) * S], np.array([0, S], np.int32), run_optimizer=False)
            torch.cuda.synchronize()
            total.add_(grads, alpha=(S - 1) / (T - 4))
            wl += lb * (S - 1) / (T - 4)
        assert abs(wl - loss) < 1e-5 * abs(loss), (wl, loss)
        err = (total - g_batch).abs()
        tol = ATOL + RTOL * g_batch.abs()
        assert bool((err <= tol).all()), f"packed batch vs sum of sequences: max err {float(err.max()):.3e}"
        rel = float(torch.linalg.vector_norm(total - g_batch) / torch.linalg.vector_norm(g_batch))
        del total, err, tol
        tok2 = np.random.default_rng(63).integers(0, c["vocab"], T).astype(np.int32)
        t.step(tok2, starts, run_optimizer=False)
        torch.cuda.synchronize()
        g_two = grads.clone()                              # the second batch's gradient alone
    finally:
        t.close()

    # (3) accumulation over two micro-steps; AdamW only after the second
    t = tr.Trainer(cfg, tr.optim_config(lr, gradient_accumulation_steps=2), max_tokens=T, max_batch=4, ext=(params, grads, m, v))
    try:
        t.step(tok, starts)
        torch.cuda.synchronize()
        assert t.optimizer_step == 0 and torch.equal(params, p0) and torch.equal(grads, g_batch)
        t.step(tok2, starts)                               # accumulates into the first micro-step's gradient, then AdamW
        torch.cuda.synchronize()
        assert t.optimizer_step == 1
        want = g_batch + g_two
        err = (grads - want).abs()
        assert bool((err <= ATOL + RTOL * want.abs()).all()), f"accumulated gradient: max err {float(err.max()):.3e}"
        del err
        # (4) AdamW at lr/2 (divided by the accumulation count, src/train.c:5461) in the warm-up, on two slices
        from oracle import oracle as orc
        step_lr = orc.lr_schedule(lr, 1, 2)
        assert abs(t.last_lr - step_lr) < 1e-12
        sl = dict((nm, (a, b)) for nm, a, b in tensor_slices(c))
        for nm, rows in (("embed", 4096 * c["hidden"]), ("layer27.down", None), ("layer13.in_norm", None)):
            a, b = sl[nm]
            b = a + rows if rows else b
            gw = grads[a:b].cpu().numpy()
            z = np.zeros_like(gw)
            rw, rm, rv = orc.adamw(p0[a:b].cpu().numpy(), gw, z, z, step_lr, 0.9, 0.999, 0.01, 1e-8, 1)
            for got, ref, what in ((params, rw, "weight"), (m, rm, "adam m"), (v, rv, "adam v")):
                got = got[a:b].cpu().numpy().astype(np.float64)
                assert (np.abs(got - ref) <= ATOL + RTOL * np.abs(ref)).all(), (nm, what)
    finally:
        t.close()
    print(f"\n  loss {loss:.5f}; packed batch vs weighted sum of its sequences: rel-L2 {rel:.2e}")
