"""Independent float64 torch.autograd statement of the training step, used only
to pin the CPU oracle.  It follows the mathematics the reference's step
computes (src/train.c:4365-5470 full, :5847-6719 LoRA, packed structure of
src/train_cuda.c:1966-2326): interleaved-pair RoPE, RMSNorm with the step's
eps, tied LM head, block-diagonal causal attention with GQA, CE averaged over
T-B predictions.  torch is a tool here, not the reference."""
import numpy as np
import torch


def split_params(cfg, flat):
    """Views into the flat parameter vector in the oracle's layout."""
    h, L = cfg.hidden, cfg.layers
    qd, kv, f, V = cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim, cfg.ffn, cfg.vocab
    o = 0

    def take(*shape):
        nonlocal o
        n = int(np.prod(shape))
        t = flat[o:o + n].view(*shape)
        o += n
        return t

    P = {"embed": take(V, h), "final_norm": take(h), "layers": []}
    for _ in range(L):
        P["layers"].append({
            "in_norm": take(h), "q": take(qd, h), "k": take(kv, h), "v": take(kv, h), "o": take(h, qd),
            "post_norm": take(h), "gate": take(f, h), "up": take(f, h), "down": take(h, f)})
    assert o == flat.numel()
    return P


def split_lora(cfg, flat):
    h = cfg.hidden
    qd, kv, r = cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim, cfg.lora_rank
    f = cfg.ffn
    ins, outs = [h, h, h, qd, h, h, f], [qd, kv, kv, h, f, f, h]
    o = 0
    layers = []
    for _ in range(cfg.layers):
        d = {}
        for p, name in enumerate(("q", "k", "v", "o", "gate", "up", "down")):
            if (cfg.lora_mask >> p) & 1:
                A = flat[o:o + r * ins[p]].view(r, ins[p]); o += r * ins[p]
                B = flat[o:o + outs[p] * r].view(outs[p], r); o += outs[p] * r
                d[name] = (A, B)
        layers.append(d)
    assert o == flat.numel()
    return layers


def rmsnorm(x, g, eps):
    return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * g


def rope(x, pos, heads, D, theta):
    T = x.shape[0]
    i = np.arange(D // 2)
    inv_freq = (np.float32(1.0) / np.power(np.float32(theta), (2 * i).astype(np.float32) / np.float32(D),
                                           dtype=np.float32)).astype(np.float32)
    ang = (pos.astype(np.float32)[:, None] * inv_freq[None, :]).astype(np.float32).astype(np.float64)
    c = torch.from_numpy(np.cos(ang))[:, None, :]
    s = torch.from_numpy(np.sin(ang))[:, None, :]
    xv = x.view(T, heads, D // 2, 2)
    x0, x1 = xv[..., 0], xv[..., 1]
    return torch.stack([x0 * c - x1 * s, x0 * s + x1 * c], -1).reshape(T, heads * D)


def qk_norm(x, eps):
    """shaders/qk_norm.comp:38-75: every token's vector over all heads divided by max(its root mean square, eps)."""
    rms = torch.sqrt((x * x).mean(-1, keepdim=True))
    return x / torch.clamp(rms, min=float(eps))


def attention(q, k, v, seq_id, H, KVH, D):
    T = q.shape[0]
    q = q.view(T, H, D).transpose(0, 1)
    k = k.view(T, KVH, D).transpose(0, 1)
    v = v.view(T, KVH, D).transpose(0, 1)
    idx = torch.arange(H) * KVH // H
    k, v = k[idx], v[idx]
    s = (q @ k.transpose(1, 2)) / np.sqrt(np.float32(D)).astype(np.float64)
    t = torch.arange(T)
    sid = torch.from_numpy(seq_id)
    mask = (t[None, :] <= t[:, None]) & (sid[None, :] == sid[:, None])
    s = s.masked_fill(~mask, float("-inf"))
    p = torch.softmax(s, -1)
    return (p @ v).transpose(0, 1).reshape(T, H * D)


def loss_fn(cfg, P, tokens, seq_starts, lora=None, drop_adapter_dgrad=True):
    T = len(tokens)
    starts = np.asarray(seq_starts if seq_starts is not None else [0, T])
    seq_id = np.searchsorted(starts, np.arange(T), side="right") - 1
    pos = np.arange(T) - starts[seq_id]
    tok = np.maximum(tokens, 0)
    H, KVH, D = cfg.heads, cfg.kv_heads, cfg.head_dim
    s = cfg.lora_alpha / cfg.lora_rank if cfg.lora_rank else 0.0

    def proj(x, W, ad):
        y = x @ W.T
        if ad is not None:
            xi = x.detach() if drop_adapter_dgrad else x
            y = y + ((xi @ ad[0].T) * s) @ ad[1].T
        return y

    x = P["embed"][torch.from_numpy(tok).long()]
    for l, W in enumerate(P["layers"]):
        ad = lora[l] if lora is not None else {}
        xn = rmsnorm(x, W["in_norm"], cfg.rms_eps)
        q = rope(proj(xn, W["q"], ad.get("q")), pos, H, D, cfg.rope_theta)
        k = rope(proj(xn, W["k"], ad.get("k")), pos, KVH, D, cfg.rope_theta)
        v = proj(xn, W["v"], ad.get("v"))
        if getattr(cfg, "use_qk_norm", 0):                   # after RoPE, before the attention (src/train.c:4687-4689)
            q, k = qk_norm(q, cfg.rms_eps), qk_norm(k, cfg.rms_eps)
        a = attention(q, k, v, seq_id, H, KVH, D)
        x = x + proj(a, W["o"], ad.get("o"))
        xn = rmsnorm(x, W["post_norm"], cfg.rms_eps)
        g, u = proj(xn, W["gate"], ad.get("gate")), proj(xn, W["up"], ad.get("up"))
        x = x + proj(torch.nn.functional.silu(g) * u, W["down"], ad.get("down"))
    logits = rmsnorm(x, P["final_norm"], cfg.rms_eps) @ P["embed"].T
    valid = np.ones(T, bool)
    valid[starts[1:] - 1] = False
    tgt = np.zeros(T, np.int64)
    tgt[:-1] = tok[1:]
    lp = torch.log_softmax(logits, -1)
    nll = -lp[torch.arange(T), torch.from_numpy(tgt)]
    return (nll * torch.from_numpy(valid)).sum() / valid.sum()
