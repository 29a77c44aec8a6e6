"""Host-side data formats (include/hip_train_io.h) against independent statements of the
reference's formats: .ttok files and batch packing, config.json, BF16 safetensors model
directories, full-weight checkpoints, the .state sidecar, LoRA adapter files.  No GPU.

Independent side of every check: files are written/read here with struct / the safetensors
package / libc's rand(), never with the code under test."""
import ctypes
import json
import struct

import numpy as np
import pytest
import torch

from seraph_amd import io as sio
from seraph_amd._lib import SeraphError
from seraph_amd.trainer import lora_layout, lora_param_count, model_config, param_count, param_layout
from tests.refmodel import split_lora, split_params

TTOK_MAGIC = 0x544F4B54           # src/train.c:20


def write_ttok(path, samples, vocab=1000, magic=TTOK_MAGIC):
    """tools/tokenize_dataset.c:113: header {magic, version 1, num_samples, vocab}, then per sample u32 n + n int32."""
    with open(path, "wb") as f:
        f.write(struct.pack("<4I", magic, 1, len(samples), vocab))
        for s in samples:
            f.write(struct.pack("<I", len(s)))
            f.write(np.asarray(s, np.int32).tobytes())


def ragged_samples(rng, n, lo=0, hi=40, vocab=1000):
    return [rng.integers(0, vocab, size=int(rng.integers(lo, hi + 1))).astype(np.int32) for _ in range(n)]


# ------------------------------------------------------------------ .ttok
def test_ttok_load_matches_file_layout(tmp_path):
    rng = np.random.default_rng(0)
    samples = ragged_samples(rng, 37)
    samples[5] = np.zeros(0, np.int32)           # an empty sample is legal
    samples[9] = np.array([7], np.int32)         # and a one-token one
    p = tmp_path / "a.ttok"
    write_ttok(p, samples, vocab=4321)
    tokens, offsets, vocab = sio.ttok_load(p)
    assert vocab == 4321
    assert offsets.tolist() == np.concatenate([[0], np.cumsum([len(s) for s in samples])]).tolist()
    assert np.array_equal(tokens, np.concatenate(samples))


def test_ttok_empty_file_and_negative_ids(tmp_path):
    p = tmp_path / "e.ttok"
    write_ttok(p, [])
    tokens, offsets, _ = sio.ttok_load(p)
    assert tokens.size == 0 and offsets.tolist() == [0]
    write_ttok(p, [np.array([-1, 5, -7], np.int32)])          # ids are stored as int32, sign and all
    tokens, _, _ = sio.ttok_load(p)
    assert tokens.tolist() == [-1, 5, -7]


def test_ttok_rejects_bad_magic_and_truncation(tmp_path):
    rng = np.random.default_rng(1)
    p = tmp_path / "bad.ttok"
    write_ttok(p, ragged_samples(rng, 3), magic=0x12345678)
    with pytest.raises(SeraphError):
        sio.ttok_load(p)
    write_ttok(p, ragged_samples(rng, 8, lo=5))
    data = p.read_bytes()
    p.write_bytes(data[:-6])                                   # last sample cut short
    with pytest.raises(SeraphError):
        sio.ttok_load(p)
    with pytest.raises(SeraphError):
        sio.ttok_load(tmp_path / "missing.ttok")


def test_ttok_writer_produces_the_reference_layout(tmp_path):
    rng = np.random.default_rng(2)
    samples = ragged_samples(rng, 11, lo=1)
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).astype(np.int32)
    p = tmp_path / "w.ttok"
    sio.ttok_write(p, tokens, offsets, 777)
    raw = p.read_bytes()
    assert struct.unpack_from("<4I", raw) == (TTOK_MAGIC, 1, 11, 777)
    at = 16
    for s in samples:
        (n,) = struct.unpack_from("<I", raw, at)
        at += 4
        assert n == len(s) and np.array_equal(np.frombuffer(raw, np.int32, n, at), s)
        at += 4 * n
    assert at == len(raw)


# ------------------------------------------------------------------ units and packing
def reference_units(offsets, max_seq, fixed):
    """src/train.c:7242-7275"""
    starts, lengths = [], []
    for i in range(len(offsets) - 1):
        start, n = int(offsets[i]), int(offsets[i + 1] - offsets[i])
        if fixed:
            for w in range(n // max_seq):
                starts.append(start + w * max_seq)
                lengths.append(max_seq)
        else:
            starts.append(start)
            lengths.append(min(n, max_seq))
    return starts, lengths


def reference_pack(tokens, offsets, batch, max_seq):
    """tools/seraph_train_cuda.c:363-402: the loop over sample_idx with its skip and truncation rules."""
    num_samples, out, idx = len(offsets) - 1, [], 0
    while idx < num_samples:
        count, packed, starts, src = 0, [], [0], idx
        while count < batch and src < num_samples:
            start = offsets[src]
            end = offsets[src + 1] if src + 1 < num_samples else len(tokens)
            n = min(end - start, max_seq)
            if n < 2:
                src += 1
                continue
            packed.extend(tokens[start:start + n])
            count += 1
            starts.append(len(packed))
            src += 1
        idx = src
        if count:
            out.append((packed, starts))
    return out


@pytest.mark.parametrize("batch,max_seq", [(1, 16), (4, 16), (8, 7), (3, 64)])
def test_pack_batches_match_the_reference_loop(batch, max_seq):
    rng = np.random.default_rng(batch * 100 + max_seq)
    samples = ragged_samples(rng, 61, lo=0, hi=40)
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).astype(np.int32)
    starts, lengths = sio.ttok_units(tokens, offsets, max_seq)
    assert (starts.tolist(), lengths.tolist()) == tuple(reference_units(offsets, max_seq, False))
    got = [(t.tolist(), s.tolist()) for t, s in sio.pack_batches(tokens, starts, lengths, batch, max_seq)]
    want = reference_pack(tokens.tolist(), offsets.tolist(), batch, max_seq)
    assert got == want
    assert all(s[-1] <= batch * max_seq for _, s in got)


def test_fixed_windows_drop_remainders():
    rng = np.random.default_rng(5)
    samples = ragged_samples(rng, 23, lo=0, hi=50)
    tokens = np.concatenate(samples)
    offsets = np.concatenate([[0], np.cumsum([len(s) for s in samples])]).astype(np.int32)
    starts, lengths = sio.ttok_units(tokens, offsets, 12, fixed_windows=True)
    assert (starts.tolist(), lengths.tolist()) == tuple(reference_units(offsets, 12, True))
    assert set(lengths.tolist()) <= {12}
    batches = list(sio.pack_batches(tokens, starts, lengths, 4, 12))
    assert sum(len(s) - 1 for _, s in batches) == len(starts)
    for t, s in batches:
        assert np.all(np.diff(s) == 12)


# ------------------------------------------------------------------ config.json
def test_model_config_reads_the_reference_keys(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps({
        "model_type": "qwen3", "vocab_size": 151936, "hidden_size": 2048, "num_hidden_layers": 28,
        "intermediate_size": 6144, "num_attention_heads": 16, "num_key_value_heads": 8, "head_dim": 128,
        "rms_norm_eps": 1e-6, "rope_theta": 1000000.0, "tie_word_embeddings": True, "architectures": ["Qwen3ForCausalLM"],
        "note": 'escaped " quote and \u00e9'}))
    c = sio.model_config_load(tmp_path)
    assert (c.vocab, c.hidden, c.layers, c.ffn, c.heads, c.kv_heads, c.head_dim) == (151936, 2048, 28, 6144, 16, 8, 128)
    assert c.rope_theta == 1e6 and abs(c.rms_eps - 1e-6) < 1e-12
    assert (c.lora_rank, c.lora_mask) == (0, 0)


def test_model_config_defaults_nesting_and_fallbacks(tmp_path):
    # src/model_config.c:232-279: text_config wins, head_dim derived, kv heads default to heads,
    # rope_theta from rope_parameters, then 10000
    (tmp_path / "config.json").write_text(json.dumps({
        "model_type": "wrapper", "hidden_size": 1, "text_config": {
            "hidden_size": 512, "num_attention_heads": 8, "num_hidden_layers": 4, "intermediate_size": 1024,
            "vocab_size": 4096, "rope_parameters": {"rope_theta": 500000.0}}}))
    c = sio.model_config_load(tmp_path)
    assert (c.hidden, c.heads, c.kv_heads, c.head_dim, c.layers, c.ffn, c.vocab) == (512, 8, 8, 64, 4, 1024, 4096)
    assert c.rope_theta == 500000.0 and abs(c.rms_eps - 1e-6) < 1e-12
    (tmp_path / "config.json").write_text("{}")
    c = sio.model_config_load(tmp_path)
    assert (c.vocab, c.hidden, c.layers, c.ffn, c.heads, c.kv_heads, c.head_dim) == (32000, 4096, 32, 11008, 32, 32, 128)
    assert c.rope_theta == 10000.0
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(SeraphError):
        sio.model_config_load(tmp_path)


# ------------------------------------------------------------------ model weights
NAMES = {"q": "self_attn.q_proj", "k": "self_attn.k_proj", "v": "self_attn.v_proj", "o": "self_attn.o_proj",
         "gate": "mlp.gate_proj", "up": "mlp.up_proj", "down": "mlp.down_proj",
         "in_norm": "input_layernorm", "post_norm": "post_attention_layernorm"}       # src/train.c:340-422


def small_cfg(**kw):
    base = dict(hidden=64, layers=3, heads=4, kv_heads=2, head_dim=32, ffn=96, vocab=200)
    base.update(kw)
    return model_config(**base)


def named_tensors(cfg, arena, prefix=""):
    """HF-named views of an arena laid out as tests/refmodel.split_params (the oracle's layout)."""
    P = split_params(cfg, torch.from_numpy(arena))
    out = {prefix + "model.embed_tokens.weight": P["embed"], prefix + "model.norm.weight": P["final_norm"]}
    for l, layer in enumerate(P["layers"]):
        for k, t in layer.items():
            out[f"{prefix}model.layers.{l}.{NAMES[k]}.weight"] = t
    return out


def test_param_layout_is_the_oracle_layout():
    cfg = small_cfg()
    L = param_layout(cfg)
    n = param_count(cfg)
    P = split_params(cfg, torch.arange(n, dtype=torch.float64))
    assert L.count == n and int(P["embed"][0, 0]) == L.embed and int(P["final_norm"][0]) == L.final_norm
    for l, layer in enumerate(P["layers"]):
        for k, t in layer.items():
            assert int(t.reshape(-1)[0]) == L.layer0 + l * L.layer_stride + getattr(L, k), (l, k)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_weights_load_single_file(tmp_path, dtype):
    from safetensors.torch import save_file
    cfg = small_cfg()
    rng = np.random.default_rng(3)
    arena = rng.standard_normal(param_count(cfg)).astype(np.float32)
    tensors = {k: v.to(dtype).contiguous() for k, v in named_tensors(cfg, arena).items()}
    tensors["lm_head.weight"] = torch.zeros(3, 3, dtype=dtype)          # tensors the trainer does not use are ignored
    save_file(tensors, str(tmp_path / "model.safetensors"))
    got, missing = sio.weights_load(tmp_path, cfg)
    want = torch.from_numpy(arena).to(dtype).to(torch.float32).numpy()    # exact widening of the stored values
    assert missing == 0
    assert np.array_equal(got, want)
    got2, _ = sio.weights_load(tmp_path / "model.safetensors", cfg)        # a file path works too
    assert np.array_equal(got2, want)


def test_weights_load_with_an_odd_header_length(tmp_path):
    """Header padding is free-form, so 16-bit tensor data can start at an odd file offset."""
    import struct
    from safetensors.torch import save_file
    cfg = small_cfg(layers=1)
    arena = np.random.default_rng(5).standard_normal(param_count(cfg)).astype(np.float32)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in named_tensors(cfg, arena).items()},
              str(tmp_path / "even.safetensors"))
    raw = (tmp_path / "even.safetensors").read_bytes()
    n = struct.unpack("<Q", raw[:8])[0]
    header, data = raw[8:8 + n], raw[8 + n:]
    pad = b" " if (n + 1) % 2 else b"  "
    assert (8 + n + len(pad)) % 2 == 1
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", n + len(pad)) + header + pad + data)
    got, missing = sio.weights_load(tmp_path / "model.safetensors", cfg)
    assert missing == 0
    assert np.array_equal(got, torch.from_numpy(arena).to(torch.bfloat16).to(torch.float32).numpy())


def test_weights_load_shards_prefixes_and_missing(tmp_path):
    from safetensors.torch import save_file
    cfg = small_cfg(layers=2)
    rng = np.random.default_rng(4)
    arena = rng.standard_normal(param_count(cfg)).astype(np.float32)
    named = {k: v.to(torch.bfloat16).contiguous() for k, v in named_tensors(cfg, arena, prefix="language_model.").items()}
    del named["language_model.model.layers.1.mlp.up_proj.weight"]
    keys = sorted(named)
    for i in range(3):                                                     # src/model_config.c:349-368
        save_file({k: named[k] for k in keys[i::3]}, str(tmp_path / f"model-{i + 1:05d}-of-00003.safetensors"))
    got, missing = sio.weights_load(tmp_path, cfg)
    assert missing == 1
    want = torch.from_numpy(arena).to(torch.bfloat16).to(torch.float32).numpy()
    L = param_layout(cfg)
    lo = L.layer0 + L.layer_stride + L.up
    hi = lo + cfg.ffn * cfg.hidden
    assert np.all(got[lo:hi] == 0)                                         # the reference leaves an absent tensor at zero
    want[lo:hi] = 0
    assert np.array_equal(got, want)


def test_weights_load_rejects_wrong_sizes(tmp_path):
    from safetensors.torch import save_file
    cfg = small_cfg(layers=1)
    arena = np.ones(param_count(cfg), np.float32)
    named = {k: v.to(torch.bfloat16).contiguous() for k, v in named_tensors(cfg, arena).items()}
    named["model.layers.0.mlp.down_proj.weight"] = torch.zeros(5, 5, dtype=torch.bfloat16)
    save_file(named, str(tmp_path / "model.safetensors"))
    with pytest.raises(SeraphError):
        sio.weights_load(tmp_path, cfg)
    with pytest.raises(SeraphError):
        sio.weights_load(tmp_path / "nothing_here", cfg)


def test_embedding_rows_beyond_the_file_get_the_seeded_he_init(tmp_path):
    """src/train.c:318-332: srand(42), Box-Muller over rand(), scale sqrt(2/hidden)."""
    from safetensors.torch import save_file
    cfg = small_cfg(layers=1, vocab=200)
    file_rows = 150
    rng = np.random.default_rng(6)
    arena = rng.standard_normal(param_count(cfg)).astype(np.float32)
    named = {k: v.to(torch.bfloat16).contiguous() for k, v in named_tensors(cfg, arena).items()}
    named["model.embed_tokens.weight"] = named["model.embed_tokens.weight"][:file_rows].contiguous()
    save_file(named, str(tmp_path / "model.safetensors"))
    got, _ = sio.weights_load(tmp_path, cfg)
    h = cfg.hidden
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(42)
    rand_max = np.float32(2147483647)
    scale = np.sqrt(np.float32(2.0) / np.float32(h), dtype=np.float32)
    n_new = (cfg.vocab - file_rows) * h
    u = np.array([libc.rand() for _ in range(2 * n_new)], np.float32) / rand_max
    u1, u2 = u[0::2] + np.float32(1e-7), u[1::2]
    want = np.sqrt(np.float32(-2.0) * np.log(u1)) * np.cos(np.float32(2.0) * np.float32(3.14159265) * u2) * scale
    new = got[file_rows * h:cfg.vocab * h]
    assert np.allclose(new, want.astype(np.float32), rtol=2e-6, atol=1e-7)
    assert abs(new.std() / scale - 1.0) < 0.05
    kept = torch.from_numpy(arena[:file_rows * h]).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(got[:file_rows * h], kept)


# ------------------------------------------------------------------ checkpoints
def test_checkpoint_is_a_bf16_safetensors_file_in_the_reference_order(tmp_path):
    from safetensors import safe_open
    cfg = small_cfg()
    rng = np.random.default_rng(7)
    arena = rng.standard_normal(param_count(cfg)).astype(np.float32)
    p = tmp_path / "checkpoint_10.safetensors"
    sio.checkpoint_save(p, cfg, arena)
    want = named_tensors(cfg, arena)
    trunc = lambda t: (t.contiguous().view(torch.int32) >> 16).to(torch.int16)       # src/train.c:262-266
    with safe_open(str(p), framework="pt") as f:
        assert f.metadata() == {"format": "pt", "framework": "tetyah", "trained": "full_weight_fp32_adamw"}
        assert set(f.keys()) == set(want)
        for k in want:
            t = f.get_tensor(k)
            assert t.dtype == torch.bfloat16 and tuple(t.shape) == tuple(want[k].shape), k
            assert torch.equal(t.view(torch.int16), trunc(want[k])), k
    # data section order: embed, per layer q k v o gate up down input_norm post_norm, final norm (src/train.c:470-506)
    raw = p.read_bytes()
    (hlen,) = struct.unpack_from("<Q", raw)
    header = json.loads(raw[8:8 + hlen])
    order = sorted((v["data_offsets"][0], k) for k, v in header.items() if k != "__metadata__")
    expect = ["model.embed_tokens.weight"]
    for l in range(cfg.layers):
        expect += [f"model.layers.{l}.{NAMES[k]}.weight" for k in ("q", "k", "v", "o", "gate", "up", "down", "in_norm", "post_norm")]
    expect.append("model.norm.weight")
    assert [k for _, k in order] == expect
    assert order[0][0] == 0 and all(header[a]["data_offsets"][1] == header[b]["data_offsets"][0]
                                    for a, b in zip(expect, expect[1:]))
    assert 8 + hlen + header[expect[-1]]["data_offsets"][1] == len(raw)


def test_checkpoint_reader_is_sequential_like_the_reference(tmp_path):
    cfg = small_cfg(layers=2)
    rng = np.random.default_rng(8)
    arena = rng.standard_normal(param_count(cfg)).astype(np.float32)
    p = tmp_path / "c.safetensors"
    sio.checkpoint_save(p, cfg, arena)
    back = sio.checkpoint_load(p, cfg)
    assert np.array_equal(back.view(np.uint32), arena.view(np.uint32) & np.uint32(0xFFFF0000))
    # the reference's reader skips the header and never looks inside it (src/train.c:579-580): any header works
    raw = p.read_bytes()
    (hlen,) = struct.unpack_from("<Q", raw)
    junk = b'{"x":1}'
    p.write_bytes(struct.pack("<Q", len(junk)) + junk + raw[8 + hlen:])
    assert np.array_equal(sio.checkpoint_load(p, cfg), back)
    p.write_bytes(raw[:-10])
    with pytest.raises(SeraphError):
        sio.checkpoint_load(p, cfg)
    # and the by-name loader reads a checkpoint as a model file
    p.write_bytes(raw)
    named, missing = sio.weights_load(p, cfg)
    assert missing == 0 and np.array_equal(named, back)


def test_state_sidecar_layout(tmp_path):
    p = tmp_path / "checkpoint_5.safetensors"
    sio.train_state_save(p, 2, 5000, 1.25, 1250)
    raw = (tmp_path / "checkpoint_5.safetensors.state").read_bytes()
    assert raw == struct.pack("<iifi", 2, 5000, 1.25, 1250)              # src/train.c:7796-7799
    assert sio.train_state_load(p) == dict(epoch=2, step=5000, loss=1.25, optimizer_step=1250)
    assert sio.train_state_load(tmp_path / "none") is None


# ------------------------------------------------------------------ LoRA adapters
def libc_kaiming(libc, state, n, fan_in):
    """src/lora.c:20-49 in float32 over libc's rand()."""
    out = np.empty(n, np.float32)
    rm = np.float32(2147483647)
    std = np.sqrt(np.float32(2.0) / np.float32(fan_in), dtype=np.float32)
    for i in range(n):
        if state["have"]:
            state["have"] = False
            out[i] = state["spare"] * std
            continue
        while True:
            u = np.float32(libc.rand()) / rm * np.float32(2) - np.float32(1)
            v = np.float32(libc.rand()) / rm * np.float32(2) - np.float32(1)
            s = u * u + v * v
            if np.float32(0) < s < np.float32(1):
                break
        m = np.sqrt(np.float32(-2.0) * np.log(s) / s, dtype=np.float32)
        state["spare"], state["have"] = v * m, True
        out[i] = u * m * std
    return out


@pytest.mark.parametrize("mask", [0b0000101, 0b1111111])
def test_lora_init_draws_the_reference_sequence(mask):
    cfg = small_cfg(layers=2, lora_rank=4, lora_alpha=8.0, lora_mask=mask)
    got = sio.lora_init(cfg, 1234)
    layers = split_lora(cfg, torch.from_numpy(got))
    libc = ctypes.CDLL("libc.so.6")
    libc.srand(1234)
    state = {"have": False, "spare": np.float32(0)}
    for layer in layers:
        for name in ("q", "k", "v", "o", "gate", "up", "down"):        # creation order, src/lora.c:372-396
            if name not in layer:
                continue
            A, B = layer[name]
            want = libc_kaiming(libc, state, A.numel(), A.shape[1])
            assert np.allclose(A.reshape(-1).numpy(), want, rtol=2e-6, atol=1e-7), name
            assert torch.count_nonzero(B) == 0


def test_lora_file_header_and_body_follow_the_reference(tmp_path):
    cfg = small_cfg(layers=2, lora_rank=4, lora_alpha=16.0, lora_mask=0b0000101)
    rng = np.random.default_rng(9)
    arena = rng.standard_normal(lora_param_count(cfg)).astype(np.float32)
    p = tmp_path / "checkpoint_final.bin"
    sio.lora_save(p, cfg, arena)
    raw = p.read_bytes()
    h, qd, kv, r = cfg.hidden, cfg.heads * cfg.head_dim, cfg.kv_heads * cfg.head_dim, cfg.lora_rank
    # src/lora.c:445-475
    assert struct.unpack_from("<IIiifiiiI", raw) == (0x4C4F5241, 2, 2, r, 16.0, h, qd, kv, 1 | 4)
    at = 36
    layers = split_lora(cfg, torch.from_numpy(arena))
    for layer in layers:                                                   # per layer q then v, A then B (src/lora.c:478-489)
        for name in ("q", "v"):
            for t in layer[name]:
                n = t.numel()
                assert np.array_equal(np.frombuffer(raw, np.float32, n, at), t.reshape(-1).numpy())
                at += 4 * n
    assert at == len(raw)                                                  # nothing appended for a q+v adapter set
    assert np.array_equal(sio.lora_load(p, cfg), arena)


def test_lora_file_with_all_adapters_round_trips_and_keeps_the_v2_body(tmp_path):
    cfg = small_cfg(layers=2, lora_rank=4, lora_alpha=16.0, lora_mask=0b1111111)
    rng = np.random.default_rng(10)
    arena = rng.standard_normal(lora_param_count(cfg)).astype(np.float32)
    p = tmp_path / "all.bin"
    sio.lora_save(p, cfg, arena)
    assert np.array_equal(sio.lora_load(p, cfg), arena)
    raw = p.read_bytes()
    assert struct.unpack_from("<I", raw, 32)[0] == 1 | 2 | 4 | 8 | 16
    # a q+v reader (the reference's) finds its adapters where it expects them
    qv = small_cfg(layers=2, lora_rank=4, lora_alpha=16.0, lora_mask=0b0000101)
    got = split_lora(qv, torch.from_numpy(sio.lora_load(p, qv)))
    full = split_lora(cfg, torch.from_numpy(arena))
    for a, b in zip(got, full):
        for name in ("q", "v"):
            assert torch.equal(a[name][0], b[name][0]) and torch.equal(a[name][1], b[name][1])
    other = small_cfg(layers=3, lora_rank=4, lora_alpha=16.0, lora_mask=0b0000101)
    with pytest.raises(SeraphError):
        sio.lora_load(p, other)


def test_lora_layout_is_the_oracle_layout():
    cfg = small_cfg(layers=2, lora_rank=4, lora_alpha=8.0, lora_mask=0b1010101)
    L = lora_layout(cfg)
    n = lora_param_count(cfg)
    layers = split_lora(cfg, torch.arange(n, dtype=torch.float64))
    assert L.count == n
    for l, layer in enumerate(layers):
        for p, name in enumerate(("q", "k", "v", "o", "gate", "up", "down")):
            if name in layer:
                assert int(layer[name][0].reshape(-1)[0]) == l * L.layer_stride + L.A[p]
                assert int(layer[name][1].reshape(-1)[0]) == l * L.layer_stride + L.B[p]
                assert tuple(layer[name][0].shape) == (cfg.lora_rank, L.in_dim[p])
                assert tuple(layer[name][1].shape) == (L.out_dim[p], cfg.lora_rank)
            else:
                assert L.A[p] == -1 and L.B[p] == -1
