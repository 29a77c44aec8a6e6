"""ctypes binding of the CPU oracle (oracle/liboracle.so) over numpy arrays.

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
CPU-baseline leg of the benchmark; never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"])
    return _SO


class Config(C.Structure):
    _fields_ = [("hidden", C.c_int32), ("layers", C.c_int32), ("heads", C.c_int32),
                ("kv_heads", C.c_int32), ("head_dim", C.c_int32), ("ffn", C.c_int32),
                ("vocab", C.c_int32), ("rms_eps", C.c_float), ("rope_theta", C.c_float),
                ("lora_rank", C.c_int32), ("lora_alpha", C.c_float), ("lora_mask", C.c_int32),
                ("use_qk_norm", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_SO)
        _lib.orc_step_full.restype = C.c_float
        _lib.orc_step_lora.restype = C.c_float
        _lib.orc_lr_schedule.restype = C.c_float
        _lib.orc_lr_schedule.argtypes = [C.c_float, C.c_int, C.c_int]
        _lib.orc_param_count.restype = C.c_int64
        _lib.orc_lora_param_count.restype = C.c_int64
        _lib.orc_nan_check.restype = C.c_int
    return _lib


def _f(a):
    assert a.dtype == np.float32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u(a):
    if a is None:
        return None
    assert a.dtype == np.uint32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


def _i(a):
    if a is None:
        return None
    assert a.dtype == np.int32 and a.flags.c_contiguous
    return a.ctypes.data_as(C.POINTER(C.c_int32))


i64 = C.c_int64
f32 = C.c_float


def cross_entropy_grad(logits, targets, valid_rows=None):
    rows, cols = logits.shape
    grad = np.empty_like(logits)
    loss = np.empty(rows, np.float32)
    lib().orc_cross_entropy_grad(_f(logits), _u(targets), _f(grad), _f(loss), i64(rows), i64(cols),
                                 i64(rows if valid_rows is None else valid_rows))
    return grad, loss


def cross_entropy_grad_packed(logits, targets, seq_starts, num_valid):
    rows, cols = logits.shape
    grad = np.empty_like(logits)
    loss = np.empty(rows, np.float32)
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    lib().orc_cross_entropy_grad_packed(_f(logits), _u(targets), _f(grad), _f(loss), _u(seq_starts),
                                        i64(rows), C.c_int(batch), i64(cols), i64(num_valid))
    return grad, loss


def reduce_sum(x):
    out = np.empty((x.size + 511) // 512, np.float32)
    lib().orc_reduce_sum(_f(x), _f(out), i64(x.size))
    return out


def matmul(A, B, M, N, K, tA=0, tB=0, C_in=None, exact=False):
    """exact: the plain double-accumulated loop nest whatever the size (orc_matmul switches to a
    cache-blocked form for large products)."""
    out = np.zeros((M, N), np.float32) if C_in is None else C_in.copy()
    (lib().orc_matmul_exact if exact else lib().orc_matmul)(_f(A), _f(B), _f(out), i64(M), i64(N), i64(K), C.c_int(tA), C.c_int(tB),
                     C.c_int(0 if C_in is None else 1))
    return out


def attention_forward(Q, K, V, H, KVH, D, seq_starts=None, scale=None):
    T = Q.shape[0]
    out = np.empty_like(Q)
    lse = np.empty((T, H), np.float32)
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    lib().orc_attention_forward(_f(Q), _f(K), _f(V), _f(out), _f(lse), _u(seq_starts), C.c_int(batch),
                                i64(T), C.c_int(H), C.c_int(KVH), C.c_int(D), f32(scale))
    return out, lse


def attention_backward(Q, K, V, dO, H, KVH, D, seq_starts=None, scale=None, dK0=None, dV0=None):
    T = Q.shape[0]
    dQ = np.empty_like(Q)
    dK = np.zeros_like(K) if dK0 is None else dK0.copy()
    dV = np.zeros_like(V) if dV0 is None else dV0.copy()
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    lib().orc_attention_backward(_f(Q), _f(K), _f(V), _f(dO), _f(dQ), _f(dK), _f(dV), _u(seq_starts),
                                 C.c_int(batch), i64(T), C.c_int(H), C.c_int(KVH), C.c_int(D), f32(scale))
    return dQ, dK, dV


def rmsnorm(x, scale, eps):
    y = np.empty_like(x)
    lib().orc_rmsnorm(_f(x), _f(scale), _f(y), i64(x.shape[0]), i64(x.shape[1]), f32(eps))
    return y


def rmsnorm_backward_batch(x, scale, dy, eps, gscale0=None):
    dx = np.empty_like(x)
    gs = np.zeros(x.shape[1], np.float32) if gscale0 is None else gscale0.copy()
    lib().orc_rmsnorm_backward_batch(_f(x), _f(scale), _f(dy), _f(dx), _f(gs), i64(x.shape[0]),
                                     i64(x.shape[1]), f32(eps))
    return dx, gs


def rope_inv_freq(D, theta):
    out = np.empty(D // 2, np.float32)
    lib().orc_rope_inv_freq(_f(out), C.c_int(D), f32(theta))
    return out


def rope(x, heads, D, theta, seq_starts=None, backward=False):
    out = np.empty_like(x)
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    lib().orc_rope(_f(x), _f(out), _u(seq_starts), C.c_int(batch), i64(x.shape[0]), C.c_int(heads),
                   C.c_int(D), f32(theta), C.c_int(1 if backward else 0))
    return out


def qk_norm(x, heads, D, eps):
    y = x.copy()
    lib().orc_qk_norm(_f(y), i64(x.shape[0]), C.c_int(heads), C.c_int(D), f32(eps))
    return y


def qk_norm_backward(x_pre, dy, heads, D, eps):
    dx = np.empty_like(x_pre)
    lib().orc_qk_norm_backward(_f(x_pre), _f(dy), _f(dx), i64(x_pre.shape[0]), C.c_int(heads), C.c_int(D), f32(eps))
    return dx


def silu(x):
    y = np.empty_like(x)
    lib().orc_silu(_f(x), _f(y), i64(x.size))
    return y


def silu_backward(x, dy):
    dx = np.empty_like(x)
    lib().orc_silu_backward(_f(x), _f(dy), _f(dx), i64(x.size))
    return dx


def mul_backward(A, B, dC):
    dA, dB = np.empty_like(A), np.empty_like(A)
    lib().orc_mul_backward(_f(A), _f(B), _f(dC), _f(dA), _f(dB), i64(A.size))
    return dA, dB


def swiglu_backward(gate, up, dH):
    dG, dU = np.empty_like(gate), np.empty_like(gate)
    lib().orc_swiglu_backward(_f(gate), _f(up), _f(dH), _f(dG), _f(dU), i64(gate.size))
    return dG, dU


def embed_lookup(tokens, embed):
    out = np.empty((tokens.size, embed.shape[1]), np.float32)
    lib().orc_embed_lookup(_u(tokens), _f(embed), _f(out), i64(tokens.size), i64(embed.shape[1]), i64(embed.shape[0]))
    return out


def embedding_backward(tokens, dH, grad_embed):
    g = grad_embed.copy()
    lib().orc_embedding_backward(_u(tokens), _f(dH), _f(g), i64(tokens.size), i64(dH.shape[1]), i64(g.shape[0]))
    return g


def adamw(w, g, m, v, lr, beta1, beta2, wd, eps, step, clip=0.0):
    w, m, v = w.copy(), m.copy(), v.copy()
    lib().orc_adamw(_f(w), _f(g), _f(m), _f(v), i64(w.size), f32(lr), f32(beta1), f32(beta2), f32(wd),
                    f32(eps), C.c_int(step), f32(clip))
    return w, m, v


def nan_check(x):
    return int(lib().orc_nan_check(_f(x), i64(x.size)))


def lr_schedule(base_lr, optimizer_step, accum_steps=1):
    return float(lib().orc_lr_schedule(base_lr, optimizer_step, accum_steps))


def make_config(hidden, layers, heads, kv_heads, head_dim, ffn, vocab, rms_eps=1e-5, rope_theta=10000.0,
                lora_rank=0, lora_alpha=0.0, lora_mask=0, use_qk_norm=0):
    return Config(hidden, layers, heads, kv_heads, head_dim, ffn, vocab, rms_eps, rope_theta,
                  lora_rank, lora_alpha, lora_mask, use_qk_norm)


def param_count(cfg):
    return int(lib().orc_param_count(C.byref(cfg)))


def lora_param_count(cfg):
    return int(lib().orc_lora_param_count(C.byref(cfg)))


def step_full(cfg, params, tokens, seq_starts=None, grads0=None):
    T = tokens.size
    grads = np.zeros_like(params) if grads0 is None else grads0.copy()
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    loss = lib().orc_step_full(C.byref(cfg), _f(params), _f(grads), _i(tokens), _i(seq_starts), C.c_int(batch), i64(T))
    return float(loss), grads


def step_lora(cfg, params, lora, tokens, seq_starts=None, grads0=None):
    T = tokens.size
    grads = np.zeros_like(lora) if grads0 is None else grads0.copy()
    batch = 1 if seq_starts is None else len(seq_starts) - 1
    loss = lib().orc_step_lora(C.byref(cfg), _f(params), _f(lora), _f(grads), _i(tokens), _i(seq_starts),
                               C.c_int(batch), i64(T))
    return float(loss), grads


def num_threads():
    return int(lib().orc_num_threads())
