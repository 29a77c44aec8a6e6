"""Thin Python mirror of the C-ABI kernel library over torch CUDA tensors.

torch supplies device memory and the stream only; every computation goes through
libseraph_hip.so.  Names and argument meaning follow the backend ops of the reference
(include/vulkan_backend.h:431-603), with the packed-batch arguments of
include/cuda_train_context.h:273-288 where they apply.
"""
import ctypes as C

import torch

from ._lib import check, kernels

i64, f32, sz = C.c_int64, C.c_float, C.c_size_t


def _p(t):
    if t is None:
        return None
    assert t.is_cuda and t.is_contiguous(), "expected a contiguous CUDA tensor"
    return C.c_void_p(t.data_ptr())


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


_ws = {}


def _workspace(nbytes):
    dev = torch.cuda.current_device()
    t = _ws.get(dev)
    if t is None or t.numel() < nbytes:
        t = torch.empty(max(int(nbytes), 1 << 20), dtype=torch.uint8, device="cuda")
        _ws[dev] = t
    return t


def init(device=0):
    check(kernels().seraph_hip_init(C.c_int(device)), "seraph_hip_init")


def _batch(seq_starts):
    return 1 if seq_starts is None else seq_starts.numel() - 1


def fill_u32(t, value):
    check(kernels().seraph_fill_u32(_p(t), C.c_uint32(value), sz(t.numel()), _stream()), "fill_u32")


def add(a, b, out):
    check(kernels().seraph_add(_p(a), _p(b), _p(out), sz(a.numel()), _stream()), "add")
    return out


def mul(a, b, out):
    check(kernels().seraph_mul(_p(a), _p(b), _p(out), sz(a.numel()), _stream()), "mul")
    return out


def scale_(a, alpha):
    check(kernels().seraph_scale(_p(a), sz(a.numel()), f32(alpha), _stream()), "scale")
    return a


def nan_check(x, flags, flag_index):
    check(kernels().seraph_nan_check(_p(x), sz(x.numel()), _p(flags), C.c_uint32(flag_index), _stream()), "nan_check")


def reduce_sum(x):
    out = torch.empty((x.numel() + 511) // 512, dtype=torch.float32, device=x.device)
    check(kernels().seraph_reduce_sum(_p(x), _p(out), sz(x.numel()), _stream()), "reduce_sum")
    return out


def cross_entropy_grad(logits, targets, valid_rows, seq_starts=None, grad=None):
    rows, cols = logits.shape
    grad = torch.empty_like(logits) if grad is None else grad
    loss = torch.empty(rows, dtype=torch.float32, device=logits.device)
    check(kernels().seraph_cross_entropy_grad(_p(logits), _p(targets), _p(grad), _p(loss), _p(seq_starts),
                                              C.c_int(_batch(seq_starts)), i64(rows), i64(cols), i64(valid_rows),
                                              _stream()), "cross_entropy_grad")
    return grad, loss


def gemm(A, B, M, N, K, tA=0, tB=0, out=None, accumulate=False):
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    check(kernels().seraph_gemm(_p(A), _p(B), _p(out), i64(M), i64(N), i64(K), C.c_int(tA), C.c_int(tB),
                                C.c_int(1 if accumulate else 0), _stream()), "gemm")
    return out


class GemmProblem(C.Structure):
    _fields_ = [("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p), ("M", C.c_int64), ("N", C.c_int64)]


def gemm_grouped(problems, K, tA=0, tB=0, accumulate=False):
    """problems: list of (A, B, out, M, N) sharing K, the orientations and the accumulate flag; one launch."""
    arr = (GemmProblem * len(problems))(*[GemmProblem(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n) for a, b, c, m, n in problems])
    check(kernels().seraph_gemm_grouped(arr, C.c_int(len(problems)), i64(K), C.c_int(tA), C.c_int(tB),
                                        C.c_int(1 if accumulate else 0), _stream()), "gemm_grouped")
    return [c for _, _, c, _, _ in problems]


class GemmTerm(C.Structure):
    _fields_ = [("A", C.c_void_p), ("B", C.c_void_p), ("K", C.c_int64)]


def gemm_chain(terms, M, N, tA=0, tB=0, out=None, accumulate=False):
    """out (+)= sum of op(A_i) op(B_i) over terms (A_i, B_i, K_i) that share M, N and the orientations."""
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=terms[0][0].device)
    arr = (GemmTerm * len(terms))(*[GemmTerm(a.data_ptr(), b.data_ptr(), k) for a, b, k in terms])
    check(kernels().seraph_gemm_chain(arr, C.c_int(len(terms)), _p(out), i64(M), i64(N), C.c_int(tA), C.c_int(tB),
                                      C.c_int(1 if accumulate else 0), _stream()), "gemm_chain")
    return out


def gemm_chain_kernel_name(terms, out, M, N, tA=0, tB=0):
    arr = (GemmTerm * len(terms))(*[GemmTerm(a.data_ptr(), b.data_ptr(), k) for a, b, k in terms])
    return kernels().seraph_gemm_chain_kernel_name(arr, C.c_int(len(terms)), _p(out), i64(M), i64(N), C.c_int(tA), C.c_int(tB)).decode()


def gemm_scaled(A, B, M, N, K, tA=0, tB=0, out=None, accumulate=False, alpha=1.0, scratch=True):
    """out (+)= alpha * op(A) op(B); with scratch, small outputs with a long K are computed in runs of K."""
    if out is None:
        out = torch.empty((M, N), dtype=torch.float32, device=A.device)
    k = kernels()
    nbytes = k.seraph_gemm_scaled_ws_bytes(i64(M), i64(N), i64(K), C.c_int(tA), C.c_int(tB)) if scratch else 0
    ws = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=A.device) if scratch else None
    check(k.seraph_gemm_scaled(_p(A), _p(B), _p(out), i64(M), i64(N), i64(K), C.c_int(tA), C.c_int(tB),
                               C.c_int(1 if accumulate else 0), f32(alpha), _p(ws), C.c_size_t(int(nbytes)), _stream()),
          "gemm_scaled")
    return out


class GemmScaledProblem(C.Structure):
    _fields_ = [("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p), ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64)]


def gemm_scaled_grouped(problems, tA=0, tB=0, accumulate=False, alpha=1.0):
    """problems: list of (A, B, out, M, N, K) sharing the orientations, alpha and the accumulate flag; one launch each."""
    k = kernels()
    arr = (GemmScaledProblem * len(problems))(*[GemmScaledProblem(a.data_ptr(), b.data_ptr(), c.data_ptr(), m, n, kk)
                                                 for a, b, c, m, n, kk in problems])
    k.seraph_gemm_scaled_grouped_ws_bytes.restype = C.c_size_t
    nbytes = k.seraph_gemm_scaled_grouped_ws_bytes(arr, C.c_int(len(problems)), C.c_int(tA), C.c_int(tB))
    ws = torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=problems[0][0].device)
    check(k.seraph_gemm_scaled_grouped(arr, C.c_int(len(problems)), C.c_int(tA), C.c_int(tB), C.c_int(1 if accumulate else 0),
                                       f32(alpha), _p(ws), C.c_size_t(int(nbytes)), _stream()), "gemm_scaled_grouped")
    return [p[2] for p in problems]


def attention_forward(Q, K, V, heads, kv_heads, head_dim, seq_starts=None, scale=None, want_lse=True):
    T = Q.shape[0]
    out = torch.empty_like(Q)
    lse = torch.empty((T, heads), dtype=torch.float32, device=Q.device) if want_lse else None
    scale = head_dim ** -0.5 if scale is None else scale
    check(kernels().seraph_attention_forward(_p(Q), _p(K), _p(V), _p(out), _p(lse), _p(seq_starts),
                                             C.c_int(_batch(seq_starts)), i64(T), C.c_int(heads), C.c_int(kv_heads),
                                             C.c_int(head_dim), f32(scale), _stream()), "attention_forward")
    return out, lse


def attention_backward(Q, K, V, dO, heads, kv_heads, head_dim, seq_starts=None, scale=None, out=None, lse=None,
                       dK=None, dV=None, max_seq_len=None, dQ=None):
    """max_seq_len: a bound on the longest packed sequence; when given, the scratch is sized for the
    dS band and the 5-product path runs (seraph_attention_backward_banded)."""
    T = Q.shape[0]
    dQ = torch.empty_like(Q) if dQ is None else dQ
    dK = torch.zeros_like(K) if dK is None else dK
    dV = torch.zeros_like(V) if dV is None else dV
    scale = head_dim ** -0.5 if scale is None else scale
    if max_seq_len is None:
        nbytes = kernels().seraph_attention_backward_ws_bytes(i64(T), C.c_int(heads), C.c_int(kv_heads), C.c_int(head_dim))
    else:
        nbytes = kernels().seraph_attention_backward_ws_bytes_banded(i64(T), C.c_int(heads), C.c_int(kv_heads),
                                                                     C.c_int(head_dim), i64(max_seq_len))
    ws = _workspace(nbytes)
    check(kernels().seraph_attention_backward_banded(_p(Q), _p(K), _p(V), _p(dO), _p(out), _p(lse), _p(dQ), _p(dK), _p(dV),
                                                     _p(seq_starts), C.c_int(_batch(seq_starts)), i64(T), C.c_int(heads),
                                                     C.c_int(kv_heads), C.c_int(head_dim), f32(scale),
                                                     i64(T if max_seq_len is None else max_seq_len), _p(ws), sz(nbytes),
                                                     _stream()), "attention_backward")
    return dQ, dK, dV


def attention_backward_assign(Q, K, V, dO, heads, kv_heads, head_dim, seq_starts=None, host_starts=None, scale=None,
                              out=None, lse=None, dQ=None, dK=None, dV=None):
    """dK / dV assigned (given buffers may hold anything); the dS band sized from the host copy of the offsets."""
    T = Q.shape[0]
    dQ = torch.empty_like(Q) if dQ is None else dQ
    dK = torch.empty_like(K) if dK is None else dK
    dV = torch.empty_like(V) if dV is None else dV
    scale = head_dim ** -0.5 if scale is None else scale
    hs = None
    longest = T
    if seq_starts is not None:
        hs = (C.c_uint32 * len(host_starts))(*[int(x) for x in host_starts])
        longest = max(1, max(int(host_starts[i + 1]) - int(host_starts[i]) for i in range(len(host_starts) - 1)))
    nbytes = kernels().seraph_attention_backward_ws_bytes_banded(i64(T), C.c_int(heads), C.c_int(kv_heads),
                                                                 C.c_int(head_dim), i64(longest))
    ws = _workspace(nbytes)
    check(kernels().seraph_attention_backward_assign(_p(Q), _p(K), _p(V), _p(dO), _p(out), _p(lse), _p(dQ), _p(dK), _p(dV),
                                                     _p(seq_starts), hs, C.c_int(_batch(seq_starts)), i64(T), C.c_int(heads),
                                                     C.c_int(kv_heads), C.c_int(head_dim), f32(scale), _p(ws), sz(nbytes),
                                                     _stream()), "attention_backward_assign")
    return dQ, dK, dV


def rmsnorm(x, scale, eps):
    y = torch.empty_like(x)
    check(kernels().seraph_rmsnorm(_p(x), _p(scale), _p(y), i64(x.shape[0]), i64(x.shape[1]), f32(eps), _stream()),
          "rmsnorm")
    return y


def add_rmsnorm(x, addend, scale, eps):
    """(x + addend, rmsnorm(x + addend)) in one pass."""
    total, y = torch.empty_like(x), torch.empty_like(x)
    check(kernels().seraph_add_rmsnorm(_p(x), _p(addend), _p(total), _p(scale), _p(y), i64(x.shape[0]), i64(x.shape[1]),
                                       f32(eps), _stream()), "add_rmsnorm")
    return total, y


def rmsnorm_backward(x, scale, dy, eps, grad_scale=None, residual=None, out=None):
    """residual: added to the input gradient as it is stored (out may be the residual itself)."""
    dx = torch.empty_like(x) if out is None else out
    gs = torch.zeros_like(scale) if grad_scale is None else grad_scale
    rows, cols = x.shape
    nbytes = kernels().seraph_rmsnorm_backward_ws_bytes(i64(rows), i64(cols))
    ws = _workspace(nbytes)
    if residual is None:
        check(kernels().seraph_rmsnorm_backward(_p(x), _p(scale), _p(dy), _p(dx), _p(gs), i64(rows), i64(cols), f32(eps),
                                                _p(ws), sz(nbytes), _stream()), "rmsnorm_backward")
    else:
        check(kernels().seraph_rmsnorm_backward_residual(_p(x), _p(scale), _p(dy), _p(residual), _p(dx), _p(gs), i64(rows),
                                                         i64(cols), f32(eps), _p(ws), sz(nbytes), _stream()),
              "rmsnorm_backward_residual")
    return dx, gs


class ColsumJob(C.Structure):
    _fields_ = [("partial", C.c_void_p), ("nparts", C.c_int), ("grad_scale", C.c_void_p)]


def rmsnorm_backward_rows(x, scale, dy, eps, residual=None, out=None):
    """The row pass alone: returns (dx, partial rows kept for rmsnorm_colsum_multi, their number)."""
    dx = torch.empty_like(x) if out is None else out
    rows, cols = x.shape
    nbytes = kernels().seraph_rmsnorm_backward_ws_bytes(i64(rows), i64(cols))
    part = torch.empty(max(nbytes // 4, 1), dtype=torch.float32, device=x.device)
    nparts = C.c_int(0)
    check(kernels().seraph_rmsnorm_backward_rows(_p(x), _p(scale), _p(dy), _p(residual), _p(dx), i64(rows), i64(cols), f32(eps),
                                                 _p(part), sz(nbytes), C.byref(nparts), _stream()), "rmsnorm_backward_rows")
    return dx, part, nparts.value


def rmsnorm_colsum_multi(jobs, cols):
    """jobs: (partial, nparts, grad_scale) of row passes of one width; adds each pass's column sums to its grad_scale."""
    arr = (ColsumJob * len(jobs))()
    for i, (part, nparts, gs) in enumerate(jobs):
        arr[i].partial, arr[i].nparts, arr[i].grad_scale = part.data_ptr(), nparts, gs.data_ptr()
    check(kernels().seraph_rmsnorm_colsum_multi(arr, C.c_int(len(jobs)), i64(cols), _stream()), "rmsnorm_colsum_multi")


def rmsnorm_backward_static(x, scale, dy, eps, grad_scale, dx, residual=None):
    """The backward over the library's built-in scratch array: every buffer is the caller's, nothing is allocated."""
    rows, cols = x.shape
    check(kernels().seraph_rmsnorm_backward_static(_p(x), _p(scale), _p(dy), _p(residual), _p(dx), _p(grad_scale), i64(rows),
                                                   i64(cols), f32(eps), _stream()), "rmsnorm_backward_static")
    return dx, grad_scale


def rope(x, heads, head_dim, theta, seq_starts=None, backward=False, out=None):
    out = torch.empty_like(x) if out is None else out
    check(kernels().seraph_rope(_p(x), _p(out), _p(seq_starts), C.c_int(_batch(seq_starts)), i64(x.shape[0]),
                                C.c_int(heads), C.c_int(head_dim), f32(theta), C.c_int(1 if backward else 0),
                                _stream()), "rope")
    return out


def qk_norm_(x, heads, head_dim, eps, use_qk_norm=1):
    check(kernels().seraph_qk_norm(_p(x), i64(x.shape[0]), C.c_int(heads), C.c_int(head_dim), C.c_int(use_qk_norm),
                                   f32(eps), _stream()), "qk_norm")
    return x


def qk_norm_backward(x_pre, dy, heads, head_dim, eps, out=None):
    dx = torch.empty_like(x_pre) if out is None else out
    check(kernels().seraph_qk_norm_backward(_p(x_pre), _p(dy), _p(dx), i64(x_pre.shape[0]), C.c_int(heads),
                                            C.c_int(head_dim), f32(eps), _stream()), "qk_norm_backward")
    return dx


def qk_norm_saved_(x, heads, head_dim, eps):
    """In place; returns (x, rms per token) as the training step keeps them."""
    rms = torch.empty(x.shape[0], dtype=torch.float32, device=x.device)
    check(kernels().seraph_qk_norm_saved(_p(x), _p(rms), i64(x.shape[0]), C.c_int(heads), C.c_int(head_dim), f32(eps), _stream()),
          "qk_norm_saved")
    return x, rms


def qk_norm_backward_saved(y, rms, dy, heads, head_dim, eps, out=None):
    dx = torch.empty_like(y) if out is None else out
    check(kernels().seraph_qk_norm_backward_saved(_p(y), _p(rms), _p(dy), _p(dx), i64(y.shape[0]), C.c_int(heads),
                                                  C.c_int(head_dim), f32(eps), _stream()), "qk_norm_backward_saved")
    return dx


def silu(x):
    y = torch.empty_like(x)
    check(kernels().seraph_silu(_p(x), _p(y), sz(x.numel()), _stream()), "silu")
    return y


def silu_backward(x, dy, out=None):
    dx = torch.empty_like(x) if out is None else out
    check(kernels().seraph_silu_backward(_p(x), _p(dy), _p(dx), sz(x.numel()), _stream()), "silu_backward")
    return dx


def mul_backward(A, B, dC):
    dA, dB = torch.empty_like(A), torch.empty_like(A)
    check(kernels().seraph_mul_backward(_p(A), _p(B), _p(dC), _p(dA), _p(dB), sz(A.numel()), _stream()), "mul_backward")
    return dA, dB


def swiglu_backward(gate, up, dH, out=None):
    dG, dU = (torch.empty_like(gate), torch.empty_like(gate)) if out is None else out
    check(kernels().seraph_swiglu_backward(_p(gate), _p(up), _p(dH), _p(dG), _p(dU), sz(gate.numel()), _stream()),
          "swiglu_backward")
    return dG, dU


def swiglu(gate, up):
    out = torch.empty_like(gate)
    check(kernels().seraph_swiglu(_p(gate), _p(up), _p(out), sz(gate.numel()), _stream()), "swiglu")
    return out


def embed_lookup(tokens, embed):
    T, (V, h) = tokens.numel(), embed.shape
    out = torch.empty((T, h), dtype=torch.float32, device=embed.device)
    check(kernels().seraph_embed_lookup(_p(tokens), _p(embed), _p(out), i64(T), i64(h), i64(V), _stream()), "embed_lookup")
    return out


def embedding_backward(tokens, dH, grad_embed):
    T, (V, h) = tokens.numel(), grad_embed.shape
    nbytes = kernels().seraph_embedding_backward_ws_bytes(i64(T), i64(V))
    ws = _workspace(nbytes)
    check(kernels().seraph_embedding_backward(_p(tokens), _p(dH), _p(grad_embed), i64(T), i64(h), i64(V), _p(ws),
                                              sz(nbytes), _stream()), "embedding_backward")
    return grad_embed


def adamw_(w, g, m, v, lr, beta1, beta2, weight_decay, eps, step, clip=0.0):
    check(kernels().seraph_adamw(_p(w), _p(g), _p(m), _p(v), sz(w.numel()), f32(lr), f32(beta1), f32(beta2),
                                 f32(weight_decay), f32(eps), C.c_int(step), f32(clip), _stream()), "adamw")
    return w, m, v
