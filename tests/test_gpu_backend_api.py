"""The vulkan_* compatible backend (the API src/train.c links against) driven the way the
reference's step drives it: context, buffers, a recorded batch of ops, one submit, a
download - every result checked against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


class Buf(C.Structure):
    _fields_ = [("buffer", C.c_void_p), ("memory", C.c_void_p), ("size", C.c_size_t), ("mapped", C.c_void_p)]


@pytest.fixture(scope="module")
def vk():
    from seraph_amd._lib import backend
    lib = backend()
    lib.vulkan_init_ex.restype = C.c_void_p
    lib.vulkan_buffer_create.restype = C.POINTER(Buf)
    lib.vulkan_buffer_create.argtypes = [C.c_void_p, C.c_size_t]
    ctx = lib.vulkan_init_ex(0, -1)
    assert ctx
    yield lib, C.c_void_p(ctx)
    lib.vulkan_free(C.c_void_p(ctx))


def rng(seed):
    return np.random.default_rng(seed)


def up(vk, a):
    lib, ctx = vk
    a = np.ascontiguousarray(a)
    b = lib.vulkan_buffer_create(ctx, a.nbytes)
    assert b and b.contents.size == a.nbytes and not b.contents.mapped
    lib.vulkan_buffer_upload_bytes(ctx, b, a.ctypes.data_as(C.c_void_p), C.c_size_t(a.nbytes))
    return b


def down(vk, b, shape, dtype=np.float32):
    lib, ctx = vk
    out = np.empty(shape, dtype)
    lib.vulkan_buffer_download_bytes(ctx, b, out.ctypes.data_as(C.c_void_p), C.c_size_t(out.nbytes))
    return out


def close(got, ref, rtol=1e-4, atol=1e-5):
    got, ref = got.astype(np.float64), np.asarray(ref, np.float64)
    assert (np.abs(got - ref) <= atol + rtol * np.abs(ref)).all(), np.abs(got - ref).max()


def test_buffers_and_fill_range(vk):
    lib, ctx = vk
    x = rng(0).standard_normal(1024).astype(np.float32)            # tests/test_vulkan.c: 4 KB round trip
    b = up(vk, x)
    assert (down(vk, b, 1024) == x).all()
    lib.vulkan_fill_buffer_range(ctx, b, C.c_size_t(18), C.c_uint32(0), C.c_size_t(23))   # aligned down: bytes 16..35
    y = down(vk, b, 1024)
    assert (y[4:9] == 0).all() and (y[:4] == x[:4]).all() and (y[9:] == x[9:]).all()
    lib.vulkan_fill_buffer(ctx, b, C.c_uint32(0x3f800000), C.c_size_t(1 << 20))          # clamped to the buffer
    assert (down(vk, b, 1024) == 1.0).all()
    lib.vulkan_buffer_free(ctx, b)
    lib.vulkan_silu(ctx, None, None, C.c_size_t(5))                 # NULL buffers are ignored, not fatal
    assert lib.hip_backend_error_count(ctx) == 0


def test_recorded_backward_slice(vk, orc):
    """One attention block's backward ops in the reference's order (src/train.c:5205-5351),
    recorded between cmd_begin and cmd_end_submit."""
    lib, ctx = vk
    r = rng(1)
    T, H, KVH, D, h = 96, 4, 2, 32, 64
    qd, kv = H * D, KVH * D
    q, k, v = (r.standard_normal((T, w)).astype(np.float32) * 0.4 for w in (qd, kv, kv))
    g_hidden = (1e-2 * r.standard_normal((T, h))).astype(np.float32)
    w_o = (0.05 * r.standard_normal((h, qd))).astype(np.float32)
    w_q = (0.05 * r.standard_normal((qd, h))).astype(np.float32)
    xn = r.standard_normal((T, h)).astype(np.float32)
    layer_in = r.standard_normal((T, h)).astype(np.float32)
    w_norm = (1 + 0.02 * r.standard_normal(h)).astype(np.float32)
    g_wq0 = (1e-3 * r.standard_normal((qd, h))).astype(np.float32)

    B = {n: up(vk, a) for n, a in dict(q=q, k=k, v=v, g_hidden=g_hidden, w_o=w_o, w_q=w_q, xn=xn, layer_in=layer_in,
                                       w_norm=w_norm, g_wq=g_wq0).items()}
    for n, shape in dict(g_attn=(T, qd), g_q=(T, qd), g_k=(T, kv), g_v=(T, kv), g_xn=(T, h), g_tmp=(T, h), g_norm=(h,)).items():
        B[n] = up(vk, np.full(shape, 7.0, np.float32))              # stale contents the ops must overwrite or be told to zero

    assert lib.vulkan_cmd_begin(ctx) == 1
    lib.vulkan_matmul(ctx, B["g_hidden"], B["w_o"], B["g_attn"], T, qd, h)
    lib.vulkan_fill_buffer(ctx, B["g_k"], C.c_uint32(0), C.c_size_t(T * kv * 4))
    lib.vulkan_fill_buffer(ctx, B["g_v"], C.c_uint32(0), C.c_size_t(T * kv * 4))
    lib.vulkan_fill_buffer(ctx, B["g_norm"], C.c_uint32(0), C.c_size_t(h * 4))
    lib.vulkan_batch_attention_backward(ctx, B["q"], B["k"], B["v"], B["g_attn"], B["g_q"], B["g_k"], B["g_v"], T, H, KVH, D)
    lib.vulkan_rope_backward(ctx, B["g_q"], B["g_q"], T, H, D, C.c_float(10000.0))
    lib.vulkan_matmul_transpose(ctx, B["g_q"], B["xn"], B["g_wq"], qd, h, T, 1, 0, 1)
    lib.vulkan_matmul(ctx, B["g_q"], B["w_q"], B["g_xn"], T, h, qd)
    lib.vulkan_rmsnorm_backward_batch(ctx, B["layer_in"], B["w_norm"], B["g_xn"], B["g_tmp"], B["g_norm"], T, h, C.c_float(1e-5))
    lib.vulkan_add(ctx, B["g_tmp"], B["g_hidden"], B["g_hidden"], C.c_size_t(T * h))
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    assert lib.vulkan_cmd_end_submit(ctx) == 0                      # nothing recording any more

    g_attn = orc.matmul(g_hidden, w_o, T, qd, h)
    dq, dk, dv = orc.attention_backward(q, k, v, g_attn, H, KVH, D)
    dq = orc.rope(dq, H, D, 10000.0, backward=True)
    close(down(vk, B["g_k"], (T, kv)), dk); close(down(vk, B["g_v"], (T, kv)), dv)
    close(down(vk, B["g_q"], (T, qd)), dq)
    close(down(vk, B["g_wq"], (qd, h)), orc.matmul(dq, xn, qd, h, T, 1, 0, g_wq0))
    g_xn = orc.matmul(dq, w_q, T, h, qd)
    dx, gs = orc.rmsnorm_backward_batch(layer_in, w_norm, g_xn, 1e-5)
    close(down(vk, B["g_norm"], (h,)), gs)
    close(down(vk, B["g_hidden"], (T, h)), dx + g_hidden)
    for b in B.values():
        lib.vulkan_buffer_free(ctx, b)
    assert lib.hip_backend_error_count(ctx) == 0


def test_loss_chain_and_adamw(vk, orc):
    """cross_entropy_grad + the 512-wide reduce_sum ping-pong (src/train.c:4887-4913), then
    AdamW with the host-side bias corrections (src/vulkan_backend.c:2151-2152)."""
    lib, ctx = vk
    r = rng(2)
    T, V = 1200, 1000
    x = (2 * r.standard_normal((T, V))).astype(np.float32)
    t = r.integers(0, V, T).astype(np.uint32)
    bx, bt = up(vk, x), up(vk, t)
    bg, bl = up(vk, np.zeros((T, V), np.float32)), up(vk, np.zeros(T, np.float32))
    ra, rb = up(vk, np.zeros(T, np.float32)), up(vk, np.zeros(T, np.float32))
    lib.vulkan_cmd_begin(ctx)
    lib.vulkan_cross_entropy_grad(ctx, bx, bt, bg, bl, T - 1, V, T - 1)
    n, rin, rout = T - 1, bl, ra
    while n > 1:
        lib.vulkan_reduce_sum(ctx, rin, rout, C.c_size_t(n))
        n = (n + 511) // 512
        rin, rout = rout, (rb if rout is ra else ra)
    lib.vulkan_cmd_end_submit(ctx)
    rg, rl = orc.cross_entropy_grad(x[:T - 1], t[:T - 1], valid_rows=T - 1)
    close(down(vk, bg, (T, V))[:T - 1], rg, atol=1e-7)
    close(down(vk, rin, (1,)), [rl.astype(np.float64).sum()], rtol=1e-5, atol=1e-3)

    n = 5000
    w = r.standard_normal(n).astype(np.float32)
    g = (1e-3 * r.standard_normal(n)).astype(np.float32)
    z = np.zeros(n, np.float32)
    bw, bgr, bm, bv = up(vk, w), up(vk, g), up(vk, z), up(vk, z)
    f = C.c_float
    lib.vulkan_adamw_update(ctx, bw, bgr, bm, bv, f(3.14e-4), f(0.9), f(0.999), f(0.01), f(1e-8), 3, C.c_size_t(n))
    rw, rm, rv = orc.adamw(w, g, z, z, 3.14e-4, 0.9, 0.999, 0.01, 1e-8, 3)
    close(down(vk, bw, n), rw, atol=1e-7); close(down(vk, bm, n), rm, atol=1e-9); close(down(vk, bv, n), rv, atol=1e-12)
    assert lib.hip_backend_error_count(ctx) == 0


def test_lora_products_through_the_backend(vk, orc):
    """The LoRA adapter's forward the way src/train.c:5785-5792 issues it (product, scale, product into the
    output), once with the reference's three ops and once with hip_matmul_scaled in place of the first two."""
    lib, ctx = vk
    r = rng(21)
    T, d_in, d_out, rank, s = 512, 256, 192, 16, 2.0
    x = r.standard_normal((T, d_in)).astype(np.float32)
    A = (0.05 * r.standard_normal((rank, d_in))).astype(np.float32)
    B = (0.05 * r.standard_normal((d_out, rank))).astype(np.float32)
    y0 = r.standard_normal((T, d_out)).astype(np.float32)
    tmp_ref = s * orc.matmul(x, A, T, rank, d_in, 0, 1)
    ref = orc.matmul(tmp_ref.astype(np.float32), B, T, d_out, rank, 0, 1, y0)
    bx, bA, bB = up(vk, x), up(vk, A), up(vk, B)
    outs = []
    for fused in (False, True):
        btmp, by = up(vk, np.zeros((T, rank), np.float32)), up(vk, y0)
        assert lib.vulkan_cmd_begin(ctx) == 1
        if fused:
            lib.hip_matmul_scaled(ctx, bx, bA, btmp, T, rank, d_in, 0, 1, 0, C.c_float(s))
        else:
            lib.vulkan_matmul_transpose(ctx, bx, bA, btmp, T, rank, d_in, 0, 1, 0)
            lib.vulkan_scale(ctx, btmp, C.c_size_t(T * rank), C.c_float(s))
        lib.vulkan_matmul_transpose(ctx, btmp, bB, by, T, d_out, rank, 0, 1, 1)
        assert lib.vulkan_cmd_end_submit(ctx) == 1
        close(down(vk, btmp, (T, rank)), tmp_ref)
        outs.append(down(vk, by, (T, d_out)))
        close(outs[-1], ref)
        lib.vulkan_buffer_free(ctx, btmp); lib.vulkan_buffer_free(ctx, by)
    for b in (bx, bA, bB):
        lib.vulkan_buffer_free(ctx, b)
    assert lib.hip_backend_error_count(ctx) == 0


def test_norm_column_sums_deferred_through_the_backend(vk):
    """Three norms' backward as vulkan_rmsnorm_backward_batch issues them, and as row passes followed by one
    hip_rmsnorm_colsum_multi over the kept partial rows: the same bits in grad_input and grad_scale."""
    lib, ctx = vk
    lib.hip_rmsnorm_backward_partial_bytes.restype = C.c_size_t
    r = rng(23)
    rows, cols, eps = 300, 512, C.c_float(1e-5)
    s = (1 + 0.02 * r.standard_normal(cols)).astype(np.float32)
    bs = up(vk, s)
    nbytes = lib.hip_rmsnorm_backward_partial_bytes(rows, cols)
    assert nbytes > 0
    keep, parts, nparts, gs_new, want = [], [], [], [], []
    assert lib.vulkan_cmd_begin(ctx) == 1
    for i in range(3):
        x, dy = (r.standard_normal((rows, cols)).astype(np.float32) for _ in range(2))
        g0 = r.standard_normal(cols).astype(np.float32)
        bx, bdy = up(vk, x), up(vk, dy)
        dx1, dx2 = up(vk, np.zeros((rows, cols), np.float32)), up(vk, np.zeros((rows, cols), np.float32))
        gs1, gs2 = up(vk, g0), up(vk, g0)
        part = lib.vulkan_buffer_create(ctx, C.c_size_t(nbytes))
        lib.vulkan_rmsnorm_backward_batch(ctx, bx, bs, bdy, dx1, gs1, rows, cols, eps)
        n = lib.hip_rmsnorm_backward_rows(ctx, bx, bs, bdy, None, dx2, part, rows, cols, eps)
        assert n > 0
        parts.append(part); nparts.append(n); gs_new.append(gs2); want.append((dx1, dx2, gs1))
        keep += [bx, bdy]
    P = (C.c_void_p * 3)(*[C.cast(b, C.c_void_p) for b in parts])
    G = (C.c_void_p * 3)(*[C.cast(b, C.c_void_p) for b in gs_new])
    N = (C.c_int * 3)(*nparts)
    lib.hip_rmsnorm_colsum_multi(ctx, 3, P, N, G, cols)
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    for (dx1, dx2, gs1), gs2 in zip(want, gs_new):
        assert (down(vk, dx1, (rows, cols)) == down(vk, dx2, (rows, cols))).all()
        assert (down(vk, gs1, cols) == down(vk, gs2, cols)).all()
    for buf in keep + parts + gs_new + [b for w in want for b in w] + [bs]:
        lib.vulkan_buffer_free(ctx, buf)
    assert lib.hip_backend_error_count(ctx) == 0


def test_residual_adds_folded_into_the_norms(vk):
    """hip_add_rmsnorm and hip_rmsnorm_backward_residual against the reference's op pairs, bit for bit."""
    lib, ctx = vk
    r = rng(22)
    rows, cols, eps = 300, 512, C.c_float(1e-5)
    x, b, dy = (r.standard_normal((rows, cols)).astype(np.float32) for _ in range(3))
    s = (1 + 0.02 * r.standard_normal(cols)).astype(np.float32)
    bx, bb, bdy, bs = up(vk, x), up(vk, b), up(vk, dy), up(vk, s)
    zeros = lambda shape: up(vk, np.zeros(shape, np.float32))
    sum1, y1, sum2, y2 = (zeros((rows, cols)) for _ in range(4))
    dx1, gs1, gs2 = zeros((rows, cols)), zeros(cols), zeros(cols)
    res2 = up(vk, b)
    assert lib.vulkan_cmd_begin(ctx) == 1
    lib.vulkan_add(ctx, bx, bb, sum1, C.c_size_t(rows * cols))
    lib.vulkan_rmsnorm(ctx, sum1, bs, y1, rows, cols, eps)
    lib.hip_add_rmsnorm(ctx, bx, bb, sum2, bs, y2, rows, cols, eps)
    lib.vulkan_rmsnorm_backward_batch(ctx, bx, bs, bdy, dx1, gs1, rows, cols, eps)
    lib.vulkan_add(ctx, dx1, bb, dx1, C.c_size_t(rows * cols))
    lib.hip_rmsnorm_backward_residual(ctx, bx, bs, bdy, res2, res2, gs2, rows, cols, eps)      # in place
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    assert (down(vk, sum1, (rows, cols)) == down(vk, sum2, (rows, cols))).all()
    assert (down(vk, y1, (rows, cols)) == down(vk, y2, (rows, cols))).all()
    assert (down(vk, dx1, (rows, cols)) == down(vk, res2, (rows, cols))).all()
    assert (down(vk, gs1, cols) == down(vk, gs2, cols)).all()
    for buf in (bx, bb, bdy, bs, sum1, y1, sum2, y2, dx1, gs1, gs2, res2):
        lib.vulkan_buffer_free(ctx, buf)
    assert lib.hip_backend_error_count(ctx) == 0


def test_adamw_update_multi_equals_per_tensor_updates(vk, orc):
    """hip_adamw_update_multi over a tensor list (the 2 + 9 L tensors of a model, src/train.c:4225-4284) in one recorded
    op: bit-identical to one vulkan_adamw_update per tensor, and within tolerance of the oracle.  More tensors than one
    launch carries (48), odd sizes, an empty and a missing entry."""
    lib, ctx = vk
    r = rng(40)
    sizes = [8192 * 64, 64] + [64, 64 * 64, 48 * 64, 48 * 64, 64 * 64, 64, 96 * 64, 96 * 64, 64 * 96] * 8 + [1, 3, 1027, 0]
    n = len(sizes)
    host = [[(0.1 * r.standard_normal(s)).astype(np.float32) for s in sizes] for _ in range(2)]     # w, g
    host_m = [(1e-3 * r.standard_normal(s)).astype(np.float32) for s in sizes]
    host_v = [(1e-6 * r.random(s)).astype(np.float32) for s in sizes]
    hp = (C.c_float(3e-4), C.c_float(0.9), C.c_float(0.999), C.c_float(0.01), C.c_float(1e-8), C.c_int(7))

    def buffers():
        return [[up(vk, a) if a.size else None for a in arrs] for arrs in (host[0], host[1], host_m, host_v)]

    one = buffers()
    lib.vulkan_cmd_begin(ctx)
    for i in range(n):
        if sizes[i]:
            lib.vulkan_adamw_update(ctx, one[0][i], one[1][i], one[2][i], one[3][i], *hp, C.c_size_t(sizes[i]))
    assert lib.vulkan_cmd_end_submit(ctx) == 1

    many = buffers()
    many[1][5] = None                                              # a missing gradient: that tensor is skipped
    arr = lambda bufs: (C.POINTER(Buf) * n)(*[b if b is not None else C.POINTER(Buf)() for b in bufs])
    lib.vulkan_cmd_begin(ctx)
    lib.hip_adamw_update_multi(ctx, C.c_int(n), arr(many[0]), arr(many[1]), arr(many[2]), arr(many[3]),
                               (C.c_size_t * n)(*sizes), *hp, C.c_float(0.0))
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    assert lib.hip_backend_error_count(ctx) == 0
    for i in range(n):
        if not sizes[i]:
            continue
        for which, src in ((0, host[0]), (2, host_m), (3, host_v)):
            got = down(vk, many[which][i], sizes[i])
            if i == 5:
                assert (got == src[i]).all()                       # skipped: untouched
            else:
                assert (got == down(vk, one[which][i], sizes[i])).all(), (i, which)
    rw, rm, rv = orc.adamw(host[0][2], host[1][2], host_m[2], host_v[2], 3e-4, 0.9, 0.999, 0.01, 1e-8, 7)
    close(down(vk, many[0][2], sizes[2]), rw, atol=1e-7)
    for bufs in one + many:
        for b in bufs:
            if b is not None:
                lib.vulkan_buffer_free(ctx, b)


def test_shapes_that_do_not_fit_their_buffers_are_refused():
    """An op whose shape reaches past the end of one of its buffers is not launched: the op reports an error, counts it
    and leaves every buffer as it was.  (Elsewhere such a call reads garbage; on this device it would be a memory fault.)
    A context of its own, because the error count is the context's."""
    from seraph_amd._lib import backend
    lib = backend()
    lib.vulkan_init_ex.restype = C.c_void_p
    lib.vulkan_buffer_create.restype = C.POINTER(Buf)
    lib.vulkan_buffer_create.argtypes = [C.c_void_p, C.c_size_t]
    ctx = C.c_void_p(lib.vulkan_init_ex(0, -1))
    me = (lib, ctx)
    r = rng(90)
    T, h, w = 24, 32, 48
    a = r.standard_normal((T, h)).astype(np.float32)
    b = r.standard_normal((h, w)).astype(np.float32)
    stale = np.full((T, h), 3.0, np.float32)                     # T x h where the product needs T x w
    A, B, Csmall, tok = up(me, a), up(me, b), up(me, stale), up(me, np.arange(T, dtype=np.uint32))
    errors = 0
    calls = [
        lambda: lib.vulkan_matmul(ctx, A, B, Csmall, T, w, h),
        lambda: lib.vulkan_matmul_transpose(ctx, A, B, Csmall, T, w, h, 0, 0, 1),
        lambda: lib.vulkan_add(ctx, A, A, Csmall, C.c_size_t(T * h + 1)),
        lambda: lib.vulkan_scale(ctx, Csmall, C.c_size_t(T * w), C.c_float(2.0)),
        lambda: lib.vulkan_silu(ctx, A, Csmall, C.c_size_t(T * w)),
        lambda: lib.vulkan_rmsnorm(ctx, A, B, Csmall, T, w, C.c_float(1e-5)),
        lambda: lib.vulkan_rope(ctx, Csmall, Csmall, T, 2, 32, C.c_float(10000.0)),
        lambda: lib.vulkan_batch_attention(ctx, A, A, A, Csmall, T, 2, 2, 32),
        lambda: lib.vulkan_embed_lookup(ctx, tok, B, Csmall, T, w, h),
        lambda: lib.vulkan_cross_entropy_grad(ctx, A, tok, Csmall, Csmall, T, w, T),
        lambda: lib.vulkan_rmsnorm_backward_batch(ctx, A, B, A, Csmall, B, T, w, C.c_float(1e-5)),
        lambda: lib.vulkan_batch_attention_backward(ctx, A, A, A, A, Csmall, Csmall, Csmall, T, 2, 2, 32),
        lambda: lib.vulkan_embedding_backward(ctx, tok, A, Csmall, T, h, w),
        lambda: lib.vulkan_silu_backward(ctx, A, A, Csmall, C.c_size_t(T * w)),
        lambda: lib.vulkan_adamw_update(ctx, Csmall, A, A, A, C.c_float(1e-3), C.c_float(0.9), C.c_float(0.999), C.c_float(0.01),
                                        C.c_float(1e-8), 1, C.c_size_t(T * w)),
    ]
    lib.vulkan_cmd_begin(ctx)
    for i, call in enumerate(calls):
        call()
        errors += 1
        assert lib.hip_backend_error_count(ctx) == errors, i
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    assert (down(me, Csmall, (T, h)) == stale).all() and (down(me, A, (T, h)) == a).all()
    # the same ops with shapes that fit still run
    lib.vulkan_cmd_begin(ctx)
    lib.vulkan_matmul(ctx, A, B, Csmall, T, h // 2, h)            # T x 16 of B's first rows: inside every buffer
    lib.vulkan_cmd_end_submit(ctx)
    assert lib.hip_backend_error_count(ctx) == errors
    assert not (down(me, Csmall, (T, h)) == stale).all()
    for buf in (A, B, Csmall, tok):
        lib.vulkan_buffer_free(ctx, buf)
    lib.vulkan_free(ctx)


def test_packed_and_fused_additions_through_the_backend(vk, orc):
    """The entry points the backend adds for packed batches and fused ops (arguments of include/cuda_train_context.h:273-288),
    and the single-op forms the reference's step does not reach in the slices above, each against the oracle: one layer's
    worth of a packed batch, forward and backward, in issue order between cmd_begin and cmd_end_submit."""
    lib, ctx = vk
    r = rng(31)
    f = C.c_float
    starts = np.array([0, 40, 41, 100], np.uint32)
    T, batch, H, KVH, D, V, ffn = 100, 3, 4, 2, 32, 211, 96
    hdim, qd, kvd = 64, H * D, KVH * D
    theta, eps = 10000.0, 1e-6
    tok = r.integers(0, V, T).astype(np.uint32)
    E = r.standard_normal((V, hdim)).astype(np.float32)
    q, k, v = (0.5 * r.standard_normal((T, w)).astype(np.float32) for w in (qd, kvd, kvd))
    d_out = (0.1 * r.standard_normal((T, qd))).astype(np.float32)
    logits = (2 * r.standard_normal((T, V))).astype(np.float32)
    gate, upv, d_h = (r.standard_normal((T, ffn)).astype(np.float32) for _ in range(3))
    dk0, dv0 = (r.standard_normal((T, kvd)).astype(np.float32) for _ in range(2))
    ge0 = r.standard_normal((V, hdim)).astype(np.float32)
    d_hidden = r.standard_normal((T, hdim)).astype(np.float32)

    B = {n: up(vk, a) for n, a in dict(tok=tok, E=E, q=q, k=k, v=v, d_out=d_out, logits=logits, gate=gate, up=upv, d_h=d_h,
                                       starts=starts, dk=dk0, dv=dv0, dk2=dk0, dv2=dv0, ge=ge0, d_hidden=d_hidden).items()}
    for n, shape in dict(hid=(T, hdim), qn=(T, qd), qr=(T, qd), kr=(T, kvd), att=(T, qd), lse=(T, H), dq=(T, qd), dq2=(T, qd),
                         dqr=(T, qd), dqn=(T, qd), gl=(T, V), loss=(T,), act=(T, ffn), sil=(T, ffn), g_gate=(T, ffn), g_up=(T, ffn),
                         g_sil=(T, ffn), g_a=(T, ffn), g_b=(T, ffn), copy=(T, qd), att1=(T, qd)).items():
        B[n] = up(vk, np.full(shape, 7.0, np.float32))
    B["flags"] = up(vk, np.zeros(4, np.uint32))
    n_valid = T - batch

    assert lib.vulkan_cmd_begin(ctx) == 1
    lib.vulkan_embed_lookup(ctx, B["tok"], B["E"], B["hid"], T, hdim, V)
    lib.vulkan_copy_buffer(ctx, B["q"], B["qn"], C.c_size_t(T * qd * 4))
    lib.vulkan_qk_norm(ctx, B["qn"], T, H, D, 1, f(eps))
    lib.hip_rope_packed(ctx, B["qn"], B["qr"], B["starts"], T, batch, H, D, f(theta))
    lib.hip_rope_packed(ctx, B["k"], B["kr"], B["starts"], T, batch, KVH, D, f(theta))
    lib.hip_batch_attention_packed(ctx, B["qr"], B["kr"], B["v"], B["att"], B["lse"], B["starts"], T, batch, H, KVH, D)
    lib.vulkan_copy_buffer_cache(ctx, B["att"], B["copy"], C.c_size_t(T * qd * 4))
    lib.hip_cross_entropy_grad_packed(ctx, B["logits"], B["tok"], B["gl"], B["loss"], B["starts"], T, batch, V, n_valid)
    lib.hip_batch_attention_backward_packed(ctx, B["qr"], B["kr"], B["v"], B["att"], B["lse"], B["d_out"], B["dq"], B["dk"], B["dv"],
                                            B["starts"], T, batch, H, KVH, D)
    lib.hip_batch_attention_backward_packed(ctx, B["qr"], B["kr"], B["v"], None, None, B["d_out"], B["dq2"], B["dk2"], B["dv2"],
                                            B["starts"], T, batch, H, KVH, D)             # nothing saved: recomputed
    lib.hip_rope_backward_packed(ctx, B["dq"], B["dqr"], B["starts"], T, batch, H, D, f(theta))
    lib.hip_qk_norm_backward(ctx, B["q"], B["dqr"], B["dqn"], T, H, D, f(eps))
    lib.hip_swiglu(ctx, B["gate"], B["up"], B["act"], C.c_size_t(T * ffn))
    lib.hip_swiglu_backward(ctx, B["gate"], B["up"], B["d_h"], B["g_gate"], B["g_up"], C.c_size_t(T * ffn))
    lib.vulkan_silu(ctx, B["gate"], B["sil"], C.c_size_t(T * ffn))                        # the reference's two ops for the same
    lib.vulkan_mul(ctx, B["sil"], B["up"], B["sil"], C.c_size_t(T * ffn))
    lib.vulkan_elementwise_mul_backward(ctx, B["gate"], B["up"], B["d_h"], B["g_a"], B["g_b"], C.c_size_t(T * ffn))
    lib.vulkan_silu_backward(ctx, B["gate"], B["d_h"], B["g_sil"], C.c_size_t(T * ffn))
    lib.vulkan_embedding_backward(ctx, B["tok"], B["d_hidden"], B["ge"], T, hdim, V)
    lib.vulkan_nan_check(ctx, B["att"], C.c_size_t(T * qd), B["flags"], 2)
    lib.vulkan_barrier_transfer_to_compute(ctx)
    assert lib.vulkan_cmd_end_submit(ctx) == 1
    # one sequence through the unpacked forms (outside a recording: synchronous)
    lib.vulkan_rope(ctx, B["q"], B["dq2"], T, H, D, f(theta))
    lib.vulkan_batch_attention(ctx, B["q"], B["k"], B["v"], B["att1"], T, H, KVH, D)
    assert lib.hip_backend_error_count(ctx) == 0

    assert (down(vk, B["hid"], (T, hdim)) == orc.embed_lookup(tok, E)).all()
    qn = orc.qk_norm(q, H, D, eps)
    close(down(vk, B["qn"], (T, qd)), qn)
    qr, kr = orc.rope(qn, H, D, theta, starts), orc.rope(k, KVH, D, theta, starts)
    close(down(vk, B["qr"], (T, qd)), qr); close(down(vk, B["kr"], (T, kvd)), kr)
    att, lse = orc.attention_forward(qr, kr, v, H, KVH, D, starts)
    close(down(vk, B["att"], (T, qd)), att); close(down(vk, B["lse"], (T, H)), lse)
    assert (down(vk, B["copy"], (T, qd)) == down(vk, B["att"], (T, qd))).all()
    gl, loss = orc.cross_entropy_grad_packed(logits, tok, starts, n_valid)
    close(down(vk, B["gl"], (T, V)), gl, atol=1e-7); close(down(vk, B["loss"], (T,)), loss)
    dq, dk, dv = orc.attention_backward(qr, kr, v, d_out, H, KVH, D, starts, dK0=dk0, dV0=dv0)
    for a, b, ref, shape in (("dq", "dq2", dq, (T, qd)), ("dk", "dk2", dk, (T, kvd)), ("dv", "dv2", dv, (T, kvd))):
        if a != "dq":
            close(down(vk, B[b], shape), ref)                      # dq2 was reused by vulkan_rope below
        close(down(vk, B[a], shape), ref)
    dqr = orc.rope(dq, H, D, theta, starts, backward=True)
    close(down(vk, B["dqr"], (T, qd)), dqr)
    close(down(vk, B["dqn"], (T, qd)), orc.qk_norm_backward(q, dqr, H, D, eps), atol=2e-5)
    act = orc.silu(gate) * upv
    close(down(vk, B["act"], (T, ffn)), act); close(down(vk, B["sil"], (T, ffn)), act)
    gg, gu = orc.swiglu_backward(gate, upv, d_h)
    close(down(vk, B["g_gate"], (T, ffn)), gg); close(down(vk, B["g_up"], (T, ffn)), gu)
    ga, gb = orc.mul_backward(gate, upv, d_h)
    assert (down(vk, B["g_a"], (T, ffn)) == ga).all() and (down(vk, B["g_b"], (T, ffn)) == gb).all()
    close(down(vk, B["g_sil"], (T, ffn)), orc.silu_backward(gate, d_h))
    close(down(vk, B["ge"], (V, hdim)), orc.embedding_backward(tok, d_hidden, ge0))
    assert (down(vk, B["flags"], 4, np.uint32) == 0).all()
    close(down(vk, B["dq2"], (T, qd)), orc.rope(q, H, D, theta))
    close(down(vk, B["att1"], (T, qd)), orc.attention_forward(q, k, v, H, KVH, D)[0])
    for b in B.values():
        lib.vulkan_buffer_free(ctx, b)


def test_video_mode_ops_report_that_they_are_not_provided():
    """The four video-only symbols exist so that train.o links (include/vulkan_backend.h:600-642); calling one is an error
    that is reported and counted, nothing more.  A context of its own (vulkan_init, the pool-size form), because the error
    count is the context's."""
    from seraph_amd._lib import backend
    lib = backend()
    lib.vulkan_init.restype = C.c_void_p
    ctx = C.c_void_p(lib.vulkan_init(0))
    assert ctx
    lib.vulkan_patch_extract(ctx, None, None, 1, 1, 1, 1, 1, 1)
    lib.vulkan_add_bias(ctx, None, None, 1, 1)
    lib.vulkan_bce_loss_grad(ctx, None, None, None, None, C.c_size_t(1))
    lib.vulkan_sum_cols(ctx, None, None, 1, 1)
    assert lib.hip_backend_error_count(ctx) == 4
    lib.vulkan_free(ctx)
