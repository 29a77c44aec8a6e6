// embedding.hip - embedding lookup and its deterministic scatter-add backward.
//
// shaders/embedding_backward.comp:22-44 adds every element of dH into the table with a
// compare-and-swap loop, so rows of repeated tokens serialise and the summation order
// changes from run to run.  Here positions are grouped by token first (count, exclusive
// scan, fill, in-group rank - all integer work, O(T + vocab)); then one workgroup per
// touched row adds that row's positions in ascending order and performs a single
// read-modify-write of the table row.  HBM traffic: dH once, each touched row once in
// and once out.
#include "common.hpp"

namespace seraph {

// ---------------------------------------------------------------- lookup
__global__ __launch_bounds__(256) void embed_lookup_kernel(const uint32_t* __restrict__ tokens,
                                                           const float* __restrict__ embed,
                                                           float* __restrict__ out,
                                                           int64_t T, int64_t hidden, int64_t vocab, int vec) {
    const int64_t t = blockIdx.x;
    const uint32_t tok = tokens[t];
    const bool ok = (int64_t)tok < vocab;                      // embed_lookup.comp:32-36: zero row otherwise
    const float* src = embed + (int64_t)tok * hidden;
    float* dst = out + t * hidden;
    if (vec) {
        const int64_t n4 = hidden >> 2;
        for (int64_t i = threadIdx.x; i < n4; i += 256)
            reinterpret_cast<float4*>(dst)[i] = ok ? reinterpret_cast<const float4*>(src)[i] : make_float4(0, 0, 0, 0);
    } else {
        for (int64_t i = threadIdx.x; i < hidden; i += 256) dst[i] = ok ? src[i] : 0.0f;
    }
}

// ---------------------------------------------------------------- backward: grouping
struct EmbWs {
    uint32_t* cnt;      // [vocab + 1]  per-token count, then fill cursor
    uint32_t* off;      // [vocab + 1]  exclusive scan of cnt
    uint32_t* uniq;     // [T]          tokens that occur, ascending
    uint32_t* nuniq;    // [1]
    uint32_t* perm;     // [T]          positions grouped by token, arbitrary order inside a group
    uint32_t* sorted;   // [T]          the same, ascending inside each group
};

static size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

static size_t emb_ws_layout(int64_t T, int64_t vocab, char* base, EmbWs* w) {
    size_t o = 0;
    auto take = [&](size_t count) { uint32_t* p = (uint32_t*)(base + o); o += align_up(count * 4); return p; };
    uint32_t* cnt = take((size_t)vocab + 1);
    uint32_t* off = take((size_t)vocab + 1);
    uint32_t* uniq = take((size_t)T);
    uint32_t* nuniq = take(1);
    uint32_t* perm = take((size_t)T);
    uint32_t* sorted = take((size_t)T);
    if (w) { w->cnt = cnt; w->off = off; w->uniq = uniq; w->nuniq = nuniq; w->perm = perm; w->sorted = sorted; }
    return o;
}

__global__ __launch_bounds__(256) void emb_count_kernel(const uint32_t* __restrict__ tokens, uint32_t* cnt,
                                                        int64_t T, int64_t vocab) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p < T && (int64_t)tokens[p] < vocab) atomicAdd(&cnt[tokens[p]], 1u);     // integer: order-independent
}

// One workgroup scans the whole vocabulary: off = exclusive scan(cnt), uniq = tokens with
// cnt > 0, and cnt is cleared so the fill kernel can reuse it as a cursor.
__global__ __launch_bounds__(1024) void emb_scan_kernel(uint32_t* cnt, uint32_t* off, uint32_t* uniq,
                                                        uint32_t* nuniq, int64_t vocab) {
    __shared__ uint32_t s_sum[1024], s_nz[1024];
    const int tid = threadIdx.x;
    const int64_t per = (vocab + 1023) / 1024;
    const int64_t lo = tid * per, hi = (lo + per < vocab) ? lo + per : vocab;
    uint32_t sum = 0, nz = 0;
    for (int64_t v = lo; v < hi; v++) { uint32_t c = cnt[v]; sum += c; nz += c ? 1u : 0u; }
    s_sum[tid] = sum; s_nz[tid] = nz;
    __syncthreads();
    for (int d = 1; d < 1024; d <<= 1) {                       // Hillis-Steele inclusive scan
        uint32_t a = tid >= d ? s_sum[tid - d] : 0u, b = tid >= d ? s_nz[tid - d] : 0u;
        __syncthreads();
        s_sum[tid] += a; s_nz[tid] += b;
        __syncthreads();
    }
    uint32_t run = s_sum[tid] - sum, urun = s_nz[tid] - nz;    // exclusive prefixes of this lane's chunk
    for (int64_t v = lo; v < hi; v++) {
        uint32_t c = cnt[v];
        off[v] = run;
        if (c) uniq[urun++] = (uint32_t)v;
        run += c;
        cnt[v] = 0;
    }
    if (tid == 1023) { off[vocab] = s_sum[1023]; *nuniq = s_nz[1023]; }
}

__global__ __launch_bounds__(256) void emb_fill_kernel(const uint32_t* __restrict__ tokens, uint32_t* cnt,
                                                       const uint32_t* __restrict__ off, uint32_t* perm,
                                                       int64_t T, int64_t vocab) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= T) return;
    uint32_t tok = tokens[p];
    if ((int64_t)tok >= vocab) return;
    perm[off[tok] + atomicAdd(&cnt[tok], 1u)] = (uint32_t)p;
}

// Rank of each position inside its group: makes the order independent of the fill race.
__global__ __launch_bounds__(256) void emb_rank_kernel(const uint32_t* __restrict__ tokens,
                                                       const uint32_t* __restrict__ off,
                                                       const uint32_t* __restrict__ perm, uint32_t* sorted,
                                                       int64_t vocab) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)off[vocab]) return;
    uint32_t p = perm[i], tok = tokens[p];
    uint32_t lo = off[tok], hi = off[tok + 1], rank = 0;
    for (uint32_t q = lo; q < hi; q++) rank += perm[q] < p ? 1u : 0u;
    sorted[lo + rank] = p;
}

__global__ __launch_bounds__(256) void emb_sum_kernel(const uint32_t* __restrict__ uniq,
                                                      const uint32_t* __restrict__ nuniq,
                                                      const uint32_t* __restrict__ off,
                                                      const uint32_t* __restrict__ sorted,
                                                      const float* __restrict__ dH, float* __restrict__ grad_embed,
                                                      int64_t hidden, int vec) {
    if (blockIdx.x >= *nuniq) return;
    const uint32_t tok = uniq[blockIdx.x];
    const uint32_t lo = off[tok], hi = off[tok + 1];
    float* row = grad_embed + (int64_t)tok * hidden;
    if (vec) {
        const int64_t n4 = hidden >> 2;
        for (int64_t i = threadIdx.x; i < n4; i += 256) {
            float4 a = make_float4(0, 0, 0, 0);
            for (uint32_t q = lo; q < hi; q++) {
                float4 g = reinterpret_cast<const float4*>(dH + (int64_t)sorted[q] * hidden)[i];
                a.x += g.x; a.y += g.y; a.z += g.z; a.w += g.w;
            }
            float4 r = reinterpret_cast<float4*>(row)[i];
            r.x += a.x; r.y += a.y; r.z += a.z; r.w += a.w;
            reinterpret_cast<float4*>(row)[i] = r;
        }
    } else {
        for (int64_t i = threadIdx.x; i < hidden; i += 256) {
            float a = 0.0f;
            for (uint32_t q = lo; q < hi; q++) a += dH[(int64_t)sorted[q] * hidden + i];
            row[i] += a;
        }
    }
}

}  // namespace seraph

using namespace seraph;

extern "C" {

int seraph_embed_lookup(const uint32_t* tokens, const float* embed, float* out,
                        int64_t T, int64_t hidden, int64_t vocab, seraph_stream_t s) {
    if (T == 0 || hidden == 0) return SERAPH_OK;
    SERAPH_REQUIRE(tokens && embed && out, "embed_lookup: NULL pointer");
    SERAPH_REQUIRE(T > 0 && T <= 0x7fffffff && hidden > 0 && vocab > 0, "embed_lookup: bad shape");
    int vec = (hidden % 4 == 0) && aligned16(embed) && aligned16(out);
    hipLaunchKernelGGL(embed_lookup_kernel, dim3((unsigned)T), dim3(256), 0, as_stream(s), tokens, embed, out, T, hidden, vocab, vec);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

size_t seraph_embedding_backward_ws_bytes(int64_t T, int64_t vocab) {
    if (T <= 0 || vocab <= 0) return 0;
    return emb_ws_layout(T, vocab, nullptr, nullptr);
}

int seraph_embedding_backward(const uint32_t* tokens, const float* dH, float* grad_embed,
                              int64_t T, int64_t hidden, int64_t vocab,
                              void* ws, size_t ws_bytes, seraph_stream_t s) {
    if (T == 0 || hidden == 0) return SERAPH_OK;
    SERAPH_REQUIRE(tokens && dH && grad_embed, "embedding_backward: NULL pointer");
    SERAPH_REQUIRE(T > 0 && T <= 0x7fffffff && hidden > 0 && vocab > 0 && vocab < 0xffffffffLL, "embedding_backward: bad shape");
    if (!ws || ws_bytes < seraph_embedding_backward_ws_bytes(T, vocab) || !aligned16(ws)) {
        set_error("embedding_backward: 16-byte aligned scratch of %zu bytes required", seraph_embedding_backward_ws_bytes(T, vocab));
        return SERAPH_ERR_WORKSPACE;
    }
    EmbWs w;
    emb_ws_layout(T, vocab, (char*)ws, &w);
    hipStream_t st = as_stream(s);
    int rc = seraph_fill_u32(w.cnt, 0u, (size_t)vocab + 1, s);
    if (rc != SERAPH_OK) return rc;
    const dim3 tgrid((unsigned)ceil_div(T, 256));
    hipLaunchKernelGGL(emb_count_kernel, tgrid, dim3(256), 0, st, tokens, w.cnt, T, vocab);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_scan_kernel, dim3(1), dim3(1024), 0, st, w.cnt, w.off, w.uniq, w.nuniq, vocab);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_fill_kernel, tgrid, dim3(256), 0, st, tokens, w.cnt, w.off, w.perm, T, vocab);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_rank_kernel, tgrid, dim3(256), 0, st, tokens, w.off, w.perm, w.sorted, vocab);
    SERAPH_LAUNCH_CHECK();
    int vec = (hidden % 4 == 0) && aligned16(dH) && aligned16(grad_embed);
    int64_t nblocks = T < vocab ? T : vocab;                  // upper bound on the number of touched rows
    hipLaunchKernelGGL(emb_sum_kernel, dim3((unsigned)nblocks), dim3(256), 0, st, w.uniq, w.nuniq, w.off, w.sorted,
                       dH, grad_embed, hidden, vec);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // extern "C"
