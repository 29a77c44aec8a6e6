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
    uint32_t* csum;     // [chunks]     per-chunk count totals, then bases
    uint32_t* cnz;      // [chunks]     per-chunk distinct-token totals, then bases
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
    const size_t chunks = (size_t)((vocab + 4095) / 4096);
    uint32_t* csum = take(chunks);
    uint32_t* cnz = take(chunks);
    if (w) { w->csum = csum; w->cnz = cnz; w->cnt = cnt; w->off = off; w->uniq = uniq; w->nuniq = nuniq; w->perm = perm; w->sorted = sorted; }
    return o;
}

__global__ __launch_bounds__(256) void emb_count_kernel(const uint32_t* __restrict__ tokens, uint32_t* cnt,
                                                        int64_t T, int64_t vocab) {
    int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p < T && (int64_t)tokens[p] < vocab) atomicAdd(&cnt[tokens[p]], 1u);     // integer: order-independent
}

// Exclusive scan of the per-token counts over the vocabulary in three small launches:
// per-chunk totals (4096 tokens per workgroup, coalesced 16-byte loads), a serial scan of the
// few chunk totals, then a rescan of every chunk from its base.  The last pass writes
// off = exclusive scan(cnt) and uniq = tokens with cnt > 0 in ascending order, and clears cnt
// so the fill kernel can reuse it as a cursor.
constexpr int kScanBlock = 1024;
constexpr int kScanChunk = 4 * kScanBlock;

__device__ __forceinline__ uint4 load_cnt4(const uint32_t* cnt, int64_t v0, int64_t vocab) {
    uint4 c = make_uint4(0, 0, 0, 0);
    if (v0 + 3 < vocab && ((v0 & 3) == 0)) return *reinterpret_cast<const uint4*>(cnt + v0);
    if (v0 < vocab) c.x = cnt[v0];
    if (v0 + 1 < vocab) c.y = cnt[v0 + 1];
    if (v0 + 2 < vocab) c.z = cnt[v0 + 2];
    if (v0 + 3 < vocab) c.w = cnt[v0 + 3];
    return c;
}

__global__ __launch_bounds__(kScanBlock) void emb_chunk_sums_kernel(const uint32_t* __restrict__ cnt, int64_t vocab,
                                                                    uint32_t* __restrict__ csum, uint32_t* __restrict__ cnz) {
    __shared__ uint32_t s_sum[kScanBlock / 64], s_nz[kScanBlock / 64];
    const int64_t v0 = (int64_t)blockIdx.x * kScanChunk + 4 * threadIdx.x;
    const uint4 c = load_cnt4(cnt, v0, vocab);
    uint32_t sum = c.x + c.y + c.z + c.w;
    uint32_t nz = (c.x ? 1u : 0u) + (c.y ? 1u : 0u) + (c.z ? 1u : 0u) + (c.w ? 1u : 0u);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) { sum += __shfl_xor(sum, o, 64); nz += __shfl_xor(nz, o, 64); }
    if ((threadIdx.x & 63) == 0) { s_sum[threadIdx.x >> 6] = sum; s_nz[threadIdx.x >> 6] = nz; }
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t a = 0, b = 0;
        for (int w = 0; w < kScanBlock / 64; w++) { a += s_sum[w]; b += s_nz[w]; }
        csum[blockIdx.x] = a;
        cnz[blockIdx.x] = b;
    }
}

// chunk totals -> exclusive chunk bases (in place); also off[vocab] and the number of distinct tokens
__global__ void emb_chunk_scan_kernel(uint32_t* csum, uint32_t* cnz, int nchunks, uint32_t* off, uint32_t* nuniq, int64_t vocab) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    uint32_t a = 0, b = 0;
    for (int i = 0; i < nchunks; i++) {
        uint32_t x = csum[i], y = cnz[i];
        csum[i] = a; cnz[i] = b;
        a += x; b += y;
    }
    off[vocab] = a;
    *nuniq = b;
}

__global__ __launch_bounds__(kScanBlock) void emb_chunk_write_kernel(uint32_t* __restrict__ cnt, int64_t vocab,
                                                                     const uint32_t* __restrict__ csum,
                                                                     const uint32_t* __restrict__ cnz,
                                                                     uint32_t* __restrict__ off, uint32_t* __restrict__ uniq) {
    __shared__ uint32_t s_sum[kScanBlock], s_nz[kScanBlock];
    const int tid = threadIdx.x;
    const int64_t v0 = (int64_t)blockIdx.x * kScanChunk + 4 * tid;
    const uint4 c = load_cnt4(cnt, v0, vocab);
    const uint32_t sum = c.x + c.y + c.z + c.w;
    const uint32_t nz = (c.x ? 1u : 0u) + (c.y ? 1u : 0u) + (c.z ? 1u : 0u) + (c.w ? 1u : 0u);
    s_sum[tid] = sum; s_nz[tid] = nz;
    __syncthreads();
    for (int d = 1; d < kScanBlock; d <<= 1) {                 // Hillis-Steele inclusive scan
        uint32_t a = tid >= d ? s_sum[tid - d] : 0u, b = tid >= d ? s_nz[tid - d] : 0u;
        __syncthreads();
        s_sum[tid] += a; s_nz[tid] += b;
        __syncthreads();
    }
    uint32_t run = csum[blockIdx.x] + s_sum[tid] - sum;         // exclusive prefix of this lane's four tokens
    uint32_t urun = cnz[blockIdx.x] + s_nz[tid] - nz;
    const uint32_t cs[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int e = 0; e < 4; e++) {
        const int64_t v = v0 + e;
        if (v < vocab) {
            off[v] = run;
            if (cs[e]) uniq[urun++] = (uint32_t)v;
            run += cs[e];
            cnt[v] = 0;
        }
    }
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
    const int nchunks = (int)ceil_div(vocab, kScanChunk);
    hipLaunchKernelGGL(emb_chunk_sums_kernel, dim3(nchunks), dim3(kScanBlock), 0, st, w.cnt, vocab, w.csum, w.cnz);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_chunk_scan_kernel, dim3(1), dim3(64), 0, st, w.csum, w.cnz, nchunks, w.off, w.nuniq, vocab);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_chunk_write_kernel, dim3(nchunks), dim3(kScanBlock), 0, st, w.cnt, vocab, w.csum, w.cnz, w.off, w.uniq);
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
