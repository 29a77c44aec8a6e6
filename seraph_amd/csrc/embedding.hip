// embedding.hip - embedding lookup and its deterministic scatter-add backward.
//
// shaders/embedding_backward.comp:22-44 adds every element of dH into the table with a
// compare-and-swap loop, so rows of repeated tokens serialise and the summation order
// changes from run to run.  Here every position joins its token's chain with one exchange on a
// per-token table (integer work; the chain's order is arbitrary), the one position of each token that
// found the chain empty becomes the token's owner, and one wavefront per owner gathers the token's
// positions, puts them in ascending order and adds their rows of dH in that order, with a single
// read-modify-write of the table row.  Three launches; HBM traffic: dH once, each touched row once in and
// once out.  The sum does not depend on the order in which positions joined, so reruns are bit-identical.
// A token that fills a large part of the batch (padding, a begin-of-sequence token in thousands of short packed
// sequences) would leave one wavefront adding thousands of rows alone: such a group is cut along the row's width
// instead, the first positions of the group to arrive taking one 64-slot slab of columns each, every slab added in
// the same ascending order - still no scratch, no second level of sums, and the same bits whoever takes which slab.
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

// ---------------------------------------------------------------- backward
constexpr uint32_t kNil = 0xffffffffu;
struct EmbWs {
    uint4* tab;         // [vocab]  x = most recent position that joined the token's chain (kNil: none), y = positions so far,
                        //          z = column slabs of a long group handed out so far
    uint32_t* link;     // [T]      the position that had joined the same token's chain before this one; kNil for the first
};

static size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

static size_t emb_ws_layout(int64_t T, int64_t vocab, char* base, EmbWs* w) {
    size_t o = 0;
    char* tab = base + o; o += align_up((size_t)vocab * 16);
    char* link = base + o; o += align_up((size_t)T * 4);
    if (w) { w->tab = (uint4*)tab; w->link = (uint32_t*)link; }
    return o;
}

__global__ __launch_bounds__(256) void emb_init_kernel(uint4* __restrict__ tab, int64_t vocab) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v < vocab) tab[v] = make_uint4(kNil, 0u, 0u, 0u);
}

__global__ __launch_bounds__(256) void emb_link_kernel(const uint32_t* __restrict__ tokens, uint4* tab, uint32_t* __restrict__ link,
                                                       int64_t T, int64_t vocab) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= T) return;
    const uint32_t tok = tokens[p];
    if ((int64_t)tok >= vocab) { link[p] = 0u; return; }      // skipped position (embedding_backward.comp:31): owns nothing (its token is checked again)
    atomicAdd(&tab[tok].y, 1u);
    link[p] = atomicExch(&tab[tok].x, (uint32_t)p);
}

// One wavefront per position; only a token's owner (the position whose exchange found the chain empty) works.
// The owner's own row of dH is requested before anything is known about the token, the table row as soon as the
// token is: for a token that occurs once, which is most of them, two dependent loads precede the payload.
constexpr int kEmbList = 1024;          // positions gathered per batch
constexpr int kEmbWalk = 16;            // up to this many positions the chain is walked; longer groups are found by scanning the tokens
constexpr int kEmbVpl = 8;              // float4 per lane and pass: 2048 floats of a row
constexpr uint32_t kEmbLong = 128;      // from this many positions on a group is cut into column slabs (rows of more than one slab)
constexpr int kEmbAhead = 32;           // rows in flight per slab wavefront (32 KB: a round trip of memory at some 10 GB/s per wavefront)

// One slab (64 float4 slots of the row's width) of a long group: draw a slab number, leave if all are taken, else sweep the
// token array for the group's positions (ascending by construction) a batch at a time and add the slab's part of their
// rows in that order, kEmbAhead rows' loads in flight; one read-modify-write of the slab's part of the table row.
__device__ __forceinline__ void emb_sum_slab(const uint32_t* __restrict__ tokens, uint4* entry, const float* __restrict__ dH,
                                             float* row, int64_t T, int64_t hidden, uint32_t tok, uint32_t count, uint32_t* list) {
    const int lane = threadIdx.x;
    const int64_t n4 = hidden >> 2, nslabs = (n4 + 63) / 64;
    uint32_t slab = 0;
    if (lane == 0) slab = atomicAdd(&entry->z, 1u);
    slab = __shfl(slab, 0, 64);
    if ((int64_t)slab >= nslabs) return;
    const int64_t i4 = (int64_t)slab * 64 + lane;
    const bool ok = i4 < n4;
    float4 acc = make_float4(0, 0, 0, 0);
    int64_t cursor = 0;
    uint32_t found = 0;
    while (found < count && cursor < T) {
        constexpr int U = 8;
        int len = 0;
        while (len + 64 * U <= kEmbList && cursor < T && found + (uint32_t)len < count) {
            uint32_t tk[U];
#pragma unroll
            for (int j = 0; j < U; j++) {
                const int64_t q = cursor + 64 * j + lane;
                tk[j] = q < T ? tokens[q] : kNil;
            }
#pragma unroll
            for (int j = 0; j < U; j++) {
                const bool hit = tk[j] == tok;
                const unsigned long long mask = __ballot(hit);
                if (hit) list[len + __popcll(mask & ((1ull << lane) - 1ull))] = (uint32_t)(cursor + 64 * j + lane);
                len += __popcll(mask);
            }
            cursor += 64 * U;
        }
        __syncthreads();
        found += (uint32_t)len;
        int m = 0;
        for (; m + kEmbAhead <= len; m += kEmbAhead) {
            float4 g[kEmbAhead];
#pragma unroll
            for (int u = 0; u < kEmbAhead; u++)
                g[u] = ok ? reinterpret_cast<const float4*>(dH + (int64_t)list[m + u] * hidden)[i4] : make_float4(0, 0, 0, 0);
#pragma unroll
            for (int u = 0; u < kEmbAhead; u++) { acc.x += g[u].x; acc.y += g[u].y; acc.z += g[u].z; acc.w += g[u].w; }
        }
        for (; m < len; m++) {
            if (ok) { const float4 g = reinterpret_cast<const float4*>(dH + (int64_t)list[m] * hidden)[i4]; acc.x += g.x; acc.y += g.y; acc.z += g.z; acc.w += g.w; }
        }
        __syncthreads();
    }
    if (ok) {
        float4 r = reinterpret_cast<float4*>(row)[i4];
        r.x += acc.x; r.y += acc.y; r.z += acc.z; r.w += acc.w;
        reinterpret_cast<float4*>(row)[i4] = r;
    }
}

__global__ __launch_bounds__(64) void emb_sum_kernel(const uint32_t* __restrict__ tokens, uint4* tab,
                                                     const uint32_t* __restrict__ link,
                                                     const float* __restrict__ dH, float* __restrict__ grad_embed,
                                                     int64_t T, int64_t hidden, int64_t vocab, int vec) {
    __shared__ uint32_t list[kEmbList], tmp[kEmbWalk];
    const int lane = threadIdx.x;
    const int64_t p = blockIdx.x;
    const int64_t n4 = hidden >> 2;
    // speculative: the first pass of this position's own row
    float4 own[kEmbVpl];
    if (vec) {
#pragma unroll
        for (int k = 0; k < kEmbVpl; k++) {
            const int64_t i = lane + 64 * k;
            own[k] = i < n4 ? reinterpret_cast<const float4*>(dH + p * hidden)[i] : make_float4(0, 0, 0, 0);
        }
    }
    const uint32_t tok = tokens[p];
    const uint32_t lk = link[p];
    if ((int64_t)tok >= vocab) return;
    float* row = grad_embed + (int64_t)tok * hidden;
    const int64_t nslabs = (n4 + 63) / 64;
    if (lk != kNil) {
        // Not the owner.  Positions of a long group each offer to take a slab of columns; the rest leave.
        if (!vec || nslabs < 2) return;
        const uint4 e = tab[tok];
        if (e.y < kEmbLong || (int64_t)e.z >= nslabs) return;  // a stale z only costs the draw below
        emb_sum_slab(tokens, &tab[tok], dH, row, T, hidden, tok, e.y, list);
        return;
    }
    float4 old[kEmbVpl];
    if (vec) {
#pragma unroll
        for (int k = 0; k < kEmbVpl; k++) {
            const int64_t i = lane + 64 * k;
            old[k] = i < n4 ? reinterpret_cast<const float4*>(row)[i] : make_float4(0, 0, 0, 0);
        }
    }
    const uint4 e = tab[tok];
    const uint32_t count = e.y;
    if (vec && nslabs >= 2 && count >= kEmbLong) {             // a long group: the owner is one slab taker among the others
        emb_sum_slab(tokens, &tab[tok], dH, row, T, hidden, tok, count, list);
        return;
    }

    if (count == 1 && vec) {                                   // the common case: nothing to gather
#pragma unroll
        for (int k = 0; k < kEmbVpl; k++) {
            const int64_t i = lane + 64 * k;
            if (i < n4) reinterpret_cast<float4*>(row)[i] = make_float4(old[k].x + own[k].x, old[k].y + own[k].y, old[k].z + own[k].z, old[k].w + own[k].w);
        }
        for (int64_t i0 = 64 * kEmbVpl; i0 < n4; i0 += 64) {   // rows wider than one pass
            const int64_t i = i0 + lane;
            if (i < n4) {
                const float4 g = reinterpret_cast<const float4*>(dH + p * hidden)[i];
                float4 r = reinterpret_cast<float4*>(row)[i];
                r.x += g.x; r.y += g.y; r.z += g.z; r.w += g.w;
                reinterpret_cast<float4*>(row)[i] = r;
            }
        }
        return;
    }

    // The token's positions in ascending order, a batch of at most kEmbList at a time.  Short chains are walked (one
    // dependent load per position) and ranked; long ones are found by sweeping the token array from the smallest
    // position on, which costs T / count loads per position found.
    int64_t cursor = 0;                                        // scan: next token index to look at
    uint32_t found = 0;
    bool first_batch = true;
    while (found < count) {
        int len = 0;
        if (count <= (uint32_t)kEmbWalk) {
            if (lane == 0) {
                uint32_t q = e.x;
                for (uint32_t i = 0; i < count; i++) { tmp[i] = q; q = link[q]; }
            }
            __syncthreads();
            if (lane < (int)count) {
                const uint32_t mine = tmp[lane];
                int rank = 0;
                for (uint32_t j = 0; j < count; j++) rank += tmp[j] < mine ? 1 : 0;
                list[rank] = mine;
            }
            len = (int)count;
        } else {
            constexpr int U = 8;                               // token loads in flight per lane
            while (len + 64 * U <= kEmbList && cursor < T && found + (uint32_t)len < count) {
                uint32_t tk[U];
#pragma unroll
                for (int j = 0; j < U; j++) {
                    const int64_t q = cursor + 64 * j + lane;
                    tk[j] = q < T ? tokens[q] : kNil;          // kNil is no token (tok < vocab < 2^32 - 1)
                }
#pragma unroll
                for (int j = 0; j < U; j++) {
                    const bool hit = tk[j] == tok;
                    const unsigned long long mask = __ballot(hit);
                    if (hit) list[len + __popcll(mask & ((1ull << lane) - 1ull))] = (uint32_t)(cursor + 64 * j + lane);
                    len += __popcll(mask);
                }
                cursor += 64 * U;
            }
        }
        __syncthreads();
        found += (uint32_t)len;
        if (len == 0) break;                                   // cannot happen while the counts are consistent; never spin
        // add the batch's rows in list order, pass by pass over the row's width
        if (vec) {
            for (int64_t i0 = 0; i0 < n4; i0 += 64 * kEmbVpl) {
                float4 acc[kEmbVpl];
#pragma unroll
                for (int k = 0; k < kEmbVpl; k++) acc[k] = make_float4(0, 0, 0, 0);
                int m = 0;
                for (; m + 4 <= len; m += 4) {                 // four rows' loads in flight, added in list order
                    float4 g[4][kEmbVpl];
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        const float4* src = reinterpret_cast<const float4*>(dH + (int64_t)list[m + u] * hidden);
#pragma unroll
                        for (int k = 0; k < kEmbVpl; k++) {
                            const int64_t i = i0 + lane + 64 * k;
                            g[u][k] = i < n4 ? src[i] : make_float4(0, 0, 0, 0);
                        }
                    }
#pragma unroll
                    for (int u = 0; u < 4; u++)
#pragma unroll
                        for (int k = 0; k < kEmbVpl; k++) { acc[k].x += g[u][k].x; acc[k].y += g[u][k].y; acc[k].z += g[u][k].z; acc[k].w += g[u][k].w; }
                }
                for (; m < len; m++) {
                    const float4* src = reinterpret_cast<const float4*>(dH + (int64_t)list[m] * hidden);
#pragma unroll
                    for (int k = 0; k < kEmbVpl; k++) {
                        const int64_t i = i0 + lane + 64 * k;
                        if (i < n4) { const float4 g = src[i]; acc[k].x += g.x; acc[k].y += g.y; acc[k].z += g.z; acc[k].w += g.w; }
                    }
                }
#pragma unroll
                for (int k = 0; k < kEmbVpl; k++) {
                    const int64_t i = i0 + lane + 64 * k;
                    if (i < n4) {
                        float4 r = (first_batch && i0 == 0) ? old[k] : reinterpret_cast<float4*>(row)[i];
                        r.x += acc[k].x; r.y += acc[k].y; r.z += acc[k].z; r.w += acc[k].w;
                        reinterpret_cast<float4*>(row)[i] = r;
                    }
                }
            }
        } else {
            for (int64_t i = lane; i < hidden; i += 64) {
                float a = 0.0f;
                for (int m = 0; m < len; m++) a += dH[(int64_t)list[m] * hidden + i];
                row[i] += a;
            }
        }
        first_batch = false;
        __syncthreads();
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
    hipLaunchKernelGGL(emb_init_kernel, dim3((unsigned)ceil_div(vocab, 256)), dim3(256), 0, st, w.tab, vocab);
    SERAPH_LAUNCH_CHECK();
    hipLaunchKernelGGL(emb_link_kernel, dim3((unsigned)ceil_div(T, 256)), dim3(256), 0, st, tokens, w.tab, w.link, T, vocab);
    SERAPH_LAUNCH_CHECK();
    int vec = (hidden % 4 == 0) && aligned16(dH) && aligned16(grad_embed);
    hipLaunchKernelGGL(emb_sum_kernel, dim3((unsigned)T), dim3(64), 0, st, tokens, w.tab, w.link, dH, grad_embed, T, hidden, vocab, vec);
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // extern "C"
