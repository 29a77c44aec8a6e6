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
#include <atomic>
#include <mutex>

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

// One entry per token.  Every word carries the call's epoch in its upper half: an entry whose epoch is not the
// current call's is an empty entry, so no launch has to clear the table between calls.
struct EmbEntry {
    unsigned long long head;     // epoch | most recent position that joined the token's chain
    unsigned long long count;    // epoch | positions so far
    unsigned long long slabs;    // epoch | column slabs of a long group handed out so far
    unsigned long long unused;
};
__device__ __forceinline__ uint32_t emb_value(unsigned long long word, uint32_t epoch, uint32_t empty) {
    return (uint32_t)(word >> 32) == epoch ? (uint32_t)word : empty;
}
// value += 1 under the epoch; returns the value before (0 for a word of another epoch)
__device__ __forceinline__ uint32_t emb_bump(unsigned long long* word, uint32_t epoch) {
    unsigned long long seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    for (;;) {
        const uint32_t before = emb_value(seen, epoch, 0u);
        const unsigned long long want = ((unsigned long long)epoch << 32) | (before + 1u);
        const unsigned long long got = atomicCAS(word, seen, want);
        if (got == seen) return before;
        seen = got;
    }
}

// Tables kept by the library (zero at load: epoch 0 is never used), one per call in rotation, so that a call finds
// a table without clearing one.  Vocabularies beyond their size use a table in the caller's scratch that is cleared
// first.  More than kEmbTables calls in flight on one device at a time would share a table: not supported.
constexpr int64_t kEmbLibVocab = 1 << 18;
constexpr int kEmbTables = 4;
static __device__ EmbEntry g_emb_tables[kEmbTables][kEmbLibVocab];

static size_t align_up(size_t x) { return (x + 255) & ~(size_t)255; }

struct EmbWs {
    uint32_t* link;     // [T]      the position that had joined the same token's chain before this one; kNil for the first
    EmbEntry* tab;      // [vocab]  only for vocabularies beyond kEmbLibVocab
};
static size_t emb_ws_layout(int64_t T, int64_t vocab, char* base, EmbWs* w) {
    size_t o = 0;
    char* link = base + o; o += align_up((size_t)T * 4);
    char* tab = base + o;
    if (vocab > kEmbLibVocab) o += align_up((size_t)vocab * sizeof(EmbEntry));
    if (w) { w->link = (uint32_t*)link; w->tab = vocab > kEmbLibVocab ? (EmbEntry*)tab : nullptr; }
    return o;
}

__global__ __launch_bounds__(256) void emb_init_kernel(EmbEntry* __restrict__ tab, int64_t vocab) {
    const int64_t v = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (v < vocab) { tab[v].head = 0ull; tab[v].count = 0ull; tab[v].slabs = 0ull; tab[v].unused = 0ull; }
}

__global__ __launch_bounds__(256) void emb_link_kernel(const uint32_t* __restrict__ tokens, EmbEntry* tab, uint32_t* __restrict__ link,
                                                       int64_t T, int64_t vocab, uint32_t epoch) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= T) return;
    const uint32_t tok = tokens[p];
    if ((int64_t)tok >= vocab) { link[p] = 0u; return; }      // skipped position (embedding_backward.comp:31): owns nothing (its token is checked again)
    emb_bump(&tab[tok].count, epoch);
    const unsigned long long before = atomicExch(&tab[tok].head, ((unsigned long long)epoch << 32) | (uint32_t)p);
    link[p] = emb_value(before, epoch, kNil);
}

// One wavefront per position; only a token's owner (the position whose exchange found the chain empty) works.
// The owner's own row of dH is requested before anything is known about the token, the table row as soon as the
// token is: for a token that occurs once, which is most of them, two dependent loads precede the payload.  The
// kernel is held to 80 registers a lane (six wavefronts per SIMD): it lives on the number of rows in flight.
constexpr int kEmbList = 1024;          // positions gathered per batch
constexpr int kEmbWalk = 16;            // below this many positions the chain is walked and one wavefront adds the rows;
                                        // from it on the group is cut into column slabs (rows of more than one slab)
constexpr int kEmbAhead = 16;           // rows in flight per slab wavefront
constexpr int kEmbGatherVpl = 4;        // float4 per lane and pass where one wavefront adds the rows of a short chain

// Gathers the next batch of the token's positions (ascending) into `list` by sweeping the token array from `cursor`.
__device__ __forceinline__ int emb_scan(const uint32_t* __restrict__ tokens, int64_t T, uint32_t tok, uint32_t wanted,
                                        int64_t& cursor, uint32_t* list) {
    constexpr int U = 8;                                       // token loads in flight per lane
    const int lane = threadIdx.x;
    int len = 0;
    while (len + 64 * U <= kEmbList && cursor < T && (uint32_t)len < wanted) {
        uint32_t tk[U];
#pragma unroll
        for (int j = 0; j < U; j++) {
            const int64_t q = cursor + 64 * j + lane;
            tk[j] = q < T ? tokens[q] : kNil;                  // kNil is no token (tok < vocab < 2^32 - 1)
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
    return len;
}

// Column slabs (64 float4 slots of the row's width) of a long group: draw a slab number until all are taken; for each,
// sweep the token array for the group's positions (ascending by construction) a batch at a time and add the slab's part
// of their rows in that order, kEmbAhead rows' loads in flight; one read-modify-write of the slab's part of the table row.
__device__ __forceinline__ void emb_sum_slabs(const uint32_t* __restrict__ tokens, EmbEntry* entry, uint32_t epoch,
                                              const float* __restrict__ dH, float* row, int64_t T, int64_t hidden,
                                              uint32_t tok, uint32_t count, uint32_t* list) {
    const int lane = threadIdx.x;
    const int64_t n4 = hidden >> 2, nslabs = (n4 + 63) / 64;
    for (;;) {
        uint32_t slab = 0;
        if (lane == 0) slab = emb_bump(&entry->slabs, epoch);
        slab = __shfl(slab, 0, 64);
        if ((int64_t)slab >= nslabs) return;
        const int64_t i4 = (int64_t)slab * 64 + lane;
        const bool ok = i4 < n4;
        float4 acc = make_float4(0, 0, 0, 0);
        int64_t cursor = 0;
        uint32_t found = 0;
        while (found < count && cursor < T) {
            const int len = emb_scan(tokens, T, tok, count - found, cursor, list);
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
}

// VPL float4 per lane make the first pass over a row; EXACT: the row holds at least that many and the pass needs no
// test against its end (the tests cost 8 us of 66 at 16384 x 2048: the loads of a pass no longer issue back to back).
// Streamed (nontemporal) accesses for the row read-modify-write were measured and are not used: with table rows that no
// earlier call left in the last-level cache they change nothing (87.5 against 87.2 us at 16384 x 2048 into 151936 rows),
// with rows that are still there they lose them (87.1 against 69.6 us).
template <int VPL, bool EXACT>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 8)))
void emb_sum_kernel(const uint32_t* __restrict__ tokens, EmbEntry* tab, const uint32_t* __restrict__ link,
                    const float* __restrict__ dH, float* __restrict__ grad_embed,
                    int64_t T, int64_t hidden, int64_t vocab, uint32_t epoch, int vec) {
    __shared__ uint32_t list[kEmbList], tmp[kEmbWalk];
    const int lane = threadIdx.x;
    const int64_t p = blockIdx.x;
    const int64_t n4 = hidden >> 2;
    // speculative: the first pass of this position's own row
    float4 own[VPL];
    if (vec) {
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const int64_t i = lane + 64 * k;
            own[k] = (EXACT || i < n4) ? reinterpret_cast<const float4*>(dH + p * hidden)[i] : make_float4(0, 0, 0, 0);
        }
    }
    const uint32_t tok = tokens[p];
    const uint32_t lk = link[p];
    if ((int64_t)tok >= vocab) return;
    float* row = grad_embed + (int64_t)tok * hidden;
    const int64_t nslabs = (n4 + 63) / 64;
    const bool slabs_ok = vec && nslabs >= 2;
    if (lk != kNil) {
        // Not the owner.  Positions of a long group each offer to take slabs of columns; the rest leave.
        if (!slabs_ok) return;
        const uint32_t count = emb_value(tab[tok].count, epoch, 0u);
        if (count < (uint32_t)kEmbWalk || (int64_t)emb_value(tab[tok].slabs, epoch, 0u) >= nslabs) return;  // a stale slab count only costs a draw
        emb_sum_slabs(tokens, &tab[tok], epoch, dH, row, T, hidden, tok, count, list);
        return;
    }
    float4 old[VPL];
    if (vec) {
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const int64_t i = lane + 64 * k;
            old[k] = (EXACT || i < n4) ? reinterpret_cast<const float4*>(row)[i] : make_float4(0, 0, 0, 0);
        }
    }
    const uint32_t count = emb_value(tab[tok].count, epoch, 0u);
    const uint32_t head = emb_value(tab[tok].head, epoch, kNil);
    if (slabs_ok && count >= (uint32_t)kEmbWalk) {             // a long group: the owner is one slab taker among the others
        emb_sum_slabs(tokens, &tab[tok], epoch, dH, row, T, hidden, tok, count, list);
        return;
    }

    if (count == 1 && vec) {                                   // the common case: nothing to gather
#pragma unroll
        for (int k = 0; k < VPL; k++) {
            const int64_t i = lane + 64 * k;
            if (EXACT || i < n4) reinterpret_cast<float4*>(row)[i] = make_float4(old[k].x + own[k].x, old[k].y + own[k].y, old[k].z + own[k].z, old[k].w + own[k].w);
        }
        for (int64_t i0 = 64 * VPL; i0 < n4; i0 += 64) {       // what the first pass left of the row
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
    // dependent load per position) and ranked; long ones (only rows of a single slab, or unaligned ones, get here
    // with a long chain) are found by sweeping the token array from the smallest position on.
    int64_t cursor = 0;                                        // scan: next token index to look at
    uint32_t found = 0;
    while (found < count) {
        int len = 0;
        if (count < (uint32_t)kEmbWalk) {
            if (lane == 0) {
                uint32_t q = head;
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
            len = emb_scan(tokens, T, tok, count - found, cursor, list);
        }
        __syncthreads();
        found += (uint32_t)len;
        if (len == 0) break;                                   // cannot happen while the counts are consistent; never spin
        // add the batch's rows in list order, pass by pass over the row's width
        if (vec) {
            for (int64_t i0 = 0; i0 < n4; i0 += 64 * kEmbGatherVpl) {
                float4 acc[kEmbGatherVpl];
#pragma unroll
                for (int k = 0; k < kEmbGatherVpl; k++) acc[k] = make_float4(0, 0, 0, 0);
                int m = 0;
                float4 g[kEmbGatherVpl];
                auto fetch = [&](int at) {
                    const float4* src = reinterpret_cast<const float4*>(dH + (int64_t)list[at] * hidden);
#pragma unroll
                    for (int k = 0; k < kEmbGatherVpl; k++) {
                        const int64_t i = i0 + lane + 64 * k;
                        g[k] = i < n4 ? src[i] : make_float4(0, 0, 0, 0);
                    }
                };
                for (; m < len; m++) {
                    fetch(m);
#pragma unroll
                    for (int k = 0; k < kEmbGatherVpl; k++) { acc[k].x += g[k].x; acc[k].y += g[k].y; acc[k].z += g[k].z; acc[k].w += g[k].w; }
                }
#pragma unroll
                for (int k = 0; k < kEmbGatherVpl; k++) {
                    const int64_t i = i0 + lane + 64 * k;
                    if (i < n4) {
                        float4 r = reinterpret_cast<float4*>(row)[i];   // (requested once before for a single position: a cache hit)
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
        __syncthreads();
    }
}

// device address of the library's tables on the current device
static int emb_tables(EmbEntry** out, int* device) {
    static std::mutex mu;
    static EmbEntry* base[64] = {nullptr};
    int dev = 0;
    SERAPH_HIP_CHECK(hipGetDevice(&dev));
    SERAPH_REQUIRE(dev >= 0 && dev < 64, "device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lk(mu);
    if (!base[dev]) SERAPH_HIP_CHECK(hipGetSymbolAddress((void**)&base[dev], HIP_SYMBOL(g_emb_tables)));
    *out = base[dev];
    *device = dev;
    return SERAPH_OK;
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
    // The epoch of a call: 1 ... 2^32 - 1, then around again (0 is the epoch of an entry that was never written).
    static std::atomic<uint64_t> calls{0};
    const uint64_t call = calls.fetch_add(1);
    const uint32_t epoch = (uint32_t)(call % 0xffffffffull) + 1u;
    const uint64_t era = call / 0xffffffffull;
    EmbEntry* tab = w.tab;
    bool clear = true;
    if (!tab) {
        // The library's tables are cleared only when the epochs start over: an entry left untouched since the same
        // epoch of the era before would look current.
        int dev = 0;
        int rc = emb_tables(&tab, &dev);
        if (rc != SERAPH_OK) return rc;
        const int slot = (int)(call % kEmbTables);
        tab += (size_t)slot * kEmbLibVocab;
        static std::mutex mu;
        static uint64_t cleared_in_era[64][kEmbTables];
        std::lock_guard<std::mutex> lk(mu);
        clear = cleared_in_era[dev][slot] != era;
        cleared_in_era[dev][slot] = era;
    }
    if (clear) {
        const int64_t entries = w.tab ? vocab : kEmbLibVocab;
        hipLaunchKernelGGL(emb_init_kernel, dim3((unsigned)ceil_div(entries, 256)), dim3(256), 0, st, tab, entries);
        SERAPH_LAUNCH_CHECK();
    }
    hipLaunchKernelGGL(emb_link_kernel, dim3((unsigned)ceil_div(T, 256)), dim3(256), 0, st, tokens, tab, w.link, T, vocab, epoch);
    SERAPH_LAUNCH_CHECK();
    int vec = (hidden % 4 == 0) && aligned16(dH) && aligned16(grad_embed);
    // first pass over a row: as many float4 per lane as fit it exactly, up to 8 (2048 floats)
    const int64_t whole = vec && hidden % 256 == 0 ? hidden / 256 : 0;
#define SUM(VPL, EXACT) \
    hipLaunchKernelGGL((emb_sum_kernel<VPL, EXACT>), dim3((unsigned)T), dim3(64), 0, st, tokens, tab, w.link, dH, grad_embed, T, hidden, vocab, epoch, vec)
    if (whole >= 8) SUM(8, true);
    else if (whole >= 4) SUM(4, true);
    else if (whole >= 2) SUM(2, true);
    else if (whole >= 1) SUM(1, true);
    else SUM(8, false);
#undef SUM
    SERAPH_LAUNCH_CHECK();
    return SERAPH_OK;
}

}  // extern "C"
