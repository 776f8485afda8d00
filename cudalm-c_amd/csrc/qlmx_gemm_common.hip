/* qlmx_gemm_common.hip -- problem-table upload ring and argument checks of the grouped GEMMs. */
#include "qlmx_gemm.h"
#include <string.h>
#include <algorithm>

#define RING_SLOTS 64
static DevProb   *g_ring_h = nullptr, *g_ring_d = nullptr;
static hipEvent_t g_ring_ev[RING_SLOTS];
static bool       g_ring_used[RING_SLOTS];
static int        g_ring_next = 0;

static int ring_init(void){
    if(g_ring_h) return QLMX_OK;
    const size_t bytes = (size_t)RING_SLOTS * QLMX_MAX_PROBLEMS * sizeof(DevProb);
    QLMX_HIP(hipHostMalloc((void **)&g_ring_h, bytes, hipHostMallocDefault), "problem ring (pinned)");
    QLMX_HIP(hipMalloc((void **)&g_ring_d, bytes), "problem ring (device)");
    for(int i = 0; i < RING_SLOTS; i++){
        QLMX_HIP(hipEventCreateWithFlags(&g_ring_ev[i], hipEventDisableTiming), "problem ring event");
        g_ring_used[i] = false;
    }
    return QLMX_OK;
}

int qlmx_upload_problems(const qlmx_gemm_prob *probs, int nprob, int mode, int K, int N,
                         int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot_out){
    QLMX_REQUIRE(probs && nprob >= 0, "grouped gemm: NULL problem list");
    if(nprob > QLMX_MAX_PROBLEMS){
        qlmx_set_error("grouped gemm: %d problems exceed the limit of %d", nprob, QLMX_MAX_PROBLEMS);
        return QLMX_E_LIMIT;
    }
    int rc = ring_init(); if(rc) return rc;
    const int slot = g_ring_next; g_ring_next = (g_ring_next + 1) % RING_SLOTS;
    if(g_ring_used[slot]) QLMX_HIP(hipEventSynchronize(g_ring_ev[slot]), "problem ring wait");
    DevProb *h = g_ring_h + (size_t)slot * QLMX_MAX_PROBLEMS;
    DevProb *dv = g_ring_d + (size_t)slot * QLMX_MAX_PROBLEMS;
    const int tiles_n = (N + tile_cols - 1) / tile_cols;
    long long tiles = 0; int n = 0;
    /* Weight gradients: every problem has the same number of tiles but a cost proportional to its
     * row count, and the kernel gives table slot p to XCD p % 8 so that all tiles of an expert share
     * one L2. The slots are therefore filled heaviest first, dealt to the XCDs back and forth. */
    static int order[QLMX_MAX_PROBLEMS];
    int live = 0;
    for(int i = 0; i < nprob; i++) if(probs[i].M != 0) order[live++] = i;
    if(mode == GEMM_NT && live > 8){
        static int sorted[QLMX_MAX_PROBLEMS];
        memcpy(sorted, order, (size_t)live * sizeof(int));
        std::stable_sort(sorted, sorted + live, [&](int x, int y){ return probs[x].M > probs[y].M; });
        for(int i = 0; i < live; i++){
            const int grp = i >> 3, pos = i & 7, cnt = std::min(8, live - grp * 8);
            const int x = (cnt == 8 && (grp & 1)) ? 7 - pos : pos;
            order[grp * 8 + x] = sorted[i];
        }
    }
    for(int oi = 0; oi < live; oi++){
        const int i = order[oi];
        const qlmx_gemm_prob &p = probs[i];
        QLMX_REQUIRE(p.M >= 0, "grouped gemm: problem %d has M=%d", i, p.M);
        if(p.M == 0) continue;
        QLMX_REQUIRE(p.A && p.C, "grouped gemm: problem %d has a NULL operand", i);
        QLMX_REQUIRE(mode != GEMM_NT || p.B, "grouped gemm nt: problem %d has no B operand", i);
        QLMX_REQUIRE(p.beta == 0.0f || p.beta == 1.0f, "grouped gemm: beta must be 0 or 1");
        const int rows = mode == GEMM_NT ? K : p.M;
        DevProb &q = h[n++];
        q.A = p.A; q.B = p.B; q.C = p.C; q.wq = p.wq; q.wg = p.wg; q.M = p.M;
        q.beta = mode == GEMM_NN ? 0.0f : p.beta;
        q.tile0 = (int)tiles; q.tiles_n = tiles_n;
        tiles += (long long)((rows + tile_rows - 1) / tile_rows) * tiles_n;
        QLMX_REQUIRE(tiles < (1LL << 30), "grouped gemm: too many tiles");
    }
    if(n) QLMX_HIP(hipMemcpyAsync(dv, h, (size_t)n * sizeof(DevProb), hipMemcpyHostToDevice, stream), "problem table h2d");
    out->dev = dv; out->ntiles = (int)tiles; out->nprob = n;
    *slot_out = slot;
    return QLMX_OK;
}

int qlmx_upload_done(int slot, hipStream_t stream){
    QLMX_HIP(hipEventRecord(g_ring_ev[slot], stream), "problem ring record");
    g_ring_used[slot] = true;
    return QLMX_OK;
}
