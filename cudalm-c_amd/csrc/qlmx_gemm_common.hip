/* qlmx_gemm_common.hip -- problem-table rings and argument checks of the grouped GEMMs.
 *
 * The tables of a launch (problems, and for scheduled launches the unit table) are put together in
 * ordinary host memory and then written, with one streaming copy by the CPU, into a slot of a ring that
 * lies in DEVICE memory the host can write directly (fine-grained device memory, mapped through the PCIe
 * BAR; only where the device reports a large BAR, i.e. all of its memory host-visible). The writes are
 * write-combined, so a store fence follows them: the launch's doorbell is a later store of the same
 * thread and must not overtake them. No copy kernel or DMA stands in front of the launch (a 4 us copy kernel and its dependency cost 20 us of a 1 ms training
 * step), and the kernels' dependent table reads at the start of every tile cost a trip to local memory
 * or L2 (170-420 cycles measured) instead of one across PCIe to pinned host memory (1300). Where such
 * memory cannot be had the ring falls back to pinned host memory. A slot is handed out again only after
 * the host has waited for an event recorded behind the kernel that last read it. Because the slots are
 * rewritten, launches that use them must not be captured into a HIP graph. */
#include "qlmx_gemm.h"
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <algorithm>
#include <atomic>
#include <immintrin.h>

/* Reuse guard of a ring: an event behind every launch costs about 6 us of idle GPU between that kernel
 * and the next (the record makes the end of the kernel visible to the host), so the slots are guarded
 * by segments instead: when the ring moves on to the next segment, one event is recorded on each stream
 * the segment's launches went to, and those events are waited for when the ring comes round to the
 * segment's first slot again -- three segments' worth of launches later. Closing a segment on the way
 * out covers every launch made from it, also when a call that took its last slot returned without
 * launching (an error, or nothing but empty problems). */
#define GUARD_STREAMS 4
struct RingSeg { hipStream_t st[GUARD_STREAMS]; hipEvent_t ev[GUARD_STREAMS]; int nst, nrec; bool made; };
struct RingGuard { int nslots, per_seg, next; RingSeg seg[8]; };

static int guard_close(RingSeg &sg){
    sg.nrec = 0;
    for(int i = 0; i < sg.nst; i++){
        if(hipEventRecord(sg.ev[sg.nrec], sg.st[i]) == hipSuccess) sg.nrec++;
        else {
            /* e.g. a stream destroyed since its launch: fall back to waiting for the whole device */
            (void)hipGetLastError();
            QLMX_HIP(hipDeviceSynchronize(), "table ring device wait");
        }
    }
    sg.nst = 0;
    return QLMX_OK;
}
static int guard_take(RingGuard &g, int *slot_out){
    const int slot = g.next; g.next = (g.next + 1) % g.nslots;
    if(slot % g.per_seg == 0){
        const int nseg = g.nslots / g.per_seg, cur = slot / g.per_seg;
        /* a launch held back for a pair owns a slot of the segment that is closed here: issue it first, so
         * that the segment's events come after it */
        int rc = qlmx_pair_flush(); if(rc) return rc;
        rc = guard_close(g.seg[(cur + nseg - 1) % nseg]); if(rc) return rc;
        RingSeg &sg = g.seg[cur];
        for(int i = 0; i < sg.nrec; i++) QLMX_HIP(hipEventSynchronize(sg.ev[i]), "table ring wait");
        sg.nrec = 0;
    }
    *slot_out = slot;
    return QLMX_OK;
}
static int guard_launched(RingGuard &g, int slot, hipStream_t stream){
    RingSeg &sg = g.seg[slot / g.per_seg];
    if(!sg.made){
        for(int i = 0; i < GUARD_STREAMS; i++) QLMX_HIP(hipEventCreateWithFlags(&sg.ev[i], hipEventDisableTiming), "table ring event");
        sg.made = true;
    }
    int k = 0;
    while(k < sg.nst && sg.st[k] != stream) k++;
    if(k == sg.nst){
        if(sg.nst == GUARD_STREAMS){
            /* more streams than events in one segment: wait for this one now */
            QLMX_HIP(hipStreamSynchronize(stream), "table ring stream wait");
            return QLMX_OK;
        }
        sg.st[sg.nst++] = stream;
    }
    return QLMX_OK;
}

/* Table memory the host writes and the kernels read: device memory mapped into the host's address space,
 * else pinned host memory. Never read back by the host (reads across the BAR are slow) and never freed. */
static int table_alloc(void **p, size_t bytes, const char *what){
    int dev = 0, large_bar = 0;
    if(hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&large_bar, hipDeviceAttributeIsLargeBar, dev) != hipSuccess) large_bar = 0;
    (void)hipGetLastError();
    const bool say = getenv("QLMX_VERBOSE") != nullptr;
    if(large_bar && hipExtMallocWithFlags(p, bytes, hipDeviceMallocFinegrained) == hipSuccess && *p){
        if(say) fprintf(stderr, "[qlmx] %s: %zu bytes of host-writable device memory\n", what, bytes);
        return QLMX_OK;
    }
    (void)hipGetLastError();
    QLMX_HIP(hipHostMalloc(p, bytes, hipHostMallocDefault), what);
    if(say) fprintf(stderr, "[qlmx] %s: %zu bytes of pinned host memory (large BAR: %d)\n", what, bytes, large_bar);
    return QLMX_OK;
}
/* Everything written into a table so far is on its way to the device before anything the thread stores next
 * (the queue's doorbell): sfence drains the write-combining buffers, the thread fence keeps the compiler
 * from moving the copies past it. */
static inline void table_publish(void){
    std::atomic_thread_fence(std::memory_order_seq_cst);
    _mm_sfence();
}

#define RING_SLOTS 64
static DevProb   *g_ring_h = nullptr;
static RingGuard  g_ring_guard = {RING_SLOTS, 16, 0, {}};

static int ring_init(void){
    if(g_ring_h) return QLMX_OK;
    const size_t bytes = (size_t)RING_SLOTS * QLMX_MAX_PROBLEMS * sizeof(DevProb);
    return table_alloc((void **)&g_ring_h, bytes, "problem ring");
}

/* `second` (else NULL): problem i has a second half. tn: it continues its contraction over second[i].A
 * and the weight matrix at second[i].wq / wg. nn: its tiles hold columns of two weight matrices, the
 * second at second[i].wq / wg with its output at second[i].C and the combined output at second[i].B.
 * Such a problem is followed in the table by an entry that carries the second half's fields and owns
 * no tile (its tile0 is the next problem's), and has `chunk` set to 1. */
static int upload_problems(const qlmx_gemm_prob *probs, const qlmx_gemm_prob *second, int nprob, int mode, int K, int N,
                           int tile_rows, int tile_cols, const RowBytes *rb, hipStream_t stream, ProbUpload *out, int *slot_out){
    QLMX_REQUIRE(probs && nprob >= 0, "grouped gemm: NULL problem list");
    const int per = (second ? 2 : 1) * (rb ? 2 : 1);                 /* table entries a problem may take */
    if(nprob * per > QLMX_MAX_PROBLEMS){
        qlmx_set_error("grouped gemm: %d problems exceed the limit of %d", nprob, QLMX_MAX_PROBLEMS / per);
        return QLMX_E_LIMIT;
    }
    int rc = ring_init(); if(rc) return rc;
    int slot; rc = guard_take(g_ring_guard, &slot); if(rc) return rc;
    static DevProb stage[QLMX_MAX_PROBLEMS];                 /* built here, copied to the slot in one go */
    DevProb *h = stage;
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
        QLMX_REQUIRE(p.A && (p.C || (second && mode == GEMM_NN)), "grouped gemm: problem %d has a NULL operand", i);
        QLMX_REQUIRE(mode != GEMM_NT || p.B, "grouped gemm nt: problem %d has no B operand", i);
        QLMX_REQUIRE(p.beta == 0.0f || p.beta == 1.0f, "grouped gemm: beta must be 0 or 1");
        if(second){
            const qlmx_gemm_prob &p2 = second[i];
            QLMX_REQUIRE(p2.M == p.M, "grouped gemm: problem %d and its second half differ in rows (%d, %d)", i, p.M, p2.M);
            QLMX_REQUIRE(mode == GEMM_TN ? p2.A != nullptr : (p2.B != nullptr && (p2.C != nullptr) == (p.C != nullptr)), "grouped gemm: the second half of problem %d lacks a pointer", i);
        }
    }
    /* One table entry (two for a problem with a second half) covering rows [r0, r0 + m) of problem i. */
    auto emit = [&](int i, int r0, int m){
        const qlmx_gemm_prob &p = probs[i];
        const int rows = mode == GEMM_NT ? K : m;
        auto adv = [&](const void *ptr, size_t row_bytes) -> const void * { return (ptr && r0) ? (const void *)((const char *)ptr + (size_t)r0 * row_bytes) : ptr; };
        DevProb &q = h[n++];
        q.A = adv(p.A, rb ? rb->a : 0); q.B = p.B; q.C = (float *)adv(p.C, rb ? rb->c : 0); q.wq = p.wq; q.wg = p.wg; q.M = m;
        q.beta = mode == GEMM_NN ? 0.0f : p.beta;
        q.tile0 = (int)tiles; q.tiles_n = tiles_n; q.chunk = second ? 1 : 0; q.flag0 = 0;
        tiles += (long long)((rows + tile_rows - 1) / tile_rows) * tiles_n;
        if(second){
            const qlmx_gemm_prob &p2 = second[i];
            DevProb &c = h[n++];
            c = q; c.A = adv(p2.A, rb ? rb->a2 : 0); c.B = adv(p2.B, rb ? rb->b2 : 0); c.C = (float *)adv(p2.C, rb ? rb->c2 : 0);
            c.wq = p2.wq; c.wg = p2.wg; c.tile0 = (int)tiles; c.chunk = 0;
        }
    };
    int nfull = 0;
    if(rb){
        /* Longest tiles first: a launch ends when its last workgroup does, workgroups start in table order, and
         * under a skewed load a full-height tile handed out at the very end leaves most of the device waiting for
         * it. Every problem is therefore entered twice: its whole row tiles in the first part of the table (in the
         * caller's order, so that an expert's tiles stay together), its ragged last row tile in the second part,
         * tallest first. Rows are independent in these products, so a part is a problem of its own whose row
         * pointers start further down. */
        for(int oi = 0; oi < live; oi++){ const int i = order[oi], full = probs[i].M / tile_rows * tile_rows; if(full) emit(i, 0, full); }
        QLMX_REQUIRE(tiles < (1LL << 30), "grouped gemm: too many tiles");
        nfull = (int)tiles;
        static int tails[QLMX_MAX_PROBLEMS];
        int nt = 0;
        for(int oi = 0; oi < live; oi++) if(probs[order[oi]].M % tile_rows) tails[nt++] = order[oi];
        std::stable_sort(tails, tails + nt, [&](int x, int y){ return probs[x].M % tile_rows > probs[y].M % tile_rows; });
        for(int k = 0; k < nt; k++){ const int i = tails[k], full = probs[i].M / tile_rows * tile_rows; emit(i, full, probs[i].M - full); }
    } else {
        for(int oi = 0; oi < live; oi++) emit(order[oi], 0, probs[order[oi]].M);
        nfull = (int)tiles;
    }
    QLMX_REQUIRE(tiles < (1LL << 30), "grouped gemm: too many tiles");
    (void)stream;
    DevProb *dst = g_ring_h + (size_t)slot * QLMX_MAX_PROBLEMS;
    memcpy(dst, stage, (size_t)n * sizeof(DevProb));
    table_publish();
    out->dev = dst; out->ntiles = (int)tiles; out->nprob = n; out->nfull = nfull;
    *slot_out = slot;
    return QLMX_OK;
}

int qlmx_upload_problems(const qlmx_gemm_prob *probs, int nprob, int mode, int K, int N,
                         int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot_out){
    return upload_problems(probs, nullptr, nprob, mode, K, N, tile_rows, tile_cols, nullptr, stream, out, slot_out);
}
int qlmx_upload_problem_pairs(const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int mode, int K, int N,
                              int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot_out){
    QLMX_REQUIRE(second && (mode == GEMM_TN || mode == GEMM_NN), "grouped gemm: NULL list of second halves");
    return upload_problems(first, second, nprob, mode, K, N, tile_rows, tile_cols, nullptr, stream, out, slot_out);
}
int qlmx_upload_problems_split(const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int mode, int K, int N,
                               int tile_rows, int tile_cols, const RowBytes *rb, hipStream_t stream, ProbUpload *out, int *slot_out){
    QLMX_REQUIRE(rb && (mode == GEMM_TN || mode == GEMM_NN), "grouped gemm: row sizes are needed to split problems");
    return upload_problems(first, second, nprob, mode, K, N, tile_rows, tile_cols, rb, stream, out, slot_out);
}

int qlmx_upload_done(int slot, hipStream_t stream){ return guard_launched(g_ring_guard, slot, stream); }

/* ---- unit tables of scheduled launches: a ring of pinned slots like the one above, each holding a
 * problem table and a unit table; chain flags handed out round the ring of a fixed array
 * (a launch's flags carry its epoch, so nothing is ever cleared). ---- */
#define UNIT_SLOTS 32
/* A launch takes at most CHAIN_MAX_PER_LAUNCH flags from a cursor that wraps; a unit-ring slot is only handed out
 * again after its launch has finished, so at most UNIT_SLOTS launches are in flight and the array holds all of
 * their flags plus the stretch a wrap may skip: flags of two live launches never overlap. */
#define CHAIN_MAX_PER_LAUNCH (1 << 16)
#define CHAIN_FLAGS ((UNIT_SLOTS + 1) * CHAIN_MAX_PER_LAUNCH)
static char      *g_unit_h = nullptr;
static RingGuard  g_unit_guard = {UNIT_SLOTS, 8, 0, {}};
static int       *g_chain_flags = nullptr;
static unsigned  *g_chain_status = nullptr;      /* pinned: a kernel whose wait ran out sets it */
static int        g_chain_cursor = 0;
static unsigned   g_chain_epoch = 0;
static const size_t UNIT_SLOT_BYTES = (size_t)QLMX_MAX_PROBLEMS * sizeof(DevProb) + (size_t)QLMX_MAX_UNITS * sizeof(DevUnit);

/* the unit table follows the problem table */
static size_t unit_offset(int nprob){ return ((size_t)nprob * sizeof(DevProb) + 63) & ~(size_t)63; }

static int unit_init(void){
    if(g_unit_h) return QLMX_OK;
    { int rc = table_alloc((void **)&g_unit_h, UNIT_SLOTS * UNIT_SLOT_BYTES, "unit ring"); if(rc) return rc; }
    QLMX_HIP(hipMalloc((void **)&g_chain_flags, CHAIN_FLAGS * sizeof(int)), "chain flags");
    QLMX_HIP(hipMemset(g_chain_flags, 0, CHAIN_FLAGS * sizeof(int)), "chain flags clear");
    QLMX_HIP(hipHostMalloc((void **)&g_chain_status, sizeof(unsigned), hipHostMallocDefault), "chain status (pinned)");
    *g_chain_status = 0;
    return QLMX_OK;
}

int qlmx_unit_slot(int nprob, UnitUpload *out, int *slot_out){
    int rc = unit_init(); if(rc) return rc;
    if(*(volatile unsigned *)g_chain_status){
        *g_chain_status = 0;                      /* reported once, by this call */
        qlmx_set_error("grouped gemm: an earlier launch gave up waiting for a partial sum of a split contraction; its output is incomplete");
        return QLMX_E_HIP;
    }
    int slot; rc = guard_take(g_unit_guard, &slot); if(rc) return rc;
    /* the caller fills the staging copy and calls qlmx_unit_commit before it launches */
    static char stage[UNIT_SLOT_BYTES];
    char *h = g_unit_h + slot * UNIT_SLOT_BYTES;
    const size_t uoff = unit_offset(nprob);
    out->hprob = (DevProb *)stage; out->hunit = (DevUnit *)(stage + uoff);
    out->dprob = (const DevProb *)h; out->dunit = (const DevUnit *)(h + uoff);
    out->flags = g_chain_flags; out->status = g_chain_status;
    *slot_out = slot;
    return QLMX_OK;
}

void qlmx_unit_commit(const UnitUpload *u, int nprob, int nunits){
    const size_t uoff = unit_offset(nprob);
    memcpy((void *)u->dprob, u->hprob, (size_t)nprob * sizeof(DevProb));
    memcpy((void *)u->dunit, u->hunit, (size_t)nunits * sizeof(DevUnit));
    table_publish();
    (void)uoff;
}
int qlmx_unit_done(int slot, hipStream_t stream){ return guard_launched(g_unit_guard, slot, stream); }

int qlmx_chain_reserve(int nflags, int *first, unsigned *epoch){
    QLMX_REQUIRE(nflags <= CHAIN_MAX_PER_LAUNCH, "grouped gemm: %d chained tiles in one launch", nflags);
    if(g_chain_cursor + nflags > CHAIN_FLAGS) g_chain_cursor = 0;
    *first = g_chain_cursor; g_chain_cursor += nflags;
    g_chain_epoch = (g_chain_epoch + 1) & 0x0FFFFFFFu;
    *epoch = g_chain_epoch;
    return QLMX_OK;
}

/* ---- time-out tests: the host arms a one-shot switch; the next launch of that kind then waits, for a single
 * poll, for a hand-over tag that nobody publishes, so every one of its waits gives up, every workgroup still runs to
 * its end, the output is wrong and the status word is set -- exactly what a real time-out leaves behind. ---- */
static bool g_forced[3] = {false, false, false};
bool qlmx_test_take_forced_timeout(int which){
    if(which < 1 || which > 2 || !g_forced[which]) return false;
    g_forced[which] = false;
    return true;
}
extern "C" int qlmx_test_force_wait_timeout(int which){
    QLMX_REQUIRE(which == 1 || which == 2, "qlmx_test_force_wait_timeout: 1 = decode layer, 2 = split weight-gradient contraction");
    g_forced[which] = true;
    return QLMX_OK;
}
