/* qlmx_gemm_nt_lds.hip -- launch side of the weight-gradient grouped GEMM (nt) for bf16 operands; the kernel
 * body is in qlmx_gemm_nt_body.h (mg_atb, cudalm.cu:3204-3256; call sites 4334-4366). */
#include "qlmx_gemm_nt_body.h"
#include <algorithm>
#include <stdlib.h>

template<int BN, int NW>
__global__ void __launch_bounds__(NW * 64, (Nt3Shape<BN, NW>::WG_PER_CU)) k_gemm_nt_lds(Nt3Args a){
    nt3_block<BN, NW>(a, blockIdx.x);
}

static void *g_nt3_zeros = nullptr;

/* Lays out a scheduled launch. Every live problem owns T = tile rows x tile columns output tiles whose
 * cost is its row count, so a Zipf-loaded layer has a few tiles that outlast all others: contractions
 * longer than about the mean load of a workgroup slot are cut into slices that add up through a
 * chain. Groups (problem, tile row) -- the tiles that share the activation slab -- are dealt to the
 * XCDs heaviest first, each to the XCD with the least work so far. A table entry stands for the g
 * column tiles of one (problem, tile row, slice); XCD x runs its entries in order, g workgroups each.
 * Returns the grid size, or 0 when the launch does not fit the table. */
struct Nt3Group { int prob, ti, cost; };
/* whole problems up to num/den of an XCD's share (QLMX_NT_WHOLE = num, 0 = never). Config-3 step, reads of the two
 * weight-gradient launches by FETCH_SIZE and their times: never 278 + 436 MiB, 77.7 + 140.6 us; 2/4 185 + 312 MiB,
 * 82.6 + 137.8; 3/4 159 + 292 MiB, 75.1 + 136.2; 4/4 the same as 3/4 (no expert lies between). */
static int g_nt3_whole_num = -1, g_nt3_whole_den = 4;
static int nt3_schedule(DevProb *pr, int n, int K, int N, int BN, int slots_per_cu, int cus, DevUnit *units, int *nflags_out, int *nent_out){
    if(g_nt3_whole_num < 0){ const char *e = getenv("QLMX_NT_WHOLE"); g_nt3_whole_num = e ? atoi(e) : 3; }
    const int g = N / BN, rp = (K + NT3_BM - 1) / NT3_BM;
    if(rp > 64) return 0;                                              /* the packed entry has 6 bits for the tile row */
    long long work = 0;
    for(int p = 0; p < n; p++) work += (long long)pr[p].M * rp * g;
    const long long slots = (long long)slots_per_cu * cus;
    long long mean = (work + slots - 1) / slots;                       /* rows of contraction per workgroup slot */
    if(mean < 256) mean = 256;
    static int nchunk[QLMX_MAX_PROBLEMS], chunk[QLMX_MAX_PROBLEMS];
    long long nunits = 0;
    for(int p = 0; p < n; p++){
        int nc = 1;
        if(pr[p].M > mean + mean / 4){ nc = (int)((pr[p].M + mean - 1) / mean); if(nc > 15) nc = 15; }
        chunk[p] = ((pr[p].M + nc - 1) / nc + NT3_BK - 1) / NT3_BK * NT3_BK;
        nc = (pr[p].M + chunk[p] - 1) / chunk[p];                       /* rounding the slice up can make the last one empty */
        nchunk[p] = nc;
        nunits += (long long)nc * rp;
    }
    if(nunits + 8LL * 15 > QLMX_MAX_UNITS) return 0;
    /* A problem whose whole cost is at most `whole` of an XCD's share stays on one XCD with all its tile rows
     * (ti = -1): they read the same rows of dY, which then come from HBM once instead of once per tile row. */
    static Nt3Group groups[QLMX_MAX_UNITS];
    int ng = 0;
    const long long share = (work + 7) / 8;
    for(int p = 0; p < n; p++){
        if(rp > 1 && (long long)pr[p].M * rp * g * g_nt3_whole_den <= share * g_nt3_whole_num) groups[ng++] = {p, -1, pr[p].M * rp};
        else for(int ti = 0; ti < rp; ti++) groups[ng++] = {p, ti, pr[p].M};
    }
    std::stable_sort(groups, groups + ng, [](const Nt3Group &x, const Nt3Group &y){ return x.cost > y.cost; });
    static int gx[QLMX_MAX_UNITS];
    long long load[8] = {0, 0, 0, 0, 0, 0, 0, 0}; int len[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for(int i = 0; i < ng; i++){
        int x = 0;
        for(int y = 1; y < 8; y++) if(load[y] < load[x]) x = y;
        gx[i] = x; load[x] += (long long)groups[i].cost * g; len[x] += nchunk[groups[i].prob] * (groups[i].ti < 0 ? rp : 1);
    }
    int longest = 0;
    for(int x = 0; x < 8; x++) if(len[x] > longest) longest = len[x];
    const int nent = 8 * longest;                                      /* table entries; each stands for g workgroups */
    if(nent > QLMX_MAX_UNITS || (long long)nent * g >= (1LL << 30)) return 0;
    for(int b = 0; b < nent; b++) units[b] = QX_UNIT_NONE;
    int nflags = 0;
    for(int p = 0; p < n; p++){
        pr[p].chunk = chunk[p]; pr[p].flag0 = nflags;
        if(nchunk[p] > 1) nflags += rp * g;
    }
    int pos[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for(int i = 0; i < ng; i++){
        const int p = groups[i].prob, x = gx[i], nc = nchunk[p];
        const int t0 = groups[i].ti < 0 ? 0 : groups[i].ti, t1 = groups[i].ti < 0 ? rp : groups[i].ti + 1;
        for(int c = 0; c < nc; c++)                                   /* a slice's tile rows side by side: they share its rows of dY */
            for(int ti = t0; ti < t1; ti++) units[8 * pos[x]++ + x] = QX_UNIT(p, ti, 0, c, nc);
    }
    *nflags_out = nflags;
    *nent_out = nent;
    return nent * g;
}

template<int BN, int NW> static int nt3_launch(const Nt3Args &a, int grid, hipStream_t st){
    static bool attr_set = false;
    if(!attr_set){
        QLMX_HIP(hipFuncSetAttribute((const void *)(k_gemm_nt_lds<BN, NW>), hipFuncAttributeMaxDynamicSharedMemorySize, (Nt3Shape<BN, NW>::LDS_BYTES)), "nt LDS size");
        attr_set = true;
    }
    hipLaunchKernelGGL((k_gemm_nt_lds<BN, NW>), dim3(grid), dim3(NW * 64), (Nt3Shape<BN, NW>::LDS_BYTES), st, a);
    return QLMX_OK;
}
static int nt3_launch_any(int BN, const Nt3Args &a, int grid, hipStream_t st){
    return BN == 128 ? nt3_launch<128, 4>(a, grid, st) : nt3_launch<256, 8>(a, grid, st);
}
int qlmx_pair_hold_nt(const Nt3Args &a, int grid, int slot, bool units, hipStream_t st, bool *held);
/* the launch of the 256 x 128 form (also what issues a launch that was held for a pair and found no partner) */
int qlmx_gemm_nt_lds_issue(const Nt3Args &a, int grid, int slot, bool units, hipStream_t st){
    int rc = nt3_launch<128, 4>(a, grid, st); if(rc) return rc;
    QLMX_LAUNCH_CHECK("grouped gemm nt (direct-to-LDS) launch");
    return units ? qlmx_unit_done(slot, st) : qlmx_upload_done(slot, st);
}
/* a launch ready to go: held for a pair, or launched */
static int nt3_submit(int BN, const Nt3Args &a, int grid, int slot, bool units, hipStream_t st){
    if(BN == 128){
        bool held;
        int rc = qlmx_pair_hold_nt(a, grid, slot, units, st, &held); if(rc) return rc;
        return held ? QLMX_OK : qlmx_gemm_nt_lds_issue(a, grid, slot, units, st);
    }
    int rc = qlmx_pair_flush(); if(rc) return rc;          /* the wide tile is never held: what is held goes first */
    rc = nt3_launch_any(BN, a, grid, st); if(rc) return rc;
    QLMX_LAUNCH_CHECK("grouped gemm nt (direct-to-LDS) launch");
    return units ? qlmx_unit_done(slot, st) : qlmx_upload_done(slot, st);
}

/* Which tile. Uniform experts, K=768 N=2048, TFLOP/s at 512 / 2048 / 8192 rows per expert (8 experts at 8192, which
 * leaves the wide form 192 tiles for 256 CUs): 128 columns 778 / 950 / 934; 256 columns on eight wavefronts with four
 * tiles in LDS 724 / 1036 / 905 (with three 690 / 972 / 872, with five 719 / 1003 / 892; on four wavefronts of
 * 128 x 128 and three tiles 636 / 935 / 824). The wide form wins where experts have a few thousand rows and the
 * device is not held back by its power limit; the config-3 step has 512-row experts and the config-5 step runs at
 * the clock its load allows (861.6 against 863.3 TFLOP/s), so the wide tile is only taken on request:
 * QLMX_NT_TILE=256 in the environment (read at the first call) or qlmx_nt_tile(256). */
static int g_nt3_forced = -1;
static int nt3_pick_bn(int N){
    if(g_nt3_forced < 0){ const char *e = getenv("QLMX_NT_TILE"); g_nt3_forced = e ? atoi(e) : 0; }
    return (g_nt3_forced == 256 && N % 256 == 0) ? 256 : 128;
}
extern "C" int qlmx_nt_tile(int tile){
    QLMX_REQUIRE(tile == 128 || tile == 256, "qlmx_nt_tile: 128 or 256, not %d", tile);
    g_nt3_forced = tile;
    return QLMX_OK;
}

/* bf16 operands only; N % 128 == 0, K % 8 == 0, operands 16-byte aligned (checked by the caller) */
int qlmx_gemm_nt_lds_launch(const qlmx_gemm_prob *probs, int nprob, int K, int N, hipStream_t st){
    const int BN = nt3_pick_bn(N);
    if(!g_nt3_zeros){
        QLMX_HIP(hipMalloc(&g_nt3_zeros, 256), "nt zero block");
        QLMX_HIP(hipMemset(g_nt3_zeros, 0, 256), "nt zero block clear");
    }
    /* scheduled launch when the unit table holds it; the index-mapped one otherwise */
    {
        int live = 0;
        for(int i = 0; i < nprob; i++) if(probs[i].M > 0) live++;
        if(live == 0) return QLMX_OK;
        if(nprob <= QLMX_MAX_PROBLEMS){
            UnitUpload uu; int uslot;
            int rc = qlmx_unit_slot(live, &uu, &uslot); if(rc) return rc;
            int n = 0;
            for(int i = 0; i < nprob; i++){
                const qlmx_gemm_prob &p = probs[i];
                QLMX_REQUIRE(p.M >= 0, "grouped gemm: problem %d has M=%d", i, p.M);
                if(p.M == 0) continue;
                QLMX_REQUIRE(p.A && p.B && p.C, "grouped gemm nt: problem %d has a NULL operand", i);
                QLMX_REQUIRE(p.beta == 0.0f || p.beta == 1.0f, "grouped gemm: beta must be 0 or 1");
                DevProb &q = uu.hprob[n++];
                q.A = p.A; q.B = p.B; q.C = p.C; q.wq = 0; q.wg = 0; q.M = p.M; q.beta = p.beta; q.tile0 = 0; q.tiles_n = N / BN;
            }
            int nflags = 0, nent = 0;
            const int grid = nt3_schedule(uu.hprob, n, K, N, BN, BN == 128 ? 2 : 1, qlmx_cu_count(), uu.hunit, &nflags, &nent);
            if(grid > 0){
                Nt3Args a; a.pr = uu.dprob; a.units = uu.dunit; a.flags = uu.flags; a.status = uu.status;
                a.nprob = n; a.ntiles = grid; a.tiles_n = N / BN; a.rows_p = 1; a.K = K; a.N = N; a.zeros = g_nt3_zeros;
                int first = 0; a.epoch = 0;
                if(nflags){ rc = qlmx_chain_reserve(nflags, &first, &a.epoch); if(rc) return rc; }
                a.wait_epoch = a.epoch; a.wait_limit = QX_CHAIN_SPINS;
                if(nflags && qlmx_test_take_forced_timeout(2)){ a.wait_epoch = a.epoch ^ 0x00A5A5A5u; a.wait_limit = 1; }
                for(int p = 0; p < n; p++) uu.hprob[p].flag0 += first;
                qlmx_unit_commit(&uu, n, nent);
                return nt3_submit(BN, a, grid, uslot, true, st);
            }
        }
    }
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, GEMM_NT, K, N, NT3_BM, BN, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Nt3Args a; a.units = nullptr; a.flags = nullptr; a.status = nullptr; a.epoch = 0; a.wait_epoch = 0; a.wait_limit = 0; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.tiles_n = N / BN; a.K = K; a.N = N; a.zeros = g_nt3_zeros;
    a.rows_p = up.ntiles / (a.tiles_n * up.nprob);
    int grid;
    if(a.rows_p & 7) grid = 8 * a.tiles_n * a.rows_p * ((up.nprob + 7) / 8);
    else             grid = 8 * a.tiles_n * ((up.ntiles / a.tiles_n + 7) / 8);
    return nt3_submit(BN, a, grid, slot, false, st);
}
