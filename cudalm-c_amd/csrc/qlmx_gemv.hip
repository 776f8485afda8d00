/* qlmx_gemv.hip -- few-row expert GEMV over packed 4-bit weights (decode shape), bound by HBM.
 *
 * Serves the reference's decode step, where moe_forward runs on N = batch rows (dec_step,
 * cudalm.cu:7163-7204) and each expert GEMM of cudalm.cu:4211-4225 has at most a few rows: the
 * work is one pass over the hit experts' digits and scales. Two parts: the small-row path of
 * qlmx_moe_gemm_nn (the reference's CPU SGEMM has the same split at R<=4, cpu_rt.h:233-258), and
 * further down the whole decode layer fused into one launch.
 *
 * y[m, n] = sum_k x[m, k] * s[k, n/group] * digit[k, n], W row-major [K, N].
 *
 * Mapping of the small-row GEMV. A thread owns one 16-byte chunk column (32 consecutive n) and walks down the rows of
 * its workgroup's K-slice; consecutive threads own consecutive chunks, and when a row is narrower
 * than the workgroup the next threads continue on the following rows, so every load instruction
 * of a wave covers one contiguous 1 KiB of the weight matrix. Per chunk: xor 0x88888888 turns the
 * two's-complement nibbles into offset-8 bytes, two masks split even and odd nibbles, the
 * byte-to-float converts feed fp32 FMAs against x*s, and the offset (8 * sum of x*s) is taken out
 * once per row. The K dimension is split over workgroups for parallelism; slices leave partial sums
 * in a scratch buffer and the finishing kernel adds them in slice order, so results do not depend on
 * scheduling and no workgroup ever waits for another.
 *
 * Algorithmic HBM bytes per expert hit: K*N/2 digits + K*N/group*4 scales per matrix
 * (D=768, F=2048, three matrices: 2,506,752 B).
 */
#include "qlmx_gemm.h"
#include <math.h>
#include <string.h>
#include <stdlib.h>
#include <algorithm>

#define GV_THREADS 256
#define GV_MAXROWS 4          /* rows per problem (larger row counts are split by the callers) */
#define GV_MAXSLICE 512       /* K rows per workgroup slice held in LDS */
#define GV_BATCH 4            /* rows a thread has in flight */


struct GvProb {               /* 64 bytes */
    const float *x[GV_MAXROWS];   /* the input rows (each K floats)           */
    float *out;                   /* finish kernel: [M, N] rows, pitch N      */
    unsigned long long wq, wg;
    int M, pad;
};

struct GvArgs {
    const GvProb *pr; const int *nprob_dev; int nprob;
    const signed char *d; const float *s; int group, K, N;
    int nmat; unsigned long long mat_dq, mat_dg;     /* second matrix of a pair: +mat_dq elements, +mat_dg groups */
    int S, rps;                                      /* K slices, rows per slice */
    float *part;                                     /* out: [task][slice][MR][N] partial sums */
};

__device__ __forceinline__ float ub(uint32_t w, int k){ return (float)((w >> (8 * k)) & 0xFFu); }

#define GV_MAXSPLIT 16
/* sum of S <= GV_MAXSPLIT partial sums `stride` apart, added in slice order; all loads are issued
 * before the first add so the chain costs one memory latency, not S of them */
__device__ __forceinline__ float sum_slices(const float *src, size_t stride, int S){
    float t[GV_MAXSPLIT];
#pragma unroll
    for(int u = 0; u < GV_MAXSPLIT; u++) t[u] = u < S ? src[(size_t)u * stride] : 0.0f;
    float v = 0.0f;
#pragma unroll
    for(int u = 0; u < GV_MAXSPLIT; u++) v += t[u];
    return v;
}

template<int MR>
__global__ void __launch_bounds__(GV_THREADS) k_qlmx_gemv(GvArgs a){
    __shared__ float xs[MR][GV_MAXSLICE];
    __shared__ float red[GV_THREADS * 33];
    const int split = blockIdx.x, task = blockIdx.y;
    const int p = task / a.nmat, mat = task - p * a.nmat;
    const int nprob = a.nprob_dev ? *a.nprob_dev : a.nprob;
    if(p >= nprob) return;
    const GvProb *Pp = a.pr + p;
    const int PM = Pp->M;
    const int tid = threadIdx.x;
    const int ncc = a.N >> 5;                        /* 16-byte chunks per row */
    const int nph = GV_THREADS / ncc > 0 ? GV_THREADS / ncc : 1;
    const int ncol_pass = ncc < GV_THREADS ? 1 : (ncc + GV_THREADS - 1) / GV_THREADS;   /* column passes when a row is wider than the workgroup */
    const int kb0 = split * a.rps, kb1 = min(a.K, kb0 + a.rps);
    const unsigned long long wq = Pp->wq + (unsigned long long)mat * a.mat_dq;
    const unsigned long long wg = Pp->wg + (unsigned long long)mat * a.mat_dg;

    /* ---- input rows of this K slice into LDS ---- */
    for(int i = tid; i < MR * a.rps; i += GV_THREADS){
        const int m = i / a.rps, r = i - m * a.rps;
        float v = 0.0f;
        if(m < PM && kb0 + r < kb1) v = Pp->x[m][kb0 + r];
        xs[m][r] = v;
    }
    __syncthreads();

    for(int cp = 0; cp < ncol_pass; cp++){
        const int width = ncc < GV_THREADS ? ncc : GV_THREADS;          /* chunk columns in this pass */
        const int lc = ncc < GV_THREADS ? tid % ncc : tid;              /* chunk column inside the pass */
        const int c = lc + cp * GV_THREADS;
        const int ph = ncc < GV_THREADS ? tid / ncc : 0;
        const bool active = ph < nph && c < ncc;
        float acc[MR][32], corr[MR];
#pragma unroll
        for(int m = 0; m < MR; m++){ corr[m] = 0.0f;
#pragma unroll
            for(int j = 0; j < 32; j++) acc[m][j] = 0.0f; }
        if(active){
            /* GV_BATCH rows of this thread's chunk column are loaded before any is consumed, so a
             * slice costs one or two memory latencies rather than one per row */
            const signed char *dbase = a.d + ((wq + (size_t)c * 32) >> 1);
            const size_t rowb = (size_t)a.N >> 1;
            for(int rb = kb0 + ph; rb < kb1; rb += GV_BATCH * nph){
                uint4 wv[GV_BATCH]; float sv[GV_BATCH];
#pragma unroll
                for(int b = 0; b < GV_BATCH; b++){
                    const int r = rb + b * nph;
                    wv[b] = make_uint4(0x88888888u, 0x88888888u, 0x88888888u, 0x88888888u); sv[b] = 0.0f;     /* digit 0 */
                    if(r < kb1){
                        wv[b] = *(const uint4 *)(dbase + (size_t)r * rowb);
                        sv[b] = a.s[wg + ((size_t)r * a.N + (size_t)c * 32) / (size_t)a.group];
                    }
                }
#pragma unroll
                for(int b = 0; b < GV_BATCH; b++){
                    const int r = rb + b * nph;
                    float xv[MR];
#pragma unroll
                    for(int m = 0; m < MR; m++){ xv[m] = (r < kb1 ? xs[m][r - kb0] : 0.0f) * sv[b]; corr[m] += xv[m]; }
                    const uint32_t wd[4] = {wv[b].x, wv[b].y, wv[b].z, wv[b].w};
#pragma unroll
                    for(int q = 0; q < 4; q++){
                        const uint32_t u = wd[q] ^ 0x88888888u;
                        const uint32_t lo = u & 0x0F0F0F0Fu, hi = (u >> 4) & 0x0F0F0F0Fu;
#pragma unroll
                        for(int k = 0; k < 4; k++){
                            const float f0 = ub(lo, k), f1 = ub(hi, k);
#pragma unroll
                            for(int m = 0; m < MR; m++){
                                acc[m][q * 8 + 2 * k]     = fmaf(xv[m], f0, acc[m][q * 8 + 2 * k]);
                                acc[m][q * 8 + 2 * k + 1] = fmaf(xv[m], f1, acc[m][q * 8 + 2 * k + 1]);
                            }
                        }
                    }
                }
            }
        }
        /* reduce the row phases through LDS, one x-row at a time, and leave the slice's partial
         * sums in the scratch buffer */
#pragma unroll
        for(int m = 0; m < MR; m++){
            if(m < PM){                                  /* uniform over the workgroup */
                __syncthreads();
                if(active){
#pragma unroll
                    for(int j = 0; j < 32; j++) red[(ph * 32 + j) * width + lc] = acc[m][j] - 8.0f * corr[m];
                }
                __syncthreads();
                /* phase sums, turned to natural column order through LDS (pitch 33 keeps both the
                 * transposing write and the row read free of bank conflicts), then stored coalesced */
                float *dst = a.part + (((size_t)task * a.S + split) * MR + m) * a.N + (size_t)cp * GV_THREADS * 32;
                const int nph_eff = ncc < GV_THREADS ? nph : 1;
                float vsum[32];
#pragma unroll
                for(int it = 0; it < 32; it++){
                    const int i = tid + it * GV_THREADS;
                    float v = 0.0f;
                    if(i < 32 * width) for(int h = 0; h < nph_eff; h++) v += red[(size_t)h * 32 * width + i];
                    vsum[it] = v;
                }
                __syncthreads();
#pragma unroll
                for(int it = 0; it < 32; it++){
                    const int i = tid + it * GV_THREADS;
                    if(i < 32 * width){ const int j = i / width, cc = i - j * width; red[cc * 33 + j] = vsum[it]; }
                }
                __syncthreads();
                const int ncols = min(width, ncc - cp * GV_THREADS) * 32;
                for(int n = tid; n < ncols; n += GV_THREADS) dst[n] = red[(n >> 5) * 33 + (n & 31)];
            }
        }
    }
}

/* out[m, n] = sum over slices (in slice order) of the partial sums: the small-row GEMM's last step */
template<int MR>
__global__ void __launch_bounds__(256) k_qlmx_gemv_finish(const GvProb *pr, const float *part, int S, int N){
    const int p = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
    if(n >= N) return;
    const int M = pr[p].M; float *out = pr[p].out;
    for(int m = 0; m < M; m++){
        const float *src = part + (((size_t)p * S) * MR + m) * N + n;
        out[(size_t)m * N + n] = sum_slices(src, (size_t)MR * N, S);
    }
}

/* ------------------------------------------------------------------------------------------
 * Workspace owned by the library (grow-only): partial sums, device problem tables and the row maps
 * of the fused decode layer.
 * ---------------------------------------------------------------------------------------- */
struct GvWorkspace { float *part[1] = {nullptr}; size_t part_floats[1] = {0}; };
static GvWorkspace g_ws;

static int ws_reserve(int which, size_t floats, hipStream_t st){
    if(floats > g_ws.part_floats[which]){
        QLMX_HIP(hipStreamSynchronize(st), "gemv workspace sync");
        if(g_ws.part[which]) QLMX_HIP(hipFree(g_ws.part[which]), "gemv workspace free");
        QLMX_HIP(hipMalloc((void **)&g_ws.part[which], floats * sizeof(float)), "gemv partial sums");
        g_ws.part_floats[which] = floats;
    }
    return QLMX_OK;
}

/* number of K slices: about four workgroups per CU over the expected tasks, at least two row
 * sweeps per slice, at most GV_MAXSLICE rows per slice, at most 16 slices (partial-sum traffic) */
static void choose_split(int K, int N, int ntask, int *S, int *rps){
    const int ncc = N / 32, nph = GV_THREADS / ncc > 0 ? GV_THREADS / ncc : 1;
    int want = (1024 + ntask - 1) / (ntask > 0 ? ntask : 1);
    int smax = K / (2 * nph); if(smax < 1) smax = 1; if(smax > GV_MAXSPLIT) smax = GV_MAXSPLIT;
    int s = want < 1 ? 1 : (want > smax ? smax : want);
    int r = (K + s - 1) / s;
    r = ((r + nph - 1) / nph) * nph;                 /* whole sweeps */
    if(r > GV_MAXSLICE) r = GV_MAXSLICE / nph * nph;
    s = (K + r - 1) / r;
    *S = s; *rps = r;
}

template<int MR>
static int launch_gemv(GvArgs &a, int ntask_max, hipStream_t st){
    hipLaunchKernelGGL((k_qlmx_gemv<MR>), dim3(a.S, ntask_max), dim3(GV_THREADS), 0, st, a);
    QLMX_LAUNCH_CHECK("gemv launch");
    return QLMX_OK;
}

/* ---- small-row path of qlmx_moe_gemm_nn (fp32 activations, every problem M <= GV_MAXROWS) ---- */
int qlmx_gemv_nn_dispatch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                          int K, int N, hipStream_t st){
    QLMX_REQUIRE(N % 32 == 0 && group % 32 == 0, "gemv: N and group must be multiples of 32");
    QLMX_REQUIRE(((uintptr_t)d & 15) == 0, "gemv: digit array must be 16-byte aligned");
    /* The problem table is written into one of 16 slots of pinned host memory and read by the kernels
     * from there. The slots are guarded in two halves: an event is recorded behind the launch that
     * uses the last slot of a half and waited for when the ring re-enters that half (an event behind
     * every launch would leave the GPU idle for some microseconds each time). */
    enum { GV_SLOTS = 16, GV_HALF = 8 };
    static GvProb *ring = nullptr; static hipEvent_t ev[2]; static bool recorded[2] = {false, false};
    static hipStream_t ev_stream[2] = {nullptr, nullptr}; static int next_slot = 0;
    if(!ring){
        QLMX_HIP(hipHostMalloc((void **)&ring, (size_t)GV_SLOTS * QLMX_MAX_PROBLEMS * sizeof(GvProb), hipHostMallocDefault), "gemv table ring (pinned)");
        for(int i = 0; i < 2; i++) QLMX_HIP(hipEventCreateWithFlags(&ev[i], hipEventDisableTiming), "gemv table event");
    }
    const int slot = next_slot, half = slot / GV_HALF;
    if(slot % GV_HALF == 0 && recorded[half]){ QLMX_HIP(hipEventSynchronize(ev[half]), "gemv table wait"); recorded[half] = false; }
    /* a half whose launches went to more than one stream is closed by waiting for the odd stream at once */
    if(slot % GV_HALF == 0) ev_stream[half] = st;
    GvProb *h_tab = ring + (size_t)slot * QLMX_MAX_PROBLEMS, *d_tab = h_tab;
    int n = 0;
    for(int i = 0; i < nprob; i++){
        if(probs[i].M == 0) continue;
        QLMX_REQUIRE(((probs[i].wq >> 1) & 15ULL) == 0, "gemv: problem %d weight offset must be a multiple of 32 elements", i);
        GvProb &g = h_tab[n++];
        for(int m = 0; m < GV_MAXROWS; m++) g.x[m] = m < probs[i].M ? (const float *)probs[i].A + (size_t)m * K : nullptr;
        g.out = probs[i].C; g.wq = probs[i].wq; g.wg = probs[i].wg; g.M = probs[i].M; g.pad = 0;
    }
    if(n == 0) return QLMX_OK;
    GvArgs a; a.pr = d_tab; a.nprob_dev = nullptr; a.nprob = n; a.d = d; a.s = s; a.group = group; a.K = K; a.N = N;
    a.nmat = 1; a.mat_dq = 0; a.mat_dg = 0;
    choose_split(K, N, n, &a.S, &a.rps);
    int rc = ws_reserve(0, (size_t)n * a.S * GV_MAXROWS * N, st); if(rc) return rc;
    a.part = g_ws.part[0];
    rc = launch_gemv<GV_MAXROWS>(a, n, st); if(rc) return rc;
    hipLaunchKernelGGL(k_qlmx_gemv_finish<GV_MAXROWS>, dim3((N + 255) / 256, n), dim3(256), 0, st, d_tab, g_ws.part[0], a.S, N);
    QLMX_LAUNCH_CHECK("gemv finish launch");
    next_slot = (slot + 1) % GV_SLOTS;
    if(st != ev_stream[half]) QLMX_HIP(hipStreamSynchronize(st), "gemv table stream wait");
    if(slot % GV_HALF == GV_HALF - 1){ QLMX_HIP(hipEventRecord(ev[half], ev_stream[half]), "gemv table record"); recorded[half] = true; }
    return QLMX_OK;
}

/* ------------------------------------------------------------------------------------------
 * Fused decode layer: one launch for grouping, gate|up GEMV, SwiGLU, down GEMV and the gated
 * combine (moe_forward on decode rows, cudalm.cu:4189-4228).
 *
 * At decode sizes a layer moves a few tens of MB, i.e. a handful of microseconds of HBM time, so a
 * chain of launches costs more than the data. The layer therefore runs as one grid of resident
 * workgroups that walk three task lists in order:
 *   1. gate|up tasks  (problem, matrix w1|w3, 256-column chunk of F, K slice of D)  -> part1
 *   2. down tasks     (problem, 256-column chunk of D, K slice of F)                -> part2
 *      input rows h = silu(g) * u come from part1
 *   3. combine tasks  (token, 256-column chunk of D): out += gate * y from part2, passes in order.
 * Hand-over between lists: every partial sum is stored as one 8-byte word {value, tag of this
 * call}; a consumer re-reads a word until it carries the current tag (`epoch` below; the kernel
 * derives it from a device word, see its first lines). There are no flags to set,
 * clear or fence, and a consumer pays one memory round trip when its producer is already done.
 * Every workgroup finishes all of its tasks of one list before it starts the next, tasks of list 1
 * never wait, and the grid is sized to be co-resident, so the waits cannot deadlock; they are also
 * bounded (DF_SPIN_LIMIT polls) and report through a status word in pinned host memory if ever
 * exceeded. Partial sums are added in slice order by their consumer, so results do not depend on
 * timing. The 8-byte words are written and read with device-scope atomic accesses, which go to the
 * point where all XCDs (each has its own L2) agree, so no cache-wide write-back or invalidate is
 * needed around them.
 *
 * A "problem" is up to DF_MB (pass, token) pairs that hit the same expert; every workgroup derives
 * the same problem table from `assign` in LDS (stable counting sort by expert, the order of the
 * reference's host permutation, cudalm.cu:3586-3599).
 *
 * Task kernel (a template over two multiply loops). fp32 loop, the default: 256 threads cover 16 rows x 256
 * columns per step (a lane owns 16 columns = 8 bytes of digits of one row; 16 lanes cover the 128 contiguous
 * bytes of a row's chunk). fp16-input loop (qlmx_decode_math(1)): 32 rows per step, a lane owns the same columns
 * of two consecutive rows and multiplies both at once (see df_task). Either way a task is two halves of
 * DF_BATCH 8-byte loads per lane, both in flight (the next task's halves are requested as soon as this task has
 * consumed them). The input rows are staged in LDS already multiplied by the row's group scales, so the loop
 * loads digits only. Tasks of one (problem, matrix) are given to workgroups of one XCD so that the 64-byte scale
 * sectors shared by neighbouring chunks are fetched into one L2 only (the groups left over after a full round of
 * 8 XCDs are cut into pieces, see the kernel).
 * ---------------------------------------------------------------------------------------- */
#define DEC_MAXPAIR 64
#define DF_THREADS 256
#define DF_MB 2               /* pairs per problem: an expert hit by more pairs is several problems (a task of four rows took
                                 2.3 times as long as one of one row and held up everything that waited for it; its digits are
                                 fetched by neighbouring workgroups at about the same time, mostly once from HBM) */
#define DF_CW 256             /* columns per task */
#define DF_NG 2               /* scale groups per task row: group 128, or one when the group is a multiple of 256 */
#define DF_RMAX 256           /* rows per task at most */
#define DF_BATCH 8            /* 8-byte digit loads per lane and half task (fp32 loop: 8 steps of 16 rows; fp16-input loop: 4 steps of
                                 32 rows, a lane's two rows each): a task is two halves of at most 128 rows */
#define DF_SPIN_LIMIT (1 << 17)
#define DF_MAXTASKS 128        /* tasks of one workgroup at most (both lists); the host refuses shapes that would need more */
typedef unsigned long long u64;
/* Tracing build (-DQLMX_DF_TRACE): thread 0 of every workgroup stamps the 100 MHz wall clock at the phases
 * of its tasks into LDS (a store to memory per stamp would be waited for with the loads it sits among and
 * stretch the phases of a saturated launch); the workgroup copies its stamps to a device table when it is
 * done, and qlmx_debug_trace copies that out. Not part of the shipped library. */
#ifdef QLMX_DF_TRACE
#define DF_TRACE_WG 1024
#define DF_TRACE_EV 64
static __device__ u64 df_trace_tab[DF_TRACE_WG][DF_TRACE_EV];
#define DF_STAMP(code) do{ if(threadIdx.x == 0 && df_nev < DF_TRACE_EV) \
    df_ev[df_nev++] = (wall_clock64() << 8) | (u64)(code); }while(0)
#define DF_TRACE_PARAM , int &df_nev, u64 *df_ev
#define DF_TRACE_ARG , df_nev, df_ev
#else
#define DF_STAMP(code) do{}while(0)
#define DF_TRACE_PARAM
#define DF_TRACE_ARG
#endif

struct DfArgs {
    const float *x; const int *assign; const float *gate; float *out;
    const signed char *d; const float *s;
    u64 w1q, w3q, w2q; int group;
    u64 w1g, w3g, w2g, dfg;   /* the matrices' first scale groups, and scale groups per expert matrix (host-side divisions) */
    int T, K, E, D, F;
    int R1, S1, NC1, R2, S2, NC2;
    u64 *part1, *part2; unsigned epoch; unsigned *status;
    unsigned wait_xor; int spin_limit;   /* waits look for epoch ^ wait_xor (0) for at most spin_limit polls; the time-out test changes both */
    unsigned *ctl;            /* device words: [0] tag of the last finished call, [1] workgroups of this call that are done */
    u64 parts1, parts2;       /* byte n: pieces a group's chunks are cut into when n groups are left over after the last round of 8 (a table in a
                                 word: indexing an array inside the kernel arguments would move them all to scratch memory) */
};

struct DfMeta {
    int nprob;
    int p_e[DEC_MAXPAIR], p_M[DEC_MAXPAIR], p_row0[DEC_MAXPAIR];
    int rowpair[DEC_MAXPAIR], rowtok[DEC_MAXPAIR], pair_prob[DEC_MAXPAIR], pair_m[DEC_MAXPAIR];
    int se[DEC_MAXPAIR], sj[DEC_MAXPAIR], ein[DEC_MAXPAIR], rk[4][DEC_MAXPAIR];
};

/* a / b for 0 <= a < 2^22, b > 0, rb = 1/b as a float: the quotient of the floats is off by at most one,
 * which the remainder shows. (The compiler's integer division is some fifty instructions, and the
 * bookkeeping between two tasks is made of divisions.) */
__device__ __forceinline__ int df_div(int a, int b, float rb){
    int q = (int)((float)a * rb);
    const int r = a - q * b;
    q += (r >= b) - (r < 0);
    return q;
}
__device__ __forceinline__ int df_uni(int v){ return __builtin_amdgcn_readfirstlane(v); }

__device__ __forceinline__ void df_st(u64 *p, float v, unsigned epoch){
    __hip_atomic_store(p, ((u64)epoch << 32) | (u64)__float_as_uint(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* Sums of S tagged partial sums `stride` words apart from each of NSRC sources, in slice order;
 * re-reads until every word carries `epoch`. All loads of a pass are issued before the first is
 * looked at. */
template<int NSRC, int DF_SLICE_STEP>
__device__ __forceinline__ void df_sum_wait(const u64 *const (&src)[NSRC], size_t stride, int S, unsigned epoch, int limit,
                                            volatile int *giveup, unsigned *status, float (&v)[NSRC]){
    int spins = 0;
    for(;;){
        bool ok = true;
#pragma unroll
        for(int q = 0; q < NSRC; q++) v[q] = 0.0f;
        for(int b = 0; b < S; b += DF_SLICE_STEP){
            u64 t[NSRC][DF_SLICE_STEP];
#pragma unroll
            for(int q = 0; q < NSRC; q++)
#pragma unroll
                for(int u = 0; u < DF_SLICE_STEP; u++)
                    t[q][u] = __hip_atomic_load(src[q] + (size_t)min(b + u, S - 1) * stride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for(int q = 0; q < NSRC; q++)
#pragma unroll
                for(int u = 0; u < DF_SLICE_STEP; u++){
                    ok = ok && (unsigned)(t[q][u] >> 32) == epoch;
                    if(b + u < S) v[q] += __uint_as_float((unsigned)t[q][u]);
                }
        }
        if(ok) break;
        if(++spins > limit || *giveup){ *(volatile unsigned *)status = 1u; *giveup = 1; break; }
        __builtin_amdgcn_s_sleep(2);
    }
}

/* Cheap wait in front of the tagged reads: thread i < n polls one word of producer i until it carries
 * the epoch, then the workgroup meets. A producer's words become visible within a short time of each
 * other, so the full read that follows rarely has to repeat, and while a producer is still busy only
 * n threads per workgroup poll instead of all of them. */
template<class ADDR>
__device__ __forceinline__ void df_wait_first(int n, unsigned epoch, int limit, volatile int *giveup, unsigned *status, ADDR addr){
    for(int i = threadIdx.x; i < n; i += DF_THREADS){
        const u64 *p = addr(i);
        if(!p) continue;
        int spins = 0;
        while((unsigned)(__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 32) != epoch){
            if(++spins > limit || *giveup){ *(volatile unsigned *)status = 1u; *giveup = 1; break; }
            __builtin_amdgcn_s_sleep(4);
        }
    }
    __syncthreads();
}

__device__ __forceinline__ uint32_t df_and(uint32_t v){
    uint32_t r; asm("v_and_b32 %0, %1, %2" : "=v"(r) : "s"(0x0F0F0F0Fu), "v"(v)); return r;
}

/* (v & mask) | magic in one instruction; written out because the compiler emits an and and an or */
__device__ __forceinline__ uint32_t df_and_or(uint32_t v, uint32_t mask, uint32_t magic){
    uint32_t r; asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "s"(mask), "v"(magic)); return r;
}
typedef _Float16 df_h2 __attribute__((ext_vector_type(2)));
/* a.x * b.x + a.y * b.y + c: fp16 pairs, exact products, fp32 sum (v_dot2_f32_f16) */
__device__ __forceinline__ float df_dot2(uint32_t a, uint32_t b, float c){
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(df_h2, a), __builtin_bit_cast(df_h2, b), c, false);
}
__device__ __forceinline__ uint32_t df_pack_h2(float a, float b){
    const df_h2 h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

/* Staging of a task's inputs. v[g][m] is this thread's row (thread = row of the task; zeros past its rows)
 * times the row's scale of column group g, for the task's input rows m. The multiply loop takes them as fp16
 * pairs of two consecutive rows, so they are first brought to [2^14, 2^15) at the task's largest magnitude by a
 * power of two (its inverse is returned and applied to the task's sums) and stored per scale group and row
 * pair as {pair of m = 0, pair of m = 1, the same two divided by 16}. Two barriers: the first also separates
 * the previous task's reads of xs from the writes here. */
__device__ __forceinline__ float df_stage(const float (&v)[DF_NG][DF_MB], bool live, uint32_t (*xs)[DF_RMAX / 2][2 * DF_MB], float *wmax){
    const int tid = threadIdx.x;
    float mx = 0.0f;
#pragma unroll
    for(int gg = 0; gg < DF_NG; gg++)
#pragma unroll
        for(int m = 0; m < DF_MB; m++) mx = fmaxf(mx, fabsf(v[gg][m]));
#pragma unroll
    for(int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if((tid & 63) == 0) wmax[tid >> 6] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    /* 2^(14 - floor(log2 mx)), kept where it and its inverse are both normal numbers */
    const int ex = (int)((__float_as_uint(mx) >> 23) & 0xFFu);
    int se = 268 - ex; if(se > 252) se = 252; if(se < 2) se = 2;
    const float scale = __uint_as_float((uint32_t)se << 23), inv = __uint_as_float((uint32_t)(254 - se) << 23);
#pragma unroll
    for(int gg = 0; gg < DF_NG; gg++){
        uint32_t hi[DF_MB], lo[DF_MB];
#pragma unroll
        for(int m = 0; m < DF_MB; m++){
            const float p = v[gg][m] * scale, q = __shfl_xor(p, 1, 64);   /* the odd row of the pair is the next lane's */
            hi[m] = df_pack_h2(p, q); lo[m] = df_pack_h2(p * 0.0625f, q * 0.0625f);
        }
        if(live && !(tid & 1)) *(uint4 *)&xs[gg][tid >> 1][0] = make_uint4(hi[0], hi[1], lo[0], lo[1]);
    }
    __syncthreads();
    return inv;
}

/* The same for the fp32 loop: the values as they are, xs[g][row][m]; nothing to undo (returns 1). */
__device__ __forceinline__ float df_stage_f32(const float (&v)[DF_NG][DF_MB], bool live, float (*xs)[DF_RMAX][DF_MB]){
    __syncthreads();                                 /* the previous task is done with xs */
    if(live){
#pragma unroll
        for(int gg = 0; gg < DF_NG; gg++) *(float2 *)&xs[gg][threadIdx.x][0] = make_float2(v[gg][0], v[gg][1]);
    }
    __syncthreads();
    return 1.0f;
}

/* One task: which slice of which matrix, for which problem. list 0 = none. */
struct DfT { u64 wq, wg; int list, N, k0, rows, chunk, M, prob, mat, sl, ngl; };   /* ngl: scale groups of the chunk that lie inside the row (1 or 2) */

/* first DF_BATCH steps of a task's digits into W (the caller keeps them in flight across the end of
 * the previous task) */
template<bool H>
__device__ __forceinline__ const signed char *df_digits(const DfArgs &a, const DfT &t){
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cl = lane & 15, rp = wave * 4 + (lane >> 4);
    const int col0 = t.chunk * DF_CW + cl * 16;
    return a.d + ((t.wq + (size_t)(t.k0 + (H ? 2 * rp : rp)) * t.N + (col0 < t.N ? col0 : 0)) >> 1);
}
/* Requests half h of a task's digits into W. fp16 loop (H): a step is 32 rows, the 16 row pairs of the
 * workgroup's 16 lane groups, and W[2 s + par] holds row `par` of the lane's pair in step s of the half; fp32
 * loop: a step is 16 rows, W[s] the lane's row in step s. rows is a multiple of 32, so a step is live or not
 * for the whole workgroup. Every load is issued unconditionally (a dead step re-reads step 0): loads under a
 * branch make the compiler wait for each one where the branches join, which turns a batch into a chain of
 * memory round trips. */
template<bool H>
__device__ __forceinline__ void df_load(uint2 (&W)[DF_BATCH], const signed char *dp, size_t rowb, int rows, int hsteps, int h){
#pragma unroll
    for(int b = 0; b < DF_BATCH; b++){
        if(H){
            const int st = h * hsteps + (b >> 1);
            const int sc = ((b >> 1) < hsteps && st * 32 < rows) ? st : 0;
            W[b] = *(const uint2 *)(dp + (size_t)(sc * 32 + (b & 1)) * rowb);
        } else {
            const int st = h * hsteps + b;
            const int sc = (b < hsteps && st * 16 < rows) ? st : 0;
            W[b] = *(const uint2 *)(dp + (size_t)sc * 16 * rowb);
        }
    }
}

/* dst[m*mstride + chunk*256 + c] = sum_{r<rows} x[m][r] * s * digit(k0+r, chunk*256+c), m < M, stored
 * tagged. w0, w1 hold the digits of the task's two halves, requested earlier. `prep` stages the inputs
 * (df_stage) and returns the power of two to apply to the sums. `next0` and `next1` request the following
 * task's halves into w0 and w1 as soon as this task has consumed them, so the reduction, the stores and the
 * next task's staging overlap that trip from HBM.
 *
 * The multiply-adds are v_dot2_f32_f16: two products per instruction, exact, summed in fp32. One operand is the
 * pair of digits of a lane's two rows as fp16, built without a conversion: with u = digit + 8 (two's complement
 * nibble xor 8), 0x6400 | u is the fp16 number 1024 + u (even columns, low nibble) and 0x6400 | u << 4 is
 * 1024 + 16 u (odd columns, the nibble stays where it is), so one byte permute puts two bytes of both rows side
 * by side and one and-or per column does the rest: 14 instructions per 16 digits. The other operand is the pair
 * of staged inputs (divided by 16 for the odd columns). What the offsets add -- (1024 + 8) and (64 + 8) times
 * the sum of the staged inputs -- is taken out at the end. The inputs thus carry 11 significant bits. */
template<bool H, int MT, class PREP, class NEXT0, class NEXT1>
__device__ __forceinline__ void df_task(const DfArgs &a, const DfT &t, uint2 (&w0)[DF_BATCH], uint2 (&w1)[DF_BATCH], int hsteps,
                                        const uint32_t *xs_raw, float *red, u64 *dst, size_t mstride,
                                        PREP prep, NEXT0 next0, NEXT1 next1 DF_TRACE_PARAM){
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int cl = lane & 15, rp = wave * 4 + (lane >> 4);
    const int N = t.N, rows = t.rows, M = t.M, chunk = t.chunk;
    const int gl = a.group >= DF_CW ? 0 : (cl >> 3);          /* this lane's scale group inside the chunk */
    float acc[MT][16], corr[MT];
#pragma unroll
    for(int m = 0; m < MT; m++){ corr[m] = 0.0f;
#pragma unroll
        for(int j = 0; j < 16; j++) acc[m][j] = 0.0f; }
    const uint32_t magic = 0x64006400u;
    const uint32_t (*xs)[DF_RMAX / 2][2 * DF_MB] = (const uint32_t (*)[DF_RMAX / 2][2 * DF_MB])xs_raw;
    const float (*xf)[DF_RMAX][DF_MB] = (const float (*)[DF_RMAX][DF_MB])xs_raw;
#define DF_COMPUTE_H(W, h)                                                          \
    _Pragma("unroll")                                                              \
    for(int s_ = 0; s_ < DF_BATCH / 2; s_++){                                      \
        if(s_ < hsteps && ((h) * hsteps + s_) * 32 < rows){                        \
            const uint4 x4 = *(const uint4 *)&xs[gl][((h) * hsteps + s_) * 16 + rp][0]; \
            const uint32_t xh[DF_MB] = {x4.x, x4.y}, xl[DF_MB] = {x4.z, x4.w};     \
            uint32_t P[16];                                                        \
            _Pragma("unroll")                                                      \
            for(int hf = 0; hf < 2; hf++){                                         \
                const uint32_t r0_ = (hf ? W[2 * s_].y : W[2 * s_].x) ^ 0x88888888u;         \
                const uint32_t r1_ = (hf ? W[2 * s_ + 1].y : W[2 * s_ + 1].x) ^ 0x88888888u; \
                const uint32_t E0 = __builtin_amdgcn_perm(r1_, r0_, 0x05040100u);  \
                const uint32_t E1 = __builtin_amdgcn_perm(r1_, r0_, 0x07060302u);  \
                const uint32_t S0 = E0 >> 8, S1 = E1 >> 8;                         \
                P[hf * 8 + 0] = df_and_or(E0, 0x000F000Fu, magic);                 \
                P[hf * 8 + 1] = df_and_or(E0, 0x00F000F0u, magic);                 \
                P[hf * 8 + 2] = df_and_or(S0, 0x000F000Fu, magic);                 \
                P[hf * 8 + 3] = df_and_or(S0, 0x00F000F0u, magic);                 \
                P[hf * 8 + 4] = df_and_or(E1, 0x000F000Fu, magic);                 \
                P[hf * 8 + 5] = df_and_or(E1, 0x00F000F0u, magic);                 \
                P[hf * 8 + 6] = df_and_or(S1, 0x000F000Fu, magic);                 \
                P[hf * 8 + 7] = df_and_or(S1, 0x00F000F0u, magic);                 \
            }                                                                      \
            _Pragma("unroll")                                                      \
            for(int m = 0; m < MT; m++){                                           \
                corr[m] = df_dot2(0x3C003C00u, xh[m], corr[m]);                    \
                _Pragma("unroll")                                                  \
                for(int j = 0; j < 16; j++) acc[m][j] = df_dot2(P[j], (j & 1) ? xl[m] : xh[m], acc[m][j]); \
            }                                                                      \
        }                                                                          \
    }
    /* The fp32 loop: one row per lane and step, digits to fp32 one by one (v_cvt_f32_ubyteN; the nibble masks go
     * through df_and so that those converts survive: seen through, the compiler rewrites mask + byte select into
     * a bit-field extract per digit and doubles the instruction count), 16 fp32 multiply-adds per input row. */
#define DF_COMPUTE_S(W, h)                                                        \
    _Pragma("unroll")                                                              \
    for(int b = 0; b < DF_BATCH; b++){                                             \
        if(b < hsteps && ((h) * hsteps + b) * 16 < rows){                          \
            const int r = ((h) * hsteps + b) * 16 + rp;                            \
            const float2 x2 = *(const float2 *)&xf[gl][r][0];                      \
            const float xm[DF_MB] = {x2.x, x2.y};                                  \
            float f[16];                                                           \
            const uint32_t u0 = W[b].x ^ 0x88888888u, u1 = W[b].y ^ 0x88888888u;   \
            const uint32_t l0 = df_and(u0), h0 = df_and(u0 >> 4);                  \
            const uint32_t l1 = df_and(u1), h1 = df_and(u1 >> 4);                  \
            _Pragma("unroll")                                                      \
            for(int k = 0; k < 4; k++){ f[2 * k] = ub(l0, k); f[2 * k + 1] = ub(h0, k); f[8 + 2 * k] = ub(l1, k); f[9 + 2 * k] = ub(h1, k); } \
            _Pragma("unroll")                                                      \
            for(int m = 0; m < MT; m++){                                           \
                const float xv = xm[m];                                            \
                corr[m] += xv;                                                     \
                _Pragma("unroll")                                                  \
                for(int j = 0; j < 16; j++) acc[m][j] = fmaf(xv, f[j], acc[m][j]); \
            }                                                                      \
        }                                                                          \
    }
    DF_STAMP(10 + 16 * t.list);
    const float unscale = prep();
    DF_STAMP(11);
    /* The multiply loop saturates the vector ALU; everything else a workgroup does -- listing its tasks, requesting
     * digits, staging, reducing -- is short chains of dependent instructions that other workgroups wait for. Those
     * run at a raised wave priority, the loop at the lowest, so that a workgroup still on its way to its first
     * task is not starved by its neighbours' loops (the fourth workgroup of a CU otherwise reached its first task
     * 8 us after the first). */
    __builtin_amdgcn_s_setprio(0);
    if(H){ DF_COMPUTE_H(w0, 0) } else { DF_COMPUTE_S(w0, 0) }
    next0();
    DF_STAMP(12);
    if(H){ DF_COMPUTE_H(w1, 1) } else { DF_COMPUTE_S(w1, 1) }
    next1();
    __builtin_amdgcn_s_setprio(3);
    DF_STAMP(13);
#undef DF_COMPUTE_H
#undef DF_COMPUTE_S
    /* four row phases of a wave: reduce-scatter over lane bits 5 and 4, then the four waves via LDS */
    const bool hi32 = lane & 32, hi16 = lane & 16;
    __syncthreads();
#pragma unroll
    for(int m = 0; m < MT; m++){
        if(m < M){
            float k8[8], k4[4];
            const float off_even = (H ? 1032.0f : 8.0f) * corr[m], off_odd = (H ? 72.0f : 8.0f) * corr[m];
#pragma unroll
            for(int j = 0; j < 8; j++){
                const float off = (j & 1) ? off_odd : off_even;
                const float lo = acc[m][j] - off, hi = acc[m][8 + j] - off;
                const float mine = hi32 ? hi : lo, send = hi32 ? lo : hi;
                k8[j] = mine + __shfl_xor(send, 32, 64);
            }
#pragma unroll
            for(int j = 0; j < 4; j++){
                const float mine = hi16 ? k8[4 + j] : k8[j], send = hi16 ? k8[j] : k8[4 + j];
                k4[j] = mine + __shfl_xor(send, 16, 64);
            }
            *(float4 *)&red[(wave * DF_MB + m) * DF_CW + cl * 16 + (hi32 ? 8 : 0) + (hi16 ? 4 : 0)] = make_float4(k4[0], k4[1], k4[2], k4[3]);
        }
    }
    __syncthreads();
    const int col = chunk * DF_CW + tid;
    if(col < N){
        for(int m = 0; m < M; m++){
            const float v = ((red[(0 * DF_MB + m) * DF_CW + tid] + red[(1 * DF_MB + m) * DF_CW + tid])
                           + red[(2 * DF_MB + m) * DF_CW + tid]) + red[(3 * DF_MB + m) * DF_CW + tid];
            df_st(dst + (size_t)m * mstride + col, v * unscale, a.epoch);
        }
    }
    DF_STAMP(14);
}

template<bool H>
__global__ void __launch_bounds__(DF_THREADS, 4) k_decode_fused(DfArgs a){
    __shared__ DfMeta mt;
    __shared__ __align__(16) uint32_t xs_raw[DF_NG * DF_RMAX * DF_MB];   /* staged inputs: df_stage (fp16 pairs) or df_stage_f32 */
    __shared__ float wmax[4];
    __shared__ DfT tasks[DF_MAXTASKS];
    __shared__ int wcount[4];
    __shared__ float red[4 * DF_MB * DF_CW];
    __shared__ int giveup;
    const int tid = threadIdx.x;
    __builtin_amdgcn_s_setprio(3);
#ifdef QLMX_DF_TRACE
    int df_nev = 0;
    __shared__ u64 df_ev[DF_TRACE_EV];
    if(tid < DF_TRACE_EV) df_ev[tid] = 0;
    __syncthreads();
#endif
    DF_STAMP(1);
    /* The tag of this call's partial sums is one more than the last finished call's, which lives in
     * device memory: the host passes no counter, so a launch recorded in a graph tags every replay
     * afresh. Every workgroup reads the word here; the last workgroup to finish moves it on (end of
     * the kernel), which cannot happen before all of them have read it. 0 is the cleared state. */
    const int npair = a.T * a.K;
    const int ng = a.group >= DF_CW ? 1 : DF_CW / a.group;
    /* the two first loads -- the pairs' experts and the tag -- are both on their way before either is used
     * (under branches they went one after the other, a memory round trip each) */
    const int e_in = a.assign[min(tid, npair - 1)];
    const unsigned last = __hip_atomic_load(a.ctl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if(tid == 0) giveup = 0;

    /* ---- problem table (identical in every workgroup): rank of pair j among (expert, j) ---- */
    if(tid < DEC_MAXPAIR){
        int e = tid < npair ? e_in : 0x7FFFFFFF;
        if(tid < npair && (unsigned)e >= (unsigned)a.E) e = 0x7FFFFFFE;   /* invalid: sorts after every valid expert */
        mt.ein[tid] = e;
    }
    __syncthreads();
    {
        const int j = tid & 63, part = tid >> 6, e = mt.ein[j];
        int rank = 0;
        for(int i = part * 16; i < min(npair, part * 16 + 16); i++){
            const int ei = mt.ein[i];
            rank += (ei < e) || (ei == e && i < j);
        }
        mt.rk[part][j] = rank;
    }
    __syncthreads();
    if(tid < 64){
        const bool live = tid < npair;
        const int e = mt.ein[tid];
        const bool bad = live && e == 0x7FFFFFFE;
        const int rank = mt.rk[0][tid] + mt.rk[1][tid] + mt.rk[2][tid] + mt.rk[3][tid];
        if(live){ mt.se[rank] = e; mt.sj[rank] = tid; }
        if(bad){ mt.pair_prob[tid] = -1; mt.pair_m[tid] = 0; }
    }
    __syncthreads();
    if(tid < 64){
        const bool live = tid < npair;
        const int nvalid = __popcll(__ballot(live && mt.ein[tid] != 0x7FFFFFFE));
        const int r = tid; const bool valid = r < nvalid;
        const int er = valid ? mt.se[r] : -1;
        const bool head = valid && (r == 0 || mt.se[r - 1] != er);
        const u64 upto = r == 63 ? ~0ull : ((2ull << r) - 1ull);
        const u64 hm = __ballot(head);
        const int hidx = 63 - __clzll((long long)((hm & upto) | 1ull));
        const u64 after = hm & ~upto;
        const int nidx = after ? __ffsll((long long)after) - 1 : nvalid;
        const int pos = r - hidx, cnt = nidx - hidx;
        const bool start = valid && (pos % DF_MB == 0);
        const u64 sm = __ballot(start);
        const int prob = __popcll(sm & upto) - 1;
        if(valid){
            const int j = mt.sj[r];
            mt.rowpair[r] = j; mt.rowtok[r] = j % a.T; mt.pair_prob[j] = prob; mt.pair_m[j] = pos % DF_MB;
            if(start){ mt.p_e[prob] = er; mt.p_M[prob] = min(DF_MB, cnt - pos); mt.p_row0[prob] = r; }
        }
        if(tid == 0) mt.nprob = __popcll(sm);
    }
    __syncthreads();
    const int nprob = mt.nprob;
    DF_STAMP(2);
    const int G = gridDim.x, xcd = blockIdx.x & 7, slot0 = blockIdx.x >> 3, nslot = G >> 3;
    const u64 DF = (u64)a.D * a.F;

    /* ---- this workgroup's tasks, list 1 (gate|up) then list 2 (down), in one stream so that the
     * first digits of a task are already on their way while the task before it finishes ---- */
    /* Groups -- (problem, matrix) in list 1, problems in list 2 -- go to the XCDs round robin, whole, so that the
     * scale sectors that a group's column chunks share meet in one L2. The groups left over after the last full
     * round of 8 would give some XCDs a whole group more than others (a second task for a sixth of their
     * workgroups while others have none; with a single token: 4 groups, half the device idle), so the chunks of
     * each of those are cut into `parts` pieces that go to different XCDs (host table by the number left over). */
    const int ngrp1 = 2 * nprob;
    const int rem1 = ngrp1 & 7, rem2 = nprob & 7, full1 = ngrp1 - rem1, full2 = nprob - rem2;
    const int parts1 = (int)((a.parts1 >> (8 * rem1)) & 0xFFu), parts2 = (int)((a.parts2 >> (8 * rem2)) & 0xFFu);
    const int cpp1 = df_div(a.NC1, parts1, 1.0f / (float)parts1), cpp2 = df_div(a.NC2, parts2, 1.0f / (float)parts2);   /* chunks per piece */
    const int tpw1 = a.NC1 * a.S1, tpw2 = a.NC2 * a.S2;               /* tasks of a whole group */
    const int tpg1 = cpp1 * a.S1, tpg2 = cpp2 * a.S2;                 /* tasks of a piece */
    const int nw1 = (full1 >> 3) * tpw1, nw2 = (full2 >> 3) * tpw2;   /* tasks that whole groups give each XCD */
    const int nvg1 = rem1 * parts1, nvg2 = rem2 * parts2;             /* pieces */
    const int lim1 = nw1 + ((nvg1 + 7) >> 3) * tpg1, lim2 = nw2 + ((nvg2 + 7) >> 3) * tpg2;
    const float rtpw1 = 1.0f / (float)tpw1, rtpw2 = 1.0f / (float)tpw2;
    const float rtpg1 = 1.0f / (float)tpg1, rtpg2 = 1.0f / (float)tpg2, rS1 = 1.0f / (float)a.S1, rS2 = 1.0f / (float)a.S2;
    const float rparts1 = 1.0f / (float)parts1, rparts2 = 1.0f / (float)parts2;
    /* The task list of this workgroup is worked out once, one candidate per thread, and kept in LDS: candidate k
     * of list 1 is slot slot0 + k * nslot of this XCD's tasks, list 2's follow; candidates that fall behind the
     * last group of the XCD are dropped and the rest keeps its order. (Worked out one after the other by every
     * wavefront in front of each task, this arithmetic -- a microsecond of dependent instructions -- stood between
     * any two tasks.) */
    const int nc1 = nslot > 0 ? (lim1 - slot0 + nslot - 1) / nslot : 0, nc2 = nslot > 0 ? (lim2 - slot0 + nslot - 1) / nslot : 0;
    const int c1 = nc1 > 0 ? nc1 : 0, c2 = nc2 > 0 ? nc2 : 0;           /* candidates of the two lists */
    {
        DfT t; t.list = 0; t.wq = 0; t.wg = 0; t.N = t.k0 = t.rows = t.chunk = t.M = t.prob = t.mat = t.sl = t.ngl = 0;
        if(tid < c1){
            const int q = slot0 + tid * nslot;
            /* slot q of this XCD: first its whole groups, then its pieces of the groups left over */
            const bool whole = q < nw1;
            const int qq = whole ? q : q - nw1, tp = whole ? tpw1 : tpg1;
            const int qd = df_div(qq, tp, whole ? rtpw1 : rtpg1), vg = qd * 8 + xcd, sub = qq - qd * tp;
            if(whole || vg < nvg1){
                const int gp = df_div(vg, parts1, rparts1);
                const int g = whole ? vg : full1 + gp, part = whole ? 0 : vg - gp * parts1, cl = df_div(sub, a.S1, rS1);
                t.list = 1; t.prob = g >> 1; t.mat = g & 1; t.chunk = part * cpp1 + cl; t.sl = sub - cl * a.S1;
                t.N = a.F; t.k0 = t.sl * a.R1; t.rows = min(a.R1, a.D - t.k0); t.M = mt.p_M[t.prob];
                t.ngl = (ng == 2 && t.N - t.chunk * DF_CW > a.group) ? 2 : 1;
                const int ex = mt.p_e[t.prob];
                t.wq = (t.mat ? a.w3q : a.w1q) + (u64)ex * DF;
                t.wg = (t.mat ? a.w3g : a.w1g) + (u64)ex * a.dfg;
            }
        } else if(tid < c1 + c2){
            const int q = slot0 + (tid - c1) * nslot;
            const bool whole = q < nw2;
            const int qq = whole ? q : q - nw2, tp = whole ? tpw2 : tpg2;
            const int qd = df_div(qq, tp, whole ? rtpw2 : rtpg2), vg = qd * 8 + xcd, sub = qq - qd * tp;
            if(whole || vg < nvg2){
                const int gp = df_div(vg, parts2, rparts2);
                const int prob = whole ? vg : full2 + gp, part = whole ? 0 : vg - gp * parts2, cl = df_div(sub, a.S2, rS2);
                t.list = 2; t.prob = prob; t.mat = 0; t.chunk = part * cpp2 + cl; t.sl = sub - cl * a.S2;
                t.N = a.D; t.k0 = t.sl * a.R2; t.rows = min(a.R2, a.F - t.k0); t.M = mt.p_M[prob];
                t.ngl = (ng == 2 && t.N - t.chunk * DF_CW > a.group) ? 2 : 1;
                const int ex = mt.p_e[prob];
                t.wq = a.w2q + (u64)ex * DF;
                t.wg = a.w2g + (u64)ex * a.dfg;
            }
        }
        /* keep the live ones, in order: rank inside the wavefront by a ballot, wavefronts added up through LDS */
        const u64 bal = __ballot(t.list != 0);
        const int lane = tid & 63, wv = tid >> 6;
        if(lane == 0) wcount[wv] = __popcll(bal);
        __syncthreads();
        int base = 0;
        for(int w = 0; w < wv; w++) base += wcount[w];
        if(t.list != 0){
            const int pos = base + __popcll(bal & ((1ull << lane) - 1ull));
            if(pos < DF_MAXTASKS) tasks[pos] = t;
        }
        __syncthreads();
    }
    /* the tag is first needed when a partial sum is stored: its load (past the caches) has had the table and the
     * task list to come back */
    a.epoch = __builtin_amdgcn_readfirstlane(last == 0xFFFFFFFFu ? 1u : last + 1u);
    const int ntasks = min(DF_MAXTASKS, wcount[0] + wcount[1] + wcount[2] + wcount[3]);
    int ti = 0;
    auto fetch = [&]() -> DfT {
        DfT t; t.list = 0; t.wq = 0; t.wg = 0; t.N = t.k0 = t.rows = t.chunk = t.M = t.prob = t.mat = t.sl = t.ngl = 0;
        if(ti < ntasks){
            const DfT &s = tasks[ti++];
            t.list = df_uni(s.list); t.N = df_uni(s.N); t.k0 = df_uni(s.k0); t.rows = df_uni(s.rows); t.chunk = df_uni(s.chunk);
            t.M = df_uni(s.M); t.prob = df_uni(s.prob); t.mat = df_uni(s.mat); t.sl = df_uni(s.sl); t.ngl = df_uni(s.ngl);
            t.wq = ((u64)(unsigned)df_uni((int)(s.wq >> 32)) << 32) | (unsigned)df_uni((int)(unsigned)s.wq);
            t.wg = ((u64)(unsigned)df_uni((int)(s.wg >> 32)) << 32) | (unsigned)df_uni((int)(unsigned)s.wg);
        }
        return t;
    };
    uint2 w0[DF_BATCH], w1[DF_BATCH];
    const int hs1 = a.R1 >> (H ? 6 : 5), hs2 = a.R2 >> (H ? 6 : 5);   /* steps (of 32 rows, fp32 loop: 16) per half task */
    const int gprF = a.F / a.group, gprD = a.D / a.group;     /* scale groups per row of w1|w3 and of w2 */
    const int cpg = a.group >= DF_CW ? a.group / DF_CW : 1;   /* chunks per scale group when the group is wider than a chunk */
    /* first scale of a task: its first row, its chunk's first group */
    auto scales_of = [&](const DfT &t) -> const float * {
        const int cg = a.group >= DF_CW ? t.chunk / cpg : t.chunk * (DF_CW / a.group);
        return a.s + t.wg + (size_t)t.k0 * (t.list == 1 ? gprF : gprD) + cg;
    };
    /* The group scales of row `tid` of a task, requested together with the task's digits -- a task ahead -- so
     * that the staging finds them in registers instead of waiting for HBM. Requested without conditions (a
     * dead position re-reads a live one); the staging zeroes what lies outside the matrix. */
    auto scales_ahead = [&](const DfT &t, float (&sc)[DF_NG]){
        const float *sp = scales_of(t) + (size_t)min(tid, t.rows - 1) * (t.list == 1 ? gprF : gprD);
#pragma unroll
        for(int gg = 0; gg < DF_NG; gg++) sc[gg] = sp[gg < t.ngl ? gg : 0];   /* a group past the row's end re-reads the first */
    };
    float csc[DF_NG];
    DF_STAMP(20);
    DfT cur = fetch();
    DF_STAMP(21);
    if(cur.list){
        const signed char *dp = df_digits<H>(a, cur); const int hs = cur.list == 1 ? hs1 : hs2;
        scales_ahead(cur, csc);
        df_load<H>(w0, dp, (size_t)cur.N >> 1, cur.rows, hs, 0);
        df_load<H>(w1, dp, (size_t)cur.N >> 1, cur.rows, hs, 1);
    }
    DF_STAMP(22);
    while(cur.list){
        const DfT nxt = fetch();
        DF_STAMP(23);
        /* after the last task the same loads go to the current task's digits again and are dropped */
        const DfT &pre = nxt.list ? nxt : cur;
        /* older than the digits requested below, so taking them over at the end of this task waits for nothing
         * that is still on its way */
        float nsc[DF_NG];
        scales_ahead(pre, nsc);
        const signed char *ndp = df_digits<H>(a, pre); const int nhs = pre.list == 1 ? hs1 : hs2;
        auto next0 = [&](){ df_load<H>(w0, ndp, (size_t)pre.N >> 1, pre.rows, nhs, 0); };
        auto next1 = [&](){ df_load<H>(w1, ndp, (size_t)pre.N >> 1, pre.rows, nhs, 1); };
        const int hs = cur.list == 1 ? hs1 : hs2;
        const int prob = cur.prob, chunk = cur.chunk, k0 = cur.k0, rows = cur.rows, M = cur.M;
        u64 *dst; size_t mstride;
        if(cur.list == 1){ dst = a.part1 + ((((size_t)prob * 2 + cur.mat) * a.S1 + cur.sl) * DF_MB) * a.F; mstride = (size_t)a.F; }
        else             { dst = a.part2 + (((size_t)prob * a.S2 + cur.sl) * DF_MB) * a.D;                  mstride = (size_t)a.D; }
        auto prep = [&]() -> float {
            /* thread = row of the task (rows <= DF_RMAX = the threads) */
            const int r = tid; const bool live = r < rows;
            float v[DF_NG][DF_MB];
            if(cur.list == 1){
                float xv[DF_MB];
#pragma unroll
                for(int m = 0; m < DF_MB; m++)
                    xv[m] = (live && m < M) ? a.x[(size_t)mt.rowtok[mt.p_row0[prob] + m] * a.D + k0 + r] : 0.0f;
#pragma unroll
                for(int gg = 0; gg < DF_NG; gg++){
                    const float sc = (gg < ng && chunk * DF_CW + gg * a.group < a.F) ? csc[gg] : 0.0f;
#pragma unroll
                    for(int m = 0; m < DF_MB; m++) v[gg][m] = xv[m] * sc;
                }
            } else {
                const u64 *p1 = a.part1 + (((size_t)prob * 2) * a.S1 * DF_MB) * a.F + k0;
                const size_t sstride = (size_t)DF_MB * a.F;
                /* with a full grid, one polling thread per producer first (everybody re-reading its sums until they
                 * are there slows the producers down: T=16 +0.6 us per layer); with few workgroups the poll and its
                 * barrier only add to the chain (T=1, 4: -0.3 us without) */
                if(lim1 * 2 > nslot) df_wait_first(2 * a.S1, a.epoch ^ a.wait_xor, a.spin_limit, &giveup, a.status, [=](int i){ return p1 + (size_t)i * sstride; });
                float hv[DF_MB];
#pragma unroll
                for(int m = 0; m < DF_MB; m++) hv[m] = 0.0f;
                if(live){
                    /* h = silu(gate) * up (k_swiglu, cudalm.cu:2430-2432), both summed over the K slices in order.
                     * The sums of both input rows are read in one round trip (a second row that does not exist
                     * re-reads the first: its words are never written). */
                    const u64 *src[2 * DF_MB];
#pragma unroll
                    for(int m = 0; m < DF_MB; m++){
                        const int mm = m < M ? m : 0;
                        src[2 * m] = p1 + (size_t)mm * a.F + r; src[2 * m + 1] = p1 + (size_t)a.S1 * sstride + (size_t)mm * a.F + r;
                    }
                    float gu[2 * DF_MB];
                    if(a.S1 <= 3) df_sum_wait<2 * DF_MB, 3>(src, sstride, a.S1, a.epoch ^ a.wait_xor, a.spin_limit, &giveup, a.status, gu);
                    else          df_sum_wait<2 * DF_MB, 6>(src, sstride, a.S1, a.epoch ^ a.wait_xor, a.spin_limit, &giveup, a.status, gu);
#pragma unroll
                    for(int m = 0; m < DF_MB; m++)
                        if(m < M) hv[m] = (gu[2 * m] / (1.0f + expf(-gu[2 * m]))) * gu[2 * m + 1];
                }
#pragma unroll
                for(int gg = 0; gg < DF_NG; gg++){
                    const float sc = (gg < ng && chunk * DF_CW + gg * a.group < a.D) ? csc[gg] : 0.0f;
#pragma unroll
                    for(int m = 0; m < DF_MB; m++) v[gg][m] = hv[m] * sc;
                }
            }
            if(H) return df_stage(v, live, (uint32_t (*)[DF_RMAX / 2][2 * DF_MB])xs_raw, wmax);
            return df_stage_f32(v, live, (float (*)[DF_RMAX][DF_MB])xs_raw);
        };
        /* the inner loop is compiled for 1 and 2 input rows */
        if(M == 1) df_task<H, 1>(a, cur, w0, w1, hs, xs_raw, red, dst, mstride, prep, next0, next1 DF_TRACE_ARG);
        else       df_task<H, 2>(a, cur, w0, w1, hs, xs_raw, red, dst, mstride, prep, next0, next1 DF_TRACE_ARG);
        cur = nxt;
#pragma unroll
        for(int gg = 0; gg < DF_NG; gg++) csc[gg] = nsc[gg];
    }
    DF_STAMP(3);
    /* ---- 3. out[n,:] += gate[k][n] * y[row(k,n),:], passes in order (cudalm.cu:4227). A pair whose
     * expert index was out of range adds nothing (the reference aborts the run, cudalm.cu:3476-3478). ---- */
    {
        const int ntask = a.T * a.NC2;
        for(int q3 = blockIdx.x; q3 < ntask; q3 += G){
            const int n = q3 / a.NC2, chunk = q3 - n * a.NC2;
            const int col = chunk * DF_CW + tid;
            if(col < a.D){
                float o = a.out[(size_t)n * a.D + col];
                /* two passes' sums per round trip; an invalid pair re-reads the other's words and adds nothing */
                for(int k = 0; k < a.K; k += 2){
                    const int j0 = k * a.T + n, j1 = min(k + 1, a.K - 1) * a.T + n;
                    const int prob0 = mt.pair_prob[j0], prob1 = k + 1 < a.K ? mt.pair_prob[j1] : -1;
                    if(prob0 < 0 && prob1 < 0) continue;
                    const int ja = prob0 >= 0 ? j0 : j1, jb = prob1 >= 0 ? j1 : j0;
                    const u64 *const src[2] = { a.part2 + (((size_t)mt.pair_prob[ja] * a.S2) * DF_MB + mt.pair_m[ja]) * a.D + col,
                                                a.part2 + (((size_t)mt.pair_prob[jb] * a.S2) * DF_MB + mt.pair_m[jb]) * a.D + col };
                    float y[2];
                    df_sum_wait<2, 12>(src, (size_t)DF_MB * a.D, a.S2, a.epoch ^ a.wait_xor, a.spin_limit, &giveup, a.status, y);
                    if(prob0 >= 0) o = o + a.gate[j0] * y[0];
                    if(prob1 >= 0) o = o + a.gate[j1] * y[1];
                }
                a.out[(size_t)n * a.D + col] = o;
            }
        }
    }
    DF_STAMP(4);
#ifdef QLMX_DF_TRACE
    __syncthreads();
    if(tid < DF_TRACE_EV && blockIdx.x < DF_TRACE_WG) df_trace_tab[blockIdx.x][tid] = df_ev[tid];
#endif
    /* the last workgroup to get here closes the call: clears the count and publishes the tag */
    if(tid == 0){
        const unsigned done = __hip_atomic_fetch_add(a.ctl + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if(done == gridDim.x - 1){
            __hip_atomic_store(a.ctl + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(a.ctl, a.epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Host side. Per device: the launch shape, a status word in pinned host memory, a grow-only
 * workspace for qlmx_moe_decode_forward, and the address of the fixed device array that
 * qlmx_moe_decode_forward_noalloc uses instead. All of it is set up by qlmx_init (nothing is
 * allocated by the entry points afterwards, except when the grow-only workspace has to grow).
 * ---------------------------------------------------------------------------------------- */
#define DF_CTL_BYTES 256
/* Scratch of the allocation-free entry point: control words, then both lists of tagged partial sums.
 * Every call on a device shares this one array; it is never cleared (words carry the tag of the call
 * that wrote them, and static device memory starts as zeros = "never written"). */
static __device__ __align__(256) unsigned char scratch[DF_CTL_BYTES + QLMX_DECODE_SCRATCH_BYTES];

struct DfSpace { u64 *part[2] = {nullptr, nullptr}; size_t words[2] = {0, 0}; unsigned *ctl = nullptr; };
struct DfDevice {
    bool ready = false;
    unsigned *status = nullptr;            /* pinned host word a kernel sets when a bounded wait ran out */
    int grid = 0;                          /* co-resident workgroups */
    unsigned char *fixed = nullptr;        /* device address of `scratch` on this device */
    DfSpace grown;                         /* qlmx_moe_decode_forward's workspace */
};
#define DF_MAX_DEVICES 16
static DfDevice g_dfdev[DF_MAX_DEVICES];

/* called by qlmx_init with `device` current */
int qlmx_decode_setup(int device){
    QLMX_REQUIRE(device >= 0 && device < DF_MAX_DEVICES, "decode setup: device %d is beyond the %d this library keeps state for", device, DF_MAX_DEVICES);
    DfDevice &dv = g_dfdev[device];
    if(dv.ready) return QLMX_OK;
    QLMX_HIP(hipHostMalloc((void **)&dv.status, 64, hipHostMallocDefault), "decode status word");
    *dv.status = 0;
    int nb = 0; hipDeviceProp_t pr;
    QLMX_HIP(hipGetDeviceProperties(&pr, device), "decode device properties");
    int nb32 = 0;
    QLMX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb, k_decode_fused<true>, DF_THREADS, 0), "decode occupancy");
    QLMX_HIP(hipOccupancyMaxActiveBlocksPerMultiprocessor(&nb32, k_decode_fused<false>, DF_THREADS, 0), "decode occupancy");
    if(nb32 < nb) nb = nb32;                  /* one grid size for both loops: every workgroup of a launch must be resident */
    if(nb > 4) nb = 4;
    dv.grid = (nb * pr.multiProcessorCount) & ~7;
    QLMX_REQUIRE(dv.grid >= 8, "decode setup: device too small (%d resident workgroups)", dv.grid);
    /* `scratch` names the array in host code; its memory on this device is wherever the loader put it */
    void *sym = nullptr;
    QLMX_HIP(hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)), "decode scratch address");
    dv.fixed = (unsigned char *)sym;
    QLMX_HIP(hipMalloc((void **)&dv.grown.ctl, DF_CTL_BYTES), "decode control words");
    QLMX_HIP(hipMemset(dv.grown.ctl, 0, DF_CTL_BYTES), "decode control words clear");
    dv.ready = true;
    return QLMX_OK;
}

/* tagged partial sums: grow-only, cleared when (re)allocated so that no word carries a live tag */
static int df_reserve(DfSpace &ws, int which, size_t words, hipStream_t st){
    if(words <= ws.words[which]) return QLMX_OK;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    QLMX_HIP(hipStreamIsCapturing(st, &cap), "decode capture query");
    QLMX_REQUIRE(cap == hipStreamCaptureStatusNone,
                 "qlmx_moe_decode_forward: the workspace would have to grow while the stream is being captured; run the largest "
                 "shape once outside the capture first, or use qlmx_moe_decode_forward_noalloc");
    QLMX_HIP(hipStreamSynchronize(st), "decode workspace sync");
    if(ws.part[which]) QLMX_HIP(hipFree(ws.part[which]), "decode workspace free");
    ws.part[which] = nullptr; ws.words[which] = 0;
    QLMX_HIP(hipMalloc((void **)&ws.part[which], words * sizeof(u64)), "decode partial sums");
    QLMX_HIP(hipMemset(ws.part[which], 0, words * sizeof(u64)), "decode partial sums clear");
    ws.words[which] = words;
    return QLMX_OK;
}

/* Rows per task of list 1: 256 keeps the per-task fixed cost (staging, reduction, hand-over) small against
 * the streaming part; the slices are halved only while they leave fewer than 0.15 x the grid with a gate|up task
 * (a single token: 128 rows, 192 tasks). More, shorter slices cost the down tasks a second round trip for their
 * sums: measured at E=32 D=768 F=2048 top-2, rows 256 / 128 / 64 give 16.3 / 15.6 / 18.2 us per layer for one
 * token, 18.8 / 21.4 / 26.4 for four, 29.7 / 32.7 / 42.0 for sixteen. The number of problems is only known on the
 * device; the host uses the expected number of distinct experts hit by `npair` uniform picks out of E. */
static int df_rows(int Kdim, double tasks_per_slice, int grid){
    int R = DF_RMAX;
    while(R > 64 && tasks_per_slice * ((Kdim + R - 1) / R) < 0.15 * grid) R >>= 1;
    while((Kdim + R - 1) / R > 32 && R < DF_RMAX) R <<= 1;
    return R;
}
/* Rows per task of list 2 (a multiple of 64, two halves of whole 32-row steps): as many slices of the contraction as still leave one task per
 * resident workgroup -- a second round of tasks would double the list's time -- but at most 12, which is what
 * the combine reads in one round trip, and none shorter than 64 rows. */
static int df_rows_down(int Kdim, double tasks_per_slice, int grid){
    int S = tasks_per_slice > 0.0 ? (int)(0.95 * grid / tasks_per_slice) : 1;
    const int smin = (Kdim + DF_RMAX - 1) / DF_RMAX, smax = Kdim >= 64 ? Kdim / 64 : 1;
    if(S > 12) S = 12;
    if(S > smax) S = smax;
    if(S < smin) S = smin;
    int R = ((Kdim + S - 1) / S + 63) & ~63;
    if(R > DF_RMAX) R = DF_RMAX;
    return R;
}

/* Which multiply loop the decode layer runs. fp32 (the default): inputs as they are, 2.6 / 3.6 vector
 * instructions per digit for one / two input rows, 4e-7 relative L2 on a layer's output against the fp32 oracle.
 * fp16 inputs: the staged inputs as fp16 pairs and v_dot2_f32_f16, 1.4 / 2.0 instructions per digit, inputs
 * rounded to 11 bits (3.7e-4), 1-4 % faster per layer (the layer is bound by its chain of hand-overs and by HBM,
 * not by this loop). QLMX_DECODE_MATH=fp16 in the environment (read at the first call) or qlmx_decode_math(1)
 * selects the fp16 loop, qlmx_decode_math(0) the fp32 one. */
static int g_df_math = -1;
static bool df_math_fp16(){
    if(g_df_math < 0){ const char *e = getenv("QLMX_DECODE_MATH"); g_df_math = (e && !strcmp(e, "fp16")) ? 1 : 0; }
    return g_df_math != 0;
}
extern "C" int qlmx_decode_math(int fp16_inputs){
    QLMX_REQUIRE(fp16_inputs == 0 || fp16_inputs == 1, "qlmx_decode_math: 0 (fp32 loop) or 1 (fp16 inputs), not %d", fp16_inputs);
    g_df_math = fp16_inputs;
    return QLMX_OK;
}

/* Both entry points: checks, launch shape, workspace (`fixed`: the static array, else the grow-only one), launch. */
static int df_forward(bool fixed, const char *who, const float *x, const int *assign, const float *gate, float *out,
                      const signed char *d, const float *s, int group, u64 w1q, u64 w3q, u64 w2q,
                      int T, int K, int E, int D, int F, hipStream_t st){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(x && assign && gate && out && d && s, "%s: NULL buffer", who);
    QLMX_REQUIRE(T > 0 && K > 0 && E > 0, "%s: T=%d K=%d E=%d", who, T, K, E);
    if(T * K > DEC_MAXPAIR){ qlmx_set_error("%s: %d (pass, token) pairs exceed the limit of %d", who, T * K, DEC_MAXPAIR); return QLMX_E_LIMIT; }
    QLMX_REQUIRE(D % 32 == 0 && F % 32 == 0 && D <= 8192 && F <= 8192, "%s: D=%d F=%d must be multiples of 32, at most 8192", who, D, F);
    QLMX_REQUIRE(group == 128 || (group > 0 && group % DF_CW == 0), "%s: group %d is not supported (128 or a multiple of 256)", who, group);
    QLMX_REQUIRE(F % group == 0 && D % group == 0, "%s: group %d must divide D and F", who, group);
    QLMX_REQUIRE(w1q % group == 0 && w3q % group == 0 && w2q % group == 0 && ((uintptr_t)d & 15) == 0,
                 "%s: weight offsets must be multiples of the group and the digit array 16-byte aligned", who);
    int device = -1;
    QLMX_HIP(hipGetDevice(&device), "decode device");
    QLMX_REQUIRE(device >= 0 && device < DF_MAX_DEVICES && g_dfdev[device].ready, "%s: qlmx_init has not run for device %d", who, device);
    DfDevice &dv = g_dfdev[device];
    if(*(volatile unsigned *)dv.status){
        *dv.status = 0;
        qlmx_set_error("%s: an earlier decode call gave up waiting for a task of its own grid; its output is invalid", who);
        return QLMX_E_HIP;
    }
    const int npair = T * K;
    DfArgs a;
    a.x = x; a.assign = assign; a.gate = gate; a.out = out; a.d = d; a.s = s; a.w1q = w1q; a.w3q = w3q; a.w2q = w2q; a.group = group;
    a.w1g = w1q / group; a.w3g = w3q / group; a.w2g = w2q / group; a.dfg = (u64)D * F / group;
    a.T = T; a.K = K; a.E = E; a.D = D; a.F = F;
    a.NC1 = (F + DF_CW - 1) / DF_CW; a.NC2 = (D + DF_CW - 1) / DF_CW;
    const double hits = E * (1.0 - pow(1.0 - 1.0 / E, (double)npair));
    a.R1 = df_rows(D, 2.0 * hits * a.NC1, dv.grid); a.S1 = (D + a.R1 - 1) / a.R1;
    a.R2 = df_rows_down(F, hits * a.NC2, dv.grid);   a.S2 = (F + a.R2 - 1) / a.R2;
    const size_t words1 = (size_t)npair * 2 * a.S1 * DF_MB * F, words2 = (size_t)npair * a.S2 * DF_MB * D;
    if(fixed){
        if((words1 + words2) * sizeof(u64) > (size_t)QLMX_DECODE_SCRATCH_BYTES){
            qlmx_set_error("%s: T=%d K=%d D=%d F=%d needs %zu bytes of partial sums, the fixed scratch holds %zu",
                           who, T, K, D, F, (words1 + words2) * sizeof(u64), (size_t)QLMX_DECODE_SCRATCH_BYTES);
            return QLMX_E_LIMIT;
        }
        a.ctl = (unsigned *)dv.fixed;
        a.part1 = (u64 *)(dv.fixed + DF_CTL_BYTES); a.part2 = a.part1 + words1;
    } else {
        rc = df_reserve(dv.grown, 0, words1, st); if(rc) return rc;
        rc = df_reserve(dv.grown, 1, words2, st); if(rc) return rc;
        a.ctl = dv.grown.ctl; a.part1 = dv.grown.part[0]; a.part2 = dv.grown.part[1];
    }
    /* n groups left over after the last full round of 8: the number of pieces (a divisor of the chunk count) that
     * leaves the fullest XCD with the fewest chunks, the smallest such number */
    a.parts1 = 0; a.parts2 = 0;
    for(int n = 0; n < 8; n++){
        auto pieces = [&](int NC){
            int best = 1, load = NC;
            for(int c = 1; c <= NC && n > 0; c++) if(NC % c == 0){ const int l = ((n * c + 7) / 8) * (NC / c); if(l < load){ load = l; best = c; } }
            return best; };
        a.parts1 |= (u64)pieces(a.NC1) << (8 * n); a.parts2 |= (u64)pieces(a.NC2) << (8 * n);
    }
    a.status = dv.status; a.epoch = 0;
    a.wait_xor = 0; a.spin_limit = DF_SPIN_LIMIT;
    if(qlmx_test_take_forced_timeout(1)){ a.wait_xor = 0x40000000u; a.spin_limit = 0; }
    const long long most = (long long)2 * npair * a.NC1 * a.S1;
    const int grid = (int)std::min<long long>(dv.grid, (most + 7) & ~7LL);
    {   /* a workgroup lists its tasks once, one candidate per thread: bound them for the worst case (every pair its own expert) */
        const long long nslot = grid / 8;
        const long long lim1 = ((2LL * npair + 7) / 8) * a.NC1 * a.S1, lim2 = (((long long)npair + 7) / 8) * a.NC2 * a.S2;
        const long long cand = (lim1 + nslot - 1) / nslot + (lim2 + nslot - 1) / nslot;
        if(cand > DF_MAXTASKS){
            qlmx_set_error("%s: T=%d K=%d D=%d F=%d gives a workgroup up to %lld tasks, more than the %d it can list", who, T, K, D, F, cand, DF_MAXTASKS);
            return QLMX_E_LIMIT;
        }
    }
    if(df_math_fp16()) hipLaunchKernelGGL(k_decode_fused<true>, dim3(grid), dim3(DF_THREADS), 0, st, a);
    else               hipLaunchKernelGGL(k_decode_fused<false>, dim3(grid), dim3(DF_THREADS), 0, st, a);
    QLMX_LAUNCH_CHECK("decode launch");
    return QLMX_OK;
}

/* Host-only query for callers whose decode launches do not pass through df_forward (HIP-graph replays): reads
 * and clears the pinned word a launch sets when one of its bounded waits gave up. No GPU call. */
extern "C" int qlmx_decode_status(void){
    int rc = qlmx_check_ready(); if(rc) return rc;
    int device = -1;
    QLMX_HIP(hipGetDevice(&device), "decode device");
    QLMX_REQUIRE(device >= 0 && device < DF_MAX_DEVICES && g_dfdev[device].ready, "qlmx_decode_status: qlmx_init has not run for device %d", device);
    DfDevice &dv = g_dfdev[device];
    if(*(volatile unsigned *)dv.status){
        *dv.status = 0;
        qlmx_set_error("qlmx_decode_status: a decode launch gave up waiting for a task of its own grid; its output is invalid");
        return QLMX_E_HIP;
    }
    return QLMX_OK;
}

#ifdef QLMX_DF_TRACE
extern "C" int qlmx_debug_trace(unsigned long long *host, int words){
    if(words > DF_TRACE_WG * DF_TRACE_EV) words = DF_TRACE_WG * DF_TRACE_EV;
    QLMX_HIP(hipMemcpyFromSymbol(host, HIP_SYMBOL(df_trace_tab), (size_t)words * 8), "trace copy");
    return QLMX_OK;
}
#endif

extern "C" int qlmx_moe_decode_forward(const float *x, const int *assign, const float *gate, float *out,
                                       const signed char *d, const float *s, int group,
                                       unsigned long long w1q, unsigned long long w3q, unsigned long long w2q,
                                       int T, int K, int E, int D, int F, void *stream){
    return df_forward(false, "qlmx_moe_decode_forward", x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, (hipStream_t)stream);
}

/* The same layer over the fixed device array: no hipMalloc, hipFree or other allocating call on any path. */
extern "C" int qlmx_moe_decode_forward_noalloc(const float *x, const int *assign, const float *gate, float *out,
                                               const signed char *d, const float *s, int group,
                                               unsigned long long w1q, unsigned long long w3q, unsigned long long w2q,
                                               int T, int K, int E, int D, int F, void *stream){
    return df_forward(true, "qlmx_moe_decode_forward_noalloc", x, assign, gate, out, d, s, group, w1q, w3q, w2q, T, K, E, D, F, (hipStream_t)stream);
}
