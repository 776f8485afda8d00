/* qlmx_gemv.hip -- few-row expert GEMV over packed 4-bit weights (decode shape), bound by HBM.
 *
 * Serves the reference's decode step, where moe_forward runs on N = batch rows (dec_step,
 * cudalm.cu:7163-7204) and each expert GEMM of cudalm.cu:4211-4225 has at most a few rows: the
 * work is one pass over the hit experts' digits and scales. Also the small-row path of
 * qlmx_moe_gemm_nn (the reference's CPU SGEMM has the same split at R<=4, cpu_rt.h:233-258).
 *
 * y[m, n] = sum_k x[m, k] * s[k, n/group] * digit[k, n], W row-major [K, N].
 *
 * Mapping. A thread owns one 16-byte chunk column (32 consecutive n) and walks down the rows of
 * its workgroup's K-slice; consecutive threads own consecutive chunks, and when a row is narrower
 * than the workgroup the next threads continue on the following rows, so every load instruction
 * of a wave covers one contiguous 1 KiB of the weight matrix. Per chunk: xor 0x88888888 turns the
 * two's-complement nibbles into offset-8 bytes, two masks split even and odd nibbles, the
 * byte-to-float converts feed fp32 FMAs against x*s, and the offset (8 * sum of x*s) is taken out
 * once per row. The K dimension is split over workgroups for parallelism; slices leave partial sums
 * in a scratch buffer and whoever consumes them (the next stage's prologue, the combine kernel or
 * the finishing kernel) adds them in slice order, so results do not depend on scheduling and no
 * workgroup ever waits for another.
 *
 * Algorithmic HBM bytes per expert hit: K*N/2 digits + K*N/group*4 scales per matrix
 * (D=768, F=2048, three matrices: 2,506,752 B).
 */
#include "qlmx_gemm.h"
#include <math.h>
#include <algorithm>

#define GV_THREADS 256
#define GV_MAXROWS 4          /* rows per problem (larger row counts are split by the callers) */
#define GV_MAXSLICE 512       /* K rows per workgroup slice held in LDS */
#define GV_BATCH 4            /* rows a thread has in flight */

enum { PRO_ROWS = 0, PRO_SWIGLU = 1 };   /* where a problem's input rows come from */

struct GvProb {               /* 64 bytes */
    const float *x[GV_MAXROWS];   /* PRO_ROWS: the input rows (each K floats) */
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
    const float *prev; int prevS;                    /* PRO_SWIGLU: partial sums of the gate|up stage (its N == this K) */
};

__device__ __forceinline__ float ub(uint32_t w, int k){ return (float)((w >> (8 * k)) & 0xFFu); }
/* position of output column n inside a partial-sum row (natural order) */
__device__ __forceinline__ int part_index(int n, int){ return n; }

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

template<int PRO, int MR>
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
        if(m < PM && kb0 + r < kb1){
            if(PRO == PRO_ROWS) v = Pp->x[m][kb0 + r];
            else {
                /* x = silu(gate) * up, both summed over the previous stage's slices in slice order
                 * (k_swiglu, cudalm.cu:2430-2432) */
                const int ix = part_index(kb0 + r, a.K);
                const float *g0 = a.prev + (((size_t)(2 * p) * a.prevS) * MR + m) * a.K + ix;
                const float *u0 = a.prev + (((size_t)(2 * p + 1) * a.prevS) * MR + m) * a.K + ix;
                const float g = sum_slices(g0, (size_t)MR * a.K, a.prevS), u = sum_slices(u0, (size_t)MR * a.K, a.prevS);
                v = (g / (1.0f + expf(-g))) * u;
            }
        }
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
    const int ix = part_index(n, N);
    for(int m = 0; m < M; m++){
        const float *src = part + (((size_t)p * S) * MR + m) * N + ix;
        out[(size_t)m * N + n] = sum_slices(src, (size_t)MR * N, S);
    }
}

/* ------------------------------------------------------------------------------------------
 * Workspace owned by the library (grow-only): partial sums, device problem tables and the row maps
 * of the fused decode layer.
 * ---------------------------------------------------------------------------------------- */
struct GvWorkspace {
    float *part[2] = {nullptr, nullptr}; size_t part_floats[2] = {0, 0};
    GvProb *prob = nullptr;                 /* device problem table of the decode path: 2 x 64 */
    int *meta = nullptr;
};
static GvWorkspace g_ws;

static int ws_reserve(int which, size_t floats, hipStream_t st){
    if(!g_ws.prob){
        QLMX_HIP(hipMalloc((void **)&g_ws.prob, 2 * 64 * sizeof(GvProb)), "gemv problem table");
        QLMX_HIP(hipMalloc((void **)&g_ws.meta, 512 * sizeof(int)), "gemv meta");
    }
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

template<int PRO, int MR>
static int launch_gemv(GvArgs &a, int ntask_max, hipStream_t st){
    hipLaunchKernelGGL((k_qlmx_gemv<PRO, MR>), dim3(a.S, ntask_max), dim3(GV_THREADS), 0, st, a);
    QLMX_LAUNCH_CHECK("gemv launch");
    return QLMX_OK;
}

/* ---- small-row path of qlmx_moe_gemm_nn (fp32 activations, every problem M <= GV_MAXROWS) ---- */
int qlmx_gemv_nn_dispatch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                          int K, int N, hipStream_t st){
    QLMX_REQUIRE(N % 32 == 0 && group % 32 == 0, "gemv: N and group must be multiples of 32");
    QLMX_REQUIRE(((uintptr_t)d & 15) == 0, "gemv: digit array must be 16-byte aligned");
    static GvProb *h_tab = nullptr, *d_tab = nullptr; static hipEvent_t ev; static bool used = false;
    if(!h_tab){
        QLMX_HIP(hipHostMalloc((void **)&h_tab, QLMX_MAX_PROBLEMS * sizeof(GvProb), hipHostMallocDefault), "gemv table (pinned)");
        QLMX_HIP(hipMalloc((void **)&d_tab, QLMX_MAX_PROBLEMS * sizeof(GvProb)), "gemv table (device)");
        QLMX_HIP(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "gemv table event");
    }
    if(used) QLMX_HIP(hipEventSynchronize(ev), "gemv table wait");
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
    a.nmat = 1; a.mat_dq = 0; a.mat_dg = 0; a.prev = nullptr; a.prevS = 0;
    choose_split(K, N, n, &a.S, &a.rps);
    int rc = ws_reserve(0, (size_t)n * a.S * GV_MAXROWS * N, st); if(rc) return rc;
    a.part = g_ws.part[0];
    QLMX_HIP(hipMemcpyAsync(d_tab, h_tab, (size_t)n * sizeof(GvProb), hipMemcpyHostToDevice, st), "gemv table h2d");
    rc = launch_gemv<PRO_ROWS, GV_MAXROWS>(a, n, st); if(rc) return rc;
    hipLaunchKernelGGL(k_qlmx_gemv_finish<GV_MAXROWS>, dim3((N + 255) / 256, n), dim3(256), 0, st, d_tab, g_ws.part[0], a.S, N);
    QLMX_LAUNCH_CHECK("gemv finish launch");
    QLMX_HIP(hipEventRecord(ev, st), "gemv table record"); used = true;
    return QLMX_OK;
}

/* ------------------------------------------------------------------------------------------
 * Fused decode layer
 * ---------------------------------------------------------------------------------------- */
#define DEC_MAXPAIR 64
/* meta layout (ints): [0] nprob, [1] invalid-expert flag, [8 + j] row of pair j,
 * [8 + 64 + r] pair of row r, [8 + 128 + r] problem*GV_MAXROWS + row-in-problem of row r */

/* Groups the (pass, token) pairs by expert: a stable counting sort over j = k*T + n, i.e. rows are
 * ordered by (expert, pass, token), the order of the reference's host permutation
 * (cudalm.cu:3586-3599) applied to the merged passes. Experts with more than MR rows are cut into
 * several problems. One wavefront, lane j owns pair j; ranks come from 64 lane broadcasts, so no
 * serial chain of global-memory round trips sits in front of the first GEMV. */
template<int MR>
__global__ void __launch_bounds__(64) k_decode_group(const int *assign, int npair, int T, int E, int D, int F,
                               const float *x, unsigned long long w1q, unsigned long long w2q, int group,
                               GvProb *prob1, GvProb *prob2, int *meta){
    __shared__ int rowpair[DEC_MAXPAIR], isstart[DEC_MAXPAIR];
    const int j = threadIdx.x;
    const bool live = j < npair;
    int e = live ? assign[j] : 0x7FFFFFFF;
    const bool bad = live && (unsigned)e >= (unsigned)E;
    if(bad) e = 0x7FFFFFFE;                               /* sorts after every valid expert */
    int rank = 0, pos = 0, cnt = 0;
    for(int i = 0; i < DEC_MAXPAIR; i++){
        const int ei = __shfl(e, i, 64);
        rank += (ei < e) || (ei == e && i < j);
        pos  += (ei == e && i < j);
        cnt  += (ei == e);
    }
    isstart[j] = 0;
    __syncthreads();
    const bool start = live && !bad && (pos % MR == 0);
    if(live && !bad){ rowpair[rank] = j; isstart[rank] = start ? 1 : 0; meta[8 + j] = rank; meta[8 + DEC_MAXPAIR + rank] = j; }
    if(bad) meta[8 + j] = -1;
    __syncthreads();
    if(live && !bad){
        const int first = rank - (pos % MR);              /* row of the problem's first pair */
        int np = 0;
        for(int r = 0; r < first; r++) np += isstart[r];
        meta[8 + 2 * DEC_MAXPAIR + rank] = np * GV_MAXROWS + (pos % MR);
        if(start){
            const int M = min(MR, cnt - pos);
            GvProb g1, g2;
#pragma unroll
            for(int m = 0; m < GV_MAXROWS; m++){
                g1.x[m] = nullptr; g2.x[m] = nullptr;
                if(m < M) g1.x[m] = x + (size_t)(rowpair[rank + m] % T) * D;
            }
            const unsigned long long eo = (unsigned long long)e * D * F;
            g1.out = nullptr; g1.wq = w1q + eo; g1.wg = (w1q + eo) / group; g1.M = M; g1.pad = 0;
            g2.out = nullptr; g2.wq = w2q + eo; g2.wg = (w2q + eo) / group; g2.M = M; g2.pad = 0;
            prob1[np] = g1; prob2[np] = g2;
        }
    }
    const unsigned long long sm = __ballot(start), bm = __ballot(bad);
    if(j == 0){ meta[0] = __popcll(sm); meta[1] = bm ? 1 : 0; }
}

/* out[n,:] += gate[k][n] * y[row(k,n),:], passes in order (cudalm.cu:4227); y is summed here from
 * the down-projection's slices in slice order. A pair whose expert index was out of range adds
 * nothing (the reference aborts the run in that case, cudalm.cu:3476-3478). */
template<int MR>
__global__ void __launch_bounds__(256) k_decode_combine(const float *part, int S, const float *gate, const int *meta,
                                                        float *out, int T, int K, int D){
    const int n = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
    if(c >= D) return;
    const int ix = part_index(c, D);
    float o = out[(size_t)n * D + c];
    for(int k = 0; k < K; k++){
        const int j = k * T + n, row = meta[8 + j];
        if(row < 0) continue;
        const int pm = meta[8 + 2 * DEC_MAXPAIR + row], p = pm / GV_MAXROWS, m = pm - p * GV_MAXROWS;
        const float *src = part + (((size_t)p * S) * MR + m) * D + ix;
        const float y = sum_slices(src, (size_t)MR * D, S);
        o = o + gate[j] * y;
    }
    out[(size_t)n * D + c] = o;
}

extern "C" int qlmx_moe_decode_forward(const float *x, const int *assign, const float *gate, float *out,
                                       const signed char *d, const float *s, int group,
                                       unsigned long long w1q, unsigned long long w3q, unsigned long long w2q,
                                       int T, int K, int E, int D, int F, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    QLMX_REQUIRE(x && assign && gate && out && d && s, "qlmx_moe_decode_forward: NULL buffer");
    QLMX_REQUIRE(T > 0 && K > 0 && E > 0 && E <= 256, "qlmx_moe_decode_forward: T=%d K=%d E=%d", T, K, E);
    if(T * K > DEC_MAXPAIR){ qlmx_set_error("qlmx_moe_decode_forward: %d (pass, token) pairs exceed the limit of %d", T * K, DEC_MAXPAIR); return QLMX_E_LIMIT; }
    QLMX_REQUIRE(D % 32 == 0 && F % 32 == 0 && D <= 8192 && F <= 8192, "qlmx_moe_decode_forward: D=%d F=%d must be multiples of 32, at most 8192", D, F);
    QLMX_REQUIRE(group % 32 == 0 && F % group == 0 && D % group == 0, "qlmx_moe_decode_forward: group %d must divide D and F", group);
    QLMX_REQUIRE(w1q % 32 == 0 && w3q % 32 == 0 && w2q % 32 == 0 && ((uintptr_t)d & 15) == 0, "qlmx_moe_decode_forward: weight offsets must be multiples of 32 elements");
    QLMX_REQUIRE(w3q >= w1q, "qlmx_moe_decode_forward: w3 must follow w1 in the digit array");
    const int npair = T * K;
    const int MR = T == 1 ? 1 : 2;
    GvArgs a1, a2;
    a1.nmat = 2; a2.nmat = 1;
    choose_split(D, F, 2 * npair, &a1.S, &a1.rps);
    choose_split(F, D, npair, &a2.S, &a2.rps);
    rc = ws_reserve(0, (size_t)npair * 2 * a1.S * MR * F, st); if(rc) return rc;
    rc = ws_reserve(1, (size_t)npair * a2.S * MR * D, st); if(rc) return rc;
    GvProb *p1 = g_ws.prob, *p2 = g_ws.prob + 64;
    if(MR == 1) hipLaunchKernelGGL(k_decode_group<1>, dim3(1), dim3(64), 0, st, assign, npair, T, E, D, F, x, w1q, w2q, group, p1, p2, g_ws.meta);
    else        hipLaunchKernelGGL(k_decode_group<2>, dim3(1), dim3(64), 0, st, assign, npair, T, E, D, F, x, w1q, w2q, group, p1, p2, g_ws.meta);
    QLMX_LAUNCH_CHECK("decode group launch");
    a1.pr = p1; a1.nprob_dev = g_ws.meta; a1.nprob = npair; a1.d = d; a1.s = s; a1.group = group; a1.K = D; a1.N = F;
    a1.mat_dq = w3q - w1q; a1.mat_dg = (w3q - w1q) / group; a1.part = g_ws.part[0]; a1.prev = nullptr; a1.prevS = 0;
    a2.pr = p2; a2.nprob_dev = g_ws.meta; a2.nprob = npair; a2.d = d; a2.s = s; a2.group = group; a2.K = F; a2.N = D;
    a2.mat_dq = 0; a2.mat_dg = 0; a2.part = g_ws.part[1]; a2.prev = g_ws.part[0]; a2.prevS = a1.S;
    const dim3 cg((D + 255) / 256, T);
    if(MR == 1){
        rc = launch_gemv<PRO_ROWS, 1>(a1, 2 * npair, st); if(rc) return rc;
        rc = launch_gemv<PRO_SWIGLU, 1>(a2, npair, st); if(rc) return rc;
        hipLaunchKernelGGL(k_decode_combine<1>, cg, dim3(256), 0, st, g_ws.part[1], a2.S, gate, g_ws.meta, out, T, K, D);
    } else {
        rc = launch_gemv<PRO_ROWS, 2>(a1, 2 * npair, st); if(rc) return rc;
        rc = launch_gemv<PRO_SWIGLU, 2>(a2, npair, st); if(rc) return rc;
        hipLaunchKernelGGL(k_decode_combine<2>, cg, dim3(256), 0, st, g_ws.part[1], a2.S, gate, g_ws.meta, out, T, K, D);
    }
    QLMX_LAUNCH_CHECK("decode combine launch");
    return QLMX_OK;
}
