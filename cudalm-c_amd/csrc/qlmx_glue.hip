/* qlmx_glue.hip -- the pieces of a top-K MoE layer that sit between the expert GEMMs: router,
 * grouping permutation, row gather / gated scatter, gate gradient, SwiGLU forward and backward.
 *
 * Reference: k_router_topk (cudalm.cu:2515-2534, CPU cpu_kern.h:413-425), k_gp_hist / k_gp_scan /
 * k_gp_scatter (cudalm.cu:3504-3530; the host form of the same permutation is 3586-3599),
 * k_gather / k_scatter_gate / k_gather4 / k_scatter_add4 (cudalm.cu:2536-2567, cpu_kern.h:426-450),
 * k_moe_dgate (cudalm.cu:2591, cpu_kern.h:454-468), k_swiglu / k_swiglu_bwd (cudalm.cu:2430-2453,
 * cpu_kern.h:376-394).
 *
 * Indices (assign, perm, off) and gate probabilities are part of the bit-exact contract: the
 * router restates the CPU build's polynomial exponential operation for operation (this file is
 * compiled without FMA contraction), sums the softmax in expert order, and breaks ties towards
 * the lower expert index; the permutation is the stable counting sort. Everything here is bound by
 * HBM: one read and one write per element, rows moved with 16-byte accesses.
 */
#include "qlmx_dev.h"
#include "qlmx_gemm.h"

/* ---- router: one thread per token, experts visited in order so the softmax sum rounds exactly as
 * the reference's loop does. `logit` points at the token's E logits and `pr` at E floats for its
 * probabilities (the two may be the same place). ---- */
__device__ __forceinline__ void route_token(const float *logit, float *pr, int n, int *assign, float *gate,
                                            int N, int E, int K, const float *bias, int bs){
    float mx = -1e30f;
    for(int e = 0; e < E; e++) if(logit[e] > mx) mx = logit[e];
    float sum = 0.0f;
    for(int e = 0; e < E; e++){ const float p = qx_fexp(logit[e] - mx); pr[e] = p; sum += p; }
    const float inv = 1.0f / sum;
    for(int e = 0; e < E; e++) pr[e] *= inv;
    int chosen[8];
    for(int k = 0; k < K; k++){
        int best = -1; float bestp = -1e30f;
        for(int e = 0; e < E; e++){
            bool taken = false;
#pragma unroll
            for(int j = 0; j < 8; j++) taken = taken || (j < k && chosen[j] == e);
            if(taken) continue;
            const float sc = pr[e] + (bias ? bias[k * bs + e] : 0.0f);
            if(sc > bestp){ bestp = sc; best = e; }
        }
        if(best < 0) best = k;
#pragma unroll
        for(int j = 0; j < 8; j++) if(j == k) chosen[j] = best;
        assign[(size_t)k * N + n] = best;
        gate[(size_t)k * N + n] = pr[best];
    }
}

/* rows straight from memory: consecutive threads are E floats apart, for any E */
__global__ void __launch_bounds__(256) k_router_topk(const float *rt, float *rprobs, int *assign, float *gate,
                                                     int N, int E, int K, const float *bias, int bs){
    const int n = blockIdx.x * 256 + threadIdx.x;
    if(n >= N) return;
    route_token(rt + (size_t)n * E, rprobs + (size_t)n * E, n, assign, gate, N, E, K, bias, bs);
}

/* The rows of RT_TOK consecutive tokens are one contiguous piece of `rt`: it is copied to LDS with
 * consecutive threads on consecutive floats, each thread then routes its token out of LDS (rows an odd
 * number of floats apart, so the lanes of a wavefront hit different banks), and the probabilities go
 * back the way the logits came. Same arithmetic in the same order as the kernel above. */
#define RT_TOK 64
#define RT_MAXE 96
__global__ void __launch_bounds__(RT_TOK) k_router_topk_lds(const float *rt, float *rprobs, int *assign, float *gate,
                                                            int N, int E, int K, const float *bias, int bs){
    extern __shared__ float rows[];
    const int n0 = blockIdx.x * RT_TOK, tid = threadIdx.x;
    const int ld = E | 1;
    const int cnt = min(RT_TOK, N - n0) * E;
    const float *src = rt + (size_t)n0 * E;
    int t = tid / E, e = tid - t * E;
    const int dt = RT_TOK / E, de = RT_TOK - dt * E;
    for(int i = tid; i < cnt; i += RT_TOK){
        rows[t * ld + e] = src[i];
        t += dt; e += de; if(e >= E){ e -= E; t++; }
    }
    __syncthreads();
    if(n0 + tid < N) route_token(rows + tid * ld, rows + tid * ld, n0 + tid, assign, gate, N, E, K, bias, bs);
    __syncthreads();
    float *dst = rprobs + (size_t)n0 * E;
    t = tid / E; e = tid - t * E;
    for(int i = tid; i < cnt; i += RT_TOK){
        dst[i] = rows[t * ld + e];
        t += dt; e += de; if(e >= E){ e -= E; t++; }
    }
}

/* Expert count known at compile time (at most 64): the token's row lives in registers between the
 * staged load and the staged store, the chosen experts in a bit mask. Same operations in the same
 * order as route_token. */
template<int EE>
__global__ void __launch_bounds__(RT_TOK) k_router_topk_reg(const float *rt, float *rprobs, int *assign, float *gate,
                                                            int N, int K, const float *bias, int bs){
    __shared__ float rows[RT_TOK * (EE | 1)];
    constexpr int ld = EE | 1;
    const int n0 = blockIdx.x * RT_TOK, tid = threadIdx.x;
    const int cnt = min(RT_TOK, N - n0) * EE;
    const float *src = rt + (size_t)n0 * EE;
    for(int i = tid; i < cnt; i += RT_TOK) rows[(i / EE) * ld + (i % EE)] = src[i];
    __syncthreads();
    const int n = n0 + tid;
    if(n < N){
        float p[EE];
#pragma unroll
        for(int e = 0; e < EE; e++) p[e] = rows[tid * ld + e];
        float mx = -1e30f;
#pragma unroll
        for(int e = 0; e < EE; e++) if(p[e] > mx) mx = p[e];
        float sum = 0.0f;
#pragma unroll
        for(int e = 0; e < EE; e++){ p[e] = qx_fexp(p[e] - mx); sum += p[e]; }
        const float inv = 1.0f / sum;
#pragma unroll
        for(int e = 0; e < EE; e++){ p[e] *= inv; rows[tid * ld + e] = p[e]; }
        unsigned long long taken = 0ULL;
        for(int k = 0; k < K; k++){
            int best = -1; float bestp = -1e30f;
#pragma unroll
            for(int e = 0; e < EE; e++){
                const float sc = p[e] + (bias ? bias[k * bs + e] : 0.0f);
                if(!((taken >> e) & 1ULL) && sc > bestp){ bestp = sc; best = e; }
            }
            if(best < 0) best = k;
            taken |= 1ULL << best;
            float gv = 0.0f;
#pragma unroll
            for(int e = 0; e < EE; e++) if(e == best) gv = p[e];
            assign[(size_t)k * N + n] = best;
            gate[(size_t)k * N + n] = gv;
        }
    }
    __syncthreads();
    float *dst = rprobs + (size_t)n0 * EE;
    for(int i = tid; i < cnt; i += RT_TOK) dst[i] = rows[(i / EE) * ld + (i % EE)];
}

/* ---- grouping permutation of one pass: perm lists the tokens expert by expert, tokens of one
 * expert in ascending order; off[e] is the first row of expert e, off[E] = N.
 * Launches: clear, per-chunk histograms (which also add up the experts' totals), scan, stable placement. ---- */
#define GP_CHUNK 256
/* workspace: ch[K][NC][E] chunk histograms, then 4 ints (the first is the out-of-range flag), then
 * tot[K][E] per-expert totals */
__global__ void __launch_bounds__(256) k_gp_clear(int *bad, int ntot){
    for(int i = threadIdx.x; i < 4 + ntot; i += 256) bad[i] = 0;
}
__global__ void __launch_bounds__(GP_CHUNK) k_gp_hist(const int *asn, int N, int E, int NC, int *ch, int *bad){
    extern __shared__ int hist[];
    const int c = blockIdx.x, k = blockIdx.y, n = c * GP_CHUNK + threadIdx.x;
    int *tot = bad + 4;
    for(int e = threadIdx.x; e < E; e += GP_CHUNK) hist[e] = 0;
    __syncthreads();
    if(n < N){
        const int e = asn[(size_t)k * N + n];
        if((unsigned)e >= (unsigned)E) atomicExch(bad, -1 - e); else atomicAdd(&hist[e], 1);
    }
    __syncthreads();
    for(int e = threadIdx.x; e < E; e += GP_CHUNK){
        const int h = hist[e];
        ch[((size_t)k * NC + c) * E + e] = h;
        if(h) atomicAdd(&tot[(size_t)k * E + e], h);
    }
}
__device__ __forceinline__ int wave_incl_scan(int v, int lane){
#pragma unroll
    for(int d = 1; d < 64; d <<= 1){ const int u = __shfl_up(v, d, 64); if(lane >= d) v += u; }
    return v;
}
/* one wavefront per (pass, expert), and one more per pass for off[E]: the expert's first row is the
 * sum of the totals of the experts before it; ch[k][c][e] becomes the first output row of
 * (chunk c, expert e), 64 chunks per scan step */
__global__ void __launch_bounds__(256) k_gp_scan(int *ch, const int *tot, int E, int NC, int *off){
    const int k = blockIdx.y, lane = threadIdx.x & 63, e = blockIdx.x * 4 + (threadIdx.x >> 6);
    if(e > E) return;
    int base = 0;
    for(int j0 = 0; j0 < e; j0 += 64){
        const int j = j0 + lane;
        base += j < e ? tot[(size_t)k * E + j] : 0;
    }
#pragma unroll
    for(int d = 32; d >= 1; d >>= 1) base += __shfl_xor(base, d, 64);
    if(lane == 0) off[(size_t)k * (E + 1) + e] = base;
    if(e == E) return;
    int *col = ch + (size_t)k * NC * E + e;
    int run = base;
    for(int c0 = 0; c0 < NC; c0 += 64){
        const int c = c0 + lane;
        const int t = c < NC ? col[(size_t)c * E] : 0;
        const int incl = wave_incl_scan(t, lane);
        if(c < NC) col[(size_t)c * E] = run + incl - t;
        run += __shfl(incl, 63, 64);
    }
}
/* stable placement: a token's row = start of (its chunk, its expert) + the number of earlier
 * tokens of the chunk with the same expert. Inside a wavefront that number is a population count
 * over the lanes that share the expert; the four wavefronts add up in order through LDS. */
__global__ void __launch_bounds__(GP_CHUNK) k_gp_scatter(const int *asn, int N, int E, int NC, const int *co, int *perm){
    extern __shared__ int wcnt[];                       /* [4][E] */
    const int c = blockIdx.x, k = blockIdx.y, n = c * GP_CHUNK + threadIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for(int i = threadIdx.x; i < 4 * E; i += GP_CHUNK) wcnt[i] = 0;
    __syncthreads();
    int e = -1;
    if(n < N){ e = asn[(size_t)k * N + n]; if((unsigned)e >= (unsigned)E) e = -1; }
    int rank = 0;
    unsigned long long remaining = __ballot(e >= 0);
    while(remaining){
        const int leader = __ffsll((long long)remaining) - 1;
        const int e0 = __shfl(e, leader, 64);
        const unsigned long long m = __ballot(e == e0);
        if(e == e0){
            rank = __popcll(m & ((1ull << lane) - 1ull));
            if(lane == leader) wcnt[wave * E + e0] = __popcll(m);
        }
        remaining &= ~m;
    }
    __syncthreads();
    if(e >= 0){
        for(int w = 0; w < wave; w++) rank += wcnt[w * E + e];
        perm[(size_t)k * N + co[((size_t)k * NC + c) * E + e] + rank] = n;
    }
}

__global__ void __launch_bounds__(256) k_fill_i32(int *p, int v, int n){
    const int i = blockIdx.x * 256 + threadIdx.x;
    if(i < n) p[i] = v;
}

/* ---- row movers. One workgroup per row; D % 4 == 0. ---- */
template<bool OUT_BF16>
__global__ void __launch_bounds__(256) k_gather_rows(const float4 *src, const int *perm, void *Xp, int D4){
    const int j = blockIdx.x, n = perm[j];
    const float4 *s = src + (size_t)(n < 0 ? 0 : n) * D4;
    for(int d = threadIdx.x; d < D4; d += 256){
        float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if(n >= 0) v = s[d];
        if(OUT_BF16){
            uint2 o;
            o.x = (uint32_t)qx_f32_to_bf16(v.x) | ((uint32_t)qx_f32_to_bf16(v.y) << 16);
            o.y = (uint32_t)qx_f32_to_bf16(v.z) | ((uint32_t)qx_f32_to_bf16(v.w) << 16);
            ((uint2 *)Xp)[(size_t)j * D4 + d] = o;
        } else ((float4 *)Xp)[(size_t)j * D4 + d] = v;
    }
}
/* out[perm[j],:] = out[perm[j],:] + gate[perm[j]] * yp[j,:] (multiply, then add); a pass names every
 * token at most once, so rows do not collide */
__global__ void __launch_bounds__(256) k_scatter_gate(const float4 *yp, const int *perm, const float *gate, float4 *out, int D4){
    const int j = blockIdx.x, n = perm[j];
    if(n < 0) return;
    const float g = gate[n];
    float4 *o = out + (size_t)n * D4; const float4 *y = yp + (size_t)j * D4;
    for(int d = threadIdx.x; d < D4; d += 256){
        float4 a = o[d]; const float4 b = y[d];
        a.x = a.x + g * b.x; a.y = a.y + g * b.y; a.z = a.z + g * b.z; a.w = a.w + g * b.w;
        o[d] = a;
    }
}
__global__ void __launch_bounds__(256) k_scatter_add(const float4 *dXp, const int *perm, float4 *dst, int D4){
    const int j = blockIdx.x, n = perm[j];
    if(n < 0) return;
    float4 *o = dst + (size_t)n * D4; const float4 *s = dXp + (size_t)j * D4;
    for(int d = threadIdx.x; d < D4; d += 256){
        float4 a = o[d]; const float4 b = s[d];
        a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
        o[d] = a;
    }
}
/* d_gate[n] = dout[n,:] . yp[j,:];  dyp[j,:] = gate[n] * dout[n,:] */
template<bool OUT_BF16>
__global__ void __launch_bounds__(256) k_moe_dgate(const float4 *dout, const float4 *yp, const int *perm, const float *gate,
                                                   float *d_gate, void *dyp, int D4, int tokens){
    __shared__ float red[4];
    /* one pass (tokens = 0): perm names the token, which also indexes gate and d_gate; all passes as one grouped
     * list: perm names pass * tokens + token, which indexes gate and d_gate, and the token is the remainder */
    const int j = blockIdx.x, m = perm[j], n = (tokens && m >= 0) ? m % tokens : m;
    if(n < 0){
        for(int d = threadIdx.x; d < D4; d += 256){
            if(OUT_BF16) ((uint2 *)dyp)[(size_t)j * D4 + d] = make_uint2(0u, 0u);
            else ((float4 *)dyp)[(size_t)j * D4 + d] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        }
        return;
    }
    const float4 *dr = dout + (size_t)n * D4, *y = yp + (size_t)j * D4;
    const float g = gate[m];
    float acc = 0.0f;
    for(int d = threadIdx.x; d < D4; d += 256){
        const float4 a = dr[d], b = y[d];
        acc += a.x * b.x; acc += a.y * b.y; acc += a.z * b.z; acc += a.w * b.w;
        const float4 v = make_float4(g * a.x, g * a.y, g * a.z, g * a.w);
        if(OUT_BF16){
            uint2 o;
            o.x = (uint32_t)qx_f32_to_bf16(v.x) | ((uint32_t)qx_f32_to_bf16(v.y) << 16);
            o.y = (uint32_t)qx_f32_to_bf16(v.z) | ((uint32_t)qx_f32_to_bf16(v.w) << 16);
            ((uint2 *)dyp)[(size_t)j * D4 + d] = o;
        } else ((float4 *)dyp)[(size_t)j * D4 + d] = v;
    }
    acc = qx_wave_sum(acc);
    if((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = acc;
    __syncthreads();
    if(threadIdx.x == 0) d_gate[m] = (red[0] + red[1]) + (red[2] + red[3]);
}

/* ---- all K passes as ONE expert-grouped list of K*N rows (the reference's merged top-K, cudalm.cu:3532-3561,
 * 4022-4034): the grouping permutation of the K*N assignments names entries m = pass * N + token; row p of the
 * grouped buffers holds token perm[p] % N, and inv[m] is the row that holds entry m. ---- */
__global__ void __launch_bounds__(256) k_merge_rows(const int *perm, int KN, int N, int *tok, int *inv){
    const int p = blockIdx.x * 256 + threadIdx.x;
    if(p >= KN) return;
    const int m = perm[p];
    tok[p] = m < 0 ? -1 : m % N;
    if(m >= 0) inv[m] = p;
}
/* out[n,:] = (..(out[n,:] + g[0*N+n] * y[inv[0*N+n],:]) + ..) + g[(K-1)*N+n] * y[inv[(K-1)*N+n],:], pass after pass:
 * the sums the per-pass scatters build, in their order (g NULL: plain additions; inv < 0: the pass dropped the token) */
__global__ void __launch_bounds__(256) k_combine(const float4 *y, const int *inv, const float *g, float4 *out, int N, int K, int D4){
    const int n = blockIdx.x;
    float4 *o = out + (size_t)n * D4;
    for(int d = threadIdx.x; d < D4; d += 256){
        float4 a = o[d];
        for(int k = 0; k < K; k++){
            const size_t i = (size_t)k * N + n;
            const int p = inv[i];
            if(p < 0) continue;
            const float4 b = y[(size_t)p * D4 + d];
            if(g){ const float w = g[i]; a.x = a.x + w * b.x; a.y = a.y + w * b.y; a.z = a.z + w * b.z; a.w = a.w + w * b.w; }
            else { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
        }
        o[d] = a;
    }
}

/* ---- SwiGLU between the GEMMs: O = g * sigmoid(g) * u with the polynomial sigmoid ---- */
template<bool OUT_BF16>
__global__ void __launch_bounds__(256) k_swiglu(const float4 *G, const float4 *U, void *O, size_t n4){
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= n4) return;
    const float4 g = G[i], u = U[i];
    float4 o;
    o.x = g.x * qx_fsig(g.x) * u.x; o.y = g.y * qx_fsig(g.y) * u.y;
    o.z = g.z * qx_fsig(g.z) * u.z; o.w = g.w * qx_fsig(g.w) * u.w;
    if(OUT_BF16){
        uint2 p;
        p.x = (uint32_t)qx_f32_to_bf16(o.x) | ((uint32_t)qx_f32_to_bf16(o.y) << 16);
        p.y = (uint32_t)qx_f32_to_bf16(o.z) | ((uint32_t)qx_f32_to_bf16(o.w) << 16);
        ((uint2 *)O)[i] = p;
    } else ((float4 *)O)[i] = o;
}
template<bool OUT_BF16>
__global__ void __launch_bounds__(256) k_swiglu_bwd(const float4 *Gg, const float4 *U, const float4 *dact, void *dg, void *du, size_t n4){
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if(i >= n4) return;
    const float4 g = Gg[i], u = U[i], a = dact[i];
    float4 x, y;
    qx_swiglu_bwd1(g.x, u.x, a.x, x.x, y.x); qx_swiglu_bwd1(g.y, u.y, a.y, x.y, y.y);
    qx_swiglu_bwd1(g.z, u.z, a.z, x.z, y.z); qx_swiglu_bwd1(g.w, u.w, a.w, x.w, y.w);
    if(OUT_BF16){
        uint2 p, q;
        p.x = (uint32_t)qx_f32_to_bf16(x.x) | ((uint32_t)qx_f32_to_bf16(x.y) << 16);
        p.y = (uint32_t)qx_f32_to_bf16(x.z) | ((uint32_t)qx_f32_to_bf16(x.w) << 16);
        q.x = (uint32_t)qx_f32_to_bf16(y.x) | ((uint32_t)qx_f32_to_bf16(y.y) << 16);
        q.y = (uint32_t)qx_f32_to_bf16(y.z) | ((uint32_t)qx_f32_to_bf16(y.w) << 16);
        ((uint2 *)dg)[i] = p; ((uint2 *)du)[i] = q;
    } else { ((float4 *)dg)[i] = x; ((float4 *)du)[i] = y; }
}

/* ------------------------------------------------------------------------------------------
 * C ABI
 * ---------------------------------------------------------------------------------------- */
#define GLUE_ALIGN16(p) ((((uintptr_t)(p)) & 15) == 0)

extern "C" int qlmx_router_topk(const float *rt, float *rprobs, int *assign, float *gate, int N, int E, int K,
                                const float *bias, int bs, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(rt && rprobs && assign && gate, "qlmx_router_topk: NULL buffer");
    QLMX_REQUIRE(N >= 0 && E > 0 && K > 0 && K <= 8 && K <= E, "qlmx_router_topk: N=%d E=%d K=%d (K at most 8 and at most E)", N, E, K);
    if(N == 0) return QLMX_OK;
    const dim3 rgrid((N + RT_TOK - 1) / RT_TOK);
#define ROUTE_REG(EE) hipLaunchKernelGGL(k_router_topk_reg<EE>, rgrid, dim3(RT_TOK), 0, (hipStream_t)stream, rt, rprobs, assign, gate, N, K, bias, bs)
    if(E == 8) ROUTE_REG(8);
    else if(E == 16) ROUTE_REG(16);
    else if(E == 32) ROUTE_REG(32);
    else if(E == 64) ROUTE_REG(64);
#undef ROUTE_REG
    else if(E <= RT_MAXE)
        hipLaunchKernelGGL(k_router_topk_lds, dim3((N + RT_TOK - 1) / RT_TOK), dim3(RT_TOK), (size_t)RT_TOK * (E | 1) * sizeof(float),
                           (hipStream_t)stream, rt, rprobs, assign, gate, N, E, K, bias, bs);
    else
        hipLaunchKernelGGL(k_router_topk, dim3((N + 255) / 256), dim3(256), 0, (hipStream_t)stream, rt, rprobs, assign, gate, N, E, K, bias, bs);
    QLMX_LAUNCH_CHECK("router launch");
    return QLMX_OK;
}

extern "C" size_t qlmx_moe_perm_workspace(int N, int E, int K){
    const size_t NC = (size_t)(N + GP_CHUNK - 1) / GP_CHUNK;
    return ((size_t)K * NC * E + 4 + (size_t)K * E) * sizeof(int);
}

extern "C" int qlmx_moe_perm(const int *assign, int N, int E, int K, int *perm, int *off, void *workspace, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    hipStream_t st = (hipStream_t)stream;
    QLMX_REQUIRE(assign && perm && off && workspace, "qlmx_moe_perm: NULL buffer");
    QLMX_REQUIRE(N > 0 && E > 0 && E <= 4096 && K > 0, "qlmx_moe_perm: N=%d E=%d K=%d", N, E, K);
    const int NC = (N + GP_CHUNK - 1) / GP_CHUNK;
    int *ch = (int *)workspace, *bad = ch + (size_t)K * NC * E;
    hipLaunchKernelGGL(k_gp_clear, dim3(1), dim3(256), 0, st, bad, K * E);       /* a kernel, not a memset: callers may capture this into a graph */
    QLMX_LAUNCH_CHECK("perm flag clear");
    hipLaunchKernelGGL(k_gp_hist, dim3(NC, K), dim3(GP_CHUNK), E * sizeof(int), st, assign, N, E, NC, ch, bad);
    QLMX_LAUNCH_CHECK("perm histogram launch");
    hipLaunchKernelGGL(k_gp_scan, dim3((E + 1 + 3) / 4, K), dim3(256), 0, st, ch, (const int *)(bad + 4), E, NC, off);
    QLMX_LAUNCH_CHECK("perm scan launch");
    hipLaunchKernelGGL(k_gp_scatter, dim3(NC, K), dim3(GP_CHUNK), 4 * E * sizeof(int), st, assign, N, E, NC, (const int *)ch, perm);
    QLMX_LAUNCH_CHECK("perm scatter launch");
    return QLMX_OK;
}

/* 0 when every assignment of the last qlmx_moe_perm on this workspace was in range, else -1-e for
 * one offending expert index e (the reference aborts the run, cudalm.cu:3476-3478). Synchronises. */
extern "C" int qlmx_moe_perm_status(const void *workspace, int N, int E, int K, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(workspace, "qlmx_moe_perm_status: NULL workspace");
    const int NC = (N + GP_CHUNK - 1) / GP_CHUNK;
    int bad = 0;
    QLMX_HIP(hipMemcpyAsync(&bad, (const int *)workspace + (size_t)K * NC * E, sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream), "perm flag read");
    QLMX_HIP(hipStreamSynchronize((hipStream_t)stream), "perm flag sync");
    if(bad){ qlmx_set_error("qlmx_moe_perm: expert index %d out of range [0, %d)", -1 - bad, E); return QLMX_E_ARG; }
    return QLMX_OK;
}

#define GLUE_ROWS_CHECK(name, D)                                                                   \
    QLMX_REQUIRE((D) > 0 && (D) % 4 == 0, name ": D=%d must be a positive multiple of 4", (D))

extern "C" int qlmx_moe_gather(const float *src, const int *perm, void *Xp, int N, int D, int out_dtype, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(src && perm && Xp, "qlmx_moe_gather: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_gather", D);
    QLMX_REQUIRE(GLUE_ALIGN16(src) && GLUE_ALIGN16(Xp), "qlmx_moe_gather: buffers must be 16-byte aligned");
    QLMX_REQUIRE(out_dtype == QLMX_ACT_F32 || out_dtype == QLMX_ACT_BF16, "qlmx_moe_gather: unknown output type %d", out_dtype);
    if(N <= 0) return QLMX_OK;
    if(out_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL(k_gather_rows<true>, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)src, perm, Xp, D / 4);
    else                           hipLaunchKernelGGL(k_gather_rows<false>, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)src, perm, Xp, D / 4);
    QLMX_LAUNCH_CHECK("gather launch");
    return QLMX_OK;
}

extern "C" int qlmx_moe_scatter_gate(const float *yp, const int *perm, const float *gate, float *out, int N, int D, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(yp && perm && gate && out, "qlmx_moe_scatter_gate: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_scatter_gate", D);
    QLMX_REQUIRE(GLUE_ALIGN16(yp) && GLUE_ALIGN16(out), "qlmx_moe_scatter_gate: buffers must be 16-byte aligned");
    if(N <= 0) return QLMX_OK;
    hipLaunchKernelGGL(k_scatter_gate, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)yp, perm, gate, (float4 *)out, D / 4);
    QLMX_LAUNCH_CHECK("scatter launch");
    return QLMX_OK;
}

extern "C" int qlmx_moe_scatter_add(const float *dXp, const int *perm, float *dst, int N, int D, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(dXp && perm && dst, "qlmx_moe_scatter_add: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_scatter_add", D);
    QLMX_REQUIRE(GLUE_ALIGN16(dXp) && GLUE_ALIGN16(dst), "qlmx_moe_scatter_add: buffers must be 16-byte aligned");
    if(N <= 0) return QLMX_OK;
    hipLaunchKernelGGL(k_scatter_add, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)dXp, perm, (float4 *)dst, D / 4);
    QLMX_LAUNCH_CHECK("scatter-add launch");
    return QLMX_OK;
}

extern "C" int qlmx_moe_dgate(const float *dout, const float *yp, const int *perm, const float *gate,
                              float *d_gate, void *dyp, int N, int D, int out_dtype, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(dout && yp && perm && gate && d_gate && dyp, "qlmx_moe_dgate: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_dgate", D);
    QLMX_REQUIRE(GLUE_ALIGN16(dout) && GLUE_ALIGN16(yp) && GLUE_ALIGN16(dyp), "qlmx_moe_dgate: buffers must be 16-byte aligned");
    QLMX_REQUIRE(out_dtype == QLMX_ACT_F32 || out_dtype == QLMX_ACT_BF16, "qlmx_moe_dgate: unknown output type %d", out_dtype);
    if(N <= 0) return QLMX_OK;
    if(out_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL(k_moe_dgate<true>, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)dout, (const float4 *)yp, perm, gate, d_gate, dyp, D / 4, 0);
    else                           hipLaunchKernelGGL(k_moe_dgate<false>, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)dout, (const float4 *)yp, perm, gate, d_gate, dyp, D / 4, 0);
    QLMX_LAUNCH_CHECK("dgate launch");
    return QLMX_OK;
}

/* ---- merged passes ---- */
extern "C" int qlmx_moe_merge_rows(const int *perm, int N, int K, int *tok, int *inv, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(perm && tok && inv, "qlmx_moe_merge_rows: NULL buffer");
    QLMX_REQUIRE(N > 0 && K > 0 && (long long)N * K < (1LL << 31), "qlmx_moe_merge_rows: N=%d K=%d", N, K);
    const int KN = N * K;
    /* rows a caller dropped (perm < 0) leave no inverse: -1 everywhere first, by a kernel so that a capture holds no memset node */
    hipLaunchKernelGGL(k_fill_i32, dim3((KN + 255) / 256), dim3(256), 0, (hipStream_t)stream, inv, -1, KN);
    QLMX_LAUNCH_CHECK("merge rows: inverse fill");
    hipLaunchKernelGGL(k_merge_rows, dim3((KN + 255) / 256), dim3(256), 0, (hipStream_t)stream, perm, KN, N, tok, inv);
    QLMX_LAUNCH_CHECK("merge rows launch");
    return QLMX_OK;
}

extern "C" int qlmx_moe_combine(const float *y, const int *inv, const float *gate, float *out, int N, int K, int D, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(y && inv && out, "qlmx_moe_combine: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_combine", D);
    QLMX_REQUIRE(K > 0 && GLUE_ALIGN16(y) && GLUE_ALIGN16(out), "qlmx_moe_combine: K=%d, buffers must be 16-byte aligned", K);
    if(N <= 0) return QLMX_OK;
    hipLaunchKernelGGL(k_combine, dim3(N), dim3(256), 0, (hipStream_t)stream, (const float4 *)y, inv, gate, (float4 *)out, N, K, D / 4);
    QLMX_LAUNCH_CHECK("combine launch");
    return QLMX_OK;
}

extern "C" int qlmx_moe_dgate_merged(const float *dout, const float *yp, const int *perm, const float *gate,
                                     float *d_gate, void *dyp, int N, int K, int D, int out_dtype, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(dout && yp && perm && gate && d_gate && dyp, "qlmx_moe_dgate_merged: NULL buffer");
    GLUE_ROWS_CHECK("qlmx_moe_dgate_merged", D);
    QLMX_REQUIRE(GLUE_ALIGN16(dout) && GLUE_ALIGN16(yp) && GLUE_ALIGN16(dyp), "qlmx_moe_dgate_merged: buffers must be 16-byte aligned");
    QLMX_REQUIRE(out_dtype == QLMX_ACT_F32 || out_dtype == QLMX_ACT_BF16, "qlmx_moe_dgate_merged: unknown output type %d", out_dtype);
    QLMX_REQUIRE(K > 0 && (long long)N * K < (1LL << 31), "qlmx_moe_dgate_merged: N=%d K=%d", N, K);
    if(N <= 0) return QLMX_OK;
    const int KN = N * K;
    if(out_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL(k_moe_dgate<true>, dim3(KN), dim3(256), 0, (hipStream_t)stream, (const float4 *)dout, (const float4 *)yp, perm, gate, d_gate, dyp, D / 4, N);
    else                           hipLaunchKernelGGL(k_moe_dgate<false>, dim3(KN), dim3(256), 0, (hipStream_t)stream, (const float4 *)dout, (const float4 *)yp, perm, gate, d_gate, dyp, D / 4, N);
    QLMX_LAUNCH_CHECK("merged dgate launch");
    return QLMX_OK;
}

extern "C" int qlmx_swiglu(const float *G, const float *U, void *O, size_t n, int out_dtype, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(G && U && O, "qlmx_swiglu: NULL buffer");
    QLMX_REQUIRE(n % 4 == 0 && GLUE_ALIGN16(G) && GLUE_ALIGN16(U) && GLUE_ALIGN16(O), "qlmx_swiglu: n must be a multiple of 4 and the buffers 16-byte aligned");
    QLMX_REQUIRE(out_dtype == QLMX_ACT_F32 || out_dtype == QLMX_ACT_BF16, "qlmx_swiglu: unknown output type %d", out_dtype);
    if(n == 0) return QLMX_OK;
    const size_t n4 = n / 4; const unsigned grid = (unsigned)((n4 + 255) / 256);
    if(out_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL(k_swiglu<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const float4 *)G, (const float4 *)U, O, n4);
    else                           hipLaunchKernelGGL(k_swiglu<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const float4 *)G, (const float4 *)U, O, n4);
    QLMX_LAUNCH_CHECK("swiglu launch");
    return QLMX_OK;
}

extern "C" int qlmx_swiglu_bwd(const float *Gg, const float *U, const float *dact, void *dg, void *du, size_t n, int out_dtype, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(Gg && U && dact && dg && du, "qlmx_swiglu_bwd: NULL buffer");
    QLMX_REQUIRE(n % 4 == 0 && GLUE_ALIGN16(Gg) && GLUE_ALIGN16(U) && GLUE_ALIGN16(dact) && GLUE_ALIGN16(dg) && GLUE_ALIGN16(du),
                 "qlmx_swiglu_bwd: n must be a multiple of 4 and the buffers 16-byte aligned");
    QLMX_REQUIRE(out_dtype == QLMX_ACT_F32 || out_dtype == QLMX_ACT_BF16, "qlmx_swiglu_bwd: unknown output type %d", out_dtype);
    if(n == 0) return QLMX_OK;
    const size_t n4 = n / 4; const unsigned grid = (unsigned)((n4 + 255) / 256);
    if(out_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL(k_swiglu_bwd<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const float4 *)Gg, (const float4 *)U, (const float4 *)dact, dg, du, n4);
    else                           hipLaunchKernelGGL(k_swiglu_bwd<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const float4 *)Gg, (const float4 *)U, (const float4 *)dact, dg, du, n4);
    QLMX_LAUNCH_CHECK("swiglu backward launch");
    return QLMX_OK;
}
