/* qlm_oracle.c -- TEST INFRASTRUCTURE ONLY. See qlm_oracle.h.
 *
 * Parity status (what pins each function; "ref lib" = oracle/_ref/libcudalm_ref.so built from the
 * reference's own sources, fixtures = tests/golden/ written by tests/golden/make_golden.py from it):
 *   qhashu/qsri/qclmp/qd_get/qd_set/qd_bytes  fixtures + brute force over all byte values
 *   encode/render                             fixtures (bit-exact) + half-step / 15-level invariants
 *   step (adam, lion, both lrmodes, gsp,      fixtures incl. forced carry cases (bit-exact), ref lib
 *         tail groups, unpacked, v4)          on 1e6-element seeded inputs when present
 *   step_touched                              fixture written by the reference's k_ng_q4_step (bit-exact) +
 *                                             equality with step() on a full gradient whose untouched
 *                                             groups are left out
 *   servo                                     fixtures with forced grow / shrink / idle groups
 *   gemm nn/tn/nt                             double-precision triple loop + ref lib
 *   fexp / router_topk / perm                 fixtures (bit-exact) + brute force stable-sort check
 *   gather/scatter/dgate                      closed form + ref lib
 *   swiglu fwd/bwd                            libm closed form to 1e-6 (the reference's AVX2 body uses
 *                                             explicit FMA, so tolerance rather than bits) + ref lib
 *   q4n quantize/dequantize                   fixtures (byte-exact: grid groups, off-grid raw groups, an
 *                                             all-zero group, a short tail) + round trip + ref lib
 *   sqsum / gnorm                             fixture written by the reference's k_sqsum / k_gnorm (bit-exact: chunk
 *                                             sums in double, a clipping and a non-clipping norm, a non-finite
 *                                             side sum) + closed forms (all ones, a 3-4-5 vector) + ref lib
 *   moe_forward/backward                      double-precision scalar expert FFN in the tests
 *                                             (cudalm.cu:10366-10387 style) + composition of ref lib calls
 * No function here is "parity unpinned".
 */
#include "qlm_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

void orc_set_threads(int n){
#ifdef _OPENMP
    if(n>0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
int orc_get_threads(void){
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * Integer helpers
 * ---------------------------------------------------------------------------------------- */

/* qlm.cuh:78-82: splitmix64 finaliser, low 32 bits. */
uint32_t orc_qhashu(uint64_t x){
    x += 0x9E3779B97F4A7C15ULL;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    return (uint32_t)(x ^ (x >> 31));
}

/* qlm.cuh:83-87: floor plus one with probability frac(v); the uniform is the top 24 bits of the
 * hash of (element index, step), so the draw is a pure function of both. */
int orc_qsri(float v, uint64_t i, uint64_t t){
    float fl = floorf(v);
    uint32_t h = orc_qhashu(i * 0x2545F4914F6CDD1DULL + t * 0x9E3779B97F4A7C15ULL);
    float u = (float)(h >> 8) * (1.0f / 16777216.0f);
    return (int)fl + (u < (v - fl) ? 1 : 0);
}

/* qlm.cuh:88 */
int orc_qclmp(int v, int lo, int hi){ return v < lo ? lo : (v > hi ? hi : v); }

/* qlm.cuh:96-101: element i lives in byte i/2; even i is the low nibble, odd i the high one;
 * two's complement on 4 bits. */
int orc_qd_get(const int8_t *d, uint64_t i, int packed){
    if(!packed) return (int)d[i];
    unsigned b = (uint8_t)d[i >> 1];
    int nib = (int)((i & 1) ? (b >> 4) : (b & 15u));
    return nib >= 8 ? nib - 16 : nib;
}

/* qlm.cuh:102-108 */
void orc_qd_set(int8_t *d, uint64_t i, int v, int packed){
    if(!packed){ d[i] = (int8_t)v; return; }
    uint8_t *b = (uint8_t *)&d[i >> 1];
    unsigned nib = (unsigned)v & 15u;
    *b = (uint8_t)((i & 1) ? ((*b & 0x0Fu) | (nib << 4)) : ((*b & 0xF0u) | nib));
}

/* qlm.cuh:109-111 */
uint64_t orc_qd_bytes(uint64_t nq, int packed){ return packed ? (nq + 1) / 2 : nq; }

/* ------------------------------------------------------------------------------------------
 * Span table
 * ---------------------------------------------------------------------------------------- */

/* qlm.cuh:448-455: append a span; groups are consecutive chunks of `group` elements, the last one
 * may be short. gof starts equal to pof, sref starts at 1. */
int orc_span_add(orc_span *tab, int nspan, uint64_t pof, uint64_t n, int group,
                 uint64_t *nq, uint64_t *ngrp){
    orc_span *sp = &tab[nspan];
    sp->pof = pof; sp->gof = pof; sp->qi0 = *nq; sp->n = n;
    sp->gi0 = (int)*ngrp;
    sp->ngrp = (int)((n + (uint64_t)group - 1) / (uint64_t)group);
    sp->sref = 1.0f;
    *nq += n; *ngrp += (uint64_t)sp->ngrp;
    return nspan + 1;
}

/* qlm.cuh:527-536: freeze each span's reference scale = mean of its group scales, summed in
 * double in group order. */
void orc_span_sref(orc_span *tab, int nspan, const float *s){
    for(int i = 0; i < nspan; i++){
        double acc = 0;
        for(int g = 0; g < tab[i].ngrp; g++) acc += s[tab[i].gi0 + g];
        tab[i].sref = (float)(acc / (double)tab[i].ngrp);
    }
}

/* Where group gi lives: owning span (first match of a linear scan, span 0 when nothing matches:
 * qlm.cuh:114-117), element offset inside the span and the element count (cpu_kern.h:773-776). */
typedef struct { int si, n; uint64_t j0; } grp_loc;
static grp_loc locate(const orc_span *sp, int nspan, int gi, int group){
    grp_loc L; L.si = 0;
    for(int i = 0; i < nspan; i++)
        if(gi >= sp[i].gi0 && gi < sp[i].gi0 + sp[i].ngrp){ L.si = i; break; }
    L.j0 = (uint64_t)(gi - sp[L.si].gi0) * (uint64_t)group;
    uint64_t left = sp[L.si].n - L.j0;
    L.n = (int)((uint64_t)group < left ? (uint64_t)group : left);
    return L;
}

/* qlm.cuh:119-132: write one group's digits; packed pairs (low = even element), a missing odd
 * partner of a short group is stored as 0. */
static void put_digits(int8_t *d, uint64_t qi0, const int8_t *dig, int n, int packed){
    if(!packed){ for(int j = 0; j < n; j++) d[qi0 + j] = dig[j]; return; }
    int nb = (n + 1) >> 1;
    for(int b = 0; b < nb; b++){
        int lo = dig[2*b] & 15;
        int hi = (2*b + 1 < n) ? (dig[2*b + 1] & 15) : 0;
        d[(qi0 >> 1) + b] = (int8_t)((hi << 4) | lo);
    }
}

/* ------------------------------------------------------------------------------------------
 * encode / render
 * ---------------------------------------------------------------------------------------- */

/* qlm.cuh:136-167 == cpu_kern.h:777-789. scale = absmax/dmax (1e-8 when not positive);
 * digit = clamp(rint(P/scale)); residual = clamp(rint((P/scale - digit)*128), +-64). */
void orc_encode(const float *P, int8_t *d, int8_t *r, float *s, const orc_span *sp, int nspan,
                int group, int dmax, int packed, int ngrp){
    #pragma omp parallel for schedule(static)
    for(int gi = 0; gi < ngrp; gi++){
        grp_loc L = locate(sp, nspan, gi, group);
        const float *p = P + sp[L.si].pof + L.j0;
        uint64_t qi0 = sp[L.si].qi0 + L.j0;
        float amax = 0.0f;
        for(int j = 0; j < L.n; j++) amax = fmaxf(amax, fabsf(p[j]));
        float sg = amax / (float)dmax;
        if(!(sg > 0.0f)) sg = 1e-8f;
        s[gi] = sg;
        int8_t dig[256];
        for(int j = 0; j < L.n; j++){
            float t = p[j] / sg;
            int dd = orc_qclmp((int)rintf(t), -dmax, dmax);
            int rr = orc_qclmp((int)rintf((t - (float)dd) * 128.0f), -64, 64);
            dig[j] = (int8_t)dd;
            r[qi0 + j] = (int8_t)rr;
        }
        put_digits(d, qi0, dig, L.n, packed);
    }
}

/* qlm.cuh:170-178 == cpu_kern.h:790-796: P = scale * digit, one fp32 multiply. */
void orc_render(float *P, const int8_t *d, const float *s, const orc_span *sp, int nspan,
                int group, int packed, int gi_base, int ng){
    #pragma omp parallel for schedule(static)
    for(int w = 0; w < ng; w++){
        int gi = gi_base + w;
        grp_loc L = locate(sp, nspan, gi, group);
        float *p = P + sp[L.si].pof + L.j0;
        uint64_t qi0 = sp[L.si].qi0 + L.j0;
        float sg = s[gi];
        for(int j = 0; j < L.n; j++) p[j] = sg * (float)orc_qd_get(d, qi0 + j, packed);
    }
}

/* ------------------------------------------------------------------------------------------
 * Integer AdamW
 * ---------------------------------------------------------------------------------------- */

/* One group: qlm.cuh:199-278 == cpu_kern.h:798-826, same operation order. `v4` is the QLM_V4
 * switch (qlm.cuh:62-67): the stored second moment is v^(1/4) instead of sqrt(v). */
static void step_group(int gi, float *P, const float *G, int8_t *d, int8_t *r, const float *s,
                       int8_t *m8, float *m8s, uint8_t *v8, float *v8s,
                       const orc_span *sp, int nspan, int group, int dmax,
                       float lr, float b1, float b2, float wd, float gs,
                       float inv_bc1, float inv_sqrt_bc2, int lrmode, uint64_t t, int adam,
                       int packed, int v4, long long *st, const float *Gcompact){
    grp_loc L = locate(sp, nspan, gi, group);
    const orc_span *S = &sp[L.si];
    uint64_t pof = S->pof + L.j0, qi0 = S->qi0 + L.j0, gof = S->gof + L.j0;
    float sg = s[gi];
    float lsb_rate = lr * 128.0f / (lrmode ? sg : S->sref);   /* LSBs per unit Adam step     */
    float decay = lr * wd * 128.0f;                           /* LSBs of decay per digit     */
    float ms_old = m8s[gi], vs_old = v8s ? v8s[gi] : 0.0f;
    float mnew[256], rnew[256], amax = 0.0f, vmax = 0.0f;
    int8_t dig[256];

    for(int j = 0; j < L.n; j++){
        uint64_t qi = qi0 + j;
        float gr = (Gcompact ? Gcompact[j] : G[gof + j]) * gs;
        float mv = (float)m8[qi] * ms_old;
        float u;
        rnew[j] = 0.0f;
        if(adam){
            float sv = (float)v8[qi] * vs_old; if(v4) sv = sv * sv;
            float vv = sv * sv;
            mnew[j] = b1 * mv + (1.0f - b1) * gr;
            vv = b2 * vv + (1.0f - b2) * gr * gr;
            float rv = sqrtf(vv);
            float q1 = 1.0f * vs_old; if(v4) q1 = q1 * q1;
            float veps = fmaxf(q1, 1e-8f);
            u = (mnew[j] * inv_bc1) / (rv * inv_sqrt_bc2 + veps);
            u = fmaxf(-8.0f, fminf(8.0f, u));
            rnew[j] = v4 ? sqrtf(rv) : rv;
        } else {                                      /* Lion: qlm.cuh:225-229 */
            float cc = b1 * mv + (1.0f - b1) * gr;
            u = (float)((cc > 0.0f) - (cc < 0.0f));
            mnew[j] = b2 * mv + (1.0f - b2) * gr;
        }
        int dd = orc_qd_get(d, qi, packed);
        int idl = orc_qsri(-(lsb_rate * u + decay * (float)dd), qi, t);
        int rr = (int)r[qi] + idl;
        /* the unique carry c with rr-128c in [-64,64]; rr == 64 stays put */
        int c = 0;
        if(rr > 64)       c =  (((rr - 65) >> 7) + 1);
        else if(rr < -64) c = -((((-rr) - 65) >> 7) + 1);
        rr -= c * 128;
        dd = orc_qclmp(dd + c, -dmax, dmax);
        dig[j] = (int8_t)dd;
        r[qi] = (int8_t)rr;
        if(P) P[pof + j] = sg * (float)dd;
        if(st){
            int ai = idl < 0 ? -idl : idl;
            if(ai > st[3]) st[3] = ai;
            st[0] += c < 0 ? -c : c;
            st[1] += (dd == dmax) | (dd == -dmax);
            st[2] += (dd == 0);
        }
        amax = fmaxf(amax, fabsf(mnew[j]));
        vmax = fmaxf(vmax, rnew[j]);
    }
    put_digits(d, qi0, dig, L.n, packed);

    float ms = amax > 0.0f ? amax / 127.0f : 1e-12f;
    float vs = vmax > 0.0f ? vmax / 255.0f : 1e-12f;
    m8s[gi] = ms;
    if(adam) v8s[gi] = vs;
    for(int j = 0; j < L.n; j++){
        uint64_t qi = qi0 + j;
        m8[qi] = (int8_t)orc_qclmp(orc_qsri(mnew[j] / ms, qi, t + 0x5EEDULL), -127, 127);
        if(adam){
            int vq = orc_qclmp(orc_qsri(rnew[j] / vs, qi, t + 0xBEEFULL), 0, 255);
            if(vq == 0 && rnew[j] > 0.0f) vq = 1;     /* zero is absorbing: keep v alive */
            v8[qi] = (uint8_t)vq;
        }
    }
}

/* qlm.cuh:377-397 / cpu_kern.h:827-852: groups gi_base .. gi_base+ng-1; the clip multiplier
 * comes from *gsp when gsp is not NULL. stat = {sum |carry|, railed, zero, max |idl|}. */
void orc_step(float *P, const float *G, int8_t *d, int8_t *r, const float *s, int8_t *m8, float *m8s,
              uint8_t *v8, float *v8s, const orc_span *sp, int nspan, int group, int dmax,
              float lr, float b1, float b2, float wd, float gscale, const float *gsp,
              float inv_bc1, float inv_sqrt_bc2, int lrmode, uint64_t t, int adam,
              long long *stat, int packed, int gi_base, int ng, int v4){
    float gs = gsp ? *gsp : gscale;
    long long s0 = 0, s1 = 0, s2 = 0, s3 = 0;
    #pragma omp parallel for schedule(static) reduction(+:s0,s1,s2) reduction(max:s3)
    for(int w = 0; w < ng; w++){
        long long st[4] = {0, 0, 0, 0};
        step_group(gi_base + w, P, G, d, r, s, m8, m8s, v8, v8s, sp, nspan, group, dmax,
                   lr, b1, b2, wd, gs, inv_bc1, inv_sqrt_bc2, lrmode, t, adam, packed, v4,
                   stat ? st : NULL, NULL);
        s0 += st[0]; s1 += st[1]; s2 += st[2]; if(st[3] > s3) s3 = st[3];
    }
    if(stat){ stat[0] += s0; stat[1] += s1; stat[2] += s2; if(s3 > stat[3]) stat[3] = s3; }
}

/* cpu_kern.h:620-648 (k_ng_q4_step, GPU form cudalm.cu:4472-4520): the same group update driven by a
 * list of touched groups of one packed span that starts at element 0; group w reads its gradient
 * from the compact row Gc[w*group ..]. adam, relative LR through sref, gscale = *gs or 1. */
void orc_step_touched(float *P, const float *Gc, int8_t *d, int8_t *r, const float *s, int8_t *m8, float *m8s,
                      uint8_t *v8, float *v8s, const int *touched_gi, int ntouched, int group, int dmax,
                      float lr, float b1, float b2, float wd, float sref, float inv_bc1, float inv_sqrt_bc2,
                      uint64_t t, uint64_t nt, const float *gs, int v4){
    orc_span one; memset(&one, 0, sizeof one);
    one.n = nt; one.ngrp = (int)((nt + (uint64_t)group - 1) / (uint64_t)group); one.sref = sref;
    #pragma omp parallel for schedule(static)
    for(int w = 0; w < ntouched; w++)
        step_group(touched_gi[w], P, NULL, d, r, s, m8, m8s, v8, v8s, &one, 1, group, dmax, lr, b1, b2, wd,
                   gs ? gs[0] : 1.0f, inv_bc1, inv_sqrt_bc2, 0, t, 1, 1, v4, NULL, Gc + (size_t)w * group);
}

/* ------------------------------------------------------------------------------------------
 * Scale servo: qlm.cuh:404-441 == cpu_kern.h:857-873
 * ---------------------------------------------------------------------------------------- */
void orc_servo(int8_t *d, int8_t *r, float *s, const orc_span *sp, int nspan, int group, int dmax,
               float f_hi, float f_lo, int packed, int ngrp){
    #pragma omp parallel for schedule(static)
    for(int gi = 0; gi < ngrp; gi++){
        grp_loc L = locate(sp, nspan, gi, group);
        uint64_t qi0 = sp[L.si].qi0 + L.j0;
        int railed = 0;
        for(int j = 0; j < L.n; j++){
            int dd = orc_qd_get(d, qi0 + j, packed);
            railed += (dd == dmax) | (dd == -dmax);
        }
        float f = (float)railed / (float)L.n, sg = s[gi], sn;
        if(f > f_hi)      sn = sg * 1.09051f;       /* 2^(1/8) */
        else if(f < f_lo) sn = sg / 1.09051f;
        else continue;
        float conv = sg / sn;
        s[gi] = sn;
        int8_t dig[256];
        for(int j = 0; j < L.n; j++){
            uint64_t qi = qi0 + j;
            float t = ((float)orc_qd_get(d, qi, packed) + (float)r[qi] * (1.0f / 128.0f)) * conv;
            int dd = orc_qclmp((int)rintf(t), -dmax, dmax);
            int rr = orc_qclmp((int)rintf((t - (float)dd) * 128.0f), -64, 64);
            dig[j] = (int8_t)dd;
            r[qi] = (int8_t)rr;
        }
        put_digits(d, qi0, dig, L.n, packed);
    }
}

/* ------------------------------------------------------------------------------------------
 * fp32 GEMM, strided core
 *
 * O[R,C] = X[R,K] @ Y[K,C] + beta*O with X, Y read through (row, col) strides (cpu_rt.h:178-183).
 * The reference packs 6x16 panels and sums each K chunk of 256 with one FMA chain per output
 * starting from zero, then adds the chunk to O (cpu_rt.h:196-231, 264-303); this keeps that
 * summation order (chunked FMA chains, chunk totals added in order) without the packing.
 * Rows <= 4 take the reference's unpacked path (cpu_rt.h:233-258), whose multiply-then-add
 * (no FMA under -ffp-contract=off) axpy order is kept for the non-dot case; the dot case uses a
 * SIMD reduction there whose order the compiler chooses, so agreement is to rounding, not bits.
 * ---------------------------------------------------------------------------------------- */
#define ORC_KC 256
static void gemm_core(int R, int C, int K, const float *X, ptrdiff_t xr, ptrdiff_t xc,
                      const float *Y, ptrdiff_t yr, ptrdiff_t yc, float beta, float *O, ptrdiff_t ldo){
    if(R <= 0 || C <= 0) return;
    if(K <= 0){
        for(int r = 0; r < R; r++) for(int c = 0; c < C; c++)
            O[r*ldo + c] = beta == 0 ? 0.0f : beta * O[r*ldo + c];
        return;
    }
    if(R <= 4){
        #pragma omp parallel for schedule(static)
        for(int c0 = 0; c0 < C; c0 += 64){
            int c1 = c0 + 64 < C ? c0 + 64 : C;
            for(int r = 0; r < R; r++){
                float acc[64];
                for(int c = c0; c < c1; c++) acc[c - c0] = 0.0f;
                for(int p = 0; p < K; p++){
                    float x = X[r*xr + p*xc];
                    const float *y = Y + (ptrdiff_t)p*yr;
                    for(int c = c0; c < c1; c++) acc[c - c0] = acc[c - c0] + x * y[(ptrdiff_t)c*yc];
                }
                for(int c = c0; c < c1; c++){
                    float *o = &O[r*ldo + c];
                    *o = beta == 0 ? acc[c - c0] : beta * (*o) + acc[c - c0];
                }
            }
        }
        return;
    }
    /* parallel over (row block, column block); each thread owns its outputs for all K chunks */
    const int RB = 48, CB = 64;
    int nrb = (R + RB - 1) / RB, ncb = (C + CB - 1) / CB;
    #pragma omp parallel for schedule(dynamic,1) collapse(2)
    for(int ib = 0; ib < nrb; ib++) for(int jb = 0; jb < ncb; jb++){
        int r0 = ib*RB, r1 = r0 + RB < R ? r0 + RB : R;
        int c0 = jb*CB, c1 = c0 + CB < C ? c0 + CB : C, cw = c1 - c0;
        float ytile[ORC_KC * 64];
        for(int pc = 0; pc < K; pc += ORC_KC){
            int kc = K - pc < ORC_KC ? K - pc : ORC_KC;
            for(int p = 0; p < kc; p++) for(int c = 0; c < cw; c++)
                ytile[p*64 + c] = Y[(ptrdiff_t)(pc + p)*yr + (ptrdiff_t)(c0 + c)*yc];
            for(int r = r0; r < r1; r++){
                float acc[64];
                for(int c = 0; c < cw; c++) acc[c] = 0.0f;
                const float *x = X + (ptrdiff_t)r*xr + (ptrdiff_t)pc*xc;
                for(int p = 0; p < kc; p++){
                    float xv = x[(ptrdiff_t)p*xc];
                    const float *yt = ytile + p*64;
                    #pragma omp simd
                    for(int c = 0; c < cw; c++) acc[c] = fmaf(xv, yt[c], acc[c]);
                }
                float *o = O + (ptrdiff_t)r*ldo + c0;
                if(pc > 0)          for(int c = 0; c < cw; c++) o[c] = o[c] + acc[c];
                else if(beta == 0)  for(int c = 0; c < cw; c++) o[c] = acc[c];
                else                for(int c = 0; c < cw; c++) o[c] = fmaf(1.0f, acc[c], beta * o[c]);
            }
        }
    }
}

/* cudalm.cu:3133-3145 / 3247-3249: C[M,N] = A[M,K] @ B[K,N] */
void orc_gemm_nn(const float *A, const float *B, float *C, int M, int K, int N){
    gemm_core(M, N, K, A, K, 1, B, N, 1, 0.0f, C, N);
}
/* cudalm.cu:3174-3186 / 3250-3253: C[M,N] = A[M,K] @ B[N,K]^T + beta*C */
void orc_gemm_tn(const float *A, const float *B, float *C, int M, int K, int N, float beta){
    gemm_core(M, N, K, A, K, 1, B, 1, K, beta, C, N);
}
/* cudalm.cu:3190-3202 / 3254-3256: C[K,N] += A[M,K]^T @ B[M,N] */
void orc_gemm_nt(const float *A, const float *B, float *C, int M, int K, int N){
    gemm_core(K, N, M, A, 1, K, B, N, 1, 1.0f, C, N);
}

void orc_gemm_nn_f64(const float *A, const float *B, double *C, int M, int K, int N){
    #pragma omp parallel for schedule(static)
    for(int m = 0; m < M; m++) for(int n = 0; n < N; n++){
        double acc = 0; for(int k = 0; k < K; k++) acc += (double)A[(size_t)m*K + k] * (double)B[(size_t)k*N + n];
        C[(size_t)m*N + n] = acc; }
}
void orc_gemm_tn_f64(const float *A, const float *B, double *C, int M, int K, int N){
    #pragma omp parallel for schedule(static)
    for(int m = 0; m < M; m++) for(int n = 0; n < N; n++){
        double acc = 0; for(int k = 0; k < K; k++) acc += (double)A[(size_t)m*K + k] * (double)B[(size_t)n*K + k];
        C[(size_t)m*N + n] = acc; }
}
void orc_gemm_nt_f64(const float *A, const float *B, double *C, int M, int K, int N){
    #pragma omp parallel for schedule(static)
    for(int k = 0; k < K; k++) for(int n = 0; n < N; n++){
        double acc = 0; for(int m = 0; m < M; m++) acc += (double)A[(size_t)m*K + k] * (double)B[(size_t)m*N + n];
        C[(size_t)k*N + n] = acc; }
}
/* cudalm.cu:9842-9844: relative L2 */
double orc_relerr(const float *a, const float *b, size_t n){
    double num = 0, den = 0;
    for(size_t i = 0; i < n; i++){ double e = (double)a[i] - (double)b[i]; num += e*e; den += (double)b[i]*(double)b[i]; }
    return sqrt(num / (den > 0 ? den : 1));
}
double orc_relerr_f64(const float *a, const double *b, size_t n){
    double num = 0, den = 0;
    for(size_t i = 0; i < n; i++){ double e = (double)a[i] - b[i]; num += e*e; den += b[i]*b[i]; }
    return sqrt(num / (den > 0 ? den : 1));
}

/* ------------------------------------------------------------------------------------------
 * MoE glue
 * ---------------------------------------------------------------------------------------- */

/* cpu_kern.h:29-34: clamp, Cody-Waite split of ln2, degree-6 Horner polynomial, exponent built
 * with integer bit arithmetic. No contraction, so each product and sum rounds separately. */
float orc_fexp(float x){
    x = x < -87.0f ? -87.0f : (x > 88.0f ? 88.0f : x);
    float fi = rintf(x * 1.44269504089f);
    float r = x - fi * 0.693145751953125f;
    r -= fi * 1.428606765330187e-06f;
    float p = 1.0f + r*(1.0f + r*(0.5f + r*(1.0f/6 + r*(1.0f/24 + r*(1.0f/120 + r*(1.0f/720))))));
    uint32_t bits = (uint32_t)((int)fi + 127) << 23;
    float scale; memcpy(&scale, &bits, 4);
    return p * scale;
}
static float orc_fsig(float x){ return 1.0f / (1.0f + orc_fexp(-x)); }

/* cpu_kern.h:413-425 (cudalm.cu:2515-2534): softmax over E, then K greedy picks on prob+bias with a
 * strict > so the lowest index wins a tie; pass-major outputs, gate = raw softmax prob. */
void orc_router_topk(const float *rt, float *rprobs, int *assign, float *gate, int N, int E, int K,
                     const float *bias, int bs){
    #pragma omp parallel for schedule(static) if((long)N*E >= 32768)
    for(int n = 0; n < N; n++){
        const float *logit = rt + (size_t)n*E;
        float *pr = rprobs + (size_t)n*E;
        float mx = -1e30f;
        for(int e = 0; e < E; e++) if(logit[e] > mx) mx = logit[e];
        float sum = 0;
        for(int e = 0; e < E; e++){ pr[e] = orc_fexp(logit[e] - mx); sum += pr[e]; }
        float inv = 1.0f / sum;
        for(int e = 0; e < E; e++) pr[e] *= inv;
        int chosen[8];
        for(int k = 0; k < K; k++){
            int best = -1; float bestp = -1e30f;
            for(int e = 0; e < E; e++){
                int taken = 0;
                for(int j = 0; j < k; j++) if(chosen[j] == e){ taken = 1; break; }
                if(taken) continue;
                float sc = pr[e] + (bias ? bias[k*bs + e] : 0.0f);
                if(sc > bestp){ bestp = sc; best = e; }
            }
            if(best < 0) best = k;
            chosen[k] = best;
            assign[(size_t)k*N + n] = best;
            gate[(size_t)k*N + n] = pr[best];
        }
    }
}

/* cudalm.cu:3586-3599 (no capacity padding): histogram, exclusive prefix, stable placement. */
int orc_moe_perm(const int *assign, int N, int E, int *perm, int *off){
    for(int e = 0; e <= E; e++) off[e] = 0;
    for(int n = 0; n < N; n++){
        if((unsigned)assign[n] >= (unsigned)E) return -1 - assign[n];
        off[assign[n] + 1]++;
    }
    for(int e = 0; e < E; e++) off[e + 1] += off[e];
    int *cur = (int *)malloc(sizeof(int) * (size_t)(E > 0 ? E : 1));
    for(int e = 0; e < E; e++) cur[e] = off[e];
    for(int n = 0; n < N; n++) perm[cur[assign[n]]++] = n;
    free(cur);
    return 0;
}

/* cpu_kern.h:426-430 */
void orc_gather(const float *src, const int *perm, float *Xp, int N, int D){
    #pragma omp parallel for schedule(static) if((long)N*D >= 32768)
    for(int j = 0; j < N; j++){
        float *o = Xp + (size_t)j*D;
        if(perm[j] < 0) memset(o, 0, (size_t)D*4);
        else memcpy(o, src + (size_t)perm[j]*D, (size_t)D*4);
    }
}
/* cpu_kern.h:431-436: out[perm[j]] += gate[perm[j]] * yp[j] (multiply, then add) */
void orc_scatter_gate(const float *yp, const int *perm, const float *gate, float *out, int N, int D){
    #pragma omp parallel for schedule(static) if((long)N*D >= 32768)
    for(int j = 0; j < N; j++){
        int n = perm[j]; if(n < 0) continue;
        float g = gate[n]; float *o = out + (size_t)n*D; const float *y = yp + (size_t)j*D;
        for(int k = 0; k < D; k++) o[k] = o[k] + g * y[k];
    }
}
/* cpu_kern.h:445-450 */
void orc_scatter_add(const float *dXp, const int *perm, float *dst, int N, int D){
    #pragma omp parallel for schedule(static) if((long)N*D >= 32768)
    for(int j = 0; j < N; j++){
        int n = perm[j]; if(n < 0) continue;
        float *o = dst + (size_t)n*D; const float *x = dXp + (size_t)j*D;
        for(int k = 0; k < D; k++) o[k] += x[k];
    }
}
/* cpu_kern.h:454-468: d_gate[n] = dout[n] . yp[j]; dyp[j] = gate[n] * dout[n] */
void orc_moe_dgate(const float *dout, const float *yp, const int *perm, const float *gate,
                   float *d_gate, float *dyp, int N, int D){
    #pragma omp parallel for schedule(static) if((long)N*D >= 32768)
    for(int j = 0; j < N; j++){
        int n = perm[j]; float *dy = dyp + (size_t)j*D;
        if(n < 0){ memset(dy, 0, (size_t)D*4); continue; }
        const float *dr = dout + (size_t)n*D, *y = yp + (size_t)j*D;
        double acc = 0;                          /* the reference sums in fp32 SIMD lanes; order-free to 1e-6 */
        for(int k = 0; k < D; k++) acc += (double)dr[k] * (double)y[k];
        d_gate[n] = (float)acc;
        float g = gate[n];
        for(int k = 0; k < D; k++) dy[k] = g * dr[k];
    }
}
/* cpu_kern.h:376-383: silu(g) * u with the polynomial sigmoid */
void orc_swiglu(const float *G, const float *U, float *O, size_t n){
    #pragma omp parallel for schedule(static) if(n >= 32768)
    for(long i = 0; i < (long)n; i++){ float z = G[i]; O[i] = z * orc_fsig(z) * U[i]; }
}
/* cpu_kern.h:384-394 */
void orc_swiglu_bwd(const float *Gg, const float *U, const float *dact, float *dg, float *du, size_t n){
    #pragma omp parallel for schedule(static) if(n >= 32768)
    for(long i = 0; i < (long)n; i++){
        float z = Gg[i], sg = orc_fsig(z), silu = z * sg, ds = sg + z * sg * (1.0f - sg);
        dg[i] = dact[i] * U[i] * ds;
        du[i] = dact[i] * silu;
    }
}

/* ------------------------------------------------------------------------------------------
 * One MoE expert-FFN layer on the rendered view
 * ---------------------------------------------------------------------------------------- */
orc_moe_ws *orc_moe_ws_new(int N, int D, int F, int E, int K){
    orc_moe_ws *w = (orc_moe_ws *)calloc(1, sizeof *w);
    w->N = N; w->D = D; w->F = F; w->E = E; w->K = K;
    size_t nd = (size_t)N*D, nf = (size_t)N*F;
    w->perm = (int *)malloc(sizeof(int)*(size_t)K*N);
    w->off  = (int *)malloc(sizeof(int)*(size_t)K*(E+1));
    w->Xp = (float *)malloc(4*nd); w->yp = (float *)malloc(4*nd);
    w->gp = (float *)malloc(4*nf); w->up = (float *)malloc(4*nf); w->ap = (float *)malloc(4*nf);
    w->dyp = (float *)malloc(4*nd); w->dXp = (float *)malloc(4*nd);
    w->dap = (float *)malloc(4*nf); w->dgp = (float *)malloc(4*nf); w->dup = (float *)malloc(4*nf);
    return w;
}
void orc_moe_ws_bf16(orc_moe_ws *w, int on){ w->bf16_inter = on; }
void orc_bf16_round_n(float *x, size_t n);
static void inter(const orc_moe_ws *w, float *x, size_t n){ if(w->bf16_inter) orc_bf16_round_n(x, n); }
void orc_moe_ws_free(orc_moe_ws *w){
    if(!w) return;
    free(w->perm); free(w->off); free(w->Xp); free(w->yp); free(w->gp); free(w->up); free(w->ap);
    free(w->dyp); free(w->dXp); free(w->dap); free(w->dgp); free(w->dup); free(w);
}

static void experts_fwd(orc_moe_ws *w, const int *off, const float *w1, const float *w3, const float *w2){
    int D = w->D, F = w->F; size_t DF = (size_t)D*F;
    for(int e = 0; e < w->E; e++){
        int ne = off[e+1] - off[e]; if(!ne) continue;
        orc_gemm_nn(w->Xp + (size_t)off[e]*D, w1 + e*DF, w->gp + (size_t)off[e]*F, ne, D, F);
        orc_gemm_nn(w->Xp + (size_t)off[e]*D, w3 + e*DF, w->up + (size_t)off[e]*F, ne, D, F);
    }
    orc_swiglu(w->gp, w->up, w->ap, (size_t)w->N*F);
    inter(w, w->ap, (size_t)w->N*F);
    for(int e = 0; e < w->E; e++){
        int ne = off[e+1] - off[e]; if(!ne) continue;
        orc_gemm_nn(w->ap + (size_t)off[e]*F, w2 + e*DF, w->yp + (size_t)off[e]*D, ne, F, D);
    }
}

/* cudalm.cu:4189-4228 with grouped fp32 GEMMs: per pass gather -> w1,w3 -> swiglu -> w2 ->
 * gated scatter into out. */
int orc_moe_forward(orc_moe_ws *w, const float *x, const float *w1, const float *w3, const float *w2,
                    const int *assign, const float *gate, float *out){
    int N = w->N, D = w->D, E = w->E;
    for(int k = 0; k < w->K; k++){
        int *prm = w->perm + (size_t)k*N, *off = w->off + (size_t)k*(E+1);
        int rc = orc_moe_perm(assign + (size_t)k*N, N, E, prm, off);
        if(rc) return rc;
    }
    for(int k = 0; k < w->K; k++){
        int *prm = w->perm + (size_t)k*N, *off = w->off + (size_t)k*(E+1);
        orc_gather(x, prm, w->Xp, N, D);
        inter(w, w->Xp, (size_t)N*D);
        experts_fwd(w, off, w1, w3, w2);
        orc_scatter_gate(w->yp, prm, gate + (size_t)k*N, out, N, D);
    }
    return 0;
}

/* cudalm.cu:4286-4371, stash off: per pass recompute the forward, dgate, w2 wgrad+dgrad,
 * swiglu backward, w1/w3 wgrad + dgrad (second one accumulates), scatter-add into dx. */
void orc_moe_backward(orc_moe_ws *w, const float *x, const float *w1, const float *w3, const float *w2,
                      const float *gate, const float *dout, float *dx, float *dgate,
                      float *Gw1, float *Gw3, float *Gw2){
    int N = w->N, D = w->D, F = w->F, E = w->E; size_t DF = (size_t)D*F;
    memset(dx, 0, (size_t)N*D*4);
    for(int k = 0; k < w->K; k++){
        int *prm = w->perm + (size_t)k*N, *off = w->off + (size_t)k*(E+1);
        orc_gather(x, prm, w->Xp, N, D);
        inter(w, w->Xp, (size_t)N*D);
        experts_fwd(w, off, w1, w3, w2);
        orc_moe_dgate(dout, w->yp, prm, gate + (size_t)k*N, dgate + (size_t)k*N, w->dyp, N, D);
        inter(w, w->dyp, (size_t)N*D);
        for(int e = 0; e < E; e++){
            int ne = off[e+1] - off[e]; if(!ne) continue;
            orc_gemm_nt(w->ap + (size_t)off[e]*F, w->dyp + (size_t)off[e]*D, Gw2 + e*DF, ne, F, D);
            orc_gemm_tn(w->dyp + (size_t)off[e]*D, w2 + e*DF, w->dap + (size_t)off[e]*F, ne, D, F, 0.0f);
        }
        orc_swiglu_bwd(w->gp, w->up, w->dap, w->dgp, w->dup, (size_t)N*F);
        inter(w, w->dgp, (size_t)N*F); inter(w, w->dup, (size_t)N*F);
        for(int e = 0; e < E; e++){
            int ne = off[e+1] - off[e]; if(!ne) continue;
            orc_gemm_nt(w->Xp + (size_t)off[e]*D, w->dgp + (size_t)off[e]*F, Gw1 + e*DF, ne, D, F);
            orc_gemm_nt(w->Xp + (size_t)off[e]*D, w->dup + (size_t)off[e]*F, Gw3 + e*DF, ne, D, F);
            orc_gemm_tn(w->dgp + (size_t)off[e]*F, w1 + e*DF, w->dXp + (size_t)off[e]*D, ne, F, D, 0.0f);
            orc_gemm_tn(w->dup + (size_t)off[e]*F, w3 + e*DF, w->dXp + (size_t)off[e]*D, ne, F, D, 1.0f);
        }
        orc_scatter_add(w->dXp, prm, dx, N, D);
    }
}

/* ------------------------------------------------------------------------------------------
 * q4n wire format
 * ---------------------------------------------------------------------------------------- */
/* cudalm.cu:638-656. For each group: amax; candidate scales amax/k for k = 7..1 and their two
 * neighbours on each side; the first candidate for which every value is exactly scale * an integer
 * of magnitude <= 7 wins. An all-zero group keeps scale 0. */
size_t orc_q4n_quantize(const float *P, size_t n, int group, unsigned char *out, size_t cap, size_t *nraw){
    size_t o = 0, raw = 0;
    for(size_t i = 0; i < n; i += (size_t)group){
        int g = (i + (size_t)group <= n) ? group : (int)(n - i), ok = 0;
        float amax = 0, s = 0;
        for(int j = 0; j < g; j++){ float a = fabsf(P[i+j]); if(a > amax) amax = a; }
        if(amax == 0) ok = 1;
        for(int k = 7; k >= 1 && !ok; k--){
            float s0 = amax / (float)k, c[5];
            c[0] = s0; c[1] = nextafterf(s0, 0); c[2] = nextafterf(s0, INFINITY);
            c[3] = nextafterf(c[1], 0); c[4] = nextafterf(c[2], INFINITY);
            for(int t = 0; t < 5 && !ok; t++){
                s = c[t]; ok = 1;
                for(int j = 0; j < g && ok; j++){ float d = rintf(P[i+j] / s); if(fabsf(d) > 7 || d * s != P[i+j]) ok = 0; }
            }
        }
        if(!ok){
            float nanv = NAN;
            if(o + 4 + 4*(size_t)g <= cap){ memcpy(out + o, &nanv, 4); memcpy(out + o + 4, P + i, 4*(size_t)g); }
            o += 4 + 4*(size_t)g; raw++; continue;
        }
        if(o + 4 <= cap) memcpy(out + o, &s, 4);
        o += 4;
        for(int j = 0; j < g; j += 2){
            int a = s ? (int)rintf(P[i+j] / s) : 0, b = (j + 1 < g && s) ? (int)rintf(P[i+j+1] / s) : 0;
            if(o < cap) out[o] = (unsigned char)((a & 15) | ((b & 15) << 4));
            o++;
        }
    }
    if(nraw) *nraw = raw;
    return o;
}
/* cudalm.cu:688-696; returns 0 on a short buffer */
int orc_q4n_dequantize(const unsigned char *buf, size_t len, float *P, size_t n, int group){
    size_t o = 0;
    for(size_t i = 0; i < n; i += (size_t)group){
        int g = (i + (size_t)group <= n) ? group : (int)(n - i);
        float s;
        if(o + 4 > len) return 0;
        memcpy(&s, buf + o, 4); o += 4;
        if(s != s){ if(o + 4*(size_t)g > len) return 0; memcpy(P + i, buf + o, 4*(size_t)g); o += 4*(size_t)g; continue; }
        for(int j = 0; j < g; j += 2){
            if(o + 1 > len) return 0;
            unsigned char b = buf[o++];
            P[i+j] = (float)((int)((b & 15) ^ 8) - 8) * s;
            if(j + 1 < g) P[i+j+1] = (float)((int)((b >> 4) ^ 8) - 8) * s;
        }
    }
    return 1;
}

/* ------------------------------------------------------------------------------------------
 * Reciprocal-and-correct division identity (used by the GPU step kernel for the per-group divisors)
 * ---------------------------------------------------------------------------------------- */
size_t orc_recip_div_mismatches(uint64_t seed, size_t n){
    size_t bad = 0;
    #pragma omp parallel for reduction(+:bad) schedule(static)
    for(long i = 0; i < (long)n; i++){
        uint64_t h = orc_splitmix64(seed * 0x9E3779B97F4A7C15ULL + (uint64_t)i), h2 = orc_splitmix64(h);
        uint32_t be = 127 - 60 + (uint32_t)(h % 121), bm = (uint32_t)(h >> 20) & 0x7FFFFF;
        uint32_t bb = (be << 23) | bm;
        int ae = (int)be + 8 - (int)(h2 % 40); if(ae < 1) ae = 1;
        uint32_t ab = ((uint32_t)ae << 23) | ((uint32_t)(h2 >> 10) & 0x7FFFFF) | ((uint32_t)(h2 >> 63) << 31);
        float a, b; memcpy(&a, &ab, 4); memcpy(&b, &bb, 4);
        float y = 1.0f / b, q = a * y, r = fmaf(-q, b, a), q2 = fmaf(r, y, q), ref = a / b;
        if(memcmp(&q2, &ref, 4) != 0) bad++;
    }
    return bad;
}

/* ------------------------------------------------------------------------------------------
 * Deterministic synthetic inputs
 * ---------------------------------------------------------------------------------------- */
uint64_t orc_splitmix64(uint64_t x){
    x += 0x9E3779B97F4A7C15ULL;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    return x ^ (x >> 31);
}
static inline uint64_t stream_key(uint64_t seed, uint64_t tensor_id){ return (seed << 32) + tensor_id; }
/* uniform in [0,1): top 24 bits of splitmix64(key*GOLD + counter) */
static inline float u24(uint64_t key, uint64_t ctr){
    uint64_t h = orc_splitmix64(key * 0xD1342543DE82EF95ULL + ctr);
    return (float)(h >> 40) * (1.0f / 16777216.0f);
}
void orc_fill_normal(float *dst, size_t n, uint64_t seed, uint64_t tensor_id, float scale){
    uint64_t key = stream_key(seed, tensor_id);
    #pragma omp parallel for schedule(static) if(n >= 65536)
    for(long i = 0; i < (long)n; i++){
        float acc = 0.0f;
        for(int k = 0; k < 12; k++) acc = acc + u24(key, (uint64_t)i*12 + (uint64_t)k);
        dst[i] = (acc - 6.0f) * scale;
    }
}
void orc_fill_uniform(float *dst, size_t n, uint64_t seed, uint64_t tensor_id, float lo, float hi){
    uint64_t key = stream_key(seed, tensor_id);
    #pragma omp parallel for schedule(static) if(n >= 65536)
    for(long i = 0; i < (long)n; i++) dst[i] = lo + (hi - lo) * u24(key, (uint64_t)i);
}
static inline int irange(uint64_t key, uint64_t ctr, int lo, int hi){
    uint64_t h = orc_splitmix64(key * 0xD1342543DE82EF95ULL + ctr);
    return lo + (int)((h >> 33) % (uint64_t)(hi - lo + 1));
}
void orc_fill_int8(int8_t *dst, size_t n, uint64_t seed, uint64_t tensor_id, int lo, int hi){
    uint64_t key = stream_key(seed, tensor_id);
    #pragma omp parallel for schedule(static) if(n >= 65536)
    for(long i = 0; i < (long)n; i++) dst[i] = (int8_t)irange(key, (uint64_t)i, lo, hi);
}
void orc_fill_u8(uint8_t *dst, size_t n, uint64_t seed, uint64_t tensor_id, int lo, int hi){
    uint64_t key = stream_key(seed, tensor_id);
    #pragma omp parallel for schedule(static) if(n >= 65536)
    for(long i = 0; i < (long)n; i++) dst[i] = (uint8_t)irange(key, (uint64_t)i, lo, hi);
}
void orc_fill_digits(int8_t *d, size_t nq, uint64_t seed, uint64_t tensor_id, int dmax, int packed){
    uint64_t key = stream_key(seed, tensor_id);
    if(!packed){
        #pragma omp parallel for schedule(static) if(nq >= 65536)
        for(long i = 0; i < (long)nq; i++) d[i] = (int8_t)irange(key, (uint64_t)i, -dmax, dmax);
        return;
    }
    size_t nb = (nq + 1) / 2;
    #pragma omp parallel for schedule(static) if(nb >= 65536)
    for(long b = 0; b < (long)nb; b++){
        int lo = irange(key, (uint64_t)(2*b), -dmax, dmax) & 15;
        int hi = ((size_t)(2*b + 1) < nq) ? (irange(key, (uint64_t)(2*b + 1), -dmax, dmax) & 15) : 0;
        d[b] = (int8_t)((hi << 4) | lo);
    }
}
/* cudalm.cu:334-338: round to nearest even on the top 16 bits */
float orc_bf16_round(float x){
    uint32_t u; memcpy(&u, &x, 4);
    u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
    float y; memcpy(&y, &u, 4); return y;
}
void orc_bf16_round_n(float *x, size_t n){
    #pragma omp parallel for schedule(static) if(n >= 65536)
    for(long i = 0; i < (long)n; i++) x[i] = orc_bf16_round(x[i]);
}

/* ---- gradient-norm clipping: k_sqsum and k_gnorm, cpu_kern.h:533-546 (GPU forms cudalm.cu:2794-2816) ---- */
void orc_sqsum(const float *G, uint64_t n, float *part64){
    for(int c = 0; c < 64; c++){
        const uint64_t i0 = n * (uint64_t)c / 64, i1 = n * (uint64_t)(c + 1) / 64;
        double s = 0.0;
        for(uint64_t i = i0; i < i1; i++) s += (double)G[i] * G[i];
        part64[c] = (float)s;
    }
}
void orc_gnorm(const float *part, int nside, int clip_side, float *gs){
    double ss = 0.0, sd = 0.0;
    for(int i = 0; i < 64; i++) ss += part[i];
    for(int i = 64; i < 64 * (1 + nside); i++) sd += part[i];
    float gn = (float)sqrt(clip_side ? ss + sd : ss);
    if(!isfinite(sd)) gn = NAN;
    gs[0] = gn > 1.0f ? 1.0f / gn : 1.0f;
    gs[1] = gn;
}
