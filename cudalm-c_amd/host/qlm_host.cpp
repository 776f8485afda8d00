/* qlm_host.cpp -- see qlm_host.h. Host logic only; every device operation goes through libqlmx. */
#include "qlm_host.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

static void ck(int rc, const char *what){
    if(rc != QLMX_OK){ fprintf(stderr, "HIP error: %s at %s\n", qlmx_last_error(), what); exit(1); }
}
void *dmalloc(size_t bytes){ void *p = NULL; ck(qlmx_malloc(&p, bytes), "hipMalloc"); return p; }

/* qlm.cuh:448-455 */
void qlm_add_span(Qlm *q, unsigned long long pof, unsigned long long n){
    if(q->nspan >= QLM_MAXSPAN) return;
    QSpanD *sp = &q->spanH[q->nspan];
    sp->pof = pof; sp->gof = pof; sp->qi0 = q->nq; sp->n = n;
    sp->gi0 = (int)q->ngrp; sp->ngrp = (int)((n + q->group - 1) / q->group);
    sp->sref = 1.0f;
    q->nq += n; q->ngrp += sp->ngrp; q->nspan++;
}

/* qlm.cuh:458-541: environment, span table, float gaps, allocation, encode, frozen reference scales,
 * first render. */
void qlm_gpu_init(Qlm *q, const QlmSpanDesc *spans, int nspan, float *P, size_t np){
    memset(q, 0, sizeof(*q));
    const char *e;
    int bits = (e = getenv("QLM_BITS")) ? atoi(e) : 4;
    q->dmax  = bits <= 2 ? 1 : bits == 3 ? 3 : bits == 4 ? 7 : 127;
    q->group = (e = getenv("QLM_GROUP")) ? atoi(e) : 128;
    if(q->group < 32) q->group = 32;
    if(q->group > 256) q->group = 256;
    q->lrmode = (e = getenv("QLM_LRMODE")) ? (!strcmp(e, "abs") ? 1 : 0) : 0;
    q->servo_every = (e = getenv("QLM_SERVO")) ? atoi(e) : 100;
    q->adam = 1;
    q->v4 = (e = getenv("QLM_V4")) ? (atoi(e) != 0) : 0;
    if((e = getenv("QLM_OPT")) && !strcmp(e, "qlion")) q->adam = 0;
    q->fstar = (e = getenv("QLM_FSTAR")) ? (float)atof(e) : (q->dmax == 1 ? 0.60f : 1.5f / (float)q->group);
    q->f_hi = q->fstar * 1.5f; q->f_lo = q->fstar * 0.5f;
    q->np = np;
    q->render_p = P != NULL;

    q->spanH = (QSpanD *)calloc(QLM_MAXSPAN, sizeof(QSpanD));
    for(int i = 0; i < nspan; i++) qlm_add_span(q, spans[i].pof, spans[i].n);
    {   /* float spans = the gaps between quantized spans */
        unsigned long long cur = 0;
        for(int i = 0; i < q->nspan; i++){
            if(q->spanH[i].pof > cur){ q->fs_off[q->nfs] = cur; q->fs_n[q->nfs] = q->spanH[i].pof - cur; q->nfs++; }
            cur = q->spanH[i].pof + q->spanH[i].n;
        }
        if(cur < np){ q->fs_off[q->nfs] = cur; q->fs_n[q->nfs] = np - cur; q->nfs++; }
        unsigned long long acc = 0;
        for(int i = 0; i < q->nfs; i++){ q->fs_cs[i] = acc; acc += q->fs_n[i]; }
        q->nfloat = acc;
    }
    q->packed = (q->dmax <= 7);
    q->d  = (signed char *)dmalloc((size_t)qlmx_qd_bytes(q->nq, q->packed));
    q->r  = (signed char *)dmalloc(q->nq);
    q->m8 = (signed char *)dmalloc(q->nq);
    q->v8 = q->adam ? (unsigned char *)dmalloc(q->nq) : NULL;
    ck(qlmx_memset(q->m8, 0, q->nq, NULL), "qlm m8 zero");
    if(q->adam) ck(qlmx_memset(q->v8, 0, q->nq, NULL), "qlm v8 zero");
    q->s   = (float *)dmalloc(q->ngrp * 4);
    q->m8s = (float *)dmalloc(q->ngrp * 4);
    q->v8s = q->adam ? (float *)dmalloc(q->ngrp * 4) : NULL;
    ck(qlmx_memset(q->m8s, 0, q->ngrp * 4, NULL), "qlm m8s zero");
    if(q->adam) ck(qlmx_memset(q->v8s, 0, q->ngrp * 4, NULL), "qlm v8s zero");
    q->statD = (long long *)dmalloc(4 * 8);
    ck(qlmx_memset(q->statD, 0, 32, NULL), "qlm stat zero");
    q->spanD = (QSpanD *)dmalloc((size_t)q->nspan * sizeof(QSpanD));
    ck(qlmx_memcpy_h2d(q->spanD, q->spanH, (size_t)q->nspan * sizeof(QSpanD)), "qlm span h2d");
    if(P){
        ck(qlmx_encode(P, q->d, q->r, q->s, q->spanD, q->nspan, q->group, q->dmax, q->packed, (int)q->ngrp, NULL), "qlm encode");
        /* freeze each span's reference scale: mean of its group scales, in double (qlm.cuh:527-536) */
        std::vector<float> sh(q->ngrp);
        ck(qlmx_memcpy_d2h(sh.data(), q->s, q->ngrp * 4), "qlm s d2h");
        for(int i = 0; i < q->nspan; i++){
            double acc = 0;
            for(int g = 0; g < q->spanH[i].ngrp; g++) acc += sh[q->spanH[i].gi0 + g];
            q->spanH[i].sref = (float)(acc / (double)q->spanH[i].ngrp);
        }
        ck(qlmx_memcpy_h2d(q->spanD, q->spanH, (size_t)q->nspan * sizeof(QSpanD)), "qlm span h2d 2");
        ck(qlmx_render(P, q->d, q->s, q->spanD, q->nspan, q->group, q->packed, 0, (int)q->ngrp, NULL), "qlm render");
    }
    q->on = 1;
}

void qlm_gpu_render(Qlm *q, float *P){
    ck(qlmx_render(P, q->d, q->s, q->spanD, q->nspan, q->group, q->packed, 0, (int)q->ngrp, NULL), "qlm render");
}
/* qlm.cuh:586-591 generalised: render the groups of spans [span0, span0+nspans) */
void qlm_render_spans(Qlm *q, float *P, int span0, int nspans){
    int gi0 = q->spanH[span0].gi0, ng = 0;
    for(int i = span0; i < span0 + nspans; i++) ng += q->spanH[i].ngrp;
    ck(qlmx_render(P, q->d, q->s, q->spanD, q->nspan, q->group, q->packed, gi0, ng, NULL), "qlm render layer");
}

/* qlm.cuh:377-397. The QLM_V4 switch travels as an argument of the C ABI; here it is read from
 * the environment once, as the reference does (qlm.cuh:68-72). */
void qlm_step_launch(float *P, const float *G, signed char *d, signed char *r, float *s,
                     signed char *m8, float *m8s, unsigned char *v8, float *v8s,
                     const QSpanD *sp, int nspan, int group, int dmax,
                     float lr, float b1, float b2, float wd, float gscale, const float *gsp,
                     float inv_bc1, float inv_sqrt_bc2, int lrmode,
                     unsigned long long t, int adam, long long *stat, int packed, int gi_base, int ng){
    static int v4 = -1;
    if(v4 < 0){ const char *e = getenv("QLM_V4"); v4 = e && atoi(e); }
    ck(qlmx_step(P, G, d, r, s, m8, m8s, v8, v8s, sp, nspan, group, dmax, lr, b1, b2, wd, gscale, gsp,
                 inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4, NULL), "qlm step");
}

/* cudalm.cu:6082-6103 without the float spans' AdamW */
void qlm_gpu_update(Qlm *q, float *P, float *G, float lr, float b1, float b2, float wd,
                    float bc1, float bc2, int t, const float *gs){
    float inv_bc1 = 1.0f / bc1, inv_sqrt_bc2 = 1.0f / sqrtf(bc2);
    qlm_step_launch(q->render_p ? P : NULL, G, q->d, q->r, q->s, q->m8, q->m8s, q->v8, q->v8s, q->spanD, q->nspan,
                    q->group, q->dmax, lr, b1, b2, wd, 1.0f, gs, inv_bc1, inv_sqrt_bc2, q->lrmode,
                    (unsigned long long)t, q->adam, getenv("CUDALM_QLM_DIAG") ? q->statD : NULL, q->packed, 0, (int)q->ngrp);
    if(q->servo_every > 0 && (t % q->servo_every) == 0)
        ck(qlmx_servo(q->d, q->r, q->s, q->spanD, q->nspan, q->group, q->dmax, q->f_hi, q->f_lo, q->packed, (int)q->ngrp, NULL), "qlm servo");
}

/* cudalm.cu:6110-6135 without the float spans' AdamW and the diagnostics */
void qlm_fused_spans(Qlm *q, float *P, float *G, int span0, int nspans, size_t g0, size_t gn, float *part64,
                     float lr, float wd, int t, float prev_gn){
    const float b1 = 0.9f, b2 = 0.95f;
    const float bc1 = 1.0f - powf(b1, (float)t), bc2 = 1.0f - powf(b2, (float)t);
    const float inv_bc1 = 1.0f / bc1, inv_sqrt_bc2 = 1.0f / sqrtf(bc2);
    const float gscale = prev_gn > 1.0f ? 1.0f / prev_gn : 1.0f;
    ck(qlmx_sqsum(G + g0, (unsigned long long)gn, part64, NULL), "fused sqsum");
    int gi0 = q->spanH[span0].gi0, ng = 0;
    for(int i = span0; i < span0 + nspans; i++) ng += q->spanH[i].ngrp;
    qlm_step_launch(q->render_p ? P : NULL, G, q->d, q->r, q->s, q->m8, q->m8s, q->v8, q->v8s, q->spanD, q->nspan,
                    q->group, q->dmax, lr, b1, b2, wd, gscale, NULL, inv_bc1, inv_sqrt_bc2, q->lrmode,
                    (unsigned long long)t, q->adam, NULL, q->packed, gi0, ng);
}
void qlm_fused_layer(Qlm *q, float *P, float *G, size_t layer_g0, size_t layer_gn, float *gnpart, int l,
                     float lr, float wd, int t, float prev_gn){
    qlm_fused_spans(q, P, G, 7 * l, 7, layer_g0, layer_gn, gnpart + 64 * (size_t)l, lr, wd, t, prev_gn);
}
/* cudalm.cu:6176-6186 */
float qlm_fused_tail(const float *gnpart, int L, const float *extra, int nextra){
    const size_t nsl = 64 * (size_t)L, nex = 64 * (size_t)nextra;
    std::vector<float> ph(nsl + nex);
    if(nsl) ck(qlmx_memcpy_d2h(ph.data(), gnpart, nsl * 4), "fused sqsum d2h");
    if(nex) ck(qlmx_memcpy_d2h(ph.data() + nsl, extra, nex * 4), "fused tail sqsum d2h");
    double ss = 0;
    for(size_t i = 0; i < nsl + nex; i++) ss += ph[i];
    return (float)sqrt(ss);
}

/* qlm.cuh:678-683 */
double qlm_persist_bytes(const Qlm *q){
    return (double)qlmx_qd_bytes(q->nq, q->packed) + (double)q->nq * 1.0 + (double)q->nq * (q->adam ? 2.0 : 1.0)
         + (double)q->ngrp * 4.0 * (q->adam ? 3.0 : 2.0);
}

/* ---- .opt.q checkpoint: magic QLMH, int hdr[6] = {dmax, group, adam, nspan, packed, iter},
 * u64 nq, ngrp, nfloat, bf16 Mc, Vc (float spans), packed d, r, m8, [v8], fp32 s, m8s, [v8s],
 * trailer "SREF" + nspan + per-span sref, trailer "PGN1" + previous grad norm (qlm.cuh:702-738).
 * Written to <path>.tmp and renamed, as the reference does. ---- */
int qlm_save(const Qlm *q, const char *path, int iter, float prev_gn){
    char tmp[1300]; snprintf(tmp, sizeof tmp, "%s.tmp", path);
    FILE *f = fopen(tmp, "wb"); if(!f) return 0;
    int hdr[6] = {q->dmax, q->group, q->adam, q->nspan, q->packed, iter};
    unsigned long long nq = q->nq, ng = q->ngrp, nf = q->nfloat, nd = qlmx_qd_bytes(nq, q->packed);
    std::vector<signed char> hd(nd), hr(nq), hm(nq);
    std::vector<unsigned char> hv(q->adam ? nq : 0);
    std::vector<float> hs(ng), hms(ng), hvs(q->adam ? ng : 0);
    std::vector<bf16> hM(nf, 0), hV(nf, 0);
    if(q->Mc && nf) ck(qlmx_memcpy_d2h(hM.data(), q->Mc, nf * 2), "qlm save Mc");
    if(q->Vc && nf) ck(qlmx_memcpy_d2h(hV.data(), q->Vc, nf * 2), "qlm save Vc");
    ck(qlmx_memcpy_d2h(hd.data(), q->d, nd), "qlm save d");
    ck(qlmx_memcpy_d2h(hr.data(), q->r, nq), "qlm save r");
    ck(qlmx_memcpy_d2h(hm.data(), q->m8, nq), "qlm save m8");
    if(q->adam) ck(qlmx_memcpy_d2h(hv.data(), q->v8, nq), "qlm save v8");
    ck(qlmx_memcpy_d2h(hs.data(), q->s, ng * 4), "qlm save s");
    ck(qlmx_memcpy_d2h(hms.data(), q->m8s, ng * 4), "qlm save m8s");
    if(q->adam) ck(qlmx_memcpy_d2h(hvs.data(), q->v8s, ng * 4), "qlm save v8s");
    int ok = fwrite("QLMH", 1, 4, f) == 4 && fwrite(hdr, 4, 6, f) == 6
          && fwrite(&nq, 8, 1, f) == 1 && fwrite(&ng, 8, 1, f) == 1 && fwrite(&nf, 8, 1, f) == 1
          && fwrite(hM.data(), 2, nf, f) == nf && fwrite(hV.data(), 2, nf, f) == nf
          && fwrite(hd.data(), 1, nd, f) == nd && fwrite(hr.data(), 1, nq, f) == nq
          && fwrite(hm.data(), 1, nq, f) == nq && (q->adam ? fwrite(hv.data(), 1, nq, f) == nq : 1)
          && fwrite(hs.data(), 4, ng, f) == ng && fwrite(hms.data(), 4, ng, f) == ng
          && (q->adam ? fwrite(hvs.data(), 4, ng, f) == ng : 1);
    if(ok){ int ns = q->nspan; ok = fwrite("SREF", 1, 4, f) == 4 && fwrite(&ns, 4, 1, f) == 1;
            for(int i = 0; ok && i < ns; i++) ok = fwrite(&q->spanH[i].sref, 4, 1, f) == 1; }
    if(ok) ok = fwrite("PGN1", 1, 4, f) == 4 && fwrite(&prev_gn, 4, 1, f) == 1;
    if(fflush(f) != 0) ok = 0;
    if(fclose(f) != 0) ok = 0;
    if(!ok){ remove(tmp); return 0; }
    return rename(tmp, path) == 0;
}

/* qlm.cuh:740-788: a file of another shape is ignored with a warning and 0 is returned */
int qlm_load(Qlm *q, const char *path, int *iter, float *prev_gn){
    FILE *f = fopen(path, "rb"); if(!f) return 0;
    char mg[4]; int hdr[6]; unsigned long long nq, ng, nf;
    if(fread(mg, 1, 4, f) != 4 || memcmp(mg, "QLMH", 4)){ fclose(f); return 0; }
    if(fread(hdr, 4, 6, f) != 6 || fread(&nq, 8, 1, f) != 1 || fread(&ng, 8, 1, f) != 1 || fread(&nf, 8, 1, f) != 1){ fclose(f); return 0; }
    if(hdr[0] != q->dmax || hdr[1] != q->group || hdr[2] != q->adam || hdr[4] != q->packed
       || nq != q->nq || ng != q->ngrp || nf > q->nfloat){
        fprintf(stderr, "[qlm] %s has a different shape (bits/group/opt) -- ignoring\n", path);
        fclose(f); return 0;
    }
    if(iter) *iter = hdr[5];
    unsigned long long nd = qlmx_qd_bytes(nq, q->packed);
    std::vector<signed char> hd(nd), hr(nq), hm(nq);
    std::vector<unsigned char> hv(q->adam ? nq : 0);
    std::vector<float> hs(ng), hms(ng), hvs(q->adam ? ng : 0);
    std::vector<bf16> hM(nf), hV(nf);
    int ok = fread(hM.data(), 2, nf, f) == nf && fread(hV.data(), 2, nf, f) == nf
          && fread(hd.data(), 1, nd, f) == nd && fread(hr.data(), 1, nq, f) == nq
          && fread(hm.data(), 1, nq, f) == nq && (q->adam ? fread(hv.data(), 1, nq, f) == nq : 1)
          && fread(hs.data(), 4, ng, f) == ng && fread(hms.data(), 4, ng, f) == ng
          && (q->adam ? fread(hvs.data(), 4, ng, f) == ng : 1);
    std::vector<float> sr; int have_sref = 0;
    if(ok){ char tm[4]; int ns = 0;
        if(fread(tm, 1, 4, f) == 4 && !memcmp(tm, "SREF", 4) && fread(&ns, 4, 1, f) == 1 && ns == q->nspan){
            sr.resize(ns); have_sref = fread(sr.data(), 4, (size_t)ns, f) == (size_t)ns; }
        float pg;
        if(have_sref && fread(tm, 1, 4, f) == 4 && !memcmp(tm, "PGN1", 4) && fread(&pg, 4, 1, f) == 1 && pg > 0.0f && isfinite(pg) && prev_gn) *prev_gn = pg; }
    fclose(f);
    if(!ok) return 0;
    if(have_sref){
        for(int i = 0; i < q->nspan; i++) q->spanH[i].sref = sr[i];
        ck(qlmx_memcpy_h2d(q->spanD, q->spanH, (size_t)q->nspan * sizeof(QSpanD)), "qlm load span");
    } else
        fprintf(stderr, "[qlm] %s has no reference-scale record: sref is re-derived from the current weights\n", path);
    if(q->Mc && nf) ck(qlmx_memcpy_h2d(q->Mc, hM.data(), nf * 2), "qlm load Mc");
    if(q->Vc && nf) ck(qlmx_memcpy_h2d(q->Vc, hV.data(), nf * 2), "qlm load Vc");
    ck(qlmx_memcpy_h2d(q->d, hd.data(), nd), "qlm load d");
    ck(qlmx_memcpy_h2d(q->r, hr.data(), nq), "qlm load r");
    ck(qlmx_memcpy_h2d(q->m8, hm.data(), nq), "qlm load m8");
    if(q->adam) ck(qlmx_memcpy_h2d(q->v8, hv.data(), nq), "qlm load v8");
    ck(qlmx_memcpy_h2d(q->s, hs.data(), ng * 4), "qlm load s");
    ck(qlmx_memcpy_h2d(q->m8s, hms.data(), ng * 4), "qlm load m8s");
    if(q->adam) ck(qlmx_memcpy_h2d(q->v8s, hvs.data(), ng * 4), "qlm load v8s");
    return 1;
}

void qlm_free(Qlm *q){
    void *p[] = {q->d, q->r, q->m8, q->v8, q->s, q->m8s, q->v8s, q->statD, q->spanD};
    for(void *x : p) if(x) qlmx_free(x);
    free(q->spanH);
    memset(q, 0, sizeof(*q));
}

/* ---------------------------------------------------------------------------------------------
 * Grouped expert GEMM queue (cudalm.cu:3204-3256). Queue 0: beta = 0 problems (nn and tn), queue 1:
 * tn problems with beta != 0, which accumulate into a C a queue-0 problem writes and therefore run
 * strictly after queue 0, queue 2: nt weight gradients. A flush issues each queue as one grouped
 * launch per (orientation, K, N).
 * ------------------------------------------------------------------------------------------- */
struct MgItem { int mode, K, N; qlmx_gemm_prob p; };
static std::vector<MgItem> g_q[3];
static const Qlm *g_mg_q = NULL; static const float *g_mg_P = NULL; static int g_mg_act = QLMX_ACT_F32, g_mg_math = QLMX_MATH_F32;

void mg_bind(const Qlm *q, const float *Pbase, int act_dtype, int math){ g_mg_q = q; g_mg_P = Pbase; g_mg_act = act_dtype; g_mg_math = math; }

/* pointer into P -> (digit offset, scale group) through the span table */
static void weight_of(const float *B, unsigned long long *wq, unsigned long long *wg){
    if(!g_mg_q){ fprintf(stderr, "mg: mg_bind() was not called\n"); exit(1); }
    const unsigned long long off = (unsigned long long)(B - g_mg_P);
    for(int i = 0; i < g_mg_q->nspan; i++){
        const QSpanD *sp = &g_mg_q->spanH[i];
        if(off >= sp->pof && off < sp->pof + sp->n){
            const unsigned long long in = off - sp->pof;
            if(in % (unsigned long long)g_mg_q->group){ fprintf(stderr, "mg: weight operand does not start on a scale group\n"); exit(1); }
            *wq = sp->qi0 + in; *wg = (unsigned long long)sp->gi0 + in / (unsigned long long)g_mg_q->group; return;
        }
    }
    fprintf(stderr, "mg: weight operand is not inside a quantized span\n"); exit(1);
}
static void mg_push(int qn, int mode, const void *A, const void *B, float *C, unsigned long long wq, unsigned long long wg,
                    int M, int K, int N, float beta){
    if(g_q[qn].size() >= QLMX_MAX_PROBLEMS){ fprintf(stderr, "mg queue overflow\n"); exit(1); }
    MgItem it; it.mode = mode; it.K = K; it.N = N;
    it.p.A = A; it.p.B = B; it.p.C = C; it.p.wq = wq; it.p.wg = wg; it.p.M = M; it.p.beta = beta;
    g_q[qn].push_back(it);
}
void mg_ab(const void *A, const float *B, float *C, int M, int K, int N){
    unsigned long long wq, wg; weight_of(B, &wq, &wg); mg_push(0, 0, A, NULL, C, wq, wg, M, K, N, 0.0f);
}
void mg_abt_b(const void *A, const float *B, float *C, int M, int K, int N, float beta){
    unsigned long long wq, wg; weight_of(B, &wq, &wg); mg_push(beta != 0.0f, 1, A, NULL, C, wq, wg, M, K, N, beta);
}
void mg_abt(const void *A, const float *B, float *C, int M, int K, int N){ mg_abt_b(A, B, C, M, K, N, 0.0f); }
void mg_atb(const void *A, const void *B, float *C, int M, int K, int N){ mg_push(2, 2, A, B, C, 0, 0, M, K, N, 1.0f); }

/* gate|up problems with the SwiGLU behind them: queued apart, flushed first as one call per (K, N) */
struct MgDual { int K, N; qlmx_gemm_prob gate, up; };
static std::vector<MgDual> g_qdual;
void mg_ab_swiglu(const void *A, const float *B1, const float *B3, float *gp, float *up, void *ap, int M, int K, int N){
    if(g_qdual.size() >= QLMX_MAX_PROBLEMS / 2){ fprintf(stderr, "mg queue overflow\n"); exit(1); }
    MgDual it; it.K = K; it.N = N;
    unsigned long long wq, wg;
    weight_of(B1, &wq, &wg);
    it.gate.A = A; it.gate.B = NULL; it.gate.C = gp; it.gate.wq = wq; it.gate.wg = wg; it.gate.M = M; it.gate.beta = 0.0f;
    weight_of(B3, &wq, &wg);
    it.up.A = NULL; it.up.B = ap; it.up.C = up; it.up.wq = wq; it.up.wg = wg; it.up.M = M; it.up.beta = 0.0f;
    g_qdual.push_back(it);
}
static void mg_run_dual(void){
    std::vector<char> done(g_qdual.size(), 0);
    for(size_t i = 0; i < g_qdual.size(); i++){
        if(done[i]) continue;
        std::vector<qlmx_gemm_prob> gate, up;
        for(size_t j = i; j < g_qdual.size(); j++)
            if(!done[j] && g_qdual[j].K == g_qdual[i].K && g_qdual[j].N == g_qdual[i].N){ gate.push_back(g_qdual[j].gate); up.push_back(g_qdual[j].up); done[j] = 1; }
        const int rc = qlmx_moe_gemm_nn_swiglu(g_mg_q->d, g_mg_q->s, g_mg_q->group, gate.data(), up.data(), (int)gate.size(),
                                               g_qdual[i].K, g_qdual[i].N, g_mg_act, g_mg_math, NULL);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped (gate|up): %s\n", rc, qlmx_last_error()); exit(1); }
    }
    g_qdual.clear();
}

static void mg_run(std::vector<MgItem> &v){
    std::vector<char> done(v.size(), 0);
    for(size_t i = 0; i < v.size(); i++){
        if(done[i]) continue;
        std::vector<qlmx_gemm_prob> batch;
        for(size_t j = i; j < v.size(); j++)
            if(!done[j] && v[j].mode == v[i].mode && v[j].K == v[i].K && v[j].N == v[i].N){ batch.push_back(v[j].p); done[j] = 1; }
        int rc;
        if(v[i].mode == 0)      rc = qlmx_moe_gemm_nn(g_mg_q->d, g_mg_q->s, g_mg_q->group, batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, NULL);
        else if(v[i].mode == 1) rc = qlmx_moe_gemm_tn(g_mg_q->d, g_mg_q->s, g_mg_q->group, batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, NULL);
        else                    rc = qlmx_moe_gemm_nt(batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, NULL);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped: %s\n", rc, qlmx_last_error()); exit(1); }
    }
    v.clear();
}
/* A queue-1 problem (tn, beta = 1) whose output a queue-0 tn problem of the same shape writes is that
 * problem's second half (cudalm.cu:4365-4366): on the MFMA path the two run as one continued
 * contraction per (K, N) instead of two launches with the output stored and read back in between. */
static void mg_run_pairs(void){
    if(g_mg_act != QLMX_ACT_BF16 || g_mg_math != QLMX_MATH_MFMA) return;
    std::vector<MgItem> &v0 = g_q[0], &v1 = g_q[1];
    std::vector<int> mate(v1.size(), -1);
    std::vector<char> used(v0.size(), 0);
    bool any = false;
    for(size_t j = 0; j < v1.size(); j++){
        if(v1[j].mode != 1 || v1[j].p.beta != 1.0f || v1[j].p.M == 0) continue;
        for(size_t i = 0; i < v0.size(); i++)
            if(!used[i] && v0[i].mode == 1 && v0[i].p.C == v1[j].p.C && v0[i].p.M == v1[j].p.M && v0[i].K == v1[j].K && v0[i].N == v1[j].N){
                mate[j] = (int)i; used[i] = 1; any = true; break;
            }
    }
    if(!any) return;
    std::vector<char> done(v1.size(), 0);
    for(size_t j = 0; j < v1.size(); j++){
        if(done[j] || mate[j] < 0) continue;
        std::vector<qlmx_gemm_prob> first, second;
        for(size_t k = j; k < v1.size() && first.size() < QLMX_MAX_PROBLEMS / 2; k++)
            if(!done[k] && mate[k] >= 0 && v1[k].K == v1[j].K && v1[k].N == v1[j].N){ first.push_back(v0[mate[k]].p); second.push_back(v1[k].p); done[k] = 1; }
        const int rc = qlmx_moe_gemm_tn_pair(g_mg_q->d, g_mg_q->s, g_mg_q->group, first.data(), second.data(), (int)first.size(),
                                             v1[j].K, v1[j].N, g_mg_act, g_mg_math, NULL);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped (pairs): %s\n", rc, qlmx_last_error()); exit(1); }
    }
    std::vector<MgItem> r0, r1;
    for(size_t i = 0; i < v0.size(); i++) if(!used[i]) r0.push_back(v0[i]);
    for(size_t j = 0; j < v1.size(); j++) if(!done[j]) r1.push_back(v1[j]);
    v0.swap(r0); v1.swap(r1);
}
void mg_flush(void){ mg_run_dual(); mg_run_pairs(); mg_run(g_q[0]); mg_run(g_q[1]); mg_run(g_q[2]); }
