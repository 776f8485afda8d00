/* qlm_host.h -- C++ host mirror of the reference's QLM call surface on top of the C ABI (include/qlmx.h).
 *
 * Same names, argument order and error behaviour as the reference's host code so that cudalm.cu's
 * call sites keep compiling against it: the Qlm / QSpanD types (qlm.cuh:30-58), qlm_add_span,
 * qlm_gpu_init, qlm_gpu_render, qlm_render_layer, qlm_step_launch, qlm_gpu_update, qlm_fused_layer /
 * qlm_fused_tail, qlm_save / qlm_load (qlm.cuh:448-541, 577-591, 377-397, 702-788; cudalm.cu:6082-6103,
 * 6110-6187) and the grouped expert
 * GEMM queue mg_ab / mg_abt / mg_abt_b / mg_atb / mg_flush (cudalm.cu:3204-3256). Failures print
 * and exit(1) like ck()/ckb() (cudalm.cu:147-152).
 *
 * What differs, because the weights are never rendered for the GEMMs:
 *   - qlm_gpu_init takes the span list explicitly (the reference derives it from its Cfg/Off model
 *     description, qlm.cuh:479-490, which is outside this path);
 *   - the GEMM wrappers take the weight operand as a pointer INTO the fp32 view `P`, exactly as the
 *     reference call sites pass it (P + offset), but only its offset is used: mg_bind() registers
 *     the Qlm and the base of P, and the offset is mapped through the span table to digits + scales.
 *     P itself may be unallocated (P rendering is optional, see qlm_gpu_update);
 *   - the float spans' bf16 AdamW (k_adamw, cudalm.cu:6092-6096) is not part of this path; the
 *     table of float gaps is still built so a caller can run its own update over them.
 */
#ifndef QLM_HOST_H
#define QLM_HOST_H
#include <stddef.h>
#include <stdint.h>
#include "../../include/qlmx.h"

#define QLM_MAXSPAN 4096
typedef qlmx_span QSpanD;
typedef unsigned short bf16;

typedef struct {
    int on, adam, dmax, group, lrmode, servo_every, packed, v4;
    float fstar, f_hi, f_lo;
    int nspan;
    QSpanD *spanH, *spanD;
    unsigned long long nq, ngrp, np;
    signed char *d, *r, *m8;
    unsigned char *v8;
    float *s, *m8s, *v8s;
    unsigned long long fs_off[QLM_MAXSPAN], fs_n[QLM_MAXSPAN], fs_cs[QLM_MAXSPAN];
    int nfs; unsigned long long nfloat;
    bf16 *Mc, *Vc;                       /* owned by the caller's float-span optimizer; may be NULL */
    long long *statD; long long statH[4];
    int render_p;                        /* 1: the step keeps the fp32 view P up to date (reference behaviour) */
} Qlm;

typedef struct { unsigned long long pof, n; } QlmSpanDesc;

void *dmalloc(size_t bytes);                                            /* cudalm.cu:153 */
void  qlm_add_span(Qlm *q, unsigned long long pof, unsigned long long n);          /* qlm.cuh:448 */
void  qlm_gpu_init(Qlm *q, const QlmSpanDesc *spans, int nspan, float *P, size_t np); /* qlm.cuh:458 */
void  qlm_gpu_render(Qlm *q, float *P);                                 /* qlm.cuh:577 */
void  qlm_render_spans(Qlm *q, float *P, int span0, int nspans);        /* qlm.cuh:586 (one layer = 7 spans) */
void  qlm_step_launch(float *P, const float *G, signed char *d, signed char *r, float *s,
                      signed char *m8, float *m8s, unsigned char *v8, float *v8s,
                      const QSpanD *sp, int nspan, int group, int dmax,
                      float lr, float b1, float b2, float wd, float gscale, const float *gsp,
                      float inv_bc1, float inv_sqrt_bc2, int lrmode,
                      unsigned long long t, int adam, long long *stat, int packed,
                      int gi_base, int ng);                             /* qlm.cuh:377 */
void  qlm_gpu_update(Qlm *q, float *P, float *G, float lr, float b1, float b2, float wd,
                     float bc1, float bc2, int t, const float *gs);     /* cudalm.cu:6082 */
/* Fused per-layer update (cudalm.cu:6110-6135): step exactly spans [span0, span0+nspans) -- a layer is the 7
 * spans 7l..7l+6 (qlm.cuh:479-489) -- while their gradients are live, clipped by the PREVIOUS step's norm
 * (gscale = 1/prev_gn above 1), and leave the 64 partial sums of squares of G[g0 .. g0+gn) in part64.
 * qlm_fused_tail (cudalm.cu:6176-6186) closes the step: the norm over L slices of 64 layer partials plus
 * `nextra` further slices (embedding, final norm, ... summed by the caller with qlmx_sqsum), added up on
 * the host in double; it clips the next step. The float spans' AdamW in both reference functions is the
 * caller's. */
void  qlm_fused_spans(Qlm *q, float *P, float *G, int span0, int nspans, size_t g0, size_t gn, float *part64,
                      float lr, float wd, int t, float prev_gn);
void  qlm_fused_layer(Qlm *q, float *P, float *G, size_t layer_g0, size_t layer_gn, float *gnpart, int l,
                      float lr, float wd, int t, float prev_gn);
float qlm_fused_tail(const float *gnpart, int L, const float *extra, int nextra);
double qlm_persist_bytes(const Qlm *q);                                 /* qlm.cuh:678 */
int   qlm_save(const Qlm *q, const char *path, int iter, float prev_gn); /* qlm.cuh:702 */
int   qlm_load(Qlm *q, const char *path, int *iter, float *prev_gn);    /* qlm.cuh:740 */
void  qlm_free(Qlm *q);

/* The .opt.q file format over HOST memory (plain C, no device needed): what qlm_save / qlm_load write and
 * read, for tools and for byte-level checks against files written by the reference. All pointers are host
 * arrays of the sizes the header fields imply (Mc, Vc: nfloat bf16, may be NULL = zeros / skipped;
 * v8, v8s only when adam; sref: nspan floats). read fills the arrays, iter, prev_gn (left alone when the
 * file has no valid one) and have_sref; both return 1 on success, 0 otherwise. */
typedef struct {
    int dmax, group, adam, nspan, packed, iter;
    unsigned long long nq, ngrp, nfloat;
    bf16 *Mc, *Vc;
    signed char *d, *r, *m8;
    unsigned char *v8;
    float *s, *m8s, *v8s;
    float *sref;
    float prev_gn;
    int have_sref;
} QlmOptqHost;
#ifdef __cplusplus
extern "C" {
#endif
int qlm_optq_write_host(const char *path, const QlmOptqHost *v);
int qlm_optq_read_host(const char *path, QlmOptqHost *v);
#ifdef __cplusplus
}
#endif

/* grouped expert GEMMs: row-major, B points into the (possibly virtual) fp32 view P */
void mg_bind(const Qlm *q, const float *Pbase, int act_dtype, int math);
void mg_ab(const void *A, const float *B, float *C, int M, int K, int N);                /* cudalm.cu:3247 */
void mg_abt_b(const void *A, const float *B, float *C, int M, int K, int N, float beta); /* cudalm.cu:3250 */
void mg_abt(const void *A, const float *B, float *C, int M, int K, int N);               /* cudalm.cu:3253 */
void mg_atb(const void *A, const void *B, float *C, int M, int K, int N);                /* cudalm.cu:3254 */
/* mg_ab on w1 and w3 of one expert followed by the reference's e_swig (cudalm.cu:4211-4215) as one queued
 * item: gp = A.B1, up = A.B3 (fp32, kept for the backward pass), ap = bf16(SwiGLU(gp, up)) */
void mg_ab_swiglu(const void *A, const float *B1, const float *B3, float *gp, float *up, void *ap, int M, int K, int N);
void mg_flush(void);                                                                      /* cudalm.cu:3243 */

/* Label timing and fault localisation at the reference's check points (kchk, cudalm.cu:842-855; hooks e.g. at 4336,
 * 4366, 6089). Levels as the reference reads them from the environment (cudalm.cu:10764-10765): CUDALM_DEBUG != 0 or
 * CUDALM_PROF = 1, 2: wait for the device at every label, report a fault by label and layer and exit(1), charge the
 * wall time since the previous label to this one, warn when one label took more than a quarter of the watchdog
 * budget; CUDALM_PROF >= 3 (and no debug): no wait -- an event per label, GPU time between events, and a count of the
 * labels at which the GPU had already run dry. Neither set: kchk returns at once. prof_report prints the table
 * (cudalm.cu:826-840); kchk_slowest returns the label that took longest in the waiting modes. */
void kchk(const char *what, int l);
void prof_report(void);
const char *kchk_slowest(double *ms);
void kchk_levels(int debug, int prof, double tdr_seconds);        /* instead of the environment (tests, hosts with flags) */
#endif
