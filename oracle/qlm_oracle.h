/* qlm_oracle.h -- TEST INFRASTRUCTURE ONLY.
 *
 * CPU restatement of the reference's QLM 4-bit hot path, used as the checker by tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py. The shipped library must never
 * call into it. Every function names the reference lines it restates (paths are relative to the
 * reference tree). Built with -O3 -ffp-contract=off: FMA contraction changes the integer
 * optimizer bytes, so it is forbidden on both sides of every bit-exact comparison.
 *
 * Parity status of each function is listed at the top of qlm_oracle.c.
 */
#ifndef QLM_ORACLE_H
#define QLM_ORACLE_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

/* One quantized span = one whole weight tensor (qlm.cuh:30-38, same field order and sizes). */
typedef struct {
    unsigned long long pof;   /* element offset of the span in the rendered fp32 view P */
    unsigned long long gof;   /* element offset of its gradient in G                     */
    unsigned long long qi0;   /* element offset in d / r / m8 / v8                       */
    unsigned long long n;     /* elements                                                */
    int   gi0, ngrp;          /* first scale-group index, number of groups               */
    float sref;               /* frozen mean scale (relative-LR mode)                    */
} orc_span;

/* ---- integer helpers: qlm.cuh:78-111 ---- */
uint32_t orc_qhashu(uint64_t x);
int      orc_qsri(float v, uint64_t i, uint64_t t);
int      orc_qclmp(int v, int lo, int hi);
int      orc_qd_get(const int8_t *d, uint64_t i, int packed);
void     orc_qd_set(int8_t *d, uint64_t i, int v, int packed);
uint64_t orc_qd_bytes(uint64_t nq, int packed);

/* ---- span table: qlm.cuh:448-455, 527-536 ---- */
int  orc_span_add(orc_span *tab, int nspan, uint64_t pof, uint64_t n, int group,
                  uint64_t *nq, uint64_t *ngrp);
void orc_span_sref(orc_span *tab, int nspan, const float *s);

/* ---- encode / render / Integer AdamW / servo: qlm.cuh:136-441 == cpu_kern.h:771-874 ---- */
void orc_encode(const float *P, int8_t *d, int8_t *r, float *s, const orc_span *sp, int nspan,
                int group, int dmax, int packed, int ngrp);
void orc_render(float *P, const int8_t *d, const float *s, const orc_span *sp, int nspan,
                int group, int packed, int gi_base, int ng);
/* P may be NULL (no fp32 view kept); v8/v8s may be NULL when adam==0; stat may be NULL. */
void orc_step(float *P, const float *G, int8_t *d, int8_t *r, const float *s, int8_t *m8, float *m8s,
              uint8_t *v8, float *v8s, const orc_span *sp, int nspan, int group, int dmax,
              float lr, float b1, float b2, float wd, float gscale, const float *gsp,
              float inv_bc1, float inv_sqrt_bc2, int lrmode, uint64_t t, int adam,
              long long *stat, int packed, int gi_base, int ng, int v4);
/* cpu_kern.h:620-648 / cudalm.cu:4472-4520: touched-group form over one span starting at element 0 */
void orc_step_touched(float *P, const float *Gc, int8_t *d, int8_t *r, const float *s, int8_t *m8, float *m8s,
                      uint8_t *v8, float *v8s, const int *touched_gi, int ntouched, int group, int dmax,
                      float lr, float b1, float b2, float wd, float sref, float inv_bc1, float inv_sqrt_bc2,
                      uint64_t t, uint64_t nt, const float *gs, int v4);
/* cpu_kern.h:533-546: 64 chunk sums of squares (double accumulation, one rounding to float), and the clip
 * multiplier / norm pair derived from them */
void orc_sqsum(const float *G, uint64_t n, float *part64);
void orc_gnorm(const float *part, int nside, int clip_side, float *gs);

void orc_servo(int8_t *d, int8_t *r, float *s, const orc_span *sp, int nspan, int group, int dmax,
               float f_hi, float f_lo, int packed, int ngrp);

/* ---- expert GEMMs on the rendered fp32 view, row-major: cudalm.cu:3133-3256 over
 *      cpu_rt.h:178-352 ----
 *   nn: C[M,N]  = A[M,K] @ B[K,N]
 *   tn: C[M,N]  = A[M,K] @ B[N,K]^T + beta*C
 *   nt: C[K,N] += A[M,K]^T @ B[M,N]                                              */
void orc_gemm_nn(const float *A, const float *B, float *C, int M, int K, int N);
void orc_gemm_tn(const float *A, const float *B, float *C, int M, int K, int N, float beta);
void orc_gemm_nt(const float *A, const float *B, float *C, int M, int K, int N);
/* double-precision triple loops (cudalm.cu:9930-9945 style) used to pin the fp32 ones */
void orc_gemm_nn_f64(const float *A, const float *B, double *C, int M, int K, int N);
void orc_gemm_tn_f64(const float *A, const float *B, double *C, int M, int K, int N);
void orc_gemm_nt_f64(const float *A, const float *B, double *C, int M, int K, int N);
double orc_relerr(const float *a, const float *b, size_t n);
double orc_relerr_f64(const float *a, const double *b, size_t n);

/* ---- MoE glue: cpu_kern.h:29-35, 376-482; cudalm.cu:3586-3599 ---- */
float orc_fexp(float x);
void orc_router_topk(const float *rt, float *rprobs, int *assign, float *gate, int N, int E, int K,
                     const float *bias, int bs);
/* stable counting sort of one pass; returns -1-e if an assignment e is out of range */
int  orc_moe_perm(const int *assign, int N, int E, int *perm, int *off);
void orc_gather(const float *src, const int *perm, float *Xp, int N, int D);
void orc_scatter_gate(const float *yp, const int *perm, const float *gate, float *out, int N, int D);
void orc_scatter_add(const float *dXp, const int *perm, float *dst, int N, int D);
void orc_moe_dgate(const float *dout, const float *yp, const int *perm, const float *gate,
                   float *d_gate, float *dyp, int N, int D);
void orc_swiglu(const float *G, const float *U, float *O, size_t n);
void orc_swiglu_bwd(const float *Gg, const float *U, const float *dact, float *dg, float *du, size_t n);

/* ---- one top-K MoE expert FFN layer on the rendered view: call order of
 *      cudalm.cu:4193-4228 (forward) and 4299-4371 (backward, stash off) ----
 * w1,w3: [E][D][F]; w2: [E][F][D]; assign/gate pass-major [K][N].
 * out[N,D] is accumulated into (the caller seeds it with the residual or zero). */
typedef struct {
    int N, D, F, E, K;
    int *perm;      /* [K][N]      */
    int *off;       /* [K][E+1]    */
    float *Xp, *gp, *up, *ap, *yp;           /* per-pass scratch, N rows      */
    float *dyp, *dap, *dgp, *dup, *dXp;      /* backward scratch              */
    int bf16_inter;  /* 1: the GEMM inputs Xp, ap, dyp, dgp, dup are stored rounded to bf16, as the reference's
                      * GPU path stores them (hbf buffers of bfm_ffn / bfm_bwd, cudalm.cu:4001-4008, 4061-4087);
                      * everything else stays fp32. 0 (default): the CPU build's all-fp32 layer. */
} orc_moe_ws;
void orc_moe_ws_bf16(orc_moe_ws *w, int on);
orc_moe_ws *orc_moe_ws_new(int N, int D, int F, int E, int K);
void orc_moe_ws_free(orc_moe_ws *w);
int  orc_moe_forward(orc_moe_ws *w, const float *x, const float *w1, const float *w3, const float *w2,
                     const int *assign, const float *gate, float *out);
/* Needs a forward on the same ws first (perm/off). dgate [K][N]; dx zeroed here; G* accumulated. */
void orc_moe_backward(orc_moe_ws *w, const float *x, const float *w1, const float *w3, const float *w2,
                      const float *gate, const float *dout, float *dx, float *dgate,
                      float *Gw1, float *Gw3, float *Gw2);

/* ---- q4n wire format (cudalm.cu:638-656 writer, 688-696 reader): per group one fp32 scale and
 *      ceil(g/2) nibble bytes (same nibble rule as the packed digits); a group whose values are not
 *      s * integers in [-7,7] for any candidate scale is written as NaN + raw fp32. Returns the
 *      number of bytes (written only if <= cap); *nraw counts the raw groups. ---- */
size_t orc_q4n_quantize(const float *P, size_t n, int group, unsigned char *out, size_t cap, size_t *nraw);
int    orc_q4n_dequantize(const unsigned char *buf, size_t len, float *P, size_t n, int group);

/* ---- check of an identity the GPU step kernel relies on (not part of the reference): for b in
 *      [2^-60, 2^60] and |a| <= 2^9 b, with y = 1/b, q = a*y, r = fma(-q,b,a): fma(r,y,q) == a/b bit for
 *      bit. Returns the number of mismatches over n pseudo-random pairs drawn from `seed`. ---- */
size_t orc_recip_div_mismatches(uint64_t seed, size_t n);

/* ---- deterministic synthetic inputs: splitmix64 keyed by (seed, tensor id), top 24 bits as a
 *      uniform, Irwin-Hall sum of 12 uniforms minus 6 as a normal. Integer and exactly-rounded
 *      fp32 operations only, so every machine produces the same bits. ---- */
uint64_t orc_splitmix64(uint64_t x);
void orc_fill_normal(float *dst, size_t n, uint64_t seed, uint64_t tensor_id, float scale);
void orc_fill_uniform(float *dst, size_t n, uint64_t seed, uint64_t tensor_id, float lo, float hi);
void orc_fill_int8(int8_t *dst, size_t n, uint64_t seed, uint64_t tensor_id, int lo, int hi);
void orc_fill_u8(uint8_t *dst, size_t n, uint64_t seed, uint64_t tensor_id, int lo, int hi);
/* packed digits uniform in [-dmax,dmax] */
void orc_fill_digits(int8_t *d, size_t nq, uint64_t seed, uint64_t tensor_id, int dmax, int packed);
float orc_bf16_round(float x);           /* RNE to bf16, returned as fp32 (cudalm.cu:334-338) */
void  orc_bf16_round_n(float *x, size_t n);

void orc_set_threads(int n);
int  orc_get_threads(void);

#ifdef __cplusplus
}
#endif
#endif
