/* qlmx.h -- C ABI of libqlmx: cudalm's QLM 4-bit weight path on MI355X (gfx950).
 *
 * The reference (Dsg2/cudalm-c) is one translation unit with no FFI; its backend seam is the set of
 * call signatures cudalm.cu uses against qlm.cuh and against its own GEMM wrappers, swapped for the
 * CPU build by cpu_rt.h / cpu_kern.h. Every entry point below replaces one of those call sites and
 * cites it (paths relative to the reference tree). All device buffers are caller-owned; `stream`
 * is a hipStream_t passed as void* (NULL = the default stream, which is what the reference uses).
 * Launches are asynchronous and ordered by the stream.
 * ONE HOST THREAD, ONE STREAM AT A TIME (as the reference: one thread, the default stream, cudalm.cu:6628): the
 * library keeps process-wide state -- the table rings of the grouped GEMMs and their staging copies, the chain flags
 * of split contractions, the partial sums of qlmx_sqsum, the decode workspace -- so calls must come from one host
 * thread, and calls whose kernels could overlap on different streams are not supported, except the documented
 * pairing of qlmx_side_fork / qlmx_side_join (qlmx_pair_begin / qlmx_pair_end runs the two on one stream).
 * Every function returns 0 on success and a
 * negative QLMX_E_* code on failure; qlmx_last_error() holds the message of the calling thread's
 * last failure. The reference's print-and-exit(1) behaviour (ck/ckb, cudalm.cu:147-152) is kept by
 * the C++ mirror in cudalm-c_amd/host/, not here.
 *
 * Plain C: pointers and sizes only, no C++ or framework types.
 */
#ifndef QLMX_H
#define QLMX_H
#include <stddef.h>
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

#define QLMX_VERSION 1

#define QLMX_OK            0
#define QLMX_E_ARG        -1   /* bad argument (shape, alignment, NULL, unsupported combination) */
#define QLMX_E_HIP        -2   /* a HIP runtime call failed                                     */
#define QLMX_E_NODEV      -3   /* no gfx950 device / library not initialised                    */
#define QLMX_E_LIMIT      -4   /* a documented size limit was exceeded                          */

/* One quantized span = one whole weight tensor. Same layout as QSpanD (qlm.cuh:30-38), 48 bytes. */
typedef struct qlmx_span {
    unsigned long long pof;   /* element offset in the rendered fp32 view P            */
    unsigned long long gof;   /* element offset of the gradient in G                   */
    unsigned long long qi0;   /* element offset in d / r / m8 / v8 (even when packed)  */
    unsigned long long n;     /* elements                                              */
    int   gi0, ngrp;          /* first scale group, number of groups                   */
    float sref;               /* frozen mean scale for the relative-LR mode            */
} qlmx_span;

/* ---- runtime: replaces cudaSetDevice / dmalloc / cudaMemcpy / cudaMemset /
 *      cudaDeviceSynchronize as used by cudalm.cu:147-154, 6628 and qlm.cuh:505-521 ---- */
int         qlmx_version(void);
int         qlmx_init(int device);
const char *qlmx_last_error(void);
const char *qlmx_device_name(void);
int         qlmx_malloc(void **p, size_t bytes);
int         qlmx_free(void *p);
int         qlmx_memcpy_h2d(void *dst, const void *src, size_t bytes);
int         qlmx_memcpy_d2h(void *dst, const void *src, size_t bytes);
int         qlmx_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream);
int         qlmx_memset(void *dst, int value, size_t bytes, void *stream);
int         qlmx_sync(void *stream);
/* A second stream beside the caller's (no counterpart in the reference, which issues the grouped GEMMs of a
 * flush one after the other on one stream, cudalm.cu:3243-3256). The weight gradient and the input gradient of a
 * backward flush read the same operands and write different outputs; at config 3 neither fills the device to
 * the end of its last round of tiles, and side by side they take 4 % less than one after the other.
 * qlmx_side_fork(stream, &side): `side` (owned by the library, one per device) continues after everything queued
 * on `stream` so far; pass it as the `stream` argument of the independent calls. qlmx_side_join(stream): `stream`
 * continues after everything queued on the side stream. Neither blocks the host. Not for use under stream
 * capture. */
int         qlmx_side_fork(void *stream, void **side);
int         qlmx_side_join(void *stream);
/* The two grouped GEMMs of a backward flush as ONE kernel launch (no counterpart in the reference, which issues
 * them one after the other, cudalm.cu:3243-3256). Between qlmx_pair_begin(stream) and qlmx_pair_end(stream) the
 * library holds back at most one input-gradient launch (qlmx_moe_gemm_tn, _tn_pair, _tn_pair_scatter,
 * _tn_swiglu_bwd) and one weight-gradient launch (qlmx_moe_gemm_nt), both on bf16 operands with MFMA math and
 * queued on `stream`, and qlmx_pair_end issues them as one grid: the workgroups of the one kernel first, those of
 * the other behind them, each tile computed exactly as in its own launch (bit-identical results), so the second
 * kind's tiles take the compute units as the first kind's last round leaves them -- without the wait between
 * hardware queues that the side stream costs at its fork and join. The caller promises what it promises for the
 * side stream: neither of the two reads what the other writes. Everything else keeps its order on the stream:
 * a second launch of a kind already held, a launch of a shape the two direct-to-LDS kernels do not take, and any
 * other library call that queues work first issue what is held. One pair at a time; not for use across host
 * synchronisation (nothing held runs before qlmx_pair_end or one of the calls just named). */
int         qlmx_pair_begin(void *stream);
int         qlmx_pair_end(void *stream);
/* Label timing without synchronisation: prof_ev / prof_flush / prof_report behind kchk, cudalm.cu:806-840.
 * qlmx_prof_mark(label, stream) records an event on `stream` and charges the GPU time since the previous mark to
 * `label` (marks stand BEHIND the work they name, as the reference places kchk); a mark that finds the previous
 * mark's event already complete counts as `drained`: the GPU had no queued work left and the host was the bottleneck
 * there. Up to 48 labels (the rest share the last entry); events are drained every 1024 marks and by the report.
 * qlmx_prof_report writes the table (largest total first: name, ms, share, count, drained) into out[cap] and the number
 * of labels into *nlabels (may be NULL); qlmx_prof_reset forgets everything. The waiting modes of kchk (fault
 * localisation, wall time per label) live in the host mirror (cudalm-c_amd/host/qlm_host.h: kchk, prof_report). */
int         qlmx_prof_mark(const char *label, void *stream);
int         qlmx_prof_report(char *out, size_t cap, int *nlabels);
int         qlmx_prof_reset(void);

/* ---- host integer helpers: the __host__ __device__ inlines of qlm.cuh:78-111, used by the
 *      reference's checkpoint code and selftest reference (cudalm.cu:10574-10580) ---- */
unsigned int       qlmx_qhashu(unsigned long long x);                              /* qlm.cuh:78  */
int                qlmx_qsri(float v, unsigned long long i, unsigned long long t);  /* qlm.cuh:83  */
int                qlmx_qclmp(int v, int lo, int hi);                               /* qlm.cuh:88  */
int                qlmx_qd_get(const signed char *d, unsigned long long i, int packed);          /* :96  */
void               qlmx_qd_set_host(signed char *d, unsigned long long i, int v, int packed);    /* :102 */
unsigned long long qlmx_qd_bytes(unsigned long long nq, int packed);                              /* :109 */

/* ---- k_qlm_encode (qlm.cuh:136-167; launch at qlm.cuh:524): P -> digits, residual, scales.
 * `sp` is the DEVICE copy of the span table, ngrp the total number of groups. group in [2,256] and
 * even when packed; dmax <= 7 when packed. ---- */
int qlmx_encode(const float *P, signed char *d, signed char *r, float *s,
                const qlmx_span *sp, int nspan, int group, int dmax, int packed, int ngrp,
                void *stream);

/* ---- k_qlm_render (qlm.cuh:170-178; launches at 538, 578, 589): P = s * digit for groups
 * gi_base .. gi_base+ng-1. ---- */
int qlmx_render(float *P, const signed char *d, const float *s,
                const qlmx_span *sp, int nspan, int group, int packed, int gi_base, int ng,
                void *stream);

/* ---- qlm_step_launch (qlm.cuh:377-397; called from cudalm.cu:6086, 6126, 10601, 10617):
 * Integer AdamW (adam=1) or integer Lion (adam=0) over groups gi_base .. gi_base+ng-1, then the
 * moments are re-quantized with fresh per-group scales. Argument order and meaning are the
 * reference's. gsp, when not NULL, is a device pointer to the gradient clip multiplier and
 * overrides gscale (no host round trip). stat, when not NULL, is a device long long[4]
 * {sum |carry|, railed digits, zero digits, max |LSB step|} that is accumulated into.
 * Differences from the reference, both additive: P may be NULL (the fp32 view is not kept when the
 * GEMMs read the digits directly); v4 carries the QLM_V4 switch (qlm.cuh:62-67) that the reference
 * keeps in a device global. ---- */
int qlmx_step(float *P, const float *G, signed char *d, signed char *r, const float *s,
              signed char *m8, float *m8s, unsigned char *v8, float *v8s,
              const qlmx_span *sp, int nspan, int group, int dmax,
              float lr, float b1, float b2, float wd, float gscale, const float *gsp,
              float inv_bc1, float inv_sqrt_bc2, int lrmode,
              unsigned long long t, int adam, long long *stat, int packed,
              int gi_base, int ng, int v4, void *stream);

/* ---- k_ng_q4_step (cudalm.cu:4472-4520; cpu_kern.h:620-648), called from the n-gram table update
 * (cudalm.cu:4752): the Integer AdamW step over a LIST of touched groups of one packed span that
 * starts at element 0 of d/r/m8/v8/P and has `nt` elements. Group w of the list is touched_gi[w] and
 * its gradient is the compact row Gc[w*group .. +group). Relative LR through the frozen `sref`,
 * gscale = *gs (1 when NULL), no statistics; otherwise the arithmetic of qlmx_step, bit for bit.
 * A group may be listed at most once. ---- */
int qlmx_step_touched(float *P, const float *Gc, signed char *d, signed char *r, const float *s,
                      signed char *m8, float *m8s, unsigned char *v8, float *v8s,
                      const int *touched_gi, int ntouched, int group, int dmax,
                      float lr, float b1, float b2, float wd, float sref,
                      float inv_bc1, float inv_sqrt_bc2, unsigned long long t, unsigned long long nt,
                      const float *gs, int v4, void *stream);

/* ---- gradient-norm clipping around the step: k_sqsum and k_gnorm (cudalm.cu:2794-2816; CPU twins
 * cpu_kern.h:533-546), called from qlm_fused_layer / qlm_fused_tail (cudalm.cu:6122, 6181) and the
 * unfused update (6435-6444). qlmx_sqsum writes 64 partial sums of squares, partial c over
 * G[n*c/64 .. n*(c+1)/64), accumulated in double and rounded to float once (the CPU path's
 * definition). qlmx_gnorm reduces them (plus `nside` further slices of 64) on the device to
 * gs[0] = clip multiplier (1 when the norm is <= 1) and gs[1] = the norm, which qlmx_step reads
 * through its `gsp` argument. ---- */
int qlmx_sqsum(const float *G, unsigned long long n, float *part64, void *stream);
int qlmx_gnorm(const float *part, int nside, int clip_side, float *gs, void *stream);


/* ---- k_qlm_servo (qlm.cuh:404-441; launched from cudalm.cu:6099): rail-fraction scale servo
 * and re-encode of (d, r) for the groups whose scale moved. ---- */
int qlmx_servo(signed char *d, signed char *r, float *s,
               const qlmx_span *sp, int nspan, int group, int dmax,
               float f_hi, float f_lo, int packed, int ngrp, void *stream);

/* =====================================================================================
 * Expert GEMMs with the dequantisation fused in
 *
 * The reference renders P = s*digit once per step and hands fp32 slices of P to its GEMM wrappers
 * (row-major):  mg_ab   C[M,N]  = A[M,K] @ B[K,N]             cudalm.cu:3247-3249 (g_ab 3133)
 *               mg_abt_b C[M,N] = A[M,K] @ B[N,K]^T + beta*C   cudalm.cu:3250-3253 (g_abt_b 3174)
 *               mg_atb  C[K,N] += A[M,K]^T @ B[M,N]            cudalm.cu:3254-3256 (g_atb 3190)
 * queued per expert and issued together by mg_flush (cudalm.cu:3230-3243). Here the weight operand
 * is named by its position in the packed digits and scales instead of by a pointer into P, and one
 * call takes the whole queue: an array of problems that share K and N. Results equal the
 * reference's P = s*digit -> fp32 SGEMM semantics to rounding (fp32 math) or to bf16-MFMA
 * accumulation order (MFMA math); C is always fp32.
 * ===================================================================================== */
#define QLMX_ACT_F32   0     /* activation operands are fp32                         */
#define QLMX_ACT_BF16  1     /* activation operands are bf16 (high half of an fp32)  */
#define QLMX_MATH_F32  0     /* fp32 FMA on the vector ALU                           */
#define QLMX_MATH_MFMA 1     /* bf16 MFMA, fp32 accumulate                           */
#define QLMX_MATH_MFMA_F16 2 /* as QLMX_MATH_MFMA, except that qlmx_moe_gemm_nn on bf16 activations runs on the fp16
                              * matrix core: the activations are converted exactly (|x| in [2^-14, 65504]; smaller ones
                              * with an absolute error below 3e-8), every weight s*digit is rounded once to fp16
                              * (11 significant bits, full precision for 2.4e-7 <= |w| <= 255) and a product costs one
                              * MFMA instead of the two of the bf16 hi + lo split. Relative L2 error against the fp32
                              * result about 2e-4 (QLMX_MATH_MFMA: 3e-6), inside the 1e-3 bar for matmul outputs. */
#define QLMX_MAX_PROBLEMS 1024   /* like MG_MAXP, cudalm.cu:3214 */

typedef struct qlmx_gemm_prob {
    const void *A;           /* device: nn/tn [M,K]; nt [M,K] (read transposed)                  */
    const void *B;           /* device: nt: [M,N] activation/gradient rows; the second list of
                              * qlmx_moe_gemm_nn_swiglu: the bf16 output; else NULL              */
    float      *C;           /* device: nn/tn [M,N]; nt [K,N]                                    */
    unsigned long long wq;   /* nn/tn: element offset of the weight matrix in the digit array    */
    unsigned long long wg;   /* nn/tn: index of the matrix's first scale group                   */
    int   M;                 /* rows of A (0 is allowed and skipped)                             */
    float beta;              /* tn, nt: 0 (overwrite C) or 1 (accumulate, the reference's mg_atb and
                              * the second mg_abt_b of a pair). nn always overwrites.              */
} qlmx_gemm_prob;

/* nn: weights [K,N] row-major, scale groups run along N (N % group == 0). */
int qlmx_moe_gemm_nn(const signed char *d, const float *s, int group,
                     const qlmx_gemm_prob *probs_host, int nprob, int K, int N,
                     int act_dtype, int math, void *stream);
/* tn: weights [N,K] row-major, scale groups run along K (K % group == 0). */
int qlmx_moe_gemm_tn(const signed char *d, const float *s, int group,
                     const qlmx_gemm_prob *probs_host, int nprob, int K, int N,
                     int act_dtype, int math, void *stream);
/* The two mg_abt_b calls on one output (cudalm.cu:4365-4366: dXp = dgp . w1^T with beta 0, then
 * dXp += dup . w3^T with beta 1) as one call: problem i computes
 *   C = first[i].A . W(first[i].wq)^T + second[i].A . W(second[i].wq)^T   (+ C when first[i].beta = 1).
 * second[i] supplies A, wq, wg and must repeat M; its B, C and beta are ignored. On bf16 activations
 * with QLMX_MATH_MFMA both contractions run in one launch and the sum stays in the accumulators;
 * every other combination issues the two launches the reference would. At most QLMX_MAX_PROBLEMS / 2
 * problems. */
int qlmx_moe_gemm_tn_pair(const signed char *d, const float *s, int group,
                          const qlmx_gemm_prob *first_host, const qlmx_gemm_prob *second_host, int nprob,
                          int K, int N, int act_dtype, int math, void *stream);
/* The gate and up GEMMs of moe_forward and the SwiGLU that follows them (cudalm.cu:4211-4215: mg_ab(Xp, w1_e,
 * gp), mg_ab(Xp, w3_e, up), mg_flush, e_swig(gp, up, ap)) as one call: problem i computes
 *   gp = A . W(gate[i].wq),  up = A . W(up[i].wq),  ap = bf16(gp * sigmoid(gp) * up)   (k_swiglu, cudalm.cu:2430)
 * with A = gate[i].A [M, K]; gp goes to gate[i].C and up to up[i].C (fp32 [M, N], kept for the backward pass),
 * ap to up[i].B (bf16 [M, N], the down GEMM's input). up[i] must repeat M; its A and beta are ignored.
 * On bf16 activations with QLMX_MATH_MFMA (N % 64 == 0, K % 32 == 0, group a power of two >= 64, at most
 * QLMX_MAX_PROBLEMS / 2 problems) an output tile holds 64 columns of both matrices and the SwiGLU is applied
 * to the accumulators (gp and up bit-identical to the two GEMM calls; ap computed with the polynomial sigmoid of
 * qlmx_swiglu on QLMX_MATH_MFMA); every other combination runs the two GEMM launches and a SwiGLU launch per problem. */
int qlmx_moe_gemm_nn_swiglu(const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *gate_host, const qlmx_gemm_prob *up_host, int nprob,
                            int K, int N, int act_dtype, int math, void *stream);
/* The row moves of the MoE layer folded into the expert GEMMs, so that the permuted copies never exist in memory
 * (cudalm.cu:4209-4213 gather + mg_ab; 4224-4227 mg_ab + k_scatter_gate; 4365-4367 paired mg_abt_b + k_scatter_add4).
 * bf16 activations, matrix-core math (fp16 forward as QLMX_MATH_MFMA_F16, bf16 input gradient as QLMX_MATH_MFMA),
 * N % 128 == 0, K % 32 == 0 (64 for the input gradient), group a power of two >= that. An index list is int32 in
 * device memory, entry r of problem i naming a token row; an entry < 0 reads as zeros (gather) or is dropped
 * (scatter). Moves are exact: results equal the separate gather / GEMM / scatter kernels bit for bit.
 *   gather:  probs[i].A = index list; C[r, :] = x[idx[r], :] . W                     x: bf16 [tokens, K]
 *   scatter: probs[i].C = index list; out[idx[r], :] = out[idx[r], :] + gate[idx[r]] * (A . W)[r, :]   (gate NULL: + (A . W)[r, :])
 *   tn_pair_scatter: first[i].C = index list; dst[idx[r], :] += (first.A . W1^T + second.A . W3^T)[r, :]
 * A scatter call must not name an output row twice (one pass of the layer never does); calls on one stream are
 * ordered, so the passes of a layer add up in pass order as in the reference. */
int qlmx_moe_gemm_nn_gather(const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *probs_host, int nprob, int K, int N, const void *x_bf16, void *stream);
int qlmx_moe_gemm_nn_scatter(const signed char *d, const float *s, int group,
                             const qlmx_gemm_prob *probs_host, int nprob, int K, int N,
                             float *out, const float *gate, void *stream);
int qlmx_moe_gemm_tn_pair_scatter(const signed char *d, const float *s, int group,
                                  const qlmx_gemm_prob *first_host, const qlmx_gemm_prob *second_host, int nprob, int K, int N,
                                  float *dst, void *stream);
/* The SwiGLU and its gradient folded into the GEMMs next to them (fp16 forward kernel, bf16 input-gradient kernel).
 * The fp32 gate and up outputs equal the separate GEMM calls bit for bit. The epilogues take the sigmoid from the
 * transcendental unit (v_exp_f32, v_rcp_f32) where qlmx_swiglu / qlmx_swiglu_bwd use the CPU build's polynomial
 * (cpu_kern.h:376-394): the two agree to 3e-7 relative, so the bf16 outputs (activation, dgp, dup) equal the
 * separate calls except where that difference crosses a bf16 rounding boundary -- one bf16 unit in the last place on
 * fewer than 1 element in 10,000 (the bound the tests hold):
 *   qlmx_moe_gemm_nn_swiglu with QLMX_MATH_MFMA_F16: as documented above on the fp16 matrix core; gate[i].C and
 *     up[i].C may then both be NULL, and only the bf16 SwiGLU output up[i].B is written (a forward pass that does
 *     not keep gp / up for the backward: cudalm.cu:4211-4215 with the stash off).
 *   qlmx_moe_gemm_nn_gather_swiglu: the same with the gather in front (cudalm.cu:4209-4215): gate[i].A are
 *     row-index lists into the bf16 token matrix x, as in qlmx_moe_gemm_nn_gather. N % 64 == 0, K % 32 == 0,
 *     group 64, 128 or 256, at most QLMX_MAX_PROBLEMS / 2 problems.
 *   qlmx_moe_gemm_tn_swiglu_bwd: mg_abt of the down projection + e_swigb (cudalm.cu:4340-4346): the product
 *     d(act) = A . W^T is not stored; probs[i].C points at the problem's rows INSIDE gp (the forward's fp32 gate
 *     pre-activations), and with o = probs[i].C - gp the kernel reads gp[o ..], up[o ..] and writes the bf16
 *     gradients dgp[o ..], dup[o ..] ([rows, N] each, the four buffers laid out alike). */
int qlmx_moe_gemm_nn_gather_swiglu(const signed char *d, const float *s, int group,
                                   const qlmx_gemm_prob *gate_host, const qlmx_gemm_prob *up_host, int nprob, int K, int N,
                                   const void *x_bf16, void *stream);
int qlmx_moe_gemm_tn_swiglu_bwd(const signed char *d, const float *s, int group,
                                const qlmx_gemm_prob *probs_host, int nprob, int K, int N,
                                const float *gp, const float *up, void *dgp_bf16, void *dup_bf16, void *stream);
/* nt: no weight operand; both inputs are activations, fp32 result. beta = 1 reproduces the
 * reference's accumulation into a zeroed G; beta = 0 saves the read when G is known to be fresh. */
int qlmx_moe_gemm_nt(const qlmx_gemm_prob *probs_host, int nprob, int K, int N,
                     int act_dtype, int math, void *stream);

/* =====================================================================================
 * Decode-shaped expert FFN (a few tokens per step)
 *
 * The reference's decoder runs the training forward on N = batch rows (dec_step, cudalm.cu:7163-7204
 * -> moe_forward 7193), so each expert GEMM has 0..few rows and the work is reading the experts'
 * packed weights once. qlmx_moe_gemm_nn with QLMX_MATH_F32 already takes a streaming GEMV path when
 * every problem has at most 4 rows (the counterpart of the reference's R<=4 path, cpu_rt.h:233-258).
 * qlmx_moe_decode_forward fuses the whole expert part of moe_forward for such batches: it groups
 * the (pass, token) pairs by expert on the device (no host round trip, unlike cudalm.cu:3576-3602),
 * streams w1|w3 with the SwiGLU applied on the fly, streams w2, and adds gate*y into `out` in pass
 * order (cudalm.cu:4193-4228 semantics: out[n] += sum_k gate[k][n] * FFN_{assign[k][n]}(x[n])).
 *   x      [T, D] fp32                    assign [K][T] int32 (pass-major)   gate [K][T] fp32
 *   out    [T, D] fp32, accumulated into (the caller seeds it with the residual)
 *   w1q/w3q/w2q: element offsets of expert 0's matrices in d; expert e adds e*D*F. All multiples of
 *   `group`; w1, w3 are [D,F] row-major and w2 is [F,D] row-major (cudalm.cu:263-265). The scale of
 *   element q is s[q / group] (every span a multiple of the group, true of all reference presets).
 * Limits: K*T <= 64 pairs, D and F multiples of 32 and <= 8192 (QLMX_E_LIMIT for the few shapes in that range
 * whose task lists a workgroup cannot hold). Uses a library-owned workspace that
 * is (re)allocated on first use or growth; calls on different streams must not overlap. The tag that
 * orders the hand-over between workgroups lives in device memory and moves on by itself, so a call
 * may be recorded into a HIP graph and replayed (once the workspace has its size: a call that would
 * have to grow it during a capture fails with QLMX_E_ARG); a replay does not pass through the host,
 * so a wait that gave up is reported by the next direct call or by qlmx_decode_status(), which a loop of
 * replays should ask after each synchronised replay. The launch is a grid of co-resident workgroups that wait for
 * each other: it assumes that no other kernel occupies the device while it runs (with the CUs partly taken, late
 * workgroups make the others wait, and past the bound -- of the order of 0.1 s -- the launch gives up).
 * ===================================================================================== */
int qlmx_moe_decode_forward(const float *x, const int *assign, const float *gate, float *out,
                            const signed char *d, const float *s, int group,
                            unsigned long long w1q, unsigned long long w3q, unsigned long long w2q,
                            int T, int K, int E, int D, int F, void *stream);

/* Host-only, no GPU call: QLMX_OK, or QLMX_E_HIP (once) when a decode launch on the current device has given up a
 * bounded wait since the last report -- its `out` is invalid. No counterpart in the reference. */
int qlmx_decode_status(void);

/* qlmx_moe_decode_forward for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). No counterpart in the reference. Same arguments,
 * same kernel, bit-identical output; the partial sums live in a fixed device array of
 * QLMX_DECODE_SCRATCH_BYTES that is part of the library image (each GPU the library runs on holds it
 * until the process ends), and the call makes no hipMalloc, hipFree or other allocating call.
 * qlmx_init must have run for the current device. A shape whose partial sums
 *   8 * K*T * 2 * (2 * ceil(D/R1) * F + ceil(F/R2) * D)  bytes, R1, R2 = 64..256 rows per gate|up / down slice
 * exceed the array fails with QLMX_E_LIMIT (the 32-expert D=768 F=2048 layer at 16 tokens top-2
 * needs 10.6 MB). Every call on a GPU shares that GPU's array: calls that overlap on one GPU,
 * whatever their streams, race. */
#define QLMX_DECODE_SCRATCH_BYTES (32u << 20)
int qlmx_moe_decode_forward_noalloc(const float *x, const int *assign, const float *gate, float *out,
                                    const signed char *d, const float *s, int group,
                                    unsigned long long w1q, unsigned long long w3q, unsigned long long w2q,
                                    int T, int K, int E, int D, int F, void *stream);

/* =====================================================================================
 * MoE layer glue around the expert GEMMs (training shape). Indices and gate probabilities are
 * bit-exact against the reference's CPU build; float outputs follow its operation order.
 * `out_dtype` (QLMX_ACT_F32 / QLMX_ACT_BF16) selects the type of a buffer that feeds a GEMM next,
 * so the bf16 MFMA path needs no separate cast pass (bf16 = round to nearest even, cudalm.cu:334-338).
 * Row buffers must be 16-byte aligned and D a multiple of 4.
 * ===================================================================================== */

/* k_router_topk (cudalm.cu:2515-2534; cpu_kern.h:413-425): softmax over E per token with the CPU
 * build's polynomial exp (cpu_kern.h:29-34), then K greedy picks on prob + bias[k*bs + e] with a
 * strict >, lowest index winning ties. rt, rprobs [N,E]; assign, gate pass-major [K][N]; gate is the
 * raw softmax probability; bias may be NULL. K <= 8. */
int qlmx_router_topk(const float *rt, float *rprobs, int *assign, float *gate, int N, int E, int K,
                     const float *bias, int bs, void *stream);

/* k_gp_hist / k_gp_scan / k_gp_scatter (cudalm.cu:3504-3530), equal to the host permutation of
 * cudalm.cu:3586-3599: for each pass k a stable counting sort of the tokens by expert.
 * perm [K][N]: perm[k][j] = token in row j of pass k; off [K][E+1]: first row of each expert.
 * `workspace` = qlmx_moe_perm_workspace(N,E,K) bytes of device memory. Asynchronous; an expert index
 * out of range is reported by qlmx_moe_perm_status (the reference aborts, cudalm.cu:3476-3478). */
size_t qlmx_moe_perm_workspace(int N, int E, int K);
int qlmx_moe_perm(const int *assign, int N, int E, int K, int *perm, int *off, void *workspace, void *stream);
int qlmx_moe_perm_status(const void *workspace, int N, int E, int K, void *stream);

/* k_gather / k_gather4 (cudalm.cu:2536-2539, 2558-2563): Xp[j,:] = src[perm[j],:], zeros where perm[j] < 0 */
int qlmx_moe_gather(const float *src, const int *perm, void *Xp, int N, int D, int out_dtype, void *stream);
/* k_scatter_gate (cudalm.cu:2541-2545): out[perm[j],:] += gate[perm[j]] * yp[j,:] */
int qlmx_moe_scatter_gate(const float *yp, const int *perm, const float *gate, float *out, int N, int D, void *stream);
/* k_scatter_add4 (cudalm.cu:2564-2567; cpu_kern.h:445-450): dst[perm[j],:] += dXp[j,:] */
int qlmx_moe_scatter_add(const float *dXp, const int *perm, float *dst, int N, int D, void *stream);
/* k_moe_dgate (cudalm.cu:2591; cpu_kern.h:454-468): d_gate[n] = dout[n,:] . yp[j,:], dyp[j,:] = gate[n] * dout[n,:], n = perm[j] */
int qlmx_moe_dgate(const float *dout, const float *yp, const int *perm, const float *gate,
                   float *d_gate, void *dyp, int N, int D, int out_dtype, void *stream);
/* All K passes of a layer as ONE expert-grouped list of K*N rows (the reference's merged top-K: moe_gperm with
 * mrg, k_gather_bfm, k_combine_bf, k_moe_dgate_bfm; cudalm.cu:3532-3561, 4022-4047), so that every grouped GEMM
 * runs once per layer on K times the rows instead of once per pass. The grouping itself is qlmx_moe_perm over the
 * K*N assignments as a single pass (N' = K*N, K' = 1): its perm names entries m = pass * N + token.
 *   qlmx_moe_merge_rows: tok[p] = perm[p] % N (the token row p holds; what a gather or a gathering GEMM takes as
 *     its index list) and inv[m] = the row that holds entry m (-1 if none), both int32 [K*N].
 *   qlmx_moe_combine: out[n,:] = (..(out[n,:] + gate[0*N+n] * y[inv[0*N+n],:]) ..) + gate[(K-1)*N+n] * y[inv[(K-1)*N+n],:]
 *     -- the sums that K calls of qlmx_moe_scatter_gate build, in their order and to their bits; gate NULL adds
 *     the rows themselves (K calls of qlmx_moe_scatter_add). y fp32 [K*N, D].
 *   qlmx_moe_dgate_merged: qlmx_moe_dgate over the grouped list: row j holds entry m = perm[j], token n = m % N;
 *     d_gate[m] = dout[n,:] . yp[j,:], dyp[j,:] = gate[m] * dout[n,:]. */
int qlmx_moe_merge_rows(const int *perm, int N, int K, int *tok, int *inv, void *stream);
int qlmx_moe_combine(const float *y, const int *inv, const float *gate, float *out, int N, int K, int D, void *stream);
int qlmx_moe_dgate_merged(const float *dout, const float *yp, const int *perm, const float *gate,
                          float *d_gate, void *dyp, int N, int K, int D, int out_dtype, void *stream);
/* k_swiglu / k_swiglu_bwd (cudalm.cu:2430-2453; cpu_kern.h:376-394): O = g*sigmoid(g)*u and its
 * gradient (dg, du) from dact, with the CPU build's polynomial sigmoid. n % 4 == 0. */
int qlmx_swiglu(const float *G, const float *U, void *O, size_t n, int out_dtype, void *stream);
int qlmx_swiglu_bwd(const float *Gg, const float *U, const float *dact, void *dg, void *du, size_t n, int out_dtype, void *stream);

/* Test hook (no counterpart in the reference). The decode layer (which = 1) and the split contractions of
 * qlmx_moe_gemm_nt (which = 2) hand partial results from workgroup to workgroup through bounded waits. Arming the
 * hook makes the NEXT launch of that kind wait -- for one poll -- for a tag nobody publishes: every wait gives up
 * at once, every workgroup still runs to its end, the launch's output is invalid, and the following call of that
 * entry point returns QLMX_E_HIP once, exactly as after a real time-out. One-shot; the call after that is normal. */
int qlmx_test_force_wait_timeout(int which);
/* Tuning and test hook (no counterpart in the reference). qlmx_moe_gemm_nt on bf16 operands computes 256 x 128 output
 * tiles; a 256 x 256 variant (one workgroup of eight wavefronts per CU) exists and
 * is correct but not faster on MI355X, so it is never chosen by itself. tile = 256 selects it for later calls whose
 * column count is a multiple of 256, tile = 128 goes back; QLMX_NT_TILE=256 in the environment is the same switch
 * from outside the process. */
int qlmx_nt_tile(int tile);
/* Math mode of the decode layer (no counterpart in the reference, whose decode path multiplies in fp32; the same
 * kind of choice as QLMX_MATH_MFMA_F16 for the training forward). fp16_inputs = 0, the default: the fp32 loop,
 * 4e-7 relative L2 on a layer's output against the fp32 reference. fp16_inputs = 1: a task's inputs (x times the
 * group scale, or silu(gate) * up times the group scale) are rounded to fp16 -- 11 significant bits, scaled per
 * task so that nothing underflows -- and multiplied with the exact digits by v_dot2_f32_f16 into fp32 sums:
 * 3.7e-4, and 1-4 % faster per layer. Applies to both decode entry points from the next call on;
 * QLMX_DECODE_MATH=fp16 in the environment is the same switch from outside the process. */
int qlmx_decode_math(int fp16_inputs);
/* Test hook. qlmx_step takes the square roots of the second moment with a short form of the correctly rounded
 * sqrtf() that is valid for arguments in [2^-96, +infinity] (and switches to sqrtf() itself below that). This
 * compares the two forms on the device for the `count` consecutive bit patterns starting at first_bits and adds
 * the number of differing results to *mismatches_dev (device memory, unsigned long long). */
int qlmx_test_sqrt_form(unsigned first_bits, unsigned long long count, unsigned long long *mismatches_dev, void *stream);
/* Test hook. For operands in the middle of the range (divisor in [2^-40, 2^40], dividend 0 or of a magnitude in that
 * interval) qlmx_step divides with the compiler's correctly rounded sequence minus its scaling and special-case
 * instructions, which do nothing there. This compares that form with `/` on the device for `count` pseudo-random
 * operand pairs of that range (derived from `seed`) and adds the number of differing results to *mismatches_dev. */
int qlmx_test_div_form(unsigned long long seed, unsigned long long count, unsigned long long *mismatches_dev, void *stream);
/* Test hook. qlmx_step has two kernels: one group per 16 lanes (every shape and option) and, for Adam on packed groups
 * of 128 without statistics, eight groups per wavefront with 16 weights per lane. They must leave the same bytes;
 * on = 0 sends every later launch through the first, on = 1 (the default) restores the choice. */
int qlmx_test_step_wide(int on);

/* =====================================================================================
 * q4n wire format (host only, no device needed): quantize_params / dequantize_params with qtype 3
 * (cudalm.cu:638-656 and 688-696). Per group: fp32 scale + packed nibbles, or a NaN scale followed by
 * the raw fp32 values when the group is not on a 4-bit grid. Byte-identical to the reference's
 * writer; the reader reproduces every value bit for bit.
 * qlmx_q4n_bound: bytes that always suffice for n values. quantize: *out_len bytes written, *nraw
 * (may be NULL) = groups stored raw. dequantize: *used (may be NULL) = bytes consumed.
 * ===================================================================================== */
size_t qlmx_q4n_bound(size_t n, int group);
int qlmx_q4n_quantize(const float *P, size_t n, int group, unsigned char *out, size_t cap, size_t *out_len, size_t *nraw);
int qlmx_q4n_dequantize(const unsigned char *buf, size_t len, float *P, size_t n, int group, size_t *used);

#ifdef __cplusplus
}
#endif
#endif /* QLMX_H */
