/* qlmx_gemm_api.hip -- C entry points of the grouped expert GEMMs: argument checks and the choice
 * between the fp32 vector-ALU kernels and the bf16 MFMA kernels. */
#include "qlmx_gemm.h"
#include <stdlib.h>

int qlmx_gemm_f32_dispatch(int mode, const signed char *d, const float *s, int group,
                           const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, hipStream_t st);
int qlmx_gemv_nn_dispatch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                          int K, int N, hipStream_t st);
int qlmx_gemm_mfma_dispatch(int mode, const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *probs, const qlmx_gemm_prob *second, int nprob, int K, int N, int act_dtype, hipStream_t st, bool f16);

static int gemm_entry(const char *who, int mode, const signed char *d, const float *s, int group,
                      const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, int math, void *stream,
                      const qlmx_gemm_prob *second = nullptr){
    /* an input or weight gradient on bf16 operands can wait for its partner in an open pair; every other call
     * first issues what such a pair holds, so that the stream keeps the order of the calls */
    const bool pairable = mode != GEMM_NN && act_dtype == QLMX_ACT_BF16 && math != QLMX_MATH_F32;
    int rc = pairable ? qlmx_check_ready_keep() : qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(K > 0 && N > 0, "%s: K=%d N=%d", who, K, N);
    QLMX_REQUIRE(act_dtype == QLMX_ACT_F32 || act_dtype == QLMX_ACT_BF16, "%s: act_dtype %d", who, act_dtype);
    QLMX_REQUIRE(math == QLMX_MATH_F32 || math == QLMX_MATH_MFMA || math == QLMX_MATH_MFMA_F16, "%s: math %d", who, math);
    if(mode != GEMM_NT){
        QLMX_REQUIRE(d && s, "%s: NULL digits or scales", who);
        QLMX_REQUIRE(group >= 2 && group <= 256 && (group & 1) == 0, "%s: group %d", who, group);
        const int along = mode == GEMM_NN ? N : K;
        QLMX_REQUIRE(along % group == 0, "%s: the grouped dimension (%d) is not a multiple of the group (%d)", who, along, group);
        for(int i = 0; i < nprob; i++)
            QLMX_REQUIRE(probs[i].wq % (unsigned long long)group == 0 && (!second || second[i].wq % (unsigned long long)group == 0),
                         "%s: problem %d weight offset is not group aligned", who, i);
    }
    if(math != QLMX_MATH_F32)
        return qlmx_gemm_mfma_dispatch(mode, d, s, group, probs, second, nprob, K, N, act_dtype, (hipStream_t)stream, math == QLMX_MATH_MFMA_F16);
    QLMX_REQUIRE(!second, "%s: continued contractions need the MFMA path", who);
    if(mode == GEMM_NN && act_dtype == QLMX_ACT_F32 && N % 32 == 0 && group % 32 == 0 && ((uintptr_t)d & 15) == 0){
        /* every problem has a few rows only: stream the weights once (decode shape) */
        bool small = nprob > 0;
        for(int i = 0; i < nprob && small; i++) small = probs[i].M <= 4 && probs[i].wq % 32 == 0;
        if(small) return qlmx_gemv_nn_dispatch(d, s, group, probs, nprob, K, N, (hipStream_t)stream);
    }
    return qlmx_gemm_f32_dispatch(mode, d, s, group, probs, nprob, K, N, act_dtype, (hipStream_t)stream);
}

/* mg_ab + mg_flush (cudalm.cu:3247-3249, 3243) */
extern "C" int qlmx_moe_gemm_nn(const signed char *d, const float *s, int group,
                                const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                int act_dtype, int math, void *stream){
    return gemm_entry("qlmx_moe_gemm_nn", GEMM_NN, d, s, group, probs, nprob, K, N, act_dtype, math, stream);
}
/* mg_abt_b + mg_flush (cudalm.cu:3250-3253) */
extern "C" int qlmx_moe_gemm_tn(const signed char *d, const float *s, int group,
                                const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                int act_dtype, int math, void *stream){
    return gemm_entry("qlmx_moe_gemm_tn", GEMM_TN, d, s, group, probs, nprob, K, N, act_dtype, math, stream);
}
/* The pair of mg_abt_b calls on one output (cudalm.cu:4365-4366: dXp = dgp . w1^T, then dXp += dup . w3^T)
 * as one launch: problem i computes C = first[i].A . W(first[i])^T + second[i].A . W(second[i])^T
 * (+ C when first[i].beta = 1); second[i] supplies A, wq, wg and must repeat M. On bf16 activations
 * with MFMA math the two contractions run as one, the sum never leaving the accumulators; every other
 * combination runs the two launches the reference would. */
extern "C" int qlmx_moe_gemm_tn_pair(const signed char *d, const float *s, int group,
                                     const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int K, int N,
                                     int act_dtype, int math, void *stream){
    QLMX_REQUIRE(first && second && nprob >= 0, "qlmx_moe_gemm_tn_pair: NULL problem list");
    for(int i = 0; i < nprob; i++)
        QLMX_REQUIRE(second[i].M == first[i].M, "qlmx_moe_gemm_tn_pair: problem %d has %d and %d rows", i, first[i].M, second[i].M);
    if(act_dtype == QLMX_ACT_BF16 && math != QLMX_MATH_F32)
        return gemm_entry("qlmx_moe_gemm_tn_pair", GEMM_TN, d, s, group, first, nprob, K, N, act_dtype, math, stream, second);
    int rc = gemm_entry("qlmx_moe_gemm_tn_pair", GEMM_TN, d, s, group, first, nprob, K, N, act_dtype, math, stream);
    if(rc) return rc;
    qlmx_gemm_prob *tmp = (qlmx_gemm_prob *)malloc(sizeof(qlmx_gemm_prob) * (size_t)(nprob > 0 ? nprob : 1));
    QLMX_REQUIRE(tmp, "qlmx_moe_gemm_tn_pair: out of host memory");
    for(int i = 0; i < nprob; i++){ tmp[i] = second[i]; tmp[i].C = first[i].C; tmp[i].B = nullptr; tmp[i].beta = 1.0f; }
    rc = gemm_entry("qlmx_moe_gemm_tn_pair", GEMM_TN, d, s, group, tmp, nprob, K, N, act_dtype, math, stream);
    free(tmp);
    return rc;
}
int qlmx_gemm_nn_swiglu_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *gate,
                                   const qlmx_gemm_prob *up, int nprob, int K, int N, hipStream_t st);
int qlmx_gemm_nn_h_swiglu_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *gate, const qlmx_gemm_prob *up_,
                                 int nprob, int K, int N, const void *xsrc, hipStream_t st);
extern "C" int qlmx_swiglu(const float *G, const float *U, void *O, size_t n, int out_dtype, void *stream);

/* The gate and up GEMMs of moe_forward and the SwiGLU between them and the down GEMM (cudalm.cu:4211-4215:
 * mg_ab(Xp, w1_e, gp), mg_ab(Xp, w3_e, up), mg_flush, e_swig(gp, up, ap)) as one call. Problem i computes
 *   gp = A . W(gate[i].wq), up = A . W(up[i].wq), act = bf16(gp * sigmoid(gp) * up)
 * with A = gate[i].A [M, K] and the outputs at gate[i].C, up[i].C (fp32 [M, N]) and up[i].B (bf16 [M, N]).
 * On bf16 activations with MFMA math a tile holds 64 columns of both matrices and the SwiGLU is applied to
 * the accumulators; every other combination runs the two GEMM launches and one SwiGLU launch per problem. */
extern "C" int qlmx_moe_gemm_nn_swiglu(const signed char *d, const float *s, int group,
                                       const qlmx_gemm_prob *gate, const qlmx_gemm_prob *up, int nprob, int K, int N,
                                       int act_dtype, int math, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(gate && up && nprob >= 0, "qlmx_moe_gemm_nn_swiglu: NULL problem list");
    for(int i = 0; i < nprob; i++){
        QLMX_REQUIRE(up[i].M == gate[i].M, "qlmx_moe_gemm_nn_swiglu: problem %d has %d and %d rows", i, gate[i].M, up[i].M);
        const bool both_or_none = math == QLMX_MATH_MFMA_F16 && !gate[i].C && !up[i].C;       /* bf16 output only */
        QLMX_REQUIRE(gate[i].M == 0 || (gate[i].A && ((gate[i].C && up[i].C) || both_or_none) && up[i].B), "qlmx_moe_gemm_nn_swiglu: problem %d has a NULL pointer", i);
    }
    if(act_dtype == QLMX_ACT_BF16 && (math == QLMX_MATH_MFMA || math == QLMX_MATH_MFMA_F16) && N % 64 == 0 && K % 32 == 0 && group >= 64 && (group & (group - 1)) == 0 &&
       nprob * 2 <= QLMX_MAX_PROBLEMS){
        QLMX_REQUIRE(d && s && ((uintptr_t)d & 15) == 0, "qlmx_moe_gemm_nn_swiglu: digits and scales must be given, digits 16-byte aligned");
        for(int i = 0; i < nprob; i++){
            QLMX_REQUIRE(((uintptr_t)gate[i].A & 15) == 0 && ((uintptr_t)up[i].B & 1) == 0, "qlmx_moe_gemm_nn_swiglu: problem %d operand alignment", i);
            QLMX_REQUIRE(gate[i].wq % (unsigned long long)group == 0 && up[i].wq % (unsigned long long)group == 0 &&
                         (gate[i].wq & 31ULL) == 0 && (up[i].wq & 31ULL) == 0, "qlmx_moe_gemm_nn_swiglu: problem %d weight offset alignment", i);
        }
        if(math == QLMX_MATH_MFMA_F16) return qlmx_gemm_nn_h_swiglu_launch(d, s, group, gate, up, nprob, K, N, nullptr, (hipStream_t)stream);
        return qlmx_gemm_nn_swiglu_lds_launch(d, s, group, gate, up, nprob, K, N, (hipStream_t)stream);
    }
    for(int i = 0; i < nprob; i++)
        QLMX_REQUIRE(gate[i].M == 0 || (gate[i].C && up[i].C), "qlmx_moe_gemm_nn_swiglu: problem %d has no fp32 outputs and the shape is not one the fused kernel takes", i);
    rc = gemm_entry("qlmx_moe_gemm_nn_swiglu", GEMM_NN, d, s, group, gate, nprob, K, N, act_dtype, math, stream); if(rc) return rc;
    qlmx_gemm_prob *tmp = (qlmx_gemm_prob *)malloc(sizeof(qlmx_gemm_prob) * (size_t)(nprob > 0 ? nprob : 1));
    QLMX_REQUIRE(tmp, "qlmx_moe_gemm_nn_swiglu: out of host memory");
    for(int i = 0; i < nprob; i++){ tmp[i] = up[i]; tmp[i].A = gate[i].A; tmp[i].B = nullptr; }
    rc = gemm_entry("qlmx_moe_gemm_nn_swiglu", GEMM_NN, d, s, group, tmp, nprob, K, N, act_dtype, math, stream);
    free(tmp);
    for(int i = 0; i < nprob && !rc; i++)
        if(gate[i].M > 0) rc = qlmx_swiglu(gate[i].C, up[i].C, (void *)up[i].B, (size_t)gate[i].M * N, QLMX_ACT_BF16, stream);
    return rc;
}

/* ---- the row moves of the MoE glue folded into the GEMMs (fp16 forward kernel, bf16 input-gradient kernel) ---- */
int qlmx_gemm_nn_h_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob, int K, int N,
                          int io, const void *xsrc, float *out, const float *gate, hipStream_t st);
int qlmx_gemm_tn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, const qlmx_gemm_prob *second,
                            int nprob, int K, int N, float *out, const float *gate,
                            const float *gp, const float *up_, void *dg, void *du, hipStream_t st);

static int rows_entry_checks(const char *who, const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs,
                             const qlmx_gemm_prob *second, int nprob, int K, int N, int bk, bool idx_in_a, bool pairable = false){
    int rc = pairable ? qlmx_check_ready_keep() : qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(d && s && probs && nprob >= 0 && K > 0 && N > 0, "%s: NULL or empty argument", who);
    QLMX_REQUIRE(((uintptr_t)d & 15) == 0, "%s: digit array is not 16-byte aligned", who);
    QLMX_REQUIRE(N % 128 == 0 && K % bk == 0, "%s: N=%d must be a multiple of 128 and K=%d of %d", who, N, K, bk);
    QLMX_REQUIRE(group >= bk && group <= 256 && (group & (group - 1)) == 0, "%s: group %d must be a power of two in [%d, 256]", who, group, bk);
    for(int i = 0; i < nprob; i++){
        if(probs[i].M == 0) continue;
        QLMX_REQUIRE(probs[i].A && probs[i].C, "%s: problem %d has a NULL pointer", who, i);
        QLMX_REQUIRE(((uintptr_t)(idx_in_a ? (const void *)probs[i].C : probs[i].A) & 15) == 0 && ((uintptr_t)(idx_in_a ? probs[i].A : (const void *)probs[i].C) & 3) == 0,
                     "%s: problem %d operand alignment (rows 16 bytes, index list 4)", who, i);
        QLMX_REQUIRE(probs[i].wq % (unsigned long long)group == 0 && (probs[i].wq & 31ULL) == 0, "%s: problem %d weight offset alignment", who, i);
        if(second){
            QLMX_REQUIRE(second[i].M == probs[i].M && second[i].A && ((uintptr_t)second[i].A & 15) == 0, "%s: problem %d second half (rows, pointer, alignment)", who, i);
            QLMX_REQUIRE(second[i].wq % (unsigned long long)group == 0 && (second[i].wq & 31ULL) == 0, "%s: problem %d second weight offset alignment", who, i);
        }
    }
    return QLMX_OK;
}

/* k_gather + mg_ab (cudalm.cu:4209-4213) in one launch: problem i computes C = x[idx_i[0..M), :] . W, where
 * idx_i = (const int *)probs[i].A lists the rows of the bf16 token matrix x [tokens, K] (an entry < 0 reads as a row of
 * zeros). fp16 matrix core (QLMX_MATH_MFMA_F16 arithmetic). */
extern "C" int qlmx_moe_gemm_nn_gather(const signed char *d, const float *s, int group,
                                       const qlmx_gemm_prob *probs, int nprob, int K, int N, const void *x_bf16, void *stream){
    int rc = rows_entry_checks("qlmx_moe_gemm_nn_gather", d, s, group, probs, nullptr, nprob, K, N, 32, true); if(rc) return rc;
    QLMX_REQUIRE(x_bf16 && ((uintptr_t)x_bf16 & 15) == 0 && K % 8 == 0, "qlmx_moe_gemm_nn_gather: token matrix must be given and 16-byte aligned");
    return qlmx_gemm_nn_h_launch(d, s, group, probs, nprob, K, N, 1, x_bf16, nullptr, nullptr, (hipStream_t)stream);
}
/* k_gather + mg_ab w1 + mg_ab w3 + e_swig (cudalm.cu:4209-4215) in one launch: qlmx_moe_gemm_nn_swiglu with
 * QLMX_MATH_MFMA_F16 whose gate[i].A are row-index lists into the bf16 token matrix x, as in qlmx_moe_gemm_nn_gather.
 * gate[i].C and up[i].C may both be NULL: only the bf16 SwiGLU output up[i].B is written then. */
extern "C" int qlmx_moe_gemm_nn_gather_swiglu(const signed char *d, const float *s, int group,
                                              const qlmx_gemm_prob *gate, const qlmx_gemm_prob *up, int nprob, int K, int N,
                                              const void *x_bf16, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(d && s && gate && up && nprob >= 0 && K > 0 && N > 0 && nprob * 2 <= QLMX_MAX_PROBLEMS, "qlmx_moe_gemm_nn_gather_swiglu: NULL or empty argument, or too many problems");
    QLMX_REQUIRE(((uintptr_t)d & 15) == 0 && x_bf16 && ((uintptr_t)x_bf16 & 15) == 0, "qlmx_moe_gemm_nn_gather_swiglu: digits and token matrix must be 16-byte aligned");
    QLMX_REQUIRE(N % 64 == 0 && K % 32 == 0, "qlmx_moe_gemm_nn_gather_swiglu: N=%d must be a multiple of 64 and K=%d of 32", N, K);
    QLMX_REQUIRE(group >= 64 && group <= 256 && (group & (group - 1)) == 0, "qlmx_moe_gemm_nn_gather_swiglu: group %d must be 64, 128 or 256", group);
    for(int i = 0; i < nprob; i++){
        QLMX_REQUIRE(up[i].M == gate[i].M, "qlmx_moe_gemm_nn_gather_swiglu: problem %d has %d and %d rows", i, gate[i].M, up[i].M);
        if(gate[i].M == 0) continue;
        QLMX_REQUIRE(gate[i].A && up[i].B && (gate[i].C != nullptr) == (up[i].C != nullptr), "qlmx_moe_gemm_nn_gather_swiglu: problem %d has a NULL pointer (the fp32 outputs: both or none)", i);
        QLMX_REQUIRE(((uintptr_t)gate[i].A & 3) == 0 && ((uintptr_t)up[i].B & 3) == 0, "qlmx_moe_gemm_nn_gather_swiglu: problem %d operand alignment", i);
        QLMX_REQUIRE(gate[i].wq % (unsigned long long)group == 0 && up[i].wq % (unsigned long long)group == 0 &&
                     (gate[i].wq & 31ULL) == 0 && (up[i].wq & 31ULL) == 0, "qlmx_moe_gemm_nn_gather_swiglu: problem %d weight offset alignment", i);
    }
    return qlmx_gemm_nn_h_swiglu_launch(d, s, group, gate, up, nprob, K, N, x_bf16, (hipStream_t)stream);
}
/* mg_ab + k_scatter_gate (cudalm.cu:4224-4227) in one launch: problem i computes y = A . W and adds it to indexed rows,
 * out[idx_i[r], :] = out[idx_i[r], :] + gate[idx_i[r]] * y[r, :], idx_i = (const int *)probs[i].C (entries < 0 are dropped;
 * gate NULL adds y itself). No output row may be named twice in one call (true of one pass of the MoE layer). */
extern "C" int qlmx_moe_gemm_nn_scatter(const signed char *d, const float *s, int group,
                                        const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                        float *out, const float *gate, void *stream){
    int rc = rows_entry_checks("qlmx_moe_gemm_nn_scatter", d, s, group, probs, nullptr, nprob, K, N, 32, false); if(rc) return rc;
    QLMX_REQUIRE(out, "qlmx_moe_gemm_nn_scatter: NULL output");
    return qlmx_gemm_nn_h_launch(d, s, group, probs, nprob, K, N, 2, nullptr, out, gate, (hipStream_t)stream);
}
/* the paired mg_abt_b calls + k_scatter_add4 (cudalm.cu:4365-4367) in one launch: as qlmx_moe_gemm_tn_pair on bf16
 * activations with MFMA math, the sum of both products added to indexed rows, dst[idx_i[r], :] += y[r, :],
 * idx_i = (const int *)first[i].C. */
extern "C" int qlmx_moe_gemm_tn_pair_scatter(const signed char *d, const float *s, int group,
                                             const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int K, int N,
                                             float *dst, void *stream){
    int rc = rows_entry_checks("qlmx_moe_gemm_tn_pair_scatter", d, s, group, first, second, nprob, K, N, 64, false, true); if(rc) return rc;
    QLMX_REQUIRE(dst && second && nprob * 2 <= QLMX_MAX_PROBLEMS, "qlmx_moe_gemm_tn_pair_scatter: NULL output or too many problems");
    return qlmx_gemm_tn_lds_launch(d, s, group, first, second, nprob, K, N, dst, nullptr, nullptr, nullptr, nullptr, nullptr, (hipStream_t)stream);
}
/* mg_abt (the down projection's input gradient) + e_swigb (cudalm.cu:4340-4346) in one launch: problem i computes
 * d(act) = A . W^T [M, N] and, instead of storing it, applies k_swiglu_bwd to it: with o the element offset of
 * probs[i].C inside gp (probs[i].C points at the problem's rows of the forward's gate pre-activations),
 * dgp[o ..] and dup[o ..] (bf16) receive the gradients computed from gp[o ..], up[o ..] (fp32): the operations of
 * qlmx_swiglu_bwd on the product, with the sigmoid from the transcendental unit instead of the polynomial
 * (3e-7 relative apart), so a bf16 result can differ from the two separate calls by one unit in its last place. */
extern "C" int qlmx_moe_gemm_tn_swiglu_bwd(const signed char *d, const float *s, int group,
                                           const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                           const float *gp, const float *up, void *dgp, void *dup, void *stream){
    int rc = rows_entry_checks("qlmx_moe_gemm_tn_swiglu_bwd", d, s, group, probs, nullptr, nprob, K, N, 64, false, true); if(rc) return rc;
    QLMX_REQUIRE(gp && up && dgp && dup && (((uintptr_t)gp | (uintptr_t)up | (uintptr_t)dgp | (uintptr_t)dup) & 3) == 0, "qlmx_moe_gemm_tn_swiglu_bwd: NULL or misaligned buffer");
    for(int i = 0; i < nprob; i++)
        QLMX_REQUIRE(probs[i].M == 0 || (probs[i].C >= gp && (probs[i].C - gp) % 2 == 0), "qlmx_moe_gemm_tn_swiglu_bwd: problem %d: C must point into gp at an even element", i);
    return qlmx_gemm_tn_lds_launch(d, s, group, probs, nullptr, nprob, K, N, nullptr, nullptr, gp, up, dgp, dup, (hipStream_t)stream);
}

/* mg_atb + mg_flush (cudalm.cu:3254-3256) */
extern "C" int qlmx_moe_gemm_nt(const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                int act_dtype, int math, void *stream){
    return gemm_entry("qlmx_moe_gemm_nt", GEMM_NT, nullptr, nullptr, 0, probs, nprob, K, N, act_dtype, math, stream);
}
