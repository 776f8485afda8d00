/* qlmx_gemm_api.hip -- C entry points of the grouped expert GEMMs: argument checks and the choice
 * between the fp32 vector-ALU kernels and the bf16 MFMA kernels. */
#include "qlmx_gemm.h"

int qlmx_gemm_f32_dispatch(int mode, const signed char *d, const float *s, int group,
                           const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, hipStream_t st);
int qlmx_gemv_nn_dispatch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                          int K, int N, hipStream_t st);
int qlmx_gemm_mfma_dispatch(int mode, const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, hipStream_t st);

static int gemm_entry(const char *who, int mode, const signed char *d, const float *s, int group,
                      const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, int math, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(K > 0 && N > 0, "%s: K=%d N=%d", who, K, N);
    QLMX_REQUIRE(act_dtype == QLMX_ACT_F32 || act_dtype == QLMX_ACT_BF16, "%s: act_dtype %d", who, act_dtype);
    QLMX_REQUIRE(math == QLMX_MATH_F32 || math == QLMX_MATH_MFMA, "%s: math %d", who, math);
    if(mode != GEMM_NT){
        QLMX_REQUIRE(d && s, "%s: NULL digits or scales", who);
        QLMX_REQUIRE(group >= 2 && group <= 256 && (group & 1) == 0, "%s: group %d", who, group);
        const int along = mode == GEMM_NN ? N : K;
        QLMX_REQUIRE(along % group == 0, "%s: the grouped dimension (%d) is not a multiple of the group (%d)", who, along, group);
        for(int i = 0; i < nprob; i++)
            QLMX_REQUIRE(probs[i].wq % (unsigned long long)group == 0, "%s: problem %d weight offset is not group aligned", who, i);
    }
    if(math == QLMX_MATH_MFMA)
        return qlmx_gemm_mfma_dispatch(mode, d, s, group, probs, nprob, K, N, act_dtype, (hipStream_t)stream);
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
/* mg_atb + mg_flush (cudalm.cu:3254-3256) */
extern "C" int qlmx_moe_gemm_nt(const qlmx_gemm_prob *probs, int nprob, int K, int N,
                                int act_dtype, int math, void *stream){
    return gemm_entry("qlmx_moe_gemm_nt", GEMM_NT, nullptr, nullptr, 0, probs, nprob, K, N, act_dtype, math, stream);
}
