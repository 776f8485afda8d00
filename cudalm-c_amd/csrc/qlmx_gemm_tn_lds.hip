/* qlmx_gemm_tn_lds.hip -- launch side of the input-gradient grouped GEMM (tn) for bf16 activations; the kernel
 * body is in qlmx_gemm_tn_body.h (mg_abt_b, cudalm.cu:3204-3256; call sites 4340-4366). */
#include "qlmx_gemm_tn_body.h"

__global__ void __launch_bounds__(256, 2) k_gemm_tn_lds(Tn3Args a){
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    tn3_block(a, blockIdx.x, lds);
}

int qlmx_pair_hold_tn(const Tn3Args &a, int grid, int slot, hipStream_t st, bool *held);

/* the launch itself (also what issues a launch that was held for a pair and found no partner) */
int qlmx_gemm_tn_lds_issue(const Tn3Args &a, int grid, int slot, hipStream_t st){
    static bool attr_set = false;
    if(!attr_set){
        QLMX_HIP(hipFuncSetAttribute((const void *)k_gemm_tn_lds, hipFuncAttributeMaxDynamicSharedMemorySize, TN3_LDS_BYTES), "tn LDS size");
        attr_set = true;
    }
    hipLaunchKernelGGL(k_gemm_tn_lds, dim3(grid), dim3(256), TN3_LDS_BYTES, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm tn (direct-to-LDS) launch");
    return qlmx_upload_done(slot, st);
}

/* bf16 activations only; N % 128 == 0, K % 64 == 0, group a power of two >= 64 (checked by the caller) */
int qlmx_gemm_tn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs,
                            const qlmx_gemm_prob *second, int nprob, int K, int N, float *out, const float *gate,
                            const float *gp, const float *up_, void *dg, void *du, hipStream_t st){
    ProbUpload up; int slot;
    /* a problem's C field is its output rows, its rows of gp (SwiGLU gradient behind), or a list of row indices */
    const RowBytes rb = {(size_t)K * 2, out ? sizeof(int) : (size_t)N * 4, (size_t)K * 2, 0, 0};
    int rc = qlmx_upload_problems_split(probs, second, nprob, GEMM_TN, K, N, TN3_BM, TN3_BN, &rb, st, &up, &slot);
    if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Tn3Args a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.nfull = up.nfull; a.tiles_n = N / TN3_BN; a.d = d; a.s = s; a.K = K; a.N = N; a.out = out; a.gate = gate;
    a.gp = gp; a.up = up_; a.dg = (unsigned short *)dg; a.du = (unsigned short *)du;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = qx_lpt_grid(up.nfull, up.ntiles, a.tiles_n);
    bool held;
    rc = qlmx_pair_hold_tn(a, grid, slot, st, &held); if(rc) return rc;
    return held ? QLMX_OK : qlmx_gemm_tn_lds_issue(a, grid, slot, st);
}
