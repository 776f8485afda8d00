/* qlmx_gemm_f32.hip -- grouped expert GEMMs in fp32 on the vector ALU, dequantisation fused into
 * the weight-tile load.
 *
 * This is the path whose results track the reference's CPU SGEMM to rounding error: the weight is
 * formed as the single fp32 product s*digit (exactly the value the reference renders into P,
 * qlm.cuh:177) and every multiply-accumulate is an fp32 FMA, as in the reference's 6x16 micro-kernel
 * (cpu_rt.h:196-208); only the summation order differs. It serves fp32 activations of any shape
 * and is the correctness vehicle for the MFMA kernels; large bf16 problems belong on those.
 *
 * One 256-thread workgroup computes a 64x64 output tile, 4x4 per thread, stepping the contraction
 * 16 at a time through two LDS tiles. All three transposition cases share the kernel:
 *   nn: out[m,n] = sum_k A[m,k] * W[k,n]      W row-major [K,N], groups along n
 *   tn: out[m,n] = sum_k A[m,k] * W[n,k]      W row-major [N,K], groups along k   (+ beta*out)
 *   nt: out[k,n] += sum_m A[m,k] * B[m,n]     no weight operand
 * A flattened tile list covers every problem of the call, so one launch serves all experts.
 */
#include "qlmx_gemm.h"

#define TM 64
#define TN_ 64
#define TK 16

struct F32Args { const DevProb *pr; int nprob; const signed char *d; const float *s; int group; int K, N; };

template<bool BF16> __device__ __forceinline__ float ld_act(const void *p, size_t i){
    if constexpr(BF16) return qx_bf16_to_f32(((const unsigned short *)p)[i]);
    return ((const float *)p)[i];
}
/* s*digit for element e of the packed digit array; group index relative to the matrix start */
__device__ __forceinline__ float ld_weight(const signed char *d, const float *s, unsigned long long wq,
                                           unsigned long long wg, size_t e, int group){
    const unsigned long long q = wq + e;
    const unsigned b = (unsigned char)d[q >> 1];
    const int v = (q & 1ULL) ? (int)(b >> 4) : (int)(b & 15u);
    return s[wg + e / (size_t)group] * (float)(v >= 8 ? v - 16 : v);
}

template<int MODE, bool BF16>
__global__ void __launch_bounds__(256) k_gemm_f32(F32Args a){
    __shared__ float Xs[TK][TM + 4];
    __shared__ float Ys[TK][TN_ + 4];
    const int t = blockIdx.x;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * TM, j0 = tj * TN_;
    const int rows = MODE == GEMM_NT ? a.K : P.M;      /* output rows   */
    const int cols = a.N;                              /* output cols   */
    const int depth = MODE == GEMM_NT ? P.M : a.K;     /* contraction   */
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
    float acc[4][4];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 4; j++) acc[i][j] = 0.0f;

    for(int p0 = 0; p0 < depth; p0 += TK){
        /* X tile: Xs[p][i] */
#pragma unroll
        for(int e = 0; e < 4; e++){
            const int idx = threadIdx.x + 256 * e;
            int i, p;
            if constexpr(MODE == GEMM_NT){ p = idx >> 6; i = idx & 63; }     /* consecutive threads walk k (contiguous) */
            else               { i = idx >> 4; p = idx & 15; }     /* consecutive threads walk k (contiguous) */
            float v = 0.0f;
            if(i0 + i < rows && p0 + p < depth){
                if constexpr(MODE == GEMM_NT) v = ld_act<BF16>(P.A, (size_t)(p0 + p) * a.K + (i0 + i));
                else                v = ld_act<BF16>(P.A, (size_t)(i0 + i) * a.K + (p0 + p));
            }
            Xs[p][i] = v;
        }
        /* Y tile: Ys[p][j] */
#pragma unroll
        for(int e = 0; e < 4; e++){
            const int idx = threadIdx.x + 256 * e;
            int j, p;
            if constexpr(MODE == GEMM_TN){ j = idx >> 4; p = idx & 15; }     /* W[n,k]: k contiguous */
            else               { p = idx >> 6; j = idx & 63; }     /* W[k,n] / B[m,n]: n contiguous */
            float v = 0.0f;
            if(j0 + j < cols && p0 + p < depth){
                if constexpr(MODE == GEMM_NN)      v = ld_weight(a.d, a.s, P.wq, P.wg, (size_t)(p0 + p) * a.N + (j0 + j), a.group);
                else if constexpr(MODE == GEMM_TN) v = ld_weight(a.d, a.s, P.wq, P.wg, (size_t)(j0 + j) * a.K + (p0 + p), a.group);
                else                     v = ld_act<BF16>(P.B, (size_t)(p0 + p) * a.N + (j0 + j));
            }
            Ys[p][j] = v;
        }
        __syncthreads();
#pragma unroll
        for(int p = 0; p < TK; p++){
            const float4 x = *(const float4 *)&Xs[p][ty * 4];
            const float4 y = *(const float4 *)&Ys[p][tx * 4];
            const float xv[4] = {x.x, x.y, x.z, x.w}, yv[4] = {y.x, y.y, y.z, y.w};
#pragma unroll
            for(int i = 0; i < 4; i++)
#pragma unroll
                for(int j = 0; j < 4; j++) acc[i][j] = fmaf(xv[i], yv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for(int i = 0; i < 4; i++){
        const int r = i0 + ty * 4 + i;
        if(r >= rows) continue;
#pragma unroll
        for(int j = 0; j < 4; j++){
            const int c = j0 + tx * 4 + j;
            if(c >= cols) continue;
            float *o = P.C + (size_t)r * a.N + c;
            *o = P.beta != 0.0f ? *o + acc[i][j] : acc[i][j];
        }
    }
}

template<int MODE>
static int launch_f32(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                      int K, int N, int act_dtype, hipStream_t st){
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, MODE, K, N, TM, TN_, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    F32Args a; a.pr = up.dev; a.nprob = up.nprob; a.d = d; a.s = s; a.group = group; a.K = K; a.N = N;
    if(act_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL((k_gemm_f32<MODE, true>),  dim3(up.ntiles), dim3(256), 0, st, a);
    else                           hipLaunchKernelGGL((k_gemm_f32<MODE, false>), dim3(up.ntiles), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm (fp32) launch");
    return qlmx_upload_done(slot, st);
}

int qlmx_gemm_f32_dispatch(int mode, const signed char *d, const float *s, int group,
                           const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, hipStream_t st){
    if(mode == GEMM_NN) return launch_f32<GEMM_NN>(d, s, group, probs, nprob, K, N, act_dtype, st);
    if(mode == GEMM_TN) return launch_f32<GEMM_TN>(d, s, group, probs, nprob, K, N, act_dtype, st);
    return launch_f32<GEMM_NT>(d, s, group, probs, nprob, K, N, act_dtype, st);
}
