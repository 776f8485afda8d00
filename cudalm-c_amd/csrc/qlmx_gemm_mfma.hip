/* qlmx_gemm_mfma.hip -- grouped expert GEMMs on the gfx950 matrix cores (v_mfma_f32_32x32x16_bf16),
 * 4-bit weights dequantised on the way into LDS.
 *
 * Replaces the reference's grouped expert GEMM calls at training sizes (mg_ab / mg_abt_b / mg_atb +
 * mg_flush, cudalm.cu:3204-3256, called from moe_forward 4211-4225 and moe_backward 4334-4366). The
 * reference multiplies by a rendered fp32 copy of the weights; here the packed digits and the group
 * scales are the operand, and what reaches the matrix core is chosen per orientation so that no
 * weight is rounded to 8 significant bits:
 *
 *   nn (forward, W[K,N], groups along N, scale differs for every contraction index k):
 *       w = s*digit is formed in fp32 (the exact value the reference renders) and split into
 *       bf16 hi + bf16 lo; two MFMAs per step add both parts (16 significant bits).
 *   tn (input gradient, W[N,K], groups along the contraction): the exact integer digits go to the
 *       matrix core; each 128-deep partial sum is scaled by s[n, chunk] in fp32 and added to the
 *       running result. No weight rounding at all.
 *   nt (weight gradient): both operands are bf16 activations / gradients; fp32 accumulate into G.
 *
 * Tiling: 256 threads = 4 wavefronts per 128x128 output tile, each wave a 64x64 quadrant held as
 * 2x2 accumulators of 32x32 (64 accumulator registers). The contraction advances 32 at a time
 * through LDS tiles stored contraction-contiguous ([row][k], 80-byte pitch) so that a lane's MFMA
 * operand (8 consecutive k of one row) is a single 128-bit LDS read. Global loads for step t+1 are
 * issued before the MFMAs of step t. One launch covers every expert of the call through a
 * flattened (problem, row tile, column tile) list.
 */
#include "qlmx_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));

#define BM 128
#define BN 128
#define BK 32
#define LDP 40              /* LDS row pitch in bf16 elements: 32 + 8 pad (80 bytes) */

struct MfmaArgs { const DevProb *pr; int nprob; const signed char *d; const float *s; int group; int K, N; };

__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi){
    return (uint32_t)qx_f32_to_bf16(lo) | ((uint32_t)qx_f32_to_bf16(hi) << 16);
}
__device__ __forceinline__ bf16x8 lds_frag(const unsigned short *p){
    const uint4 v = *(const uint4 *)p;
    return __builtin_bit_cast(bf16x8, v);
}

/* activation value as bf16 bits */
template<bool BF16> __device__ __forceinline__ unsigned short act_bits(const void *p, size_t i){
    if constexpr(BF16) return ((const unsigned short *)p)[i];
    return qx_f32_to_bf16(((const float *)p)[i]);
}

template<int MODE, bool BF16>
__global__ void __launch_bounds__(256) k_gemm_mfma(MfmaArgs a){
    /* As: rows of the output's first index; Bs: rows of the second. NN keeps two B tiles (hi, lo). */
    __shared__ __attribute__((aligned(16))) unsigned short As[BM * LDP];
    __shared__ __attribute__((aligned(16))) unsigned short Bs[(MODE == GEMM_NN ? 2 : 1) * BN * LDP];

    const int t = blockIdx.x;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * BM, j0 = tj * BN;
    const int rows  = MODE == GEMM_NT ? a.K : P.M;
    const int depth = MODE == GEMM_NT ? P.M : a.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * 64, wj = (wave & 1) * 64;      /* quadrant of this wave */

    f32x16 acc[2][2], part[2][2];
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++){ acc[i][j] = (f32x16)(0.0f); part[i][j] = (f32x16)(0.0f); }

    /* ---- per-thread staging registers for one 32-deep step ---- */
    uint4 ra[2];            /* NN/TN: two 16-byte pieces of A rows. NT: two row-pairs x 8 k of A */
    uint4 rb[2];            /* NT: two row-pairs x 8 n of B. */
    uint32_t rw[2];         /* NN: digits of rows k,k+1 (8 n each). TN: two dwords (8 k each) */
    float rs[2];            /* NN: scales of rows k, k+1 */

    auto load_step = [&](int p0){
        if constexpr(MODE == GEMM_NT){
            /* A^T tile: As[k][m], B^T tile: Bs[n][m]; thread takes the row pair (m, m+1) and 8
             * consecutive k (resp. n): task = pair 0..15 x octet 0..15 */
            const int pr_ = tid & 15, oc = tid >> 4;
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int m = p0 + 2 * pr_ + h;
                uint4 va = make_uint4(0, 0, 0, 0), vb = make_uint4(0, 0, 0, 0);
                if(m < depth){
                    if constexpr(BF16){
                        va = *(const uint4 *)((const unsigned short *)P.A + (size_t)m * a.K + i0 + oc * 8);
                        vb = *(const uint4 *)((const unsigned short *)P.B + (size_t)m * a.N + j0 + oc * 8);
                    } else {
                        const float *pa = (const float *)P.A + (size_t)m * a.K + i0 + oc * 8;
                        const float *pb = (const float *)P.B + (size_t)m * a.N + j0 + oc * 8;
                        va = make_uint4(pack_bf16(pa[0], pa[1]), pack_bf16(pa[2], pa[3]), pack_bf16(pa[4], pa[5]), pack_bf16(pa[6], pa[7]));
                        vb = make_uint4(pack_bf16(pb[0], pb[1]), pack_bf16(pb[2], pb[3]), pack_bf16(pb[4], pb[5]), pack_bf16(pb[6], pb[7]));
                    }
                }
                ra[h] = va; rb[h] = vb;
            }
        } else {
            /* A tile 128 rows x 32 k: 512 pieces of 8 k, two per thread */
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int piece = tid + 256 * h, r = piece >> 2, kq = piece & 3;
                uint4 v = make_uint4(0, 0, 0, 0);
                if(i0 + r < rows){
                    if constexpr(BF16) v = *(const uint4 *)((const unsigned short *)P.A + (size_t)(i0 + r) * a.K + p0 + kq * 8);
                    else {
                        const float *pa = (const float *)P.A + (size_t)(i0 + r) * a.K + p0 + kq * 8;
                        v = make_uint4(pack_bf16(pa[0], pa[1]), pack_bf16(pa[2], pa[3]), pack_bf16(pa[4], pa[5]), pack_bf16(pa[6], pa[7]));
                    }
                }
                ra[h] = v;
            }
            if constexpr(MODE == GEMM_NN){
                /* W[k, n]: thread = (k pair 0..15, n octet 0..15) */
                const int kp = tid & 15, oc = tid >> 4;
#pragma unroll
                for(int h = 0; h < 2; h++){
                    const size_t e = (size_t)(p0 + 2 * kp + h) * a.N + j0 + oc * 8;
                    rw[h] = *(const uint32_t *)(a.d + ((P.wq + e) >> 1));
                    rs[h] = a.s[P.wg + e / (size_t)a.group];
                }
            } else {
                /* W[n, k]: 128 rows x 4 k-octets = 512 dwords, two per thread */
#pragma unroll
                for(int h = 0; h < 2; h++){
                    const int piece = tid + 256 * h, r = piece >> 2, kq = piece & 3;
                    const size_t e = (size_t)(j0 + r) * a.K + p0 + kq * 8;
                    rw[h] = *(const uint32_t *)(a.d + ((P.wq + e) >> 1));
                }
            }
        }
    };

    auto store_step = [&](){
        if constexpr(MODE == GEMM_NT){
            const int pr_ = tid & 15, oc = tid >> 4;
            const uint32_t a0[4] = {ra[0].x, ra[0].y, ra[0].z, ra[0].w}, a1[4] = {ra[1].x, ra[1].y, ra[1].z, ra[1].w};
            const uint32_t b0[4] = {rb[0].x, rb[0].y, rb[0].z, rb[0].w}, b1[4] = {rb[1].x, rb[1].y, rb[1].z, rb[1].w};
#pragma unroll
            for(int j = 0; j < 8; j++){
                const int w = j >> 1, sh = (j & 1) * 16;
                const uint32_t pa = ((a0[w] >> sh) & 0xFFFFu) | (((a1[w] >> sh) & 0xFFFFu) << 16);
                const uint32_t pb = ((b0[w] >> sh) & 0xFFFFu) | (((b1[w] >> sh) & 0xFFFFu) << 16);
                *(uint32_t *)&As[(oc * 8 + j) * LDP + 2 * pr_] = pa;
                *(uint32_t *)&Bs[(oc * 8 + j) * LDP + 2 * pr_] = pb;
            }
        } else {
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int piece = tid + 256 * h, r = piece >> 2, kq = piece & 3;
                *(uint4 *)&As[r * LDP + kq * 8] = ra[h];
            }
            if constexpr(MODE == GEMM_NN){
                const int kp = tid & 15, oc = tid >> 4;
#pragma unroll
                for(int j = 0; j < 8; j++){
                    const float w0 = rs[0] * (float)qx_nib(rw[0], j), w1 = rs[1] * (float)qx_nib(rw[1], j);
                    const unsigned short h0 = qx_f32_to_bf16(w0), h1 = qx_f32_to_bf16(w1);
                    const float l0 = w0 - qx_bf16_to_f32(h0), l1 = w1 - qx_bf16_to_f32(h1);
                    *(uint32_t *)&Bs[(oc * 8 + j) * LDP + 2 * kp] = (uint32_t)h0 | ((uint32_t)h1 << 16);
                    *(uint32_t *)&Bs[BN * LDP + (oc * 8 + j) * LDP + 2 * kp] = pack_bf16(l0, l1);
                }
            } else {
#pragma unroll
                for(int h = 0; h < 2; h++){
                    const int piece = tid + 256 * h, r = piece >> 2, kq = piece & 3;
                    uint4 v;
                    v.x = pack_bf16((float)qx_nib(rw[h], 0), (float)qx_nib(rw[h], 1));
                    v.y = pack_bf16((float)qx_nib(rw[h], 2), (float)qx_nib(rw[h], 3));
                    v.z = pack_bf16((float)qx_nib(rw[h], 4), (float)qx_nib(rw[h], 5));
                    v.w = pack_bf16((float)qx_nib(rw[h], 6), (float)qx_nib(rw[h], 7));
                    *(uint4 *)&Bs[r * LDP + kq * 8] = v;
                }
            }
        }
    };

    const int fr = lane & 31, fk = (lane >> 5) * 8;       /* operand row and k-offset of this lane */
    const int steps = (depth + BK - 1) / BK;
    const int steps_per_group = MODE == GEMM_TN ? a.group / BK : 0;

    load_step(0);
    for(int st = 0; st < steps; st++){
        store_step();
        __syncthreads();
        if(st + 1 < steps) load_step((st + 1) * BK);
#pragma unroll
        for(int ks = 0; ks < BK; ks += 16){
            bf16x8 fa[2], fb[2], fl[2];
#pragma unroll
            for(int i = 0; i < 2; i++) fa[i] = lds_frag(&As[(wi + i * 32 + fr) * LDP + ks + fk]);
#pragma unroll
            for(int j = 0; j < 2; j++){
                fb[j] = lds_frag(&Bs[(wj + j * 32 + fr) * LDP + ks + fk]);
                if constexpr(MODE == GEMM_NN) fl[j] = lds_frag(&Bs[BN * LDP + (wj + j * 32 + fr) * LDP + ks + fk]);
            }
#pragma unroll
            for(int i = 0; i < 2; i++)
#pragma unroll
                for(int j = 0; j < 2; j++){
                    if constexpr(MODE == GEMM_TN){
                        part[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], part[i][j], 0, 0, 0);
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
                        if constexpr(MODE == GEMM_NN)
                            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fl[j], acc[i][j], 0, 0, 0);
                    }
                }
        }
        if(MODE == GEMM_TN && ((st + 1) % steps_per_group == 0)){
            /* one scale group of the contraction is complete: fold it in with its fp32 scale */
            const int chunk = (st * BK) / a.group;
#pragma unroll
            for(int j = 0; j < 2; j++){
                const int n = j0 + wj + j * 32 + fr;              /* this lane's output column */
                const float sc = a.s[P.wg + (size_t)n * (a.K / a.group) + chunk];
#pragma unroll
                for(int i = 0; i < 2; i++){
#pragma unroll
                    for(int v = 0; v < 16; v++) acc[i][j][v] = fmaf(sc, part[i][j][v], acc[i][j][v]);
                    part[i][j] = (f32x16)(0.0f);
                }
            }
        }
        __syncthreads();
    }

    /* ---- epilogue: lane holds column fr of each 32x32 tile, rows (v/4)*8 + (lane/32)*4 + v%4 ---- */
#pragma unroll
    for(int i = 0; i < 2; i++)
#pragma unroll
        for(int j = 0; j < 2; j++){
            const int c = j0 + wj + j * 32 + fr;
#pragma unroll
            for(int v = 0; v < 16; v++){
                const int r = i0 + wi + i * 32 + (v >> 2) * 8 + (lane >> 5) * 4 + (v & 3);
                if(r < rows){
                    float *o = P.C + (size_t)r * a.N + c;
                    *o = P.beta != 0.0f ? *o + acc[i][j][v] : acc[i][j][v];
                }
            }
        }
}

template<int MODE>
static int launch_mfma(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                       int K, int N, int act_dtype, hipStream_t st){
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, MODE, K, N, BM, BN, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    MfmaArgs a; a.pr = up.dev; a.nprob = up.nprob; a.d = d; a.s = s; a.group = group; a.K = K; a.N = N;
    if(act_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL((k_gemm_mfma<MODE, true>),  dim3(up.ntiles), dim3(256), 0, st, a);
    else                           hipLaunchKernelGGL((k_gemm_mfma<MODE, false>), dim3(up.ntiles), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm (mfma) launch");
    return qlmx_upload_done(slot, st);
}

int qlmx_gemm_mfma_dispatch(int mode, const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *probs, int nprob, int K, int N, int act_dtype, hipStream_t st){
    /* shapes the tiling assumes; anything else must use QLMX_MATH_F32 */
    QLMX_REQUIRE(N % BN == 0, "mfma gemm: N=%d is not a multiple of %d (use QLMX_MATH_F32)", N, BN);
    if(mode == GEMM_NT) QLMX_REQUIRE(K % BM == 0, "mfma gemm nt: K=%d is not a multiple of %d (use QLMX_MATH_F32)", K, BM);
    else                QLMX_REQUIRE(K % BK == 0, "mfma gemm: K=%d is not a multiple of %d (use QLMX_MATH_F32)", K, BK);
    if(mode != GEMM_NT) QLMX_REQUIRE(group % BK == 0, "mfma gemm: group %d is not a multiple of %d", group, BK);
    for(int i = 0; i < nprob; i++){
        const int al = act_dtype == QLMX_ACT_BF16 ? 15 : 3;
        QLMX_REQUIRE(((uintptr_t)probs[i].A & al) == 0 && (mode != GEMM_NT || ((uintptr_t)probs[i].B & al) == 0),
                     "mfma gemm: problem %d operand is not 16-byte aligned", i);
        QLMX_REQUIRE(mode == GEMM_NT || (probs[i].wq & 7ULL) == 0, "mfma gemm: problem %d weight offset not a multiple of 8", i);
    }
    QLMX_REQUIRE(((uintptr_t)d & 3) == 0, "mfma gemm: digit array is not 4-byte aligned");
    QLMX_REQUIRE(act_dtype != QLMX_ACT_BF16 || (K % 8 == 0 && N % 8 == 0), "mfma gemm: bf16 rows must be multiples of 8 elements");
    if(mode == GEMM_NN) return launch_mfma<GEMM_NN>(d, s, group, probs, nprob, K, N, act_dtype, st);
    if(mode == GEMM_TN) return launch_mfma<GEMM_TN>(d, s, group, probs, nprob, K, N, act_dtype, st);
    return launch_mfma<GEMM_NT>(d, s, group, probs, nprob, K, N, act_dtype, st);
}
