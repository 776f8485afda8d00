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
 * Tiling: 256 threads = 4 wavefronts in a 2x2 arrangement; a wave owns (32*WM) x 64 of the output as
 * WM x 2 accumulators of 32x32. nn and nt use WM = 4 (256x128 per workgroup, which halves the
 * dequantisation work per flop); tn keeps a second set of accumulators for the per-group partial
 * sums and uses WM = 2 (128x128). The contraction advances 32 at a time.
 *
 * LDS holds operands as 16-byte items of 8 consecutive contraction elements, item (ko, row) at
 * index ko*ROWS + (row ^ swizzle), swizzle = ((row >> 4) ^ 4*ko) & 15 on the low four bits. A lane's
 * MFMA operand is then one 128-bit read; the 128-bit writes of straight copies, the 32-bit writes of
 * transposing stores and the operand reads each hit all 64 banks without (or with 2-way) conflicts,
 * with no padding. Global loads walk the contiguous index fastest so every wave instruction covers
 * 64-512 contiguous bytes per row. Two LDS buffers: the stores and loads for the next steps are
 * issued around the MFMAs of the current one and a single barrier closes a step. One launch covers
 * every expert of the call through a flattened (problem, row tile, column tile) list.
 */
#include "qlmx_gemm.h"
int qlmx_gemm_tn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, const qlmx_gemm_prob *second,
                            int nprob, int K, int N, float *out, const float *gate,
                            const float *gp, const float *up_, void *dg, void *du, hipStream_t st);
int qlmx_gemm_nn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob, int K, int N, hipStream_t st);
int qlmx_gemm_nn_h_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob, int K, int N,
                          int io, const void *xsrc, float *out, const float *gate, hipStream_t st);
int qlmx_gemm_nt_lds_launch(const qlmx_gemm_prob *probs, int nprob, int K, int N, hipStream_t st);

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  f32x2  __attribute__((ext_vector_type(2)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));

#define BN 128
#define BK 32                /* contraction depth of a step for nn and nt */
#define KO 4                 /* 16-byte items per row per step */
#define BK_TN 64             /* tn: 64 deep, so that a step reads whole 128-byte lines of the bf16 rows and
                              * carries 16 MFMAs per wavefront between barriers */

struct MfmaArgs { const DevProb *pr; int nprob, ntiles, tiles_n, rows_p; const signed char *d; const float *s; int group, gshift; int K, N; };

/* two floats -> packed bf16 pair, round to nearest even (one v_cvt_pk_bf16_f32) */
__device__ __forceinline__ uint32_t pk_bf16(float lo, float hi){
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
__device__ __forceinline__ uint4 pk8_bf16(const float *p){
    const float4 a = *(const float4 *)p, b = *(const float4 *)(p + 4);
    return make_uint4(pk_bf16(a.x, a.y), pk_bf16(a.z, a.w), pk_bf16(b.x, b.y), pk_bf16(b.z, b.w));
}
template<int ROWS, int KOT = KO> __device__ __forceinline__ int item_at(int ko, int row){
    if constexpr(KOT == 8) return ko * ROWS + (row ^ ((ko << 1) & 15));      /* 128-bit accesses only: 8 items x 2 rows fill the banks */
    return ko * ROWS + (row ^ (((row >> 4) ^ (ko << 2)) & 15));
}

template<int MODE, bool BF16, int WM, bool DEEP>
__global__ void __launch_bounds__(256, 2) k_gemm_mfma(MfmaArgs a){
    constexpr int BM = 64 * WM;
    constexpr int NB = MODE == GEMM_NN ? 2 : 1;                 /* B planes: hi (+ lo) */
    constexpr int KOT = MODE == GEMM_TN ? BK_TN / 8 : KO;      /* items per row per step */
    constexpr int BKT = KOT * 8;                               /* contraction depth of a step */
    constexpr int A_BYTES = KOT * BM * 16, B_BYTES = KOT * BN * 16;
    /* one LDS block: [buffer 0: A | B hi | B lo][buffer 1: ...] */
    constexpr int BUF_BYTES = A_BYTES + NB * B_BYTES;
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * BUF_BYTES];

    /* Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. nn/tn (tiles of equal
     * cost): XCD x takes the x-th contiguous eighth of the tile list, so tiles sharing an expert's
     * rows and weights meet in one L2. nt (cost = the expert's row count): whole problems per XCD, or
     * output tile-rows dealt round-robin when their number per problem is a multiple of 8. */
    const int t = MODE != GEMM_NT ? qx_xcd_tile(blockIdx.x, gridDim.x)
                : (a.rows_p & 7) ? qx_xcd_tile_probs(blockIdx.x, a.tiles_n, a.rows_p) : qx_xcd_tile_rows(blockIdx.x, a.tiles_n);
    if(t >= a.ntiles) return;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * BM, j0 = tj * BN;
    const int rows  = MODE == GEMM_NT ? a.K : P.M;
    const int depth = MODE == GEMM_NT ? P.M : a.K;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (32 * WM), wj = (wave & 1) * 64;
    const int fr = lane & 31, hf = lane >> 5;

    f32x16 acc[WM][2];
    f32x16 part[MODE == GEMM_TN ? WM : 1][2];
#pragma unroll
    for(int i = 0; i < WM; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.0f);
    if constexpr(MODE == GEMM_TN){
#pragma unroll
        for(int i = 0; i < WM; i++)
#pragma unroll
            for(int j = 0; j < 2; j++) part[i][j] = (f32x16)(0.0f);
    }

    /* ---- everything that does not change from step to step is computed once: global pointers
     * (advanced by a constant per step), LDS byte offsets of this thread's stores and of its MFMA
     * operand reads. Rows past the end of a problem are clamped to its last row instead of being
     * zero-filled when they only feed output rows that are never stored. ---- */
    constexpr int NA = MODE == GEMM_NT ? 4 : WM * KOT / 4;    /* 16-byte A-side loads per thread per step */
    constexpr int ESZ = BF16 ? 2 : 4;
    const char *pa[NA];                                /* A-side source pointers                    */
    const char *pb[2];                                 /* nt: B-side source pointers                */
    const signed char *pw0 = a.d, *pw1 = a.d;          /* nn: digit rows k, k+1; tn: row n          */
    const float *ps0 = a.s, *ps1 = a.s;                /* nn: their scales                          */
    int sa_off[MODE == GEMM_NT ? 2 : NA];              /* LDS store offsets, A side (nt: per task)  */
    int sj_off[8];                                     /* transposing stores: the 8 row offsets     */
    int sb_off = 0, sbj_off[8];                        /* B side                                    */
    size_t astep, bstep = 0, wstep = 0, sstep = 0;     /* per-step advances in bytes / elements     */

    if constexpr(MODE == GEMM_NT){
#pragma unroll
        for(int h = 0; h < 2; h++){
            const int id = tid + 256 * h, oc = id & 31, mp = id >> 5;
            const int kk = (i0 + oc * 8 < a.K) ? i0 + oc * 8 : 0;          /* columns past K feed unstored rows */
#pragma unroll
            for(int e = 0; e < 2; e++) pa[2 * h + e] = (const char *)P.A + ((size_t)(2 * mp + e) * a.K + kk) * ESZ;
            sa_off[h] = (mp >> 2) * BM * 16 + (mp & 3) * 4;
        }
        { const int oc = (tid & 31), ko = (tid >> 5) >> 2;                 /* task 1 has ko + 2: its swizzle differs in bit 3 */
          const int sw = ((oc >> 1) ^ (ko << 2)) & 15;
#pragma unroll
          for(int j = 0; j < 8; j++) sj_off[j] = ((oc * 8 + j) ^ sw) * 16; }
        { const int oc = tid & 15, mp = tid >> 4, ko = mp >> 2;
#pragma unroll
          for(int e = 0; e < 2; e++) pb[e] = (const char *)P.B + ((size_t)(2 * mp + e) * a.N + j0 + oc * 8) * ESZ;
          sb_off = A_BYTES + ko * BN * 16 + (mp & 3) * 4;
          const int sw = ((oc >> 1) ^ (ko << 2)) & 15;
#pragma unroll
          for(int j = 0; j < 8; j++) sbj_off[j] = ((oc * 8 + j) ^ sw) * 16; }
        astep = (size_t)BK * a.K * ESZ; bstep = (size_t)BK * a.N * ESZ;
    } else {
#pragma unroll
        for(int h = 0; h < NA; h++){
            const int id = tid + 256 * h, kq = id & (KOT - 1), r = id / KOT;
            const int rr = (i0 + r < rows) ? i0 + r : rows - 1;            /* clamp: feeds unstored rows only */
            pa[h] = (const char *)P.A + ((size_t)rr * a.K + kq * 8) * ESZ;
            sa_off[h] = item_at<BM, KOT>(kq, r) * 16;
        }
        astep = (size_t)BKT * ESZ;
        if constexpr(MODE == GEMM_NN){
            const int oc = tid & 15, kp = tid >> 4, ko = kp >> 2;
            const size_t e0 = (size_t)(2 * kp) * a.N + j0 + oc * 8;
            pw0 = a.d + ((P.wq + e0) >> 1); pw1 = pw0 + (a.N >> 1);
            ps0 = a.s + P.wg + (e0 >> a.gshift); ps1 = a.s + P.wg + ((e0 + a.N) >> a.gshift);
            wstep = (size_t)BK * a.N >> 1; sstep = (size_t)BK * a.N >> a.gshift;
            sb_off = A_BYTES + ko * BN * 16 + (kp & 3) * 4;
            const int sw = ((oc >> 1) ^ (ko << 2)) & 15;
#pragma unroll
            for(int j = 0; j < 8; j++) sbj_off[j] = ((oc * 8 + j) ^ sw) * 16;
        } else {
            /* thread = (row n, half of the step's 64 digits): 16 bytes = 32 digits = 4 items */
            const int n = tid & (BN - 1), half = tid >> 7;
            pw0 = a.d + ((P.wq + (size_t)(j0 + n) * a.K) >> 1) + half * 16;
            wstep = BKT >> 1;
#pragma unroll
            for(int ko = 0; ko < 4; ko++) sbj_off[ko] = A_BYTES + item_at<BN, KOT>(half * 4 + ko, n) * 16;
        }
    }
    /* MFMA operand read offsets: [k16 half][tile] */
    int ra_off[KOT / 2][WM], rb_off[KOT / 2][2];
#pragma unroll
    for(int ks = 0; ks < KOT / 2; ks++){
#pragma unroll
        for(int i = 0; i < WM; i++) ra_off[ks][i] = item_at<BM, KOT>(ks * 2 + hf, wi + i * 32 + fr) * 16;
#pragma unroll
        for(int j = 0; j < 2; j++) rb_off[ks][j] = A_BYTES + item_at<BN, KOT>(ks * 2 + hf, wj + j * 32 + fr) * 16;
    }

    struct Stage {
        uint4 ra[NA];
        uint4 rb[2];
        uint4 rw;                                      /* nn: .x,.y digits of rows k,k+1; tn: 32 digits of one n row */
        float rs0, rs1;
    };
    Stage S0, S1;
    S0.rw = make_uint4(0, 0, 0, 0); S1.rw = S0.rw; S0.rs0 = S0.rs1 = S1.rs0 = S1.rs1 = 0.0f;

    auto ld16 = [&](const char *p) -> uint4 {
        if constexpr(BF16) return *(const uint4 *)p;
        else return pk8_bf16((const float *)p);
    };
    /* loads the tile of the next step in program order (pointers advance as a side effect) */
    auto load_step = [&](Stage &G, int p0){
        if constexpr(MODE == GEMM_NT){
            /* Rows past the end of the expert exist only in its last step. They are loaded from row 0
             * (always valid) and zeroed when the tile is written to LDS: a load inside a branch would
             * make every one of the six loads wait for the previous one. */
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int mp = (tid + 256 * h) >> 5;
#pragma unroll
                for(int e = 0; e < 2; e++){
                    const char *q = (p0 + 2 * mp + e < depth) ? pa[2 * h + e] : (const char *)P.A;
                    G.ra[2 * h + e] = ld16(q);
                    pa[2 * h + e] += astep;
                }
            }
            { const int mp = tid >> 4;
#pragma unroll
              for(int e = 0; e < 2; e++){
                  const char *q = (p0 + 2 * mp + e < depth) ? pb[e] : (const char *)P.B;
                  G.rb[e] = ld16(q);
                  pb[e] += bstep;
              } }
            G.rw.x = (uint32_t)p0;                     /* remembered for the zeroing at store time */
        } else {
#pragma unroll
            for(int h = 0; h < NA; h++){ G.ra[h] = ld16(pa[h]); pa[h] += astep; }
            if constexpr(MODE == GEMM_NN){
                G.rw.x = *(const uint32_t *)pw0; G.rw.y = *(const uint32_t *)pw1;
                G.rs0 = *ps0; G.rs1 = *ps1;
                pw0 += wstep; pw1 += wstep; ps0 += sstep; ps1 += sstep;
            } else {
                G.rw = *(const uint4 *)pw0;
                pw0 += wstep;
            }
        }
    };

    auto store_step = [&](const Stage &G, int nb){
        unsigned char *L = lds + nb * BUF_BYTES;
        if constexpr(MODE == GEMM_NT){
            const int p0 = (int)G.rw.x;
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int m0 = p0 + 2 * ((tid + 256 * h) >> 5);
                const uint32_t k0 = m0 < depth ? 0xFFFFFFFFu : 0u, k1 = m0 + 1 < depth ? 0xFFFFFFFFu : 0u;
                const uint32_t x0[4] = {G.ra[2 * h].x & k0, G.ra[2 * h].y & k0, G.ra[2 * h].z & k0, G.ra[2 * h].w & k0};
                const uint32_t x1[4] = {G.ra[2 * h + 1].x & k1, G.ra[2 * h + 1].y & k1, G.ra[2 * h + 1].z & k1, G.ra[2 * h + 1].w & k1};
#pragma unroll
                for(int j = 0; j < 8; j++)
                    *(uint32_t *)(L + sa_off[h] + (sj_off[j] ^ (h * 128))) = __builtin_amdgcn_perm(x1[j >> 1], x0[j >> 1], (j & 1) ? 0x07060302u : 0x05040100u);
            }
            { const int m0 = p0 + 2 * (tid >> 4);
              const uint32_t k0 = m0 < depth ? 0xFFFFFFFFu : 0u, k1 = m0 + 1 < depth ? 0xFFFFFFFFu : 0u;
              const uint32_t y0[4] = {G.rb[0].x & k0, G.rb[0].y & k0, G.rb[0].z & k0, G.rb[0].w & k0}, y1[4] = {G.rb[1].x & k1, G.rb[1].y & k1, G.rb[1].z & k1, G.rb[1].w & k1};
#pragma unroll
              for(int j = 0; j < 8; j++)
                  *(uint32_t *)(L + sb_off + sbj_off[j]) = __builtin_amdgcn_perm(y1[j >> 1], y0[j >> 1], (j & 1) ? 0x07060302u : 0x05040100u); }
        } else {
#pragma unroll
            for(int h = 0; h < NA; h++) *(uint4 *)(L + sa_off[h]) = G.ra[h];
            if constexpr(MODE == GEMM_NN){
#pragma unroll
                for(int j = 0; j < 8; j++){
                    const float w0 = G.rs0 * (float)qx_nib(G.rw.x, j), w1 = G.rs1 * (float)qx_nib(G.rw.y, j);
                    const uint32_t hi = pk_bf16(w0, w1);
                    const float l0 = w0 - __uint_as_float(hi << 16), l1 = w1 - __uint_as_float(hi & 0xFFFF0000u);
                    *(uint32_t *)(L + sb_off + sbj_off[j]) = hi;
                    *(uint32_t *)(L + sb_off + B_BYTES + sbj_off[j]) = pk_bf16(l0, l1);
                }
            } else {
                const uint32_t wd[4] = {G.rw.x, G.rw.y, G.rw.z, G.rw.w};
#pragma unroll
                for(int ko = 0; ko < 4; ko++){
                    uint4 v;
                    v.x = pk_bf16((float)qx_nib(wd[ko], 0), (float)qx_nib(wd[ko], 1));
                    v.y = pk_bf16((float)qx_nib(wd[ko], 2), (float)qx_nib(wd[ko], 3));
                    v.z = pk_bf16((float)qx_nib(wd[ko], 4), (float)qx_nib(wd[ko], 5));
                    v.w = pk_bf16((float)qx_nib(wd[ko], 6), (float)qx_nib(wd[ko], 7));
                    *(uint4 *)(L + sbj_off[ko]) = v;
                }
            }
        }
    };

    auto compute = [&](int cb){
        const unsigned char *L = lds + cb * BUF_BYTES;
#pragma unroll
        for(int ks = 0; ks < KOT / 2; ks++){
            bf16x8 fa[WM], fb[2], fl[2];
#pragma unroll
            for(int i = 0; i < WM; i++) fa[i] = __builtin_bit_cast(bf16x8, *(const uint4 *)(L + ra_off[ks][i]));
#pragma unroll
            for(int j = 0; j < 2; j++){
                fb[j] = __builtin_bit_cast(bf16x8, *(const uint4 *)(L + rb_off[ks][j]));
                if constexpr(MODE == GEMM_NN) fl[j] = __builtin_bit_cast(bf16x8, *(const uint4 *)(L + rb_off[ks][j] + B_BYTES));
            }
#pragma unroll
            for(int i = 0; i < WM; i++)
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
    };

    const int steps = (depth + BKT - 1) / BKT;
    const int steps_per_group = MODE == GEMM_TN ? (1 << a.gshift) / BKT : 1;
    const float *pfold[2] = {a.s, a.s};                /* tn: scale of (this lane's column, current group) */
    if constexpr(MODE == GEMM_TN){
#pragma unroll
        for(int j = 0; j < 2; j++) pfold[j] = a.s + P.wg + (size_t)(j0 + wj + j * 32 + fr) * (a.K >> a.gshift);
    }

    auto fold_group = [&](int st){
        if constexpr(MODE == GEMM_TN){
            if((st + 1) % steps_per_group == 0){
                /* one scale group of the contraction is complete: fold it in with its fp32 scale */
#pragma unroll
                for(int j = 0; j < 2; j++){
                    const float sc = *pfold[j]; pfold[j] += 1;
#pragma unroll
                    for(int i = 0; i < WM; i++){
#pragma unroll
                        for(int v = 0; v < 16; v++) acc[i][j][v] = fmaf(sc, part[i][j][v], acc[i][j][v]);
                        part[i][j] = (f32x16)(0.0f);
                    }
                }
            }
        }
    };

    /* step st computes from LDS buffer st&1. While it computes, the tile of step st+1 is written to
     * the other buffer and the tile of a later step is requested from global memory (two steps ahead
     * with DEEP, which keeps two sets of staging registers; one otherwise). */
    if constexpr(DEEP){
        load_step(S0, 0);
        if(steps > 1) load_step(S1, BKT);
        store_step(S0, 0);
        if(steps > 2) load_step(S0, 2 * BKT);
        __syncthreads();
        for(int st = 0; st < steps; st += 2){
            compute(0);
            if(st + 1 < steps) store_step(S1, 1);
            if(st + 3 < steps) load_step(S1, (st + 3) * BKT);
            fold_group(st);
            __syncthreads();
            if(st + 1 < steps){
                compute(1);
                if(st + 2 < steps) store_step(S0, 0);
                if(st + 4 < steps) load_step(S0, (st + 4) * BKT);
                fold_group(st + 1);
                __syncthreads();
            }
        }
    } else {
        load_step(S0, 0);
        store_step(S0, 0);
        if(steps > 1) load_step(S0, BKT);
        __syncthreads();
        for(int st = 0; st < steps; st++){
            compute(st & 1);
            if(st + 1 < steps) store_step(S0, (st + 1) & 1);
            if(st + 2 < steps) load_step(S0, (st + 2) * BKT);
            fold_group(st);
            __syncthreads();
        }
    }

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int row = i0 + wi + hf * 4;
    qx_store_tiles<WM, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, rows, (size_t)a.N, P.beta != 0.0f);
}

template<int MODE, int WM, bool DEEP>
static int launch_mfma(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                       int K, int N, int act_dtype, hipStream_t st){
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, MODE, K, N, 64 * WM, BN, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    MfmaArgs a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.tiles_n = N / BN; a.d = d; a.s = s; a.group = group; a.gshift = 0; while((1 << a.gshift) < group) a.gshift++; a.K = K; a.N = N;
    int grid = (up.ntiles + 7) / 8 * 8;
    a.rows_p = 1;
    if(MODE == GEMM_NT){
        a.rows_p = up.ntiles / (a.tiles_n * up.nprob);
        if(a.rows_p & 7) grid = 8 * a.tiles_n * a.rows_p * ((up.nprob + 7) / 8);
        else             grid = 8 * a.tiles_n * ((up.ntiles / a.tiles_n + 7) / 8);
    }
    if(act_dtype == QLMX_ACT_BF16) hipLaunchKernelGGL((k_gemm_mfma<MODE, true, WM, DEEP>),  dim3(grid), dim3(256), 0, st, a);
    else                           hipLaunchKernelGGL((k_gemm_mfma<MODE, false, WM, DEEP>), dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm (mfma) launch");
    return qlmx_upload_done(slot, st);
}

/* `second`: tn on bf16 activations only, the continuation of every problem's contraction (else NULL) */
int qlmx_gemm_mfma_dispatch(int mode, const signed char *d, const float *s, int group,
                            const qlmx_gemm_prob *probs, const qlmx_gemm_prob *second, int nprob, int K, int N, int act_dtype, hipStream_t st, bool f16){
    QLMX_REQUIRE(!second || (mode == GEMM_TN && act_dtype == QLMX_ACT_BF16), "mfma gemm: continued contractions exist for tn on bf16 activations only");
    /* shapes the tiling assumes; anything else must use QLMX_MATH_F32 */
    QLMX_REQUIRE(N % BN == 0, "mfma gemm: N=%d is not a multiple of %d (use QLMX_MATH_F32)", N, BN);
    if(mode == GEMM_NT) QLMX_REQUIRE(K % 8 == 0, "mfma gemm nt: K=%d is not a multiple of 8 (use QLMX_MATH_F32)", K);
    else {
        const int bk = mode == GEMM_TN ? BK_TN : BK;
        QLMX_REQUIRE(K % bk == 0, "mfma gemm: K=%d is not a multiple of %d (use QLMX_MATH_F32)", K, bk);
        QLMX_REQUIRE(group >= bk && (group & (group - 1)) == 0, "mfma gemm: group %d must be a power of two >= %d (use QLMX_MATH_F32)", group, bk);
    }
    for(int i = 0; i < nprob; i++){
        QLMX_REQUIRE(((uintptr_t)probs[i].A & 15) == 0 && (mode != GEMM_NT || ((uintptr_t)probs[i].B & 15) == 0),
                     "mfma gemm: problem %d operand is not 16-byte aligned", i);
        QLMX_REQUIRE(mode == GEMM_NT || (probs[i].wq & 31ULL) == 0, "mfma gemm: problem %d weight offset not a multiple of 32", i);
        if(second && probs[i].M != 0){
            QLMX_REQUIRE(((uintptr_t)second[i].A & 15) == 0, "mfma gemm: problem %d continuation operand is not 16-byte aligned", i);
            QLMX_REQUIRE((second[i].wq & 31ULL) == 0, "mfma gemm: problem %d continuation weight offset not a multiple of 32", i);
        }
    }
    QLMX_REQUIRE(mode == GEMM_NT || ((uintptr_t)d & 15) == 0, "mfma gemm: digit array is not 16-byte aligned");
    /* bf16 operands take the direct-to-LDS kernels; fp32 activations need the converting ones */
    if(mode == GEMM_TN && act_dtype == QLMX_ACT_BF16) return qlmx_gemm_tn_lds_launch(d, s, group, probs, second, nprob, K, N, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, st);
    if(mode == GEMM_NT && act_dtype == QLMX_ACT_BF16) return qlmx_gemm_nt_lds_launch(probs, nprob, K, N, st);
    if(mode == GEMM_NN && act_dtype == QLMX_ACT_BF16 && f16) return qlmx_gemm_nn_h_launch(d, s, group, probs, nprob, K, N, 0, nullptr, nullptr, nullptr, st);
    if(mode == GEMM_NN && act_dtype == QLMX_ACT_BF16) return qlmx_gemm_nn_lds_launch(d, s, group, probs, nprob, K, N, st);
    if(mode == GEMM_NN) return launch_mfma<GEMM_NN, 4, true>(d, s, group, probs, nprob, K, N, act_dtype, st);
    if(mode == GEMM_TN) return launch_mfma<GEMM_TN, 2, false>(d, s, group, probs, nprob, K, N, act_dtype, st);
    return launch_mfma<GEMM_NT, 4, false>(d, s, group, probs, nprob, K, N, act_dtype, st);
}
