/* qlmx_gemm_nt_lds.hip -- weight-gradient grouped GEMM (nt) for bf16 operands, built on two gfx950
 * features: global loads that write straight into LDS, and LDS reads that transpose 16-bit elements.
 *
 * G_e[K,N] (+)= X_e[M,K]^T . dY_e[M,N]   (mg_atb, cudalm.cu:3204-3256; call sites 4334-4366)
 *
 * Both operands are row-major with the contraction index M as the row index, while the matrix core
 * wants, per lane, 8 consecutive contraction elements of one output row or column. The general
 * kernel transposes on the way into LDS (register staging, byte permutes, 4-byte stores that hit the
 * same bank twice). Here a tile keeps its global layout in LDS -- 32 rows of M, 256 columns of X and
 * 128 of dY -- so that
 *   * every 16-byte piece goes from global memory to LDS without passing through registers
 *     (lane l of a wave instruction lands at base + 16*l; which piece a lane fetches is free, and
 *     that freedom is the XOR swizzle below), three tiles deep, one barrier per step;
 *   * an MFMA operand is two ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i & 3)
 *     of the 8-byte pieces addressed by lanes 4v + (i >> 2), v = 0..3; pointing lane 4v + q at
 *     (row r0 + v, columns c0 + 4q .. +3) therefore hands lane i the four consecutive rows
 *     r0 .. r0+3 of column c0 + i.
 * Swizzle: 16-byte unit u of tile row r is stored at unit u ^ 4*(r & 3). The four rows a transpose
 * read touches then fall into different quarters of the banks, so the reads are conflict-free.
 * Rows past the end of an expert are fetched from a zero block instead of being masked.
 */
#include "qlmx_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short  s16x4  __attribute__((ext_vector_type(4)));
typedef short  s16x8  __attribute__((ext_vector_type(8)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));

#define NT3_BM 256
#define NT3_BN 128
#define NT3_BK 32
#define NT3_STAGES 3
#define NT3_A_BYTES (NT3_BK * NT3_BM * 2)      /* 16384 */
#define NT3_B_BYTES (NT3_BK * NT3_BN * 2)      /*  8192 */
#define NT3_STAGE_BYTES (NT3_A_BYTES + NT3_B_BYTES)

struct Nt3Args { const DevProb *pr; int nprob, ntiles, tiles_n, rows_p; int K, N; const void *zeros; };

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;

/* The transposing LDS reads and the waits that order them are written as inline assembly. The
 * compiler treats a load-to-LDS as a store to all of LDS and, left to itself, puts vmcnt(0) in front
 * of the first LDS read after one -- which would make every step wait for the tile it has just
 * requested. Here the only wait on outstanding loads is the explicit one at the top of a step, which
 * still allows the next tile's six requests to be in flight. Each read leaves 4 bf16 in a register
 * pair; the wait takes the pairs as in/out operands so that nothing that uses them can move above it. */
typedef int i32x2 __attribute__((ext_vector_type(2)));
typedef int i32x4 __attribute__((ext_vector_type(4)));
template<int OFF> __device__ __forceinline__ i32x2 nt3_tr(uint32_t addr){
    i32x2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
struct Nt3Ops { i32x2 a[4][2], b[2][2]; };
template<int KS> __device__ __forceinline__ void nt3_read(Nt3Ops &o, const uint32_t (&adA)[4], const uint32_t (&adB)[2]){
#pragma unroll
    for(int i = 0; i < 4; i++){
        o.a[i][0] = nt3_tr<KS * 16 * NT3_BM * 2>(adA[i]);
        o.a[i][1] = nt3_tr<KS * 16 * NT3_BM * 2 + 4 * NT3_BM * 2>(adA[i]);
    }
#pragma unroll
    for(int j = 0; j < 2; j++){
        o.b[j][0] = nt3_tr<KS * 16 * NT3_BN * 2>(adB[j]);
        o.b[j][1] = nt3_tr<KS * 16 * NT3_BN * 2 + 4 * NT3_BN * 2>(adB[j]);
    }
}
__device__ __forceinline__ void nt3_wait_reads(Nt3Ops &o){
    asm volatile("s_waitcnt lgkmcnt(0)"
        : "+v"(o.a[0][0]), "+v"(o.a[0][1]), "+v"(o.a[1][0]), "+v"(o.a[1][1]), "+v"(o.a[2][0]), "+v"(o.a[2][1]),
          "+v"(o.a[3][0]), "+v"(o.a[3][1]), "+v"(o.b[0][0]), "+v"(o.b[0][1]), "+v"(o.b[1][0]), "+v"(o.b[1][1]));
}
__device__ __forceinline__ bf16x8 nt3_pack(const i32x2 lo, const i32x2 hi){
    const i32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(bf16x8, v);
}

__global__ void __launch_bounds__(256, 2) k_gemm_nt_lds(Nt3Args a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[NT3_STAGES * NT3_STAGE_BYTES];
    const int t = (a.rows_p & 7) ? qx_xcd_tile_probs(blockIdx.x, a.tiles_n, a.rows_p) : qx_xcd_tile_rows(blockIdx.x, a.tiles_n);
    if(t >= a.ntiles) return;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * NT3_BM, j0 = tj * NT3_BN;
    const int depth = P.M;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * 128, wj = (wave & 1) * 64;

    /* ---- what this thread fetches per tile: four 16-byte pieces of X, two of dY. Piece p of a tile
     * (LDS position 16*p) is row p/32 (p/16 for dY), stored unit p%32 = logical unit ^ swizzle. ---- */
    const char *srcA[4]; const char *srcB[2]; int rowA[4], rowB[2];
#pragma unroll
    for(int h = 0; h < 4; h++){
        const int p = h * 256 + tid, row = p >> 5, lu = (p & 31) ^ ((row & 3) << 2);
        const int col = i0 + lu * 8;
        rowA[h] = row;
        srcA[h] = (const char *)P.A + ((size_t)row * a.K + (col < a.K ? col : 0)) * 2;   /* columns past K feed rows that are never stored */
    }
#pragma unroll
    for(int h = 0; h < 2; h++){
        const int p = h * 256 + tid, row = p >> 4, lu = (p & 15) ^ ((row & 3) << 2);
        rowB[h] = row;
        srcB[h] = (const char *)P.B + ((size_t)row * a.N + j0 + lu * 8) * 2;
    }
    const size_t stepA = (size_t)NT3_BK * a.K * 2, stepB = (size_t)NT3_BK * a.N * 2;
    const int wave_off = __builtin_amdgcn_readfirstlane(wave * 1024);

    /* request h of a tile: 0..3 are the X pieces, 4..5 the dY pieces */
    auto issue_one = [&](int tile, int stage, int h){
        const int k0 = tile * NT3_BK;
        unsigned char *base = lds + stage * NT3_STAGE_BYTES + wave_off;
        if(h < 4){
            const char *g = (k0 + rowA[h] < depth) ? srcA[h] + (size_t)tile * stepA : (const char *)a.zeros;
            __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(base + h * 4096), 16, 0, 0);
        } else {
            const char *g = (k0 + rowB[h - 4] < depth) ? srcB[h - 4] + (size_t)tile * stepB : (const char *)a.zeros;
            __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(base + NT3_A_BYTES + (h - 4) * 4096), 16, 0, 0);
        }
    };
    auto issue = [&](int tile, int stage){
#pragma unroll
        for(int h = 0; h < 6; h++) issue_one(tile, stage, h);
    };

    /* ---- operand read addresses inside a stage (k16 slice 0; slice 1 is 16 rows further) ---- */
    const int g16 = lane >> 4, s16 = lane & 15, v = s16 >> 2, q = s16 & 3, khalf = g16 >> 1, chalf = g16 & 1;
    const int row0 = khalf * 8 + v;                         /* + 4 for the second read, + 16 for slice 1: row & 3 unchanged */
    const int sw = (row0 & 3) << 2;
    uint32_t offA[4], offB[2];
#pragma unroll
    for(int i = 0; i < 4; i++){
        const int col = wi + i * 32 + chalf * 16 + q * 4;
        offA[i] = row0 * (NT3_BM * 2) + ((((col >> 3) ^ sw)) << 4) + (col & 7) * 2;
    }
#pragma unroll
    for(int j = 0; j < 2; j++){
        const int col = wj + j * 32 + chalf * 16 + q * 4;
        offB[j] = NT3_A_BYTES + row0 * (NT3_BN * 2) + ((((col >> 3) ^ sw)) << 4) + (col & 7) * 2;
    }

    f32x16 acc[4][2];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.0f);

    const int steps = (depth + NT3_BK - 1) / NT3_BK;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    issue(0, 0);
    issue(1, 1);
    for(int st = 0; st < steps; st++){
        /* tile st has landed once at most the 6 requests of tile st+1 are still in flight */
        asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
        __builtin_amdgcn_s_barrier();                       /* everybody's pieces are in; stage (st+2)%3 is free again */
        const uint32_t sb = lds_base + (uint32_t)(st % NT3_STAGES) * NT3_STAGE_BYTES;
        uint32_t adA[4], adB[2];
#pragma unroll
        for(int i = 0; i < 4; i++) adA[i] = sb + offA[i];
#pragma unroll
        for(int j = 0; j < 2; j++) adB[j] = sb + offB[j];
        Nt3Ops o0, o1;
        nt3_read<0>(o0, adA, adB);
        nt3_wait_reads(o0);
        nt3_read<1>(o1, adA, adB);                          /* in flight while slice 0 multiplies */
        /* The six requests of tile st+2 go out between the multiplications, one after every other
         * MFMA: a request can wait a hundred cycles for the address unit when eight wavefronts ask at
         * once, and behind an MFMA that wait costs nothing. The fences keep the compiler from
         * gathering them again. */
        const int nt = st + 2, ns = (st + 2) % NT3_STAGES;
#pragma unroll
        for(int i = 0; i < 4; i++){
#pragma unroll
            for(int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nt3_pack(o0.a[i][0], o0.a[i][1]), nt3_pack(o0.b[j][0], o0.b[j][1]), acc[i][j], 0, 0, 0);
            if(i < 3){ __builtin_amdgcn_sched_barrier(0); issue_one(nt, ns, i); __builtin_amdgcn_sched_barrier(0); }
        }
        nt3_wait_reads(o1);
#pragma unroll
        for(int i = 0; i < 4; i++){
#pragma unroll
            for(int j = 0; j < 2; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nt3_pack(o1.a[i][0], o1.a[i][1]), nt3_pack(o1.b[j][0], o1.b[j][1]), acc[i][j], 0, 0, 0);
            if(i < 3){ __builtin_amdgcn_sched_barrier(0); issue_one(nt, ns, 3 + i); __builtin_amdgcn_sched_barrier(0); }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                    /* vmcnt(0), as a builtin so that the compiler knows it: no request may outlive the workgroup's LDS */

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int fr = lane & 31, hf = lane >> 5, row = i0 + wi + hf * 4;
    qx_store_tiles<4, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, a.K, (size_t)a.N, P.beta != 0.0f);
}

static void *g_nt3_zeros = nullptr;

/* bf16 operands only; N % 128 == 0, K % 8 == 0, operands 16-byte aligned (checked by the caller) */
int qlmx_gemm_nt_lds_launch(const qlmx_gemm_prob *probs, int nprob, int K, int N, hipStream_t st){
    if(!g_nt3_zeros){
        QLMX_HIP(hipMalloc(&g_nt3_zeros, 256), "nt zero block");
        QLMX_HIP(hipMemset(g_nt3_zeros, 0, 256), "nt zero block clear");
    }
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, GEMM_NT, K, N, NT3_BM, NT3_BN, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Nt3Args a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.tiles_n = N / NT3_BN; a.K = K; a.N = N; a.zeros = g_nt3_zeros;
    a.rows_p = up.ntiles / (a.tiles_n * up.nprob);
    int grid;
    if(a.rows_p & 7) grid = 8 * a.tiles_n * a.rows_p * ((up.nprob + 7) / 8);
    else             grid = 8 * a.tiles_n * ((up.ntiles / a.tiles_n + 7) / 8);
    hipLaunchKernelGGL(k_gemm_nt_lds, dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm nt (direct-to-LDS) launch");
    return qlmx_upload_done(slot, st);
}
