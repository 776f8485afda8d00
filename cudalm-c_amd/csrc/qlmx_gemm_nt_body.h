/* qlmx_gemm_nt_body.h -- device code of the weight-gradient grouped GEMM (nt) for bf16 operands, built on two gfx950
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
 *     that freedom is the XOR swizzle below), three tiles deep (four in the wide form), one barrier per step;
 *   * an MFMA operand is two ds_read_b64_tr_b16: within 16 lanes, lane i receives element (i & 3)
 *     of the 8-byte pieces addressed by lanes 4v + (i >> 2), v = 0..3; pointing lane 4v + q at
 *     (row r0 + v, columns c0 + 4q .. +3) therefore hands lane i the four consecutive rows
 *     r0 .. r0+3 of column c0 + i.
 * Swizzle: 16-byte unit u of tile row r is stored at unit u ^ 4*(r & 3). The four rows a transpose
 * read touches then fall into different quarters of the banks, so the reads are conflict-free.
 * Rows past the end of an expert are fetched from a zero block instead of being masked.
 */
#pragma once
#include "qlmx_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short  s16x4  __attribute__((ext_vector_type(4)));
typedef short  s16x8  __attribute__((ext_vector_type(8)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));

/* Two tile shapes, one kernel body (template parameters BN = columns of dY per tile, NW = wavefronts):
 *   256 x 128: four wavefronts of 128 x 64, two workgroups per CU (256 registers each), three tiles in LDS;
 *   256 x 256: eight wavefronts of 128 x 64, one workgroup per CU, four tiles in LDS (128 KB): a third fewer bytes
 *              brought into LDS per multiplication and a tile more on its way, but all eight wavefronts meet at one
 *              barrier per step, so the two on a SIMD read their operands at the same time instead of one
 *              multiplying while the other reads, and nothing else is resident to cover the prologue and the
 *              epilogue. Faster for experts of a few thousand rows, slower for short ones (see nt3_pick_bn); opt-in. */
#define NT3_BM 256
#define NT3_BK 32
#define NT3_A_BYTES (NT3_BK * NT3_BM * 2)      /* 16384 */
template<int BN, int NW> struct Nt3Shape {
    static constexpr int NT = NW * 64;                       /* threads */
    static constexpr int WN = NW / 2;                        /* wavefronts side by side along dY's columns (two along X's) */
    static constexpr int NJ = BN / (32 * WN);                /* 32-column accumulator tiles per wavefront */
    static constexpr int NA = NT3_A_BYTES / 16 / NT;         /* 16-byte pieces of X a thread fetches per tile */
    static constexpr int NB = NT3_BK * BN * 2 / 16 / NT;     /* and of dY */
    static constexpr int B_BYTES = NT3_BK * BN * 2;
    static constexpr int STAGE_BYTES = NT3_A_BYTES + B_BYTES;
    static constexpr int NREQ = NA + NB;                     /* requests per thread and tile */
    static constexpr int STAGES = NW == 8 ? 4 : 3;           /* tiles in LDS; STAGES - 1 of them on their way while one is multiplied */
    static constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static constexpr int WG_PER_CU = BN == 128 ? 2 : 1;
};

struct Nt3Args { const DevProb *pr; const DevUnit *units; int *flags; unsigned *status; unsigned epoch;
                 unsigned wait_epoch; int wait_limit;      /* what a slice waits for (= epoch) and for how many polls */
                 int nprob, ntiles, tiles_n, rows_p; int K, N; const void *zeros; };

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
template<int NJ> struct Nt3Ops { i32x2 a[4][2], b[NJ][2]; };
template<int KS, int BN, int NJ> __device__ __forceinline__ void nt3_read(Nt3Ops<NJ> &o, const uint32_t (&adA)[4], const uint32_t (&adB)[NJ]){
#pragma unroll
    for(int i = 0; i < 4; i++){
        o.a[i][0] = nt3_tr<KS * 16 * NT3_BM * 2>(adA[i]);
        o.a[i][1] = nt3_tr<KS * 16 * NT3_BM * 2 + 4 * NT3_BM * 2>(adA[i]);
    }
#pragma unroll
    for(int j = 0; j < NJ; j++){
        o.b[j][0] = nt3_tr<KS * 16 * BN * 2>(adB[j]);
        o.b[j][1] = nt3_tr<KS * 16 * BN * 2 + 4 * BN * 2>(adB[j]);
    }
}
__device__ __forceinline__ void nt3_wait_reads(Nt3Ops<2> &o){
    asm volatile("s_waitcnt lgkmcnt(0)"
        : "+v"(o.a[0][0]), "+v"(o.a[0][1]), "+v"(o.a[1][0]), "+v"(o.a[1][1]), "+v"(o.a[2][0]), "+v"(o.a[2][1]),
          "+v"(o.a[3][0]), "+v"(o.a[3][1]), "+v"(o.b[0][0]), "+v"(o.b[0][1]), "+v"(o.b[1][0]), "+v"(o.b[1][1]));
}
__device__ __forceinline__ bf16x8 nt3_pack(const i32x2 lo, const i32x2 hi){
    const i32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(bf16x8, v);
}

__device__ __forceinline__ int t_of(int b, const Nt3Args &a){
    return (a.rows_p & 7) ? qx_xcd_tile_probs(b, a.tiles_n, a.rows_p) : qx_xcd_tile_rows(b, a.tiles_n);
}

/* one workgroup's tile; bid = its index in the launch (the kernels below pass bid, the combined
 * backward launch the index counted from its first weight-gradient workgroup) */
template<int BN, int NW>
__device__ __forceinline__ void nt3_block(const Nt3Args &a, const unsigned bid){
    typedef Nt3Shape<BN, NW> SH;
    constexpr int NJ = SH::NJ, NA = SH::NA, NB = SH::NB, NT = SH::NT;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    /* scheduled launch: the unit table says what to do; otherwise the tile follows from the index */
    int pi, i0, j0, k0 = 0, depth = -1, seq = 0, nseq = 1, flag = 0;
    DevUnit u = QX_UNIT_NONE;
    if(a.units){
        /* one table entry per strip of tiles_n column tiles: workgroup 8k + x is column tile k % tiles_n
         * of entry k / tiles_n of XCD x */
        u = a.units[((bid >> 3) / a.tiles_n) * 8 + (bid & 7)];
        if(u == QX_UNIT_NONE) return;
        pi = (int)(u >> 22);
    } else {
        const int t = t_of(bid, a);
        if(t >= a.ntiles) return;
        pi = qx_find_problem(a.pr, a.nprob, t);
    }
    const DevProb P = a.pr[pi];
    if(a.units){
        const int ti = (u >> 16) & 63, tj = (int)(bid >> 3) % a.tiles_n;
        seq = (u >> 4) & 15; nseq = u & 15;
        i0 = ti * NT3_BM; j0 = tj * BN; k0 = seq * P.chunk;
        depth = P.M - k0 < P.chunk ? P.M - k0 : P.chunk;
        flag = P.flag0 + ti * P.tiles_n + tj;
    } else {
        const int lt = t_of(bid, a) - P.tile0;
        const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
        i0 = ti * NT3_BM; j0 = tj * BN; depth = P.M;
    }
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave / SH::WN) * 128, wj = (wave % SH::WN) * (BN / SH::WN);

    /* ---- what this thread fetches per tile: four 16-byte pieces of X, two of dY. Piece p of a tile
     * (LDS position 16*p) is row p/32 (p/16 for dY), stored unit p%32 = logical unit ^ swizzle. ---- */
    const char *srcA[NA]; const char *srcB[NB]; int rowA[NA], rowB[NB];
#pragma unroll
    for(int h = 0; h < NA; h++){
        const int p = h * NT + tid, row = p >> 5, lu = (p & 31) ^ ((row & 3) << 2);
        const int col = i0 + lu * 8;
        rowA[h] = row;
        srcA[h] = (const char *)P.A + ((size_t)(k0 + row) * a.K + (col < a.K ? col : 0)) * 2;   /* columns past K feed rows that are never stored */
    }
#pragma unroll
    for(int h = 0; h < NB; h++){
        const int p = h * NT + tid, row = p / (BN / 8), lu = (p & (BN / 8 - 1)) ^ ((row & 3) << 2);
        rowB[h] = row;
        srcB[h] = (const char *)P.B + ((size_t)(k0 + row) * a.N + j0 + lu * 8) * 2;
    }
    const size_t stepA = (size_t)NT3_BK * a.K * 2, stepB = (size_t)NT3_BK * a.N * 2;
    const int wave_off = __builtin_amdgcn_readfirstlane(wave * 1024);

    /* request h of a tile: 0..3 are the X pieces, 4..5 the dY pieces */
    auto issue_one = [&](int tile, int stage, int h){
        const int kt = tile * NT3_BK;
        unsigned char *base = lds + stage * SH::STAGE_BYTES + wave_off;
        if(h < NA){
            const char *g = (kt + rowA[h] < depth) ? srcA[h] + (size_t)tile * stepA : (const char *)a.zeros;
            __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(base + h * (NT * 16)), 16, 0, 0);
        } else {
            const char *g = (kt + rowB[h - NA] < depth) ? srcB[h - NA] + (size_t)tile * stepB : (const char *)a.zeros;
            __builtin_amdgcn_global_load_lds((glb_void *)g, (lds_void *)(base + NT3_A_BYTES + (h - NA) * (NT * 16)), 16, 0, 0);
        }
    };
    auto issue = [&](int tile, int stage){
#pragma unroll
        for(int h = 0; h < SH::NREQ; h++) issue_one(tile, stage, h);
    };

    /* ---- operand read addresses inside a stage (k16 slice 0; slice 1 is 16 rows further) ---- */
    const int g16 = lane >> 4, s16 = lane & 15, v = s16 >> 2, q = s16 & 3, khalf = g16 >> 1, chalf = g16 & 1;
    const int row0 = khalf * 8 + v;                         /* + 4 for the second read, + 16 for slice 1: row & 3 unchanged */
    const int sw = (row0 & 3) << 2;
    uint32_t offA[4], offB[NJ];
#pragma unroll
    for(int i = 0; i < 4; i++){
        const int col = wi + i * 32 + chalf * 16 + q * 4;
        offA[i] = row0 * (NT3_BM * 2) + ((((col >> 3) ^ sw)) << 4) + (col & 7) * 2;
    }
#pragma unroll
    for(int j = 0; j < NJ; j++){
        const int col = wj + j * 32 + chalf * 16 + q * 4;
        offB[j] = NT3_A_BYTES + row0 * (BN * 2) + ((((col >> 3) ^ sw)) << 4) + (col & 7) * 2;
    }

    f32x16 acc[4][NJ];
#pragma unroll
    for(int i = 0; i < 4; i++)
#pragma unroll
        for(int j = 0; j < NJ; j++) acc[i][j] = (f32x16)(0.0f);

    const int steps = (depth + NT3_BK - 1) / NT3_BK;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    constexpr int R0 = SH::NREQ / 2;                        /* requests issued behind the first slice's multiplications */
    auto addrs = [&](int st, uint32_t (&adA)[4], uint32_t (&adB)[NJ]){
        const uint32_t sb = lds_base + (uint32_t)(st % SH::STAGES) * SH::STAGE_BYTES;
#pragma unroll
        for(int i = 0; i < 4; i++) adA[i] = sb + offA[i];
#pragma unroll
        for(int j = 0; j < NJ; j++) adB[j] = sb + offB[j];
    };
#pragma unroll
    for(int t = 0; t < SH::STAGES - 1; t++) issue(t, t);
    for(int st = 0; st < steps; st++){
        /* tile st has landed once at most the requests of the STAGES - 2 tiles behind it are still in flight */
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"((SH::STAGES - 2) * SH::NREQ) : "memory");
        __builtin_amdgcn_s_barrier();                       /* everybody's pieces are in; the stage read in the step before is free again */
        uint32_t adA[4], adB[NJ];
        addrs(st, adA, adB);
        Nt3Ops<NJ> o0, o1;
        nt3_read<0, BN, NJ>(o0, adA, adB);
        nt3_wait_reads(o0);
        nt3_read<1, BN, NJ>(o1, adA, adB);                  /* in flight while slice 0 multiplies */
        /* The requests of tile st+2 go out between the multiplications, one after every row of them:
         * a request can wait a hundred cycles for the address unit when eight wavefronts ask at once, and
         * behind an MFMA that wait costs nothing. The fences keep the compiler from gathering them again. */
        const int nt = st + SH::STAGES - 1, ns = nt % SH::STAGES;
#pragma unroll
        for(int i = 0; i < 4; i++){
#pragma unroll
            for(int j = 0; j < NJ; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nt3_pack(o0.a[i][0], o0.a[i][1]), nt3_pack(o0.b[j][0], o0.b[j][1]), acc[i][j], 0, 0, 0);
            if(i < R0){ __builtin_amdgcn_sched_barrier(0); issue_one(nt, ns, i); __builtin_amdgcn_sched_barrier(0); }
        }
        nt3_wait_reads(o1);
#pragma unroll
        for(int i = 0; i < 4; i++){
#pragma unroll
            for(int j = 0; j < NJ; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(nt3_pack(o1.a[i][0], o1.a[i][1]), nt3_pack(o1.b[j][0], o1.b[j][1]), acc[i][j], 0, 0, 0);
            if(R0 + i < SH::NREQ){ __builtin_amdgcn_sched_barrier(0); issue_one(nt, ns, R0 + i); __builtin_amdgcn_sched_barrier(0); }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                    /* vmcnt(0), as a builtin so that the compiler knows it: no request may outlive the workgroup's LDS */

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int fr = lane & 31, hf = lane >> 5, row = i0 + wi + hf * 4;
    float *c = P.C + (size_t)row * a.N + (j0 + wj + fr);
    if(nseq == 1){
        qx_store_tiles<4, NJ>(acc, c, row, i0 + wi, a.K, (size_t)a.N, P.beta != 0.0f);
        return;
    }
    /* one slice of a split contraction: add to what the slices before have left, past the caches */
    if(seq > 0) qx_chain_wait(a.flags, flag, a.wait_epoch, seq, a.status, a.wait_limit);
    qx_store_tiles<4, NJ, true>(acc, c, row, i0 + wi, a.K, (size_t)a.N, seq > 0 || P.beta != 0.0f);
    if(seq + 1 < nseq) qx_chain_publish(a.flags, flag, a.epoch, seq);
}

