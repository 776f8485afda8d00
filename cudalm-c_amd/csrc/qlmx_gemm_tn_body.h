/* qlmx_gemm_tn_body.h -- device code of the input-gradient grouped GEMM (tn) for bf16 activations with the activation
 * tiles loaded straight into LDS.
 *
 * dX_e[M,N] (= or +=) dY_e[M,K] . W_e[N,K]^T   (mg_abt_b, cudalm.cu:3204-3256; call sites 4340-4366)
 * W_e[N,K] packed 4-bit, scale groups along K (the contraction), so the exact integer digits go to
 * the matrix core and no weight is rounded (see qlmx_gemm_mfma.hip for why).
 *
 * 256x128 output tile, 32-deep steps, four wavefronts 2x2 with 4x2 accumulators each -- the shape of the
 * forward and weight-gradient kernels, for the same reason: what a CU's loop waits for is its LDS, above all the
 * writes into it (about 70 bytes per cycle, against some 180 for reads), and per multiplication a 256x128 tile
 * receives and reads a quarter less than the 128x128 tile this kernel had.
 *
 * The scale of a group: the accumulators of a lane's column hold the sum in units of the CURRENT group's scale.
 * When the contraction enters the next group they are multiplied by old scale / new scale (one multiplication per
 * element and group, a reciprocal per column and group), and by the last scale at the end. A second set of
 * accumulators for the group's partial sum, folded in with an FMA per element and group, costs the same arithmetic
 * but 128 registers more, which the wide tile does not have. The scales are positive (absmax / dmax with a floor of
 * 1e-8), their ratios are formed with v_rcp_f32 (one unit in the last place), so a result carries one rounding of
 * about 2^-23 per group on top of the exact products: 3e-7 relative L2 over sixteen groups.
 *
 * Activations: each 16-byte piece goes from global memory into one of three LDS stages without touching a register
 * (lane l of a wave instruction lands at base + 16*l; rows of 64 bytes, piece ko of row r stored at position
 * ko ^ ((r >> 2) & 3), which makes the 128-bit operand reads conflict-free). Weights: 16 digits per thread and
 * step through registers, converted to bf16 (digit / 16, exact) and written to one of two LDS buffers a step ahead.
 * One barrier per step. LDS accesses and the register loads of the loop are inline assembly with explicit wait
 * counts: the compiler would otherwise wait for every outstanding load-to-LDS before any LDS access.
 */
#pragma once
#include "qlmx_gemm.h"
#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  f32x2  __attribute__((ext_vector_type(2)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));
typedef int    i32x2  __attribute__((ext_vector_type(2)));
typedef int    i32x4  __attribute__((ext_vector_type(4)));

#define TN3_BM 256
#define TN3_BN 128
#define TN3_BK 32
#define TN3_A_BYTES (TN3_BM * TN3_BK * 2)     /* 16384 */
#define TN3_B_BYTES (TN3_BN * TN3_BK * 2)     /*  8192 */
#define TN3_A_STAGES 3
#define TN3_B_OFF (TN3_A_STAGES * TN3_A_BYTES)  /* 49152; the second weight buffer ends at 65535, the largest immediate offset */

/* a continued problem: number of operand pairs (1 or 2) and where the second pair's activations (bytes),
 * digits (bytes) and scales (floats) lie relative to the first's */
struct Tn3Seg { int nseg; long long dA, dW, dS; };
/* out != NULL: the problems' C fields are row-index lists and the result is added to the indexed rows of `out`
 * (k_scatter_add4 behind the paired input-gradient GEMMs, cudalm.cu:4365-4367), see qx_scatter_tiles */
/* gp != NULL: k_swiglu_bwd behind the down projection's input gradient (cudalm.cu:4340-4346): the product is d(act);
 * a problem's C field points at its rows of gp, and up, dg, du hold the same rows at the same element offset */
struct Tn3Args { const DevProb *pr; int nprob, ntiles, nfull, tiles_n; const signed char *d; const float *s; int gshift; int K, N; float *out; const float *gate;
                 const float *gp, *up; unsigned short *dg, *du; };

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;

__device__ __forceinline__ uint32_t tn3_pk(float lo, float hi){
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
template<int OFF> __device__ __forceinline__ i32x4 tn3_rd(uint32_t addr){
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template<int OFF> __device__ __forceinline__ void tn3_wr(uint32_t addr, i32x4 v){
    asm volatile("ds_write_b128 %0, %1 offset:%2" :: "v"(addr), "v"(v), "n"(OFF) : "memory");
}
/* Register loads of the loop are inline assembly as well, and the step's wait names their
 * destinations as in/out operands: the compiler then neither adds a wait of its own (it would be
 * vmcnt(0) at the loop head, which also waits for the activation tile requested last) nor moves a
 * use of the loaded values above the wait. */
__device__ __forceinline__ i32x2 tn3_gld8(const void *p){
    i32x2 v;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ float tn3_gld4(const void *p){
    float v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
struct Tn3Ops { i32x4 a[4], b[2]; };
__device__ __forceinline__ void tn3_wait(Tn3Ops &o){
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o.a[0]), "+v"(o.a[1]), "+v"(o.a[2]), "+v"(o.a[3]), "+v"(o.b[0]), "+v"(o.b[1]));
}

/* One output tile of NI*64 rows: the four wavefronts 2x2, each NI x 2 accumulators. NI = 4 is the full tile; the
 * last tile of a problem takes the smallest NI that holds its rows. */
template<int NI>
__device__ __forceinline__ void tn3_tile(const Tn3Args &a, const DevProb &P, const Tn3Seg &sg, int i0, int j0, unsigned char *lds){
    const int rows = P.M;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (NI * 32), wj = (wave & 1) * 64;
    const int fr = lane & 31, hf = lane >> 5;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;

    /* ---- activation pieces of this thread: position p = h*256 + tid of a stage is row p/4, stored
     * piece p%4 = ko ^ ((row >> 2) & 3) ---- */
    const char *srcA[NI];
#pragma unroll
    for(int h = 0; h < NI; h++){
        const int p = h * 256 + tid, r = p >> 2, ko = (p & 3) ^ ((r >> 2) & 3);
        const int rr = (i0 + r < rows) ? i0 + r : rows - 1;               /* clamp: feeds unstored rows only */
        srcA[h] = (const char *)P.A + ((size_t)rr * a.K + ko * 8) * 2;
    }
    const int wave_off = __builtin_amdgcn_readfirstlane(wave * 1024);
    /* steps of one operand pair, and of the whole contraction; step T of a continued problem reads the
     * second pair's operands, which lie a constant distance from the first's */
    const int steps1 = a.K / TN3_BK, steps = steps1 * sg.nseg;
    auto off_a = [&](int T) -> long long { return T < steps1 ? (long long)T * (TN3_BK * 2) : (long long)(T - steps1) * (TN3_BK * 2) + sg.dA; };
    auto off_w = [&](int T) -> long long { return T < steps1 ? (long long)T * (TN3_BK / 2) : (long long)(T - steps1) * (TN3_BK / 2) + sg.dW; };
    auto issue_a = [&](int tile, int stage){
        const int tl = tile < steps ? tile : steps - 1;                   /* past the end: the last tile again, into a stage nobody reads */
        const long long oa = off_a(tl);
        unsigned char *base = lds + stage * TN3_A_BYTES + wave_off;
#pragma unroll
        for(int h = 0; h < NI; h++)
            __builtin_amdgcn_global_load_lds((glb_void *)(srcA[h] + oa), (lds_void *)(base + h * 4096), 16, 0, 0);
    };

    /* ---- weights: thread = (row n, half of the step's 32 digits); its two 16-byte units ko = 2*whalf, 2*whalf+1 ---- */
    const int wn = tid & 127, whalf = tid >> 7;
    const signed char *pw = a.d + ((P.wq + (size_t)(j0 + wn) * a.K) >> 1) + whalf * 8;
    uint32_t wp[2];
#pragma unroll
    for(int j = 0; j < 2; j++){
        const int ko = whalf * 2 + j;
        wp[j] = lds_base + (uint32_t)(ko * TN3_BN + (wn ^ ((ko << 1) & 15))) * 16;
    }
    auto load_w = [&](int tile) -> i32x2 {
        const int tl = tile < steps ? tile : steps - 1;                   /* past the end: re-read the last one, never used */
        return tn3_gld8(pw + off_w(tl));
    };
    auto dequant_unit = [&](uint32_t digits) -> i32x4 {
        const QxNibs nb = qx_nibs(digits);
        i32x4 v;
        v[0] = (int)tn3_pk(qx_nib16(nb, 0), qx_nib16(nb, 1));
        v[1] = (int)tn3_pk(qx_nib16(nb, 2), qx_nib16(nb, 3));
        v[2] = (int)tn3_pk(qx_nib16(nb, 4), qx_nib16(nb, 5));
        v[3] = (int)tn3_pk(qx_nib16(nb, 6), qx_nib16(nb, 7));
        return v;
    };

    /* ---- operand read addresses, stage / buffer 0; the stage, the buffer and the second column tile go into
     * the instructions' immediate offsets (the loop is unrolled over the six combinations of stage and buffer) ---- */
    uint32_t ra[2][NI], rb[2];
#pragma unroll
    for(int i = 0; i < NI; i++){
        const int r = wi + i * 32 + fr, f = (r >> 2) & 3;
#pragma unroll
        for(int ks = 0; ks < 2; ks++) ra[ks][i] = lds_base + (uint32_t)(r * 64 + (((ks * 2 + hf) ^ f) << 4));
    }
    {
        const int n = wj + fr;                                            /* column n + 32 shares the swizzle */
#pragma unroll
        for(int ks = 0; ks < 2; ks++){
            const int ko = ks * 2 + hf;
            rb[ks] = lds_base + (uint32_t)(ko * TN3_BN + (n ^ ((ko << 1) & 15))) * 16;
        }
    }

    /* ---- fp32 scale of (this lane's output column, scale group) ---- */
    const int ngroups = a.K >> a.gshift, sshift = a.gshift - 5, spg = 1 << sshift;     /* steps per scale group: a power of two */
    const float *pfold[2];
#pragma unroll
    for(int j = 0; j < 2; j++) pfold[j] = a.s + P.wg + (size_t)(j0 + wj + j * 32 + fr) * ngroups;
    auto load_scale = [&](int step, int j) -> float {
        int g = step >> sshift; g = g < ngroups * sg.nseg ? g : ngroups * sg.nseg - 1;
        const long long og = g < ngroups ? (long long)g : (long long)(g - ngroups) + sg.dS;
        return tn3_gld4(pfold[j] + og);
    };

    f32x16 acc[NI][2];
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.0f);

    /* ---- prologue: digits of step 0 into buffer 0, those of step 1 into registers, the scales of
     * step 0; all requests go out before the one wait ---- */
    float fs_cur[2], fs_new[2];
    i32x2 wcur;
    {
        i32x2 w0 = load_w(0);
        wcur = load_w(1);
        float f0 = load_scale(0, 0), f1 = load_scale(0, 1);
        issue_a(0, 0);
        issue_a(1, 1);
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w0), "+v"(wcur), "+v"(f0), "+v"(f1) : "n"(2 * NI) : "memory");
        tn3_wr<TN3_B_OFF>(wp[0], dequant_unit((uint32_t)w0[0]));
        tn3_wr<TN3_B_OFF>(wp[1], dequant_unit((uint32_t)w0[1]));
        fs_cur[0] = f0; fs_cur[1] = f1; fs_new[0] = f0; fs_new[1] = f1;
        asm volatile("s_waitcnt vmcnt(%0)" :: "n"(NI) : "memory");         /* tile 0 is in; tile 1 may still be on its way */
    }

    /* Main loop. A wavefront issues in order, and an MFMA of this shape keeps the vector ALU to itself
     * for about half of its 32 cycles: some four ALU instructions behind an MFMA cost nothing, every
     * further one its full four cycles, a memory request more, and whatever stands after the last MFMA
     * of a step runs alone. Everything else of a step is therefore cut into items and dealt evenly
     * into the gaps after the MFMAs, fences keeping the compiler from gathering them again:
     *   the load of the digits of step st+2 and, in a group's last step, of the next group's scales (waited for at
     *     the end of the step, when they have long arrived: an asynchronously loaded register must not be carried
     *     round the loop before its wait) and the activation requests of tile st+2,
     *   the conversion of the digits of step st+1 (wcur) to bf16, four digits per item, each 16-byte
     *     unit written to the buffer last read in step st-1 as soon as it is complete.
     * In the first step of a group the accumulators move to the new group's scale while the step's first operand
     * reads are on their way. */
    constexpr int SLOTS = NI * 4, ITEMS = 3 + NI + 4 + 2;
    long long oa2 = off_a(2 < steps ? 2 : steps - 1), ow2 = off_w(2 < steps ? 2 : steps - 1);
    const long long jump_a = sg.dA - (long long)steps1 * (TN3_BK * 2), jump_w = sg.dW - (long long)steps1 * (TN3_BK / 2);
    auto step = [&](auto STGC, auto PARC, int st){
        constexpr int STG = decltype(STGC)::value, PAR = decltype(PARC)::value;
        constexpr int RA = STG * TN3_A_BYTES, RB = TN3_B_OFF + PAR * TN3_B_BYTES, WB = TN3_B_OFF + (1 - PAR) * TN3_B_BYTES;
        constexpr int STG2 = (STG + 2) % TN3_A_STAGES;
        /* tile st is in (the wait at the end of the step before covers it), own LDS writes are done */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        const bool fresh = (st & (spg - 1)) == 0 && st > 0, last = ((st + 1) & (spg - 1)) == 0;
        i32x2 wnext; float fn[2];
        i32x4 wv[2];
        QxNibs nb[2];
        auto item = [&](int k){
            if(k == 0)      wnext = tn3_gld8(pw + ow2);
            else if(k < 3){ if(last) fn[k - 1] = load_scale(st + 1, k - 1); else fn[k - 1] = fs_new[k - 1]; }   /* a new scale only where a group ends */
            else if(k < 3 + NI)
                __builtin_amdgcn_global_load_lds((glb_void *)(srcA[k - 3] + oa2),
                                                 (lds_void *)(lds + STG2 * TN3_A_BYTES + wave_off + (k - 3) * 4096), 16, 0, 0);
            else if(k < 3 + NI + 4){
                const int q = k - 3 - NI, j = q >> 1, h = q & 1;
                if(h == 0) nb[j] = qx_nibs((uint32_t)wcur[j]);
                wv[j][2 * h]     = (int)tn3_pk(qx_nib16(nb[j], 4 * h),     qx_nib16(nb[j], 4 * h + 1));
                wv[j][2 * h + 1] = (int)tn3_pk(qx_nib16(nb[j], 4 * h + 2), qx_nib16(nb[j], 4 * h + 3));
            } else tn3_wr<WB>(wp[k - 3 - NI - 4], wv[k - 3 - NI - 4]);
        };
        Tn3Ops o0, o1;
        if(NI < 4){                                        /* the wait names all four; the spare ones hold nothing */
#pragma unroll
            for(int i = NI; i < 4; i++){ o0.a[i] = (i32x4)(0); o1.a[i] = (i32x4)(0); }
        }
#define TN3_READ(O, KS)                                                                                   \
        _Pragma("unroll")                                                                                 \
        for(int i = 0; i < NI; i++) O.a[i] = tn3_rd<RA>(ra[KS][i]);                                       \
        O.b[0] = tn3_rd<RB>(rb[KS]); O.b[1] = tn3_rd<RB + 32 * 16>(rb[KS]);
#define TN3_MMA(O, BLOCK)                                                                                 \
        _Pragma("unroll")                                                                                 \
        for(int m = 0; m < NI * 2; m++){                                                                  \
            const int i = m >> 1, j = m & 1;                                                              \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, O.a[i]), __builtin_bit_cast(bf16x8, O.b[j]), acc[i][j], 0, 0, 0); \
            {                                                                                             \
                const int slot = BLOCK * (SLOTS / 2) + m;                                                 \
                __builtin_amdgcn_sched_barrier(0);                                                        \
                _Pragma("unroll")                                                                         \
                for(int k = slot * ITEMS / SLOTS; k < (slot + 1) * ITEMS / SLOTS; k++) item(k);           \
                __builtin_amdgcn_sched_barrier(0);                                                        \
            }                                                                                             \
        }
        TN3_READ(o0, 0)
        if(fresh){
            /* a new scale group begins: the sums so far, held in units of the old scale, move to the new one */
#pragma unroll
            for(int j = 0; j < 2; j++){
                const float ratio = fs_cur[j] * __builtin_amdgcn_rcpf(fs_new[j]);
#pragma unroll
                for(int i = 0; i < NI; i++) acc[i][j] = acc[i][j] * ratio;
                fs_cur[j] = fs_new[j];
            }
        }
        tn3_wait(o0);
        TN3_READ(o1, 1)                                    /* in flight while slice 0 multiplies */
        TN3_MMA(o0, 0)
        tn3_wait(o1);
        TN3_MMA(o1, 1)
#undef TN3_READ
#undef TN3_MMA
        /* the digits of step st+2 and the next group's scales have arrived (only the activation requests are younger) */
        asm volatile("s_waitcnt vmcnt(%3)" : "+v"(wnext), "+v"(fn[0]), "+v"(fn[1]) : "n"(NI) : "memory");
        wcur = wnext;
        fs_new[0] = fn[0]; fs_new[1] = fn[1];
        if(st + 3 < steps){
            oa2 += TN3_BK * 2; ow2 += TN3_BK / 2;
            if(st + 3 == steps1){ oa2 += jump_a; ow2 += jump_w; }       /* on to the second operand pair */
        }
    };
    {
        typedef std::integral_constant<int, 0> I0; typedef std::integral_constant<int, 1> I1; typedef std::integral_constant<int, 2> I2;
        int st = 0;
        for(; st + 6 <= steps; st += 6){
            step(I0(), I0(), st);     step(I1(), I1(), st + 1); step(I2(), I0(), st + 2);
            step(I0(), I1(), st + 3); step(I1(), I0(), st + 4); step(I2(), I1(), st + 5);
        }
        if(st < steps){ step(I0(), I0(), st); st++; }
        if(st < steps){ step(I1(), I1(), st); st++; }
        if(st < steps){ step(I2(), I0(), st); st++; }
        if(st < steps){ step(I0(), I1(), st); st++; }
        if(st < steps){ step(I1(), I0(), st); st++; }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                    /* vmcnt(0), as a builtin so that the compiler knows it: no request may outlive the workgroup's LDS */

    /* the sums are in units of the last group's scale; the matrix core was fed digit / 16, so the scale carries the 16 */
#pragma unroll
    for(int j = 0; j < 2; j++){
        const float f = fs_cur[j] * 16.0f;
#pragma unroll
        for(int i = 0; i < NI; i++) acc[i][j] = acc[i][j] * f;
    }

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int row = i0 + wi + hf * 4;
    if(a.out) qx_scatter_tiles<NI>(acc, (const int *)P.C, a.gate, a.out, row, rows, (size_t)a.N, j0 + wj + fr);
    else if(a.gp){
        const size_t o = (size_t)(P.C - a.gp) + (size_t)row * a.N + (j0 + wj + fr);
        qx_store_swiglu_bwd<NI>(acc, a.gp + o, a.up + o, a.dg + o, a.du + o, row, rows, (size_t)a.N);
    } else qx_store_tiles<NI, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, rows, (size_t)a.N, P.beta != 0.0f);
}

/* one workgroup's tile; bid = its index in the launch */
__device__ __forceinline__ void tn3_block(const Tn3Args &a, const unsigned bid, unsigned char *lds){
    const int t = qx_lpt_tile(bid, a.nfull, a.ntiles, a.tiles_n);
    if(t >= a.ntiles) return;
    const int pi = qx_find_problem(a.pr, a.nprob, t);
    const DevProb P = a.pr[pi];
    Tn3Seg sg; sg.nseg = 1; sg.dA = 0; sg.dW = 0; sg.dS = 0;
    if(P.chunk){
        const DevProb Q = a.pr[pi + 1];
        sg.nseg = 2;
        sg.dA = (long long)((const char *)Q.A - (const char *)P.A);
        sg.dW = ((long long)Q.wq - (long long)P.wq) / 2;
        sg.dS = (long long)Q.wg - (long long)P.wg;
    }
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * TN3_BM, j0 = tj * TN3_BN, left = P.M - i0;
    if(left > 192)      tn3_tile<4>(a, P, sg, i0, j0, lds);
    else if(left > 128) tn3_tile<3>(a, P, sg, i0, j0, lds);
    else if(left > 64)  tn3_tile<2>(a, P, sg, i0, j0, lds);
    else                tn3_tile<1>(a, P, sg, i0, j0, lds);
}

#define TN3_LDS_BYTES (TN3_A_STAGES * TN3_A_BYTES + 2 * TN3_B_BYTES)
