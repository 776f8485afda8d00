/* qlmx_gemm_tn_lds.hip -- input-gradient grouped GEMM (tn) for bf16 activations with the activation
 * tiles loaded straight into LDS.
 *
 * dX_e[M,N] (= or +=) dY_e[M,K] . W_e[N,K]^T   (mg_abt_b, cudalm.cu:3204-3256; call sites 4340-4366)
 * W_e[N,K] packed 4-bit, scale groups along K (the contraction), so the exact integer digits go to
 * the matrix core and every 128-deep partial sum is folded in with its fp32 scale (see
 * qlmx_gemm_mfma.hip for why).
 *
 * 128x128 output tile, 64-deep steps, four wavefronts 2x2 with 2x2 accumulators each (plus the
 * per-group partial sums). Activations: each 16-byte piece goes from global memory into one of three
 * LDS stages without touching a register (lane l of a wave instruction lands at base + 16*l; the
 * rows keep their global order, 8 pieces = 128 bytes per row, piece ko of row r stored at position
 * ko ^ ((r >> 1) & 7), which makes the MFMA operand reads conflict-free). Weights: 32 digits per
 * thread and step through registers, converted to bf16 and written to one of two LDS buffers a step
 * ahead. One barrier per step; the wait in front of it lets the activation tile requested last stay
 * in flight. LDS accesses in the loop are inline assembly: the compiler would otherwise wait for
 * every outstanding load-to-LDS before any LDS access.
 */
#include "qlmx_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  f32x2  __attribute__((ext_vector_type(2)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));
typedef int    i32x4  __attribute__((ext_vector_type(4)));

#define TN3_BM 128
#define TN3_BN 128
#define TN3_BK 64
#define TN3_A_BYTES (TN3_BM * TN3_BK * 2)     /* 16384 */
#define TN3_B_BYTES (TN3_BN * TN3_BK * 2)     /* 16384 */
#define TN3_A_STAGES 3
#define TN3_B_OFF (TN3_A_STAGES * TN3_A_BYTES)

/* a continued problem: number of operand pairs (1 or 2) and where the second pair's activations (bytes),
 * digits (bytes) and scales (floats) lie relative to the first's */
struct Tn3Seg { int nseg; long long dA, dW, dS; };
/* out != NULL: the problems' C fields are row-index lists and the result is added to the indexed rows of `out`
 * (k_scatter_add4 behind the paired input-gradient GEMMs, cudalm.cu:4365-4367), see qx_scatter_tiles */
/* gp != NULL: k_swiglu_bwd behind the down projection's input gradient (cudalm.cu:4340-4346): the product is d(act);
 * a problem's C field points at its rows of gp, and up, dg, du hold the same rows at the same element offset */
struct Tn3Args { const DevProb *pr; int nprob, ntiles; const signed char *d; const float *s; int gshift; int K, N; float *out; const float *gate;
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
__device__ __forceinline__ void tn3_wr(uint32_t addr, i32x4 v){
    asm volatile("ds_write_b128 %0, %1" :: "v"(addr), "v"(v) : "memory");
}
/* Register loads of the loop are inline assembly as well, and the step's wait names their
 * destinations as in/out operands: the compiler then neither adds a wait of its own (it would be
 * vmcnt(0) at the loop head, which also waits for the activation tile requested last) nor moves a
 * use of the loaded values above the wait. */
__device__ __forceinline__ i32x4 tn3_gld16(const void *p){
    i32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ float tn3_gld4(const void *p){
    float v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
struct Tn3Ops { i32x4 a[2], b[2]; };
__device__ __forceinline__ void tn3_wait(Tn3Ops &o){
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(o.a[0]), "+v"(o.a[1]), "+v"(o.b[0]), "+v"(o.b[1]));
}

/* One output tile of NI*64 rows: the four wavefronts 2x2, each NI x 2 accumulators. NI = 2 is the
 * full tile; a last tile with at most 64 rows does half the work. */
template<int NI>
__device__ __forceinline__ void tn3_tile(const Tn3Args &a, const DevProb &P, const Tn3Seg &sg, int i0, int j0, unsigned char *lds){
    const int rows = P.M;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (NI * 32), wj = (wave & 1) * 64;
    const int fr = lane & 31, hf = lane >> 5;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;

    /* ---- activation pieces of this thread: position p = h*256 + tid of a stage is row p/8, stored
     * piece p%8 = ko ^ ((row >> 1) & 7) ---- */
    const char *srcA[2 * NI];
#pragma unroll
    for(int h = 0; h < 2 * NI; h++){
        const int p = h * 256 + tid, r = p >> 3, ko = (p & 7) ^ ((r >> 1) & 7);
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
        for(int h = 0; h < 2 * NI; h++)
            __builtin_amdgcn_global_load_lds((glb_void *)(srcA[h] + oa), (lds_void *)(base + h * 4096), 16, 0, 0);
    };

    /* ---- weights: thread = (row n, half of the step's 64 digits) ---- */
    const int wn = tid & 127, whalf = tid >> 7;
    const signed char *pw = a.d + ((P.wq + (size_t)(j0 + wn) * a.K) >> 1) + whalf * 16;
    uint32_t wr_off[4];
#pragma unroll
    for(int j = 0; j < 4; j++){
        const int ko = whalf * 4 + j;
        wr_off[j] = TN3_B_OFF + (uint32_t)(ko * TN3_BN + (wn ^ ((ko << 1) & 15))) * 16;
    }
    auto load_w = [&](int tile) -> i32x4 {
        const int tl = tile < steps ? tile : steps - 1;                   /* past the end: re-read the last one, never used */
        return tn3_gld16(pw + off_w(tl));
    };
    auto store_w = [&](const i32x4 w, int buf){
        const uint32_t wd[4] = {(uint32_t)w[0], (uint32_t)w[1], (uint32_t)w[2], (uint32_t)w[3]};
        const uint32_t bb = lds_base + buf * TN3_B_BYTES;
#pragma unroll
        for(int j = 0; j < 4; j++){
            i32x4 v;
            const QxNibs nb = qx_nibs(wd[j]);
            v[0] = (int)tn3_pk(qx_nib16(nb, 0), qx_nib16(nb, 1));
            v[1] = (int)tn3_pk(qx_nib16(nb, 2), qx_nib16(nb, 3));
            v[2] = (int)tn3_pk(qx_nib16(nb, 4), qx_nib16(nb, 5));
            v[3] = (int)tn3_pk(qx_nib16(nb, 6), qx_nib16(nb, 7));
            tn3_wr(bb + wr_off[j], v);
        }
    };

    /* ---- operand read offsets: [k16 slice]; the second tile of a pair is a constant further ---- */
    uint32_t ra[4], rb[4];
    {
        const int r = wi + fr, f = (r >> 1) & 7;                          /* rows r and r+32 share f */
        const int n = wj + fr;
#pragma unroll
        for(int ks = 0; ks < 4; ks++){
            const int ko = ks * 2 + hf;
            ra[ks] = (uint32_t)(r * 128 + ((ko ^ f) << 4));
            rb[ks] = TN3_B_OFF + (uint32_t)(ko * TN3_BN + (n ^ ((ko << 1) & 15))) * 16;
        }
    }

    /* ---- fp32 scale of (this lane's output column, scale group) ---- */
    const int ngroups = a.K >> a.gshift, sshift = a.gshift - 6, spg = 1 << sshift;     /* steps per scale group: a power of two */
    const float *pfold[2];
#pragma unroll
    for(int j = 0; j < 2; j++) pfold[j] = a.s + P.wg + (size_t)(j0 + wj + j * 32 + fr) * ngroups;
    auto load_scale = [&](int step, int j) -> float {
        int g = step >> sshift; g = g < ngroups * sg.nseg ? g : ngroups * sg.nseg - 1;
        const long long og = g < ngroups ? (long long)g : (long long)(g - ngroups) + sg.dS;
        return tn3_gld4(pfold[j] + og);
    };

    f32x16 acc[NI][2], part[NI][2];
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < 2; j++){ acc[i][j] = (f32x16)(0.0f); part[i][j] = (f32x16)(0.0f); }

    /* ---- prologue: digits of step 0 into buffer 0, those of step 1 into registers, the scales of
     * step 0; all requests go out before the one wait ---- */
    float fs_cur[2];
    i32x4 wcur;
    {
        i32x4 w0 = load_w(0);
        wcur = load_w(1);
        float f0 = load_scale(0, 0), f1 = load_scale(0, 1);
        issue_a(0, 0);
        issue_a(1, 1);
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w0), "+v"(wcur), "+v"(f0), "+v"(f1) : "n"(4 * NI) : "memory");
        store_w(w0, 0);
        fs_cur[0] = f0; fs_cur[1] = f1;
    }

    /* Main loop. A wavefront issues in order, and an MFMA of this shape keeps the vector ALU to itself
     * for about half of its 32 cycles: some four ALU instructions behind an MFMA cost nothing, every
     * further one its full four cycles, a memory request more, and whatever stands after the last MFMA
     * of a step runs alone. Everything else of a step is therefore cut into items and dealt evenly
     * into the gaps after the MFMAs, fences keeping the compiler from gathering them again:
     *   the loads of the digits of step st+2 and the scales of step st+1 (waited for at the end of the step, when they have
     *     long arrived: an asynchronously loaded register must not be carried round the loop before
     *     its wait) and the activation requests of tile st+2,
     *   the conversion of the digits of step st+1 (wcur) to bf16, four digits per item, each 16-byte
     *     unit written to the buffer last read in step st-1 as soon as it is complete.
     * A scale group's partial sums start from a zero operand instead of cleared registers. */
    constexpr int SLOTS = NI * 8, ITEMS = 3 + 2 * NI + 8 + 4;
    const f32x16 zero = (f32x16)(0.0f);
    /* A wavefront issues one instruction every four cycles whatever its kind, so the scalar bookkeeping of a step
     * counts like everything else: the stage numbers and the operand offsets of the tile two steps ahead are
     * carried from step to step (a compare and an add each) instead of being derived from the step number with
     * divisions and 64-bit multiplies. */
    int stg = 0, stg2 = 2 % TN3_A_STAGES;
    long long oa2 = off_a(2 < steps ? 2 : steps - 1), ow2 = off_w(2 < steps ? 2 : steps - 1);
    const long long jump_a = sg.dA - (long long)steps1 * (TN3_BK * 2), jump_w = sg.dW - (long long)steps1 * (TN3_BK / 2);
    for(int st = 0; st < steps; st++){
        /* tile st is in, own LDS writes are done; tile st+1 may still be on its way */
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(2 * NI) : "memory");
        __builtin_amdgcn_s_barrier();

        const uint32_t sa = lds_base + (uint32_t)stg * TN3_A_BYTES;
        const uint32_t sbuf = lds_base + (uint32_t)(st & 1) * TN3_B_BYTES;
        const uint32_t wbuf = lds_base + (uint32_t)((st + 1) & 1) * TN3_B_BYTES;
        const int stage2 = stg2;                        /* tile st+2 (past the end: the last one again, never used) goes there */
        const bool fresh = (st & (spg - 1)) == 0, last = ((st + 1) & (spg - 1)) == 0;
        i32x4 wnext; float fn[2];
        i32x4 wv[4];
        auto item = [&](int k){
            if(k == 0)      wnext = tn3_gld16(pw + ow2);
            else if(k < 3){ if(last) fn[k - 1] = load_scale(st + 1, k - 1); else fn[k - 1] = fs_cur[k - 1]; }   /* a new scale only where a group ends */
            else if(k < 3 + 2 * NI)
                __builtin_amdgcn_global_load_lds((glb_void *)(srcA[k - 3] + oa2),
                                                 (lds_void *)(lds + stage2 * TN3_A_BYTES + wave_off + (k - 3) * 4096), 16, 0, 0);
            else {
                /* per 16-byte unit: two conversion items, then its write */
                const int q = k - 3 - 2 * NI, j = q / 3, h = q % 3;
                if(h < 2){
                    const QxNibs nb = qx_nibs((uint32_t)wcur[j]);
                    wv[j][2 * h]     = (int)tn3_pk(qx_nib16(nb, 4 * h),     qx_nib16(nb, 4 * h + 1));
                    wv[j][2 * h + 1] = (int)tn3_pk(qx_nib16(nb, 4 * h + 2), qx_nib16(nb, 4 * h + 3));
                } else tn3_wr(wbuf + wr_off[j], wv[j]);
            }
        };
        Tn3Ops o[2];
        if(NI < 2){ o[0].a[1] = (i32x4)(0); o[1].a[1] = (i32x4)(0); }   /* the wait names both */
        o[0].a[0] = tn3_rd<0>(sa + ra[0]); if(NI > 1) o[0].a[1] = tn3_rd<32 * 128>(sa + ra[0]);
        o[0].b[0] = tn3_rd<0>(sbuf + rb[0]); o[0].b[1] = tn3_rd<32 * 16>(sbuf + rb[0]);
        tn3_wait(o[0]);
#define TN3_KS(KS, ZERO)                                                                                  \
        {                                                                                                 \
            Tn3Ops &cur = o[KS & 1], &nxt = o[(KS + 1) & 1];                                              \
            if(KS < 3){                                                                                   \
                nxt.a[0] = tn3_rd<0>(sa + ra[(KS + 1) & 3]); if(NI > 1) nxt.a[1] = tn3_rd<32 * 128>(sa + ra[(KS + 1) & 3]); \
                nxt.b[0] = tn3_rd<0>(sbuf + rb[(KS + 1) & 3]); nxt.b[1] = tn3_rd<32 * 16>(sbuf + rb[(KS + 1) & 3]);         \
            }                                                                                             \
            _Pragma("unroll")                                                                             \
            for(int m = 0; m < NI * 2; m++){                                                              \
                const int i = m >> 1, j = m & 1;                                                          \
                part[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, cur.a[i]), __builtin_bit_cast(bf16x8, cur.b[j]), ZERO ? zero : part[i][j], 0, 0, 0); \
                const int slot = KS * NI * 2 + m;                                                         \
                __builtin_amdgcn_sched_barrier(0);                                                        \
                _Pragma("unroll")                                                                         \
                for(int k = slot * ITEMS / SLOTS; k < (slot + 1) * ITEMS / SLOTS; k++) item(k);           \
                __builtin_amdgcn_sched_barrier(0);                                                        \
            }                                                                                             \
            if(KS < 3) tn3_wait(nxt);                                                                     \
        }
        if(fresh) TN3_KS(0, true) else TN3_KS(0, false)
        TN3_KS(1, false)
        TN3_KS(2, false)
        TN3_KS(3, false)
#undef TN3_KS
        if(last){
            /* one scale group of the contraction is complete: fold it in with its fp32 scale (spreading
             * these among the MFMAs as well costs some fifty registers, which spill). The matrix core was
             * fed digit / 16, so the scale carries the 16: both are exact, the product is the same. */
            const float fs16[2] = {fs_cur[0] * 16.0f, fs_cur[1] * 16.0f};
#pragma unroll
            for(int j = 0; j < 2; j++)
#pragma unroll
                for(int i = 0; i < NI; i++)
#pragma unroll
                    for(int e = 0; e < 16; e++) acc[i][j][e] = fmaf(fs16[j], part[i][j][e], acc[i][j][e]);
        }
        /* the digits of step st+2 and the scales of step st+1 have arrived (only the activation requests are younger) */
        asm volatile("s_waitcnt vmcnt(%3)" : "+v"(wnext), "+v"(fn[0]), "+v"(fn[1]) : "n"(2 * NI) : "memory");
        wcur = wnext;
        fs_cur[0] = fn[0]; fs_cur[1] = fn[1];
        stg = stg == TN3_A_STAGES - 1 ? 0 : stg + 1;
        stg2 = stg2 == TN3_A_STAGES - 1 ? 0 : stg2 + 1;
        if(st + 3 < steps){
            oa2 += TN3_BK * 2; ow2 += TN3_BK / 2;
            if(st + 3 == steps1){ oa2 += jump_a; ow2 += jump_w; }       /* on to the second operand pair */
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                    /* vmcnt(0), as a builtin so that the compiler knows it: no request may outlive the workgroup's LDS */

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int row = i0 + wi + hf * 4;
    if(a.out) qx_scatter_tiles<NI>(acc, (const int *)P.C, a.gate, a.out, row, rows, (size_t)a.N, j0 + wj + fr);
    else if(a.gp){
        const size_t o = (size_t)(P.C - a.gp) + (size_t)row * a.N + (j0 + wj + fr);
        qx_store_swiglu_bwd<NI>(acc, a.gp + o, a.up + o, a.dg + o, a.du + o, row, rows, (size_t)a.N);
    } else qx_store_tiles<NI, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, rows, (size_t)a.N, P.beta != 0.0f);
}

__global__ void __launch_bounds__(256, 2) k_gemm_tn_lds(Tn3Args a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[TN3_A_STAGES * TN3_A_BYTES + 2 * TN3_B_BYTES];
    const int t = qx_xcd_tile(blockIdx.x, gridDim.x);
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
    const int i0 = ti * TN3_BM, j0 = tj * TN3_BN;
    if(P.M - i0 > 64) tn3_tile<2>(a, P, sg, i0, j0, lds);
    else              tn3_tile<1>(a, P, sg, i0, j0, lds);
}

/* bf16 activations only; N % 128 == 0, K % 64 == 0, group a power of two >= 64 (checked by the caller) */
int qlmx_gemm_tn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs,
                            const qlmx_gemm_prob *second, int nprob, int K, int N, float *out, const float *gate,
                            const float *gp, const float *up_, void *dg, void *du, hipStream_t st){
    ProbUpload up; int slot;
    int rc = second ? qlmx_upload_problem_pairs(probs, second, nprob, GEMM_TN, K, N, TN3_BM, TN3_BN, st, &up, &slot)
                    : qlmx_upload_problems(probs, nprob, GEMM_TN, K, N, TN3_BM, TN3_BN, st, &up, &slot);
    if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Tn3Args a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.d = d; a.s = s; a.K = K; a.N = N; a.out = out; a.gate = gate;
    a.gp = gp; a.up = up_; a.dg = (unsigned short *)dg; a.du = (unsigned short *)du;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = (up.ntiles + 7) / 8 * 8;
    hipLaunchKernelGGL(k_gemm_tn_lds, dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm tn (direct-to-LDS) launch");
    return qlmx_upload_done(slot, st);
}
