/* qlmx_gemm_nn_lds.hip -- forward grouped GEMM (nn) for bf16 activations: activation tiles loaded
 * straight into LDS, dequantised weights kept row-major in LDS and read through the transposing
 * LDS read.
 *
 * Y_e[M,N] = X_e[M,K] . W_e[K,N]   (mg_ab, cudalm.cu:3204-3256; call sites 4211-4225)
 * W_e[K,N] packed 4-bit with scale groups along N, so the scale differs for every contraction index:
 * w = s*digit is formed in fp32 (the value the reference renders) and split into bf16 hi + lo; two
 * MFMAs per product add both parts (see qlmx_gemm_mfma.hip for why).
 *
 * 256x128 output tile, 32-deep steps, four wavefronts 2x2 with 4x2 accumulators each.
 *   Activations: every 16-byte piece goes from global memory into one of three LDS stages without
 *     touching a register (lane l of a wave instruction lands at base + 16*l). Rows keep their order,
 *     4 pieces per row, piece ko of row r stored at position ko ^ ((r >> 2) & 3): conflict-free
 *     128-bit operand reads.
 *   Weights: a thread loads 16 columns of one contraction row per step (8 bytes of digits, one scale),
 *     dequantises them and writes the hi and lo halves as two 16-byte units each; the unit u of row k
 *     sits at u ^ 4*(k & 3) of that row's 16 units. The rows stay in the matrix's own order (contraction index = row), and the MFMA operand
 *     -- 8 consecutive contraction elements of one column -- is two ds_read_b64_tr_b16 (within 16 lanes,
 *     lane i receives element i & 3 of the 8-byte pieces addressed by lanes 4v + (i >> 2), v = 0..3).
 *     The general kernel needs eight conflicting 4-byte stores per plane for the same transposition.
 * One barrier per step; the wait in front of it lets the activation tile requested last stay in
 * flight. All LDS accesses and register loads of the loop are inline assembly with explicit waits:
 * the compiler would wait for every outstanding load-to-LDS before any LDS access, and no
 * asynchronously loaded register is carried around the loop.
 */
#include "qlmx_gemm.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float  f32x2  __attribute__((ext_vector_type(2)));
typedef float  f32x16 __attribute__((ext_vector_type(16)));
typedef int    i32x2  __attribute__((ext_vector_type(2)));
typedef int    i32x4  __attribute__((ext_vector_type(4)));

#define NN3_BM 256
#define NN3_BN 128
#define NN3_BK 32
#define NN3_A_BYTES (NN3_BM * NN3_BK * 2)       /* 16384 */
#define NN3_A_STAGES 3
#define NN3_P_BYTES (NN3_BK * NN3_BN * 2)       /* one plane of a weight buffer: 8192 */
#define NN3_B_BYTES (2 * NN3_P_BYTES)           /* hi + lo */
#define NN3_B_OFF (NN3_A_STAGES * NN3_A_BYTES)

struct Nn3Args { const DevProb *pr; int nprob, ntiles; const signed char *d; const float *s; int gshift; int K, N; };

typedef __attribute__((address_space(3))) void lds_void;
typedef const __attribute__((address_space(1))) void glb_void;

__device__ __forceinline__ uint32_t nn3_pk(float lo, float hi){
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
}
template<int OFF> __device__ __forceinline__ i32x4 nn3_rd128(uint32_t addr){
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template<int OFF> __device__ __forceinline__ i32x2 nn3_tr(uint32_t addr){
    i32x2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template<int OFF> __device__ __forceinline__ void nn3_wr128(uint32_t addr, i32x4 v){
    asm volatile("ds_write_b128 %0, %1 offset:%2" :: "v"(addr), "v"(v), "n"(OFF) : "memory");
}
__device__ __forceinline__ int nn3_gld4(const void *p){
    int v;
    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ i32x2 nn3_gld8(const void *p){
    i32x2 v;
    asm volatile("global_load_dwordx2 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
struct Nn3Ops { i32x4 a[4]; i32x2 bh[2][2], bl[2][2]; };
__device__ __forceinline__ void nn3_wait(Nn3Ops &o){
    asm volatile("s_waitcnt lgkmcnt(0)"
        : "+v"(o.a[0]), "+v"(o.a[1]), "+v"(o.a[2]), "+v"(o.a[3]),
          "+v"(o.bh[0][0]), "+v"(o.bh[0][1]), "+v"(o.bh[1][0]), "+v"(o.bh[1][1]),
          "+v"(o.bl[0][0]), "+v"(o.bl[0][1]), "+v"(o.bl[1][0]), "+v"(o.bl[1][1]));
}
__device__ __forceinline__ bf16x8 nn3_pack(const i32x2 lo, const i32x2 hi){
    const i32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(bf16x8, v);
}

/* One output tile of NI*64 rows: the four wavefronts 2x2, each NI x 2 accumulators. NI = 4 is the
 * full tile; the last tile of a problem takes the smallest NI that holds its rows, so that an expert
 * with 130 rows does a 192-row tile's work rather than a 256-row tile's. */
/* The second half of a gate|up problem: the other weight matrix, its output, the SwiGLU output. */
struct Nn3Dual { unsigned long long wq, wg; float *C; unsigned short *act; };

template<int NI, bool DUAL = false>
__device__ __forceinline__ void nn3_tile(const Nn3Args &a, const DevProb &P, const Nn3Dual &Q, int i0, int j0, unsigned char *lds){
    const int rows = P.M;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (NI * 32), wj = (wave & 1) * 64;
    const int fr = lane & 31, hf = lane >> 5;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    const int steps = a.K / NN3_BK;

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
    auto issue_a = [&](int tile, int stage){
        const int tl = tile < steps ? tile : steps - 1;                   /* past the end: the last tile again, into a stage nobody reads */
        unsigned char *base = lds + stage * NN3_A_BYTES + wave_off;
#pragma unroll
        for(int h = 0; h < NI; h++)
            __builtin_amdgcn_global_load_lds((glb_void *)(srcA[h] + (size_t)tl * (NN3_BK * 2)), (lds_void *)(base + h * 4096), 16, 0, 0);
    };

    /* ---- weights: thread = (contraction row kr, columns oc*16 .. +15): one 8-byte load of digits and
     * one scale per step. The two 16-byte units it writes per plane are taken in opposite order by even
     * and odd rows, so that the 16 lanes of a write phase (two rows) hit 16 different units. ---- */
    const int oc = tid & 7, kr = tid >> 3, odd = kr & 1;
    /* gate|up tile: LDS column block oc holds 16 columns of gate (blocks 0, 1, 4, 5) or up (2, 3, 6, 7) */
    const bool second = DUAL && ((oc >> 1) & 1);
    const size_t e0 = (size_t)kr * a.N + j0 + (DUAL ? ((oc & 1) + ((oc >> 2) << 1)) * 16 : oc * 16);
    const signed char *pw = a.d + (((second ? Q.wq : P.wq) + e0) >> 1);
    const float *ps = a.s + (second ? Q.wg : P.wg) + (e0 >> a.gshift);
    const size_t wstep = (size_t)NN3_BK * a.N >> 1, sstep = (size_t)NN3_BK * a.N >> a.gshift;
    /* unit u of row k at u ^ 4*(k & 3) */
    const int sw = (kr & 3) << 2;
    const uint32_t wr0 = NN3_B_OFF + (uint32_t)(kr * 256 + (((2 * oc + odd) ^ sw) << 4));        /* written first  */
    const uint32_t wr1 = NN3_B_OFF + (uint32_t)(kr * 256 + (((2 * oc + 1 - odd) ^ sw) << 4));    /* written second */
    struct WLoad { i32x2 d; int s; };
    auto load_w = [&](int tile) -> WLoad {
        const size_t tl = (size_t)(tile < steps ? tile : steps - 1);      /* past the end: re-read the last one, never used */
        WLoad w;
        w.d = nn3_gld8(pw + tl * wstep); w.s = nn3_gld4(ps + tl * sstep);
        return w;
    };
    /* digits of the unit written first / second */
    auto unit_digits = [&](const WLoad &w, int which) -> uint32_t {
        return (uint32_t)((which ^ odd) ? w.d[1] : w.d[0]);
    };
    auto dequant_unit = [&](uint32_t digits, float sc, i32x4 &hi, i32x4 &lo){
        float w[8];
        const QxNibs nb = qx_nibs(digits);
#pragma unroll
        for(int j = 0; j < 8; j++) w[j] = (sc * 16.0f) * qx_nib16(nb, j);          /* 16 s * (digit / 16): both factors exact, the product is s * digit */
#pragma unroll
        for(int j = 0; j < 4; j++){
            const uint32_t h = nn3_pk(w[2 * j], w[2 * j + 1]);
            const float l0 = w[2 * j] - __uint_as_float(h << 16), l1 = w[2 * j + 1] - __uint_as_float(h & 0xFFFF0000u);
            hi[j] = (int)h; lo[j] = (int)nn3_pk(l0, l1);
        }
    };
    auto store_w = [&](const WLoad &w, int buf){
        const uint32_t bb = lds_base + buf * NN3_B_BYTES;
        i32x4 hi, lo;
        dequant_unit(unit_digits(w, 0), __int_as_float(w.s), hi, lo);
        nn3_wr128<0>(bb + wr0, hi); nn3_wr128<NN3_P_BYTES>(bb + wr0, lo);
        dequant_unit(unit_digits(w, 1), __int_as_float(w.s), hi, lo);
        nn3_wr128<0>(bb + wr1, hi); nn3_wr128<NN3_P_BYTES>(bb + wr1, lo);
    };

    /* ---- operand read offsets ---- */
    uint32_t ra[2][NI];                                  /* [k16 slice][row tile] activations, 128-bit */
#pragma unroll
    for(int i = 0; i < NI; i++){
        const int r = wi + i * 32 + fr, f = (r >> 2) & 3;
#pragma unroll
        for(int ks = 0; ks < 2; ks++) ra[ks][i] = (uint32_t)(r * 64 + (((ks * 2 + hf) ^ f) << 4));
    }
    uint32_t rb[2];                                      /* [column tile] weights, transposing reads; slice 1 is 16 rows further */
    {
        const int g16 = lane >> 4, s16 = lane & 15, v = s16 >> 2, q = s16 & 3, khalf = g16 >> 1, chalf = g16 & 1;
        const int row0 = khalf * 8 + v, sw = (row0 & 3) << 2;
#pragma unroll
        for(int j = 0; j < 2; j++){
            const int col = wj + j * 32 + chalf * 16 + q * 4;
            rb[j] = NN3_B_OFF + (uint32_t)(row0 * 256 + (((col >> 3) ^ sw) << 4) + (col & 7) * 2);
        }
    }

    f32x16 acc[NI][2];
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.0f);

    /* ---- prologue: weights of step 0 into buffer 0, those of step 1 into registers; all requests
     * go out before the one wait ---- */
    WLoad wcur;
    {
        WLoad w0 = load_w(0);
        wcur = load_w(1);
        issue_a(0, 0);
        issue_a(1, 1);
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(w0.d), "+v"(w0.s), "+v"(wcur.d), "+v"(wcur.s) : "n"(2 * NI) : "memory");
        store_w(w0, 0);
    }

    /* Main loop. A wavefront issues in order, and measured on this chip an MFMA of this shape keeps
     * the vector ALU to itself for about half of its 32 cycles: some four ALU instructions behind an
     * MFMA cost nothing, every further one its full four cycles, and whatever stands after the last
     * MFMA of a step runs alone. Everything else of a step is therefore cut into small items and
     * dealt evenly into the gaps after the MFMAs of both slices, fences keeping the compiler
     * from gathering them again:
     *   the two loads of the weights of step st+2 (into wnext, waited for at the end of the step,
     *     when they have long arrived: an asynchronously loaded register must not be carried round
     *     the loop before its wait), the activation requests of tile st+2,
     *   the dequantisation of the weights of step st+1 (wcur), two weights per pair of items,
     *   their four LDS writes into the buffer last read in step st-1. */
    constexpr int SLOTS = NI * 8, ITEMS = 2 + NI + 16 + 4;
    for(int st = 0; st < steps; st++){
        /* tile st is in, own LDS writes are done; tile st+1 may still be on its way */
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" :: "n"(NI) : "memory");
        __builtin_amdgcn_s_barrier();

        const uint32_t sa = lds_base + (uint32_t)(st % NN3_A_STAGES) * NN3_A_BYTES;
        const uint32_t sbuf = lds_base + (uint32_t)(st & 1) * NN3_B_BYTES;
        const uint32_t wbuf = lds_base + (uint32_t)((st + 1) & 1) * NN3_B_BYTES;
        const int tile2 = st + 2 < steps ? st + 2 : steps - 1, stage2 = (st + 2) % NN3_A_STAGES;   /* past the end: the last one again, never used */
        WLoad wnext;
        i32x4 whi[2], wlo[2];
        float wf[8][2];
        QxNibs dg[2];
        const float sc = __int_as_float(wcur.s) * 16.0f;     /* the digits come as digit / 16 (exact), the product is s * digit as before */
        auto item = [&](int k){
            if(k == 0)      wnext.d = nn3_gld8(pw + (size_t)tile2 * wstep);
            else if(k == 1) wnext.s = nn3_gld4(ps + (size_t)tile2 * sstep);
            else if(k < 2 + NI)
                __builtin_amdgcn_global_load_lds((glb_void *)(srcA[k - 2] + (size_t)tile2 * (NN3_BK * 2)),
                                                 (lds_void *)(lds + stage2 * NN3_A_BYTES + wave_off + (k - 2) * 4096), 16, 0, 0);
            else if(k < 2 + NI + 16){
                const int q = k - 2 - NI, p = q >> 1, r = p >> 2, j = p & 3;
                if(q == 0){ dg[0] = qx_nibs(unit_digits(wcur, 0)); dg[1] = qx_nibs(unit_digits(wcur, 1)); }
                if((q & 1) == 0){
                    wf[p][0] = sc * qx_nib16(dg[r], 2 * j); wf[p][1] = sc * qx_nib16(dg[r], 2 * j + 1);
                } else {
                    const uint32_t h = nn3_pk(wf[p][0], wf[p][1]);
                    whi[r][j] = (int)h;
                    wlo[r][j] = (int)nn3_pk(wf[p][0] - __uint_as_float(h << 16), wf[p][1] - __uint_as_float(h & 0xFFFF0000u));
                }
            } else {
                const int w = k - 2 - NI - 16;
                if(w == 0)      nn3_wr128<0>(wbuf + wr0, whi[0]);
                else if(w == 1) nn3_wr128<NN3_P_BYTES>(wbuf + wr0, wlo[0]);
                else if(w == 2) nn3_wr128<0>(wbuf + wr1, whi[1]);
                else            nn3_wr128<NN3_P_BYTES>(wbuf + wr1, wlo[1]);
            }
        };
        Nn3Ops o0, o1;
        if(NI < 4){                                        /* the wait names all four; the spare ones hold nothing */
#pragma unroll
            for(int i = NI; i < 4; i++){ o0.a[i] = (i32x4)(0); o1.a[i] = (i32x4)(0); }
        }
#define NN3_READ(O, KS)                                                                                   \
        _Pragma("unroll")                                                                                 \
        for(int i = 0; i < NI; i++) O.a[i] = nn3_rd128<0>(sa + ra[KS][i]);                                \
        _Pragma("unroll")                                                                                 \
        for(int j = 0; j < 2; j++){                                                                       \
            O.bh[j][0] = nn3_tr<KS * 16 * 256>(sbuf + rb[j]);                                             \
            O.bh[j][1] = nn3_tr<KS * 16 * 256 + 4 * 256>(sbuf + rb[j]);                                   \
            O.bl[j][0] = nn3_tr<NN3_P_BYTES + KS * 16 * 256>(sbuf + rb[j]);                               \
            O.bl[j][1] = nn3_tr<NN3_P_BYTES + KS * 16 * 256 + 4 * 256>(sbuf + rb[j]);                     \
        }
#define NN3_MMA(O, BLOCK)                                                                                 \
        _Pragma("unroll")                                                                                 \
        for(int m = 0; m < NI * 4; m++){                   /* all hi parts, then all lo parts */            \
            const int i = (m >> 1) % NI, j = m & 1;                                                       \
            if(m < NI * 2) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, O.a[i]), nn3_pack(O.bh[j][0], O.bh[j][1]), acc[i][j], 0, 0, 0); \
            else           acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, O.a[i]), nn3_pack(O.bl[j][0], O.bl[j][1]), acc[i][j], 0, 0, 0); \
            {                                                                                             \
                const int slot = BLOCK * (SLOTS / 2) + m;                                                 \
                __builtin_amdgcn_sched_barrier(0);                                                        \
                _Pragma("unroll")                                                                         \
                for(int k = slot * ITEMS / SLOTS; k < (slot + 1) * ITEMS / SLOTS; k++) item(k);           \
                __builtin_amdgcn_sched_barrier(0);                                                        \
            }                                                                                             \
        }
        NN3_READ(o0, 0)
        nn3_wait(o0);
        NN3_READ(o1, 1)                                    /* in flight while slice 0 multiplies */
        NN3_MMA(o0, 0)
        nn3_wait(o1);
        NN3_MMA(o1, 1)
#undef NN3_READ
#undef NN3_MMA
        /* the weights of step st+2 have arrived (only the activation requests are younger) */
        asm volatile("s_waitcnt vmcnt(%2)" : "+v"(wnext.d), "+v"(wnext.s) : "n"(NI) : "memory");
        wcur = wnext;
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);                    /* vmcnt(0), as a builtin so that the compiler knows it: no request may outlive the workgroup's LDS */

    /* ---- epilogue: the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
    const int row = i0 + wi + hf * 4;
    if(DUAL){
        const size_t o = (size_t)row * a.N + (j0 + (wj >> 1) + fr);
        qx_store_swiglu<NI>(acc, P.C + o, Q.C + o, Q.act + o, row, rows, (size_t)a.N);
    } else
        qx_store_tiles<NI, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, rows, (size_t)a.N, P.beta != 0.0f);
}

__global__ void __launch_bounds__(256, 2) k_gemm_nn_lds(Nn3Args a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[NN3_A_STAGES * NN3_A_BYTES + 2 * NN3_B_BYTES];
    const int t = qx_xcd_tile(blockIdx.x, gridDim.x);
    if(t >= a.ntiles) return;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * NN3_BM, j0 = tj * NN3_BN, left = P.M - i0;
    const Nn3Dual none = {0, 0, nullptr, nullptr};
    if(left > 192)      nn3_tile<4>(a, P, none, i0, j0, lds);
    else if(left > 128) nn3_tile<3>(a, P, none, i0, j0, lds);
    else if(left > 64)  nn3_tile<2>(a, P, none, i0, j0, lds);
    else                nn3_tile<1>(a, P, none, i0, j0, lds);
}

/* gate|up problems: tiles of 256 rows x 64 columns of both matrices; the entry after the problem's holds the
 * second matrix and the two further outputs */
__global__ void __launch_bounds__(256, 2) k_gemm_nn_lds_swiglu(Nn3Args a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[NN3_A_STAGES * NN3_A_BYTES + 2 * NN3_B_BYTES];
    const int t = qx_xcd_tile(blockIdx.x, gridDim.x);
    if(t >= a.ntiles) return;
    const int pi = qx_find_problem(a.pr, a.nprob, t);
    const DevProb P = a.pr[pi];
    const DevProb P2 = a.pr[pi + 1];
    const Nn3Dual Q = {P2.wq, P2.wg, P2.C, (unsigned short *)P2.B};
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * NN3_BM, j0 = tj * (NN3_BN / 2), left = P.M - i0;
    if(left > 192)      nn3_tile<4, true>(a, P, Q, i0, j0, lds);
    else if(left > 128) nn3_tile<3, true>(a, P, Q, i0, j0, lds);
    else if(left > 64)  nn3_tile<2, true>(a, P, Q, i0, j0, lds);
    else                nn3_tile<1, true>(a, P, Q, i0, j0, lds);
}

/* bf16 activations only; N % 128 == 0, K % 32 == 0, group a power of two >= 32 (checked by the caller) */
int qlmx_gemm_nn_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                            int K, int N, hipStream_t st){
    ProbUpload up; int slot;
    int rc = qlmx_upload_problems(probs, nprob, GEMM_NN, K, N, NN3_BM, NN3_BN, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Nn3Args a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.d = d; a.s = s; a.K = K; a.N = N;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = (up.ntiles + 7) / 8 * 8;
    hipLaunchKernelGGL(k_gemm_nn_lds, dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm nn (direct-to-LDS) launch");
    return qlmx_upload_done(slot, st);
}

/* gate|up pairs with the SwiGLU in the epilogue: bf16 activations only; N % 64 == 0, K % 32 == 0, group a
 * power of two >= 64 (so that a tile's 64 columns of a matrix share a scale per contraction row) */
int qlmx_gemm_nn_swiglu_lds_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *gate,
                                   const qlmx_gemm_prob *up_, int nprob, int K, int N, hipStream_t st){
    ProbUpload up; int slot;
    int rc = qlmx_upload_problem_pairs(gate, up_, nprob, GEMM_NN, K, N, NN3_BM, NN3_BN / 2, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    Nn3Args a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.d = d; a.s = s; a.K = K; a.N = N;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = (up.ntiles + 7) / 8 * 8;
    hipLaunchKernelGGL(k_gemm_nn_lds_swiglu, dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm nn + swiglu launch");
    return qlmx_upload_done(slot, st);
}
