/* qlmx_gemm_nn_h.hip -- forward grouped GEMM (nn) on the fp16 matrix core: one MFMA per product.
 *
 * Y_e[M,N] = X_e[M,K] . W_e[K,N]   (mg_ab, cudalm.cu:3204-3256; call sites 4211-4225)
 *
 * W is packed 4-bit with its scale groups along N, so the scale differs for every contraction index and
 * cannot be taken out of the sum: the weight w = s*digit has to be one matrix-core operand. In bf16 (8
 * significant bits) that rounding alone costs 1.6e-3 of relative error, which is why the bf16 kernel
 * (qlmx_gemm_nn_lds.hip) splits w into hi + lo and spends two MFMAs per product. fp16 keeps 11 bits:
 * fp16(s*digit), rounded to nearest even, is within 2^-12 of w, about 2e-4 relative L2 on the output,
 * and one v_mfma_f32_32x32x16_f16 per product is enough. The activations arrive as bf16; every bf16 value
 * between 2^-14 and 65504 in magnitude is an fp16 value, so they are converted exactly on their way into LDS
 * (smaller ones become fp16 subnormals with an absolute error below 3e-8, larger ones saturate at 65504).
 * Weights are multiplied by 2^8 before the conversion and the accumulators by 2^-8 after the last step, which
 * moves the range in which fp16 keeps all 11 bits to 2.4e-7 <= |w| <= 255.
 *
 * 256x128 output tile, 32-deep steps, four wavefronts 2x2 with 4x2 accumulators each, two LDS buffers per
 * operand. Every operand passes through registers once: a thread loads 16 bytes of four activation rows and
 * 16 weights per step two steps ahead, converts them one step ahead, and writes them into the buffer that was
 * read in the step before. Layouts in LDS as in qlmx_gemm_nn_lds.hip: activation rows of 64 bytes with the four
 * 16-byte pieces rotated by the row (conflict-free 128-bit operand reads), weight rows of 256 bytes in the
 * matrix's own order with the 16-byte units xor-swizzled, read through ds_read_b64_tr_b16.
 */
#include "qlmx_gemm.h"
#include <type_traits>

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float    f32x2 __attribute__((ext_vector_type(2)));
typedef float    f32x16 __attribute__((ext_vector_type(16)));
typedef int      i32x2 __attribute__((ext_vector_type(2)));
typedef int      i32x4 __attribute__((ext_vector_type(4)));

#define NH_BM 256
#define NH_BN 128
#define NH_BK 32
#define NH_A_BYTES (NH_BM * NH_BK * 2)          /* 16384 */
#define NH_B_BYTES (NH_BK * NH_BN * 2)          /*  8192 */
#define NH_B_OFF (2 * NH_A_BYTES)
#define NH_WSCALE 4096.0f                       /* 16 (the digits come as digit/16) * 2^8 (range shift) */
#define NH_UNSCALE (1.0f / 256.0f)

/* Row plumbing of a launch (the MoE glue folded into the GEMM):
 *   NH_PLAIN    A and C of a problem are its own row-major buffers;
 *   NH_GATHER   k_gather in front (cudalm.cu:2536-2539, 4211): a problem's A field points at its row indices
 *               (const int *), row r of the problem is row idx[r] of `xsrc` (bf16 [tokens, K]), zeros where idx[r] < 0;
 *   NH_SCATTER  k_scatter_gate / k_scatter_add4 behind (cudalm.cu:2541-2545, 2564-2567, 4227): a problem's C field
 *               points at its row indices, out[idx[r], :] = out[idx[r], :] + gate[idx[r]] * y[r, :] (gate NULL: + y[r, :]),
 *               rows with idx[r] < 0 dropped. Within one launch every output row must be named at most once. */
enum { NH_PLAIN = 0, NH_GATHER = 1, NH_SCATTER = 2 };
struct NhArgs { const DevProb *pr; int nprob, ntiles, nfull, tiles_n; const signed char *d; const float *s; int gshift; int K, N;
                const char *xsrc; float *out; const float *gate; };

/* a row of zeros as long as the longest contraction a gathering launch accepts: what a dropped row reads */
#define NH_ZERO_BYTES 32768
static __device__ __align__(16) unsigned char nh_zero_row[NH_ZERO_BYTES];

template<int OFF> __device__ __forceinline__ i32x4 nh_rd128(uint32_t addr){
    i32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template<int OFF> __device__ __forceinline__ i32x2 nh_tr(uint32_t addr){
    i32x2 v;
    asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF));
    return v;
}
template<int OFF> __device__ __forceinline__ void nh_wr128(uint32_t addr, i32x4 v){
    asm volatile("ds_write_b128 %0, %1 offset:%2" :: "v"(addr), "v"(v), "n"(OFF) : "memory");
}
/* Global loads are ordinary loads here: this kernel has no load-to-LDS instruction, so the compiler's own wait
 * counts are exact (it waits, with the right count, just before the first use of a loaded value, also when that
 * use is in the next iteration of the loop) and a tile's loads can stay in flight for a step and a half. */
typedef const __attribute__((address_space(1))) int   g_i32;
typedef const __attribute__((address_space(1))) i32x2 g_i32x2;
typedef const __attribute__((address_space(1))) i32x4 g_i32x4;
__device__ __forceinline__ int   nh_gld4(const void *p){ return *(g_i32 *)p; }
__device__ __forceinline__ i32x2 nh_gld8(const void *p){ return *(g_i32x2 *)p; }
__device__ __forceinline__ i32x4 nh_gld16(const void *p){ return *(g_i32x4 *)p; }
struct NhOps { i32x4 a[4]; i32x2 b[2][2]; };
__device__ __forceinline__ void nh_wait_lds(NhOps &o){
    asm volatile("s_waitcnt lgkmcnt(0)"
        : "+v"(o.a[0]), "+v"(o.a[1]), "+v"(o.a[2]), "+v"(o.a[3]),
          "+v"(o.b[0][0]), "+v"(o.b[0][1]), "+v"(o.b[1][0]), "+v"(o.b[1][1]));
}
__device__ __forceinline__ f16x8 nh_pack(const i32x2 lo, const i32x2 hi){
    const i32x4 v = {lo[0], lo[1], hi[0], hi[1]};
    return __builtin_bit_cast(f16x8, v);
}
/* two bf16 in a word -> the same two values as fp16 (exact inside fp16's normal range) */
__device__ __forceinline__ int nh_bf16x2_to_f16x2(int w){
    const float lo = __uint_as_float((uint32_t)w << 16), hi = __uint_as_float((uint32_t)w & 0xFFFF0000u);
    return __builtin_bit_cast(int, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}
__device__ __forceinline__ int nh_pk(float lo, float hi){          /* round to nearest even: v_cvt_pk_f16_f32 */
    f32x2 v = {lo, hi};
    return __builtin_bit_cast(int, __builtin_convertvector(v, f16x2));
}

struct NhW { i32x2 d; int s; };

/* One output tile of NI*64 rows (NI = 4: the full 256; the last tile of a problem takes the smallest NI that
 * holds its rows). */
/* The second half of a gate|up problem (DUAL): the other weight matrix, its fp32 output, the SwiGLU output. The
 * tile's 128 LDS columns are then [gate 0-31 | up 0-31 | gate 32-63 | up 32-63] of the problem's columns
 * j0 .. j0+63: a wavefront's first accumulator column holds gate and its second up of the same 32 columns. */
struct NhDual { unsigned long long wq, wg; float *C; unsigned short *act; };

template<int NI, int IO, bool DUAL = false>
__device__ __forceinline__ void nh_tile(const NhArgs &a, const DevProb &P, const NhDual &Q, int i0, int j0, unsigned char *lds){
    const int rows = P.M;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wi = (wave >> 1) * (NI * 32), wj = (wave & 1) * 64;
    const int fr = lane & 31, hf = lane >> 5;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char *)lds;
    const int steps = a.K / NH_BK;

    /* ---- activations: position p = h*256 + tid of a buffer is row p/4, stored piece p%4 = ko ^ ((row >> 2) & 3) ---- */
    const char *srcA[NI]; uint32_t posA[NI];
#pragma unroll
    for(int h = 0; h < NI; h++){
        const int p = h * 256 + tid, r = p >> 2, ko = (p & 3) ^ ((r >> 2) & 3);
        const int rr = (i0 + r < rows) ? i0 + r : rows - 1;               /* clamp: feeds unstored rows only */
        if(IO == NH_GATHER){
            const int tok = ((const int *)P.A)[rr];
            srcA[h] = (tok >= 0 ? a.xsrc + (size_t)tok * a.K * 2 : (const char *)nh_zero_row) + ko * 16;
        } else srcA[h] = (const char *)P.A + ((size_t)rr * a.K + ko * 8) * 2;
        posA[h] = (uint32_t)p * 16;
    }
    /* ---- weights: thread = (contraction row kr, columns oc*16 .. +15): one 8-byte load of digits and one scale
     * per step; its two 16-byte units are taken in opposite order by even and odd rows, so that the 16 lanes of
     * a write phase (two rows) hit 16 different units ---- */
    const int oc = tid & 7, kr = tid >> 3, odd = kr & 1;
    const bool second = DUAL && ((oc >> 1) & 1);
    const size_t e0 = (size_t)kr * a.N + j0 + (DUAL ? ((oc & 1) + ((oc >> 2) << 1)) * 16 : oc * 16);
    const signed char *pw = a.d + (((second ? Q.wq : P.wq) + e0) >> 1);
    const float *ps = a.s + (second ? Q.wg : P.wg) + (e0 >> a.gshift);
    const size_t wstep = (size_t)NH_BK * a.N >> 1, sstep = (size_t)NH_BK * a.N >> a.gshift;
    const int sw = (kr & 3) << 2;
    const uint32_t wr0 = NH_B_OFF + (uint32_t)(kr * 256 + (((2 * oc + odd) ^ sw) << 4));         /* written first  */
    const uint32_t wr1 = NH_B_OFF + (uint32_t)(kr * 256 + (((2 * oc + 1 - odd) ^ sw) << 4));     /* written second */
    auto tile_of = [&](int t){ return (size_t)(t < steps ? t : steps - 1); };   /* past the end: the last one again, never used */
    auto load_w = [&](int t) -> NhW { NhW w; w.d = nh_gld8(pw + tile_of(t) * wstep); w.s = nh_gld4(ps + tile_of(t) * sstep); return w; };
    auto load_a = [&](int t, int h) -> i32x4 { return nh_gld16(srcA[h] + tile_of(t) * (NH_BK * 2)); };
    auto unit_digits = [&](const NhW &w, int which) -> uint32_t { return (uint32_t)((which ^ odd) ? w.d[1] : w.d[0]); };
    auto convert_a = [&](const i32x4 &v) -> i32x4 {
        i32x4 r;
#pragma unroll
        for(int j = 0; j < 4; j++) r[j] = nh_bf16x2_to_f16x2(v[j]);
        return r;
    };
    auto dequant_unit = [&](uint32_t digits, float sc) -> i32x4 {
        const QxNibs nb = qx_nibs(digits);
        i32x4 r;
#pragma unroll
        for(int j = 0; j < 4; j++) r[j] = nh_pk(sc * qx_nib16(nb, 2 * j), sc * qx_nib16(nb, 2 * j + 1));
        return r;
    };

    /* ---- LDS addresses. Which of an operand's two buffers a step reads or writes is known at compile time (the
     * loop below is unrolled by two), so the buffer, the k16 slice and the second half of a transposing read all
     * go into the instructions' immediate offsets and the loop computes no LDS address at all. ---- */
    uint32_t ra[2][NI];                                  /* [k16 slice][row tile] activations, 128-bit reads */
#pragma unroll
    for(int i = 0; i < NI; i++){
        const int r = wi + i * 32 + fr, f = (r >> 2) & 3;
#pragma unroll
        for(int ks = 0; ks < 2; ks++) ra[ks][i] = lds_base + (uint32_t)(r * 64 + (((ks * 2 + hf) ^ f) << 4));
    }
    uint32_t rb[2];                                      /* [column tile] weights, transposing reads */
    {
        const int g16 = lane >> 4, s16 = lane & 15, v = s16 >> 2, q = s16 & 3, khalf = g16 >> 1, chalf = g16 & 1;
        const int row0 = khalf * 8 + v, swr = (row0 & 3) << 2;
#pragma unroll
        for(int j = 0; j < 2; j++){
            const int col = wj + j * 32 + chalf * 16 + q * 4;
            rb[j] = lds_base + (uint32_t)(row0 * 256 + (((col >> 3) ^ swr) << 4) + (col & 7) * 2);
        }
    }
    uint32_t wpa[NI];
#pragma unroll
    for(int h = 0; h < NI; h++) wpa[h] = lds_base + posA[h];
    const uint32_t wp0 = lds_base + wr0 - NH_B_OFF, wp1 = lds_base + wr1 - NH_B_OFF;

    f32x16 acc[NI][2];
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = (f32x16)(0.0f);

    /* ---- prologue: tile 0 into buffer 0, tile 1 into registers; all requests go out before the first use ---- */
    NhW wA, wB; i32x4 aA[NI], aB[NI];
    {
        NhW w0 = load_w(0); i32x4 a0[NI];
#pragma unroll
        for(int h = 0; h < NI; h++) a0[h] = load_a(0, h);
        wB = load_w(1);
#pragma unroll
        for(int h = 0; h < NI; h++) aB[h] = load_a(1, h);
#pragma unroll
        for(int h = 0; h < NI; h++) nh_wr128<0>(wpa[h], convert_a(a0[h]));
        const float sc = __int_as_float(w0.s) * NH_WSCALE;
        nh_wr128<NH_B_OFF>(wp0, dequant_unit(unit_digits(w0, 0), sc));
        nh_wr128<NH_B_OFF>(wp1, dequant_unit(unit_digits(w0, 1), sc));
    }

    /* Main loop, two steps per iteration: step `st` of parity PAR reads buffers PAR, holds tile st+1 in the
     * register set `cur` (loaded during step st-1) and loads tile st+2 into the set `nxt`; the two sets swap
     * roles from step to step, so no loaded value is ever copied and a tile's loads stay in flight from the first
     * items of step st until the conversions of step st+1 need them, more than a step later (the compiler places
     * those waits, with exact counts: this kernel has no load-to-LDS instruction to confuse it).
     * A wavefront issues in order and an MFMA of this shape leaves room for about four vector-ALU instructions
     * behind it, so everything else of a step is cut into small items that are dealt evenly into the gaps after
     * the step's MFMAs (fences keep the compiler from gathering them again):
     *   the loads of tile st+2 (weights, then the NI activation pieces),
     *   the conversion of tile st+1's activation pieces (two words per item) and their LDS writes,
     *   the dequantisation of tile st+1's weights (two weights per item) and their two LDS writes,
     * the writes going to the buffers that were read in step st-1. */
    constexpr int SLOTS = NI * 4, ITEMS = 2 + NI + 2 * NI + 8 + 2;
    auto step = [&](auto PARC, int st, const NhW &wcur, const i32x4 (&acur)[NI], NhW &wnxt, i32x4 (&anxt)[NI]){
        constexpr int PAR = decltype(PARC)::value;
        constexpr int RA = PAR * NH_A_BYTES, RB = NH_B_OFF + PAR * NH_B_BYTES;                 /* read  */
        constexpr int WA = (1 - PAR) * NH_A_BYTES, WB = NH_B_OFF + (1 - PAR) * NH_B_BYTES;     /* write */
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");     /* own LDS writes of tile st are done */
        __builtin_amdgcn_s_barrier();
        i32x4 ah[NI], wh[2];
        QxNibs dg[2];
        const float sc = __int_as_float(wcur.s) * NH_WSCALE;
        auto item = [&](int k){
            if(k == 0)      wnxt.d = nh_gld8(pw + tile_of(st + 2) * wstep);
            else if(k == 1) wnxt.s = nh_gld4(ps + tile_of(st + 2) * sstep);
            else if(k < 2 + NI) anxt[k - 2] = nh_gld16(srcA[k - 2] + tile_of(st + 2) * (NH_BK * 2));
            else if(k < 2 + 3 * NI){
                const int q = k - 2 - NI, h = q >> 1;
                if((q & 1) == 0){ ah[h][0] = nh_bf16x2_to_f16x2(acur[h][0]); ah[h][1] = nh_bf16x2_to_f16x2(acur[h][1]); }
                else { ah[h][2] = nh_bf16x2_to_f16x2(acur[h][2]); ah[h][3] = nh_bf16x2_to_f16x2(acur[h][3]); nh_wr128<WA>(wpa[h], ah[h]); }
            } else if(k < 2 + 3 * NI + 8){
                const int q = k - 2 - 3 * NI, r = q >> 2, j = q & 3;
                if(q == 0){ dg[0] = qx_nibs(unit_digits(wcur, 0)); dg[1] = qx_nibs(unit_digits(wcur, 1)); }
                wh[r][j] = nh_pk(sc * qx_nib16(dg[r], 2 * j), sc * qx_nib16(dg[r], 2 * j + 1));
            } else {
                if(k - 2 - 3 * NI - 8 == 0) nh_wr128<WB>(wp0, wh[0]); else nh_wr128<WB>(wp1, wh[1]);
            }
        };
        NhOps o0, o1;
        if(NI < 4){                                        /* the wait names all four; the spare ones hold nothing */
#pragma unroll
            for(int i = NI; i < 4; i++){ o0.a[i] = (i32x4)(0); o1.a[i] = (i32x4)(0); }
        }
#define NH_READ(O, KS)                                                                                    \
        _Pragma("unroll")                                                                                 \
        for(int i = 0; i < NI; i++) O.a[i] = nh_rd128<RA>(ra[KS][i]);                                     \
        _Pragma("unroll")                                                                                 \
        for(int j = 0; j < 2; j++){                                                                       \
            O.b[j][0] = nh_tr<RB + KS * 16 * 256>(rb[j]);                                                 \
            O.b[j][1] = nh_tr<RB + KS * 16 * 256 + 4 * 256>(rb[j]);                                       \
        }
#define NH_MMA(O, BLOCK)                                                                                  \
        _Pragma("unroll")                                                                                 \
        for(int m = 0; m < NI * 2; m++){                                                                  \
            const int i = m >> 1, j = m & 1;                                                              \
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, O.a[i]), nh_pack(O.b[j][0], O.b[j][1]), acc[i][j], 0, 0, 0); \
            {                                                                                             \
                const int slot = BLOCK * (SLOTS / 2) + m;                                                 \
                __builtin_amdgcn_sched_barrier(0);                                                        \
                _Pragma("unroll")                                                                         \
                for(int k = slot * ITEMS / SLOTS; k < (slot + 1) * ITEMS / SLOTS; k++) item(k);           \
                __builtin_amdgcn_sched_barrier(0);                                                        \
            }                                                                                             \
        }
        NH_READ(o0, 0)
        nh_wait_lds(o0);
        NH_READ(o1, 1)                                     /* in flight while slice 0 multiplies */
        NH_MMA(o0, 0)
        nh_wait_lds(o1);
        NH_MMA(o1, 1)
#undef NH_READ
#undef NH_MMA
    };
    {
        int st = 0;
        for(; st + 1 < steps; st += 2){
            step(std::integral_constant<int, 0>(), st, wB, aB, wA, aA);
            step(std::integral_constant<int, 1>(), st + 1, wA, aA, wB, aB);
        }
        if(st < steps) step(std::integral_constant<int, 0>(), st, wB, aB, wA, aA);
    }

    /* ---- epilogue: undo the range shift, then the lane holds column lane%32 of each 32x32 tile, four-row band lane/32 ---- */
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < 2; j++) acc[i][j] = acc[i][j] * NH_UNSCALE;
    const int row = i0 + wi + hf * 4;
    if(DUAL){
        const size_t o = (size_t)row * a.N + (j0 + (wj >> 1) + fr);
        qx_store_swiglu<NI, true>(acc, P.C ? P.C + o : nullptr, Q.C + o, Q.act + o, row, rows, (size_t)a.N);
    } else if(IO == NH_SCATTER) qx_scatter_tiles<NI>(acc, (const int *)P.C, a.gate, a.out, row, rows, (size_t)a.N, j0 + wj + fr);
    else qx_store_tiles<NI, 2>(acc, P.C + (size_t)row * a.N + (j0 + wj + fr), row, i0 + wi, rows, (size_t)a.N, false);
}

template<int IO>
__global__ void __launch_bounds__(256, 2) k_gemm_nn_h(NhArgs a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * NH_A_BYTES + 2 * NH_B_BYTES];
    const int t = qx_lpt_tile(blockIdx.x, a.nfull, a.ntiles, a.tiles_n);
    if(t >= a.ntiles) return;
    const DevProb P = a.pr[qx_find_problem(a.pr, a.nprob, t)];
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * NH_BM, j0 = tj * NH_BN, left = P.M - i0;
    const NhDual none = {0, 0, nullptr, nullptr};
    if(left > 192)      nh_tile<4, IO>(a, P, none, i0, j0, lds);
    else if(left > 128) nh_tile<3, IO>(a, P, none, i0, j0, lds);
    else if(left > 64)  nh_tile<2, IO>(a, P, none, i0, j0, lds);
    else                nh_tile<1, IO>(a, P, none, i0, j0, lds);
}

/* gate|up problems with the SwiGLU in the epilogue (mg_ab w1, mg_ab w3, e_swig; cudalm.cu:4211-4215): tiles of 256
 * rows x 64 columns of both matrices; the table entry after the problem's holds the second matrix, the up output
 * and the bf16 SwiGLU output. The fp32 gate / up outputs are skipped when the problem's C is NULL. */
template<int IO>
__global__ void __launch_bounds__(256, 2) k_gemm_nn_h_swiglu(NhArgs a){
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * NH_A_BYTES + 2 * NH_B_BYTES];
    const int t = qx_lpt_tile(blockIdx.x, a.nfull, a.ntiles, a.tiles_n);
    if(t >= a.ntiles) return;
    const int pi = qx_find_problem(a.pr, a.nprob, t);
    const DevProb P = a.pr[pi];
    const DevProb P2 = a.pr[pi + 1];
    const NhDual Q = {P2.wq, P2.wg, P2.C, (unsigned short *)P2.B};
    const int lt = t - P.tile0;
    const int ti = lt / P.tiles_n, tj = lt - ti * P.tiles_n;
    const int i0 = ti * NH_BM, j0 = tj * (NH_BN / 2), left = P.M - i0;
    if(left > 192)      nh_tile<4, IO, true>(a, P, Q, i0, j0, lds);
    else if(left > 128) nh_tile<3, IO, true>(a, P, Q, i0, j0, lds);
    else if(left > 64)  nh_tile<2, IO, true>(a, P, Q, i0, j0, lds);
    else                nh_tile<1, IO, true>(a, P, Q, i0, j0, lds);
}

/* bf16 activations only; N % 128 == 0, K % 32 == 0, group a power of two >= 32 (checked by the caller).
 * io = NH_GATHER: xsrc is the bf16 token matrix and the problems' A fields are row-index lists;
 * io = NH_SCATTER: out (and gate, may be NULL) is the destination and the problems' C fields are row-index lists. */
int qlmx_gemm_nn_h_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *probs, int nprob,
                          int K, int N, int io, const void *xsrc, float *out, const float *gate, hipStream_t st){
    QLMX_REQUIRE(io != NH_GATHER || (size_t)K * 2 <= NH_ZERO_BYTES, "grouped gemm nn with gather: K=%d exceeds %d", K, NH_ZERO_BYTES / 2);
    ProbUpload up; int slot;
    const RowBytes rb = {io == NH_GATHER ? sizeof(int) : (size_t)K * 2, io == NH_SCATTER ? sizeof(int) : (size_t)N * 4, 0, 0, 0};
    int rc = qlmx_upload_problems_split(probs, nullptr, nprob, GEMM_NN, K, N, NH_BM, NH_BN, &rb, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    NhArgs a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.nfull = up.nfull; a.tiles_n = N / NH_BN; a.d = d; a.s = s; a.K = K; a.N = N;
    a.xsrc = (const char *)xsrc; a.out = out; a.gate = gate;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = qx_lpt_grid(up.nfull, up.ntiles, a.tiles_n);
    if(io == NH_GATHER)       hipLaunchKernelGGL(k_gemm_nn_h<NH_GATHER>,  dim3(grid), dim3(256), 0, st, a);
    else if(io == NH_SCATTER) hipLaunchKernelGGL(k_gemm_nn_h<NH_SCATTER>, dim3(grid), dim3(256), 0, st, a);
    else                      hipLaunchKernelGGL(k_gemm_nn_h<NH_PLAIN>,   dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm nn (fp16 matrix core) launch");
    return qlmx_upload_done(slot, st);
}

/* gate|up pairs with the SwiGLU in the epilogue: N % 64 == 0, K % 32 == 0, group a power of two >= 64 (a tile's 64
 * columns of a matrix share a scale per contraction row). xsrc != NULL: the gate problems' A fields are row-index
 * lists into the bf16 token matrix xsrc (NH_GATHER). Problems whose gate C is NULL store the bf16 output only. */
int qlmx_gemm_nn_h_swiglu_launch(const signed char *d, const float *s, int group, const qlmx_gemm_prob *gate, const qlmx_gemm_prob *up_,
                                 int nprob, int K, int N, const void *xsrc, hipStream_t st){
    QLMX_REQUIRE(!xsrc || (size_t)K * 2 <= NH_ZERO_BYTES, "grouped gemm nn + swiglu with gather: K=%d exceeds %d", K, NH_ZERO_BYTES / 2);
    ProbUpload up; int slot;
    const RowBytes rb = {xsrc ? sizeof(int) : (size_t)K * 2, (size_t)N * 4, 0, (size_t)N * 2, (size_t)N * 4};
    int rc = qlmx_upload_problems_split(gate, up_, nprob, GEMM_NN, K, N, NH_BM, NH_BN / 2, &rb, st, &up, &slot); if(rc) return rc;
    if(up.ntiles == 0) return QLMX_OK;
    NhArgs a; a.pr = up.dev; a.nprob = up.nprob; a.ntiles = up.ntiles; a.nfull = up.nfull; a.tiles_n = N / (NH_BN / 2); a.d = d; a.s = s; a.K = K; a.N = N;
    a.xsrc = (const char *)xsrc; a.out = nullptr; a.gate = nullptr;
    a.gshift = 0; while((1 << a.gshift) < group) a.gshift++;
    const int grid = qx_lpt_grid(up.nfull, up.ntiles, a.tiles_n);
    if(xsrc) hipLaunchKernelGGL(k_gemm_nn_h_swiglu<NH_GATHER>, dim3(grid), dim3(256), 0, st, a);
    else     hipLaunchKernelGGL(k_gemm_nn_h_swiglu<NH_PLAIN>,  dim3(grid), dim3(256), 0, st, a);
    QLMX_LAUNCH_CHECK("grouped gemm nn + swiglu (fp16 matrix core) launch");
    return qlmx_upload_done(slot, st);
}
