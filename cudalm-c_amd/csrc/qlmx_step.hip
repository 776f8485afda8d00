/* qlmx_step.hip -- Integer AdamW / integer Lion update + moment requantisation for gfx950.
 *
 * Replaces qlm_step_launch and its two kernels (qlm.cuh:181-397; CPU twin cpu_kern.h:798-852).
 * The arithmetic is the reference's, operation for operation and in the same order, compiled
 * without FMA contraction: every float feeds a stochastic-rounding compare, so one ulp flips
 * integer state. Divisions and square roots are the correctly rounded ones.
 *
 * Mapping. The reference gives a CUDA block (or a 32-lane warp) to each group. Here a group
 * belongs to one DPP row (16 lanes) of a 64-lane wavefront, so a wave carries four groups and a
 * 256-thread workgroup sixteen. With the headline group of 128 each lane owns 8 consecutive
 * elements: one 32-bit word of packed digits, one 64-bit word each of residuals and of both
 * moments, two 128-bit words of gradient. A lane therefore writes whole bytes it alone owns, and
 * the reference's cross-lane nibble exchange (qlm.cuh:349-352) disappears. The two group maxima are
 * reduced inside the row with four DPP steps. Any other group size, a short tail group or an
 * unaligned span takes the pair-per-lane path in the same kernel (a lane still owns whole bytes).
 *
 * HBM traffic per weight: read G 4 + d 0.5 + r 1 + m8 1 + v8 1, write d 0.5 + r 1 + m8 1 + v8 1
 * = 11 B, plus 20 B of scales per group (0.16 B/weight at 128) and 4 B when P is rendered.
 */
#include "qlmx_dev.h"

struct StepParams {
    float *P; const float *G;
    signed char *d; signed char *r; const float *s;
    signed char *m8; float *m8s; unsigned char *v8; float *v8s;
    const qlmx_span *sp; int nspan, group, dmax;
    float lr, b1, b2, wd, gscale; const float *gsp;
    float inv_bc1, inv_sqrt_bc2; int lrmode;
    unsigned long long t; unsigned long long *stat;
    int packed, gi_base, ng, v4;
    int vec_ok;      /* base pointers are aligned for the 128/64/32-bit accesses of the fast path */
    int mid_ok;      /* 0 <= inv_sqrt_bc2 <= 2^10: the mid-range forms of the fast path may be tried */
    /* touched-group form (k_ng_q4_step, cudalm.cu:4472): team w steps group touched[w] of one span
     * that starts at element 0, and its gradient is the compact row Gc[w*group ..] */
    const int *touched; qlmx_span one;
};

struct GroupCtx {           /* per-group constants, uniform over the row */
    float sg, L, dec, ms_old, vs_old, veps, gs;
    float b1, b2, omb1, omb2, inv_bc1, inv_sqrt_bc2;
    int dmax, v4;
};

struct ElemRes { float mn, rv; int dd, rr, idl, carry; };

/* Division of many values by one per-group divisor (the requantisation of the moments, qlm.cuh:261-278).
 * With y = 1/b correctly rounded (one real division per group), q = a*y, r = fma(-q, b, a) exact and
 * q' = fma(r, y, q), q' is the correctly rounded a/b (Markstein's final-step theorem) as long as nothing
 * leaves the normal range; checked against a/b on 4e9 pairs on the CPU. The short form is used only
 * when b is in [2^-60, 2^60] (|a| is at most 255 b here); quotients so small that r is subnormal are
 * far below 2^-24 and round stochastically to the same integer either way. Anything else divides. */
struct GroupDiv { float b, y; bool fast; };
__device__ __forceinline__ GroupDiv qx_mkdiv(float b){
    GroupDiv d; d.b = b; d.fast = b >= 0x1p-60f && b <= 0x1p60f; d.y = 1.0f / b; return d;
}
__device__ __forceinline__ float qx_gdiv(float a, const GroupDiv &d){
    if(d.fast){ const float q = a * d.y; const float r = fmaf(-q, d.b, a); return fmaf(r, d.y, q); }
    return a / d.b;
}

/* Correctly rounded square root for a whole row of values at a lower price. sqrtf() as the compiler expands it
 * is v_sqrt_f32 (good to one unit in the last place) followed by a test of both neighbours through exact
 * residuals, wrapped in a rescaling for subnormal inputs and a pass-through for 0 and infinity: 17 instructions.
 * For x >= 2^-96 the wrapping does nothing, and what is left -- the same instruction, the same two tests, hence the
 * same bits -- takes 9. The caller uses this form only when every lane's values are above the bound (a wavefront-
 * uniform choice) and sqrtf() otherwise; infinity passes through both. */
__device__ __forceinline__ float qx_sqrt_above_2m96(float x){
    const float s = __builtin_amdgcn_sqrtf(x);
    const float dn = __uint_as_float(__float_as_uint(s) - 1u), up = __uint_as_float(__float_as_uint(s) + 1u);
    const float rdn = __builtin_fmaf(-dn, s, x), rup = __builtin_fmaf(-up, s, x);
    float r = rdn <= 0.0f ? dn : s;
    r = rup > 0.0f ? up : r;
    return r;
}
/* ---- the usual case of the 8-weights-per-lane path ----
 * The kernel is bound by the number of vector instructions it issues (single-instruction loops on the device: every
 * vector instruction takes a SIMD's issue slot for four cycles, rcp and sqrt for eight; the two-cycle rate of plain
 * fp32 / integer adds, multiplies and logic only appears when all wavefronts of a SIMD run nothing else, never in a
 * mix). The forms below therefore drop instructions that do nothing for operands in the middle of the range: the
 * correctly rounded division without its scaling and special-case steps, the row maxima as one DPP instruction per
 * step. They are checked against `/` on the device over billions of operand pairs; values outside the guarded
 * ranges take the general code. */
/* correctly rounded n / d for d in [2^-40, 2^40] and n = 0 or |n| in [2^-40, 2^40]: the compiler's division
 * sequence without v_div_scale (which leaves such operands alone), with a plain FMA for v_div_fmas and without
 * v_div_fixup */
__device__ __forceinline__ float qx_div_mid(float n, float d){
    const float y0 = __builtin_amdgcn_rcpf(d);
    const float e = __builtin_fmaf(-d, y0, 1.0f);
    const float y1 = __builtin_fmaf(e, y0, y0);
    const float q0 = n * y1;
    const float r0 = __builtin_fmaf(-d, q0, n);
    const float q1 = __builtin_fmaf(r0, y1, q0);
    const float r1 = __builtin_fmaf(-d, q1, n);
    return __builtin_fmaf(r1, y1, q1);
}
/* qx_hash of a key that already carries the hash's additive constant; returns u = top 24 bits * 2^-24 */
__device__ __forceinline__ float qx_hash_unit(uint64_t x){
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    const uint32_t h = (uint32_t)(x ^ (x >> 31));
    return (float)(h >> 8) * (1.0f / 16777216.0f);
}
/* row maximum of non-negative floats, as unsigned integers (same order, no NaN quieting in between): one
 * instruction per step; a DPP operand needs two idle cycles after the instruction that wrote its register */
__device__ __forceinline__ float qx_row16_max_nonneg(float f){
    uint32_t v = __float_as_uint(f);
    asm("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf" : "+v"(v));
    return __uint_as_float(v);
}
/* the same over the 8 lanes of a half row (lanes 0-7 and 8-15 of every row of 16 separately) */
__device__ __forceinline__ float qx_row8_max_nonneg(float f){
    uint32_t v = __float_as_uint(f);
    asm("s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf" : "+v"(v));
    return __uint_as_float(v);
}
/* byte `B` of `word` = low byte of a - b, the other bytes kept (a sub-dword destination instead of a subtract and
 * a funnel shift) */
template<int B> __device__ __forceinline__ void qx_sub_to_byte(uint32_t &word, int a, int b){
    if(B == 0) asm("v_sub_u32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(a), "v"(b));
    if(B == 1) asm("v_sub_u32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(a), "v"(b));
    if(B == 2) asm("v_sub_u32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(a), "v"(b));
    if(B == 3) asm("v_sub_u32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(word) : "v"(a), "v"(b));
}
__device__ __forceinline__ int qx_med3i(int v, int lo, int hi){            /* clamp in one instruction; lo <= hi */
    int r; asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(v), "v"(lo), "v"(hi)); return r;
}
/* the carry of a residual that left [-64, 64] (qlm.cuh:232-236: rr > 64 ? ((rr-65)>>7)+1 : rr < -64 ? -(((-rr-65)>>7)+1) : 0)
 * without branches: for rr >= 0 that is (rr + 63) >> 7, for rr < 0 it is floor((rr + 64) / 128), i.e. the same
 * shift of rr + 63 + 1. Checked against the branching form over all of [-40000, 40000] on the host. */
__host__ __device__ __forceinline__ int qx_carry(int rr){ return (rr + 63 - (rr >> 31)) >> 7; }

/* New first moment, new (stored form of the) second moment and the clamped Adam ratio u of one
 * element: qlm.cuh:209-229. */
template<bool ADAM>
__device__ __forceinline__ void elem_moments(const GroupCtx &c, float graw, int m8v, int v8v,
                                             float &mn, float &rvs, float &u){
    float gr = graw * c.gs;
    float mv = (float)m8v * c.ms_old;
    if(ADAM){
        float sv = (float)v8v * c.vs_old; if(c.v4) sv = sv * sv;
        float vv = sv * sv;
        mn = c.b1 * mv + c.omb1 * gr;
        vv = c.b2 * vv + c.omb2 * gr * gr;
        float rv = sqrtf(vv);
        u = (mn * c.inv_bc1) / (rv * c.inv_sqrt_bc2 + c.veps);
        u = fmaxf(-8.0f, fminf(8.0f, u));
        rvs = c.v4 ? sqrtf(rv) : rv;
    } else {
        float cc = c.b1 * mv + c.omb1 * gr;
        u = (float)((cc > 0.0f) - (cc < 0.0f));
        mn = c.b2 * mv + c.omb2 * gr;
        rvs = 0.0f;
    }
}

/* One element of qlm.cuh:207-242. `key` is the finished hash key of (element, step). */
template<bool ADAM>
__device__ __forceinline__ ElemRes step_elem(const GroupCtx &c, float graw, int m8v, int v8v,
                                             int dd, int rold, uint64_t key){
    ElemRes o; float u;
    elem_moments<ADAM>(c, graw, m8v, v8v, o.mn, o.rv, u);
    o.idl = qx_sround(-(c.L * u + c.dec * (float)dd), key);
    int rr = rold + o.idl;
    int cy = 0;
    if(rr > 64)       cy =  (((rr - 65) >> 7) + 1);
    else if(rr < -64) cy = -((((-rr) - 65) >> 7) + 1);
    o.carry = cy;
    o.rr = rr - cy * 128;
    o.dd = qx_clamp(dd + cy, -c.dmax, c.dmax);
    return o;
}

/* One full, aligned group of 128 for a row of 16 lanes, Adam, no statistics, operands in the middle of the range.
 * Nothing is stored before the guards have passed for the whole wavefront; when they fail the function returns
 * false and the caller runs the general code on the same registers. Guards (each makes a short form exact, none
 * changes a result): second moments >= 2^-96 with roots <= 2^25, |m * inv_bc1| in [2^-40, 2^40] (zero excluded, so
 * that the quotient's residuals cannot underflow), the lane's largest |m| in [2^-32, 2^40], eps <= 2^20; the launch
 * checks 0 <= inv_sqrt_bc2 <= 2^10 on the host (a.mid_ok). */
template<bool HASP, bool V4>
__device__ __forceinline__ bool step_row8_mid(const StepParams &a, const GroupCtx &c, int gi, int lane16, uint64_t q, uint64_t pofe,
                                              const float (&gv)[8], uint32_t dw, uint2 rw, uint2 mw, uint2 vw,
                                              uint64_t kt, uint64_t ktm, uint64_t ktv){
    float mn[8], vv[8], rv[8], uu[8];
    float vmin = 3.0e38f, amin = 3.0e38f, am = 0.0f, vm = 0.0f;
#pragma unroll
    for(int k = 0; k < 8; k++){
        const uint32_t mword = k < 4 ? mw.x : mw.y, vword = k < 4 ? vw.x : vw.y;
        const int sh = 8 * (k & 3);
        const float gr = gv[k] * c.gs;
        const float mv = (float)(int)(signed char)(mword >> sh) * c.ms_old;
        float sv = (float)((vword >> sh) & 0xFFu) * c.vs_old; if(V4) sv = sv * sv;
        mn[k] = c.b1 * mv + c.omb1 * gr;
        vv[k] = c.b2 * (sv * sv) + c.omb2 * gr * gr;
        vmin = fminf(vmin, vv[k]);
        amin = fminf(amin, fabsf(mn[k])); am = fmaxf(am, fabsf(mn[k]));
    }
    if(__builtin_amdgcn_ballot_w64(!(vmin >= 0x1p-96f)) != 0) return false;        /* NaN compares false */
#pragma unroll
    for(int k = 0; k < 8; k++){
        rv[k] = qx_sqrt_above_2m96(vv[k]);
        const float u = qx_div_mid(mn[k] * c.inv_bc1, rv[k] * c.inv_sqrt_bc2 + c.veps);
        uu[k] = __builtin_amdgcn_fmed3f(u, -8.0f, 8.0f);
        vm = fmaxf(vm, rv[k]);                           /* the guard wants the plain root also when V4 */
    }
    {   /* operands outside these ranges made the loop above compute garbage, which is dropped */
        const float nlo = amin * c.inv_bc1, nhi = am * c.inv_bc1;
        const bool lane_ok = vm <= 0x1p25f && nlo >= 0x1p-40f && nhi <= 0x1p40f && am >= 0x1p-32f && am <= 0x1p40f && c.veps <= 0x1p20f;
        if(__builtin_amdgcn_ballot_w64(!lane_ok) != 0) return false;
    }
    if(V4){
        vm = 0.0f;
#pragma unroll
        for(int k = 0; k < 8; k++){ rv[k] = qx_sqrt_above_2m96(rv[k]); vm = fmaxf(vm, rv[k]); }   /* stored as the fourth root, in [2^-24, 2^13] */
    }
    /* ---- digits and residuals (qlm.cuh:230-242) ---- */
    uint64_t ki = QLMX_KI;
    asm volatile("" : "+s"(ki));
    int dlo = -c.dmax, dhi = c.dmax;
    asm volatile("" : "+v"(dlo), "+v"(dhi));
    const uint64_t key0 = q * QLMX_KI + 0x9E3779B97F4A7C15ULL;       /* the hash's own additive constant rides along */
    float pv[8];
    uint32_t dnew = 0, rn0 = 0, rn1 = 0;
    uint64_t key = key0 + kt;
#pragma unroll
    for(int k = 0; k < 8; k++){
        const uint32_t rword = k < 4 ? rw.x : rw.y;
        const int rold = (int)(signed char)(rword >> (8 * (k & 3)));
        const int dd = qx_nib(dw, k);
        const float v = -(c.L * uu[k] + c.dec * (float)dd);
        const float fl = floorf(v);
        const int rr0 = rold + (int)fl + (qx_hash_unit(key) < (v - fl) ? 1 : 0);
        const int cyv = rr0 + 63 - (rr0 >> 31);
        const int cy = cyv >> 7;                                       /* qx_carry(rr0) */
        /* the new residual rr0 - 128 cy, of which only the low byte is kept: 128 cy and cyv agree from bit 7 up */
        if(k == 0) qx_sub_to_byte<0>(rn0, rr0, cyv & 0x80); if(k == 1) qx_sub_to_byte<1>(rn0, rr0, cyv & 0x80);
        if(k == 2) qx_sub_to_byte<2>(rn0, rr0, cyv & 0x80); if(k == 3) qx_sub_to_byte<3>(rn0, rr0, cyv & 0x80);
        if(k == 4) qx_sub_to_byte<0>(rn1, rr0, cyv & 0x80); if(k == 5) qx_sub_to_byte<1>(rn1, rr0, cyv & 0x80);
        if(k == 6) qx_sub_to_byte<2>(rn1, rr0, cyv & 0x80); if(k == 7) qx_sub_to_byte<3>(rn1, rr0, cyv & 0x80);
        const int dn = qx_med3i(dd + cy, dlo, dhi);
        if(HASP) pv[k] = c.sg * (float)dn;
        dnew = __builtin_amdgcn_alignbit((uint32_t)dn, dnew, 4);
        key += ki;
    }
    *(uint32_t *)(a.d + (q >> 1)) = dnew;
    *(uint2 *)(a.r + q) = make_uint2(rn0, rn1);
    if(HASP){
        typedef float f4 __attribute__((ext_vector_type(4)));
        f4 p0 = {pv[0], pv[1], pv[2], pv[3]}, p1 = {pv[4], pv[5], pv[6], pv[7]};
        __builtin_nontemporal_store(p0, (f4 *)(a.P + pofe));
        __builtin_nontemporal_store(p1, (f4 *)(a.P + pofe + 4));
    }
    /* ---- fresh scales and the re-quantised moments (qlm.cuh:244-278); both maxima are positive here ---- */
    am = qx_row16_max_nonneg(am); vm = qx_row16_max_nonneg(vm);
    const float ms = qx_div_mid(am, 127.0f), vs = qx_div_mid(vm, 255.0f);
    const float ym = qx_div_mid(1.0f, ms), yv = qx_div_mid(1.0f, vs);      /* ms, vs in [2^-40, 2^34]: qx_gdiv's reciprocal form holds */
    if(lane16 == 0){ a.m8s[gi] = ms; a.v8s[gi] = vs; }
    uint32_t mo0 = 0, mo1 = 0, vo0 = 0, vo1 = 0;
    uint64_t keym = key0 + ktm, keyv = key0 + ktv;
#pragma unroll
    for(int k = 0; k < 8; k++){
        const float t = mn[k] * ym;
        /* clamped before the rounding instead of after it: above 127 both give 127, below -127 both give -127
         * (floor -128 or lower, plus at most one), in between nothing is clamped */
        const float qm = __builtin_amdgcn_fmed3f(fmaf(fmaf(-t, ms, mn[k]), ym, t), -127.0f, 127.0f);
        const float w = rv[k] * yv, qv = fmaf(fmaf(-w, vs, rv[k]), yv, w);
        {
            const float fl = floorf(qm);
            const int mq = (int)fl + (qx_hash_unit(keym) < (qm - fl) ? 1 : 0);
            if(k < 4) mo0 = __builtin_amdgcn_alignbit((uint32_t)mq, mo0, 8); else mo1 = __builtin_amdgcn_alignbit((uint32_t)mq, mo1, 8);
        }
        {
            /* floor + increment stay whole numbers in floating point; the packing conversion saturates to [0, 255]
             * (the clamp of qlm.cuh:274); a positive moment never rounds to the code 0 (qlm.cuh:275), and every
             * root is positive on this path */
            const float fl = floorf(qv);
            const float vq = fmaxf(fl + (qx_hash_unit(keyv) < (qv - fl) ? 1.0f : 0.0f), 1.0f);
            if(k < 4) vo0 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo0); else vo1 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo1);
        }
        keym += ki; keyv += ki;
    }
    *(uint2 *)(a.m8 + q) = make_uint2(mo0, mo1);
    *(uint2 *)(a.v8 + q) = make_uint2(vo0, vo1);
    return true;
}

/* The same for a group spread over 8 lanes: a lane owns two runs of 8 weights, elements 8 l .. 8 l + 7 and
 * 64 + 8 l .. 64 + 8 l + 7 of its group, so that every access of a half row still covers 256 contiguous bytes of G
 * (64 of the byte arrays), a wavefront steps 8 groups, and what a lane works out once per group -- the span, the
 * addresses, the scales, the learning-rate quotient, the new scales and their reciprocals -- is spread over 16
 * weights instead of 8. Same arithmetic per element and the same guards as step_row8_mid, hence the same bytes;
 * qg, pofg, gofg are the positions of the group's first weight in the byte arrays, in P and in G. */
template<bool HASP, bool V4>
__device__ __forceinline__ bool step_row16_mid(const StepParams &a, const GroupCtx &c, int gi, int lane8, uint64_t qg, uint64_t pofg, uint64_t gofg,
                                               uint64_t kt, uint64_t ktm, uint64_t ktv){
    float mn[2][8], rv[2][8], uu[2][8];
    uint32_t dw[2]; uint2 rw[2];
    float vmin = 3.0e38f, amin = 3.0e38f, am = 0.0f, vm = 0.0f;
#pragma unroll
    for(int h = 0; h < 2; h++){
        const uint64_t e = (uint64_t)(h * 64 + lane8 * 8);
        const float4 h0 = *(const float4 *)(a.G + gofg + e), h1 = *(const float4 *)(a.G + gofg + e + 4);
        const uint2 mw = *(const uint2 *)(a.m8 + qg + e), vw = *(const uint2 *)(a.v8 + qg + e);
        dw[h] = *(const uint32_t *)(a.d + ((qg + e) >> 1));
        rw[h] = *(const uint2 *)(a.r + qg + e);
        const float gv[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
#pragma unroll
        for(int k = 0; k < 8; k++){
            const uint32_t mword = k < 4 ? mw.x : mw.y, vword = k < 4 ? vw.x : vw.y;
            const int sh = 8 * (k & 3);
            const float gr = gv[k] * c.gs;
            const float mv = (float)(int)(signed char)(mword >> sh) * c.ms_old;
            float sv = (float)((vword >> sh) & 0xFFu) * c.vs_old; if(V4) sv = sv * sv;
            mn[h][k] = c.b1 * mv + c.omb1 * gr;
            rv[h][k] = c.b2 * (sv * sv) + c.omb2 * gr * gr;                /* the second moment; its root below */
            vmin = fminf(vmin, rv[h][k]);
            amin = fminf(amin, fabsf(mn[h][k])); am = fmaxf(am, fabsf(mn[h][k]));
        }
    }
    if(__builtin_amdgcn_ballot_w64(!(vmin >= 0x1p-96f)) != 0) return false;        /* NaN compares false */
#pragma unroll
    for(int h = 0; h < 2; h++)
#pragma unroll
        for(int k = 0; k < 8; k++){
            rv[h][k] = qx_sqrt_above_2m96(rv[h][k]);
            const float u = qx_div_mid(mn[h][k] * c.inv_bc1, rv[h][k] * c.inv_sqrt_bc2 + c.veps);
            uu[h][k] = __builtin_amdgcn_fmed3f(u, -8.0f, 8.0f);
            vm = fmaxf(vm, rv[h][k]);                    /* the guard wants the plain root also when V4 */
        }
    {
        const float nlo = amin * c.inv_bc1, nhi = am * c.inv_bc1;
        const bool lane_ok = vm <= 0x1p25f && nlo >= 0x1p-40f && nhi <= 0x1p40f && am >= 0x1p-32f && am <= 0x1p40f && c.veps <= 0x1p20f;
        if(__builtin_amdgcn_ballot_w64(!lane_ok) != 0) return false;
    }
    if(V4){
        vm = 0.0f;
#pragma unroll
        for(int h = 0; h < 2; h++)
#pragma unroll
            for(int k = 0; k < 8; k++){ rv[h][k] = qx_sqrt_above_2m96(rv[h][k]); vm = fmaxf(vm, rv[h][k]); }
    }
    /* ---- digits and residuals (qlm.cuh:230-242) ---- */
    uint64_t ki = QLMX_KI;
    asm volatile("" : "+s"(ki));
    int dlo = -c.dmax, dhi = c.dmax;
    asm volatile("" : "+v"(dlo), "+v"(dhi));
    uint64_t key0[2];
#pragma unroll
    for(int h = 0; h < 2; h++){
        const uint64_t e = (uint64_t)(h * 64 + lane8 * 8), q = qg + e;
        key0[h] = q * QLMX_KI + 0x9E3779B97F4A7C15ULL;                   /* the hash's own additive constant rides along */
        float pv[8];
        uint32_t dnew = 0, rn0 = 0, rn1 = 0;
        uint64_t key = key0[h] + kt;
#pragma unroll
        for(int k = 0; k < 8; k++){
            const uint32_t rword = k < 4 ? rw[h].x : rw[h].y;
            const int rold = (int)(signed char)(rword >> (8 * (k & 3)));
            const int dd = qx_nib(dw[h], k);
            const float v = -(c.L * uu[h][k] + c.dec * (float)dd);
            const float fl = floorf(v);
            const int rr0 = rold + (int)fl + (qx_hash_unit(key) < (v - fl) ? 1 : 0);
            const int cyv = rr0 + 63 - (rr0 >> 31);
            const int cy = cyv >> 7;                                       /* qx_carry(rr0) */
            if(k == 0) qx_sub_to_byte<0>(rn0, rr0, cyv & 0x80); if(k == 1) qx_sub_to_byte<1>(rn0, rr0, cyv & 0x80);
            if(k == 2) qx_sub_to_byte<2>(rn0, rr0, cyv & 0x80); if(k == 3) qx_sub_to_byte<3>(rn0, rr0, cyv & 0x80);
            if(k == 4) qx_sub_to_byte<0>(rn1, rr0, cyv & 0x80); if(k == 5) qx_sub_to_byte<1>(rn1, rr0, cyv & 0x80);
            if(k == 6) qx_sub_to_byte<2>(rn1, rr0, cyv & 0x80); if(k == 7) qx_sub_to_byte<3>(rn1, rr0, cyv & 0x80);
            const int dn = qx_med3i(dd + cy, dlo, dhi);
            if(HASP) pv[k] = c.sg * (float)dn;
            dnew = __builtin_amdgcn_alignbit((uint32_t)dn, dnew, 4);
            key += ki;
        }
        *(uint32_t *)(a.d + (q >> 1)) = dnew;
        *(uint2 *)(a.r + q) = make_uint2(rn0, rn1);
        if(HASP){
            typedef float f4 __attribute__((ext_vector_type(4)));
            f4 p0 = {pv[0], pv[1], pv[2], pv[3]}, p1 = {pv[4], pv[5], pv[6], pv[7]};
            __builtin_nontemporal_store(p0, (f4 *)(a.P + pofg + e));
            __builtin_nontemporal_store(p1, (f4 *)(a.P + pofg + e + 4));
        }
    }
    /* ---- fresh scales and the re-quantised moments (qlm.cuh:244-278); both maxima are positive here ---- */
    am = qx_row8_max_nonneg(am); vm = qx_row8_max_nonneg(vm);
    const float ms = qx_div_mid(am, 127.0f), vs = qx_div_mid(vm, 255.0f);
    const float ym = qx_div_mid(1.0f, ms), yv = qx_div_mid(1.0f, vs);
    if(lane8 == 0){ a.m8s[gi] = ms; a.v8s[gi] = vs; }
#pragma unroll
    for(int h = 0; h < 2; h++){
        const uint64_t q = qg + (uint64_t)(h * 64 + lane8 * 8);
        uint32_t mo0 = 0, mo1 = 0, vo0 = 0, vo1 = 0;
        uint64_t keym = key0[h] + ktm, keyv = key0[h] + ktv;
#pragma unroll
        for(int k = 0; k < 8; k++){
            const float t = mn[h][k] * ym;
            const float qm = __builtin_amdgcn_fmed3f(fmaf(fmaf(-t, ms, mn[h][k]), ym, t), -127.0f, 127.0f);
            const float w = rv[h][k] * yv, qv = fmaf(fmaf(-w, vs, rv[h][k]), yv, w);
            {
                const float fl = floorf(qm);
                const int mq = (int)fl + (qx_hash_unit(keym) < (qm - fl) ? 1 : 0);
                if(k < 4) mo0 = __builtin_amdgcn_alignbit((uint32_t)mq, mo0, 8); else mo1 = __builtin_amdgcn_alignbit((uint32_t)mq, mo1, 8);
            }
            {
                const float fl = floorf(qv);
                const float vq = fmaxf(fl + (qx_hash_unit(keyv) < (qv - fl) ? 1.0f : 0.0f), 1.0f);
                if(k < 4) vo0 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo0); else vo1 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo1);
            }
            keym += ki; keyv += ki;
        }
        *(uint2 *)(a.m8 + q) = make_uint2(mo0, mo1);
        *(uint2 *)(a.v8 + q) = make_uint2(vo0, vo1);
    }
    return true;
}

/* STAT: the four counters are kept; HASP: the fp32 view is written; V4: the second moment is stored as its
 * fourth root (a.v4). All are fixed per launch, so they are template parameters and the usual launch (none of
 * them) carries no trace of them: as a run-time flag, v4 made the compiler compute the second square root of
 * every element and select (18 of 186 vector instructions per weight). */
template<bool ADAM, bool STAT, bool HASP, bool V4>
__device__ __forceinline__ void step_team(const StepParams &a, const int team, const int lane16){
    if(team >= a.ng) return;                       /* whole rows leave together */
    const int gi = a.touched ? a.touched[team] : a.gi_base + team;
    const qlmx_span S = a.touched ? a.one : a.sp[qx_span_of(a.sp, a.nspan, gi)];
    const uint64_t j0 = (uint64_t)(gi - S.gi0) * (uint64_t)a.group;
    const uint64_t left = S.n - j0;
    const int n = (int)((uint64_t)a.group < left ? (uint64_t)a.group : left);
    const uint64_t pof = S.pof + j0, qi0 = S.qi0 + j0;
    const uint64_t gof = a.touched ? (uint64_t)team * (uint64_t)a.group : S.gof + j0;

    GroupCtx c;
    c.gs = a.gsp ? *a.gsp : a.gscale;
    c.sg = a.s[gi];
    c.L = a.lr * 128.0f / (a.lrmode ? c.sg : S.sref);
    c.dec = a.lr * a.wd * 128.0f;
    c.ms_old = a.m8s[gi];
    c.vs_old = (ADAM && a.v8s) ? a.v8s[gi] : 0.0f;
    { float q1 = 1.0f * c.vs_old; if(V4) q1 = q1 * q1; c.veps = fmaxf(q1, 1e-8f); }
    c.b1 = a.b1; c.b2 = a.b2; c.omb1 = 1.0f - a.b1; c.omb2 = 1.0f - a.b2;
    c.inv_bc1 = a.inv_bc1; c.inv_sqrt_bc2 = a.inv_sqrt_bc2;
    c.dmax = a.dmax; c.v4 = V4;

    const uint64_t kt  = a.t * QLMX_KT;
    const uint64_t ktm = kt + 0x5EEDULL * QLMX_KT;
    const uint64_t ktv = kt + 0xBEEFULL * QLMX_KT;

    unsigned long long st_carry = 0, st_rail = 0, st_zero = 0, st_idl = 0;
    const bool want_stat = STAT;

    const bool fast = a.vec_ok && a.group == 128 && a.packed && n == 128 && ((pof | qi0 | gof) & 7ULL) == 0;
    if(fast){
        const uint64_t e0 = (uint64_t)lane16 * 8;
        const uint64_t q = qi0 + e0;
        if(ADAM && !STAT && a.mid_ok){
            const float4 h0 = *(const float4 *)(a.G + gof + e0);
            const float4 h1 = *(const float4 *)(a.G + gof + e0 + 4);
            const float hv[8] = {h0.x, h0.y, h0.z, h0.w, h1.x, h1.y, h1.z, h1.w};
            if(step_row8_mid<HASP, V4>(a, c, gi, lane16, q, pof + e0, hv, *(const uint32_t *)(a.d + (q >> 1)), *(const uint2 *)(a.r + q),
                                       *(const uint2 *)(a.m8 + q), *(const uint2 *)(a.v8 + q), kt, ktm, ktv)) return;
            /* nothing was stored; the general code loads its operands again rather than keep them in registers
             * across the attempt (the barrier keeps the compiler from merging the two sets of loads) */
            asm volatile("" ::: "memory");
        }
        const float4 g0 = *(const float4 *)(a.G + gof + e0);
        const float4 g1 = *(const float4 *)(a.G + gof + e0 + 4);
        const uint32_t dw = *(const uint32_t *)(a.d + (q >> 1));
        const uint2 rw = *(const uint2 *)(a.r + q);
        const uint2 mw = *(const uint2 *)(a.m8 + q);
        uint2 vw = make_uint2(0u, 0u);
        if(ADAM) vw = *(const uint2 *)(a.v8 + q);
        const float gv[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
        float mn[8], rv[8], uu[8];
        /* ---- moments (qlm.cuh:209-229); the square roots of a lane's eight values are taken together ---- */
        if(ADAM){
            float vv[8], vmin = 1.0f;
#pragma unroll
            for(int k = 0; k < 8; k++){
                const uint32_t mword = k < 4 ? mw.x : mw.y, vword = k < 4 ? vw.x : vw.y;
                const int sh = 8 * (k & 3);
                const float gr = gv[k] * c.gs;
                const float mv = (float)(int)(signed char)(mword >> sh) * c.ms_old;
                float sv = (float)((vword >> sh) & 0xFFu) * c.vs_old; if(V4) sv = sv * sv;
                mn[k] = c.b1 * mv + c.omb1 * gr;
                vv[k] = c.b2 * (sv * sv) + c.omb2 * gr * gr;
                vmin = fminf(vmin, vv[k]);
            }
            /* NaN compares false and takes the general form with the rest of its wavefront */
            if(__builtin_amdgcn_ballot_w64(!(vmin >= 0x1p-96f)) == 0){
#pragma unroll
                for(int k = 0; k < 8; k++) rv[k] = qx_sqrt_above_2m96(vv[k]);
            } else {
#pragma unroll
                for(int k = 0; k < 8; k++) rv[k] = sqrtf(vv[k]);
            }
#pragma unroll
            for(int k = 0; k < 8; k++){
                const float u = (mn[k] * c.inv_bc1) / (rv[k] * c.inv_sqrt_bc2 + c.veps);
                uu[k] = fmaxf(-8.0f, fminf(8.0f, u));
                if(V4) rv[k] = sqrtf(rv[k]);
            }
        } else {
#pragma unroll
            for(int k = 0; k < 8; k++){
                const uint32_t mword = k < 4 ? mw.x : mw.y;
                float r0;
                elem_moments<false>(c, gv[k], (int)(signed char)(mword >> (8 * (k & 3))), 0, mn[k], r0, uu[k]);
                rv[k] = r0;
            }
        }
        /* ---- digits and residuals (qlm.cuh:230-242). Every new byte or nibble enters its word from the top
         * (one funnel shift each), so after all eight the first element sits lowest. ---- */
        float pv[8];
        uint32_t dnew = 0, rn0 = 0, rn1 = 0;
        float am = 0.0f, vm = 0.0f;
        /* The hash keys of the lane's eight elements are kept as running sums: the element stride as a value the
         * compiler cannot see through (left as the literal, every key is rebuilt as q * KI + k * KI with the
         * second product moved into a register pair first: five instructions per key instead of one), and the
         * three step offsets added once. The clamp bounds likewise live in registers of their own: v_med3_i32
         * takes one scalar operand at most, and without this both were copied into registers per element. */
        uint64_t ki = QLMX_KI;
        asm volatile("" : "+s"(ki));
        int dlo = -c.dmax, dhi = c.dmax, mlo = -127, mhi = 127;
        asm volatile("" : "+v"(dlo), "+v"(dhi), "+v"(mlo), "+v"(mhi));
        const uint64_t key0 = q * QLMX_KI;
        uint64_t key = key0 + kt;
#pragma unroll
        for(int k = 0; k < 8; k++){
            const uint32_t rword = k < 4 ? rw.x : rw.y;
            const int rold = (int)(signed char)(rword >> (8 * (k & 3)));
            const int dd = qx_nib(dw, k);
            const int idl = qx_sround(-(c.L * uu[k] + c.dec * (float)dd), key);
            const int rr0 = rold + idl;
            const int cy = qx_carry(rr0);
            const int rr = rr0 - cy * 128;
            const int dn = qx_med3i(dd + cy, dlo, dhi);
            if(HASP) pv[k] = c.sg * (float)dn;
            dnew = __builtin_amdgcn_alignbit((uint32_t)dn, dnew, 4);
            if(k < 4) rn0 = __builtin_amdgcn_alignbit((uint32_t)rr, rn0, 8); else rn1 = __builtin_amdgcn_alignbit((uint32_t)rr, rn1, 8);
            am = fmaxf(am, fabsf(mn[k])); vm = fmaxf(vm, rv[k]);
            if(STAT){
                unsigned ai = (unsigned)(idl < 0 ? -idl : idl);
                st_idl = st_idl > ai ? st_idl : ai;
                st_carry += (unsigned)(cy < 0 ? -cy : cy);
                st_rail += (dn == c.dmax) | (dn == -c.dmax);
                st_zero += (dn == 0);
            }
            key += ki;
        }
        *(uint32_t *)(a.d + (q >> 1)) = dnew;
        *(uint2 *)(a.r + q) = make_uint2(rn0, rn1);
        if(HASP){
            /* the rendered view is not read again by this launch: written past the caches */
            typedef float f4 __attribute__((ext_vector_type(4)));
            f4 p0 = {pv[0], pv[1], pv[2], pv[3]}, p1 = {pv[4], pv[5], pv[6], pv[7]};
            __builtin_nontemporal_store(p0, (f4 *)(a.P + pof + e0));
            __builtin_nontemporal_store(p1, (f4 *)(a.P + pof + e0 + 4));
        }
        /* ---- fresh scales and the re-quantised moments (qlm.cuh:244-278) ---- */
        am = qx_row16_max(am); vm = qx_row16_max(vm);
        const float ms = am > 0.0f ? am / 127.0f : 1e-12f;
        const float vs = vm > 0.0f ? vm / 255.0f : 1e-12f;
        const GroupDiv dms = qx_mkdiv(ms), dvs = qx_mkdiv(vs);
        if(lane16 == 0){ a.m8s[gi] = ms; if(ADAM) a.v8s[gi] = vs; }
        /* one choice for the wavefront: the reciprocal form when all four groups allow it (the usual case) */
        const bool recip = __builtin_amdgcn_ballot_w64(!(dms.fast && (!ADAM || dvs.fast))) == 0;
        uint32_t mo0 = 0, mo1 = 0, vo0 = 0, vo1 = 0;
        uint64_t keym = key0 + ktm, keyv = key0 + ktv;
#pragma unroll
        for(int k = 0; k < 8; k++){
            float qm, qv = 0.0f;
            if(recip){
                const float t = mn[k] * dms.y; qm = fmaf(fmaf(-t, dms.b, mn[k]), dms.y, t);
                if(ADAM){ const float w = rv[k] * dvs.y; qv = fmaf(fmaf(-w, dvs.b, rv[k]), dvs.y, w); }
            } else {
                qm = mn[k] / ms;
                if(ADAM) qv = rv[k] / vs;
            }
            const int mq = qx_med3i(qx_sround(qm, keym), mlo, mhi);
            if(k < 4) mo0 = __builtin_amdgcn_alignbit((uint32_t)mq, mo0, 8); else mo1 = __builtin_amdgcn_alignbit((uint32_t)mq, mo1, 8);
            if(ADAM){
                /* floor + stochastic increment stay in floating point (whole numbers, exact); the conversion that
                 * packs the byte saturates to [0, 255], which is the clamp of qlm.cuh:274; a positive moment
                 * never rounds to the code 0 (qlm.cuh:275) */
                const float fl = floorf(qv);
                const uint32_t h = qx_hash(keyv);
                const float ur = (float)(h >> 8) * (1.0f / 16777216.0f);
                float vq = fl + (ur < (qv - fl) ? 1.0f : 0.0f);
                vq = fmaxf(vq, rv[k] > 0.0f ? 1.0f : 0.0f);
                if(k < 4) vo0 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo0); else vo1 = __builtin_amdgcn_cvt_pk_u8_f32(vq, k & 3, vo1);
            }
            keym += ki; keyv += ki;
        }
        *(uint2 *)(a.m8 + q) = make_uint2(mo0, mo1);
        if(ADAM) *(uint2 *)(a.v8 + q) = make_uint2(vo0, vo1);
    } else {
        /* pair-per-lane path: lane owns elements {2*lane16, 2*lane16+1} + 32*k, i.e. whole bytes
         * of packed digits. Sweep one updates digits, residuals and P; sweep two recomputes the
         * moments from m8/v8/G, which sweep one does not write (same operations, hence the same
         * bits), and requantises them. Nothing is held in registers across the reduction. */
        float am = 0.0f, vm = 0.0f;
        for(int jb = 2 * lane16; jb < n; jb += 32){
            int ddn[2] = {0, 0};
            unsigned oldb = 0;
            if(a.packed) oldb = (unsigned char)a.d[(qi0 + jb) >> 1];
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int j = jb + h;
                if(j < n){
                    const uint64_t qi = qi0 + j;
                    int dd;
                    if(a.packed){ int v = h ? (int)(oldb >> 4) : (int)(oldb & 15u); dd = v >= 8 ? v - 16 : v; }
                    else dd = (int)a.d[qi];
                    ElemRes o = step_elem<ADAM>(c, a.G[gof + j], (int)a.m8[qi], ADAM ? (int)a.v8[qi] : 0, dd,
                                                (int)a.r[qi], qi * QLMX_KI + kt);
                    a.r[qi] = (signed char)o.rr;
                    if(a.P) a.P[pof + j] = c.sg * (float)o.dd;
                    if(!a.packed) a.d[qi] = (signed char)o.dd;
                    ddn[h] = o.dd;
                    am = fmaxf(am, fabsf(o.mn)); vm = fmaxf(vm, o.rv);
                    if(want_stat){
                        unsigned ai = (unsigned)(o.idl < 0 ? -o.idl : o.idl);
                        st_idl = st_idl > ai ? st_idl : ai;
                        st_carry += (unsigned)(o.carry < 0 ? -o.carry : o.carry);
                        st_rail += (o.dd == c.dmax) | (o.dd == -c.dmax);
                        st_zero += (o.dd == 0);
                    }
                }
            }
            if(a.packed) a.d[(qi0 + jb) >> 1] = (signed char)(((ddn[1] & 15) << 4) | (ddn[0] & 15));
        }
        am = qx_row16_max(am); vm = qx_row16_max(vm);
        const float ms = am > 0.0f ? am / 127.0f : 1e-12f;
        const float vs = vm > 0.0f ? vm / 255.0f : 1e-12f;
        for(int jb = 2 * lane16; jb < n; jb += 32){
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int j = jb + h;
                if(j < n){
                    const uint64_t qi = qi0 + j;
                    float mn, rvs, u;
                    elem_moments<ADAM>(c, a.G[gof + j], (int)a.m8[qi], ADAM ? (int)a.v8[qi] : 0, mn, rvs, u);
                    a.m8[qi] = (signed char)qx_clamp(qx_sround(mn / ms, qi * QLMX_KI + ktm), -127, 127);
                    if(ADAM){
                        int vq = qx_clamp(qx_sround(rvs / vs, qi * QLMX_KI + ktv), 0, 255);
                        if(vq == 0 && rvs > 0.0f) vq = 1;
                        a.v8[qi] = (unsigned char)vq;
                    }
                }
            }
        }
        /* written last: the recomputation above reads the old per-group moment scales via `c` */
        if(lane16 == 0){ a.m8s[gi] = ms; if(ADAM) a.v8s[gi] = vs; }
    }

    if(want_stat){
        /* row totals, then one lane per group updates the four counters */
        unsigned sc = (unsigned)qx_row16_sum((int)st_carry), sr = (unsigned)qx_row16_sum((int)st_rail),
                 sz = (unsigned)qx_row16_sum((int)st_zero);
        unsigned mi = (unsigned)qx_row16_maxi((int)st_idl);
        if(lane16 == 0){
            atomicAdd(&a.stat[0], (unsigned long long)sc);
            atomicAdd(&a.stat[1], (unsigned long long)sr);
            atomicAdd(&a.stat[2], (unsigned long long)sz);
            atomicMax(&a.stat[3], (unsigned long long)mi);
        }
    }
}

/* one group per row of 16 lanes: every shape, every option */
template<bool ADAM, bool STAT, bool HASP, bool V4>
__global__ void __launch_bounds__(256) k_qlmx_step(StepParams a){
    step_team<ADAM, STAT, HASP, V4>(a, (int)((blockIdx.x * (unsigned)blockDim.x + threadIdx.x) >> 4), threadIdx.x & 15);
}
/* Adam on packed groups of 128 without statistics (what a training step launches): one group per 8 lanes, eight
 * groups per wavefront, through step_row16_mid when all eight are whole, aligned groups with operands in the middle
 * of the range -- a choice per wavefront, made before anything is stored; otherwise the wavefront's groups go through
 * the code above, four at a time. */
template<bool HASP, bool V4>
__global__ void __launch_bounds__(256) k_qlmx_step_wide(StepParams a){
    const int lane = threadIdx.x & 63;
    const int g0 = (int)((blockIdx.x * (unsigned)blockDim.x + threadIdx.x) >> 6) * 8;       /* first group of the wavefront */
    if(g0 >= a.ng) return;
    if(g0 + 8 <= a.ng){
        const int gi = a.gi_base + g0 + (lane >> 3);
        const qlmx_span S = a.sp[qx_span_of(a.sp, a.nspan, gi)];
        const uint64_t j0 = (uint64_t)(gi - S.gi0) * 128u;
        const uint64_t pof = S.pof + j0, qi0 = S.qi0 + j0, gof = S.gof + j0;
        const bool whole = S.n - j0 >= 128u && ((pof | qi0 | gof) & 7ULL) == 0;
        if(__builtin_amdgcn_ballot_w64(!whole) == 0){
            GroupCtx c;
            c.gs = a.gsp ? *a.gsp : a.gscale;
            c.sg = a.s[gi];
            c.L = a.lr * 128.0f / (a.lrmode ? c.sg : S.sref);
            c.dec = a.lr * a.wd * 128.0f;
            c.ms_old = a.m8s[gi];
            c.vs_old = a.v8s[gi];
            { float q1 = 1.0f * c.vs_old; if(V4) q1 = q1 * q1; c.veps = fmaxf(q1, 1e-8f); }
            c.b1 = a.b1; c.b2 = a.b2; c.omb1 = 1.0f - a.b1; c.omb2 = 1.0f - a.b2;
            c.inv_bc1 = a.inv_bc1; c.inv_sqrt_bc2 = a.inv_sqrt_bc2;
            c.dmax = a.dmax; c.v4 = V4;
            const uint64_t kt = a.t * QLMX_KT;
            if(step_row16_mid<HASP, V4>(a, c, gi, lane & 7, qi0, pof, gof, kt, kt + 0x5EEDULL * QLMX_KT, kt + 0xBEEFULL * QLMX_KT)) return;
            asm volatile("" ::: "memory");         /* nothing was stored; the general code loads its operands itself */
        }
    }
#pragma unroll 1
    for(int p = 0; p < 2; p++) step_team<true, false, HASP, V4>(a, g0 + 4 * p + (lane >> 4), lane & 15);
}

template<bool ADAM, bool V4> static void step_launch_opt(const StepParams &a, unsigned blocks, hipStream_t st){
    const bool stat = a.stat != nullptr, hasp = a.P != nullptr;
    if(stat && hasp)  hipLaunchKernelGGL((k_qlmx_step<ADAM, true, true, V4>),   dim3(blocks), dim3(256), 0, st, a);
    else if(stat)     hipLaunchKernelGGL((k_qlmx_step<ADAM, true, false, V4>),  dim3(blocks), dim3(256), 0, st, a);
    else if(hasp)     hipLaunchKernelGGL((k_qlmx_step<ADAM, false, true, V4>),  dim3(blocks), dim3(256), 0, st, a);
    else              hipLaunchKernelGGL((k_qlmx_step<ADAM, false, false, V4>), dim3(blocks), dim3(256), 0, st, a);
}
static void step_launch(const StepParams &a, bool adam, unsigned blocks, hipStream_t st){
    /* v4 only exists for Adam's second moment (Lion keeps none) */
    if(adam){ if(a.v4) step_launch_opt<true, true>(a, blocks, st); else step_launch_opt<true, false>(a, blocks, st); }
    else step_launch_opt<false, false>(a, blocks, st);
}

static bool g_step_wide = true;
/* qlm_step_launch (qlm.cuh:377-397) */
extern "C" int qlmx_step(float *P, const float *G, signed char *d, signed char *r, const float *s,
              signed char *m8, float *m8s, unsigned char *v8, float *v8s,
              const qlmx_span *sp, int nspan, int group, int dmax,
              float lr, float b1, float b2, float wd, float gscale, const float *gsp,
              float inv_bc1, float inv_sqrt_bc2, int lrmode,
              unsigned long long t, int adam, long long *stat, int packed,
              int gi_base, int ng, int v4, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(G && d && r && s && m8 && m8s && sp, "qlmx_step: NULL buffer");
    QLMX_REQUIRE(!adam || (v8 && v8s), "qlmx_step: adam needs v8 and v8s");
    QLMX_REQUIRE(nspan > 0 && ng >= 0 && gi_base >= 0, "qlmx_step: bad span/group range");
    QLMX_REQUIRE(group >= 2 && group <= 256, "qlmx_step: group %d outside [2,256]", group);
    QLMX_REQUIRE(!packed || (dmax <= 7 && (group & 1) == 0), "qlmx_step: packed digits need dmax<=7 and an even group");
    QLMX_REQUIRE(dmax >= 1 && dmax <= 127, "qlmx_step: dmax %d", dmax);
    if(ng == 0) return QLMX_OK;
    StepParams a;
    a.P = P; a.G = G; a.d = d; a.r = r; a.s = s; a.m8 = m8; a.m8s = m8s; a.v8 = v8; a.v8s = v8s;
    a.sp = sp; a.nspan = nspan; a.group = group; a.dmax = dmax;
    a.lr = lr; a.b1 = b1; a.b2 = b2; a.wd = wd; a.gscale = gscale; a.gsp = gsp;
    a.inv_bc1 = inv_bc1; a.inv_sqrt_bc2 = inv_sqrt_bc2; a.lrmode = lrmode;
    a.t = t; a.stat = (unsigned long long *)stat; a.packed = packed; a.gi_base = gi_base; a.ng = ng; a.v4 = v4;
    a.touched = nullptr;
    a.mid_ok = inv_sqrt_bc2 >= 0.0f && inv_sqrt_bc2 <= 1024.0f;
    a.vec_ok = (((uintptr_t)P | (uintptr_t)G) & 15) == 0 && (((uintptr_t)r | (uintptr_t)m8 | (uintptr_t)v8) & 7) == 0
               && ((uintptr_t)d & 3) == 0;
    hipStream_t st = (hipStream_t)stream;
    if(adam && !stat && packed && group == 128 && a.mid_ok && a.vec_ok && g_step_wide){
        /* a training step's launch: eight groups per wavefront (k_qlmx_step_wide) */
        const unsigned wblocks = (unsigned)((ng + 31) / 32);
        if(v4){ if(P) hipLaunchKernelGGL((k_qlmx_step_wide<true, true>), dim3(wblocks), dim3(256), 0, st, a);
                else  hipLaunchKernelGGL((k_qlmx_step_wide<false, true>), dim3(wblocks), dim3(256), 0, st, a); }
        else  { if(P) hipLaunchKernelGGL((k_qlmx_step_wide<true, false>), dim3(wblocks), dim3(256), 0, st, a);
                else  hipLaunchKernelGGL((k_qlmx_step_wide<false, false>), dim3(wblocks), dim3(256), 0, st, a); }
    } else {
        const unsigned blocks = (unsigned)((ng + 15) / 16);
        step_launch(a, adam != 0, blocks, st);
    }
    QLMX_LAUNCH_CHECK("qlmx_step launch");
    return QLMX_OK;
}
/* Test hook: 0 sends every launch through the one-group-per-16-lanes kernel (the two kernels must agree byte for
 * byte), 1 (the default) lets training-shaped launches take the eight-groups-per-wavefront kernel. */
extern "C" int qlmx_test_step_wide(int on){ g_step_wide = on != 0; return QLMX_OK; }

/* k_ng_q4_step (cudalm.cu:4472-4520; CPU twin cpu_kern.h:620-648): the step restricted to a list of
 * touched groups of ONE packed 4-bit span that starts at element 0 of d/r/m8/v8/P (the n-gram
 * table). Same arithmetic as qlmx_step with adam = 1, relative LR through the frozen `sref`,
 * no statistics, clip multiplier *gs (1 when NULL); group w of the list reads its gradient from the
 * compact buffer Gc[w*group .. w*group+group). A group must appear at most once in the list. */
extern "C" int qlmx_step_touched(float *P, const float *Gc, signed char *d, signed char *r, const float *s,
              signed char *m8, float *m8s, unsigned char *v8, float *v8s,
              const int *touched_gi, int ntouched, int group, int dmax,
              float lr, float b1, float b2, float wd, float sref,
              float inv_bc1, float inv_sqrt_bc2, unsigned long long t, unsigned long long nt,
              const float *gs, int v4, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(Gc && d && r && s && m8 && m8s && v8 && v8s && touched_gi, "qlmx_step_touched: NULL buffer");
    QLMX_REQUIRE(group >= 2 && group <= 256 && (group & 1) == 0, "qlmx_step_touched: group %d must be even and in [2,256]", group);
    QLMX_REQUIRE(dmax >= 1 && dmax <= 7, "qlmx_step_touched: dmax %d (packed digits)", dmax);
    QLMX_REQUIRE(ntouched >= 0 && nt > 0, "qlmx_step_touched: bad sizes");
    if(ntouched == 0) return QLMX_OK;
    StepParams a;
    a.P = P; a.G = Gc; a.d = d; a.r = r; a.s = s; a.m8 = m8; a.m8s = m8s; a.v8 = v8; a.v8s = v8s;
    a.sp = nullptr; a.nspan = 1; a.group = group; a.dmax = dmax;
    a.lr = lr; a.b1 = b1; a.b2 = b2; a.wd = wd; a.gscale = 1.0f; a.gsp = gs;
    a.inv_bc1 = inv_bc1; a.inv_sqrt_bc2 = inv_sqrt_bc2; a.lrmode = 0;
    a.t = t; a.stat = nullptr; a.packed = 1; a.gi_base = 0; a.ng = ntouched; a.v4 = v4;
    a.vec_ok = (((uintptr_t)P | (uintptr_t)Gc) & 15) == 0 && (((uintptr_t)r | (uintptr_t)m8 | (uintptr_t)v8) & 7) == 0
               && ((uintptr_t)d & 3) == 0;
    a.touched = touched_gi;
    a.mid_ok = inv_sqrt_bc2 >= 0.0f && inv_sqrt_bc2 <= 1024.0f;
    a.one.pof = 0; a.one.gof = 0; a.one.qi0 = 0; a.one.n = nt; a.one.gi0 = 0;
    a.one.ngrp = (int)((nt + (unsigned long long)group - 1) / (unsigned long long)group); a.one.sref = sref;
    const unsigned blocks = (unsigned)((ntouched + 15) / 16);
    step_launch(a, true, blocks, (hipStream_t)stream);
    QLMX_LAUNCH_CHECK("qlmx_step_touched launch");
    return QLMX_OK;
}

/* ---- gradient-norm clipping around the step (cudalm.cu:2794-2820, CPU twins cpu_kern.h:533-546) ----
 * k_sqsum: 64 partial sums of squares; partial c covers G[n*c/64 .. n*(c+1)/64), is accumulated in
 * double and rounded to float once (the CPU path's definition; the reference's GPU kernel sums
 * strided in fp32 and differs from its own CPU kernel in the last bits). The 64 partials are the
 * contract, 64 workgroups are not: each chunk is cut into SQ_W pieces, one workgroup each (1024
 * workgroups for the 256 CUs), which sum in double -- lanes strided, then a fixed tree -- and leave
 * their sum in a device array; the workgroup that arrives last at a chunk (a counter) adds the SQ_W
 * sums in piece order, so the result does not depend on arrival order. The order of the double
 * additions is not the CPU's, which can move the double sum by a few units in its last place -- far
 * below half a float ulp except on an exact tie. The array and the counters are static device
 * memory (the last workgroup resets its counter): calls that overlap on different streams would
 * mix their pieces and are not supported. */
#define SQ_W 16
static __device__ double   g_sq_piece[64 * SQ_W];
static __device__ unsigned g_sq_count[64];
__global__ void __launch_bounds__(256) k_qlmx_sqsum(const float *G, unsigned long long n, float *part){
    __shared__ double red[256];
    const unsigned c = blockIdx.x / SQ_W, w = blockIdx.x % SQ_W;
    const unsigned long long c0 = n * c / 64, c1 = n * (c + 1) / 64, len = c1 - c0;
    const unsigned long long i0 = c0 + len * w / SQ_W, i1 = c0 + len * (w + 1) / SQ_W;
    double s = 0.0;
    /* 16-byte loads over the aligned middle, single elements at both ends */
    unsigned long long a0 = (i0 + 3) & ~3ULL; if(a0 > i1) a0 = i1;
    const unsigned long long a1 = a0 + ((i1 - a0) & ~3ULL);
    for(unsigned long long i = i0 + threadIdx.x; i < a0; i += 256){ const double g = (double)G[i]; s += g * g; }
    if((((uintptr_t)G) & 15) == 0){
        for(unsigned long long i = a0 + 4ULL * threadIdx.x; i < a1; i += 1024){
            const float4 v = *(const float4 *)(G + i);
            s += (double)v.x * (double)v.x; s += (double)v.y * (double)v.y; s += (double)v.z * (double)v.z; s += (double)v.w * (double)v.w;
        }
    } else {
        for(unsigned long long i = a0 + threadIdx.x; i < a1; i += 256){ const double g = (double)G[i]; s += g * g; }
    }
    for(unsigned long long i = a1 + threadIdx.x; i < i1; i += 256){ const double g = (double)G[i]; s += g * g; }
    red[threadIdx.x] = s;
    __syncthreads();
    for(int o = 128; o > 0; o >>= 1){
        if((int)threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
        __syncthreads();
    }
    if(threadIdx.x == 0){
        __hip_atomic_store(&g_sq_piece[c * SQ_W + w], red[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned before = __hip_atomic_fetch_add(&g_sq_count[c], 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if(before == SQ_W - 1){
            double t = 0.0;
            for(int k = 0; k < SQ_W; k++) t += __hip_atomic_load(&g_sq_piece[c * SQ_W + k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            part[c] = (float)t;
            __hip_atomic_store(&g_sq_count[c], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

/* k_gnorm (cudalm.cu:2811-2816 = cpu_kern.h:541-546): part = G's 64 partials followed by nside more
 * slices of 64; gs[0] = clip multiplier (exactly 1 when the norm is <= 1), gs[1] = the norm; a
 * non-finite side sum makes the norm NaN. One thread, the reference's order of additions. */
__global__ void k_qlmx_gnorm(const float *part, int nside, int clip_side, float *gs){
    double ss = 0.0, sd = 0.0;
    for(int i = 0; i < 64; i++) ss += (double)part[i];
    for(int i = 64; i < 64 * (1 + nside); i++) sd += (double)part[i];
    float gn = (float)sqrt(clip_side ? ss + sd : ss);
    if(!isfinite(sd)) gn = __builtin_nanf("");
    gs[0] = gn > 1.0f ? 1.0f / gn : 1.0f;
    gs[1] = gn;
}

extern "C" int qlmx_sqsum(const float *G, unsigned long long n, float *part64, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(G && part64, "qlmx_sqsum: NULL buffer");
    hipLaunchKernelGGL(k_qlmx_sqsum, dim3(64 * SQ_W), dim3(256), 0, (hipStream_t)stream, G, n, part64);
    QLMX_LAUNCH_CHECK("qlmx_sqsum launch");
    return QLMX_OK;
}

extern "C" int qlmx_gnorm(const float *part, int nside, int clip_side, float *gs, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(part && gs && nside >= 0, "qlmx_gnorm: bad arguments");
    hipLaunchKernelGGL(k_qlmx_gnorm, dim3(1), dim3(1), 0, (hipStream_t)stream, part, nside, clip_side, gs);
    QLMX_LAUNCH_CHECK("qlmx_gnorm launch");
    return QLMX_OK;
}

/* ---- test hook: the short division form against `/` on pseudo-random operand pairs inside its range ---- */
__global__ void __launch_bounds__(256) k_qlmx_test_div(unsigned long long seed, unsigned long long count, unsigned long long *mismatches){
    unsigned long long bad = 0;
    for(unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < count; i += (unsigned long long)gridDim.x * 256){
        uint64_t r = seed + i * 0x9E3779B97F4A7C15ULL;
        r = (r ^ (r >> 30)) * 0xBF58476D1CE4E5B9ULL; r = (r ^ (r >> 27)) * 0x94D049BB133111EBULL; r ^= r >> 31;
        /* |n| and d with exponents 2^-40 .. 2^40 and random significands, n of either sign */
        const uint32_t en = 87u + (uint32_t)((r >> 23) % 81u), ed = 87u + (uint32_t)((r >> 55) % 81u);
        const float n = __uint_as_float(((uint32_t)r & 0x807FFFFFu) | (en << 23));
        const float d = __uint_as_float(((uint32_t)(r >> 32) & 0x007FFFFFu) | (ed << 23));
        bad += __float_as_uint(qx_div_mid(n, d)) != __float_as_uint(n / d);
        bad += __float_as_uint(qx_div_mid(0.0f, d)) != 0u;
    }
    if(bad) atomicAdd(mismatches, bad);
}
extern "C" int qlmx_test_div_form(unsigned long long seed, unsigned long long count, unsigned long long *mismatches_dev, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(mismatches_dev, "qlmx_test_div_form: NULL counter");
    hipLaunchKernelGGL(k_qlmx_test_div, dim3(4096), dim3(256), 0, (hipStream_t)stream, seed, count, mismatches_dev);
    QLMX_LAUNCH_CHECK("division test launch");
    return QLMX_OK;
}

/* ---- test hook: the short square-root form against sqrtf() over a range of bit patterns ---- */
__global__ void __launch_bounds__(256) k_qlmx_test_sqrt(unsigned first, unsigned long long count, unsigned long long *mismatches){
    unsigned long long bad = 0;
    for(unsigned long long i = (unsigned long long)blockIdx.x * 256 + threadIdx.x; i < count; i += (unsigned long long)gridDim.x * 256){
        const float x = __uint_as_float(first + (unsigned)i);
        const float a = qx_sqrt_above_2m96(x), b = sqrtf(x);
        bad += __float_as_uint(a) != __float_as_uint(b);
    }
    if(bad) atomicAdd(mismatches, bad);
}
extern "C" int qlmx_test_sqrt_form(unsigned first_bits, unsigned long long count, unsigned long long *mismatches_dev, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(mismatches_dev, "qlmx_test_sqrt_form: NULL counter");
    QLMX_REQUIRE(first_bits >= 0x0F800000u && (unsigned long long)first_bits + count <= 0x7F800001ULL,
                 "qlmx_test_sqrt_form: the range must lie inside [2^-96, +infinity]");
    hipLaunchKernelGGL(k_qlmx_test_sqrt, dim3(4096), dim3(256), 0, (hipStream_t)stream, first_bits, count, mismatches_dev);
    QLMX_LAUNCH_CHECK("sqrt test launch");
    return QLMX_OK;
}
