/* qlmx_codec.hip -- encode, render and scale servo of the nibble-packed 4-bit weight format.
 *
 * Replaces k_qlm_encode (qlm.cuh:136-167), k_qlm_render (qlm.cuh:170-178) and k_qlm_servo
 * (qlm.cuh:404-441); CPU twins cpu_kern.h:777-796, 857-873. Format: element i of d/r lives at
 * qi0+i; packed digits sit two per byte, even element in the low nibble, two's complement; one
 * fp32 scale per group of `group` consecutive elements of a span, the last group may be short.
 *
 * As in the optimizer kernel a group belongs to one DPP row of 16 lanes. With group 128, full and
 * 8-element aligned, each lane handles 8 consecutive elements through 128/64/32-bit accesses;
 * everything else goes pair-per-lane so that a lane always owns whole bytes of packed digits.
 * All three are streaming kernels bound by HBM (encode: read 4 B, write 1.5 B per weight; render:
 * read 0.5 B, write 4 B; servo: read 1.5 B, write at most 1.5 B).
 */
#include "qlmx_dev.h"

struct GroupLoc { int n; uint64_t pof, qi0; };
__device__ __forceinline__ GroupLoc group_loc(const qlmx_span *sp, int nspan, int gi, int group){
    const int si = qx_span_of(sp, nspan, gi);
    const qlmx_span S = sp[si];
    const uint64_t j0 = (uint64_t)(gi - S.gi0) * (uint64_t)group;
    const uint64_t left = S.n - j0;
    GroupLoc L;
    L.n = (int)((uint64_t)group < left ? (uint64_t)group : left);
    L.pof = S.pof + j0; L.qi0 = S.qi0 + j0;
    return L;
}
__device__ __forceinline__ int load_digit(const signed char *d, uint64_t qi, int packed){
    if(!packed) return (int)d[qi];
    const unsigned b = (unsigned char)d[qi >> 1];
    const int v = (qi & 1ULL) ? (int)(b >> 4) : (int)(b & 15u);
    return v >= 8 ? v - 16 : v;
}
/* digit and residual of t = value/scale (qlm.cuh:160-162, 434-436) */
__device__ __forceinline__ void quantize(float t, int dmax, int &dd, int &rr){
    dd = qx_clamp((int)rintf(t), -dmax, dmax);
    rr = qx_clamp((int)rintf((t - (float)dd) * 128.0f), -64, 64);
}

__global__ void __launch_bounds__(256) k_qlmx_encode(const float *P, signed char *d, signed char *r, float *s,
                                                     const qlmx_span *sp, int nspan, int group, int dmax,
                                                     int packed, int ngrp, int vec_ok){
    const int lane16 = threadIdx.x & 15;
    const int gi = (int)((blockIdx.x * (unsigned)blockDim.x + threadIdx.x) >> 4);
    if(gi >= ngrp) return;
    const GroupLoc L = group_loc(sp, nspan, gi, group);
    const bool fast = vec_ok && group == 128 && packed && L.n == 128 && ((L.pof | L.qi0) & 7ULL) == 0;
    if(fast){
        const uint64_t e0 = (uint64_t)lane16 * 8;
        const float4 p0 = *(const float4 *)(P + L.pof + e0), p1 = *(const float4 *)(P + L.pof + e0 + 4);
        const float pv[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
        float amax = 0.0f;
#pragma unroll
        for(int k = 0; k < 8; k++) amax = fmaxf(amax, fabsf(pv[k]));
        amax = qx_row16_max(amax);
        float sg = amax / (float)dmax; if(!(sg > 0.0f)) sg = 1e-8f;
        if(lane16 == 0) s[gi] = sg;
        uint32_t dw = 0, r0 = 0, r1 = 0;
#pragma unroll
        for(int k = 0; k < 8; k++){
            int dd, rr; quantize(pv[k] / sg, dmax, dd, rr);
            dw |= ((uint32_t)dd & 15u) << (4 * k);
            if(k < 4) r0 |= ((uint32_t)rr & 0xFFu) << (8 * k); else r1 |= ((uint32_t)rr & 0xFFu) << (8 * (k - 4));
        }
        *(uint32_t *)(d + ((L.qi0 + e0) >> 1)) = dw;
        *(uint2 *)(r + L.qi0 + e0) = make_uint2(r0, r1);
    } else {
        float amax = 0.0f;
        for(int j = lane16; j < L.n; j += 16) amax = fmaxf(amax, fabsf(P[L.pof + j]));
        amax = qx_row16_max(amax);
        float sg = amax / (float)dmax; if(!(sg > 0.0f)) sg = 1e-8f;
        if(lane16 == 0) s[gi] = sg;
        for(int jb = 2 * lane16; jb < L.n; jb += 32){
            int dn[2] = {0, 0};
#pragma unroll
            for(int h = 0; h < 2; h++){
                const int j = jb + h;
                if(j < L.n){
                    int dd, rr; quantize(P[L.pof + j] / sg, dmax, dd, rr);
                    dn[h] = dd; r[L.qi0 + j] = (signed char)rr;
                    if(!packed) d[L.qi0 + j] = (signed char)dd;
                }
            }
            if(packed) d[(L.qi0 + jb) >> 1] = (signed char)(((dn[1] & 15) << 4) | (dn[0] & 15));
        }
    }
}

__global__ void __launch_bounds__(256) k_qlmx_render(float *P, const signed char *d, const float *s,
                                                     const qlmx_span *sp, int nspan, int group, int packed,
                                                     int gi_base, int ng, int vec_ok){
    const int lane16 = threadIdx.x & 15;
    const int w = (int)((blockIdx.x * (unsigned)blockDim.x + threadIdx.x) >> 4);
    if(w >= ng) return;
    const int gi = gi_base + w;
    const GroupLoc L = group_loc(sp, nspan, gi, group);
    const float sg = s[gi];
    const bool fast = vec_ok && group == 128 && packed && L.n == 128 && ((L.pof | L.qi0) & 7ULL) == 0;
    if(fast){
        /* a lane renders elements 4*lane16 .. +3 and the same 64 further on: each of the two stores of
         * a 16-lane row covers 256 contiguous bytes of P, written past the caches */
        typedef float f4 __attribute__((ext_vector_type(4)));
        const uint64_t e0 = (uint64_t)lane16 * 4;
        const unsigned short *dh = (const unsigned short *)(d + (L.qi0 >> 1));
        const uint32_t w0 = dh[lane16], w1 = dh[16 + lane16];
        f4 o0, o1;
        o0.x = sg * (float)qx_nib(w0, 0); o0.y = sg * (float)qx_nib(w0, 1);
        o0.z = sg * (float)qx_nib(w0, 2); o0.w = sg * (float)qx_nib(w0, 3);
        o1.x = sg * (float)qx_nib(w1, 0); o1.y = sg * (float)qx_nib(w1, 1);
        o1.z = sg * (float)qx_nib(w1, 2); o1.w = sg * (float)qx_nib(w1, 3);
        __builtin_nontemporal_store(o0, (f4 *)(P + L.pof + e0));
        __builtin_nontemporal_store(o1, (f4 *)(P + L.pof + e0 + 64));
    } else {
        for(int j = lane16; j < L.n; j += 16) P[L.pof + j] = sg * (float)load_digit(d, L.qi0 + j, packed);
    }
}

__global__ void __launch_bounds__(256) k_qlmx_servo(signed char *d, signed char *r, float *s,
                                                    const qlmx_span *sp, int nspan, int group, int dmax,
                                                    float f_hi, float f_lo, int packed, int ngrp, int vec_ok){
    const int lane16 = threadIdx.x & 15;
    const int gi = (int)((blockIdx.x * (unsigned)blockDim.x + threadIdx.x) >> 4);
    if(gi >= ngrp) return;
    const GroupLoc L = group_loc(sp, nspan, gi, group);
    if(vec_ok && group == 128 && packed && L.n == 128 && (L.qi0 & 7ULL) == 0){
        /* 8 consecutive elements per lane: one 32-bit word of digits, and 8 residual bytes only where the
         * group is rescaled */
        const uint64_t e0 = L.qi0 + (uint64_t)lane16 * 8;
        const uint32_t dw = *(const uint32_t *)(d + (e0 >> 1));
        int dv[8], railed = 0;
#pragma unroll
        for(int k = 0; k < 8; k++){ dv[k] = qx_nib(dw, k); railed += (dv[k] == dmax) | (dv[k] == -dmax); }
        railed = qx_row16_sum(railed);
        const float f = (float)railed / 128.0f, sg = s[gi];
        float sn;
        if(f > f_hi)      sn = sg * 1.09051f;
        else if(f < f_lo) sn = sg / 1.09051f;
        else return;
        const float conv = sg / sn;
        if(lane16 == 0) s[gi] = sn;
        const uint2 rw = *(const uint2 *)(r + e0);
        uint32_t dn = 0, r0 = 0, r1 = 0;
#pragma unroll
        for(int k = 0; k < 8; k++){
            const int rb = (int)(signed char)(((k < 4 ? rw.x : rw.y) >> (8 * (k & 3))) & 0xFFu);
            const float t = ((float)dv[k] + (float)rb * (1.0f / 128.0f)) * conv;
            int dd, rr; quantize(t, dmax, dd, rr);
            dn |= ((uint32_t)dd & 15u) << (4 * k);
            if(k < 4) r0 |= ((uint32_t)rr & 0xFFu) << (8 * k); else r1 |= ((uint32_t)rr & 0xFFu) << (8 * (k - 4));
        }
        *(uint32_t *)(d + (e0 >> 1)) = dn;
        *(uint2 *)(r + e0) = make_uint2(r0, r1);
        return;
    }
    int railed = 0;
    for(int jb = 2 * lane16; jb < L.n; jb += 32)
        for(int h = 0; h < 2; h++){
            const int j = jb + h;
            if(j < L.n){ const int dd = load_digit(d, L.qi0 + j, packed); railed += (dd == dmax) | (dd == -dmax); }
        }
    railed = qx_row16_sum(railed);
    const float f = (float)railed / (float)L.n, sg = s[gi];
    float sn;
    if(f > f_hi)      sn = sg * 1.09051f;          /* 2^(1/8) */
    else if(f < f_lo) sn = sg / 1.09051f;
    else return;                                   /* uniform over the row */
    const float conv = sg / sn;
    if(lane16 == 0) s[gi] = sn;
    for(int jb = 2 * lane16; jb < L.n; jb += 32){
        int dn[2] = {0, 0};
#pragma unroll
        for(int h = 0; h < 2; h++){
            const int j = jb + h;
            if(j < L.n){
                const uint64_t qi = L.qi0 + j;
                const float t = ((float)load_digit(d, qi, packed) + (float)r[qi] * (1.0f / 128.0f)) * conv;
                int dd, rr; quantize(t, dmax, dd, rr);
                dn[h] = dd; r[qi] = (signed char)rr;
                if(!packed) d[qi] = (signed char)dd;
            }
        }
        if(packed) d[(L.qi0 + jb) >> 1] = (signed char)(((dn[1] & 15) << 4) | (dn[0] & 15));
    }
}

static int codec_args_ok(const char *who, int nspan, int group, int dmax, int packed){
    QLMX_REQUIRE(nspan > 0, "%s: nspan %d", who, nspan);
    QLMX_REQUIRE(group >= 2 && group <= 256, "%s: group %d outside [2,256]", who, group);
    QLMX_REQUIRE(dmax >= 1 && dmax <= 127, "%s: dmax %d", who, dmax);
    QLMX_REQUIRE(!packed || (dmax <= 7 && (group & 1) == 0), "%s: packed digits need dmax<=7 and an even group", who);
    return QLMX_OK;
}

extern "C" int qlmx_encode(const float *P, signed char *d, signed char *r, float *s,
                           const qlmx_span *sp, int nspan, int group, int dmax, int packed, int ngrp,
                           void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(P && d && r && s && sp, "qlmx_encode: NULL buffer");
    rc = codec_args_ok("qlmx_encode", nspan, group, dmax, packed); if(rc) return rc;
    if(ngrp <= 0) return QLMX_OK;
    const int vec_ok = ((uintptr_t)P & 15) == 0 && ((uintptr_t)r & 7) == 0 && ((uintptr_t)d & 3) == 0;
    hipLaunchKernelGGL(k_qlmx_encode, dim3((unsigned)((ngrp + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                       P, d, r, s, sp, nspan, group, dmax, packed, ngrp, vec_ok);
    QLMX_LAUNCH_CHECK("qlmx_encode launch");
    return QLMX_OK;
}

extern "C" int qlmx_render(float *P, const signed char *d, const float *s,
                           const qlmx_span *sp, int nspan, int group, int packed, int gi_base, int ng,
                           void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(P && d && s && sp, "qlmx_render: NULL buffer");
    rc = codec_args_ok("qlmx_render", nspan, group, packed ? 7 : 127, packed); if(rc) return rc;
    QLMX_REQUIRE(gi_base >= 0, "qlmx_render: gi_base %d", gi_base);
    if(ng <= 0) return QLMX_OK;
    const int vec_ok = ((uintptr_t)P & 15) == 0 && ((uintptr_t)d & 3) == 0;
    hipLaunchKernelGGL(k_qlmx_render, dim3((unsigned)((ng + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                       P, d, s, sp, nspan, group, packed, gi_base, ng, vec_ok);
    QLMX_LAUNCH_CHECK("qlmx_render launch");
    return QLMX_OK;
}

extern "C" int qlmx_servo(signed char *d, signed char *r, float *s,
                          const qlmx_span *sp, int nspan, int group, int dmax,
                          float f_hi, float f_lo, int packed, int ngrp, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(d && r && s && sp, "qlmx_servo: NULL buffer");
    rc = codec_args_ok("qlmx_servo", nspan, group, dmax, packed); if(rc) return rc;
    if(ngrp <= 0) return QLMX_OK;
    const int vec_ok = ((uintptr_t)r & 7) == 0 && ((uintptr_t)d & 3) == 0;
    hipLaunchKernelGGL(k_qlmx_servo, dim3((unsigned)((ngrp + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                       d, r, s, sp, nspan, group, dmax, f_hi, f_lo, packed, ngrp, vec_ok);
    QLMX_LAUNCH_CHECK("qlmx_servo launch");
    return QLMX_OK;
}
