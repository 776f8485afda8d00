/* qlmx_dev.h -- device-side building blocks shared by the gfx950 kernels. */
#ifndef QLMX_DEV_H
#define QLMX_DEV_H
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/qlmx.h"

#define QLMX_WAVE 64

/* ---- error plumbing (host) ---- */
void qlmx_set_error(const char *fmt, ...);
int qlmx_cu_count(void);
int  qlmx_check_ready(void);
int  qlmx_check_ready_keep(void);        /* the same without issuing what an open pair holds */
int  qlmx_pair_flush(void);              /* issues the launches held back for a pair, if any */
int  qlmx_decode_setup(int device);   /* per-device state of the decode entry points; qlmx_init calls it */
#define QLMX_HIP(call, what)                                                                  \
    do { hipError_t e_ = (call);                                                              \
         if(e_ != hipSuccess){ qlmx_set_error("%s: %s", what, hipGetErrorString(e_));         \
                               return QLMX_E_HIP; } } while(0)
#define QLMX_REQUIRE(cond, ...)                                                               \
    do { if(!(cond)){ qlmx_set_error(__VA_ARGS__); return QLMX_E_ARG; } } while(0)
#define QLMX_LAUNCH_CHECK(what) QLMX_HIP(hipGetLastError(), what)

/* ---- 64-bit hash and stochastic rounding (qlm.cuh:78-87) ----
 * The key of element i at step t is i*KI + t*KT; callers add KI per consecutive element and a
 * per-stream constant instead of multiplying again. */
#define QLMX_KI 0x2545F4914F6CDD1DULL
#define QLMX_KT 0x9E3779B97F4A7C15ULL

__host__ __device__ __forceinline__ uint32_t qx_hash(uint64_t x){
    x += 0x9E3779B97F4A7C15ULL;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
    return (uint32_t)(x ^ (x >> 31));
}
/* floor(v) + [u < frac(v)] with u = top 24 hash bits * 2^-24; `key` is the finished hash key */
__host__ __device__ __forceinline__ int qx_sround(float v, uint64_t key){
    float fl = floorf(v);
    uint32_t h = qx_hash(key);
    float u = (float)(h >> 8) * (1.0f / 16777216.0f);
    return (int)fl + (u < (v - fl) ? 1 : 0);
}
__host__ __device__ __forceinline__ int qx_clamp(int v, int lo, int hi){ return v < lo ? lo : (v > hi ? hi : v); }

/* signed 4-bit field k (0..7) of a 32-bit word holding 8 consecutive digits (qlm.cuh:96-101) */
__device__ __forceinline__ int qx_nib(uint32_t w, int k){ return ((int)(w << (28 - 4*k))) >> 28; }
/* digit k of a packed word as digit / 16 in fp32 (exact): one shift and v_cvt_off_f32_i4, against two
 * shifts and a convert for the integer route. Whoever uses it carries the factor 16 in a scale. */
__device__ __forceinline__ float qx_nib16(uint32_t w, int k){ return __builtin_amdgcn_cvt_off_f32_i4((int)(w >> (4 * k))); }
/* The same for all eight digits of a word at nine instructions: the convert takes its operand from a byte
 * of a register (an operand modifier, no shift), so the even digits come from the bytes of w and the odd ones
 * from the bytes of w >> 4. The empty asm keeps the shifted word a value of its own; seen through, the
 * compiler turns "byte of w >> 4" back into a bit-field extract per digit. */
struct QxNibs { uint32_t w, h; };
__device__ __forceinline__ QxNibs qx_nibs(uint32_t w){ QxNibs n; n.w = w; n.h = w >> 4; asm("" : "+v"(n.h)); return n; }
__device__ __forceinline__ float qx_nib16(const QxNibs &n, int k){
    const uint32_t src = (k & 1) ? n.h : n.w;
    return __builtin_amdgcn_cvt_off_f32_i4((int)((src >> (8 * (k >> 1))) & 0xFFu));
}

/* ---- span lookup: the owner of group gi. The table is ascending in gi0, so a binary search
 * returns what the reference's first-match linear scan returns (qlm.cuh:114-117). ---- */
__device__ __forceinline__ int qx_span_of(const qlmx_span *sp, int nspan, int gi){
    int lo = 0, hi = nspan - 1;
    while(lo < hi){
        int mid = (lo + hi + 1) >> 1;
        if(sp[mid].gi0 <= gi) lo = mid; else hi = mid - 1;
    }
    return lo;
}

/* ---- DPP reductions over a row of 16 lanes ----
 * quad_perm [1,0,3,2] = 0xB1, [2,3,0,1] = 0x4E, row_half_mirror = 0x141, row_mirror = 0x140.
 * After the four steps every lane of the row holds the row's maximum. */
template<int CTRL> __device__ __forceinline__ float qx_dpp(float v){
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}
template<int CTRL> __device__ __forceinline__ int qx_dpp_i(int v){
    return __builtin_amdgcn_mov_dpp(v, CTRL, 0xF, 0xF, true);
}
__device__ __forceinline__ float qx_row16_max(float v){
    v = fmaxf(v, qx_dpp<0xB1>(v));
    v = fmaxf(v, qx_dpp<0x4E>(v));
    v = fmaxf(v, qx_dpp<0x141>(v));
    v = fmaxf(v, qx_dpp<0x140>(v));
    return v;
}
__device__ __forceinline__ int qx_row16_maxi(int v){
    v = max(v, qx_dpp_i<0xB1>(v));
    v = max(v, qx_dpp_i<0x4E>(v));
    v = max(v, qx_dpp_i<0x141>(v));
    v = max(v, qx_dpp_i<0x140>(v));
    return v;
}
__device__ __forceinline__ int qx_row16_sum(int v){
    v += qx_dpp_i<0xB1>(v);
    v += qx_dpp_i<0x4E>(v);
    v += qx_dpp_i<0x141>(v);
    v += qx_dpp_i<0x140>(v);
    return v;
}
/* full 64-lane sum / max built from the row step plus two cross-row exchanges */
__device__ __forceinline__ float qx_wave_sum(float v){
    for(int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float qx_wave_max(float v){
    for(int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

/* cpu_kern.h:29-34: clamp, Cody-Waite split of ln 2, degree-6 Horner polynomial, exponent built
 * with integer bit arithmetic */
__device__ __forceinline__ float qx_fexp(float x){
    x = x < -87.0f ? -87.0f : (x > 88.0f ? 88.0f : x);
    const float fi = rintf(x * 1.44269504089f);
    float r = x - fi * 0.693145751953125f;
    r -= fi * 1.428606765330187e-06f;
    const float p = 1.0f + r * (1.0f + r * (0.5f + r * (1.0f / 6 + r * (1.0f / 24 + r * (1.0f / 120 + r * (1.0f / 720))))));
    const float scale = __uint_as_float((uint32_t)((int)fi + 127) << 23);
    return p * scale;
}
__device__ __forceinline__ float qx_fsig(float x){ return 1.0f / (1.0f + qx_fexp(-x)); }
/* The sigmoid on the transcendental unit (v_exp_f32, v_rcp_f32: one unit in the last place each) for the GEMM
 * epilogues, where the polynomial and the IEEE division above, some forty instructions, would cost as much as the
 * tile's matrix products: within 3e-7 of qx_fsig relative to the result for |x| < 10, 0 and 1 at the far ends. */
__device__ __forceinline__ float qx_fsig_hw(float x){ return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * -1.44269504089f)); }


#endif
