/* qlmx_q4n.hip -- the reference's "q4n" wire format (qtype 3): how a model quantised on the 4-bit
 * grid travels in a checkpoint. Host code only; no device is needed.
 *
 * Writer quantize_params(..., qtype 3, ...) cudalm.cu:638-656, reader dequantize_params
 * cudalm.cu:688-696. Layout per group of `group` values (the last group may be shorter):
 *   fp32 scale, then ceil(g/2) bytes of two's-complement nibbles, even element in the low nibble
 *   (the nibble rule of the packed digits, qlm.cuh:96-101); value = scale * nibble.
 *   A NaN scale marks a group stored as g raw fp32 values instead.
 * The writer accepts a group only if some candidate scale reproduces every value exactly:
 * candidates are amax/k for k = 7..1, each with its two neighbours below and above; the first hit
 * wins. A rendered QLM view (P = s * digit) always passes, possibly with a scale one or two ulps
 * away from s; anything else is kept bit-exact as raw fp32.
 */
#include "qlmx_dev.h"
#include <math.h>
#include <string.h>

extern "C" size_t qlmx_q4n_bound(size_t n, int group){
    if(group <= 0) return 0;
    return 4 * ((n + (size_t)group - 1) / (size_t)group) + 4 * n;
}

extern "C" int qlmx_q4n_quantize(const float *P, size_t n, int group, unsigned char *out, size_t cap,
                                 size_t *out_len, size_t *nraw){
    QLMX_REQUIRE(P && out && out_len, "qlmx_q4n_quantize: NULL buffer");
    QLMX_REQUIRE(group > 0 && group % 2 == 0, "qlmx_q4n_quantize: group %d must be positive and even", group);
    QLMX_REQUIRE(cap >= qlmx_q4n_bound(n, group), "qlmx_q4n_quantize: output buffer smaller than qlmx_q4n_bound()");
    size_t o = 0, raw = 0;
    for(size_t i = 0; i < n; i += (size_t)group){
        const int g = (i + (size_t)group <= n) ? group : (int)(n - i);
        const float *v = P + i;
        float amax = 0.0f, scale = 0.0f;
        for(int j = 0; j < g; j++) amax = fmaxf(amax, fabsf(v[j]));
        bool found = amax == 0.0f;
        for(int k = 7; k >= 1 && !found; k--){
            const float s0 = amax / (float)k;
            const float below = nextafterf(s0, 0.0f), above = nextafterf(s0, INFINITY);
            const float cand[5] = {s0, below, above, nextafterf(below, 0.0f), nextafterf(above, INFINITY)};
            for(int t = 0; t < 5 && !found; t++){
                scale = cand[t];
                found = true;
                for(int j = 0; j < g; j++){
                    const float dgt = rintf(v[j] / scale);
                    if(fabsf(dgt) > 7.0f || dgt * scale != v[j]){ found = false; break; }
                }
            }
        }
        if(!found){
            const float marker = NAN;
            memcpy(out + o, &marker, 4); o += 4;
            memcpy(out + o, v, 4 * (size_t)g); o += 4 * (size_t)g;
            raw++;
            continue;
        }
        memcpy(out + o, &scale, 4); o += 4;
        for(int j = 0; j < g; j += 2){
            const int lo = scale != 0.0f ? (int)rintf(v[j] / scale) : 0;
            const int hi = (j + 1 < g && scale != 0.0f) ? (int)rintf(v[j + 1] / scale) : 0;
            out[o++] = (unsigned char)((lo & 15) | ((hi & 15) << 4));
        }
    }
    *out_len = o;
    if(nraw) *nraw = raw;
    return QLMX_OK;
}

extern "C" int qlmx_q4n_dequantize(const unsigned char *buf, size_t len, float *P, size_t n, int group, size_t *used){
    QLMX_REQUIRE(buf && P, "qlmx_q4n_dequantize: NULL buffer");
    QLMX_REQUIRE(group > 0, "qlmx_q4n_dequantize: group %d", group);
    size_t o = 0;
    for(size_t i = 0; i < n; i += (size_t)group){
        const int g = (i + (size_t)group <= n) ? group : (int)(n - i);
        float scale;
        QLMX_REQUIRE(o + 4 <= len, "qlmx_q4n_dequantize: buffer ends inside group %zu", i / (size_t)group);
        memcpy(&scale, buf + o, 4); o += 4;
        if(scale != scale){
            QLMX_REQUIRE(o + 4 * (size_t)g <= len, "qlmx_q4n_dequantize: buffer ends inside raw group %zu", i / (size_t)group);
            memcpy(P + i, buf + o, 4 * (size_t)g); o += 4 * (size_t)g;
            continue;
        }
        QLMX_REQUIRE(o + (size_t)(g + 1) / 2 <= len, "qlmx_q4n_dequantize: buffer ends inside group %zu", i / (size_t)group);
        for(int j = 0; j < g; j += 2){
            const unsigned char b = buf[o++];
            P[i + j] = (float)((int)((b & 15) ^ 8) - 8) * scale;
            if(j + 1 < g) P[i + j + 1] = (float)((int)((b >> 4) ^ 8) - 8) * scale;
        }
    }
    if(used) *used = o;
    return QLMX_OK;
}
