/* selftest.cpp -- the QLM section of the reference's in-binary selftest (cudalm.cu:10477-10649)
 * rewritten against the host mirror: encode+render within half a quantisation step and at most
 * 2*dmax+1 levels per group; one Integer AdamW step against a scalar host restatement that reuses
 * the host helpers (digits/residuals must agree bit for bit here because both sides are compiled
 * without FMA contraction); a save/load round trip; an expert FFN forward through the grouped GEMM
 * queue against a host triple loop, the paired input-gradient GEMMs of w1 and w3, and the gate|up GEMMs with the SwiGLU behind them. Prints one line per check and exits 0 only if all pass. */
#include "qlm_host.h"
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <vector>

static uint64_t rng = 0x9E3779B97F4A7C15ULL;
static float urand(){ rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return (float)((rng >> 40) * (1.0 / 16777216.0)); }
static float nrand(){ float u1 = urand(); if(u1 < 1e-9f) u1 = 1e-9f; float u2 = urand(); return sqrtf(-2.0f * logf(u1)) * cosf(6.28318530718f * u2); }
static int ok_all = 1;
static void check(const char *name, double v, double tol){ printf("  %-34s %.3e  %s\n", name, v, v <= tol ? "OK" : "FAIL"); if(!(v <= tol)) ok_all = 0; }

/* Spans of the given sizes laid out behind `prefix` float parameters with `gap` more between them. */
static std::vector<QlmSpanDesc> layout(int prefix, int gap, int nsizes, char **sizes, size_t *np){
    std::vector<QlmSpanDesc> sp; size_t at = (size_t)prefix;
    for(int i = 0; i < nsizes; i++){ const size_t n = strtoull(sizes[i], NULL, 10); sp.push_back({at, n}); at += n + (size_t)gap; }
    *np = at - (size_t)gap + 2;
    return sp;
}
static std::vector<unsigned char> slurp(const char *path){
    std::vector<unsigned char> b; FILE *f = fopen(path, "rb"); if(!f) return b;
    fseek(f, 0, SEEK_END); b.resize((size_t)ftell(f)); fseek(f, 0, SEEK_SET);
    if(fread(b.data(), 1, b.size(), f) != b.size()) b.clear();
    fclose(f); return b;
}

/* qlm_selftest optq IN OUT PREFIX GAP N0 [N1 ...]: a Qlm of that layout without weights, qlm_load(IN) into its
 * device state, qlm_save(OUT) from it. The caller compares the two files.
 * qlm_selftest sref PFILE OUT PREFIX GAP N0 [N1 ...]: qlm_gpu_init from the fp32 parameters in PFILE; OUT gets
 * the frozen reference scale of every span followed by all group scales (raw fp32).
 * qlm_selftest update PFILE OUT PREFIX GAP N0 [N1 ...]: qlm_gpu_init from PFILE, then QLM_TEST_STEPS calls of
 * qlm_gpu_update (t = 1, 2, ...; lr 3e-4, betas 0.9 / 0.95, weight decay 0.1, bias corrections 1 - beta^t as
 * cudalm.cu:6454 forms them; the gradient of step t is the t-th block of np floats in QLM_TEST_GRADS; when
 * QLM_TEST_CLIP is set the step takes its clip multiplier from a device scalar holding that value). The servo
 * period, the optimizer and the LR mode come from the environment as in the reference. OUT gets, raw and in this
 * order: d, r, m8, v8 (Adam only), s, m8s, v8s (Adam only), sref per span, the fp32 view P. With CUDALM_PROF or
 * CUDALM_DEBUG set the driver's check points (kchk) time its labels and the table is printed at the end. */
static int tool(int argc, char **argv){
    if(argc < 7){ fprintf(stderr, "usage: %s optq|sref|update IN OUT PREFIX GAP N0 [N1 ...]\n", argv[0]); return 2; }
    size_t np = 0;
    std::vector<QlmSpanDesc> sp = layout(atoi(argv[4]), atoi(argv[5]), argc - 6, argv + 6, &np);
    Qlm q;
    if(!strcmp(argv[1], "optq")){
        qlm_gpu_init(&q, sp.data(), (int)sp.size(), NULL, np);
        if(q.nfloat){
            q.Mc = (bf16 *)dmalloc(q.nfloat * 2); q.Vc = (bf16 *)dmalloc(q.nfloat * 2);
            qlmx_memset(q.Mc, 0, q.nfloat * 2, NULL); qlmx_memset(q.Vc, 0, q.nfloat * 2, NULL);
        }
        int iter = -1; float pg = 1.0f;
        if(!qlm_load(&q, argv[2], &iter, &pg)){ fprintf(stderr, "qlm_load failed\n"); return 1; }
        if(!qlm_save(&q, argv[3], iter, pg)){ fprintf(stderr, "qlm_save failed\n"); return 1; }
        printf("optq: iter %d prev_gn %g nq %llu ngrp %llu nfloat %llu\n", iter, pg, q.nq, q.ngrp, q.nfloat);
        return 0;
    }
    if(!strcmp(argv[1], "sref")){
        std::vector<unsigned char> raw = slurp(argv[2]);
        if(raw.size() != np * 4){ fprintf(stderr, "sref: %s holds %zu bytes, the layout needs %zu\n", argv[2], raw.size(), np * 4); return 1; }
        float *Pd = (float *)dmalloc(np * 4);
        qlmx_memcpy_h2d(Pd, raw.data(), np * 4);
        qlm_gpu_init(&q, sp.data(), (int)sp.size(), Pd, np);
        std::vector<float> out(q.nspan + q.ngrp);
        for(int i = 0; i < q.nspan; i++) out[i] = q.spanH[i].sref;
        qlmx_memcpy_d2h(out.data() + q.nspan, q.s, q.ngrp * 4);
        FILE *f = fopen(argv[3], "wb");
        if(!f || fwrite(out.data(), 4, out.size(), f) != out.size()){ fprintf(stderr, "sref: cannot write %s\n", argv[3]); return 1; }
        fclose(f);
        printf("sref: %d spans %llu groups, %d float gaps holding %llu parameters\n", q.nspan, q.ngrp, q.nfs, q.nfloat);
        return 0;
    }
    if(!strcmp(argv[1], "update")){
        std::vector<unsigned char> raw = slurp(argv[2]);
        if(raw.size() != np * 4){ fprintf(stderr, "update: %s holds %zu bytes, the layout needs %zu\n", argv[2], raw.size(), np * 4); return 1; }
        const int steps = atoi(getenv("QLM_TEST_STEPS") ? getenv("QLM_TEST_STEPS") : "4");
        std::vector<unsigned char> graw = slurp(getenv("QLM_TEST_GRADS") ? getenv("QLM_TEST_GRADS") : "");
        if(graw.size() != np * 4 * (size_t)steps){ fprintf(stderr, "update: QLM_TEST_GRADS must hold %d x %zu floats\n", steps, np); return 1; }
        float *Pd = (float *)dmalloc(np * 4), *Gd = (float *)dmalloc(np * 4), *gsd = NULL;
        qlmx_memcpy_h2d(Pd, raw.data(), np * 4);
        if(getenv("QLM_TEST_CLIP")){
            const float clip = (float)atof(getenv("QLM_TEST_CLIP"));
            gsd = (float *)dmalloc(8); qlmx_memcpy_h2d(gsd, &clip, 4);
        }
        qlm_gpu_init(&q, sp.data(), (int)sp.size(), Pd, np);
        const float lr = 3e-4f, b1 = 0.9f, b2 = 0.95f, wd = 0.1f;
        int servo_passes = 0;
        for(int t = 1; t <= steps; t++){
            qlmx_memcpy_h2d(Gd, graw.data() + (size_t)(t - 1) * np * 4, np * 4);
            qlm_gpu_update(&q, Pd, Gd, lr, b1, b2, wd, 1.0f - powf(b1, (float)t), 1.0f - powf(b2, (float)t), t, gsd);
            servo_passes += q.servo_every > 0 && t % q.servo_every == 0;
        }
        /* the reference renders P after a servo pass only through the next step; the last step's P is what it left */
        qlmx_sync(NULL);
        FILE *f = fopen(argv[3], "wb");
        if(!f){ fprintf(stderr, "update: cannot write %s\n", argv[3]); return 1; }
        auto dump = [&](const void *dev, size_t bytes){
            std::vector<unsigned char> h(bytes);
            qlmx_memcpy_d2h(h.data(), dev, bytes);
            return fwrite(h.data(), 1, bytes, f) == bytes;
        };
        bool okw = dump(q.d, (size_t)qlmx_qd_bytes(q.nq, q.packed)) && dump(q.r, q.nq) && dump(q.m8, q.nq);
        if(q.adam) okw = okw && dump(q.v8, q.nq);
        okw = okw && dump(q.s, q.ngrp * 4) && dump(q.m8s, q.ngrp * 4);
        if(q.adam) okw = okw && dump(q.v8s, q.ngrp * 4);
        for(int i = 0; i < q.nspan; i++) okw = okw && fwrite(&q.spanH[i].sref, 4, 1, f) == 1;
        okw = okw && dump(Pd, np * 4);
        fclose(f);
        if(!okw){ fprintf(stderr, "update: short write to %s\n", argv[3]); return 1; }
        printf("update: %d steps, %d servo passes, adam %d lrmode %d group %d dmax %d, %llu weights %llu groups\n",
               steps, servo_passes, q.adam, q.lrmode, q.group, q.dmax, q.nq, q.ngrp);
        prof_report();                                     /* the table of the driver's kchk labels when CUDALM_PROF is set */
        double slow_ms = 0.0; const char *slow = kchk_slowest(&slow_ms);
        if(getenv("CUDALM_DEBUG") && atoi(getenv("CUDALM_DEBUG"))) printf("slowest label: %s, %.3f ms\n", slow, slow_ms);
        return 0;
    }
    fprintf(stderr, "unknown mode %s\n", argv[1]); return 2;
}

int main(int argc, char **argv){
    if(qlmx_init(0) != QLMX_OK){ fprintf(stderr, "%s\n", qlmx_last_error()); return 2; }
    if(argc > 1) return tool(argc, argv);
    printf("[selftest] %s\n", qlmx_device_name());
    /* a toy layer: 16 floats of "norm", then w1, w3 [D,F] x E and w2 [F,D] x E */
    const int E = 3, D = 128, F = 256, N = 40;
    const size_t nw = (size_t)E * D * F, np = 16 + 3 * nw + 8;
    QlmSpanDesc spans[3] = {{16, nw}, {16 + nw, nw}, {16 + 2 * nw, nw}};
    std::vector<float> Ph(np), Gh(np);
    for(size_t i = 0; i < np; i++){ Ph[i] = 0.02f * nrand(); Gh[i] = 0.01f * nrand(); }
    float *Pd = (float *)dmalloc(np * 4), *Gd = (float *)dmalloc(np * 4);
    qlmx_memcpy_h2d(Pd, Ph.data(), np * 4); qlmx_memcpy_h2d(Gd, Gh.data(), np * 4);
    Qlm q; qlm_gpu_init(&q, spans, 3, Pd, np);
    printf("[selftest] %d spans, %llu weights, %llu groups, %.2f B/param persistent\n", q.nspan, q.nq, q.ngrp, qlm_persist_bytes(&q) / (double)q.nq);

    /* (a) encode + render */
    std::vector<float> Pr(np), sh(q.ngrp);
    qlmx_memcpy_d2h(Pr.data(), Pd, np * 4); qlmx_memcpy_d2h(sh.data(), q.s, q.ngrp * 4);
    double worst = 0; int lvlmax = 0;
    for(int si = 0; si < q.nspan; si++) for(int g = 0; g < q.spanH[si].ngrp; g++){
        int gi = q.spanH[si].gi0 + g; std::vector<float> lv;
        for(int j = 0; j < q.group; j++){
            size_t k = q.spanH[si].pof + (size_t)g * q.group + j;
            double e = fabs((double)Pr[k] - Ph[k]) / sh[gi]; if(e > worst) worst = e;
            bool seen = false; for(float v : lv) if(v == Pr[k]) seen = true;
            if(!seen) lv.push_back(Pr[k]);
        }
        if((int)lv.size() > lvlmax) lvlmax = (int)lv.size();
    }
    check("qlm encode err/step", worst, 0.51);
    check("qlm distinct levels per group", lvlmax, 2 * q.dmax + 1);
    for(size_t i = 0; i < 16; i++) if(Pr[i] != Ph[i]) ok_all = 0;        /* float span untouched */

    /* (b) one step vs a scalar host restatement on the pre-step state */
    const int T = 3; const float lr = 3e-4f, b1 = 0.9f, b2 = 0.95f, wd = 0.1f;
    const float bc1 = 1.0f - powf(b1, (float)T), bc2 = 1.0f - powf(b2, (float)T);
    unsigned long long nq = q.nq, ng = q.ngrp, nd = qlmx_qd_bytes(nq, q.packed);
    std::vector<signed char> hd(nd), hr(nq), hm(nq), rd(nd), rr_(nq); std::vector<unsigned char> hv(nq);
    std::vector<float> hs(ng), hms(ng), hvs(ng);
    qlmx_memcpy_d2h(hd.data(), q.d, nd); qlmx_memcpy_d2h(hr.data(), q.r, nq); qlmx_memcpy_d2h(hm.data(), q.m8, nq);
    qlmx_memcpy_d2h(hv.data(), q.v8, nq); qlmx_memcpy_d2h(hs.data(), q.s, ng * 4);
    qlmx_memcpy_d2h(hms.data(), q.m8s, ng * 4); qlmx_memcpy_d2h(hvs.data(), q.v8s, ng * 4);
    const float inv_bc1 = 1.0f / bc1, inv_sqrt_bc2 = 1.0f / sqrtf(bc2);
    for(int si = 0; si < q.nspan; si++) for(int g = 0; g < q.spanH[si].ngrp; g++){
        int gi = q.spanH[si].gi0 + g; unsigned long long j0 = (unsigned long long)g * q.group;
        unsigned long long pof = q.spanH[si].pof + j0, qi0 = q.spanH[si].qi0 + j0;
        float sg = hs[gi], L = lr * 128.0f / (q.lrmode ? sg : q.spanH[si].sref), dec = lr * wd * 128.0f;
        float ms_old = hms[gi], vs_old = hvs[gi];
        for(int j = 0; j < q.group; j++){
            unsigned long long qi = qi0 + j; float gr = Gh[pof + j], mv = (float)hm[qi] * ms_old;
            float sv = (float)hv[qi] * vs_old, vv = sv * sv, mn = b1 * mv + (1.0f - b1) * gr;
            vv = b2 * vv + (1.0f - b2) * gr * gr; float rv = sqrtf(vv), veps = fmaxf(vs_old, 1e-8f);
            float u = (mn * inv_bc1) / (rv * inv_sqrt_bc2 + veps); u = fmaxf(-8.0f, fminf(8.0f, u));
            int dd = qlmx_qd_get(hd.data(), qi, q.packed), idl = qlmx_qsri(-(L * u + dec * (float)dd), qi, (unsigned long long)T);
            int r2 = (int)hr[qi] + idl, c = (r2 > 64) ? (((r2 - 65) >> 7) + 1) : ((r2 < -64) ? -((((-r2) - 65) >> 7) + 1) : 0);
            r2 -= c * 128; dd = qlmx_qclmp(dd + c, -q.dmax, q.dmax);
            qlmx_qd_set_host(rd.data(), qi, dd, q.packed); rr_[qi] = (signed char)r2;
        }
    }
    qlm_gpu_update(&q, Pd, Gd, lr, b1, b2, wd, bc1, bc2, T, NULL);
    qlmx_sync(NULL);
    std::vector<signed char> gd(nd), gr2(nq);
    qlmx_memcpy_d2h(gd.data(), q.d, nd); qlmx_memcpy_d2h(gr2.data(), q.r, nq);
    unsigned long long dmiss = 0, rmiss = 0;
    for(unsigned long long i = 0; i < nq; i++){ if(qlmx_qd_get(gd.data(), i, q.packed) != qlmx_qd_get(rd.data(), i, q.packed)) dmiss++; if(gr2[i] != rr_[i]) rmiss++; }
    check("qlm step digits differing", (double)dmiss, 0);
    check("qlm step residuals differing", (double)rmiss, 0);

    /* (c) checkpoint round trip */
    const char *path = "/tmp/qlmx_selftest.opt.q";
    int okio = qlm_save(&q, path, 77, 1.25f);
    qlmx_memset(q.d, 0, nd, NULL); qlmx_memset(q.m8, 0, nq, NULL);
    int iter = 0; float pg = 0; okio = okio && qlm_load(&q, path, &iter, &pg);
    std::vector<signed char> gd2(nd); qlmx_memcpy_d2h(gd2.data(), q.d, nd);
    check("qlm save/load round trip", (okio && iter == 77 && pg == 1.25f && !memcmp(gd.data(), gd2.data(), nd)) ? 0 : 1, 0);

    /* (c2) fused per-layer update: stepping span by span while "its gradients are live", clipped by the
     * previous step's norm, must leave the same state as one step over all groups with that multiplier;
     * the partial sums collected on the way give this step's norm */
    {
        const int T2 = 4; const float prev_gn = 2.5f;
        const float c1 = 1.0f - powf(b1, (float)T2), c2 = 1.0f - powf(b2, (float)T2);
        int okf = qlm_save(&q, path, 78, prev_gn);
        qlm_step_launch(Pd, Gd, q.d, q.r, q.s, q.m8, q.m8s, q.v8, q.v8s, q.spanD, q.nspan, q.group, q.dmax, lr, b1, b2, wd,
                        1.0f / prev_gn, NULL, 1.0f / c1, 1.0f / sqrtf(c2), q.lrmode, (unsigned long long)T2, q.adam, NULL, q.packed, 0, (int)q.ngrp);
        qlmx_sync(NULL);
        std::vector<signed char> wd_(nd), wr(nq), wm(nq), fd(nd), fr(nq), fm(nq);
        qlmx_memcpy_d2h(wd_.data(), q.d, nd); qlmx_memcpy_d2h(wr.data(), q.r, nq); qlmx_memcpy_d2h(wm.data(), q.m8, nq);
        int it2 = 0; float pg2 = 0; okf = okf && qlm_load(&q, path, &it2, &pg2);
        float *part = (float *)dmalloc(64 * 3 * 4);
        for(int si = 0; si < q.nspan; si++)
            qlm_fused_spans(&q, Pd, Gd, si, 1, (size_t)q.spanH[si].gof, (size_t)q.spanH[si].n, part + 64 * si, lr, wd, T2, pg2);
        qlmx_sync(NULL);
        qlmx_memcpy_d2h(fd.data(), q.d, nd); qlmx_memcpy_d2h(fr.data(), q.r, nq); qlmx_memcpy_d2h(fm.data(), q.m8, nq);
        check("qlm fused per-span step == whole step", (okf && !memcmp(wd_.data(), fd.data(), nd) && !memcmp(wr.data(), fr.data(), nq) && !memcmp(wm.data(), fm.data(), nq)) ? 0 : 1, 0);
        double ss = 0; for(int si = 0; si < q.nspan; si++) for(unsigned long long i = 0; i < q.spanH[si].n; i++){ double g = Gh[q.spanH[si].gof + i]; ss += g * g; }
        const float gn = qlm_fused_tail(part, 3, NULL, 0);
        check("qlm fused grad norm rel-err", fabs((double)gn - sqrt(ss)) / sqrt(ss), 1e-6);
    }
    remove(path);

    /* (d) expert forward through the grouped queue, weights addressed as P + offset */
    qlm_gpu_render(&q, Pd);                         /* host copy of what the digits mean */
    qlmx_memcpy_d2h(Pr.data(), Pd, np * 4);
    std::vector<float> X((size_t)N * D), Y((size_t)N * F, 0.f), Yref((size_t)N * F, 0.f);
    for(auto &v : X) v = nrand();
    float *Xd = (float *)dmalloc(X.size() * 4), *Yd = (float *)dmalloc(Y.size() * 4);
    qlmx_memcpy_h2d(Xd, X.data(), X.size() * 4);
    int off[4] = {0, 13, 13, 40};                   /* expert 1 gets no rows */
    mg_bind(&q, Pd, QLMX_ACT_F32, QLMX_MATH_F32);
    for(int e = 0; e < E; e++){ int ne = off[e + 1] - off[e]; if(!ne) continue;
        mg_ab(Xd + (size_t)off[e] * D, Pd + 16 + (size_t)e * D * F, Yd + (size_t)off[e] * F, ne, D, F); }
    mg_flush(); qlmx_sync(NULL);
    qlmx_memcpy_d2h(Y.data(), Yd, Y.size() * 4);
    for(int e = 0; e < E; e++) for(int m = off[e]; m < off[e + 1]; m++) for(int f = 0; f < F; f++){
        double acc = 0; for(int k = 0; k < D; k++) acc += (double)X[(size_t)m * D + k] * Pr[16 + (size_t)e * D * F + (size_t)k * F + f];
        Yref[(size_t)m * F + f] = (float)acc; }
    double num = 0, den = 0; for(size_t i = 0; i < Y.size(); i++){ double dlt = (double)Y[i] - Yref[i]; num += dlt * dlt; den += (double)Yref[i] * Yref[i]; }
    check("moe expert fwd (mg_ab) rel-err", sqrt(num / den), 1e-3);

    /* (d2) a weight-gradient problem that reads an output of the SAME flush (the reference runs its queues in
     * order on one stream, cudalm.cu:3243, so this is legal there): Gw[D,F] += X^T . Y with Y written by the queue-0
     * problem above it. The flush must notice the dependency and not run the two side by side. */
    {
        const int e = 2, ne = off[e + 1] - off[e];
        std::vector<float> Gw((size_t)D * F, 0.f), Gref((size_t)D * F, 0.f);
        float *Gwd = (float *)dmalloc(Gw.size() * 4);
        qlmx_memset(Gwd, 0, Gw.size() * 4, NULL); qlmx_memset(Yd, 0, Y.size() * 4, NULL);
        mg_ab(Xd + (size_t)off[e] * D, Pd + 16 + (size_t)e * D * F, Yd + (size_t)off[e] * F, ne, D, F);
        mg_atb(Xd + (size_t)off[e] * D, Yd + (size_t)off[e] * F, Gwd, ne, D, F);
        mg_flush(); qlmx_sync(NULL);
        qlmx_memcpy_d2h(Gw.data(), Gwd, Gw.size() * 4);
        double n2 = 0, d2 = 0;
        for(int k = 0; k < D; k++) for(int f = 0; f < F; f++){
            double acc = 0; for(int m = off[e]; m < off[e + 1]; m++) acc += (double)X[(size_t)m * D + k] * Yref[(size_t)m * F + f];
            const double dlt = (double)Gw[(size_t)k * F + f] - acc; n2 += dlt * dlt; d2 += acc * acc; }
        check("wgrad reading the flush's own output", sqrt(n2 / d2), 1e-3);
    }

    /* (e) input gradient of w1 and w3 through the queue as the reference issues it (beta 0, then beta 1
     * on the same output), bf16 activations on the matrix cores: the flush runs each pair as one launch */
    {
        auto bf16 = [](float f) -> unsigned short { unsigned u; memcpy(&u, &f, 4); u += 0x7FFFu + ((u >> 16) & 1u); return (unsigned short)(u >> 16); };
        auto f32 = [](unsigned short h) -> float { unsigned u = (unsigned)h << 16; float f; memcpy(&f, &u, 4); return f; };
        std::vector<unsigned short> dg((size_t)N * F), du((size_t)N * F);
        for(auto &v : dg) v = bf16(nrand());
        for(auto &v : du) v = bf16(nrand());
        std::vector<float> dX((size_t)N * D, 0.f);
        void *dgd = dmalloc(dg.size() * 2), *dud = dmalloc(du.size() * 2); float *dXd = (float *)dmalloc(dX.size() * 4);
        qlmx_memcpy_h2d(dgd, dg.data(), dg.size() * 2); qlmx_memcpy_h2d(dud, du.data(), du.size() * 2);
        mg_bind(&q, Pd, QLMX_ACT_BF16, QLMX_MATH_MFMA);
        for(int e = 0; e < E; e++){ int ne = off[e + 1] - off[e]; if(!ne) continue;
            mg_abt_b((const unsigned short *)dgd + (size_t)off[e] * F, Pd + 16 + (size_t)e * D * F, dXd + (size_t)off[e] * D, ne, F, D, 0.0f);
            mg_abt_b((const unsigned short *)dud + (size_t)off[e] * F, Pd + 16 + nw + (size_t)e * D * F, dXd + (size_t)off[e] * D, ne, F, D, 1.0f); }
        mg_flush(); qlmx_sync(NULL);
        qlmx_memcpy_d2h(dX.data(), dXd, dX.size() * 4);
        double num2 = 0, den2 = 0;
        for(int e = 0; e < E; e++) for(int m = off[e]; m < off[e + 1]; m++) for(int k = 0; k < D; k++){
            double acc = 0;
            for(int f = 0; f < F; f++) acc += (double)f32(dg[(size_t)m * F + f]) * Pr[16 + (size_t)e * D * F + (size_t)k * F + f]
                                            + (double)f32(du[(size_t)m * F + f]) * Pr[16 + nw + (size_t)e * D * F + (size_t)k * F + f];
            const double dlt = (double)dX[(size_t)m * D + k] - acc; num2 += dlt * dlt; den2 += acc * acc; }
        check("moe dgrad w1+w3 (mg_abt_b pair) rel-err", sqrt(num2 / den2), 1e-3);

        /* (f) gate | up | SwiGLU as one queued item per expert, bf16 activations on the matrix cores */
        std::vector<unsigned short> Xb((size_t)N * D), apb((size_t)N * F, 0);
        for(size_t i = 0; i < Xb.size(); i++) Xb[i] = bf16(X[i]);
        void *Xbd = dmalloc(Xb.size() * 2), *apd = dmalloc(apb.size() * 2);
        float *gpd = (float *)dmalloc((size_t)N * F * 4), *upd = (float *)dmalloc((size_t)N * F * 4);
        qlmx_memcpy_h2d(Xbd, Xb.data(), Xb.size() * 2);
        for(int e = 0; e < E; e++){ int ne = off[e + 1] - off[e]; if(!ne) continue;
            mg_ab_swiglu((const unsigned short *)Xbd + (size_t)off[e] * D, Pd + 16 + (size_t)e * D * F, Pd + 16 + nw + (size_t)e * D * F,
                         gpd + (size_t)off[e] * F, upd + (size_t)off[e] * F, (unsigned short *)apd + (size_t)off[e] * F, ne, D, F); }
        mg_flush(); qlmx_sync(NULL);
        qlmx_memcpy_d2h(apb.data(), apd, apb.size() * 2);
        double num3 = 0, den3 = 0;
        for(int e = 0; e < E; e++) for(int m = off[e]; m < off[e + 1]; m++) for(int f = 0; f < F; f++){
            double g = 0, u = 0;
            for(int k = 0; k < D; k++){ const double x = f32(Xb[(size_t)m * D + k]);
                g += x * Pr[16 + (size_t)e * D * F + (size_t)k * F + f]; u += x * Pr[16 + nw + (size_t)e * D * F + (size_t)k * F + f]; }
            const double want = g / (1.0 + exp(-g)) * u, dlt = (double)f32(apb[(size_t)m * F + f]) - want;
            num3 += dlt * dlt; den3 += want * want; }
        check("moe gate|up|swiglu (mg_ab_swiglu) rel-err", sqrt(num3 / den3), 5e-3);   /* bf16 output: 2^-9 per element */
    }
    qlm_free(&q);
    printf(ok_all ? "[selftest] ALL PASS\n" : "[selftest] FAILED\n");
    return ok_all ? 0 : 1;
}
