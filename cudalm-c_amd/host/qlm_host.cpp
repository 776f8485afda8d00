/* qlm_host.cpp -- see qlm_host.h. Host logic only; every device operation goes through libqlmx. */
#include "qlm_host.h"
#include <fcntl.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <sys/stat.h>
#include <unistd.h>
#include <algorithm>
#include <functional>
#include <numeric>
#include <string>
#include <vector>

typedef unsigned long long u64;

static void ck(int rc, const char *what){
    if(rc != QLMX_OK){ fprintf(stderr, "HIP error: %s at %s\n", qlmx_last_error(), what); exit(1); }
}
void *dmalloc(size_t bytes){ void *p = NULL; ck(qlmx_malloc(&p, bytes), "hipMalloc"); return p; }

/* ---------------------------------------------------------------------------------------------
 * Configuration. The reference reads its switches from the environment inside qlm_gpu_init
 * (qlm.cuh:459-474); here they are parsed once into a value that init applies. The rules are the
 * reference's: bits -> largest digit {<=2: 1, 3: 3, 4: 7, else 127}; group clamped to [32, 256];
 * "abs" selects the absolute LR mode; "qlion" the sign optimizer; the rail-fraction target defaults
 * to 0.60 for ternary digits and 1.5 elements per group otherwise, with a +-50 % dead band.
 * ------------------------------------------------------------------------------------------- */
namespace {
struct QlmKnobs { int dmax, group, lrmode, servo_every, adam, v4; float fstar; };

const char *env_or(const char *name, const char *fallback){ const char *v = getenv(name); return v ? v : fallback; }

QlmKnobs knobs_from_env(){
    QlmKnobs k;
    const int bits = atoi(env_or("QLM_BITS", "4"));
    k.dmax = bits <= 2 ? 1 : bits == 3 ? 3 : bits == 4 ? 7 : 127;
    k.group = std::min(256, std::max(32, atoi(env_or("QLM_GROUP", "128"))));
    k.lrmode = strcmp(env_or("QLM_LRMODE", "rel"), "abs") == 0;
    k.servo_every = atoi(env_or("QLM_SERVO", "100"));
    k.adam = strcmp(env_or("QLM_OPT", ""), "qlion") != 0;
    k.v4 = atoi(env_or("QLM_V4", "0")) != 0;
    const char *fs = getenv("QLM_FSTAR");
    k.fstar = fs ? (float)atof(fs) : (k.dmax == 1 ? 0.60f : 1.5f / (float)k.group);
    return k;
}

/* Every device array a Qlm owns, with its size: one table drives allocation, clearing and release. */
struct OwnedArray { void **slot; size_t bytes; bool cleared; };
std::vector<OwnedArray> owned_arrays(Qlm *q){
    const size_t nq = q->nq, ng4 = (size_t)q->ngrp * 4;
    std::vector<OwnedArray> t = {
        {(void **)&q->d,  (size_t)qlmx_qd_bytes(q->nq, q->packed), false},
        {(void **)&q->r,  nq, false},
        {(void **)&q->m8, nq, true},
        {(void **)&q->s,  ng4, false},
        {(void **)&q->m8s, ng4, true},
        {(void **)&q->statD, 4 * sizeof(long long), true},
        {(void **)&q->spanD, (size_t)q->nspan * sizeof(QSpanD), false},
    };
    if(q->adam){ t.push_back({(void **)&q->v8, nq, true}); t.push_back({(void **)&q->v8s, ng4, true}); }
    return t;
}

void upload_spans(Qlm *q, const char *what){
    ck(qlmx_memcpy_h2d(q->spanD, q->spanH, (size_t)q->nspan * sizeof(QSpanD)), what);
}

/* The parameters between and around the quantized spans stay in floating point; the reference keeps
 * their optimizer moments compact, so each gap gets its offset in P, its length and its offset in the
 * compact arrays (qlm.cuh:492-501). Spans are in ascending order of pof. */
void index_float_gaps(Qlm *q){
    q->nfs = 0; q->nfloat = 0;
    auto add = [&](u64 from, u64 to){
        if(to <= from) return;
        q->fs_off[q->nfs] = from; q->fs_n[q->nfs] = to - from; q->fs_cs[q->nfs] = q->nfloat;
        q->nfloat += to - from; q->nfs++;
    };
    u64 edge = 0;
    for(int i = 0; i < q->nspan; i++){ add(edge, q->spanH[i].pof); edge = q->spanH[i].pof + q->spanH[i].n; }
    add(edge, q->np);
}

/* sref of every span = mean of its group scales, summed in double in group order (qlm.cuh:527-536;
 * the order is part of the contract: the relative-LR step divides by this float) */
void freeze_reference_scales(Qlm *q){
    std::vector<float> scales(q->ngrp);
    ck(qlmx_memcpy_d2h(scales.data(), q->s, (size_t)q->ngrp * 4), "qlm s d2h");
    for(int i = 0; i < q->nspan; i++){
        QSpanD &sp = q->spanH[i];
        const float *first = scales.data() + sp.gi0;
        sp.sref = (float)(std::accumulate(first, first + sp.ngrp, 0.0) / (double)sp.ngrp);
    }
    upload_spans(q, "qlm span h2d (sref)");
}
}  // namespace

/* qlm.cuh:448-455: a span is appended behind everything registered so far */
void qlm_add_span(Qlm *q, unsigned long long pof, unsigned long long n){
    if(q->nspan >= QLM_MAXSPAN) return;
    QSpanD sp;
    sp.pof = sp.gof = pof; sp.n = n; sp.qi0 = q->nq;
    sp.gi0 = (int)q->ngrp; sp.ngrp = (int)((n + (u64)q->group - 1) / (u64)q->group);
    sp.sref = 1.0f;
    q->spanH[q->nspan++] = sp;
    q->nq += n; q->ngrp += (u64)sp.ngrp;
}

/* qlm.cuh:458-541: switches, span table, float gaps, device state, and -- when the caller still holds an
 * fp32 view P -- encode, frozen reference scales and the first render. */
void qlm_gpu_init(Qlm *q, const QlmSpanDesc *spans, int nspan, float *P, size_t np){
    *q = Qlm();
    const QlmKnobs k = knobs_from_env();
    q->dmax = k.dmax; q->group = k.group; q->lrmode = k.lrmode; q->servo_every = k.servo_every;
    q->adam = k.adam; q->v4 = k.v4; q->packed = k.dmax <= 7;
    q->fstar = k.fstar; q->f_hi = 1.5f * k.fstar; q->f_lo = 0.5f * k.fstar;
    q->np = np; q->render_p = P != NULL;
    q->spanH = (QSpanD *)calloc(QLM_MAXSPAN, sizeof(QSpanD));
    for(int i = 0; i < nspan; i++) qlm_add_span(q, spans[i].pof, spans[i].n);
    index_float_gaps(q);
    for(const OwnedArray &a : owned_arrays(q)){
        *a.slot = dmalloc(a.bytes);
        if(a.cleared) ck(qlmx_memset(*a.slot, 0, a.bytes, NULL), "qlm state clear");
    }
    upload_spans(q, "qlm span h2d");
    if(P){
        ck(qlmx_encode(P, q->d, q->r, q->s, q->spanD, q->nspan, q->group, q->dmax, q->packed, (int)q->ngrp, NULL), "qlm encode");
        freeze_reference_scales(q);
        qlm_gpu_render(q, P);
    }
    q->on = 1;
}

void qlm_free(Qlm *q){
    for(const OwnedArray &a : owned_arrays(q)) if(*a.slot) qlmx_free(*a.slot);
    free(q->spanH);
    *q = Qlm();
}

/* first group and number of groups of spans [span0, span0 + nspans) */
static void group_range(const Qlm *q, int span0, int nspans, int *gi0, int *ng){
    *gi0 = q->spanH[span0].gi0; *ng = 0;
    for(int i = span0; i < span0 + nspans; i++) *ng += q->spanH[i].ngrp;
}

void qlm_gpu_render(Qlm *q, float *P){
    ck(qlmx_render(P, q->d, q->s, q->spanD, q->nspan, q->group, q->packed, 0, (int)q->ngrp, NULL), "qlm render");
}
/* qlm.cuh:586-591 generalised: render the groups of spans [span0, span0+nspans) */
void qlm_render_spans(Qlm *q, float *P, int span0, int nspans){
    int gi0, ng; group_range(q, span0, nspans, &gi0, &ng);
    ck(qlmx_render(P, q->d, q->s, q->spanD, q->nspan, q->group, q->packed, gi0, ng, NULL), "qlm render layer");
}

/* qlm.cuh:377-397. The QLM_V4 switch travels as an argument of the C ABI; here it is read from
 * the environment once, as the reference does (qlm.cuh:68-72). */
void qlm_step_launch(float *P, const float *G, signed char *d, signed char *r, float *s,
                     signed char *m8, float *m8s, unsigned char *v8, float *v8s,
                     const QSpanD *sp, int nspan, int group, int dmax,
                     float lr, float b1, float b2, float wd, float gscale, const float *gsp,
                     float inv_bc1, float inv_sqrt_bc2, int lrmode,
                     unsigned long long t, int adam, long long *stat, int packed, int gi_base, int ng){
    static const int v4 = knobs_from_env().v4;
    ck(qlmx_step(P, G, d, r, s, m8, m8s, v8, v8s, sp, nspan, group, dmax, lr, b1, b2, wd, gscale, gsp,
                 inv_bc1, inv_sqrt_bc2, lrmode, t, adam, stat, packed, gi_base, ng, v4, NULL), "qlm step");
}

/* One step over groups [gi0, gi0 + ng) of q with the bias corrections already inverted */
static void step_groups(Qlm *q, float *P, const float *G, int gi0, int ng, float lr, float b1, float b2, float wd,
                        float gscale, const float *gsp, float bc1, float bc2, int t, long long *stat){
    qlm_step_launch(q->render_p ? P : NULL, G, q->d, q->r, q->s, q->m8, q->m8s, q->v8, q->v8s, q->spanD, q->nspan,
                    q->group, q->dmax, lr, b1, b2, wd, gscale, gsp, 1.0f / bc1, 1.0f / sqrtf(bc2), q->lrmode,
                    (unsigned long long)t, q->adam, stat, q->packed, gi0, ng);
}

/* cudalm.cu:6082-6103 without the float spans' AdamW: the whole-model step, then the scale servo on its period */
void qlm_gpu_update(Qlm *q, float *P, float *G, float lr, float b1, float b2, float wd,
                    float bc1, float bc2, int t, const float *gs){
    step_groups(q, P, G, 0, (int)q->ngrp, lr, b1, b2, wd, 1.0f, gs, bc1, bc2, t, getenv("CUDALM_QLM_DIAG") ? q->statD : NULL);
    kchk("qlm step", -1);                                              /* cudalm.cu:6089 */
    const bool servo_due = q->servo_every > 0 && t % q->servo_every == 0;
    if(servo_due){
        ck(qlmx_servo(q->d, q->r, q->s, q->spanD, q->nspan, q->group, q->dmax, q->f_hi, q->f_lo, q->packed, (int)q->ngrp, NULL), "qlm servo");
        kchk("qlm servo", -1);                                         /* cudalm.cu:6101 */
    }
}

/* cudalm.cu:6110-6135 without the float spans' AdamW and the diagnostics */
void qlm_fused_spans(Qlm *q, float *P, float *G, int span0, int nspans, size_t g0, size_t gn, float *part64,
                     float lr, float wd, int t, float prev_gn){
    const float b1 = 0.9f, b2 = 0.95f;
    ck(qlmx_sqsum(G + g0, (unsigned long long)gn, part64, NULL), "fused sqsum");
    int gi0, ng; group_range(q, span0, nspans, &gi0, &ng);
    step_groups(q, P, G, gi0, ng, lr, b1, b2, wd, prev_gn > 1.0f ? 1.0f / prev_gn : 1.0f, NULL,
                1.0f - powf(b1, (float)t), 1.0f - powf(b2, (float)t), t, NULL);
}
void qlm_fused_layer(Qlm *q, float *P, float *G, size_t layer_g0, size_t layer_gn, float *gnpart, int l,
                     float lr, float wd, int t, float prev_gn){
    qlm_fused_spans(q, P, G, 7 * l, 7, layer_g0, layer_gn, gnpart + 64 * (size_t)l, lr, wd, t, prev_gn);
}
/* cudalm.cu:6176-6186 */
float qlm_fused_tail(const float *gnpart, int L, const float *extra, int nextra){
    const size_t nsl = 64 * (size_t)L, nex = 64 * (size_t)nextra;
    std::vector<float> ph(nsl + nex);
    if(nsl) ck(qlmx_memcpy_d2h(ph.data(), gnpart, nsl * 4), "fused sqsum d2h");
    if(nex) ck(qlmx_memcpy_d2h(ph.data() + nsl, extra, nex * 4), "fused tail sqsum d2h");
    return (float)sqrt(std::accumulate(ph.begin(), ph.end(), 0.0));
}

/* qlm.cuh:678-683 */
double qlm_persist_bytes(const Qlm *q){
    return (double)qlmx_qd_bytes(q->nq, q->packed) + (double)q->nq * 1.0 + (double)q->nq * (q->adam ? 2.0 : 1.0)
         + (double)q->ngrp * 4.0 * (q->adam ? 3.0 : 2.0);
}

/* ---------------------------------------------------------------------------------------------
 * .opt.q checkpoint (qlm.cuh:702-788). Bytes, in order:
 *   "QLMH", int32 x6 {dmax, group, adam, nspan, packed, iter}, u64 x3 {nq, ngrp, nfloat},
 *   bf16 Mc[nfloat], bf16 Vc[nfloat], d, r, m8, [v8 when adam], fp32 s, m8s, [v8s when adam],
 *   "SREF", int32 nspan, fp32 sref[nspan], "PGN1", fp32 previous gradient norm.
 * The body is a list of sections; the writer and the reader walk the same list, and each section moves
 * through one bounce buffer piece by piece (the state of a large model does not fit the host twice).
 * A section lives in device memory (the Qlm's arrays) or in host memory (the *_host entry points that
 * tools and CPU tests use); `absent` sections are written as zeros and skipped when read.
 * ------------------------------------------------------------------------------------------- */
namespace {
struct Section { void *ptr; size_t bytes; bool absent; };
struct OptqBody {
    int hdr[6]; u64 nq, ngrp, nfloat;
    std::vector<Section> sections;
    float *sref; int nspan;
    bool device;                   /* where the sections' memory is */
};

OptqBody describe(int dmax, int group, int adam, int nspan, int packed, u64 nq, u64 ngrp, u64 nfloat,
                  void *Mc, void *Vc, void *d, void *r, void *m8, void *v8, void *s, void *m8s, void *v8s, bool device){
    OptqBody b;
    const int hdr[6] = {dmax, group, adam, nspan, packed, 0};
    memcpy(b.hdr, hdr, sizeof hdr);
    b.nq = nq; b.ngrp = ngrp; b.nfloat = nfloat; b.nspan = nspan; b.sref = NULL; b.device = device;
    const size_t nd = (size_t)qlmx_qd_bytes(nq, packed);
    b.sections = {{Mc, (size_t)nfloat * 2, Mc == NULL}, {Vc, (size_t)nfloat * 2, Vc == NULL},
                  {d, nd, false}, {r, (size_t)nq, false}, {m8, (size_t)nq, false}};
    if(adam) b.sections.push_back({v8, (size_t)nq, false});
    b.sections.push_back({s, (size_t)ngrp * 4, false});
    b.sections.push_back({m8s, (size_t)ngrp * 4, false});
    if(adam) b.sections.push_back({v8s, (size_t)ngrp * 4, false});
    return b;
}

const size_t BOUNCE = (size_t)8 << 20;

bool put(FILE *f, const void *p, size_t n){ return fwrite(p, 1, n, f) == n; }
bool get(FILE *f, void *p, size_t n){ return fread(p, 1, n, f) == n; }

bool write_section(FILE *f, const Section &sec, bool device, std::vector<unsigned char> &bounce){
    for(size_t at = 0; at < sec.bytes; at += BOUNCE){
        const size_t n = std::min(BOUNCE, sec.bytes - at);
        const void *src = (const unsigned char *)sec.ptr + at;
        if(sec.absent){ memset(bounce.data(), 0, n); src = bounce.data(); }
        else if(device){ ck(qlmx_memcpy_d2h(bounce.data(), src, n), "qlm save d2h"); src = bounce.data(); }
        if(!put(f, src, n)) return false;
    }
    return true;
}
bool read_section(FILE *f, const Section &sec, bool device, std::vector<unsigned char> &bounce){
    for(size_t at = 0; at < sec.bytes; at += BOUNCE){
        const size_t n = std::min(BOUNCE, sec.bytes - at);
        void *dst = (unsigned char *)sec.ptr + at;
        if(sec.absent || device){
            if(!get(f, bounce.data(), n)) return false;
            if(!sec.absent) ck(qlmx_memcpy_h2d(dst, bounce.data(), n), "qlm load h2d");
        } else if(!get(f, dst, n)) return false;
    }
    return true;
}

/* fflush + fsync + close, rename over the target, fsync of the directory: after an unclean shutdown the
 * name refers either to the old complete file or to the new complete one (the reference's save_commit,
 * cudalm.cu:509-519, gives the reason: a checkpoint of full length whose tail was zeros). */
bool commit_file(FILE *f, bool ok, const std::string &tmp, const std::string &path){
    ok = ok && !ferror(f) && fflush(f) == 0 && !ferror(f) && fsync(fileno(f)) == 0;
    if(fclose(f) != 0) ok = false;
    if(!ok || rename(tmp.c_str(), path.c_str()) != 0){ remove(tmp.c_str()); return false; }
    const size_t slash = path.find_last_of('/');
    const std::string dir = slash == std::string::npos ? "." : (slash == 0 ? "/" : path.substr(0, slash));
    const int dfd = open(dir.c_str(), O_RDONLY);
    if(dfd >= 0){ fsync(dfd); close(dfd); }
    return true;
}

bool write_optq(const char *path, OptqBody &b, int iter, float prev_gn){
    const std::string tmp = std::string(path) + ".tmp";
    FILE *f = fopen(tmp.c_str(), "wb");
    if(!f) return false;
    std::vector<unsigned char> bounce(BOUNCE);
    b.hdr[5] = iter;
    bool ok = put(f, "QLMH", 4) && put(f, b.hdr, sizeof b.hdr) && put(f, &b.nq, 8) && put(f, &b.ngrp, 8) && put(f, &b.nfloat, 8);
    for(size_t i = 0; ok && i < b.sections.size(); i++) ok = write_section(f, b.sections[i], b.device, bounce);
    ok = ok && put(f, "SREF", 4) && put(f, &b.nspan, 4) && put(f, b.sref, (size_t)b.nspan * 4);
    ok = ok && put(f, "PGN1", 4) && put(f, &prev_gn, 4);
    return commit_file(f, ok, tmp, path);
}

/* 0: unreadable, of another shape, or shorter than its header promises (nothing of `b` is touched);
 * 1: loaded. *have_sref says whether the reference-scale trailer was there. */
int read_optq(const char *path, OptqBody &b, int *iter, float *prev_gn, bool *have_sref){
    FILE *f = fopen(path, "rb");
    if(!f) return 0;
    struct Closer { FILE *f; ~Closer(){ fclose(f); } } closer{f};
    char magic[4]; int hdr[6]; u64 nq, ngrp, nfloat;
    if(!get(f, magic, 4) || memcmp(magic, "QLMH", 4) != 0) return 0;
    if(!get(f, hdr, sizeof hdr) || !get(f, &nq, 8) || !get(f, &ngrp, 8) || !get(f, &nfloat, 8)) return 0;
    const bool same_shape = hdr[0] == b.hdr[0] && hdr[1] == b.hdr[1] && hdr[2] == b.hdr[2] && hdr[4] == b.hdr[4]
                         && nq == b.nq && ngrp == b.ngrp && nfloat <= b.nfloat;
    if(!same_shape){ fprintf(stderr, "[qlm] %s was written for another shape (digits, group or optimizer differ): ignored\n", path); return 0; }
    if(nfloat < b.nfloat)       /* float parameters appended since the file was written keep their zero moments */
        fprintf(stderr, "[qlm] %s: %llu float parameters are newer than the file and start from zero moments\n", path, b.nfloat - nfloat);
    b.sections[0].bytes = b.sections[1].bytes = (size_t)nfloat * 2;
    size_t body = 0;
    for(const Section &s : b.sections) body += s.bytes;
    struct stat st;
    if(fstat(fileno(f), &st) != 0 || (u64)st.st_size < 4 + sizeof hdr + 24 + body) return 0;     /* truncated: leave the state alone */
    std::vector<unsigned char> bounce(BOUNCE);
    for(const Section &s : b.sections) if(!read_section(f, s, b.device, bounce)) return 0;
    if(iter) *iter = hdr[5];
    char tag[4]; int ns = 0; float pg = 0.0f;
    std::vector<float> sr;
    *have_sref = get(f, tag, 4) && memcmp(tag, "SREF", 4) == 0 && get(f, &ns, 4) && ns == b.nspan
              && (sr.resize((size_t)ns), get(f, sr.data(), (size_t)ns * 4));
    if(*have_sref){
        std::copy(sr.begin(), sr.end(), b.sref);
        if(get(f, tag, 4) && memcmp(tag, "PGN1", 4) == 0 && get(f, &pg, 4) && pg > 0.0f && isfinite(pg) && prev_gn) *prev_gn = pg;
    }
    return 1;
}
}  // namespace

int qlm_save(const Qlm *q, const char *path, int iter, float prev_gn){
    OptqBody b = describe(q->dmax, q->group, q->adam, q->nspan, q->packed, q->nq, q->ngrp, q->nfloat,
                          q->Mc, q->Vc, q->d, q->r, q->m8, q->v8, q->s, q->m8s, q->v8s, true);
    std::vector<float> sref(q->nspan);
    for(int i = 0; i < q->nspan; i++) sref[i] = q->spanH[i].sref;
    b.sref = sref.data();
    return write_optq(path, b, iter, prev_gn) ? 1 : 0;
}

int qlm_load(Qlm *q, const char *path, int *iter, float *prev_gn){
    OptqBody b = describe(q->dmax, q->group, q->adam, q->nspan, q->packed, q->nq, q->ngrp, q->nfloat,
                          q->Mc, q->Vc, q->d, q->r, q->m8, q->v8, q->s, q->m8s, q->v8s, true);
    std::vector<float> sref(q->nspan);
    b.sref = sref.data();
    bool have_sref = false;
    if(!read_optq(path, b, iter, prev_gn, &have_sref)) return 0;
    if(have_sref){
        for(int i = 0; i < q->nspan; i++) q->spanH[i].sref = sref[i];
        upload_spans(q, "qlm load span");
    } else
        fprintf(stderr, "[qlm] %s carries no reference scales: the spans keep the ones derived at init, so the relative step size may change here\n", path);
    return 1;
}

/* The same file format over host memory (no device needed): for tools and for the byte-level tests
 * against files the reference wrote. */
extern "C" int qlm_optq_write_host(const char *path, const QlmOptqHost *v){
    OptqBody b = describe(v->dmax, v->group, v->adam, v->nspan, v->packed, v->nq, v->ngrp, v->nfloat,
                          v->Mc, v->Vc, v->d, v->r, v->m8, v->v8, v->s, v->m8s, v->v8s, false);
    b.sref = v->sref;
    return write_optq(path, b, v->iter, v->prev_gn) ? 1 : 0;
}
extern "C" int qlm_optq_read_host(const char *path, QlmOptqHost *v){
    OptqBody b = describe(v->dmax, v->group, v->adam, v->nspan, v->packed, v->nq, v->ngrp, v->nfloat,
                          v->Mc, v->Vc, v->d, v->r, v->m8, v->v8, v->s, v->m8s, v->v8s, false);
    b.sref = v->sref;
    bool have_sref = false;
    const int ok = read_optq(path, b, &v->iter, &v->prev_gn, &have_sref);
    v->have_sref = have_sref;
    return ok;
}

/* ---------------------------------------------------------------------------------------------
 * Grouped expert GEMM queue (cudalm.cu:3204-3256). Queue 0: beta = 0 problems (nn and tn), queue 1:
 * tn problems with beta != 0, which accumulate into a C a queue-0 problem writes and therefore run
 * strictly after queue 0, queue 2: nt weight gradients. A flush issues each queue as one grouped
 * launch per (orientation, K, N).
 * ------------------------------------------------------------------------------------------- */
struct MgItem { int mode, K, N; qlmx_gemm_prob p; };
static std::vector<MgItem> g_q[3];
static const Qlm *g_mg_q = NULL; static const float *g_mg_P = NULL; static int g_mg_act = QLMX_ACT_F32, g_mg_math = QLMX_MATH_F32;

void mg_bind(const Qlm *q, const float *Pbase, int act_dtype, int math){ g_mg_q = q; g_mg_P = Pbase; g_mg_act = act_dtype; g_mg_math = math; }

/* pointer into P -> (digit offset, scale group) through the span table */
static void weight_of(const float *B, unsigned long long *wq, unsigned long long *wg){
    if(!g_mg_q){ fprintf(stderr, "mg: mg_bind() was not called\n"); exit(1); }
    const unsigned long long off = (unsigned long long)(B - g_mg_P);
    for(int i = 0; i < g_mg_q->nspan; i++){
        const QSpanD *sp = &g_mg_q->spanH[i];
        if(off >= sp->pof && off < sp->pof + sp->n){
            const unsigned long long in = off - sp->pof;
            if(in % (unsigned long long)g_mg_q->group){ fprintf(stderr, "mg: weight operand does not start on a scale group\n"); exit(1); }
            *wq = sp->qi0 + in; *wg = (unsigned long long)sp->gi0 + in / (unsigned long long)g_mg_q->group; return;
        }
    }
    fprintf(stderr, "mg: weight operand is not inside a quantized span\n"); exit(1);
}
static void mg_push(int qn, int mode, const void *A, const void *B, float *C, unsigned long long wq, unsigned long long wg,
                    int M, int K, int N, float beta){
    if(g_q[qn].size() >= QLMX_MAX_PROBLEMS){ fprintf(stderr, "mg queue overflow\n"); exit(1); }
    MgItem it; it.mode = mode; it.K = K; it.N = N;
    it.p.A = A; it.p.B = B; it.p.C = C; it.p.wq = wq; it.p.wg = wg; it.p.M = M; it.p.beta = beta;
    g_q[qn].push_back(it);
}
void mg_ab(const void *A, const float *B, float *C, int M, int K, int N){
    unsigned long long wq, wg; weight_of(B, &wq, &wg); mg_push(0, 0, A, NULL, C, wq, wg, M, K, N, 0.0f);
}
void mg_abt_b(const void *A, const float *B, float *C, int M, int K, int N, float beta){
    unsigned long long wq, wg; weight_of(B, &wq, &wg); mg_push(beta != 0.0f, 1, A, NULL, C, wq, wg, M, K, N, beta);
}
void mg_abt(const void *A, const float *B, float *C, int M, int K, int N){ mg_abt_b(A, B, C, M, K, N, 0.0f); }
void mg_atb(const void *A, const void *B, float *C, int M, int K, int N){ mg_push(2, 2, A, B, C, 0, 0, M, K, N, 1.0f); }

/* gate|up problems with the SwiGLU behind them: queued apart, flushed first as one call per (K, N) */
struct MgDual { int K, N; qlmx_gemm_prob gate, up; };
static std::vector<MgDual> g_qdual;
void mg_ab_swiglu(const void *A, const float *B1, const float *B3, float *gp, float *up, void *ap, int M, int K, int N){
    if(g_qdual.size() >= QLMX_MAX_PROBLEMS / 2){ fprintf(stderr, "mg queue overflow\n"); exit(1); }
    MgDual it; it.K = K; it.N = N;
    unsigned long long wq, wg;
    weight_of(B1, &wq, &wg);
    it.gate.A = A; it.gate.B = NULL; it.gate.C = gp; it.gate.wq = wq; it.gate.wg = wg; it.gate.M = M; it.gate.beta = 0.0f;
    weight_of(B3, &wq, &wg);
    it.up.A = NULL; it.up.B = ap; it.up.C = up; it.up.wq = wq; it.up.wg = wg; it.up.M = M; it.up.beta = 0.0f;
    g_qdual.push_back(it);
}
static void mg_run_dual(void){
    std::vector<char> done(g_qdual.size(), 0);
    for(size_t i = 0; i < g_qdual.size(); i++){
        if(done[i]) continue;
        std::vector<qlmx_gemm_prob> gate, up;
        for(size_t j = i; j < g_qdual.size(); j++)
            if(!done[j] && g_qdual[j].K == g_qdual[i].K && g_qdual[j].N == g_qdual[i].N){ gate.push_back(g_qdual[j].gate); up.push_back(g_qdual[j].up); done[j] = 1; }
        const int rc = qlmx_moe_gemm_nn_swiglu(g_mg_q->d, g_mg_q->s, g_mg_q->group, gate.data(), up.data(), (int)gate.size(),
                                               g_qdual[i].K, g_qdual[i].N, g_mg_act, g_mg_math, NULL);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped (gate|up): %s\n", rc, qlmx_last_error()); exit(1); }
    }
    g_qdual.clear();
}

static void mg_run(std::vector<MgItem> &v, void *stream = NULL){
    std::vector<char> done(v.size(), 0);
    for(size_t i = 0; i < v.size(); i++){
        if(done[i]) continue;
        std::vector<qlmx_gemm_prob> batch;
        for(size_t j = i; j < v.size(); j++)
            if(!done[j] && v[j].mode == v[i].mode && v[j].K == v[i].K && v[j].N == v[i].N){ batch.push_back(v[j].p); done[j] = 1; }
        int rc;
        if(v[i].mode == 0)      rc = qlmx_moe_gemm_nn(g_mg_q->d, g_mg_q->s, g_mg_q->group, batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, stream);
        else if(v[i].mode == 1) rc = qlmx_moe_gemm_tn(g_mg_q->d, g_mg_q->s, g_mg_q->group, batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, stream);
        else                    rc = qlmx_moe_gemm_nt(batch.data(), (int)batch.size(), v[i].K, v[i].N, g_mg_act, g_mg_math, stream);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped: %s\n", rc, qlmx_last_error()); exit(1); }
    }
    v.clear();
}
/* A queue-1 problem (tn, beta = 1) whose output a queue-0 tn problem of the same shape writes is that
 * problem's second half (cudalm.cu:4365-4366): on the MFMA path the two run as one continued
 * contraction per (K, N) instead of two launches with the output stored and read back in between. */
static void mg_run_pairs(void){
    if(g_mg_act != QLMX_ACT_BF16 || g_mg_math != QLMX_MATH_MFMA) return;
    std::vector<MgItem> &v0 = g_q[0], &v1 = g_q[1];
    std::vector<int> mate(v1.size(), -1);
    std::vector<char> used(v0.size(), 0);
    bool any = false;
    for(size_t j = 0; j < v1.size(); j++){
        if(v1[j].mode != 1 || v1[j].p.beta != 1.0f || v1[j].p.M == 0) continue;
        for(size_t i = 0; i < v0.size(); i++)
            if(!used[i] && v0[i].mode == 1 && v0[i].p.C == v1[j].p.C && v0[i].p.M == v1[j].p.M && v0[i].K == v1[j].K && v0[i].N == v1[j].N){
                mate[j] = (int)i; used[i] = 1; any = true; break;
            }
    }
    if(!any) return;
    std::vector<char> done(v1.size(), 0);
    for(size_t j = 0; j < v1.size(); j++){
        if(done[j] || mate[j] < 0) continue;
        std::vector<qlmx_gemm_prob> first, second;
        for(size_t k = j; k < v1.size() && first.size() < QLMX_MAX_PROBLEMS / 2; k++)
            if(!done[k] && mate[k] >= 0 && v1[k].K == v1[j].K && v1[k].N == v1[j].N){ first.push_back(v0[mate[k]].p); second.push_back(v1[k].p); done[k] = 1; }
        const int rc = qlmx_moe_gemm_tn_pair(g_mg_q->d, g_mg_q->s, g_mg_q->group, first.data(), second.data(), (int)first.size(),
                                             v1[j].K, v1[j].N, g_mg_act, g_mg_math, NULL);
        if(rc != QLMX_OK){ fprintf(stderr, "grouped GEMM error %d at mg grouped (pairs): %s\n", rc, qlmx_last_error()); exit(1); }
    }
    std::vector<MgItem> r0, r1;
    for(size_t i = 0; i < v0.size(); i++) if(!used[i]) r0.push_back(v0[i]);
    for(size_t j = 0; j < v1.size(); j++) if(!done[j]) r1.push_back(v1[j]);
    v0.swap(r0); v1.swap(r1);
}
/* The problems of a flush do not depend on each other except queue 1 on queue 0 (it accumulates into what queue 0
 * writes). The weight gradients (queue 2) of a flush that also holds input gradients go into one grid with the
 * first input-gradient launch (qlmx_pair_begin / qlmx_pair_end): neither fills the device to the end of its last
 * round of tiles, and in one grid the one's tiles take the compute units the other leaves. */
static bool q2_reads_what_the_flush_writes(void){
    /* the reference issues queue 0, 1, 2 in order on one stream (cudalm.cu:3243), so there a weight-gradient
     * problem may read an output of the same flush; in one grid that would race, so such a flush runs in order */
    const size_t asz = g_mg_act == QLMX_ACT_BF16 ? 2 : 4;
    auto overlaps = [](const void *p, size_t n, const void *q, size_t m){
        const uintptr_t a = (uintptr_t)p, b = (uintptr_t)q;
        return p && q && a < b + m && b < a + n;
    };
    for(const MgItem &w : g_q[2])
        for(int qn = 0; qn < 2; qn++)
            for(const MgItem &o : g_q[qn]){
                const size_t out = (size_t)o.p.M * (size_t)o.N * 4;
                if(overlaps(w.p.A, (size_t)w.p.M * (size_t)w.K * asz, o.p.C, out) || overlaps(w.p.B, (size_t)w.p.M * (size_t)w.N * asz, o.p.C, out))
                    return true;
            }
    return false;
}
void mg_flush(void){
    mg_run_dual();
    const bool paired = !g_q[2].empty() && (!g_q[0].empty() || !g_q[1].empty()) && !q2_reads_what_the_flush_writes();
    if(paired && qlmx_pair_begin(NULL) != QLMX_OK){ fprintf(stderr, "mg_flush: %s\n", qlmx_last_error()); exit(1); }
    if(paired) mg_run(g_q[2]);                 /* held; leaves with the first input-gradient launch */
    mg_run_pairs(); mg_run(g_q[0]); mg_run(g_q[1]);
    if(paired){ if(qlmx_pair_end(NULL) != QLMX_OK){ fprintf(stderr, "mg_flush: %s\n", qlmx_last_error()); exit(1); } }
    else mg_run(g_q[2]);
}

/* ---- kchk / prof_report (cudalm.cu:787-855) ---- */
namespace {
struct LabelTime { std::string name; double ms = 0.0; long n = 0; };
struct CheckState {
    int debug = -1, prof = -1;                 /* -1: not read yet */
    double tdr = 2.0, prev = 0.0, max_ms = 0.0;
    std::string max_what = "(none)";
    std::vector<LabelTime> tab;                /* waiting modes; the event mode's table lives in the library */
};
CheckState g_chk;
double wall_seconds(){
    struct timespec ts; clock_gettime(CLOCK_MONOTONIC, &ts);
    return (double)ts.tv_sec + 1e-9 * (double)ts.tv_nsec;
}
void chk_levels_from_env(){
    if(g_chk.debug >= 0) return;
    const char *d = getenv("CUDALM_DEBUG"), *p = getenv("CUDALM_PROF");
    g_chk.debug = (d && atoi(d) != 0) ? 1 : 0;
    g_chk.prof = p ? atoi(p) : 0;
    g_chk.prev = wall_seconds();
}
}
void kchk_levels(int debug, int prof, double tdr_seconds){
    g_chk.debug = debug ? 1 : 0; g_chk.prof = prof; g_chk.tdr = tdr_seconds > 0.0 ? tdr_seconds : 2.0;
    g_chk.prev = wall_seconds(); g_chk.max_ms = 0.0; g_chk.max_what = "(none)"; g_chk.tab.clear();
    qlmx_prof_reset();
}
void kchk(const char *what, int l){
    chk_levels_from_env();
    if(!g_chk.debug && !g_chk.prof) return;
    if(g_chk.prof >= 3 && !g_chk.debug){
        if(qlmx_prof_mark(what, NULL) != QLMX_OK){ fprintf(stderr, "kchk: %s\n", qlmx_last_error()); exit(1); }
        return;
    }
    if(qlmx_sync(NULL) != QLMX_OK){
        fprintf(stderr, "\n[FAULT] after %s (layer %d): %s\n", what, l, qlmx_last_error());
        exit(1);
    }
    const double now = wall_seconds(), ms = (now - g_chk.prev) * 1000.0;
    g_chk.prev = now;
    if(g_chk.prof){
        size_t i = 0;
        while(i < g_chk.tab.size() && g_chk.tab[i].name != what) i++;
        if(i == g_chk.tab.size()){ g_chk.tab.emplace_back(); g_chk.tab.back().name = what; }
        g_chk.tab[i].ms += ms; g_chk.tab[i].n++;
    }
    if(ms > g_chk.max_ms){
        g_chk.max_ms = ms;
        char buf[128]; snprintf(buf, sizeof buf, "%s (layer %d)", what, l);
        g_chk.max_what = buf;
    }
    if(g_chk.debug && ms > g_chk.tdr * 1000.0 * 0.25)
        fprintf(stderr, "[WARN] %s (layer %d) took %.0f ms - %.0f%% of the %.0fs TDR budget\n", what, l, ms, 100.0 * ms / (g_chk.tdr * 1000.0), g_chk.tdr);
}
const char *kchk_slowest(double *ms){ if(ms) *ms = g_chk.max_ms; return g_chk.max_what.c_str(); }
void prof_report(void){
    chk_levels_from_env();
    if(!g_chk.prof) return;
    if(g_chk.prof >= 3 && !g_chk.debug){
        static char text[8192];
        int n = 0;
        if(qlmx_prof_report(text, sizeof text, &n) != QLMX_OK){ fprintf(stderr, "prof_report: %s\n", qlmx_last_error()); exit(1); }
        if(n) printf("\n%s", text);
        fflush(stdout);
        return;
    }
    if(g_chk.tab.empty()) return;
    std::vector<LabelTime> t = g_chk.tab;
    std::stable_sort(t.begin(), t.end(), [](const LabelTime &a, const LabelTime &b){ return a.ms > b.ms; });
    double tot = 0.0;
    for(const LabelTime &e : t) tot += e.ms;
    printf("\n[prof] per-kernel totals over the run (%.0f ms tracked)\n", tot);
    for(const LabelTime &e : t) printf("  %-22s %9.1f ms  %5.1f%%   x%ld\n", e.name.c_str(), e.ms, 100.0 * e.ms / tot, e.n);
    fflush(stdout);
}
