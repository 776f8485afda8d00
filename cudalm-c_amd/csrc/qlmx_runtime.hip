/* qlmx_runtime.hip -- device selection, memory helpers, error text and the host-side integer
 * helpers of the C ABI. Mirrors what cudalm.cu does through cudaSetDevice / dmalloc / cudaMemcpy /
 * cudaMemset / cudaDeviceSynchronize (cudalm.cu:147-154, 6628). There is no CPU fallback: without
 * a gfx950 device every compute entry point fails with QLMX_E_NODEV. */
#include "qlmx_dev.h"
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

static thread_local char g_err[512] = "";
static int  g_ready = 0;
static char g_devname[256] = "";

void qlmx_set_error(const char *fmt, ...){
    va_list ap; va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
}
int qlmx_check_ready_keep(void){
    if(g_ready) return QLMX_OK;
    qlmx_set_error("libqlmx: qlmx_init() has not succeeded (no gfx950 device bound)");
    return QLMX_E_NODEV;
}
/* Every entry point that queues work starts here. Launches held back for a pair (qlmx_pair_begin) are issued
 * first, so that whatever this call queues comes after them on the stream; the two kinds of call that can be
 * held themselves use qlmx_check_ready_keep. */
int qlmx_pair_flush(void);
int qlmx_check_ready(void){
    const int rc = qlmx_check_ready_keep(); if(rc) return rc;
    return qlmx_pair_flush();
}

static int g_cus = 256;
int qlmx_cu_count(void){ return g_cus; }                   /* compute units of the initialised device */

extern "C" int qlmx_version(void){ return QLMX_VERSION; }
extern "C" const char *qlmx_last_error(void){ return g_err; }
extern "C" const char *qlmx_device_name(void){ return g_devname; }

extern "C" int qlmx_init(int device){
    int n = 0;
    hipError_t e = hipGetDeviceCount(&n);
    if(e != hipSuccess || n <= 0){
        qlmx_set_error("qlmx_init: no HIP device (%s)", e != hipSuccess ? hipGetErrorString(e) : "count 0");
        return QLMX_E_NODEV;
    }
    QLMX_REQUIRE(device >= 0 && device < n, "qlmx_init: device %d of %d", device, n);
    QLMX_HIP(hipSetDevice(device), "hipSetDevice");
    hipDeviceProp_t pr;
    QLMX_HIP(hipGetDeviceProperties(&pr, device), "hipGetDeviceProperties");
    snprintf(g_devname, sizeof g_devname, "%s (%s, %d CUs)", pr.name, pr.gcnArchName, pr.multiProcessorCount);
    g_cus = pr.multiProcessorCount;
    if(strncmp(pr.gcnArchName, "gfx950", 6) != 0){
        qlmx_set_error("qlmx_init: device is %s; this library carries gfx950 code only", pr.gcnArchName);
        return QLMX_E_NODEV;
    }
    int rc = qlmx_decode_setup(device); if(rc) return rc;
    g_ready = 1;
    return QLMX_OK;
}

extern "C" int qlmx_malloc(void **p, size_t bytes){
    QLMX_REQUIRE(p, "qlmx_malloc: NULL out pointer");
    QLMX_HIP(hipMalloc(p, bytes ? bytes : 1), "hipMalloc");
    return QLMX_OK;
}
extern "C" int qlmx_free(void *p){ QLMX_HIP(hipFree(p), "hipFree"); return QLMX_OK; }
/* copies, fills and waits come after what an open pair holds, like every call that queues work */
extern "C" int qlmx_memcpy_h2d(void *dst, const void *src, size_t bytes){
    int rc = qlmx_pair_flush(); if(rc) return rc;
    QLMX_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice), "hipMemcpy h2d"); return QLMX_OK; }
extern "C" int qlmx_memcpy_d2h(void *dst, const void *src, size_t bytes){
    int rc = qlmx_pair_flush(); if(rc) return rc;
    QLMX_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost), "hipMemcpy d2h"); return QLMX_OK; }
extern "C" int qlmx_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream){
    int rc = qlmx_pair_flush(); if(rc) return rc;
    QLMX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream), "hipMemcpy d2d"); return QLMX_OK; }
extern "C" int qlmx_memset(void *dst, int value, size_t bytes, void *stream){
    int rc = qlmx_pair_flush(); if(rc) return rc;
    QLMX_HIP(hipMemsetAsync(dst, value, bytes, (hipStream_t)stream), "hipMemset"); return QLMX_OK; }
extern "C" int qlmx_sync(void *stream){
    int rc = qlmx_pair_flush(); if(rc) return rc;
    if(stream) QLMX_HIP(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    else       QLMX_HIP(hipDeviceSynchronize(), "hipDeviceSynchronize");
    return QLMX_OK;
}

/* ---- a second stream beside the caller's, for launches that do not depend on each other ----
 * One side stream and two events per device, made at the first fork (default priority, like every stream here).
 * fork: the side stream waits for what `stream` holds so far; join: `stream` waits for what the side stream
 * holds. Both are waits between queues on the device; the host does not block. */
#define SIDE_MAX_DEVICES 16
struct SideState { hipStream_t st = nullptr; hipEvent_t fork = nullptr, join = nullptr; };
static SideState g_side[SIDE_MAX_DEVICES];
static int side_of(SideState **out){
    int rc = qlmx_check_ready(); if(rc) return rc;
    int device = -1;
    QLMX_HIP(hipGetDevice(&device), "side stream device");
    QLMX_REQUIRE(device >= 0 && device < SIDE_MAX_DEVICES, "side stream: device %d is beyond the %d this library keeps state for", device, SIDE_MAX_DEVICES);
    SideState &sd = g_side[device];
    if(!sd.st){
        QLMX_HIP(hipStreamCreateWithFlags(&sd.st, hipStreamNonBlocking), "side stream");
        QLMX_HIP(hipEventCreateWithFlags(&sd.fork, hipEventDisableTiming), "side stream event");
        QLMX_HIP(hipEventCreateWithFlags(&sd.join, hipEventDisableTiming), "side stream event");
    }
    *out = &sd;
    return QLMX_OK;
}
extern "C" int qlmx_side_fork(void *stream, void **side){
    QLMX_REQUIRE(side, "qlmx_side_fork: NULL out pointer");
    SideState *sd; int rc = side_of(&sd); if(rc) return rc;
    QLMX_HIP(hipEventRecord(sd->fork, (hipStream_t)stream), "side fork record");
    QLMX_HIP(hipStreamWaitEvent(sd->st, sd->fork, 0), "side fork wait");
    *side = (void *)sd->st;
    return QLMX_OK;
}
extern "C" int qlmx_side_join(void *stream){
    SideState *sd; int rc = side_of(&sd); if(rc) return rc;
    QLMX_HIP(hipEventRecord(sd->join, sd->st), "side join record");
    QLMX_HIP(hipStreamWaitEvent((hipStream_t)stream, sd->join, 0), "side join wait");
    return QLMX_OK;
}

/* ---- host integer helpers (qlm.cuh:78-111) ---- */
extern "C" unsigned int qlmx_qhashu(unsigned long long x){ return qx_hash(x); }
extern "C" int qlmx_qsri(float v, unsigned long long i, unsigned long long t){
    return qx_sround(v, i * QLMX_KI + t * QLMX_KT);
}
extern "C" int qlmx_qclmp(int v, int lo, int hi){ return qx_clamp(v, lo, hi); }
extern "C" int qlmx_qd_get(const signed char *d, unsigned long long i, int packed){
    if(!packed) return (int)d[i];
    const unsigned b = (unsigned char)d[i >> 1];
    const int v = (i & 1ULL) ? (int)(b >> 4) : (int)(b & 15u);
    return v >= 8 ? v - 16 : v;
}
extern "C" void qlmx_qd_set_host(signed char *d, unsigned long long i, int v, int packed){
    if(!packed){ d[i] = (signed char)v; return; }
    unsigned char *b = (unsigned char *)&d[i >> 1];
    const unsigned nib = (unsigned)v & 15u;
    *b = (unsigned char)((i & 1ULL) ? ((*b & 0x0Fu) | (nib << 4)) : ((*b & 0xF0u) | nib));
}
extern "C" unsigned long long qlmx_qd_bytes(unsigned long long nq, int packed){ return packed ? (nq + 1) / 2 : nq; }

/* ---- label timing without synchronisation (prof_ev / prof_flush / prof_report, cudalm.cu:806-840) ----
 * qlmx_prof_mark(label, stream) records an event on `stream`; a label is charged the GPU time between the mark
 * before it and its own, so marks are placed BEHIND the work they name, as the reference places kchk(). `drained`
 * counts the marks that found the previous mark's event already complete: the GPU had run out of queued work and
 * the host was the bottleneck at that point. Events live in a ring that is drained (one wait for the newest event)
 * when it is full and by the report. Host-side state only; the marks are ordinary event records. */
#define PROF_LABELS 48
#define PROF_EVENTS 1024
struct ProfLabel { char name[40]; double ms; long n, drained; };
static ProfLabel g_pl[PROF_LABELS];
static int g_pl_n = 0;
static hipEvent_t g_pe[PROF_EVENTS];
static short g_pe_label[PROF_EVENTS];
static int g_pe_n = 0;
static bool g_pe_made = false;
static int prof_label(const char *what){
    for(int i = 0; i < g_pl_n; i++) if(!strncmp(g_pl[i].name, what, sizeof g_pl[i].name - 1)) return i;
    if(g_pl_n == PROF_LABELS) return PROF_LABELS - 1;                     /* the table is full: the last entry takes the rest */
    memset(&g_pl[g_pl_n], 0, sizeof g_pl[0]);
    snprintf(g_pl[g_pl_n].name, sizeof g_pl[0].name, "%s", what);
    return g_pl_n++;
}
static int prof_drain(void){
    if(g_pe_n < 2) return QLMX_OK;
    QLMX_HIP(hipEventSynchronize(g_pe[g_pe_n - 1]), "label timing: wait for the newest mark");
    for(int i = 1; i < g_pe_n; i++){
        float ms = 0.0f;
        QLMX_HIP(hipEventElapsedTime(&ms, g_pe[i - 1], g_pe[i]), "label timing: elapsed time");
        g_pl[g_pe_label[i]].ms += ms; g_pl[g_pe_label[i]].n++;
    }
    const hipEvent_t last = g_pe[g_pe_n - 1];                             /* the newest mark starts the next interval */
    g_pe[g_pe_n - 1] = g_pe[0]; g_pe[0] = last; g_pe_n = 1;
    return QLMX_OK;
}
extern "C" int qlmx_prof_mark(const char *label, void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(label && label[0], "qlmx_prof_mark: empty label");
    if(!g_pe_made){
        for(int i = 0; i < PROF_EVENTS; i++) QLMX_HIP(hipEventCreate(&g_pe[i]), "label timing: event");
        g_pe_made = true;
    }
    const int k = prof_label(label);
    if(g_pe_n > 0 && hipEventQuery(g_pe[g_pe_n - 1]) == hipSuccess) g_pl[k].drained++;
    (void)hipGetLastError();                                              /* hipErrorNotReady from the query is not an error */
    QLMX_HIP(hipEventRecord(g_pe[g_pe_n], (hipStream_t)stream), "label timing: record");
    g_pe_label[g_pe_n++] = (short)k;
    return g_pe_n == PROF_EVENTS ? prof_drain() : QLMX_OK;
}
/* Writes the table, largest total first, one line per label: name, ms, share, count, drained (the format of
 * prof_report, cudalm.cu:826-840), and returns the number of labels through *nlabels (may be NULL). The text is
 * cut at cap - 1 characters. */
extern "C" int qlmx_prof_report(char *out, size_t cap, int *nlabels){
    int rc = prof_drain(); if(rc) return rc;
    QLMX_REQUIRE(out && cap > 0, "qlmx_prof_report: no buffer");
    int order[PROF_LABELS];
    double tot = 0.0;
    for(int i = 0; i < g_pl_n; i++){ order[i] = i; tot += g_pl[i].ms; }
    for(int i = 0; i < g_pl_n; i++) for(int j = i + 1; j < g_pl_n; j++) if(g_pl[order[j]].ms > g_pl[order[i]].ms){ const int t = order[i]; order[i] = order[j]; order[j] = t; }
    size_t at = 0;
    out[0] = 0;
    auto put = [&](const char *fmt, auto... v){ if(at + 1 < cap){ const int w = snprintf(out + at, cap - at, fmt, v...); if(w > 0) at = at + (size_t)w < cap ? at + (size_t)w : cap - 1; } };
    put("[prof] per-label totals (%.3f ms tracked, GPU time between marks)\n", tot);
    for(int i = 0; i < g_pl_n; i++){
        const ProfLabel &e = g_pl[order[i]];
        put("  %-22s %9.3f ms  %5.1f%%   x%ld   drained %ld\n", e.name, e.ms, tot > 0.0 ? 100.0 * e.ms / tot : 0.0, e.n, e.drained);
    }
    if(nlabels) *nlabels = g_pl_n;
    return QLMX_OK;
}
extern "C" int qlmx_prof_reset(void){
    int rc = prof_drain(); if(rc) return rc;
    g_pl_n = 0; g_pe_n = 0;
    return QLMX_OK;
}
