/* qlmx_gemm_bwd.hip -- the input gradient and the weight gradient of one backward flush as ONE kernel launch.
 *
 * moe_backward flushes twice (cudalm.cu:4333-4335 and 4362-4366); each flush holds a weight gradient (mg_atb) and
 * an input gradient (mg_abt_b) that read the same operands and write different outputs. Launched one after the
 * other, each leaves compute units idle while its last round of tiles drains (a third of them at the sizes of a
 * training step), and two streams side by side pay a wait between hardware queues at the fork and at the join.
 * Here the two are one grid: the first workgroups are the tiles of the one, the rest the tiles of the other,
 * each running the code of its own kernel (qlmx_gemm_tn_body.h, qlmx_gemm_nt_body.h), so the second kind's
 * tiles take the compute units as the first kind's leave them. The results are bit-identical to the separate
 * launches: every tile does the same arithmetic in the same order.
 *
 * Use: qlmx_pair_begin(stream); the calls of the flush; qlmx_pair_end(stream). Between the two, the library
 * holds back at most one input-gradient launch and one weight-gradient launch of the kinds named below and
 * qlmx_pair_end issues them together. Everything else keeps its order on the stream: a second launch of a kind
 * already held, and any other library call, first issues what is held. */
#include "qlmx_gemm_tn_body.h"
#include "qlmx_gemm_nt_body.h"
#include <stdlib.h>

#define BWD_LDS_BYTES ((int)(Nt3Shape<128, 4>::LDS_BYTES) > TN3_LDS_BYTES ? (int)(Nt3Shape<128, 4>::LDS_BYTES) : TN3_LDS_BYTES)

/* workgroups [0, first) belong to the one kernel, the rest to the other; `first` is a multiple of 8, so that a
 * workgroup's index within its own kind keeps the XCD the hardware gave it (index % 8) */
template<bool TN_FIRST>
__global__ void __launch_bounds__(256, 2) k_gemm_bwd_pair(Tn3Args ta, Nt3Args na, unsigned first){
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const unsigned b = blockIdx.x;
    if((b < first) == TN_FIRST) tn3_block(ta, TN_FIRST ? b : b - first, lds);
    else                        nt3_block<128, 4>(na, TN_FIRST ? b - first : b);
}

struct PairState {
    bool open; hipStream_t st;
    bool has_tn, has_nt;
    Tn3Args tn; int tn_grid, tn_slot;
    Nt3Args nt; int nt_grid, nt_slot; bool nt_units;
};
static PairState g_pair = {};
static int g_pair_tn_first = -1;

/* launch of a held input gradient alone: the kernel lives in qlmx_gemm_tn_lds.hip, the weight gradient's in
 * qlmx_gemm_nt_lds.hip */
int qlmx_gemm_tn_lds_issue(const Tn3Args &a, int grid, int slot, hipStream_t st);
int qlmx_gemm_nt_lds_issue(const Nt3Args &a, int grid, int slot, bool units, hipStream_t st);

/* issues what is held, in one launch when both kinds are */
int qlmx_pair_flush(void){
    PairState &p = g_pair;
    if(!p.has_tn && !p.has_nt) return QLMX_OK;
    const bool tn = p.has_tn, nt = p.has_nt;
    p.has_tn = p.has_nt = false;
    if(tn && !nt) return qlmx_gemm_tn_lds_issue(p.tn, p.tn_grid, p.tn_slot, p.st);
    if(nt && !tn) return qlmx_gemm_nt_lds_issue(p.nt, p.nt_grid, p.nt_slot, p.nt_units, p.st);
    static bool attr_set = false;
    if(!attr_set){
        QLMX_HIP(hipFuncSetAttribute((const void *)k_gemm_bwd_pair<true>, hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS_BYTES), "backward pair LDS size");
        QLMX_HIP(hipFuncSetAttribute((const void *)k_gemm_bwd_pair<false>, hipFuncAttributeMaxDynamicSharedMemorySize, BWD_LDS_BYTES), "backward pair LDS size");
        attr_set = true;
    }
    if(g_pair_tn_first < 0){ const char *e = getenv("QLMX_PAIR_ORDER"); g_pair_tn_first = (e && e[0] == 'n') ? 0 : 1; }
    if(g_pair_tn_first){
        const unsigned first = ((unsigned)p.tn_grid + 7u) & ~7u;
        hipLaunchKernelGGL(k_gemm_bwd_pair<true>, dim3(first + (unsigned)p.nt_grid), dim3(256), BWD_LDS_BYTES, p.st, p.tn, p.nt, first);
    } else {
        const unsigned first = ((unsigned)p.nt_grid + 7u) & ~7u;
        hipLaunchKernelGGL(k_gemm_bwd_pair<false>, dim3(first + (unsigned)p.tn_grid), dim3(256), BWD_LDS_BYTES, p.st, p.tn, p.nt, first);
    }
    QLMX_LAUNCH_CHECK("backward pair launch");
    int rc = qlmx_upload_done(p.tn_slot, p.st); if(rc) return rc;
    return p.nt_units ? qlmx_unit_done(p.nt_slot, p.st) : qlmx_upload_done(p.nt_slot, p.st);
}

/* The launch functions of the two kernels call these with a launch ready to go: *held = true when it is kept
 * for qlmx_pair_end (the caller returns), false when the caller has to launch it. A launch of a kind already
 * held first issues what is held. */
int qlmx_pair_hold_tn(const Tn3Args &a, int grid, int slot, hipStream_t st, bool *held){
    PairState &p = g_pair;
    *held = false;
    if(!p.open || st != p.st) return QLMX_OK;
    if(p.has_tn){ const int rc = qlmx_pair_flush(); if(rc) return rc; }
    p.tn = a; p.tn_grid = grid; p.tn_slot = slot; p.has_tn = true; *held = true;
    return QLMX_OK;
}
int qlmx_pair_hold_nt(const Nt3Args &a, int grid, int slot, bool units, hipStream_t st, bool *held){
    PairState &p = g_pair;
    *held = false;
    if(!p.open || st != p.st) return QLMX_OK;
    if(p.has_nt){ const int rc = qlmx_pair_flush(); if(rc) return rc; }
    p.nt = a; p.nt_grid = grid; p.nt_slot = slot; p.nt_units = units; p.has_nt = true; *held = true;
    return QLMX_OK;
}

extern "C" int qlmx_pair_begin(void *stream){
    int rc = qlmx_check_ready(); if(rc) return rc;
    QLMX_REQUIRE(!g_pair.open, "qlmx_pair_begin: a pair is already open (one at a time, like every call of the library from one thread)");
    g_pair.open = true; g_pair.st = (hipStream_t)stream; g_pair.has_tn = g_pair.has_nt = false;
    return QLMX_OK;
}
extern "C" int qlmx_pair_end(void *stream){
    QLMX_REQUIRE(g_pair.open, "qlmx_pair_end: no pair is open");
    QLMX_REQUIRE((hipStream_t)stream == g_pair.st, "qlmx_pair_end: not the stream of qlmx_pair_begin");
    const int rc = qlmx_pair_flush();
    g_pair.open = false;
    return rc;
}
