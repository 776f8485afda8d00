/* qlmx_gemm.h -- shared plumbing of the grouped expert GEMMs: the device problem record, the
 * pinned upload ring (the counterpart of the reference's mg_h/mg_d ring, cudalm.cu:3220-3241) and
 * the weight-tile readers. */
#ifndef QLMX_GEMM_H
#define QLMX_GEMM_H
#include "qlmx_dev.h"

enum { GEMM_NN = 0, GEMM_TN = 1, GEMM_NT = 2 };

struct DevProb {
    const void *A; const void *B; float *C;
    unsigned long long wq, wg;
    int M; float beta;
    int tile0;              /* first tile of this problem in the flattened tile list */
    int tiles_n;            /* tiles along the output's second dimension             */
};

/* Copies `nprob` problems into the next ring slot, fills tile0/tiles_n with the given tile shape
 * over an output of rows_of(p) x ncols, uploads the slot asynchronously on `stream`, and returns
 * the device pointer and the total tile count. Slots are guarded by events, so a slot is never
 * rewritten while a kernel launched with it may still read it. */
struct ProbUpload { const DevProb *dev; int ntiles; int nprob; };
int qlmx_upload_problems(const qlmx_gemm_prob *probs, int nprob, int mode, int K, int N,
                         int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot);
int qlmx_upload_done(int slot, hipStream_t stream);

/* locate the problem owning flattened tile t (tile0 ascending) */
__device__ __forceinline__ int qx_find_problem(const DevProb *pr, int nprob, int t){
    int lo = 0, hi = nprob - 1;
    while(lo < hi){
        int mid = (lo + hi + 1) >> 1;
        if(pr[mid].tile0 <= t) lo = mid; else hi = mid - 1;
    }
    return lo;
}

/* Tile handled by workgroup b when workgroups go round-robin to 8 XCDs and the grid has been
 * padded to a multiple of 8: XCD x gets the x-th contiguous eighth of the list. The caller drops
 * results >= the real tile count. */
__device__ __forceinline__ int qx_xcd_tile(int b, int grid){
    const int per = grid >> 3;
    return (b & 7) * per + (b >> 3);
}

/* Weight gradients (tile cost = the expert's row count): every problem owns rp rows of g tiles; a
 * row shares the A-side slab (activations), a column the B-side slab (output gradients).
 * qx_xcd_tile_probs: problem p goes to XCD p % 8 whole, so both operands come from HBM once and
 * from that XCD's L2 afterwards (the host orders the table so that the XCDs get equal work).
 * grid = 8 * g * rp * ceil(nprob / 8); a result >= nprob*rp*g is no tile.
 * qx_xcd_tile_rows: tile rows are dealt round-robin; when rp is a multiple of 8 XCD x always gets
 * row block x of every expert, the wide A side is still read once, only the narrow B side is read by
 * all eight, and the XCDs are balanced whatever the row counts are. Measured at K=2048 N=768
 * (rp=8) this order is 15% faster than whole problems per XCD in spite of 2.6x its HBM reads; at
 * K=768 N=2048 (rp=3) both take the same time and whole problems read half as much. */
__device__ __forceinline__ int qx_xcd_tile_probs(int b, int g, int rp){
    const int x = b & 7, k = b >> 3;
    const int lr = k / g, c = k - lr * g, ps = lr / rp, r = lr - ps * rp;
    return ((ps * 8 + x) * rp + r) * g + c;
}
__device__ __forceinline__ int qx_xcd_tile_rows(int b, int g){
    const int x = b & 7, k = b >> 3;
    return (x + 8 * (k / g)) * g + k % g;
}

__device__ __forceinline__ float qx_bf16_to_f32(unsigned short h){ return __uint_as_float((uint32_t)h << 16); }
/* round to nearest even, as cudalm.cu:334-338 */
__device__ __forceinline__ unsigned short qx_f32_to_bf16(float f){
    uint32_t x = __float_as_uint(f);
    return (unsigned short)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}

#endif
