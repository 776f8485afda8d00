/* qlmx_gemm.h -- shared plumbing of the grouped expert GEMMs: the device problem record, the
 * pinned table ring (the counterpart of the reference's mg_h/mg_d ring, cudalm.cu:3220-3241) and
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
    int chunk;              /* scheduled launches: rows per slice of the contraction */
    int flag0;              /*   and the chain flag of the problem's first tile      */
};

/* Writes `nprob` problems into the next slot of a ring in pinned host memory, fills tile0/tiles_n with
 * the given tile shape over an output of rows_of(p) x ncols, and returns the pointer the kernel reads
 * the table through and the total tile count. Slots are guarded by events, so a slot is never
 * rewritten while a kernel launched with it may still read it. */
struct ProbUpload { const DevProb *dev; int ntiles; int nprob; int nfull; };
int qlmx_upload_problems(const qlmx_gemm_prob *probs, int nprob, int mode, int K, int N,
                         int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot);
/* Problems with a second half (same M, K, N). tn: the contraction continues over second[i].A and the
 * weights at second[i].wq / wg. nn: a tile holds columns of both weight matrices; second[i] gives the other
 * matrix (wq, wg), its output (C) and the combined output (B). In the table such a problem has chunk = 1 and
 * is followed by an entry holding the second half's fields that owns no tile. */
int qlmx_upload_problem_pairs(const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int mode, int K, int N,
                              int tile_rows, int tile_cols, hipStream_t stream, ProbUpload *out, int *slot);
/* The same with every problem entered as two: its whole row tiles first (all problems, in the caller's order), then
 * the ragged last row tiles of all problems, tallest first, so that a launch hands out its longest tiles first
 * (nn and tn only: rows are independent there). `rb` says how many bytes a row of each pointer field takes (4 where
 * the field is a list of row indices); out->nfull = tiles of the first part. The kernel maps workgroups to tiles
 * with qx_lpt_tile and the grid is qx_lpt_grid(nfull, ntiles). `second` may be NULL. */
struct RowBytes { size_t a, c, a2, b2, c2; };
int qlmx_upload_problems_split(const qlmx_gemm_prob *first, const qlmx_gemm_prob *second, int nprob, int mode, int K, int N,
                               int tile_rows, int tile_cols, const RowBytes *rb, hipStream_t stream, ProbUpload *out, int *slot);
int qlmx_upload_done(int slot, hipStream_t stream);

/* Locate the problem owning flattened tile t: the last one whose tile0 <= t (tile0 ascending, empty
 * problems share the tile0 of their successor). Every lane reads the tile0 of one problem and the
 * wavefront counts the hits, so the lookup costs one memory round trip per 64 problems; a binary
 * search costs one per level, and at 24 contraction steps per tile those five or six dependent
 * round trips were a fifth of a workgroup's life. Call with all lanes active and t uniform. */
__device__ __forceinline__ int qx_find_problem(const DevProb *pr, int nprob, int t){
    const int lane = threadIdx.x & 63;
    int count = 0;
    for(int base = 0; base < nprob; base += 64){
        const int p = base + lane;
        const int t0 = p < nprob ? pr[p].tile0 : 0x7FFFFFFF;
        count += __popcll(__ballot(t0 <= t));
    }
    return __builtin_amdgcn_readfirstlane(count - 1);
}

/* Tile handled by workgroup b when workgroups go round-robin to 8 XCDs and the grid has been
 * padded to a multiple of 8: XCD x gets the x-th contiguous eighth of the list. The caller drops
 * results >= the real tile count. */
__device__ __forceinline__ int qx_xcd_tile(int b, int grid){
    const int per = grid >> 3;
    return (b & 7) * per + (b >> 3);
}

/* Tile of workgroup b for a table whose first nfull tiles are whole-height ones and whose remaining tiles are the
 * problems' last row tiles, tallest first, g tiles (one tile row) each: XCD x takes the x-th contiguous eighth of the
 * first part (tiles that share an expert's rows and weights meet in one L2), then every eighth tile ROW of the second
 * part -- a row's g tiles read the same activation rows, so they stay on one XCD -- so that all XCDs run out of
 * whole tiles and then of tall last tiles at about the same time. 0x7FFFFFFF = no tile. */
__device__ __forceinline__ int qx_lpt_tile(int b, int nfull, int ntiles, int g){
    const int x = b & 7, k = b >> 3, per = (nfull + 7) >> 3;
    if(k < per){ const int t = x * per + k; return t < nfull ? t : 0x7FFFFFFF; }
    const int k2 = k - per, r = k2 / g;
    const int t = nfull + (r * 8 + x) * g + (k2 - r * g);
    return t < ntiles ? t : 0x7FFFFFFF;
}
static inline int qx_lpt_grid(int nfull, int ntiles, int g){ return 8 * ((nfull + 7) / 8 + g * (((ntiles - nfull) / g + 7) / 8)); }

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

typedef float qx_f32x16 __attribute__((ext_vector_type(16)));
/* round to nearest even, as cudalm.cu:334-338 */
__device__ __forceinline__ unsigned short qx_f32_to_bf16(float f){
    uint32_t x = __float_as_uint(f);
    return (unsigned short)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}
typedef __attribute__((address_space(1))) float qx_gfloat;      /* known to be global memory: loads and stores complete in order */

/* Writes the NI x NJ accumulator tiles (32x32 each, as v_mfma_f32_32x32x16 leaves them) of one
 * wavefront: element e of a lane belongs to row (e/4)*8 + e%4 of the lane's four-row band and to the
 * lane's column. `c` points at the lane's element of tile (0,0) -- row `row` of the output, which has
 * `rows` valid rows and leading dimension ld; tile (i,j) lies 32*i rows and 32*j columns further.
 * The two cases are separate code paths on purpose: the counter that a wait for loaded values uses
 * also counts stores, so one path that may or may not load the old values waits, tile after tile, for
 * all stores of the tile before -- measured, that made the epilogue of a 256x128 tile 45,000 cycles
 * long. Without accumulation nothing waits; with it the old values of tile n+1 are requested before
 * the stores of tile n, so the wait for them leaves those stores in flight. That needs exact counts
 * and straight-line code: a wavefront whose tiles lie wholly inside the output stores without
 * conditions, the others -- the last tile row of a problem -- take the slow path. */
/* SYS: the access goes past both cache levels (system scope), for tiles that several workgroups
 * on different XCDs -- each with an L2 of its own -- add to in turn */
template<bool SYS> __device__ __forceinline__ float qx_gld_f32(const qx_gfloat *p){
    float v;
    if(SYS) asm volatile("global_load_dword %0, %1, off sc0 sc1" : "=v"(v) : "v"(p) : "memory");
    else    asm volatile("global_load_dword %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
template<bool SYS> __device__ __forceinline__ void qx_gst_f32(qx_gfloat *p, float v){
    if(SYS) asm volatile("global_store_dword %0, %1, off sc0 sc1" :: "v"(p), "v"(v) : "memory");
    else    __builtin_nontemporal_store(v, p);
}
/* at most N younger memory operations may still be in flight; names the 16 values it guards */
template<int N> __device__ __forceinline__ void qx_wait_old(float (&o)[16]){
    asm volatile("s_waitcnt vmcnt(%16)"
        : "+v"(o[0]), "+v"(o[1]), "+v"(o[2]), "+v"(o[3]), "+v"(o[4]), "+v"(o[5]), "+v"(o[6]), "+v"(o[7]),
          "+v"(o[8]), "+v"(o[9]), "+v"(o[10]), "+v"(o[11]), "+v"(o[12]), "+v"(o[13]), "+v"(o[14]), "+v"(o[15])
        : "n"(N) : "memory");
}

/* edge path: per-row conditions, the compiler places the waits (every one of them a full drain) */
template<int NI, int NJ, bool SYS>
__device__ __forceinline__ void qx_store_tiles_edge(const qx_f32x16 (&acc)[NI][NJ], qx_gfloat *c, int row, int rows, size_t ld, bool accumulate){
#pragma unroll
    for(int i = 0; i < NI; i++)
#pragma unroll
        for(int j = 0; j < NJ; j++){
            qx_gfloat *col = c + (size_t)(i * 32) * ld + j * 32;
            float old[16];
#pragma unroll
            for(int e = 0; e < 16; e++){
                const int ro = (e >> 2) * 8 + (e & 3);
                old[e] = 0.0f;
                if(accumulate && row + i * 32 + ro < rows)
                    old[e] = SYS ? __hip_atomic_load((float *)(col + (size_t)ro * ld), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM) : col[(size_t)ro * ld];
            }
#pragma unroll
            for(int e = 0; e < 16; e++){
                const int ro = (e >> 2) * 8 + (e & 3);
                if(row + i * 32 + ro < rows){
                    if(SYS) __hip_atomic_store((float *)(col + (size_t)ro * ld), old[e] + acc[i][j][e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    else    col[(size_t)ro * ld] = old[e] + acc[i][j][e];
                }
            }
        }
}
/* wavefront wholly inside the output: no conditions */
template<int NI, int NJ, bool SYS>
__device__ __forceinline__ void qx_store_tiles_full(const qx_f32x16 (&acc)[NI][NJ], qx_gfloat *c, size_t ld, bool accumulate){
    if(!accumulate){
#pragma unroll
        for(int i = 0; i < NI; i++)
#pragma unroll
            for(int j = 0; j < NJ; j++){
                qx_gfloat *col = c + (size_t)(i * 32) * ld + j * 32;
#pragma unroll
                for(int e = 0; e < 16; e++) qx_gst_f32<SYS>(col + (size_t)((e >> 2) * 8 + (e & 3)) * ld, acc[i][j][e]);
            }
        return;
    }
    /* Old values by inline assembly with explicit waits: request tile n+1, wait for tile n while the
     * 16 requests of n+1 and the 16 stores of n-1 (both younger than the requests of n) stay in
     * flight, store n. The compiler itself drains everything at each such point in these kernels. */
    constexpr int NT = NI * NJ;
    float old[2][16];
    auto load_old = [&](int n, float (&o)[16]){
        const qx_gfloat *col = c + (size_t)((n / NJ) * 32) * ld + (n % NJ) * 32;
#pragma unroll
        for(int e = 0; e < 16; e++) o[e] = qx_gld_f32<SYS>(col + (size_t)((e >> 2) * 8 + (e & 3)) * ld);
    };
    load_old(0, old[0]);
#pragma unroll
    for(int n = 0; n < NT; n++){
        if(n + 1 < NT) load_old(n + 1, old[(n + 1) & 1]);
        if(n == 0) qx_wait_old<(NT > 1 ? 16 : 0)>(old[0]);
        else if(n + 1 < NT) qx_wait_old<32>(old[n & 1]);
        else qx_wait_old<16>(old[n & 1]);
        qx_gfloat *col = c + (size_t)((n / NJ) * 32) * ld + (n % NJ) * 32;
#pragma unroll
        for(int e = 0; e < 16; e++) qx_gst_f32<SYS>(col + (size_t)((e >> 2) * 8 + (e & 3)) * ld, old[n & 1][e] + acc[n / NJ][n % NJ][e]);
        __builtin_amdgcn_sched_barrier(0);                                /* the waits count on this order */
    }
}
/* `row` is the lane's first row, `wave_row` the first row of the wavefront's tiles */
template<int NI, int NJ, bool SYS = false>
__device__ __forceinline__ void qx_store_tiles(const qx_f32x16 (&acc)[NI][NJ], float *c, int row, int wave_row, int rows, size_t ld, bool accumulate){
    if(wave_row + NI * 32 <= rows) qx_store_tiles_full<NI, NJ, SYS>(acc, (qx_gfloat *)c, ld, accumulate);
    else                           qx_store_tiles_edge<NI, NJ, SYS>(acc, (qx_gfloat *)c, row, rows, ld, accumulate);
}

/* k_swiglu_bwd (cudalm.cu:2440-2453; cpu_kern.h:385-394) for one element: z, u the forward's gate and up
 * pre-activations, da the gradient of their SwiGLU */
template<bool HW = false>
__device__ __forceinline__ void qx_swiglu_bwd1(float z, float u, float da, float &dg, float &du){
    const float sg = HW ? qx_fsig_hw(z) : qx_fsig(z), silu = z * sg, ds = sg + z * sg * (1.0f - sg);
    dg = da * u * ds; du = da * silu;
}
/* The SwiGLU gradient as the epilogue of the GEMM that produces its input: the NI x 2 accumulator tiles hold
 * da = d(act); gp, up (fp32) are read at the same positions and bf16(dg), bf16(du) written there, so that da
 * itself never reaches memory; the sigmoid is qx_fsig_hw. All four pointers are at the lane's first element (row `row`, its column in
 * tile (., 0)); neighbouring columns are paired into 4-byte stores as in qx_store_swiglu. */
template<int NI>
__device__ __forceinline__ void qx_store_swiglu_bwd(const qx_f32x16 (&acc)[NI][2], const float *gp, const float *up,
                                                    unsigned short *dg, unsigned short *du, int row, int rows, size_t ld){
    typedef const __attribute__((address_space(1))) float gfloat;
    typedef __attribute__((address_space(1))) uint32_t guint;
    const bool oddl = threadIdx.x & 1;
#pragma unroll
    for(int i = 0; i < NI; i++){
        float z[2][16], u[2][16];
#pragma unroll
        for(int e = 0; e < 16; e++){
            const int ro = i * 32 + (e >> 2) * 8 + (e & 3);
            const bool in = row + ro < rows;
#pragma unroll
            for(int j = 0; j < 2; j++){
                const size_t o = (size_t)ro * ld + j * 32;
                z[j][e] = in ? *((gfloat *)gp + o) : 0.0f;
                u[j][e] = in ? *((gfloat *)up + o) : 0.0f;
            }
        }
#pragma unroll
        for(int j = 0; j < 2; j++){
            uint32_t a[16];                                  /* bf16(dg) | bf16(du) << 16 of the lane's 16 rows */
#pragma unroll
            for(int e = 0; e < 16; e++){
                float x, y;
                qx_swiglu_bwd1<true>(z[j][e], u[j][e], acc[i][j][e], x, y);
                a[e] = (uint32_t)qx_f32_to_bf16(x) | ((uint32_t)qx_f32_to_bf16(y) << 16);
            }
            /* the even lane of a pair of columns stores the first eight of its rows for both, the odd lane the rest */
#pragma unroll
            for(int e = 0; e < 8; e++){
                const uint32_t mine = oddl ? a[e + 8] : a[e];
                const uint32_t got = (uint32_t)__shfl_xor((int)(oddl ? a[e] : a[e + 8]), 1, 64);
                const uint32_t lo = oddl ? got : mine, hi = oddl ? mine : got;          /* even column, odd column */
                const int e2 = oddl ? e + 8 : e;
                const int ro = i * 32 + (e2 >> 2) * 8 + (e2 & 3);
                if(row + ro < rows){
                    const size_t o = (size_t)ro * ld + j * 32 - (oddl ? 1 : 0);
                    *(guint *)(dg + o) = (lo & 0xFFFFu) | (hi << 16);
                    *(guint *)(du + o) = (lo >> 16) | (hi & 0xFFFF0000u);
                }
            }
        }
    }
}

/* The NI x 2 accumulator tiles of one wavefront added to INDEXED output rows (the gated scatter and the
 * scatter-add of the MoE glue, cudalm.cu:2541-2545, 2564-2567, as a GEMM epilogue): row r of the problem goes to
 * row idx[r] of `out`, out = out + gate[idx[r]] * y (multiply, then add, as k_scatter_gate does), or out += y when
 * gate is NULL (k_scatter_add4); idx[r] < 0 drops the row. `row` is the lane's first row, `col` its column in
 * tile (., 0); tile (., 1) lies 32 columns further. 32 lanes cover 128 contiguous bytes of an output row.
 * The additions are float atomics without a return value, sent off behind each other: a row index occurs
 * once in a launch's lists, so each element receives exactly one addition and the result is the one rounded
 * sum that a load, an add and a store would give, without the wavefront waiting a memory round trip per row. */
template<int NI>
__device__ __forceinline__ void qx_scatter_tiles(const qx_f32x16 (&acc)[NI][2], const int *idx, const float *gate, float *out,
                                                 int row, int rows, size_t ld, int col){
#pragma unroll
    for(int i = 0; i < NI; i++){
        int tok[16]; float g[16];
#pragma unroll
        for(int e = 0; e < 16; e++){
            const int r = row + i * 32 + (e >> 2) * 8 + (e & 3);
            tok[e] = r < rows ? idx[r] : -1;
        }
#pragma unroll
        for(int e = 0; e < 16; e++) g[e] = (gate && tok[e] >= 0) ? gate[tok[e]] : 1.0f;
#pragma unroll
        for(int e = 0; e < 16; e++)
            if(tok[e] >= 0){
                qx_gfloat *o = (qx_gfloat *)(out + (size_t)tok[e] * ld + col);
                const float y0 = gate ? g[e] * acc[i][0][e] : acc[i][0][e], y1 = gate ? g[e] * acc[i][1][e] : acc[i][1][e];
                (void)__builtin_amdgcn_global_atomic_fadd_f32(o, y0);
                (void)__builtin_amdgcn_global_atomic_fadd_f32(o + 32, y1);
            }
    }
}

/* ---- scheduled launches: instead of deriving its tile from its index, a workgroup reads an entry of
 * a table the host has laid out -- which problem, which row of output tiles, which slice of the
 * contraction; the workgroups that share an entry take one column tile each, which keeps the table
 * to a few hundred bytes. Slices of one output tile form a chain: slice seq waits until flag holds
 * (epoch << 4 | seq), adds its product to what is there and publishes seq + 1. A slice always sits at
 * a higher workgroup index than its predecessor, and workgroups start in index order, so whatever a
 * resident workgroup waits for is resident or done; the wait is bounded all the same. ---- */
typedef uint32_t DevUnit;                 /* prob:10 | tile row:6 | (8 spare) | seq:4 | nseq:4; all ones = nothing to do */
#define QX_UNIT_NONE 0xFFFFFFFFu
#define QX_UNIT(prob, ti, tj, seq, nseq) ((uint32_t)(prob) << 22 | (uint32_t)(ti) << 16 | (uint32_t)(tj) << 8 | (uint32_t)(seq) << 4 | (uint32_t)(nseq))
#define QLMX_MAX_UNITS 16384
#define QX_CHAIN_SPINS (1 << 22)
struct UnitUpload { DevProb *hprob; DevUnit *hunit; const DevProb *dprob; const DevUnit *dunit; int *flags; unsigned *status; };
int qlmx_unit_slot(int nprob, UnitUpload *out, int *slot);                         /* tables to fill (host staging) and where the kernel will read them; waits for the slot's last user */
void qlmx_unit_commit(const UnitUpload *u, int nprob, int nunits);                 /* staging copy -> the slot the kernel reads; before the launch */
int qlmx_unit_done(int slot, hipStream_t stream);                                  /* after the kernel launch */
int qlmx_chain_reserve(int nflags, int *first, unsigned *epoch);                   /* flags for one launch */
/* one-shot switches of the time-out tests (qlmx_test_force_wait_timeout): true once after being armed */
bool qlmx_test_take_forced_timeout(int which);

/* chain hand-over; every thread of the workgroup calls both */
/* `limit` polls at most (QX_CHAIN_SPINS in production; the time-out test passes 1 together with an epoch
 * nobody publishes, so that every wait gives up at once and the kernel still runs to its end) */
__device__ __forceinline__ void qx_chain_wait(int *flags, int flag, unsigned epoch, int seq, unsigned *status, int limit){
    if(threadIdx.x == 0){
        const int want = (int)((epoch << 4) | (unsigned)seq);
        int spins = 0;
        while(__hip_atomic_load(flags + flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != want && ++spins < limit) __builtin_amdgcn_s_sleep(16);
        if(spins >= limit) __hip_atomic_store(status, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    __syncthreads();
}
__device__ __forceinline__ void qx_chain_publish(int *flags, int flag, unsigned epoch, int seq){
    __builtin_amdgcn_s_waitcnt(0x0F70);                 /* vmcnt(0): this wavefront's system-scope stores are out */
    __syncthreads();
    if(threadIdx.x == 0) __hip_atomic_store(flags + flag, (int)((epoch << 4) | (unsigned)(seq + 1)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__device__ __forceinline__ float qx_bf16_to_f32(unsigned short h){ return __uint_as_float((uint32_t)h << 16); }

/* gate, up (fp32; both skipped when gp is NULL) and bf16(gate * sigmoid(gate) * up) of a gate|up tile (HW: the
 * sigmoid is qx_fsig_hw instead of the SwiGLU kernel's qx_fsig). The tile's 128 LDS columns are
 * [gate 0-31 | up 0-31 | gate 32-63 | up 32-63] of the problem's columns j0 .. j0+63, so a wavefront's first
 * accumulator column holds gate and its second holds up of the same 32 columns, element for element. */
template<int NI, bool HW = false>
__device__ __forceinline__ void qx_store_swiglu(const qx_f32x16 (&acc)[NI][2], float *gp, float *up, unsigned short *act,
                                                 int row, int rows, size_t ld){
    typedef __attribute__((address_space(1))) float gfloat;
    typedef __attribute__((address_space(1))) uint32_t guint;
    const bool oddl = threadIdx.x & 1;
#pragma unroll
    for(int i = 0; i < NI; i++){
        uint32_t a[16];
#pragma unroll
        for(int e = 0; e < 16; e++){
            const int ro = i * 32 + (e >> 2) * 8 + (e & 3);
            const float g = acc[i][0][e], u = acc[i][1][e];
            a[e] = qx_f32_to_bf16(g * (HW ? qx_fsig_hw(g) : qx_fsig(g)) * u);
            if(gp && row + ro < rows){
                const size_t o = (size_t)ro * ld;
                __builtin_nontemporal_store(g, (gfloat *)gp + o);
                __builtin_nontemporal_store(u, (gfloat *)up + o);
            }
        }
        /* two neighbouring columns per 4-byte store: the even lane of a pair writes the first eight of its
         * rows for both, the odd lane the other eight */
#pragma unroll
        for(int e = 0; e < 8; e++){
            const uint32_t got = (uint32_t)__shfl_xor((int)(oddl ? a[e] : a[e + 8]), 1, 64);
            const int e2 = oddl ? e + 8 : e;
            const int ro = i * 32 + (e2 >> 2) * 8 + (e2 & 3);
            const uint32_t v = oddl ? (got | (a[e + 8] << 16)) : (a[e] | (got << 16));
            if(row + ro < rows) *(guint *)(act + (size_t)ro * ld - (oddl ? 1 : 0)) = v;
        }
    }
}


#endif
