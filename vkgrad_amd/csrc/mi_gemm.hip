// C ABI of libmigemm.so: context, buffers, GEMM dispatch, timing, record/replay.
// Declarations and the reference interfaces they replace are in include/mi_gemm.h.
#include <hip/hip_runtime.h>

#include <algorithm>

#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>

#include "gemm_kernel.h"
#include "gemv_kernel.h"
#include "skinny_kernel.h"
#include "mi_gemm.h"
#include "tiles.h"

namespace mg {
extern launch_fn launch_table_nn_f16[MG_NUM_TILES][3];
extern launch_fn launch_table_nn_bf16[MG_NUM_TILES][3];
extern launch_fn launch_table_nt_f16[MG_NUM_TILES][3];
extern launch_fn launch_table_nt_bf16[MG_NUM_TILES][3];
extern launch_fn launch_table_tn_f16[MG_NUM_TILES][3];
extern launch_fn launch_table_tn_bf16[MG_NUM_TILES][3];

// ---------------------------------------------------------------------------
// Pre-pass for split-K with beta == 0: C = 0 (a fill kernel, so the sequence can
// be captured in a graph).
// ---------------------------------------------------------------------------
// Rows are walked with a grid stride; a thread clears four consecutive columns,
// as one 16-byte store when `vec` says every such group is aligned.
__global__ void zero_c_kernel(float *C, int64_t ldc, int M, int N, int64_t sc, int vec) {
    float *Cz = C + (int64_t)blockIdx.z * sc;
    const int col = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (col >= N) return;
    for (int row = blockIdx.y; row < M; row += gridDim.y) {
        float *q = Cz + (int64_t)row * ldc + col;
        if (vec && col + 3 < N) {
            *reinterpret_cast<float4 *>(q) = make_float4(0.f, 0.f, 0.f, 0.f);
        } else {
            for (int e = 0; e < 4 && col + e < N; e++) q[e] = 0.f;
        }
    }
}

// Arrival counters back to zero (a fill kernel, so that the sequence may be captured into a graph).
__global__ void zero_ints_kernel(int *p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

struct TileDesc {
    int id, bm, bn, bk, wgm, wgn;
    int nstage;     // 0: register-staged kernel; >0: direct-to-LDS ring depth
    int fallback;   // tile of the same BM x BN with weaker preconditions (self: none)
    int persistent; // 1: grid of resident workgroups looping over tiles; 2: the same with stream-K balancing
    int gemv;       // 1: the skinny-M streaming kernel (no matrix cores), 2: the one on the matrix cores; NT layout only
    int pingpong;   // 1: the two wavefronts of a SIMD alternate between LDS reads and MFMAs (gemm_pp_kernel.h)
};
#define V(id, bm, bn, bk, wgm, wgn) {id, bm, bn, bk, wgm, wgn, 0, id, 0, 0, 0},
#define D(id, bm, bn, bk, wgm, wgn, ns, fb) {id, bm, bn, bk, wgm, wgn, ns, fb, 0, 0, 0},
#define P(id, bm, bn, bk, wgm, wgn, ns, fb) {id, bm, bn, bk, wgm, wgn, ns, fb, 1, 0, 0},
#define S(id, bm, bn, bk, wgm, wgn, ns, fb) {id, bm, bn, bk, wgm, wgn, ns, fb, 2, 0, 0},
#define G(id, bm, bn, bk, fb) {id, bm, bn, bk, 1, GEMV_WAVES, 0, fb, 0, 1, 0},
#define Q(id, bm, bn, bk, wgm, wgn, ns, fb) {id, bm, bn, bk, wgm, wgn, ns, fb, 0, 0, 1},
#define W(id, bm, bn, bk, fb) {id, bm, bn, bk, 1, 4, 0, fb, 0, 2, 0},
static const TileDesc g_tiles[MG_NUM_TILES] = {MG_TILE_LIST(V, D, P, S, G, Q, W)};
#undef V
#undef D
#undef P
#undef S
#undef G
#undef Q
#undef W

static thread_local char g_err[512] = "";

static int fail(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

static int hip_fail(hipError_t e, const char *what) {
    return fail(MG_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(expr)                                  \
    do {                                               \
        hipError_t e_ = (expr);                        \
        if (e_ != hipSuccess) return hip_fail(e_, #expr); \
    } while (0)

static launch_fn (*table_for(int layout, int dtype))[3] {
    switch (layout * 2 + dtype) {
        case 0: return launch_table_nn_f16;
        case 1: return launch_table_nn_bf16;
        case 2: return launch_table_nt_f16;
        case 3: return launch_table_nt_bf16;
        case 4: return launch_table_tn_f16;
        default: return launch_table_tn_bf16;
    }
}

static int lds_bytes_for(const TileDesc &t, int layout) {
    if (t.gemv == 2) return skinny_lds_bytes(1, skinny_waves(1), SKINNY_KP, 768);   // for K = 768; grows with K
    if (t.gemv) return 0;
    if (t.nstage > 0) return t.nstage * (t.bm + t.bn) * t.bk * 2;
    const bool a_kc = layout != MG_TN, b_kc = layout == MG_NT;
    const int a = a_kc ? t.bm * (t.bk + 8) : t.bk * (t.bm + 32);
    const int b = b_kc ? t.bn * (t.bk + 8) : t.bk * (t.bn + 32);
    return 2 * (a + b) * 2;
}

// The aligned instantiation may be used when every 16-byte chunk the loader
// forms is 16-byte aligned and lies entirely inside or outside the matrix.
static bool operands_aligned(const mg_gemm_args &a) {
    const bool a_kc = a.layout != MG_TN, b_kc = a.layout == MG_NT;
    if (((uintptr_t)a.a | (uintptr_t)a.b) & 15) return false;
    if ((a.lda | a.ldb) & 7) return false;
    if (a.nbatch > 1 && ((a.sa | a.sb) & 7)) return false;
    if ((a_kc || b_kc) && (a.k & 7)) return false;
    if (!a_kc && (a.m & 7)) return false;
    if (!b_kc && (a.n & 7)) return false;
    return true;
}

static inline int64_t cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }

struct Plan {
    int tile, split_k, group_m, k_per_split, grid_m, grid_n, xcd_remap;
};

// Preconditions of the direct-to-LDS kernels (gemm_dma_kernel.h): aligned bases
// and pitches, K slices that are multiples of BK (the last may be ragged), and
// row pitches that cover the 16-byte chunk straddling a ragged edge.
// The skinny-M kernel holds MP >= M rows of A (1, 2, 4 or 8) over K <= 512, 768, 1024 or
// 2048 elements in registers and reads 16-byte pieces of both operands.
static bool gemv_shape(const mg_gemm_args &a, int *mp_log2, int *k_class) {
    if (a.m > 8 || a.k > 2048) return false;
    int lm = 0;
    while ((1 << lm) < a.m) lm++;
    if (mp_log2) *mp_log2 = lm;
    if (k_class) *k_class = gemv_k_class((int)a.k);
    return true;
}
static bool gemv_eligible(const mg_gemm_args &a, int split) {
    if (a.layout != MG_NT || split > 1) return false;
    if (!gemv_shape(a, nullptr, nullptr)) return false;
    if (((uintptr_t)a.a | (uintptr_t)a.b) & 15) return false;
    if ((a.lda | a.ldb | a.k) & 7) return false;
    if (a.nbatch > 1 && ((a.sa | a.sb) & 7)) return false;
    if (a.res && a.res != a.c) return false;   // its beta = 1 reads C
    if (a.tri) return false;
    return true;
}

// The skinny-M kernel on the matrix cores: one or two blocks of 32 rows of A, held in LDS over
// all of K beside the wavefronts' phase buffers of B; 16-byte pieces of both operands.
static int skinny_blocks(const mg_gemm_args &a) { return (int)((a.m + 31) / 32); }
static bool skinny_eligible(const mg_gemm_args &a, int split) {
    if (a.layout != MG_NT || split > 1 || a.nbatch != 1) return false;
    if (a.m > 32 * SKINNY_MAX_TMB || a.k > 8192) return false;
    const int tmb = skinny_blocks(a);
    if (skinny_lds_bytes(tmb, skinny_waves(tmb), SKINNY_KP, (int)a.k) > SKINNY_LDS_LIMIT) return false;
    if (((uintptr_t)a.a | (uintptr_t)a.b) & 15) return false;
    if ((a.lda | a.ldb | a.k) & 7) return false;
    if (a.res && a.res != a.c) return false;   // its beta = 1 reads C
    if (a.tri || a.y16) return false;
    return true;
}

static bool dma_eligible(const mg_gemm_args &a, const TileDesc &t, int64_t k_per_split, int split) {
    if (t.gemv == 2) return skinny_eligible(a, split);
    if (t.gemv) return gemv_eligible(a, split);
    if (t.nstage == 0) return true;
    const bool a_kc = a.layout != MG_TN, b_kc = a.layout == MG_NT;
    if (((uintptr_t)a.a | (uintptr_t)a.b) & 15) return false;
    if ((a.lda | a.ldb) & 7) return false;
    if (a.nbatch > 1 && ((a.sa | a.sb) & 7)) return false;
    if (split > 1 && k_per_split % t.bk != 0) return false;
    const int64_t k8 = (a.k + 7) & ~(int64_t)7, m8 = (a.m + 7) & ~(int64_t)7, n8 = (a.n + 7) & ~(int64_t)7;
    if (a_kc ? a.lda < k8 : (a.lda < m8 || a.m < 8)) return false;
    if (b_kc ? a.ldb < k8 : (a.ldb < n8 || a.n < 8)) return false;
    // A chunk that straddles a ragged edge reads row padding; on the last row that is
    // beyond the matrix, so the caller must own it (MG_FLAG_TIGHT_BUFFERS says it does not).
    const bool ragged = (a_kc ? (a.k & 7) : (a.m & 7)) || (b_kc ? (a.k & 7) : (a.n & 7));
    if (ragged && (a.flags & MG_FLAG_TIGHT_BUFFERS)) return false;
    if (t.pingpong) {
        // its loads address a lane as scalar base + 32-bit offset of up to 7 rows (K-contiguous
        // operand, 8 rows of 128 bytes per instruction) or 1 row (M/N-contiguous, 2 rows of 512)
        const int64_t lim = (int64_t)1 << 32;
        if ((a_kc ? 7 * a.lda * 2 + 128 : a.lda * 2 + 512) >= lim) return false;
        if ((b_kc ? 7 * a.ldb * 2 + 128 : a.ldb * 2 + 512) >= lim) return false;
    }
    if (t.persistent) {
        if (a.k % t.bk != 0 || k_per_split % t.bk != 0) return false;
        if (a.res && a.res != a.c) return false;   // their beta = 1 is an atomic add into C
        if (a.tri) return false;                   // the unit loop knows nothing of skipped tiles or K ranges
    }
    if (t.persistent == 2 && split > 1) return false;   // stream-K cuts K itself
    // the 256 x 256 stream-K kernel with the bias epilogue does not fit the register file, nor does
    // the persistent 256 x 256 x 64 one in the NN layout (neither is instantiated)
    if (t.persistent == 2 && a.bias && t.bm * t.bn > 128 * 128) return false;
    if (t.persistent && a.bias && t.bm * t.bn > 128 * 128 && t.bk >= 64 && a.layout == MG_NN) return false;
    return true;
}

// Cost table of the picker, fitted to timings of every (tile, split) candidate over 54
// shapes on MI355X (benchmark shapes, squares, skinny and deep-K cases, random bf16
// operands): time = 1.5 us + rounds * (overhead + K-blocks * block_time * occupancy).
// {per-workgroup overhead in us, time per K-block in us} by tile and layout NN, NT, TN.
// It only has to rank candidates; the tuner measures.
static const float g_cost[MG_NUM_TILES][3][2] = {
    {{6.63f, 0.906f}, {12.84f, 0.822f}, {5.81f, 0.848f}},   // 0 mm_256x256x32_w2x4 (half the fitted block time of its 64-wide form)
    {{5.29f, 1.046f}, {12.32f, 0.779f}, {3.73f, 1.029f}},   // 1 mm_256x128x64_w2x2
    {{5.21f, 0.991f}, {11.72f, 0.771f}, {3.63f, 1.042f}},   // 2 mm_128x256x64_w2x2
    {{4.60f, 1.014f}, {7.81f, 0.781f}, {2.82f, 0.975f}},   // 3 mm_128x128x64_w2x2
    {{1.59f, 0.581f}, {1.33f, 0.713f}, {1.76f, 0.581f}},   // 4 mm_64x64x64_w2x2
    {{4.46f, 0.640f}, {7.40f, 0.590f}, {3.02f, 0.675f}},   // 5 mm_64x256x64_w1x4
    {{2.79f, 0.531f}, {4.80f, 0.475f}, {2.92f, 0.534f}},   // 6 mm_32x256x64_w1x4
    {{4.55f, 0.654f}, {4.58f, 0.660f}, {3.04f, 0.671f}},   // 7 mm_256x64x64_w4x1
    {{2.88f, 0.565f}, {3.07f, 0.564f}, {2.65f, 0.574f}},   // 8 mm_256x32x64_w4x1
    {{4.30f, 0.731f}, {12.88f, 0.606f}, {4.01f, 0.693f}},   // 9 mmd_256x256x32_w2x4_s4
    {{5.69f, 1.360f}, {13.28f, 1.157f}, {4.76f, 1.246f}},   // 10 mmd_256x256x64_w2x4_s2
    {{5.06f, 0.852f}, {6.45f, 0.792f}, {3.04f, 0.956f}},   // 11 mmd_128x128x64_w2x2_s2
    {{4.11f, 0.856f}, {9.21f, 0.824f}, {3.90f, 0.779f}},   // 12 mmd_128x256x32_w2x2_s3
    {{4.36f, 0.904f}, {10.94f, 0.809f}, {4.15f, 0.786f}},   // 13 mmd_256x128x32_w2x2_s3
    {{4.18f, 0.503f}, {6.10f, 0.560f}, {3.20f, 0.459f}},   // 14 mmd_128x128x32_w2x2_s3
    {{5.55f, 1.469f}, {6.82f, 1.473f}, {4.49f, 1.352f}},   // 15 mmp_256x256x64_w2x4_s2
    {{5.39f, 0.852f}, {6.29f, 0.847f}, {4.06f, 0.795f}},   // 16 mmp_256x256x32_w2x4_s4
    {{5.27f, 0.871f}, {3.25f, 0.983f}, {3.08f, 0.980f}},   // 17 mmp_128x128x64_w2x2_s2
    {{4.81f, 2.006f}, {7.24f, 1.819f}, {3.05f, 2.002f}},   // 18 mmk_256x256x64_w2x4_s2
    {{5.52f, 0.907f}, {4.46f, 0.944f}, {3.88f, 1.003f}},   // 19 mmk_128x128x64_w2x2_s2
    {{0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}},                     // 20 mv_8x64x512 (priced by bytes, see plan_cost_us)
    {{5.69f, 1.230f}, {13.28f, 1.060f}, {4.76f, 1.200f}},   // 21 mmq_256x256x64_w2x4_s2 (tile 10's overhead, its own K-block time)
    {{0.f, 0.f}, {0.f, 0.f}, {0.f, 0.f}},                     // 22 ms_64x128x64 (priced by bytes, see plan_cost_us)
};

static int wgs_per_cu(const TileDesc &t, int layout) {
    if (t.gemv == 2) return 2;
    if (t.gemv) return 8;
    const int by_lds = 163840 / lds_bytes_for(t, layout);
    const int acc_regs = t.bm * t.bn / (t.wgm * t.wgn * 64);          // per lane
    const int waves_per_simd = acc_regs > 128 ? 1 : (acc_regs > 64 ? 2 : 4);
    const int by_regs = waves_per_simd * 4 / (t.wgm * t.wgn);
    int w = by_lds < by_regs ? by_lds : by_regs;
    return w < 1 ? 1 : w;
}

// Stream-K partition of `tiles` output tiles of `kblocks` K-blocks over a grid of at most
// `slots` resident workgroups: whole rounds, then the remaining tiles cut into `pieces`
// equal K pieces (at least four blocks each) so that one more, partial round fills the grid.
struct StreamK {
    int64_t grid;
    int full_rounds, rem_tiles, pieces;
};
static StreamK stream_k_partition(int64_t tiles, int64_t kblocks, int64_t slots) {
    StreamK s;
    int64_t cap = kblocks / 4;
    if (cap < 1) cap = 1;
    if (tiles < slots) {
        int64_t pc = slots / tiles;
        if (pc > cap) pc = cap;
        s.grid = tiles * pc;
    } else {
        s.grid = slots;
    }
    s.full_rounds = (int)(tiles / s.grid);
    s.rem_tiles = (int)(tiles - (int64_t)s.full_rounds * s.grid);
    int64_t pc = s.rem_tiles ? s.grid / s.rem_tiles : 1;
    if (pc > cap) pc = cap;
    s.pieces = (int)(pc < 1 ? 1 : pc);
    return s;
}

// Grid of a persistent launch: one workgroup per slot, or per unit if there are fewer.
static int64_t persistent_grid(const TileDesc &t, int64_t tiles, int split, int64_t kblocks, int64_t slots) {
    if (t.persistent == 2 && split == 1) return stream_k_partition(tiles, kblocks, slots).grid;
    const int64_t units = tiles * split;
    return units < slots ? units : slots;
}

// Estimated time (microseconds) of one (tile, split) choice: rounds of co-resident
// workgroups, each paying its overhead plus its K-blocks; a CU that holds fewer
// workgroups than it could runs each of them faster, down to a latency floor.
static double plan_cost_us(const mg_gemm_args &a, const TileDesc &t, int split, int cus) {
    if (t.gemv == 2) {
        // a stream over B at about 4.5 TB/s once the columns fill the chip (128 or 256 per
        // workgroup), the writes of C behind it, and a start-up of a few microseconds
        const double bytes = 2.0 * ((double)a.m * a.k + (double)a.k * a.n) + 4.0 * a.m * a.n * (a.beta ? 2.0 : 1.0);
        const double wgs = (double)cdiv(a.n, 32 * skinny_waves(skinny_blocks(a)));
        const double fill = wgs < cus / 2 ? (cus / 2) / wgs : 1.0;   // few workgroups: each streams alone
        return 4.5 + bytes / 4.5e6 * (fill > 4.0 ? 4.0 : fill);
    }
    if (t.gemv) {
        // a stream over B at about 5 TB/s once enough wavefronts are in flight, plus the
        // multiply-adds, which grow with the rows of A
        const double bytes = 2.0 * ((double)a.m * a.k + (double)a.k * a.n) * a.nbatch + 4.0 * a.m * a.n * a.nbatch;
        return 2.0 + 0.7 * a.m + bytes / 5.4e6 * (1.0 + 0.12 * (a.m - 1));
    }
    const int64_t gm = cdiv(a.m, t.bm), gn = cdiv(a.n, t.bn);
    const int64_t units = gm * gn * (int64_t)a.nbatch * split;
    const int wpc = wgs_per_cu(t, a.layout);
    const int64_t slots = (int64_t)cus * wpc;
    double rounds = t.persistent ? (double)units / (double)slots : (double)cdiv(units, slots);
    if (t.persistent == 2) {
        // stream-K: whole rounds, then one round of K pieces and their meeting
        const int64_t kblocks = cdiv(a.k, t.bk);
        // every batch is partitioned by itself (grid.z), over its share of the resident slots
        const int64_t slots_z = slots / a.nbatch > 0 ? slots / a.nbatch : 1;
        const StreamK sk = stream_k_partition(gm * gn, kblocks, slots_z);
        const int lay2 = a.layout == MG_NN ? 0 : (a.layout == MG_NT ? 1 : 2);
        double occ = (double)cdiv(sk.grid * a.nbatch, cus) / wpc;
        if (occ > 1.0) occ = 1.0;
        if (occ < 0.6) occ = 0.6;
        const double blocks = (double)sk.full_rounds * kblocks + (sk.rem_tiles ? (double)cdiv(kblocks, sk.pieces) : 0.0);
        const double units_wg = sk.full_rounds + (sk.rem_tiles ? 1 : 0);
        // meeting of the pieces: about 5.2 us per piece of a 256 x 256 tile, 1.4 us of a 128 x 128 one
        const double per_piece = t.bm * t.bn > 128 * 128 ? 5.2 : 1.4;
        // more workgroups than resident slots (many batches): they take turns
        double turns = (double)(sk.grid * a.nbatch) / (double)slots;
        if (turns < 1.0) turns = 1.0;
        return 1.5 + turns * (units_wg * g_cost[t.id][lay2][0] + blocks * occ * g_cost[t.id][lay2][1]) +
               (sk.pieces > 1 ? sk.pieces * per_piece : 0.0);
    }
    if (rounds < 1.0) rounds = 1.0;
    const int64_t resident = cdiv(units, cus) < wpc ? cdiv(units, cus) : wpc;
    double occupancy = (double)resident / wpc;
    if (occupancy < 0.6) occupancy = 0.6;
    const int lay = a.layout == MG_NN ? 0 : (a.layout == MG_NT ? 1 : 2);
    const double kb = (double)cdiv(cdiv(a.k, t.bk), split);
    double us = 1.5 + rounds * (g_cost[t.id][lay][0] + kb * occupancy * g_cost[t.id][lay][1]);
    if (split > 1) us += 2.0 + (double)a.m * a.n * 4.0 * a.nbatch * split * 2.0 / 3.0e6;   // partials out and back
    return us;
}

static const int MG_ACT_FALLBACK_TILE = 3;
static void finish_plan(const mg_gemm_args &a, int tile, int split, Plan &pl) {
    const TileDesc *d = &g_tiles[tile];
    int64_t kblocks = cdiv(a.k, d->bk);
    if (split > kblocks) split = (int)kblocks;
    if (split < 1) split = 1;
    // a triangular op(A) splits only on request (the K ranges of the row blocks differ: the picker's
    // cost model does not price that), the lower-triangular C never
    if (d->persistent == 2 || d->gemv || a.tri == MG_TRI_C_LOWER || (a.tri && a.split_k <= 1) ||
        a.act == MG_ACT_SOFTMAX_GRAD)
        split = 1;
    int64_t kb_per = cdiv(kblocks, split);
    split = (int)cdiv(kblocks, kb_per);   // no empty slices
    while (!dma_eligible(a, *d, kb_per * d->bk, split) && d->fallback != tile) {
        tile = d->fallback;
        d = &g_tiles[tile];
        kblocks = cdiv(a.k, d->bk);
        if (split > kblocks) split = (int)kblocks;
        kb_per = cdiv(kblocks, split);
        split = (int)cdiv(kblocks, kb_per);
    }
    if (a.y16 && !table_for(a.layout, a.dtype)[tile][2]) {
        // the fused activation epilogue exists for a few tiles; the any-alignment 128 x 128 one runs everything
        finish_plan(a, MG_ACT_FALLBACK_TILE, split, pl);
        return;
    }
    pl.tile = tile;
    pl.grid_m = (int)cdiv(a.m, d->bm);
    pl.grid_n = (int)cdiv(a.n, d->bn);
    pl.split_k = split;
    pl.k_per_split = (int)(kb_per * d->bk);
    int gm = a.group_m;
    if (gm <= 0) gm = 8;
    if (gm > pl.grid_m) gm = pl.grid_m;
    pl.group_m = gm;
    // XCD-major renumbering needs workgroup id % 8 to be the XCD in every K slice and batch:
    // a tile count in whole eights, or a grid that is nothing but tiles
    const int64_t tiles = (int64_t)pl.grid_m * pl.grid_n;
    pl.xcd_remap = (tiles % 8 == 0 || (split == 1 && a.nbatch <= 1 && tiles >= 16)) ? 1 : 0;
    // rotated walk unless the caller asks for the in-step one: operands of a training step are
    // rarely in the last-level cache, and there the rotated walk is worth up to 15 %
    if (pl.xcd_remap && !(a.flags & MG_FLAG_XCD_IN_STEP)) pl.xcd_remap = 2;
}

// Heuristic choice of tile, K split and rasterisation band (the reference's
// pick_config, autograd.py:22-41, picks the largest tile that still fills its
// 12 CUs; here the same trade-off is priced with a small cost model).  Pure
// arithmetic, so it is testable without a device.
static void pick_plan(const mg_gemm_args &a, int cus, Plan &pl) {
    if (cus <= 0) cus = 256;
    int tile = a.tile, split = a.split_k;
    if (tile < 0 || split <= 0) {
        double best = 1e300;
        int bt = tile < 0 ? 0 : tile, bs = 1;
        for (int t = 0; t < MG_NUM_TILES; t++) {
            if (tile >= 0 && t != tile) continue;
            if (tile < 0 && a.y16 && !table_for(a.layout, a.dtype)[t][2]) continue;
            const TileDesc &d = g_tiles[t];
            const int64_t kblocks = cdiv(a.k, d.bk);
            const int64_t groups = cdiv(a.m, d.bm) * cdiv(a.n, d.bn) * (int64_t)a.nbatch;
            const int64_t slots = (int64_t)cus * wgs_per_cu(d, a.layout);
            int cand[8] = {1, 0, 0, 0, 0, 0, 0, 0};
            int nc = 1;
            if (split > 0) {
                cand[0] = split;
            } else if (groups < slots && kblocks >= 4) {
                // splits that bring the grid to about a half, one or two workgroups per slot
                const int64_t cap = kblocks / 2;
                for (int64_t target : {slots / 2, slots, 2 * slots, (int64_t)cus}) {
                    int64_t s = target / groups;
                    if (s > cap) s = cap;
                    bool seen = s < 2;
                    for (int c = 0; c < nc; c++) seen = seen || cand[c] == (int)s;
                    if (!seen) cand[nc++] = (int)s;
                }
            }
            for (int c = 0; c < nc; c++) {
                const int s = cand[c];
                const int64_t kb_per = cdiv(kblocks, s);
                if (!dma_eligible(a, d, kb_per * d.bk, s)) continue;
                const double cost = plan_cost_us(a, d, s, cus);
                if (cost < best) {
                    best = cost;
                    bt = t;
                    bs = s;
                }
            }
        }
        tile = bt;
        split = bs;
    }
    finish_plan(a, tile, split, pl);
}

static int check_args(const mg_gemm_args *a) {
    if (!a) return fail(MG_ERR_ARG, "mg_gemm: args is NULL");
    if (a->struct_size != (int32_t)sizeof(mg_gemm_args))
        return fail(MG_ERR_ARG, "mg_gemm: struct_size %d != %d", a->struct_size, (int)sizeof(mg_gemm_args));
    if (a->layout < MG_NN || a->layout > MG_TN) return fail(MG_ERR_ARG, "mg_gemm: unknown layout %d", a->layout);
    if (a->dtype != MG_F16 && a->dtype != MG_BF16) return fail(MG_ERR_ARG, "mg_gemm: unknown dtype %d", a->dtype);
    if (a->beta != 0 && a->beta != 1) return fail(MG_ERR_ARG, "mg_gemm: beta must be 0 or 1, got %d", a->beta);
    if (a->m <= 0 || a->n <= 0 || a->k <= 0)
        return fail(MG_ERR_ARG, "mg_gemm: shape %lldx%lldx%lld must be positive", (long long)a->m, (long long)a->n,
                    (long long)a->k);
    if (a->m > 0x7fffffffLL - 512 || a->n > 0x7fffffffLL - 512 || a->k > 0x7fffffffLL - 512)
        return fail(MG_ERR_ARG, "mg_gemm: shape %lldx%lldx%lld exceeds 32-bit indexing", (long long)a->m,
                    (long long)a->n, (long long)a->k);
    if (!a->a || !a->b) return fail(MG_ERR_ARG, "mg_gemm: NULL operand pointer");
    if (!a->c && !(a->y16 && a->beta == 0))
        return fail(MG_ERR_ARG, "mg_gemm: C may only be NULL with y16 given and beta == 0");
    if (a->act < MG_ACT_NONE || a->act > MG_ACT_SOFTMAX_GRAD) return fail(MG_ERR_ARG, "mg_gemm: unknown activation %d", a->act);
    if (!a->y16 && a->act != MG_ACT_NONE) return fail(MG_ERR_ARG, "mg_gemm: an activation needs the y16 output");
    if (a->act == MG_ACT_SOFTMAX_GRAD) {
        if (!a->p16 || !a->rowsub) return fail(MG_ERR_ARG, "mg_gemm: MG_ACT_SOFTMAX_GRAD needs p16 and rowsub");
        if (((uintptr_t)a->p16 & 1) || ((uintptr_t)a->rowsub & 3))
            return fail(MG_ERR_ARG, "mg_gemm: p16 must be 2-byte and rowsub 4-byte aligned");
        if (a->ldp < a->n) return fail(MG_ERR_ARG, "mg_gemm: ldp %lld < N %lld", (long long)a->ldp, (long long)a->n);
        if (a->beta != 0 || a->bias) return fail(MG_ERR_ARG, "mg_gemm: MG_ACT_SOFTMAX_GRAD needs beta == 0 and no bias");
        if (a->z || a->colsum) return fail(MG_ERR_ARG, "mg_gemm: z and colsum belong to the GELU / ReLU _GRAD activations");
        if (!(a->scale == a->scale)) return fail(MG_ERR_ARG, "mg_gemm: scale is NaN");
        if (a->nbatch > 1 && (a->sc < (a->m - 1) * a->ldy + a->n || a->sc < (a->m - 1) * a->ldp + a->n))
            return fail(MG_ERR_ARG, "mg_gemm: batch stride sc %lld overlaps the batches of y16 or p16", (long long)a->sc);
    } else if (a->p16 || a->rowsub) {
        return fail(MG_ERR_ARG, "mg_gemm: p16 and rowsub belong to MG_ACT_SOFTMAX_GRAD");
    } else if (a->act >= MG_ACT_GELU_GRAD) {
        if (!a->z) return fail(MG_ERR_ARG, "mg_gemm: a _GRAD activation needs the pre-activation z");
        if ((uintptr_t)a->z & 3) return fail(MG_ERR_ARG, "mg_gemm: z must be 4-byte aligned");
        if (a->ldz < a->n) return fail(MG_ERR_ARG, "mg_gemm: ldz %lld < N %lld", (long long)a->ldz, (long long)a->n);
        if (a->beta != 0 || a->bias) return fail(MG_ERR_ARG, "mg_gemm: a _GRAD activation needs beta == 0 and no bias");
        if ((uintptr_t)a->colsum & 3) return fail(MG_ERR_ARG, "mg_gemm: colsum must be 4-byte aligned");
    } else if (a->z || a->colsum) {
        return fail(MG_ERR_ARG, "mg_gemm: z and colsum belong to the _GRAD activations");
    }
    if (a->y16) {
        if (a->layout == MG_TN) return fail(MG_ERR_ARG, "mg_gemm: the fused y16 output exists for layouts NN and NT only");
        if (a->nbatch != 1 && a->act != MG_ACT_SOFTMAX_GRAD)
            return fail(MG_ERR_ARG, "mg_gemm: the fused y16 output needs nbatch == 1 (except with MG_ACT_SOFTMAX_GRAD)");
        if ((uintptr_t)a->y16 & 1) return fail(MG_ERR_ARG, "mg_gemm: y16 must be 2-byte aligned");
        if (a->ldy < a->n) return fail(MG_ERR_ARG, "mg_gemm: ldy %lld < N %lld", (long long)a->ldy, (long long)a->n);
        if (a->flags & MG_FLAG_SPLITK_ATOMIC)
            return fail(MG_ERR_ARG, "mg_gemm: the fused y16 output cannot be combined with MG_FLAG_SPLITK_ATOMIC");
    }
    if (a->tri < MG_TRI_NONE || a->tri > MG_TRI_A_UPPER) return fail(MG_ERR_ARG, "mg_gemm: unknown tri %d", a->tri);
    if (a->tri >= MG_TRI_A_LOWER && a->m != a->k)
        return fail(MG_ERR_ARG, "mg_gemm: a triangular op(A) needs M == K, got %lld and %lld", (long long)a->m,
                    (long long)a->k);
    if (a->tri == MG_TRI_C_LOWER && a->split_k > 1)
        return fail(MG_ERR_ARG, "mg_gemm: MG_TRI_C_LOWER runs unsplit; split_k is %d", a->split_k);
    if (a->res) {
        if (a->beta != 1) return fail(MG_ERR_ARG, "mg_gemm: res is what beta == 1 adds to; beta is %d", a->beta);
        if ((uintptr_t)a->res & 3) return fail(MG_ERR_ARG, "mg_gemm: res must be 4-byte aligned");
        if (a->ldr < a->n) return fail(MG_ERR_ARG, "mg_gemm: ldr %lld < N %lld", (long long)a->ldr, (long long)a->n);
        if (a->nbatch != 1) return fail(MG_ERR_ARG, "mg_gemm: res needs nbatch == 1");
        if (a->flags & MG_FLAG_SPLITK_ATOMIC)
            return fail(MG_ERR_ARG, "mg_gemm: res cannot be combined with MG_FLAG_SPLITK_ATOMIC");
    }
    if (((uintptr_t)a->a | (uintptr_t)a->b) & 1) return fail(MG_ERR_ARG, "mg_gemm: A and B must be 2-byte aligned");
    if ((uintptr_t)a->c & 3) return fail(MG_ERR_ARG, "mg_gemm: C must be 4-byte aligned");
    if (a->bias && ((uintptr_t)a->bias & 3)) return fail(MG_ERR_ARG, "mg_gemm: bias must be 4-byte aligned");
    const int64_t a_cols = a->layout == MG_TN ? a->m : a->k;
    const int64_t b_cols = a->layout == MG_NT ? a->k : a->n;
    if (a->lda < a_cols) return fail(MG_ERR_ARG, "mg_gemm: lda %lld < %lld stored columns of A", (long long)a->lda, (long long)a_cols);
    if (a->ldb < b_cols) return fail(MG_ERR_ARG, "mg_gemm: ldb %lld < %lld stored columns of B", (long long)a->ldb, (long long)b_cols);
    if (a->c && a->ldc < a->n) return fail(MG_ERR_ARG, "mg_gemm: ldc %lld < N %lld", (long long)a->ldc, (long long)a->n);
    if (a->nbatch < 1 || a->nbatch > 65535) return fail(MG_ERR_ARG, "mg_gemm: nbatch %d out of range [1, 65535]", a->nbatch);
    if (a->nbatch > 1 && (a->sa < 0 || a->sb < 0 || a->sc < 0))
        return fail(MG_ERR_ARG, "mg_gemm: negative batch stride");
    if (a->nbatch > 1 && a->sc < a->m * a->ldc && a->sc != 0)
        return fail(MG_ERR_ARG, "mg_gemm: batch stride of C (%lld) overlaps outputs", (long long)a->sc);
    if (a->nbatch > 1 && a->sc == 0) return fail(MG_ERR_ARG, "mg_gemm: batches would overwrite one another (sc == 0)");
    if (a->tile < -1 || a->tile >= MG_NUM_TILES) return fail(MG_ERR_ARG, "mg_gemm: unknown tile id %d", a->tile);
    if (a->split_k < 0 || a->split_k > 65535) return fail(MG_ERR_ARG, "mg_gemm: split_k %d out of range", a->split_k);
    if (a->group_m < 0) return fail(MG_ERR_ARG, "mg_gemm: group_m %d is negative", a->group_m);
    if (a->flags & ~(MG_FLAG_TIGHT_BUFFERS | MG_FLAG_SPLITK_ATOMIC | MG_FLAG_SIDE_STREAM | MG_FLAG_XCD_ROTATE | MG_FLAG_XCD_IN_STEP))
        return fail(MG_ERR_ARG, "mg_gemm: unknown flags 0x%x", a->flags);
    if ((a->flags & MG_FLAG_XCD_ROTATE) && (a->flags & MG_FLAG_XCD_IN_STEP))
        return fail(MG_ERR_ARG, "mg_gemm: MG_FLAG_XCD_ROTATE and MG_FLAG_XCD_IN_STEP exclude each other");
    return MG_OK;
}

}  // namespace mg

using namespace mg;

struct mg_ctx {
    int device;
    hipStream_t stream;
    hipEvent_t ev0, ev1;
    // Side stream: GEMMs flagged MG_FLAG_SIDE_STREAM run there, concurrently with the
    // main stream between mg_side_fork and mg_side_join.
    hipStream_t side;
    hipEvent_t ev_fork, ev_join;
    bool side_forked;   // forked and not yet joined
    hipDeviceProp_t prop;
    bool capturing;
    // Split-K workspace: partial tiles of the K slices plus one arrival counter
    // per tile (zero between launches).  Allocated once, at init, so that its
    // address can be baked into captured graphs; a GEMM whose partials do not
    // fit adds into C with atomics instead.  Each stream owns one half of both.
    float *ws;
    int64_t ws_bytes;
    int *cnt;
};
static const int64_t MG_MAX_COUNTED_TILES = 1 << 18;

struct mg_graph {
    hipGraph_t graph;
    hipGraphExec_t exec;
};

extern "C" {

const char *mg_last_error(void) { return g_err; }

int mg_init(int device_index, mg_ctx **out) {
    if (!out) return fail(MG_ERR_ARG, "mg_init: out is NULL");
    *out = nullptr;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        return fail(MG_ERR_NODEVICE, "mg_init: no HIP device available (%s)", e == hipSuccess ? "count is 0" : hipGetErrorString(e));
    }
    if (device_index < 0 || device_index >= count)
        return fail(MG_ERR_ARG, "mg_init: device index %d out of range [0, %d)", device_index, count);
    HIP_TRY(hipSetDevice(device_index));
    mg_ctx *c = new (std::nothrow) mg_ctx();
    if (!c) return fail(MG_ERR_NOMEM, "mg_init: out of host memory");
    c->device = device_index;
    c->capturing = false;
    c->side_forked = false;
    c->stream = c->side = nullptr;
    c->ev0 = c->ev1 = c->ev_fork = c->ev_join = nullptr;
    c->ws = nullptr;
    c->cnt = nullptr;
    auto release = [](mg_ctx *x) {
        if (x->ev0) (void)hipEventDestroy(x->ev0);
        if (x->ev1) (void)hipEventDestroy(x->ev1);
        if (x->ev_fork) (void)hipEventDestroy(x->ev_fork);
        if (x->ev_join) (void)hipEventDestroy(x->ev_join);
        if (x->stream) (void)hipStreamDestroy(x->stream);
        if (x->side) (void)hipStreamDestroy(x->side);
        if (x->ws) (void)hipFree(x->ws);
        if (x->cnt) (void)hipFree(x->cnt);
        delete x;
    };
    e = hipGetDeviceProperties(&c->prop, device_index);
    // both streams at the default priority
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipStreamCreateWithFlags(&c->side, hipStreamNonBlocking);
    if (e == hipSuccess) e = hipEventCreate(&c->ev0);
    if (e == hipSuccess) e = hipEventCreate(&c->ev1);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_fork, hipEventDisableTiming);
    if (e == hipSuccess) e = hipEventCreateWithFlags(&c->ev_join, hipEventDisableTiming);
    if (e != hipSuccess) {
        release(c);
        return hip_fail(e, "mg_init");
    }
    if (strncmp(c->prop.gcnArchName, "gfx950", 6) != 0) {
        char arch[64];
        snprintf(arch, sizeof(arch), "%s", c->prop.gcnArchName);
        release(c);
        return fail(MG_ERR_NODEVICE, "mg_init: device is %s; this library is built for gfx950 only", arch);
    }
    c->ws_bytes = 512ll << 20;
    if (const char *env = getenv("MIGEMM_SPLITK_WORKSPACE_MB")) c->ws_bytes = (int64_t)atoll(env) << 20;
    c->ws_bytes &= ~(int64_t)511;   // two halves, each a multiple of 256 bytes
    if (c->ws_bytes > 0) {
        e = hipMalloc((void **)&c->ws, (size_t)c->ws_bytes);
        if (e == hipSuccess) e = hipMalloc((void **)&c->cnt, 2 * MG_MAX_COUNTED_TILES * sizeof(int));
        if (e == hipSuccess) e = hipMemset(c->cnt, 0, 2 * MG_MAX_COUNTED_TILES * sizeof(int));
        if (e != hipSuccess) {
            release(c);
            return hip_fail(e, "mg_init: split-K workspace");
        }
    } else {
        c->ws_bytes = 0;
    }
    *out = c;
    return MG_OK;
}

int mg_destroy(mg_ctx *ctx) {
    if (!ctx) return MG_OK;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipStreamSynchronize(ctx->side);
    (void)hipEventDestroy(ctx->ev0);
    (void)hipEventDestroy(ctx->ev1);
    (void)hipEventDestroy(ctx->ev_fork);
    (void)hipEventDestroy(ctx->ev_join);
    (void)hipStreamDestroy(ctx->stream);
    (void)hipStreamDestroy(ctx->side);
    (void)hipFree(ctx->ws);
    (void)hipFree(ctx->cnt);
    delete ctx;
    return MG_OK;
}

int mg_get_device_info(mg_ctx *ctx, mg_device_info *out) {
    if (!ctx || !out) return fail(MG_ERR_ARG, "mg_get_device_info: NULL argument");
    memset(out, 0, sizeof(*out));
    snprintf(out->name, sizeof(out->name), "%s", ctx->prop.name[0] ? ctx->prop.name : ctx->prop.gcnArchName);
    snprintf(out->arch, sizeof(out->arch), "%s", ctx->prop.gcnArchName);
    out->compute_units = ctx->prop.multiProcessorCount;
    out->clock_khz = ctx->prop.clockRate;
    out->mem_clock_khz = ctx->prop.memoryClockRate;
    out->mem_bus_bits = ctx->prop.memoryBusWidth;
    out->l2_bytes = ctx->prop.l2CacheSize;
    out->lds_bytes_per_cu = (int32_t)ctx->prop.maxSharedMemoryPerMultiProcessor;
    out->wavefront = ctx->prop.warpSize;
    out->total_mem = (int64_t)ctx->prop.totalGlobalMem;
    return MG_OK;
}

int mg_alloc(mg_ctx *ctx, size_t nbytes, int kind, void **dev_ptr, void **host_ptr) {
    if (!ctx || !dev_ptr || !host_ptr) return fail(MG_ERR_ARG, "mg_alloc: NULL argument");
    *dev_ptr = *host_ptr = nullptr;
    if (kind < MG_DEVICE || kind > MG_BAR) return fail(MG_ERR_ARG, "mg_alloc: unknown memory kind %d", kind);
    if (nbytes == 0) return fail(MG_ERR_ARG, "mg_alloc: size must be positive");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_alloc: not allowed while a graph is being recorded");
    HIP_TRY(hipSetDevice(ctx->device));
    if (kind == MG_DEVICE) {
        void *p = nullptr;
        hipError_t e = hipMalloc(&p, nbytes);
        if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? MG_ERR_NOMEM : MG_ERR_HIP, "mg_alloc: hipMalloc(%zu): %s", nbytes, hipGetErrorString(e));
        *dev_ptr = p;
    } else {
        // Pinned host memory, mapped into the device's address space and
        // coherent: the CPU pointer and the GPU pointer name the same bytes.
        void *p = nullptr;
        hipError_t e = hipHostMalloc(&p, nbytes, hipHostMallocMapped | hipHostMallocCoherent);
        if (e != hipSuccess) return fail(e == hipErrorOutOfMemory ? MG_ERR_NOMEM : MG_ERR_HIP, "mg_alloc: hipHostMalloc(%zu): %s", nbytes, hipGetErrorString(e));
        void *d = nullptr;
        e = hipHostGetDevicePointer(&d, p, 0);
        if (e != hipSuccess) {
            (void)hipHostFree(p);
            return hip_fail(e, "mg_alloc: hipHostGetDevicePointer");
        }
        *host_ptr = p;
        *dev_ptr = d;
    }
    return MG_OK;
}

int mg_free(mg_ctx *ctx, void *dev_ptr, int kind) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_free: ctx is NULL");
    if (!dev_ptr) return MG_OK;
    if (kind < MG_DEVICE || kind > MG_BAR) return fail(MG_ERR_ARG, "mg_free: unknown memory kind %d", kind);
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_free: not allowed while a graph is being recorded");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->side));
    if (kind == MG_DEVICE) HIP_TRY(hipFree(dev_ptr));
    else HIP_TRY(hipHostFree(dev_ptr));
    return MG_OK;
}

static int do_copy(mg_ctx *ctx, void *dst, const void *src, size_t nbytes, hipMemcpyKind kind, const char *who) {
    if (!ctx || !dst || !src) return fail(MG_ERR_ARG, "%s: NULL argument", who);
    if (nbytes == 0) return MG_OK;
    if (ctx->capturing) return fail(MG_ERR_STATE, "%s: not allowed while a graph is being recorded", who);
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipStreamSynchronize(ctx->side));   // a copy sees what either stream has written
    HIP_TRY(hipMemcpyAsync(dst, src, nbytes, kind, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    return MG_OK;
}

int mg_copy(mg_ctx *ctx, void *dst, const void *src, size_t nbytes) {
    return do_copy(ctx, dst, src, nbytes, hipMemcpyDefault, "mg_copy");
}
int mg_upload(mg_ctx *ctx, void *dst_dev, const void *src_host, size_t nbytes) {
    return do_copy(ctx, dst_dev, src_host, nbytes, hipMemcpyHostToDevice, "mg_upload");
}
int mg_download(mg_ctx *ctx, void *dst_host, const void *src_dev, size_t nbytes) {
    return do_copy(ctx, dst_host, src_dev, nbytes, hipMemcpyDeviceToHost, "mg_download");
}

int mg_sync(mg_ctx *ctx) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_sync: ctx is NULL");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_sync: not allowed while a graph is being recorded");
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->side));
    return MG_OK;
}

int mg_side_fork(mg_ctx *ctx) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_side_fork: ctx is NULL");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipEventRecord(ctx->ev_fork, ctx->stream));
    HIP_TRY(hipStreamWaitEvent(ctx->side, ctx->ev_fork, 0));
    ctx->side_forked = true;
    return MG_OK;
}

int mg_side_join(mg_ctx *ctx) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_side_join: ctx is NULL");
    if (!ctx->side_forked) return MG_OK;
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipEventRecord(ctx->ev_join, ctx->side));
    HIP_TRY(hipStreamWaitEvent(ctx->stream, ctx->ev_join, 0));
    ctx->side_forked = false;
    return MG_OK;
}

int mg_gemm_check(const mg_gemm_args *args) { return check_args(args); }

int mg_tile_count(void) { return MG_NUM_TILES; }

int mg_tile_info(int id, mg_tile *out) {
    if (!out) return fail(MG_ERR_ARG, "mg_tile_info: out is NULL");
    if (id < 0 || id >= MG_NUM_TILES) return fail(MG_ERR_ARG, "mg_tile_info: unknown tile id %d", id);
    const TileDesc &t = g_tiles[id];
    memset(out, 0, sizeof(*out));
    out->id = id;
    out->bm = t.bm;
    out->bn = t.bn;
    out->bk = t.bk;
    out->waves_m = t.wgm;
    out->waves_n = t.wgn;
    out->threads = t.wgm * t.wgn * 64;
    out->lds_bytes = lds_bytes_for(t, MG_NT);
    out->min_m = 1;
    if (t.gemv)
        snprintf(out->name, sizeof(out->name), "%s_%dx%dx%d", t.gemv == 2 ? "ms" : "mv", t.bm, t.bn, t.bk);
    else if (t.persistent)
        snprintf(out->name, sizeof(out->name), "%s_%dx%dx%d_w%dx%d_s%d", t.persistent == 2 ? "mmk" : "mmp", t.bm, t.bn, t.bk,
                 t.wgm, t.wgn, t.nstage);
    else if (t.nstage > 0)
        snprintf(out->name, sizeof(out->name), "%s_%dx%dx%d_w%dx%d_s%d", t.pingpong ? "mmq" : "mmd", t.bm, t.bn, t.bk, t.wgm,
                 t.wgn, t.nstage);
    else
        snprintf(out->name, sizeof(out->name), "mm_%dx%dx%d_w%dx%d", t.bm, t.bn, t.bk, t.wgm, t.wgn);
    out->stages = t.nstage;
    out->fallback = t.fallback;
    out->persistent = t.persistent;
    return MG_OK;
}

int mg_tile_fits(int id, const mg_gemm_args *args) {
    if (id < 0 || id >= MG_NUM_TILES) return 0;
    if (check_args(args) != MG_OK) return 0;
    // every tile handles ragged shapes; the only limit is the grid size
    const TileDesc &t = g_tiles[id];
    const int64_t groups = cdiv(args->m, t.bm) * cdiv(args->n, t.bn);
    return groups <= 0x7fffffffLL ? 1 : 0;
}

int mg_pick(const mg_gemm_args *args, int compute_units, int *tile, int *split_k, int *group_m) {
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    Plan pl;
    pick_plan(*args, compute_units, pl);
    if (tile) *tile = pl.tile;
    if (split_k) *split_k = pl.split_k;
    if (group_m) *group_m = pl.group_m;
    return MG_OK;
}

static int fill_stats(const KernelQuery &q, mg_kernel_stats *out) {
    memset(out, 0, sizeof(*out));
    out->vgprs = q.attr.numRegs;
    out->scratch_bytes = (int32_t)q.attr.localSizeBytes;
    out->static_lds_bytes = (int32_t)q.attr.sharedSizeBytes;
    out->dynamic_lds_bytes = q.dynamic_lds;
    out->threads = q.threads;
    out->wgs_per_cu = q.wgs_per_cu;
    out->waves_per_simd = (q.wgs_per_cu * (q.threads / 64) + 3) / 4;
    out->max_threads = q.attr.maxThreadsPerBlock;
    return MG_OK;
}

int mg_tile_kernel_stats(mg_ctx *ctx, int tile, int layout, int dtype, int variant, mg_kernel_stats *out) {
    if (!ctx || !out) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: NULL argument");
    if (tile < 0 || tile >= MG_NUM_TILES) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: unknown tile id %d", tile);
    if (layout < MG_NN || layout > MG_TN) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: unknown layout %d", layout);
    if (dtype != MG_F16 && dtype != MG_BF16) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: unknown dtype %d", dtype);
    HIP_TRY(hipSetDevice(ctx->device));
    KernelQuery q;
    memset(&q, 0, sizeof(q));
    const TileDesc &t = g_tiles[tile];
    if (t.gemv == 2) {
        if (layout != MG_NT || variant < 0 || variant >= SKINNY_MAX_TMB)
            return fail(MG_ERR_ARG, "mg_tile_kernel_stats: the skinny-M matrix-core tile has no instantiation %d for this layout", variant);
        SkinnyParams g{};
        const int tmb = variant + 1, nw = skinny_waves(tmb);
        HIP_TRY(skinny_table[dtype][variant](g, dim3(1), skinny_lds_bytes(tmb, nw, SKINNY_KP, 768), nullptr, &q));
        return fill_stats(q, out);
    }
    if (t.gemv) {
        if (layout != MG_NT || variant < 0 || variant >= 16 || !gemv_table[dtype][variant / 4][variant % 4])
            return fail(MG_ERR_ARG, "mg_tile_kernel_stats: the skinny-M tile has no instantiation %d for this layout", variant);
        GemvParams g{};
        HIP_TRY(gemv_table[dtype][variant / 4][variant % 4](g, dim3(1), nullptr, &q));
        return fill_stats(q, out);
    }
    if (variant < 0 || variant > 2) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: variant %d out of range", variant);
    launch_fn fn = table_for(layout, dtype)[tile][variant];
    if (!fn) return fail(MG_ERR_ARG, "mg_tile_kernel_stats: tile %d has no variant %d in this layout", tile, variant);
    GemmParams p{};
    HIP_TRY(fn(p, dim3(1), nullptr, &q));
    return fill_stats(q, out);
}

// Where a GEMM runs and what it may use there: a stream, that stream's share of the split-K
// workspace (partial tiles and per-tile arrival counters), and the limits of the device.
struct Lane {
    hipStream_t stream;
    float *ws;            // NULL: no workspace, K slices add into C with atomics
    int64_t ws_bytes;
    int *cnt;
    int64_t max_tiles;    // arrival counters available
    int cus;
    int lds_limit;        // LDS bytes a workgroup may use
    // The counters a launch uses are cleared by a fill kernel in front of it: for a workspace
    // that keeps what the last call left (mg_gemm_static).  A context's counters are zero
    // between launches by construction and need none.
    bool clear_counters = false;
    // Dry run: nothing is launched, every kernel that would be is counted here.
    int *dry_count = nullptr;
};

// MG_FLAG_SPLITK_ATOMIC keeps a call off the workspace altogether: no slices meeting there, no
// partial round cut into slices, no stream-K pieces.
static Lane lane_without_ws(Lane ln) {
    ln.ws = nullptr;
    ln.cnt = nullptr;
    ln.ws_bytes = 0;
    ln.max_tiles = 0;
    return ln;
}

static int lane_of(mg_ctx *ctx, const mg_gemm_args &a, Lane &ln) {
    const bool on_side = (a.flags & MG_FLAG_SIDE_STREAM) != 0;
    if (on_side && !ctx->side_forked)
        return fail(MG_ERR_STATE, "mg_gemm: MG_FLAG_SIDE_STREAM needs mg_side_fork first");
    // the stream this GEMM runs on, and that stream's half of the split-K workspace
    ln.stream = on_side ? ctx->side : ctx->stream;
    ln.ws_bytes = ctx->ws_bytes / 2;
    ln.ws = ctx->ws ? ctx->ws + (on_side ? ln.ws_bytes / (int64_t)sizeof(float) : 0) : nullptr;
    ln.cnt = ctx->cnt ? ctx->cnt + (on_side ? MG_MAX_COUNTED_TILES : 0) : nullptr;
    ln.max_tiles = MG_MAX_COUNTED_TILES;
    ln.cus = ctx->prop.multiProcessorCount;
    ln.lds_limit = (int)ctx->prop.maxSharedMemoryPerMultiProcessor;
    return MG_OK;
}

// The partial last round of an unsplit ping-pong GEMM with a long K loop.  591 tiles on 256 CUs
// are three rounds of which the last keeps 79 CUs busy; run as two GEMMs over row ranges - whole
// rounds unsplit, the remaining tile rows with a K split that fills the chip once more - the
// 50257 x 768 x 8192 dW product takes 538 us instead of 581.  Estimated in K-block times: a round
// costs the K loop, the split part its slice of it plus 1.7 per slice for the meeting of the
// partial tiles and 2.5 for the second launch.  Returns the rows of the first GEMM (0: no split).
static int64_t tail_rows(const Lane &ln, const mg_gemm_args &a, const Plan &pl, const TileDesc &t, int *slices) {
    if (!t.pingpong || pl.split_k != 1 || a.nbatch != 1 || a.tri != MG_TRI_NONE) return 0;
    if (!a.c || a.y16 || a.z || a.colsum || a.res || a.p16) return 0;
    // (cus: workgroups resident at once)
    const int64_t tiles = (int64_t)pl.grid_m * pl.grid_n, cus = (int64_t)ln.cus * wgs_per_cu(t, a.layout);
    if (cus < 8 || tiles <= cus || tiles % cus == 0) return 0;
    const int64_t rows1 = (tiles / cus) * cus / pl.grid_n;            // tile rows of the whole rounds
    const int64_t rest = (pl.grid_m - rows1) * pl.grid_n;             // tiles left over
    if (rows1 < 1 || rest < 1) return 0;
    const int64_t s = std::min<int64_t>(8, cus / rest);
    const int64_t nkb = cdiv(a.k, t.bk);
    if (s < 2 || nkb / s < 8) return 0;
    const double as_is = (double)cdiv(tiles, cus) * nkb;
    const double cut = (double)cdiv(rows1 * pl.grid_n, cus) * nkb + cdiv(nkb, s) + 1.7 * s + 2.5;
    if (cut > 0.95 * as_is) return 0;
    if (!ln.ws || rest * s * t.bm * t.bn * (int64_t)sizeof(float) > ln.ws_bytes || rest > ln.max_tiles) return 0;
    *slices = (int)s;
    return rows1 * t.bm;
}

// Which instantiation of a tile serves a call.  Direct-to-LDS tiles: eligibility was settled by
// the plan; register-staged tiles: the any-alignment instantiation unless every chunk is aligned
// and whole; persistent tiles: [1] is the epilogue with bias; [2] everywhere the fused activation.
static int variant_for(const mg_gemm_args &a, const TileDesc &t) {
    if (t.persistent) return a.bias != nullptr ? 1 : 0;
    if (a.y16) return 2;
    return t.nstage > 0 ? 0 : (operands_aligned(a) ? 0 : 1);
}

static int enqueue_gemm(const Lane &lane, const mg_gemm_args *args, const Plan &pl) {
    const mg_gemm_args &a = *args;
    const TileDesc &t = g_tiles[pl.tile];
    const Lane ln = (a.flags & MG_FLAG_SPLITK_ATOMIC) ? lane_without_ws(lane) : lane;
    {
        int slices = 1;
        const int64_t m1 = tail_rows(ln, a, pl, t, &slices);
        if (m1 > 0) {
            mg_gemm_args head = a, tail = a;
            head.m = m1;
            head.tile = tail.tile = pl.tile;
            head.split_k = 1;
            tail.m = a.m - m1;
            tail.split_k = slices;
            tail.flags &= ~MG_FLAG_SPLITK_ATOMIC;
            tail.a = (const char *)a.a + (a.layout == MG_TN ? m1 : m1 * a.lda) * 2;
            tail.c = a.c + m1 * a.ldc;
            Plan ph, pt;
            pick_plan(head, ln.cus, ph);
            pick_plan(tail, ln.cus, pt);
            // (neither part qualifies again: the head is whole rounds, the tail is split)
            if (ph.tile == pl.tile && pt.tile == pl.tile && ph.split_k == 1 && pt.split_k == slices) {
                const int rc = enqueue_gemm(ln, &head, ph);
                return rc != MG_OK ? rc : enqueue_gemm(ln, &tail, pt);
            }
        }
    }
    hipStream_t stream = ln.stream;
    const int64_t lane_bytes = ln.ws_bytes;
    float *lane_ws = ln.ws;
    int *lane_cnt = ln.cnt;
    GemmParams p;
    p.A = (const uint16_t *)a.a;
    p.B = (const uint16_t *)a.b;
    p.C = a.c;
    p.bias = a.bias;
    p.lda = a.lda;
    p.ldb = a.ldb;
    p.ldc = a.ldc;
    p.sa = a.nbatch > 1 ? a.sa : 0;
    p.sb = a.nbatch > 1 ? a.sb : 0;
    p.sc = a.nbatch > 1 ? a.sc : 0;
    p.M = (int)a.m;
    p.N = (int)a.n;
    p.K = (int)a.k;
    p.beta = a.beta;
    p.grid_m = pl.grid_m;
    p.grid_n = pl.grid_n;
    p.group_m = pl.group_m;
    p.split_k = pl.split_k;
    p.k_per_split = pl.k_per_split;
    p.xcd_remap = pl.xcd_remap;
    if ((int64_t)pl.grid_m * pl.grid_n > 0x7fffffffLL) return fail(MG_ERR_ARG, "mg_gemm: grid too large");
    if (t.gemv == 2) {
        if (!skinny_eligible(a, pl.split_k)) return fail(MG_ERR_STATE, "mg_gemm: the skinny-M matrix-core tile cannot run this call");
        const int tmb = skinny_blocks(a), nw = skinny_waves(tmb);
        SkinnyParams g;
        g.A = p.A; g.B = p.B; g.C = p.C; g.bias = p.bias;
        g.lda = p.lda; g.ldb = p.ldb; g.ldc = p.ldc;
        g.M = p.M; g.N = p.N; g.K = p.K; g.beta = p.beta;
        if (ln.dry_count) {
            ++*ln.dry_count;
            return MG_OK;
        }
        hipError_t e = skinny_table[a.dtype][tmb - 1](g, dim3((unsigned)cdiv(a.n, 32 * nw)), skinny_lds_bytes(tmb, nw, SKINNY_KP, p.K),
                                                       stream, nullptr);
        if (e != hipSuccess) return hip_fail(e, "mg_gemm: kernel launch");
        return MG_OK;
    }
    if (t.gemv) {
        int lm = 0, lc = 0;
        if (!gemv_eligible(a, pl.split_k) || !gemv_shape(a, &lm, &lc) || !gemv_table[a.dtype][lm][lc])
            return fail(MG_ERR_STATE, "mg_gemm: the skinny-M tile cannot run this call");
        GemvParams g;
        g.A = p.A; g.B = p.B; g.C = p.C; g.bias = p.bias;
        g.lda = p.lda; g.ldb = p.ldb; g.ldc = p.ldc;
        g.sa = p.sa; g.sb = p.sb; g.sc = p.sc;
        g.M = p.M; g.N = p.N; g.K = p.K; g.beta = p.beta;
        const dim3 grid((unsigned)cdiv(a.n, GEMV_ROWS_PER_WG), 1, (unsigned)a.nbatch);
        if (ln.dry_count) {
            ++*ln.dry_count;
            return MG_OK;
        }
        hipError_t e = gemv_table[a.dtype][lm][lc](g, grid, stream, nullptr);
        if (e != hipSuccess) return hip_fail(e, "mg_gemm: kernel launch");
        return MG_OK;
    }
    if (lds_bytes_for(t, a.layout) > ln.lds_limit)
        return fail(MG_ERR_ARG, "mg_gemm: tile %d needs %d bytes of LDS", pl.tile, lds_bytes_for(t, a.layout));
    p.Y = (uint16_t *)a.y16;
    p.ldy = a.ldy;
    p.act = a.act;
    p.Z = a.z;
    p.ldz = a.ldz;
    p.colsum = a.colsum;
    p.P16 = (const uint16_t *)a.p16;
    p.ldp = a.ldp;
    p.rowsub = a.rowsub;
    p.scale = a.scale;
    p.sy = (a.y16 && a.nbatch > 1) ? a.sc : 0;
    p.tri = a.tri;
    p.R = (a.res && a.res != a.c) ? a.res : nullptr;
    p.ldr = a.ldr;
    p.ws = nullptr;
    p.cnt = nullptr;
    p.stream_k = 0;
    p.stagger_clk = p.stagger_blocks = 0;
    if (t.pingpong) {
        // more than one round of tiles whose K loop is short beside their C store: spread the
        // starts of the first round over one K loop (2048 MFMA clocks a K-block)
        const int64_t wgs = (int64_t)pl.grid_m * pl.grid_n * a.nbatch * pl.split_k;
        const int64_t nkb = cdiv(pl.split_k > 1 ? pl.k_per_split : a.k, t.bk);
        const int64_t resident = (int64_t)ln.cus * wgs_per_cu(t, a.layout);
        if (wgs > resident && nkb <= 16) {
            p.stagger_clk = (int)nkb * 2048;
            p.stagger_blocks = (int)resident;
        }
    }
    p.sk_full_rounds = p.sk_rem_tiles = 0;
    p.sk_pieces = 1;
    if (pl.split_k > 1) {
        // partial tiles go through the workspace when they fit
        const int64_t tiles = (int64_t)pl.grid_m * pl.grid_n * a.nbatch;
        const int64_t need = tiles * pl.split_k * t.bm * t.bn * (int64_t)sizeof(float);
        if (lane_ws && need <= lane_bytes && tiles <= ln.max_tiles && !(a.flags & MG_FLAG_SPLITK_ATOMIC)) {
            p.ws = lane_ws;
            p.cnt = lane_cnt;
        }
        if ((a.y16 || p.R) && !p.ws) {
            // the activation is applied once, to the finished sum, and the residual is added
            // once: without a workspace for the slices to meet in, the same GEMM runs unsplit
            mg_gemm_args whole = a;
            whole.split_k = 1;
            Plan unsplit;
            pick_plan(whole, ln.cus, unsplit);
            return enqueue_gemm(ln, &whole, unsplit);
        }
    }
    if (pl.split_k > 1 && a.beta == 0 && p.ws == nullptr) {
        // A dense C (pitch == N, batches back to back) is cleared as one long row.
        const bool dense = a.ldc == a.n && (a.nbatch == 1 || p.sc == a.m * a.n) &&
                           a.m * a.n * (int64_t)a.nbatch < 0x40000000LL;
        const int zm = dense ? 1 : (int)a.m;
        const int zn = dense ? (int)(a.m * a.n * a.nbatch) : (int)a.n;
        const int zb = dense ? 1 : a.nbatch;
        const int vec = (reinterpret_cast<uintptr_t>(a.c) % 16 == 0) && (dense || (a.ldc % 4 == 0 && p.sc % 4 == 0));
        unsigned gx = (unsigned)cdiv(zn, 1024);
        unsigned gy = (unsigned)(zm < 4096 ? zm : 4096);
        if (gx > 65535u * 16u) return fail(MG_ERR_ARG, "mg_gemm: C too large for the split-K clear");
        if (ln.dry_count) {
            ++*ln.dry_count;
        } else {
            hipLaunchKernelGGL(zero_c_kernel, dim3(gx, gy, (unsigned)zb), dim3(256), 0, stream, a.c, a.ldc, zm, zn,
                               p.sc, vec);
            HIP_TRY(hipGetLastError());
        }
    }
    int general = variant_for(a, t);
    dim3 grid((unsigned)(pl.grid_m * pl.grid_n), (unsigned)pl.split_k, (unsigned)a.nbatch);
    if (t.persistent) {
        const int64_t tiles = (int64_t)pl.grid_m * pl.grid_n;
        const int64_t slots = (int64_t)ln.cus * wgs_per_cu(t, a.layout);
        // stream-K cuts tiles only when the batches together leave resident slots idle: every batch
        // (one grid.z slice) is partitioned by itself, over its share of the slots
        const int64_t slots_z = slots / a.nbatch > 0 ? slots / a.nbatch : 1;
        int64_t g = persistent_grid(t, tiles, pl.split_k, a.k / t.bk, t.persistent == 2 ? slots_z : slots);
        if (t.persistent == 2 && pl.split_k == 1) {
            // one workspace slot per piece; without the workspace the tile runs as plain persistent
            const StreamK sk = stream_k_partition(tiles, a.k / t.bk, slots_z);
            const int64_t need = (int64_t)sk.pieces * sk.rem_tiles * a.nbatch * t.bm * t.bn * (int64_t)sizeof(float);
            if (sk.pieces == 1) {
                g = tiles < slots ? tiles : slots;   // nothing to cut
            } else if (lane_ws && need <= lane_bytes && tiles * a.nbatch <= ln.max_tiles) {
                p.stream_k = 1;
                p.sk_full_rounds = sk.full_rounds;
                p.sk_rem_tiles = sk.rem_tiles;
                p.sk_pieces = sk.pieces;
                p.ws = lane_ws;
                p.cnt = lane_cnt;
            } else {
                g = tiles < slots ? tiles : slots;
            }
        }
        grid = dim3((unsigned)g, 1, (unsigned)a.nbatch);
        p.xcd_remap = 0;
    }
    launch_fn fn = table_for(a.layout, a.dtype)[pl.tile][general];
    if (!fn) return fail(MG_ERR_STATE, "mg_gemm: tile %d has no kernel for this alignment", pl.tile);
    if (p.cnt && ln.clear_counters) {
        // one counter per tile of this launch (all batches)
        const int64_t counted = (int64_t)pl.grid_m * pl.grid_n * a.nbatch;
        if (ln.dry_count) {
            ++*ln.dry_count;
        } else {
            hipLaunchKernelGGL(zero_ints_kernel, dim3((unsigned)cdiv(counted, 256)), dim3(256), 0, stream, p.cnt,
                               (int)counted);
            HIP_TRY(hipGetLastError());
        }
    }
    if (ln.dry_count) {
        ++*ln.dry_count;
        return MG_OK;
    }
    hipError_t e = fn(p, grid, stream, nullptr);
    if (e != hipSuccess) return hip_fail(e, "mg_gemm: kernel launch");
    return MG_OK;
}

int mg_gemm(mg_ctx *ctx, const mg_gemm_args *args) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_gemm: ctx is NULL");
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    Lane ln;
    rc = lane_of(ctx, *args, ln);
    if (rc != MG_OK) return rc;
    Plan pl;
    pick_plan(*args, ln.cus, pl);
    return enqueue_gemm(ln, args, pl);
}

int mg_kernel_stats_for(mg_ctx *ctx, const mg_gemm_args *args, int *tile, mg_kernel_stats *out) {
    if (!ctx || !out) return fail(MG_ERR_ARG, "mg_kernel_stats_for: NULL argument");
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    Plan pl;
    pick_plan(*args, ctx->prop.multiProcessorCount, pl);
    const TileDesc &t = g_tiles[pl.tile];
    if (tile) *tile = pl.tile;
    if (t.gemv == 2) return mg_tile_kernel_stats(ctx, pl.tile, args->layout, args->dtype, skinny_blocks(*args) - 1, out);
    if (t.gemv) {
        int lm = 0, lc = 0;
        if (!gemv_shape(*args, &lm, &lc)) return fail(MG_ERR_STATE, "mg_kernel_stats_for: the skinny-M tile cannot run this call");
        return mg_tile_kernel_stats(ctx, pl.tile, args->layout, args->dtype, 4 * lm + lc, out);
    }
    return mg_tile_kernel_stats(ctx, pl.tile, args->layout, args->dtype, variant_for(*args, t), out);
}

int mg_gemm_time(mg_ctx *ctx, const mg_gemm_args *args, int repeat, double *seconds) {
    if (!ctx || !seconds) return fail(MG_ERR_ARG, "mg_gemm_time: NULL argument");
    if (repeat < 1) return fail(MG_ERR_ARG, "mg_gemm_time: repeat must be >= 1");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_gemm_time: not allowed while a graph is being recorded");
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    if (args->flags & MG_FLAG_SIDE_STREAM) return fail(MG_ERR_ARG, "mg_gemm_time: timing runs on the main stream");
    Lane ln;
    rc = lane_of(ctx, *args, ln);
    if (rc != MG_OK) return rc;
    Plan pl;
    pick_plan(*args, ln.cus, pl);
    HIP_TRY(hipEventRecord(ctx->ev0, ctx->stream));
    for (int i = 0; i < repeat; i++) {
        rc = enqueue_gemm(ln, args, pl);
        if (rc != MG_OK) return rc;
    }
    HIP_TRY(hipEventRecord(ctx->ev1, ctx->stream));
    HIP_TRY(hipEventSynchronize(ctx->ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
    *seconds = (double)ms * 1e-3;
    return MG_OK;
}

int mg_gemm_time_rotating(mg_ctx *ctx, const mg_gemm_args *args, int nargs, int repeat, double *seconds) {
    if (!ctx || !args || !seconds) return fail(MG_ERR_ARG, "mg_gemm_time_rotating: NULL argument");
    if (nargs < 1 || nargs > 64) return fail(MG_ERR_ARG, "mg_gemm_time_rotating: nargs must be 1..64");
    if (repeat < 1) return fail(MG_ERR_ARG, "mg_gemm_time_rotating: repeat must be >= 1");
    if (ctx->capturing)
        return fail(MG_ERR_STATE, "mg_gemm_time_rotating: not allowed while a graph is being recorded");
    Plan pl[64];
    for (int i = 0; i < nargs; i++) {
        int rc = check_args(&args[i]);
        if (rc != MG_OK) return rc;
        if (args[i].flags & MG_FLAG_SIDE_STREAM)
            return fail(MG_ERR_ARG, "mg_gemm_time_rotating: timing runs on the main stream");
        pick_plan(args[i], ctx->prop.multiProcessorCount, pl[i]);
    }
    Lane ln;
    {
        int rc = lane_of(ctx, args[0], ln);
        if (rc != MG_OK) return rc;
    }
    HIP_TRY(hipEventRecord(ctx->ev0, ctx->stream));
    for (int i = 0; i < repeat; i++) {
        int rc = enqueue_gemm(ln, &args[i % nargs], pl[i % nargs]);
        if (rc != MG_OK) return rc;
    }
    HIP_TRY(hipEventRecord(ctx->ev1, ctx->stream));
    HIP_TRY(hipEventSynchronize(ctx->ev1));
    float ms = 0.f;
    HIP_TRY(hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1));
    *seconds = (double)ms * 1e-3;
    return MG_OK;
}

int mg_gemm_time_each(mg_ctx *ctx, const mg_gemm_args *args, int nargs, double *seconds_each) {
    if (!ctx || !args || !seconds_each) return fail(MG_ERR_ARG, "mg_gemm_time_each: NULL argument");
    if (nargs < 1 || nargs > 4096) return fail(MG_ERR_ARG, "mg_gemm_time_each: nargs must be 1..4096");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_gemm_time_each: not allowed while a graph is being recorded");
    Plan *pl = new (std::nothrow) Plan[nargs];
    hipEvent_t *ev = new (std::nothrow) hipEvent_t[nargs + 1]();
    if (!pl || !ev) {
        delete[] pl;
        delete[] ev;
        return fail(MG_ERR_NOMEM, "mg_gemm_time_each: out of host memory");
    }
    int rc = MG_OK, made = 0;
    Lane ln;
    for (int i = 0; i < nargs && rc == MG_OK; i++) {
        rc = check_args(&args[i]);
        if (rc == MG_OK && (args[i].flags & MG_FLAG_SIDE_STREAM))
            rc = fail(MG_ERR_ARG, "mg_gemm_time_each: timing runs on the main stream");
        if (rc == MG_OK) pick_plan(args[i], ctx->prop.multiProcessorCount, pl[i]);
    }
    if (rc == MG_OK) rc = lane_of(ctx, args[0], ln);
    if (rc == MG_OK && hipSetDevice(ctx->device) != hipSuccess) rc = fail(MG_ERR_HIP, "mg_gemm_time_each: hipSetDevice");
    for (; rc == MG_OK && made <= nargs; made++) {
        hipError_t e = hipEventCreate(&ev[made]);
        if (e != hipSuccess) {
            rc = hip_fail(e, "mg_gemm_time_each: hipEventCreate");
            break;
        }
    }
    if (rc == MG_OK) {
        hipError_t e = hipEventRecord(ev[0], ctx->stream);
        for (int i = 0; i < nargs && e == hipSuccess && rc == MG_OK; i++) {
            rc = enqueue_gemm(ln, &args[i], pl[i]);
            if (rc == MG_OK) e = hipEventRecord(ev[i + 1], ctx->stream);
        }
        if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);
        for (int i = 0; i < nargs && e == hipSuccess && rc == MG_OK; i++) {
            float ms = 0.f;
            e = hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
            seconds_each[i] = (double)ms * 1e-3;
        }
        if (e != hipSuccess && rc == MG_OK) rc = hip_fail(e, "mg_gemm_time_each");
    }
    for (int i = 0; i < made; i++) (void)hipEventDestroy(ev[i]);
    delete[] ev;
    delete[] pl;
    return rc;
}

int mg_graph_begin(mg_ctx *ctx) {
    if (!ctx) return fail(MG_ERR_ARG, "mg_graph_begin: ctx is NULL");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_graph_begin: a graph is already being recorded");
    if (ctx->side_forked) return fail(MG_ERR_STATE, "mg_graph_begin: join the side stream first (mg_side_join)");
    HIP_TRY(hipSetDevice(ctx->device));
    HIP_TRY(hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal));
    ctx->capturing = true;
    return MG_OK;
}

int mg_graph_end(mg_ctx *ctx, mg_graph **out) {
    if (!ctx || !out) return fail(MG_ERR_ARG, "mg_graph_end: NULL argument");
    *out = nullptr;
    if (!ctx->capturing) return fail(MG_ERR_STATE, "mg_graph_end: no graph is being recorded");
    if (ctx->side_forked) {
        // a capture cannot end while a forked stream is still apart
        int rc = mg_side_join(ctx);
        if (rc != MG_OK) {
            hipGraph_t dead = nullptr;
            (void)hipStreamEndCapture(ctx->stream, &dead);
            if (dead) (void)hipGraphDestroy(dead);
            ctx->capturing = false;
            ctx->side_forked = false;
            return rc;
        }
    }
    hipGraph_t g = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &g);
    ctx->capturing = false;
    if (e != hipSuccess) return hip_fail(e, "mg_graph_end: hipStreamEndCapture");
    hipGraphExec_t ex = nullptr;
    e = hipGraphInstantiate(&ex, g, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(g);
        return hip_fail(e, "mg_graph_end: hipGraphInstantiate");
    }
    mg_graph *r = new (std::nothrow) mg_graph();
    if (!r) {
        (void)hipGraphExecDestroy(ex);
        (void)hipGraphDestroy(g);
        return fail(MG_ERR_NOMEM, "mg_graph_end: out of host memory");
    }
    r->graph = g;
    r->exec = ex;
    *out = r;
    return MG_OK;
}

int mg_graph_launch(mg_ctx *ctx, mg_graph *g, double *seconds) {
    if (!ctx || !g) return fail(MG_ERR_ARG, "mg_graph_launch: NULL argument");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_graph_launch: a graph is being recorded");
    auto t0 = std::chrono::steady_clock::now();
    HIP_TRY(hipGraphLaunch(g->exec, ctx->stream));
    HIP_TRY(hipStreamSynchronize(ctx->stream));
    auto t1 = std::chrono::steady_clock::now();
    if (seconds) *seconds = std::chrono::duration<double>(t1 - t0).count();
    return MG_OK;
}

int mg_graph_enqueue(mg_ctx *ctx, mg_graph *g) {
    if (!ctx || !g) return fail(MG_ERR_ARG, "mg_graph_enqueue: NULL argument");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_graph_enqueue: a graph is being recorded");
    HIP_TRY(hipGraphLaunch(g->exec, ctx->stream));
    return MG_OK;
}

int mg_graph_time(mg_ctx *ctx, mg_graph *g, int repeat, double *seconds_each) {
    if (!ctx || !g || !seconds_each) return fail(MG_ERR_ARG, "mg_graph_time: NULL argument");
    if (repeat < 1 || repeat > 4096) return fail(MG_ERR_ARG, "mg_graph_time: repeat must be 1..4096");
    if (ctx->capturing) return fail(MG_ERR_STATE, "mg_graph_time: a graph is being recorded");
    HIP_TRY(hipSetDevice(ctx->device));
    hipEvent_t *ev = new (std::nothrow) hipEvent_t[repeat + 1]();
    if (!ev) return fail(MG_ERR_NOMEM, "mg_graph_time: out of host memory");
    int rc = MG_OK;
    int made = 0;
    for (; made <= repeat; made++) {
        hipError_t e = hipEventCreate(&ev[made]);
        if (e != hipSuccess) {
            rc = hip_fail(e, "mg_graph_time: hipEventCreate");
            break;
        }
    }
    if (rc == MG_OK) {
        hipError_t e = hipEventRecord(ev[0], ctx->stream);
        for (int i = 0; i < repeat && e == hipSuccess; i++) {
            e = hipGraphLaunch(g->exec, ctx->stream);
            if (e == hipSuccess) e = hipEventRecord(ev[i + 1], ctx->stream);
        }
        if (e == hipSuccess) e = hipEventSynchronize(ev[repeat]);
        for (int i = 0; i < repeat && e == hipSuccess; i++) {
            float ms = 0.f;
            e = hipEventElapsedTime(&ms, ev[i], ev[i + 1]);
            seconds_each[i] = (double)ms * 1e-3;
        }
        if (e != hipSuccess) rc = hip_fail(e, "mg_graph_time");
    }
    for (int i = 0; i < made; i++) (void)hipEventDestroy(ev[i]);
    delete[] ev;
    return rc;
}

int mg_graph_kernel_count(mg_ctx *ctx, mg_graph *g, int *kernels) {
    if (!ctx || !g || !kernels) return fail(MG_ERR_ARG, "mg_graph_kernel_count: NULL argument");
    size_t n = 0;
    HIP_TRY(hipGraphGetNodes(g->graph, nullptr, &n));
    hipGraphNode_t *nodes = n ? new (std::nothrow) hipGraphNode_t[n] : nullptr;
    if (n && !nodes) return fail(MG_ERR_STATE, "mg_graph_kernel_count: out of host memory");
    int count = 0;
    hipError_t e = n ? hipGraphGetNodes(g->graph, nodes, &n) : hipSuccess;
    for (size_t i = 0; e == hipSuccess && i < n; i++) {
        hipGraphNodeType ty;
        e = hipGraphNodeGetType(nodes[i], &ty);
        if (e == hipSuccess && ty == hipGraphNodeTypeKernel) count++;
    }
    delete[] nodes;
    if (e != hipSuccess) return hip_fail(e, "mg_graph_kernel_count");
    *kernels = count;
    return MG_OK;
}

int mg_graph_destroy(mg_ctx *ctx, mg_graph *g) {
    if (!g) return MG_OK;
    if (ctx) (void)hipStreamSynchronize(ctx->stream);
    (void)hipGraphExecDestroy(g->exec);
    (void)hipGraphDestroy(g->graph);
    delete g;
    return MG_OK;
}

// ---------------------------------------------------------------------------
// mg_gemm_static: the GEMM for callers that cannot allocate.  Its K slices meet in
// a workspace that is part of the library's image on every device instead of a
// hipMalloc'ed one: `scratch` holds MG_STATIC_WS_BYTES of partial tiles followed by
// MG_STATIC_MAX_TILES arrival counters.  In host code that name is a stand-in, not a
// device address: each device's copy is looked up with hipGetSymbolAddress, once per
// device with that device current, and only the pointer it returns is handed to kernels.
// ---------------------------------------------------------------------------
}  // extern "C"

static __device__ __align__(256) unsigned char scratch[MG_STATIC_WS_BYTES + MG_STATIC_MAX_TILES * sizeof(int)];

namespace mg {
struct StaticLane {
    std::atomic<int> ready{0};   // 0: not looked up, 1: ready
    float *ws = nullptr;
    int *cnt = nullptr;
    int cus = 0;
    int lds_limit = 0;
    char arch_ok = 0;
};
static const int MG_MAX_DEVICES = 64;
static StaticLane g_static[MG_MAX_DEVICES];
static std::mutex g_static_mu;

// Looks up this device's copies of the static arrays (with that device current).
static int static_lane(int device, StaticLane **out) {
    if (device < 0 || device >= MG_MAX_DEVICES)
        return fail(MG_ERR_ARG, "mg_gemm_static: device index %d out of range [0, %d)", device, MG_MAX_DEVICES);
    StaticLane &sl = g_static[device];
    if (!sl.ready.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lock(g_static_mu);
        if (!sl.ready.load(std::memory_order_relaxed)) {
            void *ptr = nullptr;
            HIP_TRY(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
            int cus = 0, lds = 0;
            HIP_TRY(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
            HIP_TRY(hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device));
            hipDeviceProp_t prop;
            HIP_TRY(hipGetDeviceProperties(&prop, device));
            sl.arch_ok = strncmp(prop.gcnArchName, "gfx950", 6) == 0;
            sl.ws = (float *)ptr;
            sl.cnt = (int *)((unsigned char *)ptr + MG_STATIC_WS_BYTES);
            sl.cus = cus;
            sl.lds_limit = lds;
            sl.ready.store(1, std::memory_order_release);
        }
    }
    if (!sl.arch_ok) return fail(MG_ERR_NODEVICE, "mg_gemm_static: device %d is not gfx950", device);
    *out = &sl;
    return MG_OK;
}
}  // namespace mg

extern "C" {

// Number of HIP devices, asked once: the count cannot change while the process runs, and the
// question must not be put while a stream of the caller is being captured.
static int static_device_count() {
    static std::atomic<int> cached{-1};
    int n = cached.load(std::memory_order_acquire);
    if (n >= 0) return n;
    if (hipGetDeviceCount(&n) != hipSuccess || n < 0) {
        (void)hipGetLastError();
        return 0;
    }
    cached.store(n, std::memory_order_release);
    return n;
}

static int static_gemm(int device_index, hipStream_t stream, const mg_gemm_args *args, int *dry_count) {
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    if (args->flags & MG_FLAG_SIDE_STREAM)
        return fail(MG_ERR_ARG, "mg_gemm_static: MG_FLAG_SIDE_STREAM belongs to a context; pass the stream itself");
    const int count = static_device_count();
    if (count <= 0) return fail(MG_ERR_NODEVICE, "mg_gemm_static: no HIP device available");
    if (device_index < 0 || device_index >= count)
        return fail(MG_ERR_ARG, "mg_gemm_static: device index %d out of range [0, %d)", device_index, count);
    // the caller's current device is left as it was
    int before = -1;
    HIP_TRY(hipGetDevice(&before));
    if (before != device_index) HIP_TRY(hipSetDevice(device_index));
    struct Restore {
        int dev, now;
        ~Restore() {
            if (dev >= 0 && dev != now) (void)hipSetDevice(dev);
        }
    } restore{before, device_index};
    StaticLane *sl = nullptr;
    rc = static_lane(device_index, &sl);
    if (rc != MG_OK) return rc;
    Lane ln;
    ln.stream = stream;
    ln.ws = sl->ws;
    ln.ws_bytes = MG_STATIC_WS_BYTES;
    ln.cnt = sl->cnt;
    ln.max_tiles = MG_STATIC_MAX_TILES;
    ln.cus = sl->cus;
    ln.lds_limit = sl->lds_limit;
    ln.clear_counters = true;   // the array keeps what the last call left
    ln.dry_count = dry_count;
    Plan pl;
    pick_plan(*args, ln.cus, pl);
    const TileDesc &t = g_tiles[pl.tile];
    // A K split the caller or the picker chose must fit the static workspace (a stream-K tile whose
    // pieces do not fit runs as a plain persistent one, a partial round is cut only if it fits).
    if (pl.split_k > 1 && !(args->flags & MG_FLAG_SPLITK_ATOMIC)) {
        const int64_t tiles = (int64_t)pl.grid_m * pl.grid_n * args->nbatch;
        const int64_t need = tiles * pl.split_k * t.bm * t.bn * (int64_t)sizeof(float);
        if (need > MG_STATIC_WS_BYTES || tiles > MG_STATIC_MAX_TILES)
            return fail(MG_ERR_ARG,
                        "mg_gemm_static: this GEMM's K split needs %lld bytes of partial tiles and %lld tile counters; the "
                        "static workspace holds %lld bytes and %d counters (use mg_gemm, a smaller split_k, or "
                        "MG_FLAG_SPLITK_ATOMIC)",
                        (long long)need, (long long)tiles, (long long)MG_STATIC_WS_BYTES, MG_STATIC_MAX_TILES);
    }
    return enqueue_gemm(ln, args, pl);
}

int mg_gemm_static(int device_index, void *hip_stream, const mg_gemm_args *args) {
    return static_gemm(device_index, (hipStream_t)hip_stream, args, nullptr);
}

int mg_gemm_static_launches(int device_index, const mg_gemm_args *args, int *kernels) {
    if (!kernels) return fail(MG_ERR_ARG, "mg_gemm_static_launches: kernels is NULL");
    *kernels = 0;
    return static_gemm(device_index, nullptr, args, kernels);
}

int mg_launch_count(const mg_gemm_args *args, int compute_units, int64_t workspace_bytes, int64_t counters,
                    int clear_counters, int *kernels) {
    if (!kernels) return fail(MG_ERR_ARG, "mg_launch_count: kernels is NULL");
    *kernels = 0;
    int rc = check_args(args);
    if (rc != MG_OK) return rc;
    if (workspace_bytes < 0 || counters < 0) return fail(MG_ERR_ARG, "mg_launch_count: negative workspace size");
    Lane ln;
    ln.stream = nullptr;
    // any non-null address: a dry run never dereferences it
    ln.ws = workspace_bytes > 0 ? reinterpret_cast<float *>(uintptr_t(256)) : nullptr;
    ln.ws_bytes = workspace_bytes;
    ln.cnt = workspace_bytes > 0 ? reinterpret_cast<int *>(uintptr_t(256)) : nullptr;
    ln.max_tiles = counters;
    ln.cus = compute_units > 0 ? compute_units : 256;
    ln.lds_limit = 160 * 1024;
    ln.clear_counters = clear_counters != 0;
    ln.dry_count = kernels;
    Plan pl;
    pick_plan(*args, ln.cus, pl);
    return enqueue_gemm(ln, args, pl);
}

}  // extern "C"

// ---- shared with elementwise.hip ----
namespace mg {
hipStream_t ctx_stream(mg_ctx *ctx) { return ctx->stream; }
int ctx_fail(int code, const char *msg) { return fail(code, "%s", msg); }
int ctx_hip_fail(hipError_t e, const char *what) { return hip_fail(e, what); }
}  // namespace mg
