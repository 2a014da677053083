/* mi_gemm.h — C ABI of libmigemm.so, the gfx950 (MI355X) training-GEMM library.
 *
 * This is the drop-in boundary for vkgrad's matmul path.  The reference has no
 * FFI of its own for this path (it drives Vulkan through ctypes), so each entry
 * point below names the reference interface it replaces, as file:line under
 * /root/reference/.
 *
 * Conventions
 *   - every function returns int: 0 (MG_OK) on success, an MG_ERR_* code otherwise;
 *     mg_last_error() then holds a message for the calling thread.
 *   - no torch types, no C++ types, no exceptions cross this boundary.
 *   - all device work of a context runs on one in-order HIP stream owned by the
 *     context (the reference separates every dispatch by a full barrier on a
 *     single queue: vk.py:834-851, 1317-1323).  A context is not thread-safe.
 *   - argument validation happens before any HIP call (mg_gemm_check is the same
 *     code mg_gemm runs first), so it can be exercised on a machine without a GPU.
 *   - matrices are dense row-major; leading dimensions are in elements.
 *       A is stored (M,K) [lda >= K], or (K,M) [lda >= M] in layout TN
 *       B is stored (K,N) [ldb >= N], or (N,K) [ldb >= K] in layout NT
 *       C is (M,N) float32 [ldc >= N]                 (kernels.py:42-43)
 *     M, N, K are arbitrary positive integers (no tile-multiple requirement,
 *     unlike kernels.py:265-276); operands need only 2-byte alignment, but
 *     16-byte-aligned bases with ld % 8 == 0 take the fast path.
 */
#ifndef MI_GEMM_H
#define MI_GEMM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct mg_ctx mg_ctx;
typedef struct mg_graph mg_graph;

enum {
    MG_OK = 0,
    MG_ERR_ARG = 1,     /* bad argument; nothing was launched */
    MG_ERR_HIP = 2,     /* a HIP runtime call failed */
    MG_ERR_STATE = 3,   /* call not legal in the current state (graph capture etc.) */
    MG_ERR_NOMEM = 4,
    MG_ERR_NODEVICE = 5
};

/* operand layouts: the (trans_a, trans_b) pairs of kernels.py:32-33.  (T,T) is
 * never used by any call site (autograd.py:186-228, transformer.py:89-104,
 * 326-330, 362-371) and is not provided. */
enum { MG_NN = 0, MG_NT = 1, MG_TN = 2 };
/* input element types; accumulation and C are always float32 */
enum { MG_F16 = 0, MG_BF16 = 1 };
/* memory kinds of vk.py:1161-1175 */
enum { MG_DEVICE = 0, MG_SHARED = 1, MG_CACHED = 2, MG_BAR = 3 };
/* activations for the companion elementwise kernels and the fused GEMM epilogues; the
 * _GRAD forms exist for mg_gemm only (result times the activation's derivative at z) */
enum { MG_TRI_NONE = 0, MG_TRI_C_LOWER = 1, MG_TRI_A_LOWER = 2, MG_TRI_A_UPPER = 3 };
enum { MG_ACT_NONE = 0, MG_ACT_GELU = 1, MG_ACT_RELU = 2, MG_ACT_GELU_GRAD = 3, MG_ACT_RELU_GRAD = 4,
       MG_ACT_SOFTMAX_GRAD = 5 };

typedef struct {
    int32_t struct_size;   /* sizeof(mg_gemm_args), checked */
    int32_t layout;        /* MG_NN / MG_NT / MG_TN */
    int32_t dtype;         /* MG_F16 / MG_BF16 */
    int32_t beta;          /* 0: C is overwritten; 1: C += result (dW accumulation) */
    int64_t m, n, k;
    const void *a;  int64_t lda;
    const void *b;  int64_t ldb;
    float *c;       int64_t ldc;    /* may be NULL when y16 is given and beta == 0 */
    const float *bias;     /* NULL, or N floats added to every row of the result */
    int32_t nbatch;        /* >= 1; batch z uses a + z*sa, b + z*sb, c + z*sc (elements) */
    int32_t tile;          /* tile id from mg_tile_info, or -1 for the built-in picker */
    int64_t sa, sb, sc;
    int32_t split_k;       /* 0 = picker decides, 1 = none, >1 = that many K slices */
    int32_t group_m;       /* 0 = picker decides; else row-blocks per rasterisation band */
    int32_t flags;         /* MG_FLAG_* */
    int32_t act;           /* MG_ACT_*: activation of the 16-bit output y16 (0 without y16) */
    /* Fused forward epilogue — replaces the separate pass of bias_gelu / bias
     * (kernels.py:709-718, 742-749): besides C = result (the pre-activation z the backward
     * pass needs, f32), the epilogue writes y16 = narrow(act(result)) in the input dtype, the
     * operand of the next layer's GEMM.  Layouts NN and NT, nbatch == 1; a K split goes
     * through the workspace (MG_FLAG_SPLITK_ATOMIC is refused). */
    void *y16;             /* NULL, or an (m, n) matrix of 16-bit elements */
    int64_t ldy;           /* its row pitch in elements (>= n) */
    /* Fused backward epilogue — replaces the separate pass of bias_gelu_bwd
     * (kernels.py:720-739; its call site autograd.py:204-207): with act = MG_ACT_GELU_GRAD or
     * MG_ACT_RELU_GRAD the dX GEMM of one layer hands the layer below its dz directly,
     *   g = result * act'(z),   y16 = narrow(g),   C = g (when C is given),
     * where z is that lower layer's pre-activation (m, n) in f32.  beta == 0 and no bias. */
    const float *z;        /* NULL unless act is a _GRAD form */
    int64_t ldz;           /* its row pitch in elements (>= n) */
    /* With a _GRAD activation: NULL, or N floats that receive the column sums of g, the bias
     * gradient of the layer below — col_sum (kernels.py:753-761; autograd.py:215) folded into
     * the same epilogue.  colsum[c] += sum over rows of g[r][c], added with float atomics once
     * per wavefront and column: clear it first unless accumulating over micro-batches; the
     * order of the additions, and so the last bits, vary from run to run. */
    float *colsum;
    /* Residual epilogue — replaces the separate pass of `residual` (tkernels.py:362-371; its
     * call sites transformer.py:216, 223): with beta == 1 and res given,
     *   C = res + result (+ bias),
     * i.e. the accumulation reads another (m, n) f32 matrix than the one it writes (res == c
     * is the plain in-place beta == 1).  nbatch == 1; MG_FLAG_SPLITK_ATOMIC is refused. */
    const float *res;      /* NULL: beta == 1 reads C itself */
    int64_t ldr;           /* row pitch of res in elements (>= n) */
    /* Triangular structure of causal attention (the six per-head GEMMs of transformer.py:144-182
     * with a causal mask, tkernels.py:105-133): work that only meets masked entries is skipped.
     *   MG_TRI_C_LOWER  only c[i][j] with j <= i is needed (scores = Q K^T, dP = dOut V^T, whose
     *                   consumers read keys <= query): tiles wholly above the diagonal are
     *                   neither computed nor written - C keeps its old contents there;
     *   MG_TRI_A_LOWER  op(A)[i][k] == 0 for k > i (P V, dS K): a row block's K loop ends at
     *                   its last row;
     *   MG_TRI_A_UPPER  op(A)[i][k] == 0 for k < i (P^T dOut, dS^T Q with A stored (k, m)): the K
     *                   loop starts at the block's first row.
     * The A forms need m == k; they split K only on request (split_k > 1: a slice wholly outside a row
 * block's range is empty), MG_TRI_C_LOWER never; every batch has the same structure. */
    int32_t tri;           /* MG_TRI_* */
    int32_t reserved;      /* 0 */
    /* Softmax-backward epilogue - replaces the separate pass of attn_softmax_bwd
     * (tkernels.py:167-187; its call site transformer.py:171-176): with act =
     * MG_ACT_SOFTMAX_GRAD the dP = dOut V^T GEMM of attention writes
     *   y16[i][j] = narrow(scale * p16[i][j] * (result[i][j] - rowsub[i]))
     * (and the same value to C in f32 when C is given), where p16 is the 16-bit softmax
     * output P (m, n) and rowsub[i] = sum_j P[i][j] dP[i][j], which the caller obtains without
     * dP as sum_d dOut[i][d] * Out[i][d] (mg_tk_attn_rowdot).  Masked entries need no test of
     * their own: P is zero there.  beta == 0, no bias, layouts NN and NT; batches are allowed:
     * y16 and p16 advance sc elements per batch (they have the shape of C), rowsub m floats. */
    const void *p16;       /* NULL unless act == MG_ACT_SOFTMAX_GRAD */
    int64_t ldp;           /* its row pitch in elements (>= n) */
    const float *rowsub;   /* m floats per batch */
    float scale;
    int32_t reserved2;     /* 0 */
} mg_gemm_args;

/* The buffers of A and B end at their last element: row padding (ld beyond the stored
 * columns) of the LAST row must not be read.  Without this flag, when an extent is not a
 * multiple of 8 but the pitch covers it rounded up to 8, the fast kernels may read (never
 * use) up to 14 bytes of the last row's padding, i.e. buffers must span rows * ld elements. */
#define MG_FLAG_TIGHT_BUFFERS 1
/* With a K split (split_k > 1, or chosen by the picker) the slices normally meet in the
 * context's workspace and are summed in slice order by the slice that finishes last: no
 * clear of C, bit-reproducible.  This flag makes them add into C with float atomics instead
 * (after a clear kernel when beta == 0), which is also what happens when the partial tiles
 * do not fit the workspace; it can be faster when C is large and the split is deep.  A call
 * with this flag uses no workspace at all: the library does not cut a partial last round of
 * tiles into K slices for it either, and a stream-K tile runs as a plain persistent one. */
#define MG_FLAG_SPLITK_ATOMIC 2
/* Run this GEMM on the context's side stream (see mg_side_fork): it overlaps with whatever the
 * main stream runs until mg_side_join.  The side stream has its own half of the split-K
 * workspace, so GEMMs of the two streams never meet there. */
#define MG_FLAG_SIDE_STREAM 4
/* The tiled kernels hand every XCD (8 per chip, an L2 each) a contiguous eighth of the tile
 * order.  Rotated walk: XCD x starts x eighths into its share and wraps around, so that the
 * XCDs do not ask for the same operand panel at the same moment.  That moment costs when the
 * operands are not in the last-level cache - a GEMM inside a training step, whose operands
 * were last touched a whole step ago - because every XCD then fetches the panel from HBM
 * (up to 15 % of a GEMM's time).  In-step walk: all XCDs start at the beginning of their
 * share; with operands resident in that cache it is the faster one by a few percent.
 * Neither flag: the library decides (today: rotated).  Both: MG_ERR_ARG.  Ignored by the
 * persistent, stream-K and skinny tiles and by grids the renumbering does not apply to.
 * No counterpart in the reference (one L2 on its target). */
#define MG_FLAG_XCD_ROTATE 8
#define MG_FLAG_XCD_IN_STEP 16

typedef struct {
    int32_t id;
    int32_t bm, bn, bk;        /* block tile */
    int32_t waves_m, waves_n;  /* 64-lane wavefronts per workgroup along M and N */
    int32_t threads;
    int32_t lds_bytes;         /* for the NT layout; other layouts differ by padding */
    int32_t min_m;             /* informational: smallest M this tile is meant for */
    int32_t stages;            /* 0: register-staged kernel (any alignment); >0: direct-to-LDS ring depth */
    int32_t fallback;          /* tile used instead when this tile's preconditions fail (self: none) */
    int32_t persistent;        /* 1: a grid of resident workgroups loops over the output tiles;
                                * 2: the same, and the tiles beyond the last whole round are cut along K into
                                *    equal pieces, one per workgroup (stream-K; needs the context's workspace,
                                *    without it the tile runs as kind 1) */
    int32_t reserved;
    char name[48];
} mg_tile;

typedef struct {
    char name[128];
    char arch[64];
    int32_t compute_units;
    int32_t clock_khz;
    int32_t mem_clock_khz;
    int32_t mem_bus_bits;
    int32_t l2_bytes;
    int32_t lds_bytes_per_cu;
    int32_t wavefront;
    int32_t reserved;
    int64_t total_mem;
} mg_device_info;

/* ---- runtime: replaces vk.Device / vk.Buffer (vk.py:892-1357, 507-617) ---- */

/* Device() — vk.py:892.  Fails with MG_ERR_NODEVICE when no HIP device exists. */
int mg_init(int device_index, mg_ctx **out);
/* Device.destroy — vk.py:1343 */
int mg_destroy(mg_ctx *ctx);
/* Device.name / shader_core_props — vk.py:1225-1240 */
int mg_get_device_info(mg_ctx *ctx, mg_device_info *out);
/* Device.buffer(size, kind) — vk.py:1251, 507-582.  *host_ptr is the CPU mapping of the
 * same bytes for host-visible kinds (shared/cached/bar -> pinned, device-accessible
 * host memory), NULL for MG_DEVICE. */
int mg_alloc(mg_ctx *ctx, size_t nbytes, int kind, void **dev_ptr, void **host_ptr);
/* Buffer.destroy — vk.py:607-617 */
int mg_free(mg_ctx *ctx, void *dev_ptr, int kind);
/* Device.copy(src, dst, size) — vk.py:1267-1293; any mix of device / host-visible
 * pointers; returns after the copy has completed. */
int mg_copy(mg_ctx *ctx, void *dst, const void *src, size_t nbytes);
/* staged upload/download between ordinary host memory and a buffer */
int mg_upload(mg_ctx *ctx, void *dst_dev, const void *src_host, size_t nbytes);
int mg_download(mg_ctx *ctx, void *dst_host, const void *src_dev, size_t nbytes);
/* fence wait — vk.py:1335; Buffer.flush/invalidate (vk.py:592-605) map to this */
int mg_sync(mg_ctx *ctx);
/* message for the last failing call on this thread — VkError text, vk.py:128-134 */
const char *mg_last_error(void);

/* ---- GEMM: replaces kernels.Matmul (kernels.py:232-315) ---- */

/* Matmul.fits + the argument errors of kernels.py:274-276, vk.py:778-790; pure. */
int mg_gemm_check(const mg_gemm_args *args);
/* Matmul.__call__ — kernels.py:269-297 (eager: enqueue, do not wait). */
int mg_gemm(mg_ctx *ctx, const mg_gemm_args *args);
/* Device.run(kernel, ..., repeat) timing — vk.py:1295-1340, but timed with HIP
 * events on the context's stream instead of host wall clock.  Launches the GEMM
 * `repeat` times back to back, waits, and returns the total seconds. */
int mg_gemm_time(mg_ctx *ctx, const mg_gemm_args *args, int repeat, double *seconds);
/* The same over `nargs` (1..64) argument sets used in turn: launch i runs
 * args[i % nargs].  With operand sets that together exceed the 256 MB last-level
 * cache, every launch finds its operands in HBM, as a training step does; the
 * reference times a shape on one set of buffers (kernels.py:433-447), which on
 * this chip would time small shapes out of cache. */
int mg_gemm_time_rotating(mg_ctx *ctx, const mg_gemm_args *args, int nargs, int repeat, double *seconds);
/* A whole sequence of different GEMMs (1..4096), each behind the previous one on the context's
 * stream with a HIP event between them: seconds_each[i] is the time from the end of GEMM i - 1
 * to the end of GEMM i, i.e. what GEMM i costs inside the sequence, launch gap included.  The
 * reference times dispatches one at a time (Device.run, vk.py:1295-1340) and has no
 * in-sequence timer; this one shows what a training step's order costs each GEMM. */
int mg_gemm_time_each(mg_ctx *ctx, const mg_gemm_args *args, int nargs, double *seconds_each);
/* No counterpart in the reference.  mg_gemm for callers that cannot allocate device memory or
 * create a context: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  Same arguments, kernels and plans as mg_gemm, on device `device_index` and on
 * `hip_stream` (a hipStream_t, NULL for the default stream), which the caller owns and
 * synchronises; the caller's current device is left as it was.  It calls no hipMalloc /
 * hipFree and needs no mg_ctx: the K slices of a split meet in a workspace that is part of the
 * library's image on every device, MG_STATIC_WS_BYTES of partial tiles and MG_STATIC_MAX_TILES
 * arrival counters, which each GPU holds until the process ends.
 *   Results are those of mg_gemm bit for bit whenever both take the same plan, which is always
 * the case for an explicit tile and split_k whose partial tiles fit MG_STATIC_WS_BYTES.  Where
 * the library itself decides to use its workspace - a partial last round of ping-pong tiles cut
 * into K slices, the K pieces of a stream-K tile - that decision depends on what fits, so a
 * shape whose partial tiles need between 32 MiB and the context's workspace is summed in a
 * different order here (same values on integer data, within tolerance otherwise): a stream-K
 * tile then runs as a plain persistent one and the partial round stays uncut.
 *   A K split that the caller or the picker chose and whose partial tiles or counters do not
 * fit is refused with MG_ERR_ARG (nothing is launched); MG_FLAG_SPLITK_ATOMIC, a smaller
 * split_k or mg_gemm are the ways out.  MG_FLAG_SIDE_STREAM is refused.
 *   All calls on one GPU share the one workspace, which keeps what the last call left: the
 * counters a launch uses are cleared by a fill kernel in front of it, and calls that may
 * overlap on a GPU (two streams, two threads) race on it.  Keep them on one stream, or pass
 * MG_FLAG_SPLITK_ATOMIC on every concurrent call but one: with that flag a call touches
 * neither the partial tiles nor the counters (its slices add into C with atomics, a partial
 * round is not cut, a stream-K tile runs plain).
 *   Under stream capture: the first call on a device looks up the workspace address and the
 * device's limits and raises the dynamic-LDS limit of the kernel it launches, which the
 * runtime may refuse while a capture is under way - make one call of the same tile, layout and
 * dtype outside the capture first. */
#define MG_STATIC_WS_BYTES (32ll << 20)
#define MG_STATIC_MAX_TILES 16384
int mg_gemm_static(int device_index, void *hip_stream, const mg_gemm_args *args);
/* How many kernels mg_gemm_static would launch for `args` (GEMM kernels, counter clears, the
 * clear of C before an atomic split); launches nothing. */
int mg_gemm_static_launches(int device_index, const mg_gemm_args *args, int *kernels);
/* The same question without a device, for a lane described by its numbers: CUs, bytes of
 * partial-tile workspace (0: none), arrival counters, and whether counters are cleared in front
 * of a launch (1 for a workspace that persists between calls).  Pure arithmetic. */
int mg_launch_count(const mg_gemm_args *args, int compute_units, int64_t workspace_bytes, int64_t counters,
                    int clear_counters, int *kernels);
/* What the matrix cores sustain with no memory traffic: two wavefronts per SIMD on every CU run
 * `iters` rounds of eight back-to-back v_mfma_f32_32x32x16 from registers.  random_operands = 0
 * multiplies zeros (the chip holds its boost clock), 1 multiplies random 16-bit values (the
 * power-managed clock drops, and with it the rate every real GEMM is bounded by).  Returns the
 * rate and the shader clock during the loop.  workgroups = 0 keeps every CU busy; a smaller
 * positive count keeps that many busy (one workgroup each), which shows how the clock depends on
 * the number of CUs multiplying.  The reference's counterpart is the hand-measured WMMA peak it
 * prices its kernels against (bench/RESULTS.md:113-119, 656-659). */
int mg_probe_mfma(mg_ctx *ctx, int dtype, int random_operands, int iters, int workgroups, double *tflops,
                  double *ghz);
/* What a launch shaped like the skinny-M stream reads from, or writes to, HBM when it does nothing
 * else: `repeat` back-to-back launches over `nsets` rotating buffers of `nbytes` each (enough
 * sets overflow the 256 MB last-level cache), microseconds per launch for the read-only and for
 * the fill-only kernel.  The floor under the memory-bound skinny GEMMs; the counterpart of the
 * reference's read and copy bandwidth probes (bench/roofline.py:27-50). */
int mg_probe_stream(mg_ctx *ctx, int64_t nbytes, int nsets, int repeat, double *read_us, double *fill_us);
/* CONFIGS — kernels.py:326-331: the tile table the tuner walks. */
int mg_tile_count(void);
int mg_tile_info(int id, mg_tile *out);
/* Kernel.statistics() - vk.py:690-736 (driver-reported VGPRs, LDS and scratch of a compiled
 * pipeline) and the inputs of occupancy() - kernels.py:384-411.  Reports, for the kernel the
 * library would launch for `args` (after the picker, the tuned tile/split in args, and every
 * fallback), what the HIP runtime says about that instantiation on the context's device:
 * registers per lane, static and dynamic LDS, scratch (spill) bytes per lane, and how many of its
 * workgroups one CU holds.  `tile` receives the tile that would run.  Launches nothing. */
typedef struct {
    int32_t vgprs;             /* registers per lane (hipFuncAttributes.numRegs) */
    int32_t scratch_bytes;     /* private memory per lane; non-zero means the kernel spills */
    int32_t static_lds_bytes;
    int32_t dynamic_lds_bytes;
    int32_t threads;           /* workgroup size */
    int32_t wgs_per_cu;        /* resident workgroups per CU for this launch shape */
    int32_t waves_per_simd;    /* wgs_per_cu * (threads / 64) / 4 SIMDs, rounded up */
    int32_t max_threads;       /* hipFuncAttributes.maxThreadsPerBlock */
} mg_kernel_stats;
int mg_kernel_stats_for(mg_ctx *ctx, const mg_gemm_args *args, int *tile, mg_kernel_stats *out);
/* The same for one instantiation named directly: tile id, layout (MG_NN..), dtype, and
 * variant 0 (aligned operands / plain epilogue), 1 (any alignment for register-staged tiles,
 * bias epilogue for persistent ones) or 2 (fused activation output).  For the skinny-M tile the
 * variant is 4 * log2(rows of A held) + K class (0: K <= 512, 1: 768, 2: 1024, 3: 2048).
 * MG_ERR_ARG when the table holds no such instantiation. */
int mg_tile_kernel_stats(mg_ctx *ctx, int tile, int layout, int dtype, int variant, mg_kernel_stats *out);
/* Matmul.fits for one tile: 1 if tile `id` can run `args`, else 0. */
int mg_tile_fits(int id, const mg_gemm_args *args);
/* pick_config — autograd.py:22-41: heuristic choice without benchmarking; pure.
 * Writes tile id, split_k and group_m it would use for `args` on a device with
 * `compute_units` CUs. */
int mg_pick(const mg_gemm_args *args, int compute_units, int *tile, int *split_k, int *group_m);

/* ---- a second stream for independent GEMMs ----
 * The reference orders every dispatch of a recorded step behind the previous one with a full
 * compute-to-compute barrier (Graph.record, vk.py:848-851), although the dX and dW products
 * of a linear layer (autograd.py:218-227) do not depend on each other.  Here a context owns a
 * second stream (same, default priority): mg_side_fork makes it wait for everything enqueued
 * on the main stream so far; GEMMs flagged MG_FLAG_SIDE_STREAM then run on it, concurrently
 * with later main-stream work, in their own order; mg_side_join makes the main stream wait for
 * everything enqueued on the side stream so far.  Both work eagerly and while a graph is being
 * recorded (the branches become parallel paths of the graph; mg_graph_end joins if the caller
 * has not).  A flagged GEMM without a preceding fork is an error; mg_sync, copies and mg_free
 * wait for both streams.  Buffers written on one stream must not be touched on the other
 * between fork and join. */
int mg_side_fork(mg_ctx *ctx);
int mg_side_join(mg_ctx *ctx);

/* ---- record / replay: replaces vk.Graph (vk.py:807-889) ---- */

/* Graph.__init__: start capturing the context's stream; launches enqueue nothing
 * until mg_graph_end. */
int mg_graph_begin(mg_ctx *ctx);
/* Graph.finish — vk.py:869-875 */
int mg_graph_end(mg_ctx *ctx, mg_graph **out);
/* Graph.submit — vk.py:877-889: replay and wait; *seconds = host wall time. */
int mg_graph_launch(mg_ctx *ctx, mg_graph *g, double *seconds);
/* Graph.submit without the fence wait (vk.py:1295 `wait=False` is the eager analogue):
 * replay on the context's stream and return; mg_sync waits for it. */
int mg_graph_enqueue(mg_ctx *ctx, mg_graph *g);
/* Replays the graph `repeat` (1..4096) times back to back with a HIP event between
 * replays and waits; seconds_each[i] = device time of replay i.  The reference times a
 * recorded step by host wall clock around submit (vk.py:877-889, bench/ab.py:36-51). */
int mg_graph_time(mg_ctx *ctx, mg_graph *g, int repeat, double *seconds_each);
/* Graph.n_dispatch — vk.py:824, 868, counted where the work is: the kernel launches a recorded
 * graph replays (one library call may record several: a clear in front of an atomic K split, a
 * long-K GEMM whose partial last round runs as a second, split launch). */
int mg_graph_kernel_count(mg_ctx *ctx, mg_graph *g, int *kernels);
int mg_graph_destroy(mg_ctx *ctx, mg_graph *g);

/* ---- companion elementwise kernels: kernels.make_kernels (kernels.py:699-862) ----
 * `dtype` is the 16-bit type of the narrowed outputs / mirrors (MG_F16 or MG_BF16). */

/* bias_gelu / bias (kernels.py:709-718, 742-749): z = acc + bias[i % ncol];
 * y16 = narrow(act(z)).  z and y16 may each be NULL; bias may be NULL (the GEMM's
 * fused bias epilogue already added it). */
int mg_ew_bias_act(mg_ctx *ctx, const float *acc, const float *bias, float *z, void *y16,
                   int64_t n, int64_t ncol, int act, int dtype);
/* bias_gelu_bwd (kernels.py:721-739): g = dy * act'(z); dz16 = narrow(g); dz32 = g (may be NULL). */
int mg_ew_act_bwd(mg_ctx *ctx, const float *dy, const float *z, void *dz16, float *dz32,
                  int64_t n, int act, int dtype);
/* col_sum (kernels.py:753-761): sums[c] = sum_r g[r*ncol + c]; accumulate != 0 adds
 * to the existing sums[c] instead (bias gradients over micro-batches). */
int mg_ew_col_sum(mg_ctx *ctx, const float *g, float *sums, int64_t ncol, int64_t nrow, int accumulate);
/* softmax_ce (kernels.py:766-791): per-row loss, gradient (p - onehot)/nrows in both
 * precisions, classes >= ncls masked to zero. */
int mg_ew_softmax_ce(mg_ctx *ctx, const float *logits, const uint32_t *labels, void *dl16,
                     float *dl32, float *loss, int64_t nrows, int64_t stride, int64_t ncls, int dtype);
/* adamw (kernels.py:832-851): hp = {lr, b1, b2, bc1, bc2, eps} read from memory. */
int mg_ew_adamw(mg_ctx *ctx, float *w, const float *g, float *m, float *v, void *w16,
                const float *hp, int64_t n, float wd, int dtype);
/* zero (kernels.py:853-854) */
/* The same update for a list of parameters in one launch (the reference launches adamw once per
 * parameter, autograd.py:331-343: 148 launches in a GPT-2-small step, most of them a few
 * microseconds of work).  table_dev: `ntensors` entries in device memory, ordered, first_block =
 * the sum of ceil(n / 1024) over the entries before; total_blocks = that sum over all entries.
 * vec != 0 promises that w, g, m, v are 16-byte and w16 8-byte aligned. */
typedef struct {
    float *w; const float *g; float *m; float *v; void *w16;
    int64_t n;
    int64_t first_block;
    float wd;
    int32_t vec;
} mg_adamw_entry;
int mg_ew_adamw_multi(mg_ctx *ctx, const mg_adamw_entry *table_dev, int ntensors, int64_t total_blocks, const float *hp,
                      int dtype);
/* g[0 .. n) = 0 for every entry of such a table (only g, n and first_block are read), in one launch:
 * the clears in front of the bias and LayerNorm gradient sums of a step (col_sum_zero,
 * tkernels.py:238-246, once per sum in the reference), gathered at the start of its backward pass. */
int mg_ew_zero_multi(mg_ctx *ctx, const mg_adamw_entry *table_dev, int ntensors, int64_t total_blocks);
int mg_ew_zero(mg_ctx *ctx, float *dst, int64_t n);
/* Device-side copy of nbytes (multiple of 4, both pointers 4-byte aligned) that can be
 * recorded into a graph, unlike mg_copy.  The reference's recorded step reads what the CPU
 * wrote into mapped buffers directly (inputs, labels, the optimiser's per-step scalars:
 * vk.py:583-590, autograd.py:313-329); on a discrete card every such read crosses PCIe, so a
 * recorded step stages them into HBM with this kernel first. */
int mg_ew_copy(mg_ctx *ctx, void *dst, const void *src, int64_t nbytes);
/* cast16 (kernels.py:857-860) */
int mg_ew_cast16(mg_ctx *ctx, const float *src, void *dst, int64_t n, int dtype);
/* Scratch operands for warm-up and tuning (kernels.py:367-375, 472-474 use uninitialised
 * memory): n 16-bit values, pseudo-random in [-1, 1), reproducible from `seed`. */
int mg_ew_fill_uniform16(mg_ctx *ctx, void *dst, int64_t n, uint32_t seed, int dtype);
/* grad_add (dataparallel.py:54-58): dst[i] += src[i] */
int mg_ew_grad_add(mg_ctx *ctx, float *dst, const float *src, int64_t n);
/* grad_pull (dataparallel.py:69-73): dst[i] = src[i] * scale - the summed gradient of several
 * micro-batches read back out of the accumulator as a mean */
int mg_ew_scale_copy(mg_ctx *ctx, float *dst, const float *src, int64_t n, float scale);

/* ---- Row kernels of the decoder block (tkernels.py), all in f32 with 16-bit outputs where the
 * next GEMM reads them.  `dtype` is the 16-bit type.  Head-side tensors are (B*H, T, hd),
 * row-side tensors (B*T, D) with D = H * hd; n counts the elements of the (B*T, D) side. */
/* layernorm (tkernels.py:32-56): y16 = narrow((x - mu) * rstd * gamma + beta), eps 1e-5 inside
 * the root; mu and rstd (one per row) are kept for the backward pass. */
int mg_tk_layernorm(mg_ctx *ctx, const float *x, const float *gamma, const float *beta, void *y16, float *mu,
                    float *rstd, int64_t rows, int64_t D, int dtype);
/* layernorm_bwd (tkernels.py:58-92): dx, plus dy * xhat and dy in 16 bits (the column sums of
 * those two are dgamma and dbeta, transformer.py:66-73). */
int mg_tk_layernorm_bwd(mg_ctx *ctx, const float *dy, const float *x, const float *gamma, const float *mu,
                        const float *rstd, float *dx, void *dyxh16, void *dy16, int64_t rows, int64_t D, int dtype);
/* attn_softmax / attn_softmax_doc (tkernels.py:105-165): rows = B*H*T rows of T scores; row r is
 * query r % T and sees keys first..query, first = 0 or seg[(r / T / H) * T + query]; scale, max
 * subtraction and normalisation in one kernel, masked keys get 0. */
int mg_tk_attn_softmax(mg_ctx *ctx, const float *s, const uint32_t *seg, void *p16, int64_t rows, int64_t T, int64_t H,
                       float scale, int dtype);
/* attn_softmax_bwd (tkernels.py:167-187): ds16 = narrow(P * (dP - sum_j dP_j P_j) * scale) */
int mg_tk_attn_softmax_bwd(mg_ctx *ctx, const float *dp, const void *p16, void *ds16, int64_t rows, int64_t T,
                           float scale, int dtype);
/* out[r] = sum_d a16[r][d] * b32[r][d] over `rows` rows of D elements.  With a16 = dOut and
 * b32 = Out (head-side) this is the row term sum_j P_j dP_j of attn_softmax_bwd
 * (tkernels.py:167-187), formed without P or dP: the `rowsub` of MG_ACT_SOFTMAX_GRAD. */
int mg_tk_attn_rowdot(mg_ctx *ctx, const void *a16, const float *b32, float *out, int64_t rows, int64_t D, int dtype);
/* P of attention in one kernel: the scores = Q K^T product over the heads (transformer.py:153-155)
 * and attn_softmax / attn_softmax_doc (tkernels.py:105-165) after it, without the f32 scores in
 * between: p16[b][i][j] = softmax over the seen keys j of scale * sum_d q16[b][i][d] * k16[b][j][d],
 * 0 for the others.  Query i of head b sees keys first .. i, first = 0 (seg NULL) or
 * seg[(b / H) * T + i].  nbh heads (a multiple of H) of T x T, head width hd in {32, 64, 128}, T a
 * multiple of 8, and at most 1024 for hd = 128 (mg_tk_attn_p_supported; other sizes take the GEMM
 * and mg_tk_attn_softmax).  All three tensors 16-byte aligned.  causal != 0: blocks of 32 queries x
 * 256 keys wholly beyond the diagonal are not written - keep p16 zero there. */
int mg_tk_attn_p_supported(int64_t hd, int64_t T);
int mg_tk_attn_p(mg_ctx *ctx, const void *q16, const void *k16, const uint32_t *seg, void *p16, int64_t nbh, int64_t T,
                 int64_t H, int64_t hd, float scale, int causal, int dtype);
/* Attention forward in one kernel: mg_tk_attn_p and the Out = P V product over the heads after it
 * (transformer.py:153-159; attn_softmax / attn_softmax_doc tkernels.py:105-165), so that P is written
 * (the backward pass reads it) but not read back: p16 as from mg_tk_attn_p, and
 *   out32[b][i][d] = sum_j p16[b][i][j] * v16[b][j][d]      (nbh, T, hd) f32, head-side,
 * the 16-bit P as stored times V with f32 sums (a GEMM over the stored P gives the same up to the
 * order of the sums).  out16 (or NULL): the same values narrowed, in the merged (B*T, H*hd) layout
 * of merge_heads (tkernels.py:274-286).  hd in {32, 64, 128}, T a multiple of 8 up to 1024
 * (mg_tk_attn_fwd_supported); q16, k16, v16 (nbh, T, hd) and p16 16-byte aligned.  causal != 0:
 * blocks of 32 queries x 256 keys wholly beyond the diagonal are not written - keep p16 zero there. */
int mg_tk_attn_fwd_supported(int64_t hd, int64_t T);
int mg_tk_attn_fwd(mg_ctx *ctx, const void *q16, const void *k16, const void *v16, const uint32_t *seg, void *p16,
                   float *out32, void *out16, int64_t nbh, int64_t T, int64_t H, int64_t hd, float scale, int causal,
                   int dtype);
/* dS of attention in one kernel: the dP = dOut V^T product over the heads (transformer.py:171-173)
 * and attn_softmax_bwd (tkernels.py:167-187) after it, without the f32 dP in between:
 *   ds16[b][i][j] = narrow(scale * p16[b][i][j] * (sum_d dout16[b][i][d] * v16[b][j][d] - rowsub[b][i]))
 * for nbh heads of T x T, head width hd in {32, 64, 128} and T a multiple of 8 (mg_tk_attn_ds_supported; other
 * sizes take mg_gemm with MG_ACT_SOFTMAX_GRAD).  dout16 and v16 are (nbh, T, hd), 16-byte aligned,
 * as are p16 and ds16; rowsub
 * from mg_tk_attn_rowdot.  causal != 0: blocks of 32 queries x 256 keys wholly beyond the diagonal
 * are neither computed nor written - keep ds16 zero there. */
int mg_tk_attn_ds_supported(int64_t hd, int64_t T);
int mg_tk_attn_ds(mg_ctx *ctx, const void *dout16, const void *v16, const void *p16, const float *rowsub, void *ds16,
                  int64_t nbh, int64_t T, int64_t hd, float scale, int causal, int dtype);
/* split_qkv (tkernels.py:195-213): (B*T, 3D) f32 + bias[3D] (or NULL) -> q16, k16, v16 head-side */
int mg_tk_split_qkv(mg_ctx *ctx, const float *qkv, const float *bias, void *q16, void *k16, void *v16, int64_t n,
                    int64_t D, int64_t T, int64_t H, int64_t hd, int dtype);
/* merge_qkv_grad (tkernels.py:215-231): head-side dq, dk, dv f32 -> (B*T, 3D) 16-bit */
int mg_tk_merge_qkv_grad(mg_ctx *ctx, const float *dq, const float *dk, const float *dv, void *dqkv16, int64_t n,
                         int64_t D, int64_t T, int64_t H, int64_t hd, int dtype);
/* merge_heads (tkernels.py:274-286): head-side f32 -> (B*T, D) 16-bit */
int mg_tk_merge_heads(mg_ctx *ctx, const float *src, void *y16, int64_t n, int64_t D, int64_t T, int64_t H, int64_t hd,
                      int dtype);
/* split_heads (tkernels.py:288-300): (B*T, D) f32 -> head-side 16-bit */
int mg_tk_split_heads(mg_ctx *ctx, const float *src, void *dst16, int64_t n, int64_t D, int64_t T, int64_t H,
                      int64_t hd, int dtype);
/* embed / embed_doc (tkernels.py:303-315, 334-345): x[bt, d] = tok[ids[bt], d] + pos[t, d],
 * t = bt % T, minus seg[bt] when seg is given (positions restart at each packed sample). */
int mg_tk_embed(mg_ctx *ctx, const float *tok, const float *pos, const uint32_t *ids, const uint32_t *seg, float *x,
                int64_t n, int64_t D, int64_t T);
/* embed_bwd / embed_doc_bwd (tkernels.py:317-332, 347-360): scatter-add of dx into dtok and dpos
 * with float atomics; the caller clears (or has a GEMM overwrite) both first. */
int mg_tk_embed_bwd(mg_ctx *ctx, const float *dx, const uint32_t *ids, const uint32_t *seg, float *dtok, float *dpos,
                    int64_t n, int64_t D, int64_t T);
/* residual (tkernels.py:362-371): out = res + acc + bias[i % D] — the separate-pass form of
 * mg_gemm_args.res */
int mg_tk_residual(mg_ctx *ctx, const float *acc, const float *bias, const float *res, float *out, int64_t n,
                   int64_t D);
/* add (tkernels.py:373-377) and add_bias (in place, tkernels.py:379-382) */
int mg_tk_add(mg_ctx *ctx, const float *a, const float *b, float *out, int64_t n);
/* out = a + b together with out16 = narrow(out): `add` followed by `to16` of the sum
 * (transformer.py:242-252, tkernels.py:372-389) in one pass. */
int mg_tk_add16(mg_ctx *ctx, const float *a, const float *b, float *out, void *out16, int64_t n, int dtype);
int mg_tk_add_bias(mg_ctx *ctx, float *x, const float *bias, int64_t n, int64_t ncol);
/* col_sum_zero + col_sum_chunk16 (tkernels.py:238-270; transformer.py:30-37): column sums of a
 * 16-bit (nrow, ncol) matrix, f32 accumulation; accumulate != 0 adds to sums. */
int mg_tk_col_sum16(mg_ctx *ctx, const void *g16, float *sums, int64_t ncol, int64_t nrow, int accumulate, int dtype);
/* softmax_ce / softmax_ce_w (kernels.py:766-823) for wide rows (the LM head): one workgroup per
 * row.  weights NULL: gradient scaled by 1 / nrows; else by weights[row], rows of weight 0 get
 * zeros and loss 0.  dl16 or dl32 may be NULL. */
int mg_tk_softmax_ce(mg_ctx *ctx, const float *logits, const uint32_t *labels, const float *weights, void *dl16,
                     float *dl32, float *loss, int64_t nrows, int64_t stride, int64_t ncls, int dtype);

#ifdef __cplusplus
}
#endif
#endif /* MI_GEMM_H */
