// MFMA GEMM kernel template for gfx950: C[M,N] (f32) = op(A) op(B) (+bias) (+C).
//
// One template covers the three operand layouts of the training path
// (reference: kernels.py:32-138 generates one GLSL body per (trans_a, trans_b)):
//   NN  A (M,K) K-contiguous,  B (K,N) N-contiguous
//   NT  A (M,K) K-contiguous,  B (N,K) K-contiguous
//   TN  A (K,M) M-contiguous,  B (K,N) N-contiguous
// A K-contiguous operand is staged in LDS as [row][BK+8] and read back with one
// 16-byte ds_read per MFMA fragment.  An operand whose contiguous axis is M or N
// is staged untransposed as [k][B?+32] and transposed on the way out of LDS by
// ds_read_b64_tr_b16, so no transposed copy ever exists in memory (the reference
// makes the same point about coopMatLoad layouts, kernels.py:45-48).
//
// Each wavefront owns a (BM/WGM) x (BN/WGN) block of 32x32 v_mfma_f32_32x32x16
// accumulators.  Global loads for K-block t+1 are issued into registers before
// the MFMAs of block t and written to the other LDS stage afterwards, so there
// is one workgroup barrier per K-block.
#pragma once
#include <atomic>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mg {

enum { L_NN = 0, L_NT = 1, L_TN = 2 };
enum { D_F16 = 0, D_BF16 = 1 };

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
// 16 bytes with only 2-byte alignment promised: the hardware's unaligned access
// mode serves these as a single dwordx4 load.
typedef u32x4 __attribute__((aligned(2))) u32x4_u;

struct GemmParams {
    const uint16_t *A;
    const uint16_t *B;
    float *C;
    const float *bias;
    int64_t lda, ldb, ldc;
    int64_t sa, sb, sc;   // batch strides in elements
    int M, N, K;
    int beta;             // 1: read C and add
    int grid_m, grid_n;   // tiles along M and N
    int group_m;          // rasterisation band height in tiles (>= 1)
    int split_k;          // number of K slices (gridDim.y)
    int k_per_split;      // K elements per slice, a multiple of BK
    int xcd_remap;        // 1: renumber workgroups so neighbours share an XCD; 2: and rotate each XCD's walk
    float *ws;            // split-K workspace (split_k * tiles * BM * BN floats) or null: add with atomics
    int *cnt;             // one arrival counter per tile, zero between launches
    // Staggered start (ping-pong kernel): the first stagger_blocks workgroups - the ones resident
    // at once - nap phase / 8 of stagger_clk clocks before they begin, so that the C stores of
    // a round of short-K tiles do not reach memory in one burst.  0: off.
    int stagger_clk, stagger_blocks;
    int stream_k;         // stream-K kernel only: cut the tiles of the last, partial round along K
    // stream-K partition, computed by the host for the launched grid: whole rounds of tiles,
    // tiles left over after them, and the number of equal K pieces each of those is cut into
    // (sk_rem_tiles * sk_pieces <= gridDim.x workgroups take one piece each)
    int sk_full_rounds, sk_rem_tiles, sk_pieces;
    // fused activation output (kernels instantiated with ACT only): Y = narrow(act(result))
    // in the input dtype; C (the pre-activation result) may then be null
    uint16_t *Y;
    int64_t ldy;
    int act;              // MG_ACT_*
    const float *Z;       // pre-activation for the _GRAD activations
    int64_t ldz;
    float *colsum;        // column sums of the _GRAD result are added here (or NULL)
    const float *R;       // beta = 1 reads this matrix instead of C (or NULL)
    int64_t ldr;
    int tri;              // MG_TRI_*: causal structure (non-persistent kernels only)
    // MG_ACT_SOFTMAX_GRAD: Y = narrow(scale * P16 * (result - rowsub[row])); Y and P16 advance
    // sy elements per batch, rowsub M floats
    const uint16_t *P16;
    int64_t ldp;
    const float *rowsub;
    float scale;
    int64_t sy;
};

template <int DT>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
    if constexpr (DT == D_F16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a),
                                                      __builtin_bit_cast(half8, b), c, 0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a),
                                                       __builtin_bit_cast(bf8, b), c, 0, 0, 0);
    }
}

typedef __attribute__((address_space(3))) short4v lds_short4;

// Transposing LDS read: within each group of 16 lanes the 16 x 8-byte pieces
// addressed by the lanes form a 4 x 16 matrix of 16-bit elements (lane j supplies
// row j/4, columns 4*(j%4)..+3); lane j receives column j.
__device__ __forceinline__ u32x2 lds_read_tr(const uint16_t *p) {
    short4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4 *)p);
    return __builtin_bit_cast(u32x2, v);
}

// Workgroup -> output tile.  Consecutive hardware workgroup ids land on
// different XCDs (8 per chip, one L2 each); renumbering them XCD-major keeps
// tiles that share operand panels behind one L2: XCD x takes the x-th eighth of
// the tile order (the first total % 8 XCDs one tile more).  Inside that order,
// bands of `group_m` row-blocks are walked column by column (the reference's
// grouped rasterisation, kernels.py:72-94).
//
// xcd_remap == 2 also rotates every XCD's walk: XCD x starts x eighths into its
// own run of tiles and wraps around.  Without it the eight XCDs walk their bands
// in step and ask for the same panel of the shared operand at the same moment;
// when that panel is not in the last-level cache each of them fetches it from
// HBM (8192 x 50257 x 768 after kernels that left nothing of its operands in
// cache: 717 us in step, 628 us rotated; with the operands in cache 590 / 620).
__device__ __forceinline__ void tile_coords(const GemmParams &p, int &pid_m, int &pid_n) {
    int pid = blockIdx.x;
    const int total = p.grid_m * p.grid_n;
    if (p.xcd_remap) {
        constexpr int NXCD = 8;
        const int q = total / NXCD, r = total % NXCD;
        const int xcd = pid % NXCD;
        int local = pid / NXCD;
        const int count = q + (xcd < r ? 1 : 0);
        if (p.xcd_remap == 2) {
            local += (int)(((int64_t)count * xcd) / NXCD);
            if (local >= count) local -= count;
        }
        pid = xcd * q + min(xcd, r) + local;
    }
    const int in_group = p.group_m * p.grid_n;
    const int gid = pid / in_group;
    const int first_m = gid * p.group_m;
    const int gsize = min(p.grid_m - first_m, p.group_m);
    const int r = pid % in_group;
    pid_m = first_m + r % gsize;
    pid_n = r / gsize;
}

// ---------------------------------------------------------------------------
// Operand staging.  KC = K-contiguous in memory.
//   KC:   tile is ROWS x BK,  LDS [ROWS][BK+8],  chunk = 8 consecutive k
//   !KC:  tile is BK x ROWS,  LDS [BK][ROWS+32], chunk = 8 consecutive rows (m or n)
// GENERAL=false promises: base 16-byte aligned, ld % 8 == 0, and the contiguous
// extent (K for KC, the row count otherwise) a multiple of 8, so a chunk is
// either entirely inside the matrix or entirely outside.
// ---------------------------------------------------------------------------
template <bool KC, int ROWS, int BK, int NTHREADS, bool GENERAL>
struct Stage {
    static constexpr int PITCH = KC ? (BK + 8) : (ROWS + 32);
    static constexpr int ELEMS = KC ? ROWS * PITCH : BK * PITCH;
    static constexpr int CPR = KC ? BK / 8 : ROWS / 8;        // chunks per LDS row
    static constexpr int NCHUNK = ROWS * BK / 8;
    static constexpr int PER = (NCHUNK + NTHREADS - 1) / NTHREADS;
    static constexpr int RSTEP = NTHREADS / CPR;              // LDS rows between a thread's chunks
    static_assert(NCHUNK % NTHREADS == 0 && NTHREADS % CPR == 0, "tile/threads mismatch");

    u32x4 reg[PER];

    // Unconditional loads for a K-block that lies entirely inside the matrix in
    // both directions.  `tile` points at the block's first element (uniform over
    // the workgroup); a thread's chunks are RSTEP*ld apart.
    __device__ __forceinline__ void load_fast(const uint16_t *tile, int64_t ld, int tid) {
        const uint16_t *src = tile + (int64_t)(tid / CPR) * ld + (tid % CPR) * 8;
        const int64_t step = (int64_t)RSTEP * ld;
#pragma unroll
        for (int i = 0; i < PER; i++) {
            if constexpr (GENERAL) reg[i] = *(const u32x4_u *)(src + i * step);
            else reg[i] = *(const u32x4 *)(src + i * step);
        }
    }

    // row0: first row (m or n) of the tile; nrows: matrix extent along that axis;
    // k0: first k of this block; kend: one past the last valid k for this slice.
    __device__ __forceinline__ void load(const uint16_t *base, int64_t ld, int row0, int nrows,
                                         int k0, int kend, int tid) {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int c = tid + i * NTHREADS;
            u32x4 v = {0u, 0u, 0u, 0u};
            {
                if constexpr (KC) {
                    const int r = c / CPR, kc = (c % CPR) * 8;
                    const int row = min(row0 + r, nrows - 1);   // clamp: feeds masked outputs only
                    const int k = k0 + kc;
                    const uint16_t *src = base + (int64_t)row * ld + k;
                    if constexpr (!GENERAL) {
                        if (k < kend) v = *(const u32x4 *)src;
                    } else {
                        if (k + 8 <= kend) {
                            v = *(const u32x4_u *)src;
                        } else if (k < kend) {
                            uint16_t e[8];
#pragma unroll
                            for (int j = 0; j < 8; j++) e[j] = (k + j < kend) ? src[j] : (uint16_t)0;
                            v = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                                      (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
                        }
                    }
                } else {
                    const int kr = c / CPR, rc = (c % CPR) * 8;
                    const int k = k0 + kr;
                    const int row = row0 + rc;
                    const uint16_t *src = base + (int64_t)k * ld + row;
                    if constexpr (!GENERAL) {
                        if (k < kend && row < nrows) v = *(const u32x4 *)src;
                    } else {
                        if (k < kend) {
                            if (row + 8 <= nrows) {
                                v = *(const u32x4_u *)src;
                            } else if (row < nrows) {
                                uint16_t e[8];
#pragma unroll
                                for (int j = 0; j < 8; j++) e[j] = (row + j < nrows) ? src[j] : (uint16_t)0;
                                v = u32x4{(uint32_t)e[0] | ((uint32_t)e[1] << 16), (uint32_t)e[2] | ((uint32_t)e[3] << 16),
                                          (uint32_t)e[4] | ((uint32_t)e[5] << 16), (uint32_t)e[6] | ((uint32_t)e[7] << 16)};
                            }
                        }
                    }
                }
            }
            reg[i] = v;
        }
    }

    __device__ __forceinline__ void store(uint16_t *lds, int tid) const {
#pragma unroll
        for (int i = 0; i < PER; i++) {
            const int c = tid + i * NTHREADS;
            {
                const int r = c / CPR, off = (c % CPR) * 8;
                *(u32x4 *)(lds + r * PITCH + off) = reg[i];
            }
        }
    }

    // One 32-row x 16-k MFMA operand fragment: lane l gets row (l % 32),
    // k = kk*16 + 8*(l/32) .. +7 of the staged tile.
    static __device__ __forceinline__ u32x4 frag(const uint16_t *lds, int row_base, int kk, int lane) {
        if constexpr (KC) {
            const int row = row_base + (lane & 31);
            const int k = kk * 16 + (lane >> 5) * 8;
            return *(const u32x4 *)(lds + row * PITCH + k);
        } else {
            const int j = lane & 15, g = lane >> 4;
            const int k = kk * 16 + (g >> 1) * 8 + (j >> 2);
            const int row = row_base + (g & 1) * 16 + (j & 3) * 4;
            const uint16_t *p = lds + k * PITCH + row;
            const u32x2 lo = lds_read_tr(p);
            const u32x2 hi = lds_read_tr(p + 4 * PITCH);
            return u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    }
};

template <int LAYOUT, int BM, int BN, int BK, int WGM, int WGN>
struct TileTraits {
    static constexpr bool A_KC = (LAYOUT != L_TN);
    static constexpr bool B_KC = (LAYOUT == L_NT);
    static constexpr int NTHREADS = WGM * WGN * 64;
    using SA = Stage<A_KC, BM, BK, NTHREADS, false>;
    using SB = Stage<B_KC, BN, BK, NTHREADS, false>;
    static constexpr int STAGE_ELEMS = SA::ELEMS + SB::ELEMS;
    static constexpr int LDS_BYTES = 2 * STAGE_ELEMS * 2;
};

template <int N>
struct IntC {
    static constexpr int value = N;
};

// ---------------------------------------------------------------------------
// Split-K through a workspace.  Every K slice of a tile stores its partial
// accumulators, then counts itself in; the slice that arrives last sums all the
// partials in slice order and goes on to write the tile.  Nobody waits for
// anybody, the sum order is fixed (so results are bit-reproducible from run to
// run), C needs no clearing beforehand, and bias and beta are applied once, by
// the writer.
//
// Visibility between workgroups (which may sit behind different L2s) comes from
// device-scope accesses: the partials are written and read with relaxed
// device-scope atomics, which go through to the coherence point and never leave
// a stale or dirty line in a private cache, and a slice counts itself in only
// after its stores have completed (vmcnt 0).  That avoids device-scope fences,
// which write back and invalidate a whole L2 under the workgroups still
// streaming their operands through it.
//
// Returns true in the workgroup that has to write the tile; its acc then holds
// the complete sum.  slot_of(s) names the workspace slot (in partial tiles) of
// slice s; `flag` points at one int of LDS nobody else is using.
// ---------------------------------------------------------------------------
template <int TM, int TN, int NTHREADS, class SlotOf>
__device__ __forceinline__ bool splitk_gather(f32x16 (&acc)[TM][TN], float *ws, int *counter, int slice, int nslices,
                                              SlotOf slot_of, int tid, int *flag) {
    constexpr int64_t TILE_FLOATS = (int64_t)TM * TN * 16 * NTHREADS;
    float *mine = ws + slot_of(slice) * TILE_FLOATS + tid;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                __hip_atomic_store(mine + (int64_t)((i * TN + j) * 16 + r) * NTHREADS, acc[i][j][r], __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's partials have reached the coherence point
    __syncthreads();
    if (tid == 0) {
        const int old = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = (old == nslices - 1);
    }
    __syncthreads();
    const bool last = *flag != 0;
    __syncthreads();      // flag may be reused (persistent kernel) once everyone has read it
    if (!last) return false;
    if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // ready for the next launch
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    for (int sl = 0; sl < nslices; sl++) {
        const float *src = ws + slot_of(sl) * TILE_FLOATS + tid;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            // a row of tiles is fetched as one batch of independent loads, then added
            float part[TN][16];
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++)
                    part[j][r] = __hip_atomic_load(src + (int64_t)((i * TN + j) * 16 + r) * NTHREADS, __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] += part[j][r];
        }
    }
    return true;
}

// Pin the instruction mix of one MFMA group for the backend scheduler: the
// group's LDS reads, LDS writes and global loads are spread evenly between its
// MFMAs instead of being issued in a burst in front of them.
template <int I, int NMFMA, int NDSR, int NDSW, int NVMEM>
__device__ __forceinline__ void interleave_step() {
    if constexpr (I < NMFMA) {
        constexpr int r = (I + 1) * NDSR / NMFMA - I * NDSR / NMFMA;
        constexpr int w = (I + 1) * NDSW / NMFMA - I * NDSW / NMFMA;
        constexpr int v = (I + 1) * NVMEM / NMFMA - I * NVMEM / NMFMA;
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
        if constexpr (r > 0) __builtin_amdgcn_sched_group_barrier(0x100, r, 0);   // LDS reads
        if constexpr (w > 0) __builtin_amdgcn_sched_group_barrier(0x200, w, 0);   // LDS writes
        if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x020, v, 0);   // global loads
        interleave_step<I + 1, NMFMA, NDSR, NDSW, NVMEM>();
    }
}
template <int NMFMA, int NDSR, int NDSW, int NVMEM>
__device__ __forceinline__ void interleave_group() {
    interleave_step<0, NMFMA, NDSR, NDSW, NVMEM>();
}

// K range of a row block when op(A) is triangular (M == K): rows m0 .. m0 + BM - 1 meet non-zero
// entries of op(A) only for k <= m0 + BM - 1 (lower) or k >= m0 (upper).  With a K split a
// slice may lie wholly outside that range: it comes back empty (kend == kbeg).
template <int BM, int BK>
__device__ __forceinline__ void tri_k_range(int tri, int m0, int &kbeg, int &kend) {
    if (tri == 2) kend = min(kend, m0 + BM);
    if (tri == 3) kbeg = max(kbeg, (m0 / BK) * BK);
    if (kend < kbeg) kend = kbeg;
}

// 16-bit narrowing (round to nearest even) and the activations of the fused output;
// same formulas as the companion kernels (reference kernels.py:625-629, 709-718).
template <int DT>
__device__ __forceinline__ float widen16_of(uint16_t b) {
    if constexpr (DT == D_F16) return (float)__builtin_bit_cast(_Float16, b);
    else return __builtin_bit_cast(float, (uint32_t)b << 16);
}
template <int DT>
__device__ __forceinline__ uint16_t narrow16_rne(float x) {
    if constexpr (DT == D_F16) {
        return __builtin_bit_cast(uint16_t, (_Float16)x);
    } else {
        uint32_t u = __builtin_bit_cast(uint32_t, x);
        if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
        u += 0x7fffu + ((u >> 16) & 1u);
        return (uint16_t)(u >> 16);
    }
}
__device__ __forceinline__ float fused_act(float x, int act) {
    if (act == 2) return fmaxf(x, 0.f);                  // MG_ACT_RELU
    if (act == 1) {
        // MG_ACT_GELU, tanh form: 0.5 x (1 + tanh u) = x / (1 + exp(-2u)), u = c (x + 0.044715 x^3);
        // one hardware exponential and one reciprocal instead of the library tanh (the
        // result is narrowed to 16 bits, far coarser than either)
        const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
        return x * __frcp_rn(1.0f + __expf(-2.0f * u));
    }
    return x;   // none, and the _GRAD forms (their factor is applied before)
}
// derivative of the activation at pre-activation x, for MG_ACT_GELU_GRAD (3) / MG_ACT_RELU_GRAD (4)
// (reference kernels.py:630-635).  With s = 1 / (1 + exp(-2u)) = (1 + tanh u) / 2:
//   gelu'(x) = s + x * 2 s (1 - s) * c (1 + 3 * 0.044715 x^2)
__device__ __forceinline__ float fused_dact(float x, int act) {
    if (act == 4) return x > 0.f ? 1.f : 0.f;
    const float c = 0.7978845608028654f;
    const float u = c * (x + 0.044715f * x * x * x);
    const float s = __frcp_rn(1.0f + __expf(-2.0f * u));
    return s + x * (2.0f * s * (1.0f - s)) * (c * (1.0f + 0.134145f * x * x));
}

// Writes one workgroup tile from the accumulators.  Accumulator register r of lane l holds
//   row (r/4)*8 + (l/32)*4 + r%4,  column l%32   of its 32x32 tile,
// so one store instruction writes two full 128-byte row segments.  mode: 0 overwrite,
// 1 C += (read, add, store), 2 atomic +=; the mode and the edge test are uniform over the
// workgroup and hoisted out of the element loops.  ACT: additionally Y = narrow(act(result))
// (modes 0 and 1 only), and C is optional; with a _GRAD activation (mode 0 only) the result
// is first multiplied by act'(Z) and goes to both outputs that way.
template <int DT, int TM, int TN, int WTM, int WTN, bool ACT>
__device__ __forceinline__ void store_tile(const GemmParams &p, float *C, f32x16 (&acc)[TM][TN], int m0, int n0,
                                           int wave_m, int wave_n, int lane, bool add_bias, int mode,
                                           bool interior) {
    const int row_l = m0 + wave_m * WTM + (lane >> 5) * 4;
    const int col_l = n0 + wave_n * WTN + (lane & 31);
    float *cl = C + (int64_t)row_l * p.ldc + col_l;
    const int64_t ldc = p.ldc;
    uint16_t *yl = ACT ? p.Y + (int64_t)blockIdx.z * p.sy + (int64_t)row_l * p.ldy + col_l : nullptr;
    const int64_t ldy = ACT ? p.ldy : 0;
    const bool have_c = !ACT || p.C != nullptr;   // (C carries the batch offset: test the argument)
    const bool grad = ACT && (p.act == 3 || p.act == 4);
    const bool sgrad = ACT && p.act == 5;   // MG_ACT_SOFTMAX_GRAD
    const uint16_t *pl = sgrad ? p.P16 + (int64_t)blockIdx.z * p.sy + (int64_t)row_l * p.ldp + col_l : nullptr;
    const int64_t ldp = sgrad ? p.ldp : 0;
    const float *rsl = sgrad ? p.rowsub + (int64_t)blockIdx.z * p.M + row_l : nullptr;
    // what beta = 1 adds to: C itself, or the residual matrix
    const float *rl = p.R ? p.R + (int64_t)row_l * p.ldr + col_l : cl;
    const int64_t ldr = p.R ? p.ldr : ldc;
    const float *zl = grad ? p.Z + (int64_t)row_l * p.ldz + col_l : nullptr;
    const int64_t ldz = grad ? p.ldz : 0;
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) bv[j] = (add_bias && col_l + j * 32 < p.N) ? p.bias[col_l + j * 32] : 0.f;

    auto write_out = [&](auto mode_c, auto edge_c) {
        constexpr int MODE = decltype(mode_c)::value;   // 0 overwrite, 1 C += , 2 atomic +=
        constexpr bool EDGE = decltype(edge_c)::value != 0;
        float cs[TN];   // this lane's share of the column sums (one column per j)
#pragma unroll
        for (int j = 0; j < TN; j++) cs[j] = 0.f;
#pragma unroll
        for (int i = 0; i < TM; i++) {
            float rsub[16];   // what MG_ACT_SOFTMAX_GRAD subtracts from this lane's 16 rows
            if constexpr (ACT && MODE == 0) {
                if (sgrad) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int ro = (r >> 2) * 8 + (r & 3);
                        rsub[r] = (!EDGE || row_l + i * 32 + ro < p.M) ? rsl[i * 32 + ro] : 0.f;
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < TN; j++) {
                float *ct = cl + (int64_t)(i * 32) * ldc + j * 32;
                uint16_t *yt = yl + (int64_t)(i * 32) * ldy + j * 32;
                const bool col_ok = !EDGE || (col_l + j * 32 < p.N);
                float old[16];
                if constexpr (MODE == 1) {
                    const float *rt = rl + (int64_t)(i * 32) * ldr + j * 32;
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int ro = (r >> 2) * 8 + (r & 3);
                        const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                        old[r] = ok ? rt[ro * ldr] : 0.f;
                    }
                }
                if constexpr (ACT && MODE == 0) {
                    if (grad) {
                        const float *zt = zl + (int64_t)(i * 32) * ldz + j * 32;
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int ro = (r >> 2) * 8 + (r & 3);
                            const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                            old[r] = ok ? __builtin_nontemporal_load(zt + ro * ldz) : 0.f;
                        }
                    }
                    if (sgrad) {
                        const uint16_t *pt = pl + (int64_t)(i * 32) * ldp + j * 32;
#pragma unroll
                        for (int r = 0; r < 16; r++) {
                            const int ro = (r >> 2) * 8 + (r & 3);
                            const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                            old[r] = ok ? widen16_of<DT>(pt[ro * ldp]) : 0.f;
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ro = (r >> 2) * 8 + (r & 3);
                    const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                    float v = acc[i][j][r] + bv[j];
                    if constexpr (MODE == 1) v = old[r] + v;
                    if constexpr (ACT && MODE == 0) {
                        if (grad) {
                            v *= fused_dact(old[r], p.act);
                            cs[j] += ok ? v : 0.f;
                        }
                        if (sgrad) v = p.scale * old[r] * (v - rsub[r]);
                    }
                    if (ok) {
                        if constexpr (MODE == 2) {
                            __hip_atomic_fetch_add(ct + ro * ldc, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        } else {
                            if (have_c) __builtin_nontemporal_store(v, ct + ro * ldc);   // written once: stream past the L2
                            if constexpr (ACT) yt[ro * ldy] = narrow16_rne<DT>(fused_act(v, p.act));
                        }
                    }
                }
            }
        }
        if constexpr (ACT && MODE == 0) {
            if (grad && p.colsum != nullptr) {
                // the two half-waves hold different rows of the same 32 columns
#pragma unroll
                for (int j = 0; j < TN; j++) {
                    const float s = cs[j] + __shfl_xor(cs[j], 32, 64);
                    if (lane < 32 && col_l + j * 32 < p.N)
                        __hip_atomic_fetch_add(p.colsum + col_l + j * 32, s, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
        }
    };
    if (interior) {
        if (mode == 0) write_out(IntC<0>{}, IntC<0>{});
        else if (mode == 1) write_out(IntC<1>{}, IntC<0>{});
        else write_out(IntC<2>{}, IntC<0>{});
    } else {
        if (mode == 0) write_out(IntC<0>{}, IntC<1>{});
        else if (mode == 1) write_out(IntC<1>{}, IntC<1>{});
        else write_out(IntC<2>{}, IntC<1>{});
    }
}

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, bool GENERAL, bool ACT = false>
__global__ void __launch_bounds__(WGM *WGN * 64)
gemm_kernel(const GemmParams p) {
    constexpr bool A_KC = (LAYOUT != L_TN);
    constexpr bool B_KC = (LAYOUT == L_NT);
    constexpr int NTHREADS = WGM * WGN * 64;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KK = BK / 16;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 32 == 0, "tile shape");
    using SA = Stage<A_KC, BM, BK, NTHREADS, GENERAL>;
    using SB = Stage<B_KC, BN, BK, NTHREADS, GENERAL>;
    constexpr int STAGE_ELEMS = SA::ELEMS + SB::ELEMS;
    // LDS read instructions per fragment: one b128, or two transposing b64
    constexpr int NDSR = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);
    constexpr int NLOAD = SA::PER + SB::PER;

    extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave / WGN, wave_n = wave % WGN;

    int pid_m, pid_n;
    tile_coords(p, pid_m, pid_n);
    const int m0 = pid_m * BM, n0 = pid_n * BN;

    const int64_t zb = blockIdx.z;
    const uint16_t *A = p.A + zb * p.sa;
    const uint16_t *B = p.B + zb * p.sb;
    float *C = p.C + zb * p.sc;

    if (p.tri == 1 && n0 > m0 + BM - 1) return;   // tile wholly above the diagonal: nobody reads it
    int kbeg = blockIdx.y * p.k_per_split;
    int kend = min(p.K, kbeg + p.k_per_split);
    tri_k_range<BM, BK>(p.tri, m0, kbeg, kend);
    // an empty slice has nothing to add to C, except the bias when it is the slice that carries it
    if (kend == kbeg && p.split_k > 1 && p.ws == nullptr && !(p.bias != nullptr && blockIdx.y == 0)) return;
    const int nkb = (kend - kbeg + BK - 1) / BK;
    // K-blocks that the unconditional loader may fetch: the whole block inside
    // K, and the tile inside M and N.
    const bool interior = (m0 + BM <= p.M) && (n0 + BN <= p.N);
    const int nkb_fast = interior ? (kend - kbeg) / BK : 0;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    SA sa;
    SB sb;
    u32x4 af[2][TM], bf[2][TN];

    // first element of K-block kb of this tile, per operand
    auto a_tile = [&](int kb) -> const uint16_t * {
        const int64_t k0 = kbeg + (int64_t)kb * BK;
        return A_KC ? A + (int64_t)m0 * p.lda + k0 : A + k0 * p.lda + m0;
    };
    auto b_tile = [&](int kb) -> const uint16_t * {
        const int64_t k0 = kbeg + (int64_t)kb * BK;
        return B_KC ? B + (int64_t)n0 * p.ldb + k0 : B + k0 * p.ldb + n0;
    };
    auto load_block = [&](int kb) {   // uniform branch: fast when the block is interior
        if (kb < nkb_fast) {
            sa.load_fast(a_tile(kb), p.lda, tid);
            sb.load_fast(b_tile(kb), p.ldb, tid);
        } else {
            sa.load(A, p.lda, m0, p.M, kbeg + kb * BK, kend, tid);
            sb.load(B, p.ldb, n0, p.N, kbeg + kb * BK, kend, tid);
        }
    };
    auto read_frags = [&](const uint16_t *As, int kk, int slot) {
        const uint16_t *Bs = As + SA::ELEMS;
#pragma unroll
        for (int i = 0; i < TM; i++) af[slot][i] = SA::frag(As, wave_m * WTM + i * 32, kk, lane);
#pragma unroll
        for (int j = 0; j < TN; j++) bf[slot][j] = SB::frag(Bs, wave_n * WTN + j * 32, kk, lane);
    };
    auto mfma_group = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = mfma32<DT>(af[slot][i], bf[slot][j], acc[i][j]);
    };

    // Prologue: K-block 0 -> LDS stage 0, K-block 1 -> registers, fragments of
    // (block 0, kk 0) -> af[0], bf[0].
    if (nkb > 0) {
        load_block(0);
        sa.store(smem, tid);
        sb.store(smem + SA::ELEMS, tid);
        if (nkb > 1) load_block(1);
    }
    __syncthreads();
    if (nkb > 0) read_frags(smem, 0, 0);

    // One K-block.  MODE 1: blocks kb+1 and kb+2 exist and kb+2 is interior, so
    // the loop body is straight-line code; MODE 0: generic tail with uniform
    // branches.  The global loads issued here are consumed one whole K-block
    // later, by the LDS writes of the next iteration.
    auto kblock = [&](auto mode, int kb) {
        constexpr int MODE = decltype(mode)::value;
        const uint16_t *As = smem + (kb & 1) * STAGE_ELEMS;
        uint16_t *An = smem + ((kb + 1) & 1) * STAGE_ELEMS;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk < KK - 1) {
                read_frags(As, kk + 1, nxt);
            } else if (MODE == 1 || kb + 1 < nkb) {
                read_frags(An, 0, nxt);   // next stage is complete: the barrier below has passed
            }
            if (kk == KK - 2) {
                if (MODE == 1 || kb + 1 < nkb) {
                    sa.store(An, tid);
                    sb.store(An + SA::ELEMS, tid);
                }
                if constexpr (MODE == 1) {
                    sa.load_fast(a_tile(kb + 2), p.lda, tid);
                    sb.load_fast(b_tile(kb + 2), p.ldb, tid);
                } else {
                    if (kb + 2 < nkb) load_block(kb + 2);
                }
            }
            mfma_group(cur);
            if constexpr (MODE == 1) {
                if (kk == KK - 2) interleave_group<TM * TN, NDSR, NLOAD, NLOAD>();
                else interleave_group<TM * TN, NDSR, 0, 0>();
            }
            if (kk == KK - 2) __syncthreads();
        }
    };

    int kb = 0;
    const int n_steady = nkb_fast - 2;   // iterations whose kb+2 prefetch is interior
    for (; kb < n_steady; kb++) kblock(IntC<1>{}, kb);
    for (; kb < nkb; kb++) kblock(IntC<0>{}, kb);

    // Epilogue.  Accumulator register r of lane l holds
    //   row (r/4)*8 + (l/32)*4 + r%4,  column l%32   of its 32x32 tile,
    // so one store instruction writes two full 128-byte row segments.  The mode
    // (overwrite / read-add / atomic-add) and the edge test are uniform over the
    // workgroup and hoisted out of the element loops.
    bool add_bias = p.bias != nullptr && blockIdx.y == 0;
    int mode = p.split_k > 1 ? 2 : (p.beta ? 1 : 0);
    if (p.split_k > 1 && p.ws != nullptr) {
        __syncthreads();   // every wave is done with the LDS stages: smem[0..1] serves as the flag
        const int64_t tile_id = (int64_t)blockIdx.z * gridDim.x + blockIdx.x, ntiles = (int64_t)gridDim.x * gridDim.z;
        if (!splitk_gather<TM, TN, WGM * WGN * 64>(acc, p.ws, p.cnt + tile_id, blockIdx.y, gridDim.y,
                                                    [&](int sl) { return (int64_t)sl * ntiles + tile_id; }, tid,
                                                    reinterpret_cast<int *>(smem)))
            return;
        add_bias = p.bias != nullptr;
        mode = p.beta ? 1 : 0;
    }
    store_tile<DT, TM, TN, WTM, WTN, ACT>(p, C, acc, m0, n0, wave_m, wave_n, lane, add_bias, mode, interior);
}

// What the runtime reports for one kernel instantiation on the current device (the counterpart of
// the reference's Kernel.statistics(), vk.py:690-736): registers, static LDS and scratch from
// hipFuncGetAttributes, the workgroups of this launch shape a CU holds from the occupancy query.
struct KernelQuery {
    hipFuncAttributes attr;
    int threads;        // workgroup size the launcher uses
    int dynamic_lds;    // dynamic LDS bytes it asks for
    int wgs_per_cu;     // hipOccupancyMaxActiveBlocksPerMultiprocessor for that launch shape
};
inline hipError_t query_kernel(const void *kern, int threads, int dynamic_lds, KernelQuery *q) {
    hipError_t e = hipFuncGetAttributes(&q->attr, kern);
    if (e != hipSuccess) return e;
    q->threads = threads;
    q->dynamic_lds = dynamic_lds;
    q->wgs_per_cu = 0;
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(&q->wgs_per_cu, kern, threads, (size_t)dynamic_lds);
}

// A launcher enqueues its kernel, or - with `query` set - only reports on it.
typedef hipError_t (*launch_fn)(const GemmParams &, dim3 grid, hipStream_t, KernelQuery *query);

// More than 64 KiB of dynamic LDS has to be allowed per kernel and per device; `done`
// remembers, one bit per device index, where that has happened for the calling launcher.
inline hipError_t allow_dynamic_lds(const void *kern, int bytes, std::atomic<uint64_t> &done) {
    if (bytes <= 65536) return hipSuccess;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    const uint64_t bit = 1ull << (dev & 63);
    if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
    return e;
}

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, bool GENERAL, bool ACT = false>
hipError_t launch_gemm(const GemmParams &p, dim3 grid, hipStream_t stream, KernelQuery *query = nullptr) {
    using TT = TileTraits<LAYOUT, BM, BN, BK, WGM, WGN>;
    auto kern = gemm_kernel<LAYOUT, DT, BM, BN, BK, WGM, WGN, GENERAL, ACT>;
    static std::atomic<uint64_t> lds_allowed{0};
    hipError_t e = allow_dynamic_lds((const void *)kern, TT::LDS_BYTES, lds_allowed);
    if (e != hipSuccess) return e;
    if (query) return query_kernel((const void *)kern, TT::NTHREADS, TT::LDS_BYTES, query);
    hipLaunchKernelGGL(kern, grid, dim3(TT::NTHREADS), TT::LDS_BYTES, stream, p);
    return hipGetLastError();
}

}  // namespace mg
