// GEMM kernel with direct global->LDS loads (global_load_lds_dwordx4) for gfx950.
//
// Same contract and MFMA/epilogue structure as gemm_kernel.h, but the operands
// never pass through registers on their way to LDS: every wavefront issues
// 16-byte-per-lane loads whose destination is a contiguous 1 KiB LDS segment,
// into a ring of NSTAGE K-block stages, so loads run NSTAGE-1 K-blocks ahead of
// the MFMAs with no staging registers and no LDS write instructions.
//
// A direct load cannot pad LDS rows, so bank conflicts are avoided by an XOR
// swizzle applied on the global side (which 16-byte chunk a lane fetches) and
// undone in the fragment read addresses:
//   K-contiguous operand  [rows][BK]:   chunk ^= (row / rows_per_256B) % chunks_per_row
//   M/N-contiguous operand [BK][rows]:  chunk ^= 2 * (k % 4)     (read by ds_read_b64_tr_b16)
//
// Preconditions (checked by the host, which otherwise uses gemm_kernel.h):
//   16-byte aligned operand bases, ld % 8 == 0, batch strides % 8 == 0,
//   K % BK == 0 and the K slice a multiple of BK,
//   for an M/N-contiguous operand its extent % 8 == 0 and >= 8.
#pragma once
#include "gemm_kernel.h"

namespace mg {

typedef __attribute__((address_space(3))) void lds_void_t;
typedef const __attribute__((address_space(1))) void glb_void_t;

template <bool KC, int ROWS, int BK, int NW>
struct DmaOp {
    static constexpr int ROW_BYTES = KC ? BK * 2 : ROWS * 2;
    static constexpr int BYTES = ROWS * BK * 2;
    static constexpr int NINSTR = BYTES / 1024;
    static constexpr int PERW = NINSTR / NW;          // load instructions per wavefront per K-block
    static constexpr int CPR = ROW_BYTES / 16;        // 16-byte chunks per LDS row
    static_assert(BYTES % 1024 == 0 && NINSTR % NW == 0 && PERW >= 1, "operand tile / wave count mismatch");
    static_assert(KC ? (ROW_BYTES == 64 || ROW_BYTES == 128) : (ROW_BYTES >= 256), "unsupported LDS row size");

    static __device__ __forceinline__ int swz(int row) {
        if constexpr (KC) {
            constexpr int RPB = 256 / ROW_BYTES;      // rows per 256-byte bank cycle
            return (row / RPB) % CPR;
        } else {
            return 2 * (row & 3);
        }
    }

    const uint16_t *g[PERW];   // this lane's global source for each of its load instructions

    // tile: first element of K-block 0 of this tile.  row0/nrows: tile origin and
    // matrix extent along the non-K axis (for clamping at the matrix edge).
    __device__ __forceinline__ void init(const uint16_t *base, int64_t ld, int row0, int nrows, int kbeg,
                                         int wave, int lane) {
#pragma unroll
        for (int t = 0; t < PERW; t++) {
            const int q = t * NW + wave;
            const int o = q * 1024 + lane * 16;
            const int r = o / ROW_BYTES;
            const int lc = ((o % ROW_BYTES) / 16) ^ swz(r);
            if constexpr (KC) {
                const int row = min(row0 + r, nrows - 1);
                g[t] = base + (int64_t)row * ld + kbeg + lc * 8;
            } else {
                const int col = min(row0 + lc * 8, nrows - 8);
                g[t] = base + (int64_t)(kbeg + r) * ld + col;
            }
        }
    }

    // Issue this wavefront's loads of one K-block into the LDS region at byte
    // address `dst` (wave-uniform), then advance to the next K-block.  The load
    // is written as inline assembly on purpose: the compiler's wait-count pass
    // must not see it, or it conservatively drains every outstanding direct load
    // (vmcnt(0)) in front of LDS reads it cannot prove disjoint, which would
    // serialise the whole ring.  Completion is awaited explicitly instead
    // (wait_dma_and_barrier).
    __device__ __forceinline__ void issue(uint32_t dst, int64_t kstep_elems, int wave) {
#pragma unroll
        for (int t = 0; t < PERW; t++) {
            const int q = t * NW + wave;
            const uint32_t m0v = dst + q * 1024;
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(m0v), "v"(g[t]) : "memory", "m0");
            g[t] += kstep_elems;
        }
    }

    // Byte offset (inside the operand's LDS region) of lane's fragment piece for
    // 32-row fragment `f` of the wave at row_base; kk selects the 16-k step.
    static __device__ __forceinline__ int frag_off(int row_base, int lane) {
        if constexpr (KC) {
            const int row = row_base + (lane & 31);
            return row * ROW_BYTES;   // chunk term added per kk (depends on swizzle)
        } else {
            const int j = lane & 15, g4 = lane >> 4;
            const int k = (g4 >> 1) * 8 + (j >> 2);
            const int col = row_base + (g4 & 1) * 16 + (j & 3) * 4;
            return k * ROW_BYTES + (((col >> 3) ^ swz(k)) * 16) + (col & 7) * 2;
        }
    }
    static __device__ __forceinline__ u32x4 frag(const char *region, int off, int kk, int lane, int row_base) {
        if constexpr (KC) {
            const int row = row_base + (lane & 31);
            const int lc = kk * 2 + (lane >> 5);
            return *(const u32x4 *)(region + off + ((lc ^ swz(row)) * 16));
        } else {
            const char *p = region + off + kk * 16 * ROW_BYTES;
            const u32x2 lo = lds_read_tr((const uint16_t *)p);
            const u32x2 hi = lds_read_tr((const uint16_t *)(p + 4 * ROW_BYTES));
            return u32x4{lo[0], lo[1], hi[0], hi[1]};
        }
    }
};

template <int N>
__device__ __forceinline__ void wait_dma_and_barrier() {
    // N = direct loads this wave may still have in flight; everything older has
    // landed in LDS.  lgkmcnt(0): this wave's own LDS reads are complete, so the
    // stage they came from may be overwritten after the barrier.
    if constexpr (N == 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

template <int LAYOUT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE>
struct DmaTraits {
    static constexpr int NTHREADS = WGM * WGN * 64;
    static constexpr int STAGE_BYTES = (BM + BN) * BK * 2;
    static constexpr int LDS_BYTES = NSTAGE * STAGE_BYTES;
};

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE>
__global__ void __launch_bounds__(WGM *WGN * 64)
gemm_dma_kernel(const GemmParams p) {
    constexpr bool A_KC = (LAYOUT != L_TN);
    constexpr bool B_KC = (LAYOUT == L_NT);
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KK = BK / 16;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && KK % 2 == 0 && NSTAGE >= 2, "tile shape");
    using OA = DmaOp<A_KC, BM, BK, NW>;
    using OB = DmaOp<B_KC, BN, BK, NW>;
    constexpr int STAGE_BYTES = OA::BYTES + OB::BYTES;
    constexpr int L = OA::PERW + OB::PERW;          // direct loads per wave per K-block
    constexpr int NDSR = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);

    extern __shared__ __attribute__((aligned(1024))) char dsm[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WGN, wave_n = wave % WGN;

    int pid_m, pid_n;
    tile_coords(p, pid_m, pid_n);
    const int m0 = pid_m * BM, n0 = pid_n * BN;
    const int64_t zb = blockIdx.z;
    const uint16_t *A = p.A + zb * p.sa;
    const uint16_t *B = p.B + zb * p.sb;
    float *C = p.C + zb * p.sc;
    const int kbeg = blockIdx.y * p.k_per_split;
    const int kend = min(p.K, kbeg + p.k_per_split);
    const int nkb = (kend - kbeg) / BK;
    const bool interior = (m0 + BM <= p.M) && (n0 + BN <= p.N);

    OA oa;
    OB ob;
    oa.init(A, p.lda, m0, p.M, kbeg, wave, lane);
    ob.init(B, p.ldb, n0, p.N, kbeg, wave, lane);
    const int64_t a_step = A_KC ? BK : (int64_t)BK * p.lda;
    const int64_t b_step = B_KC ? BK : (int64_t)BK * p.ldb;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    int a_off[TM], b_off[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) a_off[i] = OA::frag_off(wave_m * WTM + i * 32, lane);
#pragma unroll
    for (int j = 0; j < TN; j++) b_off[j] = OA::BYTES + OB::frag_off(wave_n * WTN + j * 32, lane);

    u32x4 af[2][TM], bf[2][TN];
    auto read_frags = [&](int stage, int kk, int slot) {
        const char *sp = dsm + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < TM; i++) af[slot][i] = OA::frag(sp, a_off[i], kk, lane, wave_m * WTM + i * 32);
#pragma unroll
        for (int j = 0; j < TN; j++) bf[slot][j] = OB::frag(sp, b_off[j], kk, lane, wave_n * WTN + j * 32);
    };
    auto mfma_group = [&](int slot) {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++) acc[i][j] = mfma32<DT>(af[slot][i], bf[slot][j], acc[i][j]);
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t *)dsm;
    auto issue_block = [&](int stage) {
        const uint32_t sp = lds_base + stage * STAGE_BYTES;
        oa.issue(sp, a_step, wave);
        ob.issue(sp + OA::BYTES, b_step, wave);
    };

    // Prologue: fill the ring (NSTAGE blocks, or all of them), publish block 0.
    const int npre = min(nkb, NSTAGE);
    for (int s = 0; s < npre; s++) issue_block(s);
    if (npre >= NSTAGE) wait_dma_and_barrier<(NSTAGE - 1) * L>();
    else wait_dma_and_barrier<0>();
    if (nkb > 0) read_frags(0, 0, 0);

    // Main loop.  At the barrier inside iteration kb, block kb+1 becomes visible
    // to every wave and stage kb % NSTAGE is free for block kb+NSTAGE.
    int stage = 0;
#ifdef EXP_NO_MAINLOOP
    for (int kb = 0; kb < 0; kb++) {
#else
    for (int kb = 0; kb < nkb; kb++) {
#endif
        const int nstage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk < KK - 1) {
#ifndef EXP_NO_FRAG
                read_frags(stage, kk + 1, nxt);
#endif
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
            if (kk == KK - 2) {
                // blocks still allowed in flight: kb+2 .. kb+NSTAGE-1, as far as they exist
#ifdef EXP_NO_GLOAD
                const int later = -1;
#else
                const int later = min(nkb - 1, kb + NSTAGE - 1) - (kb + 1);
#endif
#ifndef EXP_NO_BARRIER
                if (later >= NSTAGE - 2) wait_dma_and_barrier<(NSTAGE - 2) * L>();
                else if (later == 1 && NSTAGE > 3) wait_dma_and_barrier<L>();
                else wait_dma_and_barrier<0>();
#endif
#ifndef EXP_NO_GLOAD
                if (kb + NSTAGE < nkb) issue_block(stage);
#endif
            }
            if (kk == KK - 1) {
#ifndef EXP_NO_FRAG
                if (kb + 1 < nkb) read_frags(nstage, 0, nxt);
#endif
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
        }
        stage = nstage;
    }

#ifdef EXP_NO_EPILOGUE
    if (p.M > 0) { if (acc[0][0][0] == 123.456f) C[0] = 1.f; return; }
#endif
    // Epilogue: identical to gemm_kernel.h.
    const bool add_bias = p.bias != nullptr && blockIdx.y == 0;
    const int row_l = m0 + wave_m * WTM + (lane >> 5) * 4;
    const int col_l = n0 + wave_n * WTN + (lane & 31);
    float *cl = C + (int64_t)row_l * p.ldc + col_l;
    const int64_t ldc = p.ldc;
    float bv[TN];
#pragma unroll
    for (int j = 0; j < TN; j++) bv[j] = (add_bias && col_l + j * 32 < p.N) ? p.bias[col_l + j * 32] : 0.f;

    auto write_out = [&](auto mode_c, auto edge_c) {
        constexpr int MODE = decltype(mode_c)::value;
        constexpr bool EDGE = decltype(edge_c)::value != 0;
#pragma unroll
        for (int i = 0; i < TM; i++) {
#pragma unroll
            for (int j = 0; j < TN; j++) {
                float *ct = cl + (int64_t)(i * 32) * ldc + j * 32;
                const bool col_ok = !EDGE || (col_l + j * 32 < p.N);
                float old[16];
                if constexpr (MODE == 1) {
#pragma unroll
                    for (int r = 0; r < 16; r++) {
                        const int ro = (r >> 2) * 8 + (r & 3);
                        const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                        old[r] = ok ? ct[ro * ldc] : 0.f;
                    }
                }
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ro = (r >> 2) * 8 + (r & 3);
                    const bool ok = col_ok && (!EDGE || row_l + i * 32 + ro < p.M);
                    float v = acc[i][j][r] + bv[j];
                    if constexpr (MODE == 1) v = old[r] + v;
                    if (ok) {
                        if constexpr (MODE == 2)
                            __hip_atomic_fetch_add(ct + ro * ldc, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        else
                            ct[ro * ldc] = v;
                    }
                }
            }
        }
    };
    const int mode = p.split_k > 1 ? 2 : (p.beta ? 1 : 0);
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

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE>
hipError_t launch_gemm_dma(const GemmParams &p, dim3 grid, hipStream_t stream) {
    using TT = DmaTraits<LAYOUT, BM, BN, BK, WGM, WGN, NSTAGE>;
    auto kern = gemm_dma_kernel<LAYOUT, DT, BM, BN, BK, WGM, WGN, NSTAGE>;
    static bool attr_done = false;
    if (!attr_done) {
        if (TT::LDS_BYTES > 65536) {
            hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                               TT::LDS_BYTES);
            if (e != hipSuccess) return e;
        }
        attr_done = true;
    }
    hipLaunchKernelGGL(kern, grid, dim3(TT::NTHREADS), TT::LDS_BYTES, stream, p);
    return hipGetLastError();
}

}  // namespace mg
