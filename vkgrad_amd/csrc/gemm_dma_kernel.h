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
//   every K slice but the last a multiple of BK,
//   ld >= round_up(K, 8) for a K-contiguous operand and ld >= round_up(extent, 8),
//   extent >= 8 for an M/N-contiguous one, so that a 16-byte chunk that straddles
//   the matrix edge still lies inside the row pitch (what it reads beyond the
//   edge is masked: zeroed along K, unused along M/N).
// K need not be a multiple of BK: the remainder (< BK) is staged through
// registers with zero fill and multiplied first, before the ring starts.
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
                const int col = min(row0 + lc * 8, ((nrows + 7) & ~7) - 8);
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

    // Skip one K-block (another wavefront group issues it).
    __device__ __forceinline__ void advance(int64_t kstep_elems) {
#pragma unroll
        for (int t = 0; t < PERW; t++) g[t] += kstep_elems;
    }

    // K remainder: fill this operand's LDS region with the block [k0, k0 + BK) of
    // which only k < kend exists, through registers, zero beyond kend, in the same
    // swizzled layout the direct loads produce.
    template <int NTHREADS>
    static __device__ __forceinline__ void fill_tail(char *region, const uint16_t *base, int64_t ld, int row0,
                                                     int nrows, int k0, int kend, int tid) {
        constexpr int NCHUNK = ROWS * BK / 8;
        for (int c = tid; c < NCHUNK; c += NTHREADS) {
            u32x4 v = {0u, 0u, 0u, 0u};
            int off;
            if constexpr (KC) {
                const int r = c / CPR, kc = c % CPR;
                const int k = k0 + kc * 8;
                if (k < kend) {
                    const int row = min(row0 + r, nrows - 1);
                    v = *(const u32x4 *)(base + (int64_t)row * ld + k);
                    const int nvalid = kend - k;   // elements of this chunk inside K
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        const uint32_t keep = (2 * w + 1 < nvalid) ? 0xffffffffu : (2 * w < nvalid ? 0x0000ffffu : 0u);
                        v[w] &= keep;
                    }
                }
                off = r * ROW_BYTES + ((kc ^ swz(r)) * 16);
            } else {
                const int kr = c / CPR, rc = c % CPR;
                const int k = k0 + kr;
                if (k < kend) {
                    const int col = min(row0 + rc * 8, ((nrows + 7) & ~7) - 8);
                    v = *(const u32x4 *)(base + (int64_t)k * ld + col);
                }
                off = kr * ROW_BYTES + ((rc ^ swz(kr)) * 16);
            }
            *(u32x4 *)(region + off) = v;
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

// Four-wave workgroups whose accumulators take 128 registers a lane and whose ring takes at most
// half the LDS are meant to run two to a CU: the second launch bound keeps the register
// allocator under 256, which it otherwise exceeds for the 256 x 128 and 128 x 256 tiles (348
// registers, one workgroup per CU, 60.6 against 51.2 us at 8192 x 3072 x 768).  The smaller
// four-wave tiles stay under 256 by themselves and are left to the allocator.
template <int BM, int BN, int BK, int WGM, int WGN, int NSTAGE>
constexpr int dma_waves_per_simd() {
    return (WGM * WGN == 4 && BM * BN == 256 * 128 && NSTAGE * (BM + BN) * BK * 2 <= 81920) ? 2 : 1;
}

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE, bool ACT = false>
__global__ void __launch_bounds__(WGM *WGN * 64, (dma_waves_per_simd<BM, BN, BK, WGM, WGN, NSTAGE>()))
gemm_dma_kernel(const GemmParams p) {
    constexpr bool A_KC = (LAYOUT != L_TN);
    constexpr bool B_KC = (LAYOUT == L_NT);
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KK = BK / 16;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && KK % 2 == 0 && NSTAGE >= 2, "tile shape");
    // With eight waves (two per SIMD) and a two-stage ring, the loads of a K-block are
    // issued by half the waves, one per SIMD, alternating between the halves from block
    // to block.  A wave that issues a burst of direct loads stalls in the issue stage
    // until the texture path has taken them (16 clocks per instruction, 1024 per
    // K-block and CU); with every wave issuing at once all MFMA pipes idle for that
    // long, with one issuing wave per SIMD the other keeps its pipe busy meanwhile.
    constexpr bool ALT = (NW == 8 && NSTAGE == 2);
    constexpr int NWI = ALT ? NW / 2 : NW;          // waves that issue the loads of one K-block
    using OA = DmaOp<A_KC, BM, BK, NWI>;
    using OB = DmaOp<B_KC, BN, BK, NWI>;
    constexpr int STAGE_BYTES = OA::BYTES + OB::BYTES;
    constexpr int L = OA::PERW + OB::PERW;          // direct loads per issuing wave per K-block
    constexpr int NDSR = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);

    extern __shared__ __attribute__((aligned(1024))) char dsm[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WGN, wave_n = wave % WGN;
    const int wi = ALT ? (wave & (NWI - 1)) : wave;   // index among the issuing waves
    const int grp = ALT ? wave / NWI : 0;             // issues the K-blocks of this parity

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
    const int krem = (kend - kbeg) % BK;          // K remainder, multiplied first
    const int kdma = kbeg + krem;                 // the ring covers [kdma, kend)
    const int nkb = (kend - kdma) / BK;
    const bool interior = (m0 + BM <= p.M) && (n0 + BN <= p.N);

    // An issuing group starts at the block of its parity and steps two blocks at a time.
    OA oa;
    OB ob;
    oa.init(A, p.lda, m0, p.M, kdma + grp * BK, wi, lane);
    ob.init(B, p.ldb, n0, p.N, kdma + grp * BK, wi, lane);
    const int64_t a_step = (A_KC ? BK : (int64_t)BK * p.lda) * (ALT ? 2 : 1);
    const int64_t b_step = (B_KC ? BK : (int64_t)BK * p.ldb) * (ALT ? 2 : 1);

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
    // block: index of the K-block within the ring's sequence (decides the issuing group)
    auto issue_block = [&](int stage, int block) {
        if (ALT && (block & 1) != grp) return;
        const uint32_t sp = lds_base + stage * STAGE_BYTES;
        oa.issue(sp, a_step, wi);
        ob.issue(sp + OA::BYTES, b_step, wi);
    };

    if (krem > 0) {
        // [kbeg, kbeg + krem): through registers into stage 0, zero-filled to BK.
        OA::template fill_tail<NW * 64>(dsm, A, p.lda, m0, p.M, kbeg, kbeg + krem, tid);
        OB::template fill_tail<NW * 64>(dsm + OA::BYTES, B, p.ldb, n0, p.N, kbeg, kbeg + krem, tid);
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            read_frags(0, kk, 0);
            mfma_group(0);
        }
        __syncthreads();   // all reads of stage 0 done before the ring overwrites it
    }

    // Prologue: fill the ring (NSTAGE blocks, or all of them), publish block 0.
    const int npre = min(nkb, NSTAGE);
    for (int s = 0; s < npre; s++) issue_block(s, s);
    // (alternating groups: a wave has issued one block at most, so it waits for all it has)
    if (npre >= NSTAGE && !ALT) wait_dma_and_barrier<(NSTAGE - 1) * L>();
    else wait_dma_and_barrier<0>();
    if (nkb > 0) read_frags(0, 0, 0);

    // Main loop.  At the barrier inside iteration kb, block kb+1 becomes visible
    // to every wave and stage kb % NSTAGE is free for block kb+NSTAGE.
    int stage = 0;
    for (int kb = 0; kb < nkb; kb++) {
        const int nstage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk < KK - 1) {
                read_frags(stage, kk + 1, nxt);
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
            if (kk == KK - 2) {
                // blocks still allowed in flight: kb+2 .. kb+NSTAGE-1, as far as they exist
                const int later = min(nkb - 1, kb + NSTAGE - 1) - (kb + 1);
                if (later >= NSTAGE - 2) wait_dma_and_barrier<(NSTAGE - 2) * L>();
                else if (later == 1 && NSTAGE > 3) wait_dma_and_barrier<L>();
                else wait_dma_and_barrier<0>();
                if (kb + NSTAGE < nkb) issue_block(stage, kb + NSTAGE);
            }
            if (kk == KK - 1) {
                if (kb + 1 < nkb) read_frags(nstage, 0, nxt);
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
        }
        stage = nstage;
    }

    // Epilogue: shared with the register-staged kernel (store_tile, gemm_kernel.h).
    bool add_bias = p.bias != nullptr && blockIdx.y == 0;
    int mode = p.split_k > 1 ? 2 : (p.beta ? 1 : 0);
    if (p.split_k > 1 && p.ws != nullptr) {
        __syncthreads();   // every wave is done with the ring: its first word serves as the flag
        const int64_t tile_id = (int64_t)blockIdx.z * gridDim.x + blockIdx.x, ntiles = (int64_t)gridDim.x * gridDim.z;
        if (!splitk_gather<TM, TN, NW * 64>(acc, p.ws, p.cnt + tile_id, blockIdx.y, gridDim.y,
                                             [&](int sl) { return (int64_t)sl * ntiles + tile_id; }, tid,
                                             reinterpret_cast<int *>(dsm)))
            return;
        add_bias = p.bias != nullptr;
        mode = p.beta ? 1 : 0;
    }
    store_tile<DT, TM, TN, WTM, WTN, ACT>(p, C, acc, m0, n0, wave_m, wave_n, lane, add_bias, mode, interior);
}

// ---------------------------------------------------------------------------
// Global memory access of the persistent kernel's epilogue, as inline assembly.
// Any global load or store the compiler can see inside the K loop makes its
// wait-count pass insert s_waitcnt vmcnt(..) where registers are reused (and
// extra live ranges push the kernel into scratch spills, which are vector memory
// operations themselves); vmcnt also counts the direct-to-LDS loads in flight,
// so such waits would drain the ring once per tile.  The hardware reads a
// store's address and data registers when the instruction issues, so stores need
// no wait.  Addresses are per-lane 64-bit VGPR pointers plus an immediate: an
// SGPR base written by a scalar instruction just before would need wait states
// the compiler does not insert for assembly it cannot see into.
// ---------------------------------------------------------------------------
// C is written once and not read again by this kernel: the stores are marked non-temporal
// so they stream past the L2 instead of evicting the operand panels other workgroups
// are still sharing (LM-head forward on MI355X: 744 us -> 654 us).  Plain stores were tried
// again for outputs that fit the 256 MB last-level cache (8192 x 3072 f32): the persistent
// 128 x 128 kernel lost 7 % (51.7 us against 48.1 us).
template <int IMM>
__device__ __forceinline__ void hidden_store(float *ptr, float v) {
    asm volatile("global_store_dword %0, %1, off offset:%2 nt" ::"v"(ptr), "v"(v), "n"(IMM) : "memory");
}
// C += v without reading C into registers: the L2 performs the add.  One writer
// per element, so the result is the same single float add a load/add/store gives.
template <int IMM>
__device__ __forceinline__ void hidden_atomic_add(float *ptr, float v) {
    asm volatile("global_atomic_add_f32 %0, %1, off offset:%2" ::"v"(ptr), "v"(v), "n"(IMM) : "memory");
}
// Load and wait in one statement: the compiler does not know the destination is
// pending, so it must never get the chance to copy it before the wait.
__device__ __forceinline__ float hidden_load_wait(const float *ptr) {
    float v;
    asm volatile("global_load_dword %0, %1, off\n\ts_waitcnt vmcnt(0)" : "=&v"(v) : "v"(ptr) : "memory");
    return v;
}

template <int J, int N, class F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (J < N) {
        f(IntC<J>{});
        static_for<J + 1, N>(f);
    }
}

// wait_dma_and_barrier with a run-time number of K-blocks (of L loads each) that
// may stay in flight, 0 <= blocks <= MAXB.
template <int L, int MAXB>
__device__ __forceinline__ void wait_blocks_and_barrier(int blocks) {
    static_assert(L * MAXB <= 63, "vmcnt immediate is 6 bits");
    if constexpr (MAXB >= 3) {
        if (blocks >= 3) { wait_dma_and_barrier<3 * L>(); return; }
    }
    if constexpr (MAXB >= 2) {
        if (blocks == 2) { wait_dma_and_barrier<2 * L>(); return; }
    }
    if constexpr (MAXB >= 1) {
        if (blocks == 1) { wait_dma_and_barrier<L>(); return; }
    }
    wait_dma_and_barrier<0>();
}

// ---------------------------------------------------------------------------
// Persistent variant.  The grid holds at most as many workgroups as fit on the
// chip at once; workgroup w processes work units w, w + gridDim.x, ... where a
// unit is (K slice, output tile).  The K-blocks of all of a workgroup's units
// form one flat sequence through the LDS ring, so the loads of the next unit's
// first blocks are already in flight while the current unit finishes, and its
// epilogue stores drain while the next unit's MFMAs run: no pipeline refill and
// no exposed store phase between tiles.  Requires every K slice to be a multiple
// of BK.
//
// EPI_LOADS = true adds the bias epilogue (its loads drain vmcnt once per tile);
// C += (beta = 1 or split-K) is an L2 atomic add and needs no load.
// ---------------------------------------------------------------------------
template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE, bool EPI_LOADS, bool STREAMK>
__global__ void __launch_bounds__(WGM *WGN * 64)
gemm_dmap_kernel(const GemmParams p) {
    constexpr bool A_KC = (LAYOUT != L_TN);
    constexpr bool B_KC = (LAYOUT == L_NT);
    constexpr int NW = WGM * WGN;
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KK = BK / 16;
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && KK % 2 == 0 && NSTAGE >= 2, "tile shape");
    constexpr bool ALT = (NW == 8 && NSTAGE == 2);   // issuing waves alternate per K-block, as in gemm_dma_kernel
    constexpr int NWI = ALT ? NW / 2 : NW;
    using OA = DmaOp<A_KC, BM, BK, NWI>;
    using OB = DmaOp<B_KC, BN, BK, NWI>;
    constexpr int STAGE_BYTES = OA::BYTES + OB::BYTES;
    constexpr int L = OA::PERW + OB::PERW;
    constexpr int NDSR = TM * (A_KC ? 1 : 2) + TN * (B_KC ? 1 : 2);

    extern __shared__ __attribute__((aligned(1024))) char dsm[];
    __shared__ int gather_flag;   // the ring always holds prefetched blocks, so the flag lives beside it

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WGN, wave_n = wave % WGN;
    const int wi = ALT ? (wave & (NWI - 1)) : wave;
    const int grp = ALT ? wave / NWI : 0;
    const int64_t zb = blockIdx.z;
    const uint16_t *A = p.A + zb * p.sa;
    const uint16_t *B = p.B + zb * p.sb;
    float *C = p.C + zb * p.sc;

    // Work units of this workgroup.  Positions are renumbered XCD-major so the
    // workgroups behind one L2 hold neighbouring tiles.
    //   plain:    unit i is (K slice, tile) number pos + i * gridDim.x, slice-major (all
    //             tiles of slice 0, then slice 1, ...), so the slices of one tile are
    //             not meeting at the same moment.
    //   stream-K: the tiles that fill whole rounds are dealt out the same way; each of the
    //             remaining tiles (less than one round) is cut along K into sk_pieces equal
    //             pieces, one per workgroup, done first and piece-major like K slices, so
    //             that the workgroups sharing an operand panel walk the same K-blocks at the
    //             same time and keep hitting each other's lines in the L2.  (Cutting the
    //             remaining K-blocks into runs of exactly equal length instead balances
    //             better on paper, but then no two workgroups are at the same K offset and
    //             every load misses: measured twice as slow.)
    const int nwg = gridDim.x;
    const int ntiles = p.grid_m * p.grid_n;
    int pos = blockIdx.x;
    if ((nwg & 7) == 0) pos = (pos & 7) * (nwg >> 3) + (pos >> 3);

    struct Unit {
        int m0, n0, kbeg, nkb, lin, slice, nslices;
    };
    auto place = [&](int lin, Unit &q) {
        const int in_group = p.group_m * p.grid_n;
        const int gid = lin / in_group;
        const int first_m = gid * p.group_m;
        const int gsize = min(p.grid_m - first_m, p.group_m);
        const int r = lin - gid * in_group;
        q.m0 = (first_m + r % gsize) * BM;
        q.n0 = (r / gsize) * BN;
        q.lin = lin;
    };
    // stream-K bookkeeping (all zero in plain mode)
    const bool stream_k = STREAMK && p.stream_k;   // a stream-K tile without workspace runs plain
    const int nkb_tile = p.K / BK;
    const int full_rounds = stream_k ? p.sk_full_rounds : 0;
    const int rem_tiles = stream_k ? p.sk_rem_tiles : 0;
    const int pieces = stream_k ? p.sk_pieces : 1;
    const int rem_units = (STREAMK && pos < rem_tiles * pieces) ? 1 : 0;
    const int n_plain = stream_k ? full_rounds : (ntiles * p.split_k - pos + nwg - 1) / nwg;
    const int my_units = rem_units + (n_plain > 0 ? n_plain : 0);

    auto unit_at = [&](int i) -> Unit {
        Unit q;
        if (STREAMK && i < rem_units) {
            const int piece = pos / rem_tiles, t = pos - piece * rem_tiles;
            const int lo = piece * nkb_tile / pieces, hi = (piece + 1) * nkb_tile / pieces;
            place(full_rounds * nwg + t, q);
            q.kbeg = lo * BK;
            q.nkb = hi - lo;
            q.slice = piece;
            q.nslices = pieces;
            return q;
        }
        const int u = pos + (i - rem_units) * nwg;
        const int slice = stream_k ? 0 : u / ntiles;
        place(u - slice * ntiles, q);
        q.slice = slice;
        q.nslices = stream_k ? 1 : p.split_k;
        q.kbeg = slice * p.k_per_split;
        q.nkb = (min(p.K, q.kbeg + p.k_per_split) - q.kbeg) / BK;
        return q;
    };

    const int64_t a_step = A_KC ? BK : (int64_t)BK * p.lda;
    const int64_t b_step = B_KC ? BK : (int64_t)BK * p.ldb;
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t *)dsm;

    // ---- load side ----
    OA oa;
    OB ob;
    int l_i = 0;              // unit being loaded
    int l_kb = 0, l_nkb = 0;  // next block of it, and its block count
    int issued = 0;           // K-blocks issued so far (flat)
    bool l_live = my_units > 0;
    auto issue_next = [&]() {
        if (!l_live) return;
        if (l_kb == 0) {
            const Unit q = unit_at(l_i);
            l_nkb = q.nkb;
            oa.init(A, p.lda, q.m0, p.M, q.kbeg, wi, lane);
            ob.init(B, p.ldb, q.n0, p.N, q.kbeg, wi, lane);
        }
        const uint32_t sp = lds_base + (issued % NSTAGE) * STAGE_BYTES;
        if (!ALT || (issued & 1) == grp) {
            oa.issue(sp, a_step, wi);
            ob.issue(sp + OA::BYTES, b_step, wi);
        } else {
            oa.advance(a_step);
            ob.advance(b_step);
        }
        issued++;
        if (++l_kb == l_nkb) {
            l_kb = 0;
            l_live = ++l_i < my_units;
        }
    };

    // ---- compute side ----
    f32x16 acc[TM][TN];
    auto zero_acc = [&]() {
#pragma unroll
        for (int i = 0; i < TM; i++)
#pragma unroll
            for (int j = 0; j < TN; j++)
#pragma unroll
                for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;
    };
    zero_acc();

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

    // Epilogue of one unit.  The tile is walked row by row with one running
    // per-lane pointer; the TN column blocks of a row are immediate offsets.
    // beta = 1 and split-K both add into C with L2 atomics (no loads); the only
    // loads are the TN bias values.
    auto epilogue = [&](const Unit &q) {
        const bool interior = (q.m0 + BM <= p.M) && (q.n0 + BN <= p.N);
        bool add_bias = EPI_LOADS && p.bias != nullptr && q.kbeg == 0;
        bool atomic = q.nslices > 1 || p.beta;
        if (q.nslices > 1 && p.ws != nullptr) {
            const int64_t tile_id = zb * ntiles + q.lin;
            // Workspace slot of piece sl: slot planes over the tiles that are cut (all of them
            // for a plain split, the remaining ones for stream-K).
            const int64_t plane = stream_k ? (int64_t)rem_tiles * gridDim.z : (int64_t)ntiles * gridDim.z;
            const int64_t in_plane = stream_k ? zb * rem_tiles + (q.lin - full_rounds * nwg) : tile_id;
            const bool mine = splitk_gather<TM, TN, NW * 64>(
                acc, p.ws, p.cnt + tile_id, q.slice, q.nslices,
                [&](int sl) -> int64_t { return (int64_t)sl * plane + in_plane; }, tid, &gather_flag);
            if (!mine) return;
            add_bias = EPI_LOADS && p.bias != nullptr;
            atomic = p.beta != 0;
        }
        const int row_l = q.m0 + wave_m * WTM + (lane >> 5) * 4;
        const int col_l = q.n0 + wave_n * WTN + (lane & 31);
        const int64_t ldc = p.ldc;
        float bv[TN];
#pragma unroll
        for (int j = 0; j < TN; j++) {
            bv[j] = 0.f;
            if constexpr (EPI_LOADS) {
                if (add_bias) bv[j] = hidden_load_wait(p.bias + min(col_l + j * 32, p.N - 1));
            }
        }
        auto write_out = [&](auto atomic_c, auto edge_c) {
            constexpr bool ATOMIC = decltype(atomic_c)::value != 0;
            constexpr bool EDGE = decltype(edge_c)::value != 0;
            float *ptr = C + (int64_t)row_l * ldc + col_l;
#pragma unroll
            for (int i = 0; i < TM; i++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ro = i * 32 + (r >> 2) * 8 + (r & 3);
                    const bool row_ok = !EDGE || (row_l + ro < p.M);
                    static_for<0, TN>([&](auto jc) {
                        constexpr int j = decltype(jc)::value;
                        float v = acc[i][j][r];
                        if constexpr (EPI_LOADS) v += bv[j];
                        if (row_ok && (!EDGE || col_l + j * 32 < p.N)) {
                            if constexpr (ATOMIC) hidden_atomic_add<j * 128>(ptr, v);
                            else hidden_store<j * 128>(ptr, v);
                        }
                    });
                    ptr += ((r & 3) == 3) ? 5 * ldc : ldc;   // rows go 0,1,2,3, 8,9,10,11, 16, ...
                }
            }
        };
        if (interior) {
            if (atomic) write_out(IntC<1>{}, IntC<0>{});
            else write_out(IntC<0>{}, IntC<0>{});
        } else {
            if (atomic) write_out(IntC<1>{}, IntC<1>{});
            else write_out(IntC<0>{}, IntC<1>{});
        }
    };

    if (!l_live) return;   // more workgroups than units

    // Prologue: fill the ring, publish block 0.
    for (int s = 0; s < NSTAGE; s++) issue_next();
    // (alternating groups: a wave has issued one block at most, so it waits for all it has)
    wait_blocks_and_barrier<L, NSTAGE - 1>(ALT ? 0 : issued - 1);
    read_frags(0, 0, 0);

    int c_i = 0;
    Unit cq = unit_at(0);
    int c_kb = 0;
    int stage = 0;
    // Invariant at the top of iteration ci: blocks ci .. issued-1 are issued,
    // block ci is visible to all waves, its kk=0 fragments are in af[0], bf[0].
    // Epilogue stores are younger than any load waited for below, so waiting on
    // the load count alone can only over-wait, never under-wait.
    for (int ci = 0; ci < issued; ci++) {
        const int nstage = (stage + 1 == NSTAGE) ? 0 : stage + 1;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
            const int cur = kk & 1, nxt = cur ^ 1;
            if (kk < KK - 1) {
                read_frags(stage, kk + 1, nxt);
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
            if (kk == KK - 2) {
                // block ci+1 must have landed; blocks ci+2 .. issued-1 may stay in flight
                const int ahead = issued - (ci + 2);
                wait_blocks_and_barrier<L, NSTAGE - 2>(ahead < 0 ? 0 : (ahead > NSTAGE - 2 ? NSTAGE - 2 : ahead));
                issue_next();   // into the stage block ci just vacated
            }
            if (kk == KK - 1) {
                if (ci + 1 < issued) read_frags(nstage, 0, nxt);
                mfma_group(cur);
                interleave_group<TM * TN, NDSR, 0, 0>();
            }
        }
        stage = nstage;
        if (++c_kb == cq.nkb) {
            epilogue(cq);
            c_kb = 0;
            if (++c_i < my_units) {
                cq = unit_at(c_i);
                zero_acc();
            }
        }
    }
}

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE, bool ACT = false>
hipError_t launch_gemm_dma(const GemmParams &p, dim3 grid, hipStream_t stream, KernelQuery *query = nullptr) {
    using TT = DmaTraits<LAYOUT, BM, BN, BK, WGM, WGN, NSTAGE>;
    auto kern = gemm_dma_kernel<LAYOUT, DT, BM, BN, BK, WGM, WGN, NSTAGE, ACT>;
    static std::atomic<uint64_t> lds_allowed{0};
    hipError_t e = allow_dynamic_lds((const void *)kern, TT::LDS_BYTES, lds_allowed);
    if (e != hipSuccess) return e;
    if (query) return query_kernel((const void *)kern, TT::NTHREADS, TT::LDS_BYTES, query);
    hipLaunchKernelGGL(kern, grid, dim3(TT::NTHREADS), TT::LDS_BYTES, stream, p);
    return hipGetLastError();
}

// Persistent launcher: grid.x is the number of resident workgroups the host chose.
template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, int NSTAGE, bool EPI_LOADS, bool STREAMK>
hipError_t launch_gemm_dmap(const GemmParams &p, dim3 grid, hipStream_t stream, KernelQuery *query = nullptr) {
    using TT = DmaTraits<LAYOUT, BM, BN, BK, WGM, WGN, NSTAGE>;
    auto kern = gemm_dmap_kernel<LAYOUT, DT, BM, BN, BK, WGM, WGN, NSTAGE, EPI_LOADS, STREAMK>;
    static std::atomic<uint64_t> lds_allowed{0};
    hipError_t e = allow_dynamic_lds((const void *)kern, TT::LDS_BYTES, lds_allowed);
    if (e != hipSuccess) return e;
    if (query) return query_kernel((const void *)kern, TT::NTHREADS, TT::LDS_BYTES, query);
    hipLaunchKernelGGL(kern, grid, dim3(TT::NTHREADS), TT::LDS_BYTES, stream, p);
    return hipGetLastError();
}

}  // namespace mg
