// Ping-pong GEMM kernel for gfx950: the two wavefronts that share a SIMD run half a
// K-block apart instead of in lock-step.
//
// Same contract, LDS layout, direct-to-LDS loads and epilogue as gemm_dma_kernel.h
// (one 256 x 256 x 64 tile per workgroup, eight wavefronts of 128 x 64, a two-stage
// ring), but the K loop of a wavefront is cut into two phases per K-block:
//
//   MEM  read every MFMA operand of the block from LDS into registers (24 x 16 bytes
//        per lane), and - first group only - issue the direct loads of the next block;
//   MMA  32 back-to-back MFMAs on registers only, at raised priority.
//
// Wavefronts 0-3 (one per SIMD, the upper half of the tile) form group 0, wavefronts
// 4-7 group 1, and group 1 runs one phase behind group 0.  A workgroup barrier ends
// every phase, so at any moment one wavefront of each SIMD is in its MMA phase with all
// its operands in registers while its sibling reads LDS and issues loads: the matrix
// pipe never waits for an LDS read or for the issue of a load, which is what the
// lock-step loop spends its time on (there every wavefront reads fragments and
// issues MFMAs in the same rhythm, so LDS latency and load issue are exposed on all
// four SIMDs at once).
//
//   phase      0       1       2       3       4     ...
//   group 0  MEM(0)  MMA(0)  MEM(1)  MMA(1)  MEM(2)
//   group 1    -     MEM(0)  MMA(0)  MEM(1)  MMA(1)
//
// Ring: block i lives in stage i % 2, as three operand tiles: the upper half of A (read
// by group 0 only, in phase 2i), the lower half of A (group 1 only, phase 2i + 1) and B
// (both).  Issuing a direct load costs the issuing wavefront 60-80 clocks (the load
// path of the CU accepts one 1 KiB instruction every 20-30 clocks and backs up into the
// instruction stream), so the 64 instructions of a block are spread evenly: eight per
// wavefront, in its MEM phase, behind its LDS reads, each part as soon as its last
// reader is done:
//   group 0, phase 2i:      B of block i + 1              (read in phases 2i + 2 and 2i + 3)
//   group 1, phase 2i + 1:  lower A of block i + 1        (read by group 1 in phase 2i + 3)
//                           upper A of block i + 2        (read by group 0 in phase 2i + 4)
// so every load has two phases or more to land.  A wavefront waits for its own loads
// (vmcnt counts them in order, so the newest may stay in flight) in front of the barrier
// that precedes the phase that reads them.
//
// Loads are addressed with a scalar base and one 32-bit per-lane offset per operand
// (global_load_lds_dwordx4 v, s[..]): the LDS swizzle of a lane's 16-byte chunk does
// not depend on which of its wavefront's instructions carries it, so all of them
// share one offset register and differ in the scalar base only.  Rows beyond the
// matrix are redirected, per instruction, to the last 8-row group that holds a valid
// row (what they fetch feeds masked outputs only).
#pragma once
#include "gemm_dma_kernel.h"

namespace mg {


// Where one wavefront's direct loads of an operand tile come from.
struct PpAddr {
    uint32_t voff;        // this lane's byte offset from the scalar base of an instruction
    uint32_t voff_edge;   // the same with the lane's row clamped into the matrix (K-contiguous operands)
    const char *sbase;    // scalar: source of this wavefront's instruction 0 for the next K-block
    const char *sedge;    // scalar: source of the last row group that holds a valid row
    int64_t istride;      // bytes between consecutive instructions of this wavefront
    int edge_from;        // instructions t >= edge_from reach beyond the matrix (PERW: none)
};

// Direct loads of one operand tile, issued by NWI wavefronts.
template <bool KC, int ROWS, int BK, int NWI>
struct PpLoad {
    using Lay = DmaOp<KC, ROWS, BK, NWI>;   // LDS layout, swizzle, fragment reads
    static constexpr int PERW = Lay::PERW;
    static constexpr int ROW_BYTES = Lay::ROW_BYTES;
    static constexpr int RPI = 1024 / ROW_BYTES;   // LDS rows written by one load instruction
    static_assert(1024 % ROW_BYTES == 0 && RPI >= 1, "an instruction covers whole LDS rows");
    // the swizzle of LDS row r must not depend on the instruction index t (r = (t * NWI + wi) * RPI + ...)
    static_assert(KC ? ((RPI * NWI) / (256 / ROW_BYTES)) % Lay::CPR == 0 : (RPI * NWI) % 4 == 0,
                  "swizzle varies between a wavefront's instructions");

    // base: first element of the matrix (batch applied); row0/nrows: tile origin and matrix
    // extent along the non-K axis; k0: first k of the first ring block.
    static __device__ __forceinline__ void init(PpAddr &q, const uint16_t *base, int64_t ld, int row0, int nrows,
                                                int k0, int wi, int lane) {
        const int o = lane * 16;
        const int r_in = o / ROW_BYTES;                 // LDS row of this lane inside an instruction
        const int chunk = (o % ROW_BYTES) / 16;
        const int r0 = wi * RPI + r_in;                 // LDS row of instruction 0 (the swizzle's argument)
        const int lc = chunk ^ Lay::swz(r0);
        if constexpr (KC) {
            // a (half) tile that starts beyond the matrix is read as if it started at the last
            // row group that holds a valid row
            row0 = min(row0, ((nrows - 1) / RPI) * RPI);
            q.voff = (uint32_t)((int64_t)r_in * ld * 2 + lc * 16);
            q.sbase = (const char *)(base + (int64_t)(row0 + wi * RPI) * ld + k0);
            q.istride = (int64_t)NWI * RPI * ld * 2;
            const int nv = nrows - row0;                // valid rows of this tile (>= 1)
            q.edge_from = PERW;
#pragma unroll
            for (int t = PERW - 1; t >= 0; t--)
                if ((t * NWI + wi) * RPI + RPI > nv) q.edge_from = t;
            const int rbc = ((min(nv, ROWS) - 1) / RPI) * RPI;     // last row group with a valid row
            const int rin_c = min(r_in, nv - 1 - rbc);
            q.voff_edge = (uint32_t)((int64_t)rin_c * ld * 2 + lc * 16);
            q.sedge = (const char *)(base + (int64_t)(row0 + rbc) * ld + k0);
        } else {
            const int limit = ((nrows + 7) & ~7) - 8;   // last 16-byte chunk that starts inside a row
            row0 = min(row0, limit);
            const int col = min(row0 + lc * 8, limit) - row0;
            q.voff = q.voff_edge = (uint32_t)((int64_t)r_in * ld * 2 + col * 2);
            q.sbase = q.sedge = (const char *)(base + (int64_t)(k0 + wi * RPI) * ld + row0);
            q.istride = (int64_t)NWI * RPI * ld * 2;
            q.edge_from = PERW;
        }
    }

    // Issue instructions T0 .. T1-1 of this wavefront's loads of one K-block into the LDS
    // region at byte address dst (wave-uniform).
    template <int T0, int T1>
    static __device__ __forceinline__ void issue_part(const PpAddr &q, uint32_t dst, int wi) {
        const char *sb = q.sbase + (int64_t)T0 * q.istride;
        if (!KC || q.edge_from >= PERW) {
#pragma unroll
            for (int t = T0; t < T1; t++) {
                const uint32_t m0v = dst + (t * NWI + wi) * 1024;
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(q.voff), "s"(sb)
                             : "memory", "m0");
                sb += q.istride;
            }
        } else {
#pragma unroll
            for (int t = T0; t < T1; t++) {
                const uint32_t m0v = dst + (t * NWI + wi) * 1024;
                const bool e = t >= q.edge_from;
                const char *s = e ? q.sedge : sb;
                const uint32_t v = e ? q.voff_edge : q.voff;
                asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(m0v), "v"(v), "s"(s)
                             : "memory", "m0");
                sb += q.istride;
            }
        }
    }
    // next K-block
    static __device__ __forceinline__ void advance(PpAddr &q, int64_t kstep_bytes) {
        q.sbase += kstep_bytes;
        q.sedge += kstep_bytes;
    }
    static __device__ __forceinline__ void issue(PpAddr &q, uint32_t dst, int64_t kstep_bytes, int wi) {
        issue_part<0, PERW>(q, dst, wi);
        advance(q, kstep_bytes);
    }
};

// With a short K loop the tiles of a round finish together and their C stores meet the HBM
// write rate all at once (8192 x 3072 x 768: 64 MB in one burst, 11 us of a 27 us round), while
// memory idles during the K loops.  Spreading the starts of the first round over one K loop
// spreads the stores of every later round too; the early finishers take the tiles of the
// partial last round.  Workgroups are handed to the eight XCDs in turn and inside an XCD to
// its CUs in turn, so id / 8 walks the CUs of an XCD: neighbours get consecutive phases.
__device__ __forceinline__ void stagger_start(const GemmParams &p) {
    if (p.stagger_clk <= 0) return;
    const unsigned bid = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
    if (bid >= (unsigned)p.stagger_blocks) return;
    const unsigned phase = (bid >> 3) & 7;
    const int naps = (int)(((int64_t)p.stagger_clk * phase) >> 13);   // about 1024 clocks a nap
    for (int i = 0; i < naps; i++) __builtin_amdgcn_s_sleep(16);
}

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, bool ACT = false>
__global__ void __launch_bounds__(WGM *WGN * 64)
gemm_pp_kernel(const GemmParams p) {
    constexpr bool A_KC = (LAYOUT != L_TN);
    constexpr bool B_KC = (LAYOUT == L_NT);
    constexpr int NW = WGM * WGN;
    constexpr int NWI = NW / 2;               // wavefronts of one group
    constexpr int WTM = BM / WGM, WTN = BN / WGN;
    constexpr int TM = WTM / 32, TN = WTN / 32;
    constexpr int KK = BK / 16;
    static_assert(NW == 8 && WGM == 2, "two groups of four wavefronts, group = wave / 4 = upper / lower half");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "tile shape");
    // one ring stage: upper half of A, lower half of A, B
    using OA = DmaOp<A_KC, BM / 2, BK, NWI>;
    using OB = DmaOp<B_KC, BN, BK, NWI>;
    using LA = PpLoad<A_KC, BM / 2, BK, NWI>;
    using LB = PpLoad<B_KC, BN, BK, NWI>;
    constexpr int STAGE_BYTES = 2 * OA::BYTES + OB::BYTES;
    static_assert(STAGE_BYTES == (BM + BN) * BK * 2, "stage size");
    constexpr int NLA = LA::PERW, NLB = LB::PERW;   // direct loads per wavefront: half of A, B

    extern __shared__ __attribute__((aligned(1024))) char dsm[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WGN, wave_n = wave % WGN;
    const int wi = wave & (NWI - 1);
    const int grp = wave / NWI;              // == wave_m: group 0 owns the upper half of the tile

    stagger_start(p);
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

    // group 0 loads B, group 1 both halves of A: eight instructions per wavefront and block
    static_assert(NLB == 2 * NLA, "the two groups issue the same number of loads");
    PpAddr q0, q1;   // group 0: B (q1 unused); group 1: upper half of A, lower half of A
    if (grp == 0) {
        LB::init(q0, B, p.ldb, n0, p.N, kdma, wi, lane);
        q1 = q0;
    } else {
        LA::init(q0, A, p.lda, m0, p.M, kdma, wi, lane);
        LA::init(q1, A, p.lda, m0 + BM / 2, p.M, kdma, wi, lane);
    }
    const int64_t a_step = A_KC ? BK * 2 : (int64_t)BK * p.lda * 2;
    const int64_t b_step = B_KC ? BK * 2 : (int64_t)BK * p.ldb * 2;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    int a_off[TM], b_off[TN];
#pragma unroll
    for (int i = 0; i < TM; i++) a_off[i] = wave_m * OA::BYTES + OA::frag_off(i * 32, lane);
#pragma unroll
    for (int j = 0; j < TN; j++) b_off[j] = 2 * OA::BYTES + OB::frag_off(wave_n * WTN + j * 32, lane);

    u32x4 af[KK][TM], bf[KK][TN];
    auto read_block = [&](int stage) {
        const char *sp = dsm + stage * STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
#pragma unroll
            for (int i = 0; i < TM; i++) af[kk][i] = OA::frag(sp, a_off[i], kk, lane, i * 32);
#pragma unroll
            for (int j = 0; j < TN; j++) bf[kk][j] = OB::frag(sp, b_off[j], kk, lane, wave_n * WTN + j * 32);
        }
    };
    auto mma_block = [&]() {
#pragma unroll
        for (int kk = 0; kk < KK; kk++)
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++) acc[i][j] = mfma32<DT>(af[kk][i], bf[kk][j], acc[i][j]);
    };
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void_t *)dsm;
    auto issue_b = [&](int stage) { LB::issue(q0, lds_base + stage * STAGE_BYTES + 2 * OA::BYTES, b_step, wi); };
    auto issue_a_upper = [&](int stage) { LA::issue(q0, lds_base + stage * STAGE_BYTES, a_step, wi); };
    auto issue_a_lower = [&](int stage) { LA::issue(q1, lds_base + stage * STAGE_BYTES + OA::BYTES, a_step, wi); };

    if (krem > 0) {
        // [kbeg, kbeg + krem): through registers into stage 0, zero-filled to BK; every
        // wavefront multiplies it in step with the others, before the groups part.
        OA::template fill_tail<NW * 64>(dsm, A, p.lda, m0, p.M, kbeg, kbeg + krem, tid);
        OA::template fill_tail<NW * 64>(dsm + OA::BYTES, A, p.lda, m0 + BM / 2, p.M, kbeg, kbeg + krem, tid);
        OB::template fill_tail<NW * 64>(dsm + 2 * OA::BYTES, B, p.ldb, n0, p.N, kbeg, kbeg + krem, tid);
        __syncthreads();
        read_block(0);
        mma_block();
        __syncthreads();   // all reads of stage 0 done before the ring overwrites it
    }

    // Prologue.  Group 0: B of blocks 0 and 1.  Group 1: both halves of A of block 0 and the
    // upper half of block 1 (its MEM(0) issues the lower half of block 1, like every MEM(i)).
    // Each waits for its share of block 0.
    if (grp == 0) {
        if (nkb > 0) issue_b(0);
        if (nkb > 1) {
            issue_b(1);
            wait_dma_and_barrier<NLB>();
        } else {
            wait_dma_and_barrier<0>();
        }
    } else {
        if (nkb > 0) {
            issue_a_upper(0);
            issue_a_lower(0);
        }
        if (nkb > 1) {
            issue_a_upper(1);
            wait_dma_and_barrier<NLA>();
        } else {
            wait_dma_and_barrier<0>();
        }
        if (nkb > 0) asm volatile("s_barrier" ::: "memory");   // group 1 sits out phase 0
    }
    __builtin_amdgcn_sched_barrier(0);

    for (int i = 0; i < nkb; i++) {
        // ---- MEM(i): operands of block i into registers, and the loads that refill what has become
        // free - one after the other, not interleaved: a direct load is not issued while LDS reads
        // of its own wavefront are outstanding, so loads between the reads serialise the two ----
        int newest = 0;   // loads issued in this phase
        auto issue_phase = [&]() {
            if (grp == 0) {
                if (i >= 1 && i + 1 < nkb) {
                    issue_b((i + 1) & 1);
                    newest = NLB;
                }
            } else {
                if (i + 1 < nkb) {
                    issue_a_lower((i + 1) & 1);
                    newest = NLA;
                }
                if (i + 2 < nkb) {
                    issue_a_upper(i & 1);
                    newest = 2 * NLA;
                }
            }
        };
        // Odd wavefronts issue their loads before their LDS reads, even ones after: the load path
        // takes the loads of two wavefronts while the LDS serves the reads of the other two,
        // instead of all four queueing for the one and then for the other (8192^3 TN, whose
        // transposing reads make this phase the longer one: 838 -> 793 us).
        if (wi & 1) {
            issue_phase();
            __builtin_amdgcn_sched_barrier(0);
            read_block(i & 1);
        } else {
            read_block(i & 1);
            __builtin_amdgcn_sched_barrier(0);
            issue_phase();
        }
        __builtin_amdgcn_sched_barrier(0);
        // Group 1: the upper half of A of block i + 1, which group 0 reads next, has landed -
        // everything older than the loads of this phase.  Group 0 has nothing to confirm here.
        if (grp == 1) {
            if (newest == 2 * NLA) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * NLA) : "memory");
            else if (newest == NLA) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLA) : "memory");
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        // ---- MMA(i) ----
        __builtin_amdgcn_s_setprio(1);
        mma_block();
        __builtin_amdgcn_s_setprio(0);
        __builtin_amdgcn_sched_barrier(0);
        // Group 0: B of block i + 1 has landed.  Group 1: the lower half of A of block i + 1, which
        // it reads itself next (every wavefront of the group reads what the others loaded); the
        // upper half of block i + 2 behind it may still be on its way.
        if (grp == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        else if (newest == 2 * NLA) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(NLA) : "memory");
        else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if (grp == 0 || i + 1 < nkb) asm volatile("s_barrier" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
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

template <int LAYOUT, int DT, int BM, int BN, int BK, int WGM, int WGN, bool ACT = false>
hipError_t launch_gemm_pp(const GemmParams &p, dim3 grid, hipStream_t stream, KernelQuery *query = nullptr) {
    using TT = DmaTraits<LAYOUT, BM, BN, BK, WGM, WGN, 2>;
    auto kern = gemm_pp_kernel<LAYOUT, DT, BM, BN, BK, WGM, WGN, ACT>;
    static std::atomic<uint64_t> lds_allowed{0};
    hipError_t e = allow_dynamic_lds((const void *)kern, TT::LDS_BYTES, lds_allowed);
    if (e != hipSuccess) return e;
    if (query) return query_kernel((const void *)kern, TT::NTHREADS, TT::LDS_BYTES, query);
    hipLaunchKernelGGL(kern, grid, dim3(TT::NTHREADS), TT::LDS_BYTES, stream, p);
    return hipGetLastError();
}

}  // namespace mg
