// Skinny-M GEMM on the matrix cores, NT layout: C[M,N] = A[M,K] . B[N,K]^T with M <= 64.
//
// Between the 8 rows the v_dot2 stream (gemv_kernel.h) can hold and the shapes the tiled
// kernels are built for, the product is still a stream over B - 50257 x 768 weights are 77 MB,
// 63 rows of activations 97 KB - but too much arithmetic for the vector ALUs.  The tiled
// kernels stage B through a workgroup-wide ring of K-blocks and are capped by the bytes that
// ring keeps in flight (3.4-4.2 TB/s on this shape).  Here every wavefront streams its own 32
// rows of B (32 output columns) by itself: a phase is KP k of those rows, fetched with
// 16-byte-per-lane loads that each cover whole 128- or 256-byte pieces of rows, DEPTH phases
// are requested before the first is used, and a phase passes through a buffer in LDS that
// belongs to the wavefront alone - written as it arrived, read back as MFMA operands (a lane of
// v_mfma_f32_32x32x16 holds 8 consecutive k of one column: 16 bytes of one row of B) - so no
// barrier stands between the stream and the matrix cores.  Reading the operands straight from
// global memory, a lane per row, needs no LDS at all but fetches 32 bytes per row and
// instruction: measured 24.4 us against 17.9 us for 7 x 50257 x 768.  A (padded to TMB blocks
// of 32 rows) sits in LDS whole, rows padded by 16 bytes; shapes whose A does not fit beside
// the phase buffers go to the tiled kernels (a version that swapped A in 256 k at a time had to
// drain the stream at every swap, because waiting for the newest loads waits for all older
// ones: 63 rows 29.7 us against 24.7 us, beyond 96 rows slower than the tiled kernels).
//
// Role in the reference: the same `Matmul` entry (kernels.py:232-315), which pads M to its
// tile (autograd.py:234-236); this is the tile for 5 <= M <= 64 with a wide N.
#pragma once
#include "gemm_dma_kernel.h"   // static_for

namespace mg {

struct SkinnyParams {
    const uint16_t *A;
    const uint16_t *B;
    float *C;
    const float *bias;
    int64_t lda, ldb, ldc;
    int M, N, K;
    int beta;
};

constexpr int SKINNY_LDS_LIMIT = 160 * 1024;

// LDS bytes: one phase buffer of B per wavefront (32 rows of KP k each, rows padded by 16 bytes), then
// TMB * 32 rows of A over K rounded up to a phase, padded likewise
inline int skinny_lds_bytes(int tmb, int nw, int kp, int k) {
    const int kpad = (k + kp - 1) / kp * kp;
    return nw * 32 * (kp * 2 + 16) + tmb * 32 * (kpad * 2 + 16);
}

// NW: wavefronts per workgroup (32 output columns each).  KP: k per phase of B (64 or 128).
// DEPTH: phases requested ahead.
template <int DT, int TMB, int NW, int KP, int DEPTH>
__global__ void __launch_bounds__(NW * 64, 2)
skinny_nt_kernel(const SkinnyParams p) {
    constexpr int SKINNY_THREADS = NW * 64;
    constexpr int SKINNY_COLS_PER_WG = NW * 32;
    constexpr int STEPS = KP / 16;             // MFMA k-steps per phase
    constexpr int CPR = KP / 8;                // 16-byte chunks per row of a phase
    constexpr int RPI = 64 / CPR;              // rows one load instruction covers
    constexpr int NLD = 32 / RPI;              // load instructions per phase
    constexpr int BROW = KP * 2 + 16;          // bytes per row of a phase buffer
    constexpr int ROWS = TMB * 32;
    extern __shared__ __attribute__((aligned(16))) char lds[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int h = lane >> 5;
    const int nphase = (p.K + KP - 1) / KP;
    const int kpad = nphase * KP;
    const int pitch = kpad * 2 + 16;           // bytes per LDS row of A
    char *lds_b = lds + wave * 32 * BROW;
    char *lds_a = lds + NW * 32 * BROW;

    // ---- B: coalesced loads, lane l takes 16 bytes at chunk l % CPR of row l / CPR + RPI i ----
    const int n0 = blockIdx.x * SKINNY_COLS_PER_WG + wave * 32;
    const int lrow = lane / CPR, lch = lane % CPR;
    const uint16_t *bsrc[NLD];
#pragma unroll
    for (int i = 0; i < NLD; i++) bsrc[i] = p.B + (int64_t)min(n0 + lrow + RPI * i, p.N - 1) * p.ldb + lch * 8;
    u32x4 b[DEPTH][NLD];
    auto load_phase = [&](int ph, auto slot_c) {
        constexpr int slot = decltype(slot_c)::value;
        const bool inside = ph * KP + lch * 8 < p.K;
#pragma unroll
        for (int i = 0; i < NLD; i++)
            b[slot][i] = inside ? *(const u32x4 *)(bsrc[i] + ph * KP) : u32x4{0u, 0u, 0u, 0u};
    };

    // ---- A into LDS; B's first phases are requested right behind A's first loads (A is small
    // and soon in L2) ----
    {
        const int cpr = kpad / 8;              // 16-byte chunks per row
        const int total = ROWS * cpr;
        for (int c0 = 0; c0 < total; c0 += SKINNY_THREADS * 4) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int c = c0 + u * SKINNY_THREADS + tid;
                const int row = c / cpr, ch = c - row * cpr;
                v[u] = u32x4{0u, 0u, 0u, 0u};
                if (c < total && row < p.M && ch * 8 < p.K) v[u] = *(const u32x4 *)(p.A + (int64_t)row * p.lda + ch * 8);
            }
            if (c0 == 0) {
                static_for<0, DEPTH>([&](auto d) {
                    if (decltype(d)::value < nphase) load_phase(decltype(d)::value, d);
                });
            }
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const int c = c0 + u * SKINNY_THREADS + tid;
                const int row = c / cpr, ch = c - row * cpr;
                if (c < total) *(u32x4 *)(lds_a + row * pitch + ch * 16) = v[u];
            }
        }
    }
    __syncthreads();

    f32x16 acc[TMB];
#pragma unroll
    for (int i = 0; i < TMB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.f;

    // MFMA operands: lane l holds row l % 32 of its block, 8 k at 16 s + 8 (l / 32)
    const char *arow = lds_a + (lane & 31) * pitch + h * 16;
    const char *bfrag = lds_b + (lane & 31) * BROW + h * 16;
    char *bdst = lds_b + lrow * BROW + lch * 16;
    for (int ph0 = 0; ph0 < nphase; ph0 += DEPTH) {
        static_for<0, DEPTH>([&](auto d) {
            constexpr int slot = decltype(d)::value;
            const int ph = ph0 + slot;
            if (ph < nphase) {
                // this wavefront's phase buffer is its own: no barrier, only its own LDS operations in order
#pragma unroll
                for (int i = 0; i < NLD; i++) *(u32x4 *)(bdst + RPI * i * BROW) = b[slot][i];
                if (ph + DEPTH < nphase) load_phase(ph + DEPTH, d);
#pragma unroll
                for (int s = 0; s < STEPS; s++) {
                    const u32x4 bf = *(const u32x4 *)(bfrag + s * 32);
#pragma unroll
                    for (int i = 0; i < TMB; i++) {
                        const u32x4 a = *(const u32x4 *)(arow + i * 32 * pitch + (ph * KP + s * 16) * 2);
                        acc[i] = mfma32<DT>(a, bf, acc[i]);
                    }
                }
            }
        });
    }

    // ---- epilogue: register r of lane l holds row (r / 4) * 8 + (l / 32) * 4 + r % 4, column l % 32 ----
    const int ncol = n0 + (lane & 31);
    if (ncol < p.N) {
        const float bv = p.bias ? p.bias[ncol] : 0.f;
#pragma unroll
        for (int i = 0; i < TMB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int m = i * 32 + (r >> 2) * 8 + h * 4 + (r & 3);
                if (m < p.M) {
                    float *dst = p.C + (int64_t)m * p.ldc + ncol;
                    float v = acc[i][r] + bv;
                    if (p.beta) v += *dst;
                    *dst = v;
                }
            }
    }
}

typedef hipError_t (*skinny_launch_fn)(const SkinnyParams &, dim3 grid, int lds_bytes, hipStream_t, KernelQuery *query);

template <int DT, int TMB, int NW, int KP, int DEPTH>
hipError_t launch_skinny(const SkinnyParams &p, dim3 grid, int lds_bytes, hipStream_t stream, KernelQuery *query = nullptr) {
    auto kern = skinny_nt_kernel<DT, TMB, NW, KP, DEPTH>;
    // every launch may ask for a different amount: allow the most a workgroup can have
    static std::atomic<uint64_t> lds_allowed{0};
    hipError_t e = allow_dynamic_lds((const void *)kern, 160 * 1024, lds_allowed);
    if (e != hipSuccess) return e;
    if (query) return query_kernel((const void *)kern, NW * 64, lds_bytes, query);
    hipLaunchKernelGGL(kern, grid, dim3(NW * 64), lds_bytes, stream, p);
    return hipGetLastError();
}

// [dtype][TMB - 1]: one block of 32 rows runs four wavefronts to a workgroup, two workgroups to
// a CU (17.6 against 18.4 us for 7 x 50257 x 768 with eight); two blocks need the LDS of a whole
// CU for A and run eight wavefronts
constexpr int SKINNY_MAX_TMB = 2;
constexpr int SKINNY_KP = 64;
inline int skinny_waves(int tmb) { return tmb == 1 ? 4 : 8; }
extern skinny_launch_fn skinny_table[2][SKINNY_MAX_TMB];

}  // namespace mg
