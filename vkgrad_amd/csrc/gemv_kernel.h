// Skinny-M GEMM for the NT layout: C[M,N] = A[M,K] . B[N,K]^T with M <= 8.
//
// With a handful of rows in A the product is a stream over B (the weight matrix,
// one row of K contiguous elements per output column) and the matrix cores have
// nothing to amortise: the tiled kernels fetch B in 128-byte pieces of 256 rows per
// K-block and reach about 3.8 TB/s on a cold 50257 x 768 matrix, while a plain
// streaming read of the same bytes runs at 5-6 TB/s.  This kernel reads B the way
// it lies in memory: lane l covers elements [512 c + 8 l, 512 c + 8 l + 8) of a row
// for chunk c (one 16-byte load per row and chunk), A sits in registers for exactly
// those elements, products are formed two at a time with f32 accumulation
// (v_dot2_f32_f16 / _bf16), and the 64 partial sums of a row meet through lane
// exchanges.  Four rows are reduced together: two select-and-exchange steps fold four
// values per lane into one, four more steps finish the sum, so a row costs 7/4
// exchanges per row of A instead of 6.
//
// A wavefront takes 16 consecutive rows (one contiguous span) and has all of them in
// flight before anything else happens; lane l < 16 ends up holding output column
// n0 + 4 (l / 4) + 2 (l & 1) + ((l >> 1) & 1), so a row of C is written as one 64-byte
// piece.  (Dealing the rows out evenly over exactly as many wavefronts as stay resident,
// each walking its 24 or 25 rows in two steps, was measured slower - 20.7 us against
// 17.0 us for 1 x 50257 x 768: the second step's loads wait for the first step's data.)
//
// Beyond eight rows of A the multiply-adds of a wavefront (one VALU instruction per
// pair of elements and row) take longer than the stream, and the 64 x 64 tile of the
// tiled kernels is faster; the table stops there.
//
// Role in the reference: the same `Matmul` entry (kernels.py:232-315); it has no
// separate kernel for skinny shapes and pads M to its tile instead
// (autograd.py:234-236).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gemm_kernel.h"

namespace mg {

struct GemvParams {
    const uint16_t *A;
    const uint16_t *B;
    float *C;
    const float *bias;
    int64_t lda, ldb, ldc;
    int64_t sa, sb, sc;
    int M, N, K;
    int beta;
};

constexpr int GEMV_ROWS_PER_WAVE = 16;
constexpr int GEMV_WAVES = 4;
constexpr int GEMV_ROWS_PER_WG = GEMV_ROWS_PER_WAVE * GEMV_WAVES;

// acc + a.lo * b.lo + a.hi * b.hi over one 32-bit pair of 16-bit elements, f32 accumulate
template <int DT>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float acc) {
    if constexpr (DT == D_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(h2, a), __builtin_bit_cast(h2, b), acc, false);
    } else {
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(b2, a), __builtin_bit_cast(b2, b), acc, false);
    }
}

__device__ __forceinline__ float lane_xor(float v, int mask) { return __shfl_xor(v, mask, 64); }

// Registers the kernel below needs, roughly: the 16 rows of B, the rows of A, the partial
// sums and a few addresses.  The wavefronts per SIMD asked of the compiler follow from it
// (512 registers per lane and SIMD): more resident wavefronts are more bytes in flight.
constexpr int gemv_min_waves(int mp, int nch, bool half) {
    const int regs = 64 * nch + (half ? 32 : 0) + mp * (4 * nch + (half ? 4 : 0)) + 5 * mp + 16;
    const int w = 512 / regs;
    return w < 1 ? 1 : (w > 4 ? 4 : w);
}

// MP: rows of A held (M <= MP).  NCH: full 512-element chunks of K held.  HALF: one more
// chunk of at most 256 elements follows, and the rows of B share its registers in pairs -
// lanes 0-31 hold it for the even row of a pair, lanes 32-63 for the odd one - so that
// K = 768 costs 6 registers a row instead of 8, four wavefronts fit a SIMD and the 50257 x 768
// matrix is in flight all at once (3142 wavefronts against 4096 resident).
// K <= 512 NCH + 256 HALF.
template <int DT, int MP, int NCH, bool HALF>
__global__ void __launch_bounds__(GEMV_WAVES * 64, gemv_min_waves(MP, NCH, HALF)) gemv_nt_kernel(const GemvParams p) {
    constexpr int NG = GEMV_ROWS_PER_WAVE / 4;                         // groups of four rows
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t zb = blockIdx.z;
    const uint16_t *A = p.A + zb * p.sa;
    const uint16_t *B = p.B + zb * p.sb;
    float *C = p.C + zb * p.sc;
    const int n0 = (blockIdx.x * GEMV_WAVES + wave) * GEMV_ROWS_PER_WAVE;
    if (n0 >= p.N) return;
    const bool upper = lane >= 32;
    const int kh = NCH * 512 + (lane & 31) * 8;                        // this lane's elements of the half chunk

    // the stream first: everything the registers hold goes out before A is touched
    uint4 b[NG][4][NCH];
    uint4 bh[NG][2];
#pragma unroll
    for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const int row = n0 + g * 4 + r;
#pragma unroll
            for (int c = 0; c < NCH; c++) {
                const int k = c * 512 + lane * 8;
                b[g][r][c] = make_uint4(0u, 0u, 0u, 0u);
                if (row < p.N && k < p.K) b[g][r][c] = *reinterpret_cast<const uint4 *>(B + (int64_t)row * p.ldb + k);
            }
        }
        if constexpr (HALF) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const int row = n0 + g * 4 + 2 * j + (upper ? 1 : 0);
                bh[g][j] = make_uint4(0u, 0u, 0u, 0u);
                if (row < p.N && kh < p.K) bh[g][j] = *reinterpret_cast<const uint4 *>(B + (int64_t)row * p.ldb + kh);
            }
        }
    }

    // this lane's elements of every row of A
    uint4 a[MP][NCH];
    uint4 ah[MP];
#pragma unroll
    for (int m = 0; m < MP; m++) {
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int k = c * 512 + lane * 8;
            a[m][c] = make_uint4(0u, 0u, 0u, 0u);
            if (m < p.M && k < p.K) a[m][c] = *reinterpret_cast<const uint4 *>(A + (int64_t)m * p.lda + k);
        }
        if constexpr (HALF) {
            ah[m] = make_uint4(0u, 0u, 0u, 0u);
            if (m < p.M && kh < p.K) ah[m] = *reinterpret_cast<const uint4 *>(A + (int64_t)m * p.lda + kh);
        }
    }

    float res[MP];
#pragma unroll
    for (int m = 0; m < MP; m++) res[m] = 0.f;
#pragma unroll
    for (int g = 0; g < NG; g++) {
        float acc[MP][4];
#pragma unroll
        for (int m = 0; m < MP; m++)
#pragma unroll
            for (int r = 0; r < 4; r++) acc[m][r] = 0.f;
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
            for (int c = 0; c < NCH; c++) {
                const uint4 bv = b[g][r][c];
#pragma unroll
                for (int m = 0; m < MP; m++) {
                    float t = acc[m][r];
                    t = dot2<DT>(a[m][c].x, bv.x, t);
                    t = dot2<DT>(a[m][c].y, bv.y, t);
                    t = dot2<DT>(a[m][c].z, bv.z, t);
                    t = dot2<DT>(a[m][c].w, bv.w, t);
                    acc[m][r] = t;
                }
            }
        if constexpr (HALF) {
#pragma unroll
            for (int j = 0; j < 2; j++) {
                const uint4 bv = bh[g][j];
#pragma unroll
                for (int m = 0; m < MP; m++) {
                    float t = 0.f;
                    t = dot2<DT>(ah[m].x, bv.x, t);
                    t = dot2<DT>(ah[m].y, bv.y, t);
                    t = dot2<DT>(ah[m].z, bv.z, t);
                    t = dot2<DT>(ah[m].w, bv.w, t);
                    acc[m][2 * j] += upper ? 0.f : t;
                    acc[m][2 * j + 1] += upper ? t : 0.f;
                }
            }
        }
        // fold the four rows: after the two exchanges a lane holds the partial sum of row
        // 2 (lane & 1) + ((lane >> 1) & 1) of the group, summed over its quad of lanes
        const bool odd = lane & 1, high = lane & 2;
#pragma unroll
        for (int m = 0; m < MP; m++) {
            const float keep0 = odd ? acc[m][2] : acc[m][0], give0 = odd ? acc[m][0] : acc[m][2];
            const float keep1 = odd ? acc[m][3] : acc[m][1], give1 = odd ? acc[m][1] : acc[m][3];
            const float w0 = keep0 + lane_xor(give0, 1);
            const float w1 = keep1 + lane_xor(give1, 1);
            float u = (high ? w1 : w0) + lane_xor(high ? w0 : w1, 2);
            u += lane_xor(u, 4);
            u += lane_xor(u, 8);
            u += lane_xor(u, 16);
            u += lane_xor(u, 32);
            if (((lane >> 2) & 3) == g) res[m] = u;
        }
    }
    if (lane < 16) {
        const int col = n0 + 4 * (lane >> 2) + 2 * (lane & 1) + ((lane >> 1) & 1);
        if (col < p.N) {
            const float bv = p.bias ? p.bias[col] : 0.f;
#pragma unroll
            for (int m = 0; m < MP; m++) {
                if (m < p.M) {
                    float *dst = C + (int64_t)m * p.ldc + col;
                    float v = res[m] + bv;
                    if (p.beta) v += *dst;
                    *dst = v;
                }
            }
        }
    }
}

typedef hipError_t (*gemv_launch_fn)(const GemvParams &, dim3 grid, hipStream_t, KernelQuery *query);

template <int DT, int MP, int NCH, bool HALF>
hipError_t launch_gemv(const GemvParams &p, dim3 grid, hipStream_t stream, KernelQuery *query = nullptr) {
    if (query) return query_kernel((const void *)gemv_nt_kernel<DT, MP, NCH, HALF>, GEMV_WAVES * 64, 0, query);
    hipLaunchKernelGGL((gemv_nt_kernel<DT, MP, NCH, HALF>), grid, dim3(GEMV_WAVES * 64), 0, stream, p);
    return hipGetLastError();
}

// [dtype][log2 MP][K class]: K <= 512, 768, 1024, 2048
extern gemv_launch_fn gemv_table[2][4][4];
__host__ inline int gemv_k_class(int k) { return k <= 512 ? 0 : k <= 768 ? 1 : k <= 1024 ? 2 : 3; }

}  // namespace mg
