// Attention's dS in one kernel: the dP = dOut V^T product of every head (reference call site
// transformer.py:171-173) and the softmax backward that follows it (attn_softmax_bwd,
// tkernels.py:167-187), without the f32 dP matrix in between:
//
//   dS[b][i][j] = narrow(scale * P[b][i][j] * (sum_d dOut[b][i][d] V[b][j][d] - rowsub[b][i]))
//
// rowsub[i] = sum_j P[i][j] dP[i][j], which the caller forms as sum_d dOut[i][d] Out[i][d]
// (mg_tk_attn_rowdot).  The contraction is only as long as a head is wide (64 for GPT-2), so a
// tiled GEMM has one K-block per tile and spends its time waiting: for the operands, and in
// an epilogue version of this formula once more for P.  Here nothing waits twice: the dOut
// fragments are 16-byte loads straight from memory (a lane of v_mfma_f32_32x32x16 holds 8
// consecutive k of one row, which is how the tensor lies in memory), the V rows of the
// workgroup's keys pass through LDS once, and P and rowsub are requested before the first MFMA.
//
// What bounds such a kernel on this chip is the number of vector memory instructions, not their
// bytes: a 4-byte and a 16-byte access per lane cost a wavefront about the same.  So a
// wavefront owns 32 queries x 256 keys, eight accumulator blocks that share the dOut fragments,
// and since the key an accumulator column stands for is decided by the row of V its lane
// loaded, block t takes the keys 8n + t (n = lane % 32): a lane then holds eight neighbouring
// keys of each of its rows, and P arrives and dS leaves as one 16-byte access per lane and row
// (T must be a multiple of 8 for their alignment).  rowsub is one load per wavefront, handed
// round by lane reads.  Four wavefronts (128 queries) share a workgroup.
//
// With `causal` set, a wavefront whose keys all lie beyond its queries neither computes nor
// writes (P is zero there, and so is dS: the caller keeps the buffer zeroed); inside computed
// blocks the masked entries come out as zero because P is.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"

#include "ew_common.h"

namespace mg {

typedef _Float16 ak_half8 __attribute__((ext_vector_type(8)));
typedef __bf16 ak_bf8 __attribute__((ext_vector_type(8)));
typedef float ak_f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t ak_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t ak_u32x2 __attribute__((ext_vector_type(2)));
typedef short ak_short4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) ak_short4 ak_lds_short4;

// Transposing LDS read (ds_read_b64_tr_b16): within each group of 16 lanes the 16 x 8-byte pieces
// addressed by the lanes form a 4 x 16 matrix of 16-bit elements (lane j supplies row j / 4,
// columns 4 (j % 4) .. + 3); lane j receives column j.
__device__ __forceinline__ ak_u32x2 ak_read_tr(const uint16_t *p) {
    ak_short4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((ak_lds_short4 *)p);
    return __builtin_bit_cast(ak_u32x2, v);
}

template <int DT>
__device__ __forceinline__ ak_f32x16 ak_mfma(ak_u32x4 a, ak_u32x4 b, ak_f32x16 c) {
    if constexpr (DT == MG_F16)
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(ak_half8, a), __builtin_bit_cast(ak_half8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(ak_bf8, a), __builtin_bit_cast(ak_bf8, b), c, 0, 0, 0);
}

template <int DT>
__device__ __forceinline__ uint32_t ak_narrow(float x) {
    if constexpr (DT == MG_F16) return __builtin_bit_cast(uint16_t, (_Float16)x);
    else return __builtin_bit_cast(uint16_t, (__bf16)x);   // round to nearest even, one instruction on gfx950
}
template <int DT>
__device__ __forceinline__ float ak_widen(uint32_t b) {
    if constexpr (DT == MG_F16) return (float)__builtin_bit_cast(_Float16, (uint16_t)b);
    else return __builtin_bit_cast(float, b << 16);
}

constexpr int DS_BM = 128, DS_BN = 256;   // workgroup tile: 4 wavefronts of 32 queries x 256 keys

template <int DT, int HD>
__global__ void __launch_bounds__(256, 2)
k_attn_ds(const uint16_t *dout, const uint16_t *v, const uint16_t *p16, const float *rowsub, uint16_t *ds16, int T,
          float scale, int causal) {
    constexpr int KK = HD / 16, NB = DS_BN / 32;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t b = blockIdx.z;
    const int i0 = blockIdx.y * DS_BM + wave * 32;   // this wavefront's first query
    const int j0 = blockIdx.x * DS_BN;               // and first key
    if (causal && j0 > blockIdx.y * DS_BM + DS_BM - 1) return;   // the whole workgroup lies beyond the diagonal
    const uint16_t *db = dout + b * (int64_t)T * HD;
    const uint16_t *vb = v + b * (int64_t)T * HD;
    // The 256 rows of V go to LDS once per workgroup, in whole 128-byte-or-longer runs (the
    // strided 16-byte operand loads of four wavefronts were what this kernel spent its time
    // on).  Key j0 + 8 n + t is placed at row t * 32 + n, so a block's 32 rows are neighbours;
    // 16 bytes of padding per row spread a fragment read's 16 lanes over all banks.
    // (Heads 128 wide would need more than the 64 KiB a static array may hold: they keep the
    // direct loads.)
    constexpr bool STAGE = HD <= 64;
    constexpr int CPR = HD / 8, PITCH = HD * 2 + 16;   // 16-byte chunks per row, bytes per LDS row
    __shared__ __attribute__((aligned(16))) char vt[STAGE ? DS_BN * PITCH : 16];
    if constexpr (STAGE) {
        for (int c = threadIdx.x; c < DS_BN * CPR; c += 256) {
            const int key = c / CPR, part = c % CPR;
            const ak_u32x4 x = *reinterpret_cast<const ak_u32x4 *>(vb + (int64_t)min(j0 + key, T - 1) * HD + part * 8);
            *reinterpret_cast<ak_u32x4 *>(vt + ((key & 7) * 32 + (key >> 3)) * PITCH + part * 16) = x;
        }
        __syncthreads();
    }
    if (i0 >= T) return;
    if (causal && j0 > i0 + 31) return;              // every key beyond every query of this wavefront

    // MFMA operands: lane l holds row l % 32, k = 8 * (l / 32) .. + 7 of each 16-wide k step
    const int fr = lane & 31, fk = (lane >> 5) * 8;
    const uint16_t *ap = db + (int64_t)min(i0 + fr, T - 1) * HD + fk;
    ak_u32x4 af[KK];
#pragma unroll
    for (int kk = 0; kk < KK; kk++) af[kk] = *reinterpret_cast<const ak_u32x4 *>(ap + kk * 16);
    // Accumulator register r belongs to row i0 + ro + 4 * (l / 32), ro = 8 * (r / 4) + r % 4; this
    // lane's keys are jc .. jc + 7, one per block.  T is a multiple of 8: all eight exist or none.
    const int rl = i0 + (lane >> 5) * 4;
    const int jc = j0 + 8 * fr;
    const bool col_ok = jc < T;
    const int64_t cell = b * (int64_t)T * T + (col_ok ? jc : 0);
    const bool whole = i0 + 32 <= T;                 // no row of this wavefront beyond the matrix
    const float rs_lane = rowsub[b * (int64_t)T + min(i0 + fr, T - 1)] * scale;
    ak_u32x4 pp[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int ro = (r >> 2) * 8 + (r & 3);
        const int row = whole ? rl + ro : min(rl + ro, T - 1);
        pp[r] = *reinterpret_cast<const ak_u32x4 *>(p16 + cell + (int64_t)row * T);
    }
    ak_f32x16 acc[NB];
#pragma unroll
    for (int t = 0; t < NB; t++) {
        ak_u32x4 bf[KK];
        if constexpr (STAGE) {
            const char *bp = vt + (t * 32 + fr) * PITCH + fk * 2;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) bf[kk] = *reinterpret_cast<const ak_u32x4 *>(bp + kk * 32);
        } else {
            const uint16_t *bp = vb + (int64_t)min(j0 + 8 * fr + t, T - 1) * HD + fk;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) bf[kk] = *reinterpret_cast<const ak_u32x4 *>(bp + kk * 16);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) acc[t] = ak_mfma<DT>(af[kk], bf[kk], acc[t]);
    }
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const int ro = (r >> 2) * 8 + (r & 3);
        // rowsub of this lane's row: lanes 0-31 hold the 32 rows of the wavefront
        const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, rs_lane), ro));
        const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, rs_lane), ro + 4));
        const float rs = lane < 32 ? lo : hi;
        ak_u32x4 o;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float p0 = ak_widen<DT>(pp[r][w] & 0xffffu), p1 = ak_widen<DT>(pp[r][w] >> 16);
            o[w] = ak_narrow<DT>(p0 * (acc[2 * w][r] * scale - rs)) | (ak_narrow<DT>(p1 * (acc[2 * w + 1][r] * scale - rs)) << 16);
        }
        if (col_ok && (whole || rl + ro < T))
            *reinterpret_cast<ak_u32x4 *>(ds16 + cell + (int64_t)(rl + ro) * T) = o;
    }
}

// P of attention in one kernel: the scores = Q K^T product of every head (reference call site
// transformer.py:153-155) and the masked softmax over them (attn_softmax / attn_softmax_doc,
// tkernels.py:105-165), without the f32 score matrix in between.  The product is formed
// transposed, K Q^T: the 32 queries of a workgroup lie along the accumulator columns (one query
// per lane), the keys along the rows, so everything a softmax row needs - its maximum, its sum -
// is a reduction over a lane's own registers plus one exchange between the two half-waves.  (With
// the queries along the rows each of the 16 rows a lane holds had to be reduced over 32 lanes:
// 160 lane exchanges per wavefront, which an ablation showed to cost more than the loads.)
// The four wavefronts of a workgroup split the keys between them (256 each, so T <= 1024), meet
// once in LDS with their (maximum, sum) pairs, and each rescales and writes its own keys.  Which
// key an accumulator row stands for is decided by the row of K its lane loaded: row 8g + 4h + e
// of a block takes key 16h + 4g + e, so register r of half-wave h is key 16h + r and a lane
// writes 16 neighbouring keys of its query as two 16-byte stores per block.
// Query q (= row % T of its head) sees keys first .. q, first = 0 or seg[batch * T + q]; masked
// keys get 0.  With `causal` set, a wavefront whose keys all lie beyond its queries writes
// nothing: the caller keeps P zero there.
template <int DT, int HD>
__global__ void __launch_bounds__(256, 2)
k_attn_p(const uint16_t *q16, const uint16_t *k16, const uint32_t *seg, uint16_t *p16, int T, int H, float scale,
         int causal) {
    constexpr int KK = HD / 16, NB = 8;
    __shared__ float part_m[4][32], part_l[4][32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t b = blockIdx.y;
    const int i0 = blockIdx.x * 32;      // the workgroup's first query
    const int j0 = wave * 256;           // this wavefront's first key
    const int n = lane & 31, half = lane >> 5, fk = half * 8;
    const int q = i0 + n;                // this lane's query
    // keys that no query of this block may see: none of them, or (causal) all beyond the last query
    const bool idle = j0 >= T || (causal && j0 > i0 + 31);
    ak_f32x16 acc[NB];
    float m = -1e30f, l = 0.f;
    if (!idle) {
        const uint16_t *qb = q16 + b * (int64_t)T * HD + (int64_t)min(q, T - 1) * HD + fk;
        const uint16_t *kb = k16 + b * (int64_t)T * HD;
        ak_u32x4 bf[KK];                 // B operand: the queries
#pragma unroll
        for (int kk = 0; kk < KK; kk++) bf[kk] = *reinterpret_cast<const ak_u32x4 *>(qb + kk * 16);
        const int first = seg ? (int)seg[(b / H) * T + min(q, T - 1)] : 0;
        // A operand row n = 8g + 4h' + e of block t is key j0 + 32 t + 16 h' + 4 g + e
        const int arow = 16 * ((n >> 2) & 1) + 4 * (n >> 3) + (n & 3);
#pragma unroll
        for (int t = 0; t < NB; t++) {
            const uint16_t *ap = kb + (int64_t)min(j0 + 32 * t + arow, T - 1) * HD + fk;
            ak_u32x4 af[KK];
#pragma unroll
            for (int kk = 0; kk < KK; kk++) af[kk] = *reinterpret_cast<const ak_u32x4 *>(ap + kk * 16);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) acc[t] = ak_mfma<DT>(af[kk], bf[kk], acc[t]);
        }
        // Base-2 domain (scores times scale * log2 e): an exponential is one v_exp_f32.  A key that
        // is not seen holds -1e30 and its exponential is exactly 0 - unless no key of this
        // wavefront is seen by the query, in which case they are all 1 and the sum is wrong, but
        // then the factor below is 2^(-1e30 - max) = 0 and nothing of it is used.  (Keys >= T need
        // no test: key <= q < T for every query that is stored.)
        const float c2 = scale * 1.4426950408889634f;
        const int k0 = j0 + 16 * half;   // register r of block t: key k0 + 32 t + r
#pragma unroll
        for (int t = 0; t < NB; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = k0 + 32 * t + r;
                acc[t][r] = (key >= first && key <= q) ? acc[t][r] * c2 : -1e30f;
                m = fmaxf(m, acc[t][r]);
            }
        m = fmaxf(m, __shfl_xor(m, 32, 64));
#pragma unroll
        for (int t = 0; t < NB; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float e = __builtin_amdgcn_exp2f(acc[t][r] - m);
                acc[t][r] = e;
                l += e;
            }
        l += __shfl_xor(l, 32, 64);
    }
    if (half == 0) {
        part_m[wave][n] = m;
        part_l[wave][n] = l;
    }
    __syncthreads();
    if (idle || q >= T) return;
    const float m0 = part_m[0][n], m1 = part_m[1][n], m2 = part_m[2][n], m3 = part_m[3][n];
    const float mx = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
    const float sum = part_l[0][n] * __builtin_amdgcn_exp2f(m0 - mx) + part_l[1][n] * __builtin_amdgcn_exp2f(m1 - mx) +
                      part_l[2][n] * __builtin_amdgcn_exp2f(m2 - mx) + part_l[3][n] * __builtin_amdgcn_exp2f(m3 - mx);
    const float f = __builtin_amdgcn_exp2f(m - mx) / sum;   // (a query that sees no key does not occur: key q always is)
    uint16_t *pq = p16 + b * (int64_t)T * T + (int64_t)q * T + j0 + 16 * half;
#pragma unroll
    for (int t = 0; t < NB; t++)
#pragma unroll
        for (int u = 0; u < 2; u++) {
            ak_u32x4 o;
#pragma unroll
            for (int w = 0; w < 4; w++)
                o[w] = ak_narrow<DT>(acc[t][8 * u + 2 * w] * f) | (ak_narrow<DT>(acc[t][8 * u + 2 * w + 1] * f) << 16);
            // T is a multiple of 8: the eight keys of a store exist or none does
            if (j0 + 16 * half + 32 * t + 8 * u < T) *reinterpret_cast<ak_u32x4 *>(pq + 32 * t + 8 * u) = o;
        }
}

// Attention forward in one kernel: the one-walk P kernel above with the Out = P V product of
// every head (reference call site transformer.py:157-159) behind it, so that P is written (the
// backward pass reads it, transformer.py:165-176) but not read back.  P leaves the softmax in
// accumulator layout with the keys along the rows and one query per lane, 16 neighbouring keys
// per lane and block: narrowed, the eight keys of a 16-byte store are exactly what a lane holds
// of the B operand of v_mfma_f32_32x32x16 for the product Out^T = V^T P^T (k = keys, columns =
// queries), so the same 16-bit values that go to memory go to the matrix cores and the result
// is what a GEMM over the stored P gives, up to the order of the f32 sums.  The A operand, V^T,
// is 8 keys of one column of V per lane: every wavefront passes the 32 rows of V of a key block
// through a buffer of its own in LDS (rows padded so that the four rows and two column groups
// of a transposing read fall on different banks) and reads them back with ds_read_b64_tr_b16;
// the rows of the next block are requested before the current one is multiplied.  Key blocks
// wholly beyond the workgroup's queries hold P = 0 and are not multiplied.  The four
// wavefronts (256 keys each) then meet in LDS with their partial Out (32 queries x HD floats
// each) and the workgroup adds them in wavefront order and writes Out in f32 (head-side, the
// row term of the softmax backward reads it, autograd of transformer.py:171-176) and, if asked,
// narrowed in the merged (B*T, D) layout the projection reads (merge_heads, tkernels.py:274-286).
template <int HD>
constexpr int fwd_pitch() { return HD == 32 ? 64 : HD * 2 + 64; }   // bytes per row of V in LDS

// (heads 128 wide need 270 registers: one workgroup per CU there, two otherwise)
template <int DT, int HD>
__global__ void __launch_bounds__(256, (HD == 128 ? 1 : 2))
k_attn_fwd(const uint16_t *q16, const uint16_t *k16, const uint16_t *v16, const uint32_t *seg, uint16_t *p16,
           float *out32, uint16_t *out16, int T, int H, float scale, int causal) {
    constexpr int KK = HD / 16, NB = 8, MB = HD / 32;
    constexpr int PITCH = fwd_pitch<HD>(), VBUF = 32 * PITCH;
    constexpr int OPITCH = HD + 1;                       // floats per query of a partial Out
    constexpr int LDS_V = 4 * VBUF, LDS_O = 4 * 32 * OPITCH * 4;
    constexpr int CPR = HD / 8, RPI = 64 / CPR, NLD = 32 / RPI;   // staging of a key block: 16-byte chunks per row, rows per load, loads
    __shared__ __attribute__((aligned(16))) char smem[LDS_V > LDS_O ? LDS_V : LDS_O];
    __shared__ float part_m[4][32], part_l[4][32];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t b = blockIdx.y;
    const int i0 = blockIdx.x * 32;      // the workgroup's first query
    const int j0 = wave * 256;           // this wavefront's first key
    const int n = lane & 31, half = lane >> 5, fk = half * 8;
    const int q = i0 + n;                // this lane's query
    // keys that no query of this block sees hold P = 0: not written with `causal`, never multiplied
    const bool beyond = j0 >= T || j0 > i0 + 31;
    const bool idle = j0 >= T || (causal && j0 > i0 + 31);
    ak_f32x16 acc[NB];
    float m = -1e30f, l = 0.f;
    if (!idle) {
        const uint16_t *qb = q16 + b * (int64_t)T * HD + (int64_t)min(q, T - 1) * HD + fk;
        const uint16_t *kb = k16 + b * (int64_t)T * HD;
        ak_u32x4 bf[KK];                 // B operand: the queries
#pragma unroll
        for (int kk = 0; kk < KK; kk++) bf[kk] = *reinterpret_cast<const ak_u32x4 *>(qb + kk * 16);
        const int first = seg ? (int)seg[(b / H) * T + min(q, T - 1)] : 0;
        // A operand row n = 8g + 4h' + e of block t is key j0 + 32 t + 16 h' + 4 g + e
        const int arow = 16 * ((n >> 2) & 1) + 4 * (n >> 3) + (n & 3);
#pragma unroll
        for (int t = 0; t < NB; t++) {
            const uint16_t *ap = kb + (int64_t)min(j0 + 32 * t + arow, T - 1) * HD + fk;
            ak_u32x4 af[KK];
#pragma unroll
            for (int kk = 0; kk < KK; kk++) af[kk] = *reinterpret_cast<const ak_u32x4 *>(ap + kk * 16);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) acc[t] = ak_mfma<DT>(af[kk], bf[kk], acc[t]);
        }
        // base-2 domain, masked keys at -1e30 (see k_attn_p)
        const float c2 = scale * 1.4426950408889634f;
        const int k0 = j0 + 16 * half;   // register r of block t: key k0 + 32 t + r
#pragma unroll
        for (int t = 0; t < NB; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int key = k0 + 32 * t + r;
                acc[t][r] = (key >= first && key <= q) ? acc[t][r] * c2 : -1e30f;
                m = fmaxf(m, acc[t][r]);
            }
        m = fmaxf(m, __shfl_xor(m, 32, 64));
#pragma unroll
        for (int t = 0; t < NB; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const float e = __builtin_amdgcn_exp2f(acc[t][r] - m);
                acc[t][r] = e;
                l += e;
            }
        l += __shfl_xor(l, 32, 64);
    }
    if (half == 0) {
        part_m[wave][n] = m;
        part_l[wave][n] = l;
    }
    __syncthreads();
    ak_f32x16 oacc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[i][r] = 0.f;
    if (!idle) {
        const float m0 = part_m[0][n], m1 = part_m[1][n], m2 = part_m[2][n], m3 = part_m[3][n];
        const float mx = fmaxf(fmaxf(m0, m1), fmaxf(m2, m3));
        const float sum = part_l[0][n] * __builtin_amdgcn_exp2f(m0 - mx) + part_l[1][n] * __builtin_amdgcn_exp2f(m1 - mx) +
                          part_l[2][n] * __builtin_amdgcn_exp2f(m2 - mx) + part_l[3][n] * __builtin_amdgcn_exp2f(m3 - mx);
        const float f = __builtin_amdgcn_exp2f(m - mx) / sum;
        uint16_t *pq = p16 + b * (int64_t)T * T + (int64_t)min(q, T - 1) * T + j0 + 16 * half;
        // key blocks of this wavefront that some query of the workgroup sees (0 when all lie beyond)
        const int kend = min(min(T, j0 + 256), i0 + 32);
        const int nblk = beyond ? 0 : (kend - j0 + 31) / 32;
        // staging of V: lane l fetches chunk l % CPR of row l / CPR + RPI i of the block
        const uint16_t *vbase = v16 + b * (int64_t)T * HD;
        const int lrow = lane / CPR, lch = lane % CPR;
        char *vb = smem + wave * VBUF;
        char *vdst = vb + lrow * PITCH + lch * 16;
        // transposing read: lane (j = l % 16, g = l / 16) supplies the 8-byte piece of row 16 (g / 2) + j / 4
        // (+ 8 u, + 4 for the second read), columns 16 (g % 2) + 4 (j % 4) .. + 3, and receives column l % 32
        const int j = lane & 15, g4 = lane >> 4;
        const char *vsrc = vb + ((g4 >> 1) * 16 + (j >> 2)) * PITCH + ((g4 & 1) * 16 + (j & 3) * 4) * 2;
        ak_u32x4 vreg[NLD];
        auto load_v = [&](int t) {
#pragma unroll
            for (int i = 0; i < NLD; i++)
                vreg[i] = *reinterpret_cast<const ak_u32x4 *>(vbase + (int64_t)min(j0 + 32 * t + lrow + RPI * i, T - 1) * HD + lch * 8);
        };
        if (nblk > 0) load_v(0);
#pragma unroll
        for (int t = 0; t < NB; t++) {
            const bool mul = t < nblk;       // uniform over the wavefront
            if (mul) {
#pragma unroll
                for (int i = 0; i < NLD; i++) *reinterpret_cast<ak_u32x4 *>(vdst + RPI * i * PITCH) = vreg[i];
                if (t + 1 < nblk) load_v(t + 1);
                // a wavefront's LDS operations execute in order: the reads below see the block, and the next
                // block's writes come after them; the compiler only has to keep that order
                asm volatile("" ::: "memory");
            }
#pragma unroll
            for (int u = 0; u < 2; u++) {
                ak_u32x4 o;
#pragma unroll
                for (int w = 0; w < 4; w++)
                    o[w] = ak_narrow<DT>(acc[t][8 * u + 2 * w] * f) | (ak_narrow<DT>(acc[t][8 * u + 2 * w + 1] * f) << 16);
                // T is a multiple of 8: the eight keys of a store exist or none does
                if (q < T && j0 + 16 * half + 32 * t + 8 * u < T) *reinterpret_cast<ak_u32x4 *>(pq + 32 * t + 8 * u) = o;
                if (mul) {
#pragma unroll
                    for (int i = 0; i < MB; i++) {
                        const uint16_t *vp = reinterpret_cast<const uint16_t *>(vsrc + 8 * u * PITCH + i * 64);
                        const ak_u32x2 lo = ak_read_tr(vp);
                        const ak_u32x2 hi = ak_read_tr(reinterpret_cast<const uint16_t *>(reinterpret_cast<const char *>(vp) + 4 * PITCH));
                        oacc[i] = ak_mfma<DT>(ak_u32x4{lo[0], lo[1], hi[0], hi[1]}, o, oacc[i]);
                    }
                }
            }
            if (mul) asm volatile("" ::: "memory");
        }
    }
    __syncthreads();                         // every wavefront is done with its V buffer
    float *po = reinterpret_cast<float *>(smem);
    if (!beyond) {
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                po[(wave * 32 + n) * OPITCH + 32 * i + (r >> 2) * 8 + half * 4 + (r & 3)] = oacc[i][r];
    }
    __syncthreads();
    // wavefronts with keys to add: 0 .. nw - 1
    const int nw = min(4, min((T + 255) / 256, (i0 + 31) / 256 + 1));
    const int64_t bb = b / H, hh = b % H;
    for (int e = threadIdx.x; e < 32 * HD; e += 256) {
        const int qq = e / HD, d = e % HD;
        if (i0 + qq >= T) break;
        float sacc = 0.f;
        for (int w = 0; w < nw; w++) sacc += po[(w * 32 + qq) * OPITCH + d];
        out32[b * (int64_t)T * HD + (int64_t)(i0 + qq) * HD + d] = sacc;
        if (out16) out16[(bb * T + i0 + qq) * ((int64_t)H * HD) + hh * HD + d] = (uint16_t)ak_narrow<DT>(sacc);
    }
}

// The same for heads up to 64 wide and any T (a multiple of 8), for rows longer than the 1024 keys
// the kernel above can hold: a workgroup is four blocks of 32 queries (queries along the
// accumulator rows here, as in k_attn_ds) that walk the key tiles of 256 together, the K rows of
// a tile passing through LDS once for the 128 queries.  A row's keys never sit in the registers
// all at once, so the tiles are walked twice: the first walk keeps, per lane and row, a running
// maximum and a sum of exponentials relative to it over the lane's own keys (merged across the
// half-wave once, at the end), the second recomputes the scores and writes P.  Still no f32
// scores; K is read twice from L2.
template <int DT, int HD>
__global__ void __launch_bounds__(256, 2)
k_attn_p_tiled(const uint16_t *q16, const uint16_t *k16, const uint32_t *seg, uint16_t *p16, int T, int H, float scale,
               int causal) {
    constexpr int KK = HD / 16, NB = 8, BN = 256, BM = 128;
    constexpr int CPR = HD / 8, PITCH = HD * 2 + 16;
    __shared__ __attribute__((aligned(16))) char kt[BN * PITCH];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int64_t b = blockIdx.y;
    const int iw = blockIdx.x * BM;      // the workgroup's first query
    const int i0 = iw + wave * 32;       // this wavefront's
    const int fr = lane & 31, fk = (lane >> 5) * 8, half = lane >> 5;
    const int rl = i0 + half * 4;
    const uint16_t *kb = k16 + b * (int64_t)T * HD;
    int ntiles = (T + BN - 1) / BN;
    if (causal) ntiles = min(ntiles, (min(iw + BM, T) - 1) / BN + 1);   // tiles that hold a key <= the last query

    ak_u32x4 af[KK];
    {
        const uint16_t *qb = q16 + b * (int64_t)T * HD + (int64_t)min(i0 + fr, T - 1) * HD + fk;
#pragma unroll
        for (int kk = 0; kk < KK; kk++) af[kk] = *reinterpret_cast<const ak_u32x4 *>(qb + kk * 16);
    }
    // first seen key of row i0 + fr, held by lanes fr and fr + 32 and handed round by lane reads
    const int first_lane = seg ? (int)seg[(b / H) * T + min(i0 + fr, T - 1)] : 0;
    float mrow[16], lrow[16];
#pragma unroll
    for (int r = 0; r < 16; r++) {
        mrow[r] = -1e30f;
        lrow[r] = 0.f;
    }
    ak_f32x16 acc[NB];
    // scores of one tile for this wavefront: acc[t][r] = scale * q . k, or -1e30 where not seen
    auto tile_scores = [&](int j0) {
        const int jc = j0 + 8 * fr;
#pragma unroll
        for (int t = 0; t < NB; t++) {
            const char *bp = kt + (t * 32 + fr) * PITCH + fk * 2;
            ak_u32x4 bf[KK];
#pragma unroll
            for (int kk = 0; kk < KK; kk++) bf[kk] = *reinterpret_cast<const ak_u32x4 *>(bp + kk * 32);
#pragma unroll
            for (int r = 0; r < 16; r++) acc[t][r] = 0.f;
#pragma unroll
            for (int kk = 0; kk < KK; kk++) acc[t] = ak_mfma<DT>(af[kk], bf[kk], acc[t]);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int ro = (r >> 2) * 8 + (r & 3);
            const int q = rl + ro;
            const int flo = __builtin_amdgcn_readlane(first_lane, ro), fhi = __builtin_amdgcn_readlane(first_lane, ro + 4);
            const int first = half ? fhi : flo;
#pragma unroll
            for (int t = 0; t < NB; t++) {
                const int j = jc + t;
                acc[t][r] = (j >= first && j <= q && j < T) ? acc[t][r] * scale : -1e30f;
            }
        }
    };
    auto stage = [&](int j0) {
        for (int c = threadIdx.x; c < BN * CPR; c += 256) {
            const int key = c / CPR, part = c % CPR;
            const ak_u32x4 x = *reinterpret_cast<const ak_u32x4 *>(kb + (int64_t)min(j0 + key, T - 1) * HD + part * 8);
            *reinterpret_cast<ak_u32x4 *>(kt + ((key & 7) * 32 + (key >> 3)) * PITCH + part * 16) = x;
        }
    };
    for (int pass = 0; pass < 2; pass++) {
        for (int jt = 0; jt < ntiles; jt++) {
            const int j0 = jt * BN;
            __syncthreads();             // everybody is done with the tile before
            stage(j0);
            __syncthreads();
            if (i0 >= T || (causal && j0 > i0 + 31)) continue;   // no key of this tile is seen by this wavefront
            tile_scores(j0);
            if (pass == 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float m = mrow[r];
#pragma unroll
                    for (int t = 0; t < NB; t++) m = fmaxf(m, acc[t][r]);
                    float l = lrow[r] * __expf(mrow[r] - m);
#pragma unroll
                    for (int t = 0; t < NB; t++) l += acc[t][r] > -1e29f ? __expf(acc[t][r] - m) : 0.f;
                    mrow[r] = m;
                    lrow[r] = l;
                }
            } else {
                const int jc = j0 + 8 * fr;
                const bool col_ok = jc < T;      // T is a multiple of 8: all eight keys exist or none
                uint16_t *pb = p16 + b * (int64_t)T * T + (col_ok ? jc : 0);
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int ro = (r >> 2) * 8 + (r & 3);
                    ak_u32x4 o;
#pragma unroll
                    for (int w = 0; w < 4; w++) {
                        const float e0 = acc[2 * w][r] > -1e29f ? __expf(acc[2 * w][r] - mrow[r]) * lrow[r] : 0.f;
                        const float e1 = acc[2 * w + 1][r] > -1e29f ? __expf(acc[2 * w + 1][r] - mrow[r]) * lrow[r] : 0.f;
                        o[w] = ak_narrow<DT>(e0) | (ak_narrow<DT>(e1) << 16);
                    }
                    if (col_ok && rl + ro < T) *reinterpret_cast<ak_u32x4 *>(pb + (int64_t)(rl + ro) * T) = o;
                }
            }
        }
        if (pass == 0) {
            // merge the lanes' (maximum, sum) pairs over the 32 lanes that hold the same rows;
            // afterwards mrow is the row's maximum and lrow the reciprocal of its sum
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float m = mrow[r], l = lrow[r];
#pragma unroll
                for (int x = 16; x >= 1; x >>= 1) {
                    const float mo = __shfl_xor(m, x, 64), lo = __shfl_xor(l, x, 64);
                    const float mn = fmaxf(m, mo);
                    l = l * __expf(m - mn) + lo * __expf(mo - mn);
                    m = mn;
                }
                mrow[r] = m;
                lrow[r] = l > 0.f ? 1.0f / l : 0.f;
            }
        }
    }
}

template <int DT, int HD>
static void launch_attn_p(hipStream_t s, const void *q, const void *k, const uint32_t *seg, void *p16, int64_t nbh, int T,
                          int H, float scale, int causal) {
    // up to 1024 keys a row fits the registers of one workgroup and the one-walk kernel is faster
    // (163 against 127 us at 96 heads x 1024 x 1024 x 64: the second walk's exponentials and
    // masks cost more than the strided K loads it saves); beyond that only the tiled one exists
    if constexpr (HD <= 64) {
        if (T > 1024) {
            const dim3 grid((unsigned)((T + 127) / 128), (unsigned)nbh);
            hipLaunchKernelGGL((k_attn_p_tiled<DT, HD>), grid, dim3(256), 0, s, (const uint16_t *)q, (const uint16_t *)k,
                               seg, (uint16_t *)p16, T, H, scale, causal);
            return;
        }
    }
    const dim3 grid((unsigned)((T + 31) / 32), (unsigned)nbh);
    hipLaunchKernelGGL((k_attn_p<DT, HD>), grid, dim3(256), 0, s, (const uint16_t *)q, (const uint16_t *)k, seg,
                       (uint16_t *)p16, T, H, scale, causal);
}

template <int DT, int HD>
static void launch_attn_fwd(hipStream_t s, const void *q, const void *k, const void *v, const uint32_t *seg, void *p16,
                            float *out32, void *out16, int64_t nbh, int T, int H, float scale, int causal) {
    const dim3 grid((unsigned)((T + 31) / 32), (unsigned)nbh);
    hipLaunchKernelGGL((k_attn_fwd<DT, HD>), grid, dim3(256), 0, s, (const uint16_t *)q, (const uint16_t *)k,
                       (const uint16_t *)v, seg, (uint16_t *)p16, out32, (uint16_t *)out16, T, H, scale, causal);
}

template <int DT, int HD>
static void launch_attn_ds(hipStream_t s, const void *dout, const void *v, const void *p16, const float *rowsub, void *ds16,
                           int64_t nbh, int T, float scale, int causal) {
    const dim3 grid((unsigned)((T + DS_BN - 1) / DS_BN), (unsigned)((T + DS_BM - 1) / DS_BM), (unsigned)nbh);
    hipLaunchKernelGGL((k_attn_ds<DT, HD>), grid, dim3(256), 0, s, (const uint16_t *)dout, (const uint16_t *)v,
                       (const uint16_t *)p16, rowsub, (uint16_t *)ds16, T, scale, causal);
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_tk_attn_ds_supported(int64_t hd, int64_t T) { return (hd == 32 || hd == 64 || hd == 128) && T > 0 && T % 8 == 0; }

int mg_tk_attn_p_supported(int64_t hd, int64_t T) { return mg_tk_attn_ds_supported(hd, T) && (hd <= 64 || T <= 1024); }

int mg_tk_attn_p(mg_ctx *ctx, const void *q16, const void *k16, const uint32_t *seg, void *p16, int64_t nbh, int64_t T,
                 int64_t H, int64_t hd, float scale, int causal, int dtype) {
    EW_PRECHECK("mg_tk_attn_p", q16 && k16 && p16 && nbh > 0 && nbh <= 65535 && mg_tk_attn_p_supported(hd, T) &&
                                    T <= 0x7fffffff / 2 &&
                                    H > 0 && nbh % H == 0 && dtype_ok(dtype) && scale == scale &&
                                    (((uintptr_t)q16 | (uintptr_t)k16 | (uintptr_t)p16) & 15) == 0 &&
                                    ((uintptr_t)seg & 3) == 0);
    hipStream_t s = ctx_stream(ctx);
    const int t = (int)T, c = causal ? 1 : 0, h = (int)H;
    if (dtype == MG_F16) {
        if (hd == 32) launch_attn_p<MG_F16, 32>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
        else if (hd == 64) launch_attn_p<MG_F16, 64>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
        else launch_attn_p<MG_F16, 128>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
    } else {
        if (hd == 32) launch_attn_p<MG_BF16, 32>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
        else if (hd == 64) launch_attn_p<MG_BF16, 64>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
        else launch_attn_p<MG_BF16, 128>(s, q16, k16, seg, p16, nbh, t, h, scale, c);
    }
    EW_POSTCHECK("mg_tk_attn_p");
}

int mg_tk_attn_fwd_supported(int64_t hd, int64_t T) {
    return (hd == 32 || hd == 64 || hd == 128) && T > 0 && T % 8 == 0 && T <= 1024;
}

int mg_tk_attn_fwd(mg_ctx *ctx, const void *q16, const void *k16, const void *v16, const uint32_t *seg, void *p16,
                   float *out32, void *out16, int64_t nbh, int64_t T, int64_t H, int64_t hd, float scale, int causal,
                   int dtype) {
    EW_PRECHECK("mg_tk_attn_fwd", q16 && k16 && v16 && p16 && out32 && nbh > 0 && nbh <= 65535 &&
                                      mg_tk_attn_fwd_supported(hd, T) && H > 0 && nbh % H == 0 && dtype_ok(dtype) &&
                                      scale == scale &&
                                      (((uintptr_t)q16 | (uintptr_t)k16 | (uintptr_t)v16 | (uintptr_t)p16) & 15) == 0 &&
                                      ((uintptr_t)out32 & 3) == 0 && ((uintptr_t)out16 & 1) == 0 && ((uintptr_t)seg & 3) == 0);
    hipStream_t s = ctx_stream(ctx);
    const int t = (int)T, c = causal ? 1 : 0, h = (int)H;
    if (dtype == MG_F16) {
        if (hd == 32) launch_attn_fwd<MG_F16, 32>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
        else if (hd == 64) launch_attn_fwd<MG_F16, 64>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
        else launch_attn_fwd<MG_F16, 128>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
    } else {
        if (hd == 32) launch_attn_fwd<MG_BF16, 32>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
        else if (hd == 64) launch_attn_fwd<MG_BF16, 64>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
        else launch_attn_fwd<MG_BF16, 128>(s, q16, k16, v16, seg, p16, out32, out16, nbh, t, h, scale, c);
    }
    EW_POSTCHECK("mg_tk_attn_fwd");
}

int mg_tk_attn_ds(mg_ctx *ctx, const void *dout16, const void *v16, const void *p16, const float *rowsub, void *ds16,
                  int64_t nbh, int64_t T, int64_t hd, float scale, int causal, int dtype) {
    EW_PRECHECK("mg_tk_attn_ds", dout16 && v16 && p16 && rowsub && ds16 && nbh > 0 && nbh <= 65535 && T > 0 &&
                                     T <= 0x7fffffff / 2 && mg_tk_attn_ds_supported(hd, T) && dtype_ok(dtype) &&
                                     (T + DS_BM - 1) / DS_BM <= 65535 && scale == scale &&
                                     (((uintptr_t)dout16 | (uintptr_t)v16) & 15) == 0 &&
                                     (((uintptr_t)p16 | (uintptr_t)ds16) & 15) == 0 && ((uintptr_t)rowsub & 3) == 0);
    hipStream_t s = ctx_stream(ctx);
    const int t = (int)T, c = causal ? 1 : 0;
    if (dtype == MG_F16) {
        if (hd == 32) launch_attn_ds<MG_F16, 32>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
        else if (hd == 64) launch_attn_ds<MG_F16, 64>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
        else launch_attn_ds<MG_F16, 128>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
    } else {
        if (hd == 32) launch_attn_ds<MG_BF16, 32>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
        else if (hd == 64) launch_attn_ds<MG_BF16, 64>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
        else launch_attn_ds<MG_BF16, 128>(s, dout16, v16, p16, rowsub, ds16, nbh, t, scale, c);
    }
    EW_POSTCHECK("mg_tk_attn_ds");
}

}  // extern "C"
