/* Independent scalar restatement of the GEMM oracle.  TEST INFRASTRUCTURE ONLY.
 *
 * Same contract as /root/reference/kernels.py:606-610 and the operand storage of
 * kernels.py:42-43: A is (M,K) or (K,M) when trans_a, B is (K,N) or (N,K) when
 * trans_b, C is (M,N) float32.  Inputs are IEEE half or bfloat16 bit patterns,
 * widened exactly; products are summed in double (so the result is the
 * correctly rounded float of an almost exact sum) or in float, k ascending.
 * It shares no code with numpy/OpenBLAS, which is what makes it a check on
 * oracle/ref_gemm.py rather than a copy of it.
 */
#include <stdint.h>
#include <string.h>

static float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static float bf16_to_float(uint16_t h) {
    uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* dtype: 0 = f16, 1 = bf16.  acc64: sum in double when non-zero.
 * bias may be NULL; beta is 0 or 1 (C is read only when beta == 1). */
int ref_gemm_scalar(int dtype, int trans_a, int trans_b, int acc64,
                    int64_t M, int64_t N, int64_t K,
                    const uint16_t *A, int64_t lda, const uint16_t *B, int64_t ldb,
                    float *C, int64_t ldc, const float *bias, int beta) {
    if (trans_a && trans_b) return 1;
    for (int64_t m = 0; m < M; m++) {
        for (int64_t n = 0; n < N; n++) {
            double s64 = 0.0;
            float s32 = 0.0f;
            for (int64_t k = 0; k < K; k++) {
                uint16_t ab = trans_a ? A[k * lda + m] : A[m * lda + k];
                uint16_t bb = trans_b ? B[n * ldb + k] : B[k * ldb + n];
                float a = dtype ? bf16_to_float(ab) : half_to_float(ab);
                float b = dtype ? bf16_to_float(bb) : half_to_float(bb);
                if (acc64) s64 += (double)a * (double)b;
                else s32 += a * b;
            }
            float acc = acc64 ? (float)s64 : s32;
            if (bias) acc = acc + bias[n];
            if (beta) acc = C[m * ldc + n] + acc;
            C[m * ldc + n] = acc;
        }
    }
    return 0;
}

float ref_half_to_float(uint16_t h) { return half_to_float(h); }
float ref_bf16_to_float(uint16_t h) { return bf16_to_float(h); }
