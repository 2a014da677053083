// Shared by the companion kernel files: context access, 16-bit narrowing and widening,
// argument checks of the C entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"

struct mg_ctx;
namespace mg {
hipStream_t ctx_stream(mg_ctx *ctx);
int ctx_fail(int code, const char *msg);
int ctx_hip_fail(hipError_t e, const char *what);

__device__ __forceinline__ uint16_t narrow16(float x, int dtype) {
    if (dtype == MG_F16) {
        _Float16 h = (_Float16)x;   // round to nearest even
        return __builtin_bit_cast(uint16_t, h);
    }
    uint32_t u = __builtin_bit_cast(uint32_t, x);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;   // NaN
    u += 0x7fffu + ((u >> 16) & 1u);                        // round to nearest even
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float widen16(uint16_t h, int dtype) {
    if (dtype == MG_F16) return (float)__builtin_bit_cast(_Float16, h);
    return __builtin_bit_cast(float, (uint32_t)h << 16);
}

static inline unsigned blocks_for(int64_t n) { return (unsigned)((n + 255) / 256); }
static inline bool dtype_ok(int d) { return d == MG_F16 || d == MG_BF16; }
static inline bool count_ok(int64_t n) { return n > 0 && n <= (int64_t)0x7fffffff * 256; }

}  // namespace mg

#define EW_PRECHECK(name, cond)                                            \
    if (!ctx) return mg::ctx_fail(MG_ERR_ARG, name ": ctx is NULL");       \
    if (!(cond)) return mg::ctx_fail(MG_ERR_ARG, name ": bad argument");
#define EW_POSTCHECK(name)                                                 \
    do {                                                                   \
        hipError_t e_ = hipGetLastError();                                 \
        if (e_ != hipSuccess) return mg::ctx_hip_fail(e_, name);           \
        return MG_OK;                                                      \
    } while (0)
