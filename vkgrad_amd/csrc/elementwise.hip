// Companion elementwise kernels of the training step (reference: kernels.py:699-862,
// dataparallel.py:54-58).  One thread per element (or per row / column where the
// reference does that); they exist so a whole MLP train step can run on the
// device around the GEMMs, and are not tuned beyond coalesced access.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"

#include "ew_common.h"

namespace mg {

__device__ __forceinline__ float gelu_f(float x) {
    const float c = 0.7978845608028654f;   // sqrt(2/pi), kernels.py:625-629
    const float x3 = x * x * x;
    return 0.5f * x * (1.0f + tanhf(c * (x + 0.044715f * x3)));
}
__device__ __forceinline__ float dgelu_f(float x) {
    const float c = 0.7978845608028654f;   // kernels.py:630-635
    const float x3 = x * x * x;
    const float t = tanhf(c * (x + 0.044715f * x3));
    const float sech2 = 1.0f - t * t;
    return 0.5f * (1.0f + t) + 0.5f * x * sech2 * c * (1.0f + 3.0f * 0.044715f * x * x);
}
__device__ __forceinline__ float act_f(float x, int act) {
    return act == MG_ACT_GELU ? gelu_f(x) : (act == MG_ACT_RELU ? fmaxf(x, 0.f) : x);
}
__device__ __forceinline__ float dact_f(float x, int act) {
    return act == MG_ACT_GELU ? dgelu_f(x) : (act == MG_ACT_RELU ? (x > 0.f ? 1.f : 0.f) : 1.f);
}

__global__ void k_bias_act(const float *acc, const float *bias, float *z, uint16_t *y16, int64_t n,
                           int64_t ncol, int act, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = bias ? acc[i] + bias[i % ncol] : acc[i];
    if (z) z[i] = v;
    if (y16) y16[i] = narrow16(act_f(v, act), dtype);
}

__global__ void k_act_bwd(const float *dy, const float *z, uint16_t *dz16, float *dz32, int64_t n, int act,
                          int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float g = dy[i] * dact_f(z[i], act);
    if (dz16) dz16[i] = narrow16(g, dtype);
    if (dz32) dz32[i] = g;
}

// Column sums (the reference loops the rows in one thread per column, kernels.py:753-761:
// fine at batch 128 on 12 CUs, one long chain of dependent loads here).  A block takes 64
// columns and COL_SUM_ROWS rows: 8 threads per column stride through the rows (coalesced 256-byte
// row pieces), LDS adds the 8 partial sums.  One chunk of rows: the block writes (or adds to) the
// sum itself, in a fixed order.  More rows: the chunks add with atomics into sums, which the
// host has cleared unless accumulating.
constexpr int COL_SUM_ROWS = 512;
__global__ void __launch_bounds__(512) k_col_sum(const float *g, float *sums, int64_t ncol, int64_t nrow,
                                                  int accumulate, int atomic) {
    __shared__ float part[8][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + tx;
    const int64_t r0 = (int64_t)blockIdx.y * COL_SUM_ROWS;
    const int64_t r1 = r0 + COL_SUM_ROWS < nrow ? r0 + COL_SUM_ROWS : nrow;
    float s = 0.f;
    if (c < ncol) {
#pragma unroll 8
        for (int64_t r = r0 + ty; r < r1; r += 8) s += g[r * ncol + c];
    }
    part[ty][tx] = s;
    __syncthreads();
    if (ty == 0 && c < ncol) {
        float t = part[0][tx];
#pragma unroll
        for (int i = 1; i < 8; i++) t += part[i][tx];
        if (atomic) atomicAdd(sums + c, t);
        else sums[c] = accumulate ? sums[c] + t : t;
    }
}

// Device-side copy of nbytes (a multiple of 4; 16-byte pieces when both ends are aligned).
__global__ void k_copy(const uint32_t *src, uint32_t *dst, int64_t nwords, int vec) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (vec) {
        if (i * 4 + 3 < nwords) reinterpret_cast<uint4 *>(dst)[i] = reinterpret_cast<const uint4 *>(src)[i];
        else for (int64_t j = i * 4; j < nwords; j++) dst[j] = src[j];
    } else if (i < nwords) {
        dst[i] = src[i];
    }
}

__global__ void k_softmax_ce(const float *logits, const uint32_t *labels, uint16_t *dl16, float *dl32, float *loss,
                             int64_t nrows, int64_t stride, int64_t ncls, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= nrows) return;
    const float *row = logits + i * stride;
    float mx = -1e30f;
    for (int64_t c = 0; c < ncls; ++c) mx = fmaxf(mx, row[c]);
    float s = 0.f;
    for (int64_t c = 0; c < ncls; ++c) s += expf(row[c] - mx);
    const float logZ = mx + logf(s);
    const uint32_t y = labels[i];
    loss[i] = logZ - row[y];
    const float inv = 1.0f / (float)nrows;
    for (int64_t c = 0; c < stride; ++c) {
        float gv = 0.f;
        if (c < ncls) gv = (expf(row[c] - logZ) - (c == (int64_t)y ? 1.f : 0.f)) * inv;
        if (dl16) dl16[i * stride + c] = narrow16(gv, dtype);
        if (dl32) dl32[i * stride + c] = gv;
    }
}

__global__ void k_adamw(float *w, const float *g, float *m, float *v, uint16_t *w16, const float *hp, int64_t n,
                        float wd, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float lr = hp[0], b1 = hp[1], b2 = hp[2], bc1 = hp[3], bc2 = hp[4], eps = hp[5];
    const float gi = g[i];
    const float mi = b1 * m[i] + (1.0f - b1) * gi;
    const float vi = b2 * v[i] + (1.0f - b2) * gi * gi;
    m[i] = mi;
    v[i] = vi;
    const float mh = mi / bc1;
    const float vh = vi / bc2;
    float wi = w[i];
    wi -= lr * (mh / (sqrtf(vh) + eps) + wd * wi);
    w[i] = wi;
    if (w16) w16[i] = narrow16(wi, dtype);
}

// AdamW over a list of parameters in one launch.  The table holds one entry per parameter and the
// number of its first workgroup; a workgroup finds its parameter by bisection and updates 1024
// consecutive elements of it, four per thread (same arithmetic as k_adamw, element by element).
__device__ __forceinline__ float adamw_one(float &w, float g, float &m, float &v, float lr, float b1, float b2,
                                           float bc1, float bc2, float eps, float wd) {
    m = b1 * m + (1.0f - b1) * g;
    v = b2 * v + (1.0f - b2) * g * g;
    w -= lr * ((m / bc1) / (sqrtf(v / bc2) + eps) + wd * w);
    return w;
}
__global__ void __launch_bounds__(256) k_adamw_multi(const mg_adamw_entry *table, int ntensors, const float *hp, int dtype) {
    int lo = 0, hi = ntensors - 1;
    while (lo < hi) {                      // last entry whose first_block <= blockIdx.x
        const int mid = (lo + hi + 1) >> 1;
        if (table[mid].first_block <= (int64_t)blockIdx.x) lo = mid;
        else hi = mid - 1;
    }
    const mg_adamw_entry e = table[lo];
    const float lr = hp[0], b1 = hp[1], b2 = hp[2], bc1 = hp[3], bc2 = hp[4], eps = hp[5];
    const int64_t i0 = (((int64_t)blockIdx.x - e.first_block) * 256 + threadIdx.x) * 4;
    if (i0 >= e.n) return;
    float *w = e.w + i0, *m = e.m + i0, *v = e.v + i0;
    const float *g = e.g + i0;
    uint16_t *w16 = e.w16 ? (uint16_t *)e.w16 + i0 : nullptr;
    if (i0 + 3 < e.n && e.vec) {
        float4 wv = *reinterpret_cast<float4 *>(w), mv = *reinterpret_cast<float4 *>(m), vv = *reinterpret_cast<float4 *>(v);
        const float4 gv = *reinterpret_cast<const float4 *>(g);
        adamw_one(wv.x, gv.x, mv.x, vv.x, lr, b1, b2, bc1, bc2, eps, e.wd);
        adamw_one(wv.y, gv.y, mv.y, vv.y, lr, b1, b2, bc1, bc2, eps, e.wd);
        adamw_one(wv.z, gv.z, mv.z, vv.z, lr, b1, b2, bc1, bc2, eps, e.wd);
        adamw_one(wv.w, gv.w, mv.w, vv.w, lr, b1, b2, bc1, bc2, eps, e.wd);
        *reinterpret_cast<float4 *>(w) = wv;
        *reinterpret_cast<float4 *>(m) = mv;
        *reinterpret_cast<float4 *>(v) = vv;
        if (w16)
            *reinterpret_cast<uint2 *>(w16) =
                make_uint2((uint32_t)narrow16(wv.x, dtype) | ((uint32_t)narrow16(wv.y, dtype) << 16),
                           (uint32_t)narrow16(wv.z, dtype) | ((uint32_t)narrow16(wv.w, dtype) << 16));
    } else {
        for (int k = 0; k < 4 && i0 + k < e.n; k++) {
            const float wi = adamw_one(w[k], g[k], m[k], v[k], lr, b1, b2, bc1, bc2, eps, e.wd);
            if (w16) w16[k] = narrow16(wi, dtype);
        }
    }
}

// Clears the gradient of every entry of an AdamW-style table in one launch (same block numbering).
__global__ void __launch_bounds__(256) k_zero_multi(const mg_adamw_entry *table, int ntensors) {
    int lo = 0, hi = ntensors - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (table[mid].first_block <= (int64_t)blockIdx.x) lo = mid;
        else hi = mid - 1;
    }
    const mg_adamw_entry e = table[lo];
    float *g = const_cast<float *>(e.g);
    const int64_t i0 = (((int64_t)blockIdx.x - e.first_block) * 256 + threadIdx.x) * 4;
    for (int k = 0; k < 4 && i0 + k < e.n; k++) g[i0 + k] = 0.f;
}

__global__ void k_zero(float *dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = 0.f;
}

__global__ void k_cast16(const float *src, uint16_t *dst, int64_t n, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = narrow16(src[i], dtype);
}

// four elements per thread: one 16-byte load, one 8-byte store; the tail goes element by element
__global__ void k_cast16_v4(const float *src, uint16_t *dst, int64_t n, int dtype) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 * 4 + 3 < n) {
        const float4 t = reinterpret_cast<const float4 *>(src)[i4];
        reinterpret_cast<uint2 *>(dst)[i4] =
            make_uint2((uint32_t)narrow16(t.x, dtype) | ((uint32_t)narrow16(t.y, dtype) << 16),
                       (uint32_t)narrow16(t.z, dtype) | ((uint32_t)narrow16(t.w, dtype) << 16));
    } else {
        for (int64_t i = i4 * 4; i < n; i++) dst[i] = narrow16(src[i], dtype);
    }
}

__global__ void k_scale_copy(float *dst, const float *src, int64_t n, float scale) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = src[i] * scale;
}

__global__ void k_grad_add(float *dst, const float *src, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] += src[i];
}

// Pseudo-random 16-bit operands in [-1, 1) from a counter hash: timing a GEMM on
// zeros or on uninitialised memory misstates it (data toggling sets MFMA power,
// and with it the clock), so the tuner and warm-up fill their scratch with this.
__global__ void k_fill_uniform16(uint16_t *dst, int64_t n, uint32_t seed, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    uint32_t x = (uint32_t)i * 0x9E3779B1u + seed;
    x ^= x >> 16;
    x *= 0x85EBCA6Bu;
    x ^= x >> 13;
    x *= 0xC2B2AE35u;
    x ^= x >> 16;
    const float v = (float)(x >> 8) * (2.0f / 16777216.0f) - 1.0f;
    dst[i] = narrow16(v, dtype);
}

}  // namespace mg

using namespace mg;

static inline bool act_ok(int a) { return a >= MG_ACT_NONE && a <= MG_ACT_RELU; }

extern "C" {

int mg_ew_bias_act(mg_ctx *ctx, const float *acc, const float *bias, float *z, void *y16, int64_t n, int64_t ncol,
                   int act, int dtype) {
    EW_PRECHECK("mg_ew_bias_act", acc && (z || y16) && count_ok(n) && ncol > 0 && act_ok(act) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_bias_act, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), acc, bias, z, (uint16_t *)y16, n,
                       ncol, act, dtype);
    EW_POSTCHECK("mg_ew_bias_act");
}

int mg_ew_act_bwd(mg_ctx *ctx, const float *dy, const float *z, void *dz16, float *dz32, int64_t n, int act,
                  int dtype) {
    EW_PRECHECK("mg_ew_act_bwd", dy && z && (dz16 || dz32) && count_ok(n) && act_ok(act) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_act_bwd, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dy, z, (uint16_t *)dz16, dz32, n,
                       act, dtype);
    EW_POSTCHECK("mg_ew_act_bwd");
}

int mg_ew_col_sum(mg_ctx *ctx, const float *g, float *sums, int64_t ncol, int64_t nrow, int accumulate) {
    EW_PRECHECK("mg_ew_col_sum", g && sums && count_ok(ncol) && nrow > 0 && nrow <= (int64_t)65535 * COL_SUM_ROWS);
    const unsigned chunks = (unsigned)((nrow + COL_SUM_ROWS - 1) / COL_SUM_ROWS);
    if (chunks > 1 && !accumulate) hipLaunchKernelGGL(k_zero, dim3(blocks_for(ncol)), dim3(256), 0, ctx_stream(ctx), sums, ncol);
    hipLaunchKernelGGL(k_col_sum, dim3((unsigned)((ncol + 63) / 64), chunks), dim3(512), 0, ctx_stream(ctx), g, sums, ncol,
                       nrow, accumulate, chunks > 1 ? 1 : 0);
    EW_POSTCHECK("mg_ew_col_sum");
}

int mg_ew_copy(mg_ctx *ctx, void *dst, const void *src, int64_t nbytes) {
    EW_PRECHECK("mg_ew_copy", dst && src && count_ok(nbytes) && nbytes % 4 == 0 &&
                                  (((uintptr_t)dst | (uintptr_t)src) & 3) == 0);
    const int64_t nwords = nbytes / 4;
    const int vec = ((((uintptr_t)dst | (uintptr_t)src) & 15) == 0) ? 1 : 0;
    const int64_t threads = vec ? (nwords + 3) / 4 : nwords;
    hipLaunchKernelGGL(k_copy, dim3(blocks_for(threads)), dim3(256), 0, ctx_stream(ctx), (const uint32_t *)src,
                       (uint32_t *)dst, nwords, vec);
    EW_POSTCHECK("mg_ew_copy");
}

int mg_ew_softmax_ce(mg_ctx *ctx, const float *logits, const uint32_t *labels, void *dl16, float *dl32, float *loss,
                     int64_t nrows, int64_t stride, int64_t ncls, int dtype) {
    EW_PRECHECK("mg_ew_softmax_ce", logits && labels && loss && count_ok(nrows) && ncls > 0 && stride >= ncls && dtype_ok(dtype));
    hipLaunchKernelGGL(k_softmax_ce, dim3(blocks_for(nrows)), dim3(256), 0, ctx_stream(ctx), logits, labels,
                       (uint16_t *)dl16, dl32, loss, nrows, stride, ncls, dtype);
    EW_POSTCHECK("mg_ew_softmax_ce");
}

int mg_ew_adamw(mg_ctx *ctx, float *w, const float *g, float *m, float *v, void *w16, const float *hp, int64_t n,
                float wd, int dtype) {
    EW_PRECHECK("mg_ew_adamw", w && g && m && v && hp && count_ok(n) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_adamw, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), w, g, m, v, (uint16_t *)w16, hp, n,
                       wd, dtype);
    EW_POSTCHECK("mg_ew_adamw");
}

int mg_ew_adamw_multi(mg_ctx *ctx, const mg_adamw_entry *table_dev, int ntensors, int64_t total_blocks, const float *hp,
                      int dtype) {
    EW_PRECHECK("mg_ew_adamw_multi", table_dev && ntensors > 0 && total_blocks > 0 && total_blocks <= 0x7fffffff && hp &&
                                         dtype_ok(dtype));
    hipLaunchKernelGGL(k_adamw_multi, dim3((unsigned)total_blocks), dim3(256), 0, ctx_stream(ctx), table_dev, ntensors, hp,
                       dtype);
    EW_POSTCHECK("mg_ew_adamw_multi");
}

int mg_ew_zero_multi(mg_ctx *ctx, const mg_adamw_entry *table_dev, int ntensors, int64_t total_blocks) {
    EW_PRECHECK("mg_ew_zero_multi", table_dev && ntensors > 0 && total_blocks > 0 && total_blocks <= 0x7fffffff);
    hipLaunchKernelGGL(k_zero_multi, dim3((unsigned)total_blocks), dim3(256), 0, ctx_stream(ctx), table_dev, ntensors);
    EW_POSTCHECK("mg_ew_zero_multi");
}

int mg_ew_zero(mg_ctx *ctx, float *dst, int64_t n) {
    EW_PRECHECK("mg_ew_zero", dst && count_ok(n));
    hipLaunchKernelGGL(k_zero, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dst, n);
    EW_POSTCHECK("mg_ew_zero");
}

int mg_ew_cast16(mg_ctx *ctx, const float *src, void *dst, int64_t n, int dtype) {
    EW_PRECHECK("mg_ew_cast16", src && dst && count_ok(n) && dtype_ok(dtype));
    if ((((uintptr_t)src & 15) | ((uintptr_t)dst & 7)) == 0)
        hipLaunchKernelGGL(k_cast16_v4, dim3(blocks_for((n + 3) / 4)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)dst, n,
                           dtype);
    else
        hipLaunchKernelGGL(k_cast16, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)dst, n, dtype);
    EW_POSTCHECK("mg_ew_cast16");
}

int mg_ew_fill_uniform16(mg_ctx *ctx, void *dst, int64_t n, uint32_t seed, int dtype) {
    EW_PRECHECK("mg_ew_fill_uniform16", dst && count_ok(n) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_fill_uniform16, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), (uint16_t *)dst, n, seed,
                       dtype);
    EW_POSTCHECK("mg_ew_fill_uniform16");
}

int mg_ew_scale_copy(mg_ctx *ctx, float *dst, const float *src, int64_t n, float scale) {
    EW_PRECHECK("mg_ew_scale_copy", dst && src && count_ok(n));
    hipLaunchKernelGGL(k_scale_copy, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dst, src, n, scale);
    EW_POSTCHECK("mg_ew_scale_copy");
}

int mg_ew_grad_add(mg_ctx *ctx, float *dst, const float *src, int64_t n) {
    EW_PRECHECK("mg_ew_grad_add", dst && src && count_ok(n));
    hipLaunchKernelGGL(k_grad_add, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dst, src, n);
    EW_POSTCHECK("mg_ew_grad_add");
}

}  // extern "C"
