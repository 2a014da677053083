// Row kernels of the decoder block around the GEMMs (reference: tkernels.py:32-389):
// LayerNorm forward/backward, the causal attention softmax forward/backward, the head
// permutes, embeddings, residual adds, and the wide-row softmax cross-entropy of the
// LM head.  All of them are one pass (or one pass plus L2-resident re-reads of the same
// row) over HBM data.
//
// Row kernels give one 64-lane wavefront a row (the reference strides a row over one
// 32-lane subgroup, tkernels.py:24-31, 96-104): lane l takes elements l, l + 64, ... so a
// wavefront reads 256 contiguous bytes per step, and the row reductions are lane
// exchanges.  Four rows share a 256-thread workgroup.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mi_gemm.h"

#include "ew_common.h"

namespace mg {

constexpr int ROWS_PER_WG = 4;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}

// ---- LayerNorm (tkernels.py:32-56): y16 = narrow((x - mu) * rstd * gamma + beta), eps 1e-5;
// mu and rstd are kept for the backward pass.
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_layernorm(const float *x, const float *gamma, const float *beta, uint16_t *y16, float *mu, float *rstd, int64_t rows,
            int D, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *xr = x + row * D;
    float s = 0.f;
    for (int d = lane; d < D; d += 64) s += xr[d];
    const float m = wave_sum(s) / (float)D;
    float v = 0.f;
    for (int d = lane; d < D; d += 64) {
        const float t = xr[d] - m;
        v += t * t;
    }
    const float r = rsqrtf(wave_sum(v) / (float)D + 1e-5f);
    if (lane == 0) {
        mu[row] = m;
        rstd[row] = r;
    }
    uint16_t *yr = y16 + row * D;
    for (int d = lane; d < D; d += 64) yr[d] = narrow16((xr[d] - m) * r * gamma[d] + beta[d], dtype);
}

__device__ __forceinline__ uint2 narrow16x4(float a, float b, float c, float d, int dtype) {
    return make_uint2((uint32_t)narrow16(a, dtype) | ((uint32_t)narrow16(b, dtype) << 16),
                      (uint32_t)narrow16(c, dtype) | ((uint32_t)narrow16(d, dtype) << 16));
}

// LayerNorm with the row in registers (D % 4 == 0, D <= 256 NV): lane l holds the float4 groups
// l, l + 64, ...; one 16-byte load per group, statistics from registers, 8-byte stores.
template <int NV>
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_layernorm_reg(const float *x, const float *gamma, const float *beta, uint16_t *y16, float *mu, float *rstd,
                int64_t rows, int D, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int ngroups = D >> 2;
    const float4 *xr = reinterpret_cast<const float4 *>(x + row * D);
    float4 v[NV];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int g = lane + 64 * i;
        v[i] = g < ngroups ? xr[g] : make_float4(0.f, 0.f, 0.f, 0.f);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    const float m = wave_sum(s) / (float)D;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        if (lane + 64 * i < ngroups) {
            const float a = v[i].x - m, b = v[i].y - m, c = v[i].z - m, d = v[i].w - m;
            q += (a * a + b * b) + (c * c + d * d);
        }
    }
    const float r = rsqrtf(wave_sum(q) / (float)D + 1e-5f);
    if (lane == 0) {
        mu[row] = m;
        rstd[row] = r;
    }
    uint2 *yr = reinterpret_cast<uint2 *>(y16 + row * D);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int g = lane + 64 * i;
        if (g < ngroups) {
            const float4 ga = reinterpret_cast<const float4 *>(gamma)[g], be = reinterpret_cast<const float4 *>(beta)[g];
            yr[g] = narrow16x4((v[i].x - m) * r * ga.x + be.x, (v[i].y - m) * r * ga.y + be.y,
                               (v[i].z - m) * r * ga.z + be.z, (v[i].w - m) * r * ga.w + be.w, dtype);
        }
    }
}

template <int NV>
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_layernorm_bwd_reg(const float *dy, const float *x, const float *gamma, const float *mu, const float *rstd, float *dx,
                    uint16_t *dyxh16, uint16_t *dy16, int64_t rows, int D, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int ngroups = D >> 2;
    const float m = mu[row], r = rstd[row];
    const float4 *xr = reinterpret_cast<const float4 *>(x + row * D);
    const float4 *gr = reinterpret_cast<const float4 *>(dy + row * D);
    uint2 *o1 = reinterpret_cast<uint2 *>(dyxh16 + row * D), *o2 = reinterpret_cast<uint2 *>(dy16 + row * D);
    float xh[NV][4], dxh[NV][4];
    float s1 = 0.f, s2 = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int g = lane + 64 * i;
        if (g < ngroups) {
            const float4 xv = xr[g], gv = gr[g], ga = reinterpret_cast<const float4 *>(gamma)[g];
            const float xs[4] = {xv.x, xv.y, xv.z, xv.w}, gs[4] = {gv.x, gv.y, gv.z, gv.w};
            const float gm[4] = {ga.x, ga.y, ga.z, ga.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                xh[i][e] = (xs[e] - m) * r;
                dxh[i][e] = gs[e] * gm[e];
                s1 += dxh[i][e];
                s2 += dxh[i][e] * xh[i][e];
            }
            o1[g] = narrow16x4(gs[0] * xh[i][0], gs[1] * xh[i][1], gs[2] * xh[i][2], gs[3] * xh[i][3], dtype);
            o2[g] = narrow16x4(gs[0], gs[1], gs[2], gs[3], dtype);
        } else {
#pragma unroll
            for (int e = 0; e < 4; e++) xh[i][e] = dxh[i][e] = 0.f;
        }
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    const float inv = 1.0f / (float)D;
    float4 *dxr = reinterpret_cast<float4 *>(dx + row * D);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int g = lane + 64 * i;
        if (g < ngroups)
            dxr[g] = make_float4(r * (dxh[i][0] - s1 * inv - xh[i][0] * s2 * inv), r * (dxh[i][1] - s1 * inv - xh[i][1] * s2 * inv),
                                 r * (dxh[i][2] - s1 * inv - xh[i][2] * s2 * inv), r * (dxh[i][3] - s1 * inv - xh[i][3] * s2 * inv));
    }
}

// LayerNorm backward (tkernels.py:58-92): dx = rstd * (dxh - mean(dxh) - xh * mean(dxh * xh)) with
// dxh = dy * gamma; also emits dy * xh and dy in 16 bits for the column sums of dgamma and dbeta.
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_layernorm_bwd(const float *dy, const float *x, const float *gamma, const float *mu, const float *rstd, float *dx,
                uint16_t *dyxh16, uint16_t *dy16, int64_t rows, int D, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t base = row * D;
    const float m = mu[row], r = rstd[row];
    float s1 = 0.f, s2 = 0.f;
    for (int d = lane; d < D; d += 64) {
        const float g = dy[base + d];
        const float xh = (x[base + d] - m) * r;
        const float dxh = g * gamma[d];
        s1 += dxh;
        s2 += dxh * xh;
        dyxh16[base + d] = narrow16(g * xh, dtype);
        dy16[base + d] = narrow16(g, dtype);
    }
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    const float inv = 1.0f / (float)D;
    for (int d = lane; d < D; d += 64) {
        const float xh = (x[base + d] - m) * r;
        const float dxh = dy[base + d] * gamma[d];
        dx[base + d] = r * (dxh - s1 * inv - xh * s2 * inv);
    }
}

// ---- Causal attention softmax (tkernels.py:105-165).  Row = (batch * head, query q): keys
// first..q take part, the rest get probability 0; first = 0, or seg[b * T + q] (the start of
// the query's sample within its packed row).
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_attn_softmax(const float *s, const uint32_t *seg, uint16_t *p16, int64_t rows, int T, int H, float scale, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int q = (int)(row % T);
    const int first = seg ? (int)seg[(row / T / H) * T + q] : 0;
    const float *sr = s + row * T;
    float mx = -1e30f;
    for (int j = first + lane; j <= q; j += 64) mx = fmaxf(mx, sr[j] * scale);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = first + lane; j <= q; j += 64) sum += __expf(sr[j] * scale - mx);
    const float inv = 1.0f / wave_sum(sum);
    uint16_t *pr = p16 + row * T;
    for (int j = lane; j < T; j += 64) {
        float v = 0.f;
        if (j >= first && j <= q) v = __expf(sr[j] * scale - mx) * inv;
        pr[j] = narrow16(v, dtype);
    }
}

// The same two kernels for T % 4 == 0 and T <= 256 * NV: a lane holds NV groups of four
// consecutive scores (group i covers keys 256 i + 4 lane ...), loaded once with 16-byte loads
// - groups wholly beyond the query are never fetched - and the probabilities leave as 8-byte
// stores.  One pass over HBM instead of three L2-assisted ones.
template <int NV>
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_attn_softmax_reg(const float *s, const uint32_t *seg, uint16_t *p16, int64_t rows, int T, int H, float scale, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int q = (int)(row % T);
    const int first = seg ? (int)seg[(row / T / H) * T + q] : 0;
    const float4 *sr = reinterpret_cast<const float4 *>(s + row * T);
    float v[NV][4];
    float mx = -1e30f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int j0 = i * 256 + lane * 4;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        if (j0 <= q && j0 + 3 >= first && j0 < T) t = sr[j0 >> 2];
        v[i][0] = t.x * scale; v[i][1] = t.y * scale; v[i][2] = t.z * scale; v[i][3] = t.w * scale;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int j = j0 + e;
            if (j >= first && j <= q) mx = fmaxf(mx, v[i][e]);
        }
    }
    mx = wave_max(mx);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int j = i * 256 + lane * 4 + e;
            const float ex = (j >= first && j <= q) ? __expf(v[i][e] - mx) : 0.f;
            v[i][e] = ex;
            sum += ex;
        }
    const float inv = 1.0f / wave_sum(sum);
    uint2 *pr = reinterpret_cast<uint2 *>(p16 + row * T);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int j0 = i * 256 + lane * 4;
        if (j0 < T) {
            const uint32_t a = narrow16(v[i][0] * inv, dtype), b = narrow16(v[i][1] * inv, dtype);
            const uint32_t c = narrow16(v[i][2] * inv, dtype), d = narrow16(v[i][3] * inv, dtype);
            pr[j0 >> 2] = make_uint2(a | (b << 16), c | (d << 16));
        }
    }
}

template <int NV>
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_attn_softmax_bwd_reg(const float *dp, const uint16_t *p16, uint16_t *ds16, int64_t rows, int T, float scale, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int q = (int)(row % T);
    const float4 *dr = reinterpret_cast<const float4 *>(dp + row * T);
    const uint2 *pr = reinterpret_cast<const uint2 *>(p16 + row * T);
    float g[NV][4], pv[NV][4];
    float dot = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int j0 = i * 256 + lane * 4;
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        uint2 u = make_uint2(0u, 0u);
        if (j0 <= q && j0 < T) {
            t = dr[j0 >> 2];
            u = pr[j0 >> 2];
        }
        g[i][0] = t.x; g[i][1] = t.y; g[i][2] = t.z; g[i][3] = t.w;
        pv[i][0] = widen16((uint16_t)(u.x & 0xffffu), dtype); pv[i][1] = widen16((uint16_t)(u.x >> 16), dtype);
        pv[i][2] = widen16((uint16_t)(u.y & 0xffffu), dtype); pv[i][3] = widen16((uint16_t)(u.y >> 16), dtype);
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (j0 + e > q) {                     // beyond the query P is zero and dP was never written
                pv[i][e] = 0.f;
                g[i][e] = 0.f;
            }
            dot += g[i][e] * pv[i][e];
        }
    }
    dot = wave_sum(dot);
    uint2 *dr16 = reinterpret_cast<uint2 *>(ds16 + row * T);
#pragma unroll
    for (int i = 0; i < NV; i++) {
        const int j0 = i * 256 + lane * 4;
        if (j0 < T) {
            uint32_t o[4];
#pragma unroll
            for (int e = 0; e < 4; e++) o[e] = narrow16(j0 + e <= q ? pv[i][e] * (g[i][e] - dot) * scale : 0.f, dtype);
            dr16[j0 >> 2] = make_uint2(o[0] | (o[1] << 16), o[2] | (o[3] << 16));
        }
    }
}

// out[r] = sum_d a16[r][d] * b32[r][d], one wavefront per row.  With a = dOut and b = Out (both
// head-side, D = head width) this is sum_j P[r][j] dP[r][j] of the softmax backward
// (tkernels.py:167-187) without P or dP: dP = dOut V^T and Out = P V.
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_attn_rowdot(const uint16_t *a16, const float *b32, float *out, int64_t rows, int D, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int64_t base = row * D;
    float dot = 0.f;
    for (int d = lane; d < D; d += 64) dot += widen16(a16[base + d], dtype) * b32[base + d];
    dot = wave_sum(dot);
    if (lane == 0) out[row] = dot;
}

// The same with eight lanes per row and 16-byte loads (D a multiple of 8, aligned bases): a
// wavefront takes eight rows per load instruction instead of one - the cost of a kernel like
// this one is its number of memory instructions.
__global__ void __launch_bounds__(256)
k_attn_rowdot_v8(const uint16_t *a16, const float *b32, float *out, int64_t rows, int D, int dtype) {
    const int64_t row = ((int64_t)blockIdx.x * 256 + threadIdx.x) >> 3;
    const int seg = threadIdx.x & 7;
    float dot = 0.f;
    if (row < rows) {
        const int64_t base = row * D;
        for (int d = seg * 8; d < D; d += 64) {
            const uint4 a = *reinterpret_cast<const uint4 *>(a16 + base + d);
            const float4 b0 = *reinterpret_cast<const float4 *>(b32 + base + d);
            const float4 b1 = *reinterpret_cast<const float4 *>(b32 + base + d + 4);
            dot += widen16((uint16_t)(a.x & 0xffffu), dtype) * b0.x + widen16((uint16_t)(a.x >> 16), dtype) * b0.y +
                   widen16((uint16_t)(a.y & 0xffffu), dtype) * b0.z + widen16((uint16_t)(a.y >> 16), dtype) * b0.w +
                   widen16((uint16_t)(a.z & 0xffffu), dtype) * b1.x + widen16((uint16_t)(a.z >> 16), dtype) * b1.y +
                   widen16((uint16_t)(a.w & 0xffffu), dtype) * b1.z + widen16((uint16_t)(a.w >> 16), dtype) * b1.w;
        }
    }
#pragma unroll
    for (int m = 4; m >= 1; m >>= 1) dot += __shfl_xor(dot, m, 64);
    if (row < rows && seg == 0) out[row] = dot;
}

// dS = P * (dP - sum_j dP_j P_j) * scale over the unmasked keys (tkernels.py:167-187); masked keys
// hold P = 0, so only j <= q is read.
__global__ void __launch_bounds__(64 * ROWS_PER_WG)
k_attn_softmax_bwd(const float *dp, const uint16_t *p16, uint16_t *ds16, int64_t rows, int T, float scale, int dtype) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * ROWS_PER_WG + (threadIdx.x >> 6);
    if (row >= rows) return;
    const int q = (int)(row % T);
    const int64_t base = row * T;
    float dot = 0.f;
    for (int j = lane; j <= q; j += 64) dot += dp[base + j] * widen16(p16[base + j], dtype);
    dot = wave_sum(dot);
    for (int j = lane; j < T; j += 64) {
        float v = 0.f;
        if (j <= q) v = widen16(p16[base + j], dtype) * (dp[base + j] - dot) * scale;
        ds16[base + j] = narrow16(v, dtype);
    }
}

// ---- Head permutes (tkernels.py:195-301).  i indexes the (B*T, D) side; the head side is
// (B*H, T, hd).
struct HeadIdx {
    int64_t head;   // offset in a (B*H, T, hd) tensor
    int64_t bt;     // row of the (B*T, .) tensor
    int d;
};
__device__ __forceinline__ HeadIdx head_index(int64_t i, int D, int T, int H, int hd) {
    HeadIdx r;
    r.d = (int)(i % D);
    r.bt = i / D;
    const int t = (int)(r.bt % T);
    const int64_t b = r.bt / T;
    const int h = r.d / hd, j = r.d % hd;
    r.head = ((b * H + h) * T + t) * hd + j;
    return r;
}
__global__ void k_split_qkv(const float *qkv, const float *bias, uint16_t *q16, uint16_t *k16, uint16_t *v16, int64_t n,
                            int D, int T, int H, int hd, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const HeadIdx x = head_index(i, D, T, H, hd);
    const float *src = qkv + x.bt * 3 * D + x.d;
    const float b0 = bias ? bias[x.d] : 0.f, b1 = bias ? bias[x.d + D] : 0.f, b2 = bias ? bias[x.d + 2 * D] : 0.f;
    q16[x.head] = narrow16(src[0] + b0, dtype);
    k16[x.head] = narrow16(src[D] + b1, dtype);
    v16[x.head] = narrow16(src[2 * D] + b2, dtype);
}
__global__ void k_merge_qkv_grad(const float *dq, const float *dk, const float *dv, uint16_t *dqkv16, int64_t n, int D,
                                 int T, int H, int hd, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const HeadIdx x = head_index(i, D, T, H, hd);
    uint16_t *dst = dqkv16 + x.bt * 3 * D + x.d;
    dst[0] = narrow16(dq[x.head], dtype);
    dst[D] = narrow16(dk[x.head], dtype);
    dst[2 * D] = narrow16(dv[x.head], dtype);
}
__global__ void k_merge_heads(const float *src, uint16_t *y16, int64_t n, int D, int T, int H, int hd, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    y16[i] = narrow16(src[head_index(i, D, T, H, hd).head], dtype);
}
__global__ void k_split_heads(const float *src, uint16_t *dst16, int64_t n, int D, int T, int H, int hd, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    dst16[head_index(i, D, T, H, hd).head] = narrow16(src[i], dtype);
}

// The permutes four elements at a time (hd % 4 == 0: a group never straddles two heads).
__global__ void k_split_qkv_v4(const float *qkv, const float *bias, uint16_t *q16, uint16_t *k16, uint16_t *v16,
                               int64_t n4, int D, int T, int H, int hd, int dtype) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 >= n4) return;
    const HeadIdx x = head_index(i4 * 4, D, T, H, hd);
    const float *src = qkv + x.bt * 3 * D + x.d;
    uint16_t *dst[3] = {q16, k16, v16};
#pragma unroll
    for (int w = 0; w < 3; w++) {
        float4 t = *reinterpret_cast<const float4 *>(src + w * D);
        if (bias) {
            const float4 b = *reinterpret_cast<const float4 *>(bias + x.d + w * D);
            t.x += b.x; t.y += b.y; t.z += b.z; t.w += b.w;
        }
        *reinterpret_cast<uint2 *>(dst[w] + x.head) = narrow16x4(t.x, t.y, t.z, t.w, dtype);
    }
}
__global__ void k_merge_qkv_grad_v4(const float *dq, const float *dk, const float *dv, uint16_t *dqkv16, int64_t n4, int D,
                                    int T, int H, int hd, int dtype) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 >= n4) return;
    const HeadIdx x = head_index(i4 * 4, D, T, H, hd);
    uint16_t *dst = dqkv16 + x.bt * 3 * D + x.d;
    const float *src[3] = {dq, dk, dv};
#pragma unroll
    for (int w = 0; w < 3; w++) {
        const float4 t = *reinterpret_cast<const float4 *>(src[w] + x.head);
        *reinterpret_cast<uint2 *>(dst + w * D) = narrow16x4(t.x, t.y, t.z, t.w, dtype);
    }
}
__global__ void k_heads_v4(const float *src, uint16_t *dst16, int64_t n4, int D, int T, int H, int hd, int dtype,
                           int to_heads) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 >= n4) return;
    const int64_t head = head_index(i4 * 4, D, T, H, hd).head;
    const float4 t = *reinterpret_cast<const float4 *>(src + (to_heads ? i4 * 4 : head));
    *reinterpret_cast<uint2 *>(dst16 + (to_heads ? head : i4 * 4)) = narrow16x4(t.x, t.y, t.z, t.w, dtype);
}
// out = a + b (+ bias[i % D]) and 16-bit narrowing, four elements per thread
__global__ void k_add_v4(const float *a, const float *b, const float *bias, float *out, int64_t n4, int D) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 >= n4) return;
    float4 x = reinterpret_cast<const float4 *>(a)[i4];
    const float4 y = reinterpret_cast<const float4 *>(b)[i4];
    x.x += y.x; x.y += y.y; x.z += y.z; x.w += y.w;
    if (bias) {
        const float4 c = *reinterpret_cast<const float4 *>(bias + (i4 * 4) % D);
        x.x += c.x; x.y += c.y; x.z += c.z; x.w += c.w;
    }
    reinterpret_cast<float4 *>(out)[i4] = x;
}

// ---- Embeddings (tkernels.py:303-360): x = tok[ids] + pos[t]; t restarts at the sample's start
// when seg is given.  Backward is a scatter-add (several positions share a vocabulary row).
__global__ void k_embed(const float *tok, const float *pos, const uint32_t *ids, const uint32_t *seg, float *x, int64_t n,
                        int D, int T) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int d = (int)(i % D);
    const int64_t bt = i / D;
    const int t = (int)(bt % T) - (seg ? (int)seg[bt] : 0);
    x[i] = tok[(int64_t)ids[bt] * D + d] + pos[(int64_t)t * D + d];
}
__global__ void k_embed_bwd(const float *dx, const uint32_t *ids, const uint32_t *seg, float *dtok, float *dpos, int64_t n,
                            int D, int T) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int d = (int)(i % D);
    const int64_t bt = i / D;
    const int t = (int)(bt % T) - (seg ? (int)seg[bt] : 0);
    const float g = dx[i];
    atomicAdd(dtok + (int64_t)ids[bt] * D + d, g);
    atomicAdd(dpos + (int64_t)t * D + d, g);
}

// ---- Residual and friends (tkernels.py:362-389)
__global__ void k_residual(const float *acc, const float *bias, const float *res, float *out, int64_t n, int D) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = res[i] + acc[i] + bias[i % D];
}
// out = a + b and its 16-bit copy in one pass: the `add` of a residual's two gradient paths
// followed by the `to16` of the sum for the next GEMMs (transformer.py:242-252).
__global__ void k_add16_v4(const float *a, const float *b, float *out, uint16_t *out16, int64_t n4, int dtype) {
    const int64_t i4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i4 >= n4) return;
    float4 x = reinterpret_cast<const float4 *>(a)[i4];
    const float4 y = reinterpret_cast<const float4 *>(b)[i4];
    x.x += y.x; x.y += y.y; x.z += y.z; x.w += y.w;
    reinterpret_cast<float4 *>(out)[i4] = x;
    reinterpret_cast<uint2 *>(out16)[i4] = narrow16x4(x.x, x.y, x.z, x.w, dtype);
}
__global__ void k_add16(const float *a, const float *b, float *out, uint16_t *out16, int64_t n, int dtype) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float x = a[i] + b[i];
        out[i] = x;
        out16[i] = narrow16(x, dtype);
    }
}
__global__ void k_add(const float *a, const float *b, float *out, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = a[i] + b[i];
}
__global__ void k_add_bias(float *x, const float *bias, int64_t n, int64_t ncol) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] += bias[i % ncol];
}

// Column sums of a 16-bit matrix, f32 accumulation (tkernels.py:258-270): same blocking as the
// f32 column sum: 64 columns x 512 rows per block, 8 row lanes per column, chunks of rows meet
// through float atomics (the host clears sums first unless accumulating).  (Parking the chunks'
// partial sums in a scratch and letting the block that arrives last add them in order - no
// clear, no atomics, reproducible bits - was measured too: 7 us slower per call at 8192 rows,
// 0.7 ms on a GPT-2-small step, so the atomics stay.  So was a version with one 16-byte load per
// 8 columns and 256 rows per block: 6.7 us against 5.3 - 6.2 us for 8192 x 768, no gain.)
constexpr int CS16_ROWS = 512;
__global__ void __launch_bounds__(512)
k_col_sum16(const uint16_t *g, float *sums, int64_t ncol, int64_t nrow, int accumulate, int atomic, int dtype) {
    __shared__ float part[8][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int64_t c = (int64_t)blockIdx.x * 64 + tx;
    const int64_t r0 = (int64_t)blockIdx.y * CS16_ROWS;
    const int64_t r1 = r0 + CS16_ROWS < nrow ? r0 + CS16_ROWS : nrow;
    float s = 0.f;
    if (c < ncol) {
#pragma unroll 8
        for (int64_t r = r0 + ty; r < r1; r += 8) s += widen16(g[r * ncol + c], dtype);
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
__global__ void k_zero_f32(float *dst, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = 0.f;
}

// ---- Softmax cross-entropy over a wide row (the LM head: 50257 classes).  Same result as the
// one-thread-per-row kernel of the MLP (kernels.py:766-791) with the row spread over a
// workgroup: 1024 threads for a vocabulary (8192 x 50257: 0.80 ms with 256 threads per row,
// 0.66 with 512, 0.58 with 1024 - more loads in flight per row), 256 for narrower rows.  Pass 1 keeps a running maximum and a sum of exponentials relative to
// it per thread (one read of the row instead of two), the workgroup merges them; pass 2
// re-reads the row (L2 / last-level cache) and writes the gradient.  weight[row] (or
// 1 / nrows) scales the gradient (softmax_ce_w, kernels.py:793-823).  (Holding a 50304-wide row in
// the registers of one 1024-thread workgroup, so that HBM sees it once, was slower - 1.15 ms
// against 0.82 ms for 8192 rows: every wavefront of a CU is then in the same phase, and loads,
// exponentials and stores no longer overlap.)  Rows whose pitch and
// base are 16-byte aligned move as float4 / four 16-bit values.
struct MaxSum {
    float m, s;
};
__device__ __forceinline__ void ms_push(MaxSum &a, float x) {
    if (x > a.m) {
        a.s = a.s * __expf(a.m - x) + 1.0f;
        a.m = x;
    } else {
        a.s += __expf(x - a.m);
    }
}
__device__ __forceinline__ MaxSum ms_merge(MaxSum a, MaxSum b) {
    const float m = fmaxf(a.m, b.m);
    return MaxSum{m, a.s * __expf(a.m - m) + b.s * __expf(b.m - m)};
}
template <int NT>
__global__ void __launch_bounds__(NT)
k_softmax_ce_wide(const float *logits, const uint32_t *labels, const float *weights, uint16_t *dl16, float *dl32,
                  float *loss, int64_t nrows, int64_t stride, int64_t ncls, int dtype, int vec) {
    constexpr int NW = NT / 64;
    __shared__ float red_m[NW], red_s[NW];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lr = logits + row * stride;
    uint16_t *g16 = dl16 ? dl16 + row * stride : nullptr;
    float *g32 = dl32 ? dl32 + row * stride : nullptr;
    if (weights && weights[row] == 0.f) {   // masked row: no softmax, zeros (uniform over the workgroup)
        for (int64_t c = tid; c < stride; c += NT) {
            if (g16) g16[c] = 0;
            if (g32) g32[c] = 0.f;
        }
        if (tid == 0) loss[row] = 0.f;
        return;
    }
    MaxSum acc{-1e30f, 0.f};
    const int64_t n4 = vec ? ncls / 4 : 0;
    for (int64_t c = tid; c < n4; c += NT) {
        const float4 t = reinterpret_cast<const float4 *>(lr)[c];
        ms_push(acc, t.x); ms_push(acc, t.y); ms_push(acc, t.z); ms_push(acc, t.w);
    }
    for (int64_t c = n4 * 4 + tid; c < ncls; c += NT) ms_push(acc, lr[c]);
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) {
        MaxSum o{__shfl_xor(acc.m, m, 64), __shfl_xor(acc.s, m, 64)};
        acc = ms_merge(acc, o);
    }
    if (lane == 0) {
        red_m[wave] = acc.m;
        red_s[wave] = acc.s;
    }
    __syncthreads();
    MaxSum all{red_m[0], red_s[0]};
#pragma unroll
    for (int w = 1; w < NW; w++) all = ms_merge(all, MaxSum{red_m[w], red_s[w]});
    const float logZ = all.m + __logf(all.s);
    const int64_t y = labels[row];
    const float w = weights ? weights[row] : 1.0f / (float)nrows;
    if (tid == 0) loss[row] = logZ - lr[y];
    auto grad = [&](int64_t c, float x) { return c < ncls ? (__expf(x - logZ) - (c == y ? 1.f : 0.f)) * w : 0.f; };
    const int64_t s4 = vec ? stride / 4 : 0;
    for (int64_t c = tid; c < s4; c += NT) {
        const float4 t = reinterpret_cast<const float4 *>(lr)[c];
        const float a = grad(4 * c, t.x), b = grad(4 * c + 1, t.y), cc = grad(4 * c + 2, t.z), d = grad(4 * c + 3, t.w);
        if (g16)
            reinterpret_cast<uint2 *>(g16)[c] =
                make_uint2((uint32_t)narrow16(a, dtype) | ((uint32_t)narrow16(b, dtype) << 16),
                           (uint32_t)narrow16(cc, dtype) | ((uint32_t)narrow16(d, dtype) << 16));
        if (g32) reinterpret_cast<float4 *>(g32)[c] = make_float4(a, b, cc, d);
    }
    for (int64_t c = s4 * 4 + tid; c < stride; c += NT) {
        const float gv = grad(c, c < ncls ? lr[c] : 0.f);
        if (g16) g16[c] = narrow16(gv, dtype);
        if (g32) g32[c] = gv;
    }
}

static inline bool aligned16(const void *a, const void *b, const void *c) {
    return (((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) & 15) == 0;   // NULL counts as aligned
}
static inline bool aligned8(const void *a) { return ((uintptr_t)a & 7) == 0; }
static inline unsigned row_blocks(int64_t rows) { return (unsigned)((rows + ROWS_PER_WG - 1) / ROWS_PER_WG); }
static inline bool heads_ok(int64_t n, int D, int T, int H, int hd) {
    return count_ok(n) && D > 0 && T > 0 && H > 0 && hd > 0 && (int64_t)H * hd == D && n % ((int64_t)D * T) == 0;
}

}  // namespace mg

using namespace mg;

extern "C" {

int mg_tk_layernorm(mg_ctx *ctx, const float *x, const float *gamma, const float *beta, void *y16, float *mu,
                    float *rstd, int64_t rows, int64_t D, int dtype) {
    EW_PRECHECK("mg_tk_layernorm", x && gamma && beta && y16 && mu && rstd && count_ok(rows) && D > 0 &&
                                       D <= 0x7fffffff && dtype_ok(dtype));
    const bool vec = D % 4 == 0 && D <= 1024 && aligned16(x, gamma, beta) && aligned8(y16);
    const dim3 grid(row_blocks(rows)), block(64 * ROWS_PER_WG);
    uint16_t *y = (uint16_t *)y16;
    if (vec && D <= 256) hipLaunchKernelGGL(k_layernorm_reg<1>, grid, block, 0, ctx_stream(ctx), x, gamma, beta, y, mu, rstd, rows, (int)D, dtype);
    else if (vec && D <= 512) hipLaunchKernelGGL(k_layernorm_reg<2>, grid, block, 0, ctx_stream(ctx), x, gamma, beta, y, mu, rstd, rows, (int)D, dtype);
    else if (vec && D <= 768) hipLaunchKernelGGL(k_layernorm_reg<3>, grid, block, 0, ctx_stream(ctx), x, gamma, beta, y, mu, rstd, rows, (int)D, dtype);
    else if (vec) hipLaunchKernelGGL(k_layernorm_reg<4>, grid, block, 0, ctx_stream(ctx), x, gamma, beta, y, mu, rstd, rows, (int)D, dtype);
    else hipLaunchKernelGGL(k_layernorm, grid, block, 0, ctx_stream(ctx), x, gamma, beta, y, mu, rstd, rows, (int)D, dtype);
    EW_POSTCHECK("mg_tk_layernorm");
}

int mg_tk_layernorm_bwd(mg_ctx *ctx, const float *dy, const float *x, const float *gamma, const float *mu,
                        const float *rstd, float *dx, void *dyxh16, void *dy16, int64_t rows, int64_t D, int dtype) {
    EW_PRECHECK("mg_tk_layernorm_bwd", dy && x && gamma && mu && rstd && dx && dyxh16 && dy16 && count_ok(rows) &&
                                           D > 0 && D <= 0x7fffffff && dtype_ok(dtype));
    const bool vec = D % 4 == 0 && D <= 1024 && aligned16(dy, x, gamma) && aligned16(dx, dx, dx) && aligned8(dyxh16) &&
                     aligned8(dy16);
    const dim3 grid(row_blocks(rows)), block(64 * ROWS_PER_WG);
    uint16_t *o1 = (uint16_t *)dyxh16, *o2 = (uint16_t *)dy16;
    if (vec && D <= 256) hipLaunchKernelGGL(k_layernorm_bwd_reg<1>, grid, block, 0, ctx_stream(ctx), dy, x, gamma, mu, rstd, dx, o1, o2, rows, (int)D, dtype);
    else if (vec && D <= 512) hipLaunchKernelGGL(k_layernorm_bwd_reg<2>, grid, block, 0, ctx_stream(ctx), dy, x, gamma, mu, rstd, dx, o1, o2, rows, (int)D, dtype);
    else if (vec && D <= 768) hipLaunchKernelGGL(k_layernorm_bwd_reg<3>, grid, block, 0, ctx_stream(ctx), dy, x, gamma, mu, rstd, dx, o1, o2, rows, (int)D, dtype);
    else if (vec) hipLaunchKernelGGL(k_layernorm_bwd_reg<4>, grid, block, 0, ctx_stream(ctx), dy, x, gamma, mu, rstd, dx, o1, o2, rows, (int)D, dtype);
    else hipLaunchKernelGGL(k_layernorm_bwd, grid, block, 0, ctx_stream(ctx), dy, x, gamma, mu, rstd, dx, o1, o2, rows, (int)D, dtype);
    EW_POSTCHECK("mg_tk_layernorm_bwd");
}

int mg_tk_attn_softmax(mg_ctx *ctx, const float *s, const uint32_t *seg, void *p16, int64_t rows, int64_t T, int64_t H,
                       float scale, int dtype) {
    EW_PRECHECK("mg_tk_attn_softmax", s && p16 && count_ok(rows) && T > 0 && T <= 0x7fffffff && rows % T == 0 &&
                                          H > 0 && (!seg || (rows / T) % H == 0) && dtype_ok(dtype));
    const bool vec = T % 4 == 0 && T <= 1024 && (((uintptr_t)s & 15) == 0) && (((uintptr_t)p16 & 7) == 0);
    const dim3 grid(row_blocks(rows)), block(64 * ROWS_PER_WG);
    uint16_t *p = (uint16_t *)p16;
    if (vec && T <= 256) hipLaunchKernelGGL(k_attn_softmax_reg<1>, grid, block, 0, ctx_stream(ctx), s, seg, p, rows, (int)T, (int)H, scale, dtype);
    else if (vec && T <= 512) hipLaunchKernelGGL(k_attn_softmax_reg<2>, grid, block, 0, ctx_stream(ctx), s, seg, p, rows, (int)T, (int)H, scale, dtype);
    else if (vec) hipLaunchKernelGGL(k_attn_softmax_reg<4>, grid, block, 0, ctx_stream(ctx), s, seg, p, rows, (int)T, (int)H, scale, dtype);
    else hipLaunchKernelGGL(k_attn_softmax, grid, block, 0, ctx_stream(ctx), s, seg, p, rows, (int)T, (int)H, scale, dtype);
    EW_POSTCHECK("mg_tk_attn_softmax");
}

int mg_tk_attn_softmax_bwd(mg_ctx *ctx, const float *dp, const void *p16, void *ds16, int64_t rows, int64_t T,
                           float scale, int dtype) {
    EW_PRECHECK("mg_tk_attn_softmax_bwd", dp && p16 && ds16 && count_ok(rows) && T > 0 && T <= 0x7fffffff &&
                                              rows % T == 0 && dtype_ok(dtype));
    const bool vec = T % 4 == 0 && T <= 1024 && (((uintptr_t)dp & 15) == 0) &&
                     ((((uintptr_t)p16 | (uintptr_t)ds16) & 7) == 0);
    const dim3 grid(row_blocks(rows)), block(64 * ROWS_PER_WG);
    const uint16_t *p = (const uint16_t *)p16;
    uint16_t *d = (uint16_t *)ds16;
    if (vec && T <= 256) hipLaunchKernelGGL(k_attn_softmax_bwd_reg<1>, grid, block, 0, ctx_stream(ctx), dp, p, d, rows, (int)T, scale, dtype);
    else if (vec && T <= 512) hipLaunchKernelGGL(k_attn_softmax_bwd_reg<2>, grid, block, 0, ctx_stream(ctx), dp, p, d, rows, (int)T, scale, dtype);
    else if (vec) hipLaunchKernelGGL(k_attn_softmax_bwd_reg<4>, grid, block, 0, ctx_stream(ctx), dp, p, d, rows, (int)T, scale, dtype);
    else hipLaunchKernelGGL(k_attn_softmax_bwd, grid, block, 0, ctx_stream(ctx), dp, p, d, rows, (int)T, scale, dtype);
    EW_POSTCHECK("mg_tk_attn_softmax_bwd");
}

int mg_tk_attn_rowdot(mg_ctx *ctx, const void *a16, const float *b32, float *out, int64_t rows, int64_t D, int dtype) {
    EW_PRECHECK("mg_tk_attn_rowdot", a16 && b32 && out && rows > 0 && rows <= (int64_t)0x7fffffff * 4 && D > 0 &&
                                         D <= 0x7fffffff && dtype_ok(dtype));
    if (D % 8 == 0 && (((uintptr_t)a16 | (uintptr_t)b32) & 15) == 0)
        hipLaunchKernelGGL(k_attn_rowdot_v8, dim3((unsigned)((rows + 31) / 32)), dim3(256), 0, ctx_stream(ctx),
                           (const uint16_t *)a16, b32, out, rows, (int)D, dtype);
    else
        hipLaunchKernelGGL(k_attn_rowdot, dim3(row_blocks(rows)), dim3(64 * ROWS_PER_WG), 0, ctx_stream(ctx),
                           (const uint16_t *)a16, b32, out, rows, (int)D, dtype);
    EW_POSTCHECK("mg_tk_attn_rowdot");
}

int mg_tk_split_qkv(mg_ctx *ctx, const float *qkv, const float *bias, void *q16, void *k16, void *v16, int64_t n,
                    int64_t D, int64_t T, int64_t H, int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_split_qkv", qkv && q16 && k16 && v16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) &&
                                       dtype_ok(dtype));
    if (hd % 4 == 0 && aligned16(qkv, bias, bias) && aligned8(q16) && aligned8(k16) && aligned8(v16))
        hipLaunchKernelGGL(k_split_qkv_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), qkv, bias, (uint16_t *)q16,
                           (uint16_t *)k16, (uint16_t *)v16, n / 4, (int)D, (int)T, (int)H, (int)hd, dtype);
    else
        hipLaunchKernelGGL(k_split_qkv, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), qkv, bias, (uint16_t *)q16,
                           (uint16_t *)k16, (uint16_t *)v16, n, (int)D, (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_split_qkv");
}

int mg_tk_merge_qkv_grad(mg_ctx *ctx, const float *dq, const float *dk, const float *dv, void *dqkv16, int64_t n,
                         int64_t D, int64_t T, int64_t H, int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_merge_qkv_grad", dq && dk && dv && dqkv16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) &&
                                            dtype_ok(dtype));
    if (hd % 4 == 0 && aligned16(dq, dk, dv) && aligned8(dqkv16))
        hipLaunchKernelGGL(k_merge_qkv_grad_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), dq, dk, dv,
                           (uint16_t *)dqkv16, n / 4, (int)D, (int)T, (int)H, (int)hd, dtype);
    else
        hipLaunchKernelGGL(k_merge_qkv_grad, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dq, dk, dv,
                           (uint16_t *)dqkv16, n, (int)D, (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_merge_qkv_grad");
}

int mg_tk_merge_heads(mg_ctx *ctx, const float *src, void *y16, int64_t n, int64_t D, int64_t T, int64_t H, int64_t hd,
                      int dtype) {
    EW_PRECHECK("mg_tk_merge_heads", src && y16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) && dtype_ok(dtype));
    if (hd % 4 == 0 && aligned16(src, src, src) && aligned8(y16))
        hipLaunchKernelGGL(k_heads_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)y16, n / 4,
                           (int)D, (int)T, (int)H, (int)hd, dtype, 0);
    else
        hipLaunchKernelGGL(k_merge_heads, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)y16, n, (int)D,
                           (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_merge_heads");
}

int mg_tk_split_heads(mg_ctx *ctx, const float *src, void *dst16, int64_t n, int64_t D, int64_t T, int64_t H,
                      int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_split_heads", src && dst16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) && dtype_ok(dtype));
    if (hd % 4 == 0 && aligned16(src, src, src) && aligned8(dst16))
        hipLaunchKernelGGL(k_heads_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)dst16, n / 4,
                           (int)D, (int)T, (int)H, (int)hd, dtype, 1);
    else
        hipLaunchKernelGGL(k_split_heads, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)dst16, n,
                           (int)D, (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_split_heads");
}

int mg_tk_embed(mg_ctx *ctx, const float *tok, const float *pos, const uint32_t *ids, const uint32_t *seg, float *x,
                int64_t n, int64_t D, int64_t T) {
    EW_PRECHECK("mg_tk_embed", tok && pos && ids && x && count_ok(n) && D > 0 && T > 0 && D <= 0x7fffffff &&
                                   T <= 0x7fffffff && n % D == 0);
    hipLaunchKernelGGL(k_embed, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), tok, pos, ids, seg, x, n, (int)D,
                       (int)T);
    EW_POSTCHECK("mg_tk_embed");
}

int mg_tk_embed_bwd(mg_ctx *ctx, const float *dx, const uint32_t *ids, const uint32_t *seg, float *dtok, float *dpos,
                    int64_t n, int64_t D, int64_t T) {
    EW_PRECHECK("mg_tk_embed_bwd", dx && ids && dtok && dpos && count_ok(n) && D > 0 && T > 0 && D <= 0x7fffffff &&
                                       T <= 0x7fffffff && n % D == 0);
    hipLaunchKernelGGL(k_embed_bwd, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dx, ids, seg, dtok, dpos, n,
                       (int)D, (int)T);
    EW_POSTCHECK("mg_tk_embed_bwd");
}

int mg_tk_residual(mg_ctx *ctx, const float *acc, const float *bias, const float *res, float *out, int64_t n,
                   int64_t D) {
    EW_PRECHECK("mg_tk_residual", acc && bias && res && out && count_ok(n) && D > 0 && D <= 0x7fffffff);
    if (n % 4 == 0 && D % 4 == 0 && aligned16(acc, bias, res) && aligned16(out, out, out))
        hipLaunchKernelGGL(k_add_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), res, acc, bias, out, n / 4, (int)D);
    else
        hipLaunchKernelGGL(k_residual, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), acc, bias, res, out, n, (int)D);
    EW_POSTCHECK("mg_tk_residual");
}

int mg_tk_add(mg_ctx *ctx, const float *a, const float *b, float *out, int64_t n) {
    EW_PRECHECK("mg_tk_add", a && b && out && count_ok(n));
    if (n % 4 == 0 && aligned16(a, b, out))
        hipLaunchKernelGGL(k_add_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), a, b, (const float *)nullptr, out,
                           n / 4, 4);
    else
        hipLaunchKernelGGL(k_add, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), a, b, out, n);
    EW_POSTCHECK("mg_tk_add");
}

int mg_tk_add16(mg_ctx *ctx, const float *a, const float *b, float *out, void *out16, int64_t n, int dtype) {
    EW_PRECHECK("mg_tk_add16", a && b && out && out16 && count_ok(n) && dtype_ok(dtype));
    if (n % 4 == 0 && aligned16(a, b, out) && aligned8(out16))
        hipLaunchKernelGGL(k_add16_v4, dim3(blocks_for(n / 4)), dim3(256), 0, ctx_stream(ctx), a, b, out, (uint16_t *)out16,
                           n / 4, dtype);
    else
        hipLaunchKernelGGL(k_add16, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), a, b, out, (uint16_t *)out16, n, dtype);
    EW_POSTCHECK("mg_tk_add16");
}

int mg_tk_add_bias(mg_ctx *ctx, float *x, const float *bias, int64_t n, int64_t ncol) {
    EW_PRECHECK("mg_tk_add_bias", x && bias && count_ok(n) && ncol > 0);
    hipLaunchKernelGGL(k_add_bias, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), x, bias, n, ncol);
    EW_POSTCHECK("mg_tk_add_bias");
}

int mg_tk_col_sum16(mg_ctx *ctx, const void *g16, float *sums, int64_t ncol, int64_t nrow, int accumulate, int dtype) {
    EW_PRECHECK("mg_tk_col_sum16", g16 && sums && count_ok(ncol) && nrow > 0 && nrow <= (int64_t)65535 * CS16_ROWS &&
                                       dtype_ok(dtype));
    const unsigned chunks = (unsigned)((nrow + CS16_ROWS - 1) / CS16_ROWS);
    if (chunks > 1 && !accumulate)
        hipLaunchKernelGGL(k_zero_f32, dim3(blocks_for(ncol)), dim3(256), 0, ctx_stream(ctx), sums, ncol);
    hipLaunchKernelGGL(k_col_sum16, dim3((unsigned)((ncol + 63) / 64), chunks), dim3(512), 0, ctx_stream(ctx),
                       (const uint16_t *)g16, sums, ncol, nrow, accumulate, chunks > 1 ? 1 : 0, dtype);
    EW_POSTCHECK("mg_tk_col_sum16");
}

int mg_tk_softmax_ce(mg_ctx *ctx, const float *logits, const uint32_t *labels, const float *weights, void *dl16,
                     float *dl32, float *loss, int64_t nrows, int64_t stride, int64_t ncls, int dtype) {
    EW_PRECHECK("mg_tk_softmax_ce", logits && labels && loss && nrows > 0 && nrows <= 0x7fffffff && ncls > 0 &&
                                        stride >= ncls && dtype_ok(dtype));
    const int vec = stride % 4 == 0 && (((uintptr_t)logits | (uintptr_t)dl32) & 15) == 0 && ((uintptr_t)dl16 & 7) == 0;
    if (ncls >= 16384)   // a vocabulary
        hipLaunchKernelGGL(k_softmax_ce_wide<1024>, dim3((unsigned)nrows), dim3(1024), 0, ctx_stream(ctx), logits, labels, weights,
                           (uint16_t *)dl16, dl32, loss, nrows, stride, ncls, dtype, vec);
    else
        hipLaunchKernelGGL(k_softmax_ce_wide<256>, dim3((unsigned)nrows), dim3(256), 0, ctx_stream(ctx), logits, labels, weights,
                           (uint16_t *)dl16, dl32, loss, nrows, stride, ncls, dtype, vec);
    EW_POSTCHECK("mg_tk_softmax_ce");
}

}  // extern "C"
