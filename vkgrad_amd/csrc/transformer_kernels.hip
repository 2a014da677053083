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
// through float atomics (the host clears sums first unless accumulating).
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

// ---- Softmax cross-entropy over a wide row (the LM head: 50257 classes).  Same arithmetic as
// the one-thread-per-row kernel of the MLP (kernels.py:766-791), with the row spread over a
// 256-thread workgroup: max, sum of exponentials and the gradient sweep are each one coalesced
// pass; weight[row] (or 1 / nrows) scales the gradient (softmax_ce_w, transformer.py:331-337).
__global__ void __launch_bounds__(256)
k_softmax_ce_wide(const float *logits, const uint32_t *labels, const float *weights, uint16_t *dl16, float *dl32,
                  float *loss, int64_t nrows, int64_t stride, int64_t ncls, int dtype) {
    __shared__ float red[4];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float *lr = logits + row * stride;
    if (weights && weights[row] == 0.f) {   // masked row: no softmax, zeros (uniform over the workgroup)
        for (int64_t c = tid; c < stride; c += 256) {
            if (dl16) dl16[row * stride + c] = 0;
            if (dl32) dl32[row * stride + c] = 0.f;
        }
        if (tid == 0) loss[row] = 0.f;
        return;
    }
    float mx = -1e30f;
    for (int64_t c = tid; c < ncls; c += 256) mx = fmaxf(mx, lr[c]);
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float s = 0.f;
    for (int64_t c = tid; c < ncls; c += 256) s += __expf(lr[c] - mx);
    s = wave_sum(s);
    if (lane == 0) red[wave] = s;
    __syncthreads();
    s = (red[0] + red[1]) + (red[2] + red[3]);
    const float logZ = mx + __logf(s);
    const uint32_t y = labels[row];
    const float w = weights ? weights[row] : 1.0f / (float)nrows;
    if (tid == 0) loss[row] = logZ - lr[y];
    for (int64_t c = tid; c < stride; c += 256) {
        float gv = 0.f;
        if (c < ncls) gv = (__expf(lr[c] - logZ) - (c == (int64_t)y ? 1.f : 0.f)) * w;
        if (dl16) dl16[row * stride + c] = narrow16(gv, dtype);
        if (dl32) dl32[row * stride + c] = gv;
    }
}

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
    hipLaunchKernelGGL(k_layernorm, dim3(row_blocks(rows)), dim3(64 * ROWS_PER_WG), 0, ctx_stream(ctx), x, gamma, beta,
                       (uint16_t *)y16, mu, rstd, rows, (int)D, dtype);
    EW_POSTCHECK("mg_tk_layernorm");
}

int mg_tk_layernorm_bwd(mg_ctx *ctx, const float *dy, const float *x, const float *gamma, const float *mu,
                        const float *rstd, float *dx, void *dyxh16, void *dy16, int64_t rows, int64_t D, int dtype) {
    EW_PRECHECK("mg_tk_layernorm_bwd", dy && x && gamma && mu && rstd && dx && dyxh16 && dy16 && count_ok(rows) &&
                                           D > 0 && D <= 0x7fffffff && dtype_ok(dtype));
    hipLaunchKernelGGL(k_layernorm_bwd, dim3(row_blocks(rows)), dim3(64 * ROWS_PER_WG), 0, ctx_stream(ctx), dy, x, gamma,
                       mu, rstd, dx, (uint16_t *)dyxh16, (uint16_t *)dy16, rows, (int)D, dtype);
    EW_POSTCHECK("mg_tk_layernorm_bwd");
}

int mg_tk_attn_softmax(mg_ctx *ctx, const float *s, const uint32_t *seg, void *p16, int64_t rows, int64_t T, int64_t H,
                       float scale, int dtype) {
    EW_PRECHECK("mg_tk_attn_softmax", s && p16 && count_ok(rows) && T > 0 && T <= 0x7fffffff && rows % T == 0 &&
                                          H > 0 && (!seg || (rows / T) % H == 0) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_attn_softmax, dim3(row_blocks(rows)), dim3(64 * ROWS_PER_WG), 0, ctx_stream(ctx), s, seg,
                       (uint16_t *)p16, rows, (int)T, (int)H, scale, dtype);
    EW_POSTCHECK("mg_tk_attn_softmax");
}

int mg_tk_attn_softmax_bwd(mg_ctx *ctx, const float *dp, const void *p16, void *ds16, int64_t rows, int64_t T,
                           float scale, int dtype) {
    EW_PRECHECK("mg_tk_attn_softmax_bwd", dp && p16 && ds16 && count_ok(rows) && T > 0 && T <= 0x7fffffff &&
                                              rows % T == 0 && dtype_ok(dtype));
    hipLaunchKernelGGL(k_attn_softmax_bwd, dim3(row_blocks(rows)), dim3(64 * ROWS_PER_WG), 0, ctx_stream(ctx), dp,
                       (const uint16_t *)p16, (uint16_t *)ds16, rows, (int)T, scale, dtype);
    EW_POSTCHECK("mg_tk_attn_softmax_bwd");
}

int mg_tk_split_qkv(mg_ctx *ctx, const float *qkv, const float *bias, void *q16, void *k16, void *v16, int64_t n,
                    int64_t D, int64_t T, int64_t H, int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_split_qkv", qkv && q16 && k16 && v16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) &&
                                       dtype_ok(dtype));
    hipLaunchKernelGGL(k_split_qkv, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), qkv, bias, (uint16_t *)q16,
                       (uint16_t *)k16, (uint16_t *)v16, n, (int)D, (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_split_qkv");
}

int mg_tk_merge_qkv_grad(mg_ctx *ctx, const float *dq, const float *dk, const float *dv, void *dqkv16, int64_t n,
                         int64_t D, int64_t T, int64_t H, int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_merge_qkv_grad", dq && dk && dv && dqkv16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) &&
                                            dtype_ok(dtype));
    hipLaunchKernelGGL(k_merge_qkv_grad, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), dq, dk, dv,
                       (uint16_t *)dqkv16, n, (int)D, (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_merge_qkv_grad");
}

int mg_tk_merge_heads(mg_ctx *ctx, const float *src, void *y16, int64_t n, int64_t D, int64_t T, int64_t H, int64_t hd,
                      int dtype) {
    EW_PRECHECK("mg_tk_merge_heads", src && y16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) && dtype_ok(dtype));
    hipLaunchKernelGGL(k_merge_heads, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), src, (uint16_t *)y16, n, (int)D,
                       (int)T, (int)H, (int)hd, dtype);
    EW_POSTCHECK("mg_tk_merge_heads");
}

int mg_tk_split_heads(mg_ctx *ctx, const float *src, void *dst16, int64_t n, int64_t D, int64_t T, int64_t H,
                      int64_t hd, int dtype) {
    EW_PRECHECK("mg_tk_split_heads", src && dst16 && heads_ok(n, (int)D, (int)T, (int)H, (int)hd) && dtype_ok(dtype));
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
    hipLaunchKernelGGL(k_residual, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), acc, bias, res, out, n, (int)D);
    EW_POSTCHECK("mg_tk_residual");
}

int mg_tk_add(mg_ctx *ctx, const float *a, const float *b, float *out, int64_t n) {
    EW_PRECHECK("mg_tk_add", a && b && out && count_ok(n));
    hipLaunchKernelGGL(k_add, dim3(blocks_for(n)), dim3(256), 0, ctx_stream(ctx), a, b, out, n);
    EW_POSTCHECK("mg_tk_add");
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
    hipLaunchKernelGGL(k_softmax_ce_wide, dim3((unsigned)nrows), dim3(256), 0, ctx_stream(ctx), logits, labels, weights,
                       (uint16_t *)dl16, dl32, loss, nrows, stride, ncls, dtype);
    EW_POSTCHECK("mg_tk_softmax_ce");
}

}  // extern "C"
