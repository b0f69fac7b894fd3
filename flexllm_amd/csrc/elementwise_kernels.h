// Row-wise and elementwise fp32 stages: per-token quantisation, dequantisation, static per-head
// quantisation, RMSNorm, RoPE, SiLU/gate, residual add, softmax.  All are HBM-bound: one workgroup
// (256 threads, 4 waves) per row, float4 loads, the row kept in registers between the reduction and
// the write-back so each input byte is read from HBM once.
#pragma once
#include "common.h"
#include <math.h>

namespace fx {

constexpr int kBlock = 256;
constexpr int kNW = kBlock / kWave;

// ------------------------------------------------------------------ per-token symmetric int8
// VPT float4 vectors per thread are cached in registers (row length <= 1024*VPT floats).
template <int VPT>
__global__ __launch_bounds__(kBlock) void quant_sym_kernel(const float* __restrict__ x, int8_t* __restrict__ q,
                                                           float* __restrict__ s, int dim) {
    __shared__ float red[kNW];
    const int row = blockIdx.x;
    const int nvec = dim >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * dim);
    float4 v[VPT];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < nvec) {
            v[i] = xr[idx];
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))));
        }
    }
    amax = block_max<kNW>(amax, red);
    const float sc = sym_scale_127_uniform(amax);
    if (threadIdx.x == 0) s[row] = sc;
    uint32_t* qr = reinterpret_cast<uint32_t*>(q + (size_t)row * dim);
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < nvec) {
            const float f[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
            int n[4];
            quant_vector(f, sc, n);
            qr[idx] = pack4_i8(n[0], n[1], n[2], n[3]);
        }
    }
}

template <int VPT>
__global__ __launch_bounds__(kBlock) void quant_asym_kernel(const float* __restrict__ x, uint8_t* __restrict__ q,
                                                            float* __restrict__ s, float* __restrict__ b, int dim,
                                                            float scale_base, unsigned mask) {
    __shared__ float red[kNW];
    const int row = blockIdx.x;
    const int nvec = dim >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * dim);
    float4 v[VPT];
    float vmax = -1e32f, vmin = 1e32f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < nvec) {
            v[i] = xr[idx];
            vmax = fmaxf(vmax, fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)));
            vmin = fminf(vmin, fminf(fminf(v[i].x, v[i].y), fminf(v[i].z, v[i].w)));
        }
    }
    vmax = block_max<kNW>(vmax, red);
    vmin = block_min<kNW>(vmin, red);
    float sc = (vmax - vmin) / scale_base;
    if (sc == 0.0f) sc = 1.0f;
    if (threadIdx.x == 0) { s[row] = sc; b[row] = vmin; }
    uint32_t* qr = reinterpret_cast<uint32_t*>(q + (size_t)row * dim);
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * kBlock;
        if (idx < nvec) {
            // round((x - min) / s) through the reciprocal, with the division itself only next to a rounding tie: the
            // same integers (quant_vector)
            const float f[4] = {v[i].x - vmin, v[i].y - vmin, v[i].z - vmin, v[i].w - vmin};
            int nq[4];
            quant_vector(f, sc, nq);
            qr[idx] = pack4_i8(nq[0] & mask, nq[1] & mask, nq[2] & mask, nq[3] & mask);
        }
    }
}

// ------------------------------------------------------------------ RMSNorm (+ optional quant)
// BLOCK threads per row.  With BLOCK = 512 and VPT = 1 a 2048-row is reduced exactly as the persistent decode kernel
// reduces it (four values per thread, wave butterflies, the eight wave sums added in order), so the one-kernel-per-
// stage decode schedule and the persistent kernel agree bit for bit.
template <int VPT, bool QUANT, int BLOCK = kBlock>
__global__ __launch_bounds__(BLOCK) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ gamma,
                                                         float* __restrict__ y, int8_t* __restrict__ q,
                                                         float* __restrict__ s, int dim, float eps) {
    __shared__ float red[BLOCK / kWave];
    const int row = blockIdx.x;
    const int nvec = dim >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * dim);
    const float4* gr = reinterpret_cast<const float4*>(gamma);
    float4 v[VPT];
    float ss = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * BLOCK;
        if (idx < nvec) {
            v[i] = xr[idx];
            ss += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
        }
    }
    ss = block_sum<BLOCK / kWave>(ss, red);
    const float rms = 1.0f / sqrtf(ss / (float)dim + eps);
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < VPT; i++) {
        const int idx = threadIdx.x + i * BLOCK;
        if (idx < nvec) {
            const float4 g = gr[idx];
            v[i].x = v[i].x * rms * g.x;
            v[i].y = v[i].y * rms * g.y;
            v[i].z = v[i].z * rms * g.z;
            v[i].w = v[i].w * rms * g.w;
            if constexpr (QUANT)
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[i].x), fabsf(v[i].y)), fmaxf(fabsf(v[i].z), fabsf(v[i].w))));
            else
                reinterpret_cast<float4*>(y + (size_t)row * dim)[idx] = v[i];
        }
    }
    if constexpr (QUANT) {
        amax = block_max<BLOCK / kWave>(amax, red);
        const float sc = sym_scale_127_uniform(amax);
        if (threadIdx.x == 0) s[row] = sc;
        uint32_t* qr = reinterpret_cast<uint32_t*>(q + (size_t)row * dim);
#pragma unroll
        for (int i = 0; i < VPT; i++) {
            const int idx = threadIdx.x + i * BLOCK;
            if (idx < nvec) {
                const float f[4] = {v[i].x, v[i].y, v[i].z, v[i].w};
                int nq[4];
                quant_vector(f, sc, nq);
                qr[idx] = pack4_i8(nq[0], nq[1], nq[2], nq[3]);
            }
        }
    }
}

// RMSNorm + per-row int8 quantisation of rows of 2048 values, one WAVE per row (prefill: a thousand rows or more at
// once).  A row is eight 16-byte loads per lane, all in flight together, and the two reductions stay inside the wave:
// no LDS, no workgroup barrier.  The arithmetic is that of rmsnorm_kernel<1, true, 512> to the bit: lane l holds the
// values thread 64 w + l holds there (w = 0..7), the squares of each w are summed by the same wave butterfly, the
// eight sums are added in the same order, and a maximum does not depend on the order.
constexpr int kNormWaveRows = 4;                       // rows (waves) per workgroup
static __global__ __launch_bounds__(64 * kNormWaveRows) void rmsnorm_quant_2048_wave_kernel(
    const float* __restrict__ x, const float* __restrict__ gamma, int8_t* __restrict__ q, float* __restrict__ s, int rows, float eps) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kNormWaveRows + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (row >= rows) return;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * 2048);
    const float4* gr = reinterpret_cast<const float4*>(gamma);
    float4 v[8], g[8];
#pragma unroll
    for (int w = 0; w < 8; w++) v[w] = xr[w * 64 + lane];
#pragma unroll
    for (int w = 0; w < 8; w++) g[w] = gr[w * 64 + lane];
    float ss = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const float part = wave_sum((v[w].x * v[w].x + v[w].y * v[w].y) + (v[w].z * v[w].z + v[w].w * v[w].w));
        ss = w == 0 ? part : ss + part;
    }
    const float rms = 1.0f / sqrtf(ss / 2048.0f + eps);
    float amax = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        v[w].x = v[w].x * rms * g[w].x;
        v[w].y = v[w].y * rms * g[w].y;
        v[w].z = v[w].z * rms * g[w].z;
        v[w].w = v[w].w * rms * g[w].w;
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[w].x), fabsf(v[w].y)), fmaxf(fabsf(v[w].z), fabsf(v[w].w))));
    }
    amax = wave_max(amax);
    const float sc = sym_scale_127_uniform(amax);
    if (lane == 0) s[row] = sc;
    uint32_t* qr = reinterpret_cast<uint32_t*>(q + (size_t)row * 2048);
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const float f[4] = {v[w].x, v[w].y, v[w].z, v[w].w};
        int nq[4];
        quant_vector(f, sc, nq);
        qr[w * 64 + lane] = pack4_i8(nq[0], nq[1], nq[2], nq[3]);
    }
}

// The same for the W4A4 graph: RMSNorm of a row of 2048 values and its asymmetric quantisation to `levels` steps
// (uint4: scale_base 15, mask 15), one wave per row - what rmsnorm_kernel<1, false, 512> followed by quant_asym_kernel
// compute, to the bit (same sum of squares, maxima and minima do not depend on the order).
static __global__ __launch_bounds__(64 * kNormWaveRows) void rmsnorm_quant_asym_2048_wave_kernel(
    const float* __restrict__ x, const float* __restrict__ gamma, uint8_t* __restrict__ q, float* __restrict__ s,
    float* __restrict__ b, int rows, float eps, float scale_base, unsigned mask) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * kNormWaveRows + __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if (row >= rows) return;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * 2048);
    const float4* gr = reinterpret_cast<const float4*>(gamma);
    float4 v[8], g[8];
#pragma unroll
    for (int w = 0; w < 8; w++) v[w] = xr[w * 64 + lane];
#pragma unroll
    for (int w = 0; w < 8; w++) g[w] = gr[w * 64 + lane];
    float ss = 0.0f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const float part = wave_sum((v[w].x * v[w].x + v[w].y * v[w].y) + (v[w].z * v[w].z + v[w].w * v[w].w));
        ss = w == 0 ? part : ss + part;
    }
    const float rms = 1.0f / sqrtf(ss / 2048.0f + eps);
    float vmax = -1e32f, vmin = 1e32f;
#pragma unroll
    for (int w = 0; w < 8; w++) {
        v[w].x = v[w].x * rms * g[w].x;
        v[w].y = v[w].y * rms * g[w].y;
        v[w].z = v[w].z * rms * g[w].z;
        v[w].w = v[w].w * rms * g[w].w;
        vmax = fmaxf(vmax, fmaxf(fmaxf(v[w].x, v[w].y), fmaxf(v[w].z, v[w].w)));
        vmin = fminf(vmin, fminf(fminf(v[w].x, v[w].y), fminf(v[w].z, v[w].w)));
    }
    vmax = wave_max(vmax);
    vmin = wave_min(vmin);
    float sc = (vmax - vmin) / scale_base;
    if (sc == 0.0f) sc = 1.0f;
    if (lane == 0) { s[row] = sc; b[row] = vmin; }
    uint32_t* qr = reinterpret_cast<uint32_t*>(q + (size_t)row * 2048);
#pragma unroll
    for (int w = 0; w < 8; w++) {
        const float f[4] = {v[w].x - vmin, v[w].y - vmin, v[w].z - vmin, v[w].w - vmin};
        int nq[4];
        quant_vector(f, sc, nq);
        qr[w * 64 + lane] = pack4_i8(nq[0] & mask, nq[1] & mask, nq[2] & mask, nq[3] & mask);
    }
}

// ------------------------------------------------------------------ elementwise
static __global__ __launch_bounds__(kBlock) void dequant_kernel(const int32_t* __restrict__ acc, const float* __restrict__ s_x,
                                                         const float* __restrict__ b_x, const float* __restrict__ w_s,
                                                         const float* __restrict__ w_sum, float* __restrict__ y,
                                                         int n4) {
    // grid.y = row, n4 = n/4 vectors per row
    const int row = blockIdx.y;
    const float sx = s_x[row];
    const bool asym = b_x != nullptr;
    const float bx = asym ? b_x[row] : 0.0f;
    for (int i = blockIdx.x * kBlock + threadIdx.x; i < n4; i += gridDim.x * kBlock) {
        const int4 a = reinterpret_cast<const int4*>(acc)[(size_t)row * n4 + i];
        const float4 w = reinterpret_cast<const float4*>(w_s)[i];
        float4 r;
        r.x = (float)a.x * sx * w.x;
        r.y = (float)a.y * sx * w.y;
        r.z = (float)a.z * sx * w.z;
        r.w = (float)a.w * sx * w.w;
        if (asym) {
            const float4 ws = reinterpret_cast<const float4*>(w_sum)[i];
            r.x = r.x + bx * ws.x;
            r.y = r.y + bx * ws.y;
            r.z = r.z + bx * ws.z;
            r.w = r.w + bx * ws.w;
        }
        reinterpret_cast<float4*>(y)[(size_t)row * n4 + i] = r;
    }
}

__device__ __forceinline__ int static_q(float x, float div, bool is_signed) {
    int r = (int)roundf(x / div);
    if (is_signed) return r > 127 ? 127 : r < -128 ? -128 : r;
    return r > 255 ? 255 : r;
}

static __global__ __launch_bounds__(kBlock) void static_quant_kernel(const float* __restrict__ x, int8_t* __restrict__ q,
                                                              const float* __restrict__ scale, float factor,
                                                              int is_signed, size_t nvec, int heads, int dim4) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (size_t)gridDim.x * kBlock) {
        const int h = (int)((i / dim4) % heads);
        const float div = factor * scale[h];
        const float4 v = reinterpret_cast<const float4*>(x)[i];
        reinterpret_cast<uint32_t*>(q)[i] = pack4_i8(static_q(v.x, div, is_signed), static_q(v.y, div, is_signed),
                                                     static_q(v.z, div, is_signed), static_q(v.w, div, is_signed));
    }
}

static __global__ __launch_bounds__(kBlock) void static_dequant_kernel(const int32_t* __restrict__ acc, float* __restrict__ y,
                                                                const float* __restrict__ a_s,
                                                                const float* __restrict__ w_s, size_t nvec, int act_heads,
                                                                int group, int dim4) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < nvec; i += (size_t)gridDim.x * kBlock) {
        const int h = (int)((i / dim4) % act_heads);
        const float sa = a_s[h], sw = w_s[h / group];
        const int4 a = reinterpret_cast<const int4*>(acc)[i];
        float4 r;
        r.x = (float)a.x * sa * sw;
        r.y = (float)a.y * sa * sw;
        r.z = (float)a.z * sa * sw;
        r.w = (float)a.w * sa * sw;
        reinterpret_cast<float4*>(y)[i] = r;
    }
}

// one wave per (row, head): dim <= 256
static __global__ __launch_bounds__(kBlock) void head_quant_kernel(const float* __restrict__ x, int8_t* __restrict__ q,
                                                            float* __restrict__ s, int nrows, int dim) {
    const int row = blockIdx.x * kNW + (threadIdx.x >> 6);
    if (row >= nrows) return;
    const int lane = threadIdx.x & 63;
    const int nvec = dim >> 2;
    const float4* xr = reinterpret_cast<const float4*>(x + (size_t)row * dim);
    float4 v = make_float4(0, 0, 0, 0);
    if (lane < nvec) v = xr[lane];
    float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
    amax = wave_max(amax);
    const float sc = sym_scale_127_uniform(amax);
    if (lane == 0) s[row] = sc;
    if (lane < nvec)
        reinterpret_cast<uint32_t*>(q + (size_t)row * dim)[lane] =
            pack4_i8(quant_round(v.x, sc), quant_round(v.y, sc), quant_round(v.z, sc), quant_round(v.w, sc));
}

static __global__ __launch_bounds__(kBlock) void rope_kernel(const float* __restrict__ x, float* __restrict__ y,
                                                      const float* __restrict__ sin_t, const float* __restrict__ cos_t,
                                                      size_t npairs, int heads, int half, int pos0) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < npairs; i += (size_t)gridDim.x * kBlock) {
        const int k = (int)(i % half);
        const size_t th = i / half;              // token*heads + head
        const int t = (int)(th / heads);
        const size_t base = th * (size_t)(2 * half);
        const float sn = sin_t[(size_t)(pos0 + t) * half + k];
        const float cs = cos_t[(size_t)(pos0 + t) * half + k];
        const float t0 = x[base + k], t1 = x[base + k + half];
        y[base + k] = t0 * cs - t1 * sn;
        y[base + k + half] = t0 * sn + t1 * cs;
    }
}

__device__ __forceinline__ float silu(float v) { return silu_f(v); }

static __global__ __launch_bounds__(kBlock) void swish_kernel(const float* __restrict__ x, float* __restrict__ y, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) y[i] = silu(x[i]);
}
static __global__ __launch_bounds__(kBlock) void swiglu_kernel(const float* __restrict__ g, const float* __restrict__ u,
                                                        float* __restrict__ y, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
        y[i] = u[i] * silu(g[i]);
}
static __global__ __launch_bounds__(kBlock) void add_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                     float* __restrict__ y, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) y[i] = a[i] + b[i];
}

// softmax: one block per row, row re-read from cache between the three passes
static __global__ __launch_bounds__(kBlock) void softmax_kernel(const float* __restrict__ x, float* __restrict__ y, int dim) {
    __shared__ float red[kNW];
    const float* xr = x + (size_t)blockIdx.x * dim;
    float* yr = y + (size_t)blockIdx.x * dim;
    float mx = -1e32f;
    for (int i = threadIdx.x; i < dim; i += kBlock) mx = fmaxf(mx, xr[i]);
    mx = block_max<kNW>(mx, red);
    float sum = 0.0f;
    for (int i = threadIdx.x; i < dim; i += kBlock) {
        const float e = expf(xr[i] - mx);
        yr[i] = e;
        sum += e;
    }
    sum = block_sum<kNW>(sum, red);
    const float cd = 1.0f / sum;
    for (int i = threadIdx.x; i < dim; i += kBlock) yr[i] = yr[i] * cd;
}

static inline int ew_grid(size_t n) {
    size_t b = (n + kBlock - 1) / kBlock;
    return (int)(b < 1 ? 1 : b > 4096 ? 4096 : b);
}

}  // namespace fx
