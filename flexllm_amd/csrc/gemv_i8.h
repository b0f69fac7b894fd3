// int8 GEMV core for decode: acc[n] = sum_k x[k]*W[n][k], W row-major [N][K], streamed once from HBM.
//
// One wave owns a run of consecutive output rows.  A row is K bytes; lane l reads the 16-byte chunks
// l, l+64, l+128, ... of the row (each wave-wide load is one contiguous 1 KiB burst), multiplies them with
// the matching activation chunks held in registers via v_dot4_i32_i8, and the 64 partial sums are folded
// with a cross-lane butterfly.  U rows are in flight per wave so that enough bytes are outstanding to
// cover HBM latency.  Integer sums are exact in any order.
#pragma once
#include "common.h"

namespace fx {

__device__ __forceinline__ int dot16(const i32x4& a, const i32x4& b, int acc) {
    acc = __builtin_amdgcn_sdot4(a.x, b.x, acc, false);
    acc = __builtin_amdgcn_sdot4(a.y, b.y, acc, false);
    acc = __builtin_amdgcn_sdot4(a.z, b.z, acc, false);
    acc = __builtin_amdgcn_sdot4(a.w, b.w, acc, false);
    return acc;
}

// Loads the activation vector (K int8) into per-lane registers: chunk c = lane + 64*i.
template <int NCH>
__device__ __forceinline__ void load_x_chunks(const int8_t* __restrict__ x, int nchunks, int lane, i32x4 (&xr)[NCH]) {
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + 64 * i;
        xr[i] = c < nchunks ? reinterpret_cast<const i32x4*>(x)[c] : i32x4{0, 0, 0, 0};
    }
}

// Computes rows [row0, row0+nrows) of W.x for one wave and hands each finished (row, sum) to `epi`
// (called by every lane with the full sum; the functor decides which lane stores).
template <int NCH, int U, class Epi>
__device__ __forceinline__ void wave_gemv_rows(const int8_t* __restrict__ w, const i32x4 (&xr)[NCH], int k, int nchunks,
                                               int row0, int nrows, int lane, Epi epi) {
    int r = 0;
    for (; r + U <= nrows; r += U) {
        i32x4 wv[U][NCH];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const i32x4* wr = reinterpret_cast<const i32x4*>(w + (size_t)(row0 + r + u) * k);
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int c = lane + 64 * i;
                wv[u][i] = c < nchunks ? __builtin_nontemporal_load(wr + c) : i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            int acc = 0;
#pragma unroll
            for (int i = 0; i < NCH; i++) acc = dot16(wv[u][i], xr[i], acc);
            acc = wave_sum_i(acc);
            epi(row0 + r + u, acc);
        }
    }
    for (; r < nrows; r++) {
        const i32x4* wr = reinterpret_cast<const i32x4*>(w + (size_t)(row0 + r) * k);
        int acc = 0;
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + 64 * i;
            if (c < nchunks) acc = dot16(__builtin_nontemporal_load(wr + c), xr[i], acc);
        }
        acc = wave_sum_i(acc);
        epi(row0 + r, acc);
    }
}

constexpr int kGemvBlock = 256;
constexpr int kGemvWaves = kGemvBlock / kWave;

enum GemvEpi { kEpiRaw = 0, kEpiDequant = 1, kEpiSwiglu = 2 };


// rows_per_wave consecutive rows per wave; grid covers ceil(n / (4*rows_per_wave)) blocks.
//   kEpiRaw:     acc_out[row] = sum
//   kEpiDequant: y[row] = (float(sum)*s_x)*w_s[row] (+ residual[row])
//   kEpiSwiglu:  rows are interleaved (2i = gate_i, 2i+1 = up_i); y[i] = up_i * silu(gate_i), both dequantised
//                as above.  rows_per_wave is even, so a pair never straddles two waves.
template <int NCH, int U, int EPI>
__global__ __launch_bounds__(kGemvBlock) void gemv_i8_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ w,
                                                             int32_t* __restrict__ acc_out, const float* __restrict__ s_x,
                                                             const float* __restrict__ w_s,
                                                             const float* __restrict__ residual, float* __restrict__ y,
                                                             int k, int n, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kGemvWaves + (threadIdx.x >> 6);
    const int row0 = gw * rows_per_wave;
    if (row0 >= n) return;
    const int nrows = min(rows_per_wave, n - row0);
    const int nchunks = k >> 4;
    i32x4 xr[NCH];
    load_x_chunks<NCH>(x, nchunks, lane, xr);
    if constexpr (EPI == kEpiDequant) {
        const float sx = s_x[0];
        wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0, nrows, lane, [&](int row, int sum) {
            if (lane == 0) {
                float v = (float)sum * sx * w_s[row];
                if (residual) v = v + residual[row];
                y[row] = v;
            }
        });
    } else if constexpr (EPI == kEpiSwiglu) {
        const float sx = s_x[0];
        float gate = 0.0f;
        wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0, nrows, lane, [&](int row, int sum) {
            const float v = (float)sum * sx * w_s[row];
            if ((row & 1) == 0) gate = v;
            else if (lane == 0) y[row >> 1] = v * silu_f(gate);
        });
    } else {
        wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0, nrows, lane, [&](int row, int sum) {
            if (lane == 0) acc_out[row] = sum;
        });
    }
}

// The whole decode linear of one token in one launch: per-token symmetric int8 quantisation of the fp32 activation,
// GEMV, dequantisation (+ residual).  Every wave quantises the activation for itself, straight into the register
// layout the row products read (lane l holds the 16-value chunks l, l+64, ...): eight 16-byte loads per chunk pair, a
// wave-wide maximum, the library's quantiser arithmetic (sym_scale_127_uniform, quant_vector: the bytes and the scale
// are those of quant_sym_kernel) - no LDS, no workgroup barrier, no second kernel.
template <int NCH, int U>
__global__ __launch_bounds__(kGemvBlock) void gemv_f32_i8_kernel(const float* __restrict__ x, const int8_t* __restrict__ w,
                                                                 const float* __restrict__ w_s, const float* __restrict__ residual,
                                                                 float* __restrict__ y, float* __restrict__ s_x_out,
                                                                 int8_t* __restrict__ q_out, int k, int n, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kGemvWaves + (threadIdx.x >> 6);
    const int row0 = gw * rows_per_wave;
    if (row0 >= n) return;
    const int nrows = min(rows_per_wave, n - row0);
    const int nchunks = k >> 4;
    // the first two weight rows of this wave are requested before anything else: they do not depend on the activation,
    // and the quantisation below (a trip to the cache, a wave-wide maximum, a division) runs while they are on their way
    i32x4 wv[2][NCH];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const i32x4* wr = reinterpret_cast<const i32x4*>(w + (size_t)(row0 + min(u, nrows - 1)) * k);
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + 64 * i;
            wv[u][i] = c < nchunks ? __builtin_nontemporal_load(wr + c) : i32x4{0, 0, 0, 0};
        }
    }
    float4 xf[NCH][4];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + 64 * i;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            xf[i][j] = c < nchunks ? reinterpret_cast<const float4*>(x)[4 * c + j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(xf[i][j].x), fabsf(xf[i][j].y)), fmaxf(fabsf(xf[i][j].z), fabsf(xf[i][j].w))));
        }
    }
    amax = wave_max(amax);
    const float sx = sym_scale_127_uniform(amax);
    i32x4 xr[NCH];
#pragma unroll
    for (int i = 0; i < NCH; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float f[4] = {xf[i][j].x, xf[i][j].y, xf[i][j].z, xf[i][j].w};
            int nq[4];
            quant_vector(f, sx, nq);
            xr[i][j] = (int)pack4_i8(nq[0], nq[1], nq[2], nq[3]);
        }
    if (gw == 0) {                                             // the quantised activation and its scale, on request
        if (s_x_out && lane == 0) s_x_out[0] = sx;
        if (q_out) {
#pragma unroll
            for (int i = 0; i < NCH; i++)
                if (lane + 64 * i < nchunks) reinterpret_cast<i32x4*>(q_out)[lane + 64 * i] = xr[i];
        }
    }
    auto epi = [&](int row, int sum) {
        if (lane == 0) {
            float v = (float)sum * sx * w_s[row];
            if (residual) v = v + residual[row];
            y[row] = v;
        }
    };
#pragma unroll
    for (int u = 0; u < 2; u++) {
        if (u < nrows) {
            int acc = 0;
#pragma unroll
            for (int i = 0; i < NCH; i++) acc = dot16(wv[u][i], xr[i], acc);
            epi(row0 + u, wave_sum_i(acc));
        }
    }
    if (nrows > 2) wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0 + 2, nrows - 2, lane, epi);
}

// Picks rows per wave so that the chip holds ~8 waves per CU while each wave still streams several KiB.
static inline int pick_rows_per_wave(int k, int n) {
    const int target_waves = 256 * 8;  // 256 CUs x 8 waves
    int rpw = (n + target_waves - 1) / target_waves;
    if (rpw < 2) rpw = 2;
    return (rpw + 1) & ~1;
}

template <int EPI>
inline int launch_gemv(const int8_t* x, const int8_t* w, int32_t* acc, const float* s_x, const float* w_s,
                       const float* residual, float* y, int k, int n, hipStream_t st) {
    const int nch = (k / 16 + 63) / 64;
    const int rpw = pick_rows_per_wave(k, n);
    const int waves = (n + rpw - 1) / rpw;
    const int grid = (waves + kGemvWaves - 1) / kGemvWaves;
#define FX_GEMV_CASE(NCH, U)                                                                                     \
    gemv_i8_kernel<NCH, U, EPI><<<grid, kGemvBlock, 0, st>>>(x, w, acc, s_x, w_s, residual, y, k, n, rpw)
    if (nch <= 1) FX_GEMV_CASE(1, 4);
    else if (nch <= 2) FX_GEMV_CASE(2, 4);
    else if (nch <= 4) FX_GEMV_CASE(4, 2);
    else if (nch <= 8) FX_GEMV_CASE(8, 2);
    else FX_GEMV_CASE(16, 2);
#undef FX_GEMV_CASE
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

inline int launch_gemv_f32(const float* x, const int8_t* w, const float* w_s, const float* residual, float* y, float* s_x_out,
                           int8_t* q_out, int k, int n, hipStream_t st) {
    const int nch = (k / 16 + 63) / 64;
    const int rpw = pick_rows_per_wave(k, n);
    const int waves = (n + rpw - 1) / rpw;
    const int grid = (waves + kGemvWaves - 1) / kGemvWaves;
    if (nch <= 1) gemv_f32_i8_kernel<1, 4><<<grid, kGemvBlock, 0, st>>>(x, w, w_s, residual, y, s_x_out, q_out, k, n, rpw);
    else if (nch <= 2) gemv_f32_i8_kernel<2, 4><<<grid, kGemvBlock, 0, st>>>(x, w, w_s, residual, y, s_x_out, q_out, k, n, rpw);
    else gemv_f32_i8_kernel<4, 2><<<grid, kGemvBlock, 0, st>>>(x, w, w_s, residual, y, s_x_out, q_out, k, n, rpw);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx
