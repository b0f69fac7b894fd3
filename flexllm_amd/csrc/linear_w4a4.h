// W4A4 linear layers: activations asymmetric uint4 (value 0..15, scale s_x, zero point b_x = row minimum),
// weights symmetric int4 (-8..7), both packed two per byte along K: byte j of a row holds element 2j in its low
// nibble and element 2j+1 in its high nibble.  y[n] = (float(acc[n]) * s_x) * w_s[n] + b_x * w_sum[n], where
// acc = sum_k a[k]*w[n][k] and w_sum[n] is the sum of the dequantised weights of row n (supplied by the caller).
//
// Decode: the GEMV streams the packed weights once (half the bytes of the int8 path) and multiplies with
// v_dot8_i32_i4, which is signed x signed.  The unsigned activation a is fed as a-8 (one XOR with 8 per nibble)
// and 8*rowsum(w) is added back; the row sum comes from a second dot8 with all-ones, exact in int32.
#pragma once
#include "gemv_i8.h"

namespace fx {

__device__ __forceinline__ int dot32_i4(const i32x4& w, const i32x4& xs, int acc) {
    acc = __builtin_amdgcn_sdot8(w.x, xs.x, acc, false);
    acc = __builtin_amdgcn_sdot8(w.y, xs.y, acc, false);
    acc = __builtin_amdgcn_sdot8(w.z, xs.z, acc, false);
    acc = __builtin_amdgcn_sdot8(w.w, xs.w, acc, false);
    return acc;
}

enum Gemv4Epi { kEpi4Raw = 0, kEpi4Dequant = 1 };

// Same schedule as gemv_i8_kernel: a wave owns rows_per_wave consecutive rows, lane l reads the 16-byte chunks
// l, l+64, ... of a packed row (32 weights each), U rows in flight.
template <int NCH, int U, int EPI>
__global__ __launch_bounds__(kGemvBlock) void gemv_u4i4_kernel(const uint8_t* __restrict__ x4, const uint8_t* __restrict__ w4,
                                                               int32_t* __restrict__ acc_out, const float* __restrict__ s_x,
                                                               const float* __restrict__ b_x, const float* __restrict__ w_s,
                                                               const float* __restrict__ w_sum,
                                                               const float* __restrict__ residual, float* __restrict__ y,
                                                               int k, int n, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * kGemvWaves + (threadIdx.x >> 6);
    const int row0 = gw * rows_per_wave;
    if (row0 >= n) return;
    const int nrows = min(rows_per_wave, n - row0);
    const int row_bytes = k >> 1, nchunks = row_bytes >> 4;
    i32x4 xs[NCH];                                   // activations as signed nibbles a-8
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + 64 * i;
        i32x4 v = c < nchunks ? reinterpret_cast<const i32x4*>(x4)[c] : i32x4{(int)0x88888888, (int)0x88888888, (int)0x88888888, (int)0x88888888};
        v.x ^= 0x88888888; v.y ^= 0x88888888; v.z ^= 0x88888888; v.w ^= 0x88888888;   // a -> a-8; padding -> 0
        xs[i] = v;
    }
    const i32x4 ones = {0x11111111, 0x11111111, 0x11111111, 0x11111111};
    float sx = 0.0f, bx = 0.0f;
    if constexpr (EPI == kEpi4Dequant) { sx = s_x[0]; bx = b_x[0]; }
    for (int r = 0; r < nrows; r += U) {
        i32x4 wv[U][NCH];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const int row = min(row0 + r + u, n - 1);
            const i32x4* wr = reinterpret_cast<const i32x4*>(w4 + (size_t)row * row_bytes);
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                const int c = lane + 64 * i;
                wv[u][i] = c < nchunks ? __builtin_nontemporal_load(wr + c) : i32x4{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int u = 0; u < U; u++) {
            int acc = 0, wsum = 0;
#pragma unroll
            for (int i = 0; i < NCH; i++) { acc = dot32_i4(wv[u][i], xs[i], acc); wsum = dot32_i4(wv[u][i], ones, wsum); }
            acc = wave_sum_i(acc + 8 * wsum);
            const int row = row0 + r + u;
            if (lane == 0 && r + u < nrows) {
                if constexpr (EPI == kEpi4Dequant) {
                    float v = (float)acc * sx * w_s[row];
                    v = v + bx * w_sum[row];
                    if (residual) v = v + residual[row];
                    y[row] = v;
                } else {
                    acc_out[row] = acc;
                }
            }
        }
    }
}

template <int EPI>
inline int launch_gemv_u4i4(const uint8_t* x4, const uint8_t* w4, int32_t* acc, const float* s_x, const float* b_x,
                            const float* w_s, const float* w_sum, const float* residual, float* y, int k, int n, hipStream_t st) {
    const int nch = (k / 32 + 63) / 64;
    const int rpw = pick_rows_per_wave(k / 2, n);
    const int waves = (n + rpw - 1) / rpw;
    const int grid = (waves + kGemvWaves - 1) / kGemvWaves;
#define FX_GEMV4_CASE(NCH, U)                                                                                              \
    gemv_u4i4_kernel<NCH, U, EPI><<<grid, kGemvBlock, 0, st>>>(x4, w4, acc, s_x, b_x, w_s, w_sum, residual, y, k, n, rpw)
    if (nch <= 1) FX_GEMV4_CASE(1, 4);
    else if (nch <= 2) FX_GEMV4_CASE(2, 4);
    else if (nch <= 4) FX_GEMV4_CASE(4, 2);
    else FX_GEMV4_CASE(8, 2);
#undef FX_GEMV4_CASE
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

// values one per byte (low 4 bits used) -> two per byte, low nibble = even index
static __global__ __launch_bounds__(256) void pack_nibbles_kernel(const uint8_t* __restrict__ in, uint8_t* __restrict__ out, size_t n_out) {
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n_out; i += (size_t)gridDim.x * 256)
        out[i] = (uint8_t)((in[2 * i] & 0xF) | ((in[2 * i + 1] & 0xF) << 4));
}

// counts the bytes of `in` that are not 4-bit two's-complement values (-8..7) held one per byte
static __global__ __launch_bounds__(256) void nibble_range_kernel(const int8_t* __restrict__ in, size_t n, unsigned* __restrict__ bad) {
    unsigned c = 0;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) c += in[i] < -8 || in[i] > 7;
    if (c) atomicAdd(bad, c);
}

}  // namespace fx
