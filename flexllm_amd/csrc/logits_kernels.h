// Greedy head: fp16 embedding lookup, tied fp16 lm_head GEMV (fp32 accumulate), argmax.
#pragma once
#include "common.h"
#include <hip/hip_fp16.h>

namespace fx {

using h16x8 = _Float16 __attribute__((ext_vector_type(8)));

static __global__ __launch_bounds__(256) void embed_kernel(const __half* __restrict__ table, const int* __restrict__ token,
                                                    float* __restrict__ y, int hidden) {
    const size_t base = (size_t)token[0] * hidden;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < hidden; i += gridDim.x * 256) y[i] = __half2float(table[base + i]);
}

// One wave per run of rows; lane reads 16-byte chunks (8 halves) lane, lane+64, ... of the row.
template <int NCH>
__global__ __launch_bounds__(256) void lm_head_kernel(const __half* __restrict__ table, const float* __restrict__ n,
                                                      float* __restrict__ logits, int vocab, int hidden, int rows_per_wave) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int row0 = gw * rows_per_wave;
    if (row0 >= vocab) return;
    const int nrows = min(rows_per_wave, vocab - row0);
    const int nchunks = hidden >> 3;
    float nv[NCH][8];
#pragma unroll
    for (int i = 0; i < NCH; i++) {
        const int c = lane + 64 * i;
#pragma unroll
        for (int e = 0; e < 8; e++) nv[i][e] = c < nchunks ? n[c * 8 + e] : 0.0f;
    }
    for (int r = 0; r < nrows; r++) {
        const h16x8* wr = reinterpret_cast<const h16x8*>(table + (size_t)(row0 + r) * hidden);
        h16x8 wv[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const int c = lane + 64 * i;
            wv[i] = c < nchunks ? __builtin_nontemporal_load(wr + c) : h16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < NCH; i++)
#pragma unroll
            for (int e = 0; e < 8; e++) acc += (float)wv[i][e] * nv[i][e];
        acc = wave_sum(acc);
        if (lane == 0) logits[row0 + r] = acc;
    }
}

// two-stage argmax, lowest index wins ties
static __global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ x, int n, float* __restrict__ pv,
                                                             int* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ int si[4];
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n; i += gridDim.x * 256) {
        const float v = x[i];
        if (v > best || (v == best && i < bi)) { best = v; bi = i; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float ov = __shfl_xor(best, m);
        const int oi = __shfl_xor(bi, m);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++)
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
        pv[blockIdx.x] = best;
        pi[blockIdx.x] = bi;
    }
}
static __global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                                          int nparts, int* __restrict__ result) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < nparts; i += 64) {
        const float v = pv[i];
        const int idx = pi[i];
        if (v > best || (v == best && idx < bi)) { best = v; bi = idx; }
    }
#pragma unroll
    for (int m = 1; m < 64; m <<= 1) {
        const float ov = __shfl_xor(best, m);
        const int oi = __shfl_xor(bi, m);
        if (ov > best || (ov == best && oi < bi)) { best = ov; bi = oi; }
    }
    if (threadIdx.x == 0) result[0] = bi == 0x7fffffff ? 0 : bi;
}

constexpr int kArgmaxParts = 256;
inline float* g_pv = nullptr;
inline int* g_pi = nullptr;

inline int argmax_launch(const float* x, int n, int* result, float* pv, int* pi, hipStream_t st) {
    argmax_partial_kernel<<<kArgmaxParts, 256, 0, st>>>(x, n, pv, pi);
    argmax_final_kernel<<<1, 64, 0, st>>>(pv, pi, kArgmaxParts, result);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

inline int lm_head_launch(const uint16_t* embed, const float* n, float* logits, int vocab, int hidden, hipStream_t st) {
    const int nch = (hidden / 8 + 63) / 64;
    const int rpw = 16;
    const int waves = (vocab + rpw - 1) / rpw;
    const int grid = (waves + 3) / 4;
    const __half* t = reinterpret_cast<const __half*>(embed);
    if (nch <= 1) lm_head_kernel<1><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else if (nch <= 2) lm_head_kernel<2><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else if (nch <= 4) lm_head_kernel<4><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    else lm_head_kernel<8><<<grid, 256, 0, st>>>(t, n, logits, vocab, hidden, rpw);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx
