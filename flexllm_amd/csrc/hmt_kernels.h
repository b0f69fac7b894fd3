// Kernels of the HMT long-context plug-in (hierarchical memory on top of the prefill graph): everything here is
// fp32 and small next to the layer stack - a 2048 x 2048 fp32 GEMV, 64 dot products, a softmax over the memory
// slots, a weighted sum of the memories, and the row gather that assembles a stage's input sequence.
#pragma once
#include "common.h"

namespace fx {

// y[n] = sum_k w[n][k] * x[k], fp32.  One wave per output row, 16-byte loads, lanes keep four partial sums by
// k % 4 like the reference's PE and a wave-wide tree joins them: same value as the reference's sequential
// accumulation up to fp32 association (parity is a tolerance, not bit-exactness, for this stage).
static __global__ __launch_bounds__(256) void linear_f32_gemv_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                                 float* __restrict__ y, int k, int n) {
    const int lane = threadIdx.x & 63;
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= n) return;
    const float4* wr = reinterpret_cast<const float4*>(w + (size_t)row * k);
    const float4* xv = reinterpret_cast<const float4*>(x);
    float p0 = 0.0f, p1 = 0.0f, p2 = 0.0f, p3 = 0.0f;
    for (int i = lane; i < (k >> 2); i += 64) {
        const float4 a = xv[i], b = wr[i];
        p0 += a.x * b.x; p1 += a.y * b.y; p2 += a.z * b.z; p3 += a.w * b.w;
    }
    const float s = wave_sum((p0 + p1) + (p2 + p3));
    if (lane == 0) y[row] = s;
}

constexpr int kHmtMaxSlots = 1024;

// One workgroup: scores a[j] = q . kmem[j] for every slot (empty slots hold zeros and take part, as in the
// reference), then softmax((a - max) / scale) over the slots.
static __global__ __launch_bounds__(1024) void hmt_scores_softmax_kernel(const float* __restrict__ q, const float* __restrict__ kmem,
                                                                     float* __restrict__ a_sft, int mem_num, int hidden, float scale) {
    __shared__ float sc[kHmtMaxSlots];
    __shared__ float red[16];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const float4* qv = reinterpret_cast<const float4*>(q);
    for (int j = wave; j < mem_num; j += 16) {
        const float4* kr = reinterpret_cast<const float4*>(kmem + (size_t)j * hidden);
        float p0 = 0.0f, p1 = 0.0f, p2 = 0.0f, p3 = 0.0f;
        for (int i = lane; i < (hidden >> 2); i += 64) {
            const float4 a = qv[i], b = kr[i];
            p0 += a.x * b.x; p1 += a.y * b.y; p2 += a.z * b.z; p3 += a.w * b.w;
        }
        const float s = wave_sum((p0 + p1) + (p2 + p3));
        if (lane == 0) sc[j] = s;
    }
    __syncthreads();
    float mx = -1e32f;
    for (int j = t; j < mem_num; j += 1024) mx = fmaxf(mx, sc[j]);
    mx = block_max<16>(mx, red);
    float e = 0.0f, sum = 0.0f;
    if (t < mem_num) { e = expf((sc[t] - mx) / scale); sum = e; }      // mem_num <= 1024: one slot per thread
    sum = block_sum<16>(sum, red);
    if (t < mem_num) a_sft[t] = e * (1.0f / sum);
}

// p[c] = sum_j a[j] * mmem[j][c]: one thread per channel, slots in order with four partial sums by j % 4.
static __global__ __launch_bounds__(256) void hmt_weighted_sum_kernel(const float* __restrict__ a_sft, const float* __restrict__ mmem,
                                                                  float* __restrict__ p_out, int mem_num, int hidden) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= hidden) return;
    float p[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    int j = 0;
    for (; j + 8 <= mem_num; j += 8) {                       // eight loads in flight, summed in slot order
        float m[8];
#pragma unroll
        for (int u = 0; u < 8; u++) m[u] = mmem[(size_t)(j + u) * hidden + c];
#pragma unroll
        for (int u = 0; u < 8; u++) p[u & 3] += a_sft[j + u] * m[u];
    }
    for (; j < mem_num; j++) p[j & 3] += a_sft[j] * mmem[(size_t)j * hidden + c];
    p_out[c] = (p[0] + p[1]) + (p[2] + p[3]);
}

// Input sequence of one stage, row by row (grid.x = rows, float4 per thread):
//   stage 0: [T, emb[off .. off+cur_sum), T, 0...]                              (summary prompt around the segment's head)
//   stage 1: [P, emb[off-rec .. off) (zeros before the text), emb[off .. off+cur), P if tail_p, 0...]
static __global__ __launch_bounds__(256) void hmt_stage_input_kernel(const float* __restrict__ emb, const float* __restrict__ t_embed,
                                                                 const float* __restrict__ p_buf, float* __restrict__ x_out, int stage,
                                                                 int off, int cur, int cur_sum, int rec, int tail_p, int hidden) {
    const int row = blockIdx.x;
    const float* src = nullptr;
    if (stage == 0) {
        if (row == 0 || row == 1 + cur_sum) src = t_embed;
        else if (row <= cur_sum) src = emb + (size_t)(off + row - 1) * hidden;
    } else {
        const int tok = row - 1 - rec;                        // position relative to the segment start
        if (row == 0 || (tok == cur && tail_p)) src = p_buf;
        else if (tok < cur && off + tok >= 0) src = emb + (size_t)(off + tok) * hidden;
    }
    float4* dst = reinterpret_cast<float4*>(x_out + (size_t)row * hidden);
    for (int i = threadIdx.x; i < (hidden >> 2); i += 256)
        dst[i] = src ? reinterpret_cast<const float4*>(src)[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
}

}  // namespace fx
