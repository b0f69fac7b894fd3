// Measurement probes: what this GPU sustains on the two resources the rooflines are priced against, measured with
// the library's own kernels so that a benchmark can print "published peak" and "measured peak" side by side.
// They compute nothing a caller needs; they have no counterpart in the reference.
#include "common.h"

namespace fx {

// Matrix cores alone: every wave keeps a 4x4 grid of 32x32 int32 accumulator tiles and issues
// v_mfma_i32_32x32x32_i8 back to back, 16 per step.  FROM_LDS re-reads the eight operand fragments from LDS at every
// step (eight 16-byte reads per lane for sixteen matrix instructions: the ratio of a 128x128 wave tile), so the LDS
// pipe runs as it does in a GEMM; otherwise the fragments stay in registers.  The operands are pseudo-random bytes
// or zeros: the rate with zeros is higher because the chip draws less power and clocks higher.
// clocks[0] / clocks[1] = shader-clock cycles / 100 MHz wall-clock ticks that workgroup 0's first wave spent in the
// loop: the shader clock under this load.
template <bool FROM_LDS>
__global__ __launch_bounds__(256) void probe_mfma_i8_kernel(int* __restrict__ sink, unsigned long long* __restrict__ clocks,
                                                            int iters, int random_operands, unsigned seed) {
    __shared__ __attribute__((aligned(16))) int8_t lds[64 * 1024];
    i32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;
    unsigned x = seed * 2654435761u + threadIdx.x * 40503u + blockIdx.x;
    for (int i = threadIdx.x; i < 16 * 1024; i += 256) {
        x = x * 1664525u + 1013904223u;
        reinterpret_cast<unsigned*>(lds)[i] = random_operands ? x : 0u;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const i32x4* frag = reinterpret_cast<const i32x4*>(lds);
    i32x4 fa[4], fb[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { fa[i] = frag[lane + 64 * i]; fb[i] = frag[lane + 64 * (i + 4)]; }
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
        if constexpr (FROM_LDS) {
            const int base = (it & 7) * 512;
#pragma unroll
            for (int i = 0; i < 4; i++) { fa[i] = frag[base + lane + 64 * i]; fb[i] = frag[base + lane + 64 * (i + 4)]; }
        }
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    int s = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) s += acc[i][j][r];
    sink[blockIdx.x * 256 + threadIdx.x] = s;
    if (clocks && blockIdx.x == 0 && threadIdx.x == 0) { clocks[0] = c1 - c0; clocks[1] = w1 - w0; }
}

// HBM read stream: a workgroup reads contiguous blocks of 32 KiB (eight 16-byte loads in flight per thread, a wave's
// load covers 1 KiB of contiguous memory), blocks dealt to the workgroups round-robin; every word is folded into one
// word per wave.  Read-only traffic of `n16` 16-byte words, nothing else.
template <bool NT>
__global__ __launch_bounds__(256) void probe_hbm_read_kernel(const i32x4* __restrict__ src, size_t n16, unsigned* __restrict__ sink) {
    constexpr size_t kBlock16 = 8 * 256;                     // 16-byte words per block
    unsigned acc = 0;
    const size_t n_blocks = n16 / kBlock16;
    for (size_t b = blockIdx.x; b < n_blocks; b += gridDim.x) {
        const i32x4* p = src + b * kBlock16 + threadIdx.x;
        i32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = NT ? __builtin_nontemporal_load(p + u * 256) : p[u * 256];
#pragma unroll
        for (int u = 0; u < 8; u++) acc ^= (unsigned)(v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3]);
    }
    for (size_t i = n_blocks * kBlock16 + (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) {
        const i32x4 a = src[i];
        acc ^= (unsigned)(a[0] ^ a[1] ^ a[2] ^ a[3]);
    }
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) acc ^= (unsigned)__shfl_xor((int)acc, m);
    if ((threadIdx.x & 63) == 0) sink[blockIdx.x * 4 + (threadIdx.x >> 6)] = acc;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_probe_mfma_i8(int iters, int random_operands, int from_lds, int workgroups, int* sink, unsigned long long* clocks,
                          void* stream) {
    FX_REQUIRE(sink && iters > 0 && workgroups > 0 && workgroups <= 65536, "probe_mfma_i8: iters=%d workgroups=%d", iters, workgroups);
    if (from_lds)
        probe_mfma_i8_kernel<true><<<workgroups, 256, 0, as_stream(stream)>>>(sink, clocks, iters, random_operands, 1u);
    else
        probe_mfma_i8_kernel<false><<<workgroups, 256, 0, as_stream(stream)>>>(sink, clocks, iters, random_operands, 1u);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_probe_hbm_read(const void* src, size_t bytes, int workgroups, int non_temporal, unsigned* sink, void* stream) {
    FX_REQUIRE(src && sink && bytes % 16 == 0 && workgroups > 0 && workgroups <= 65536, "probe_hbm_read: bytes=%zu workgroups=%d", bytes, workgroups);
    FX_REQUIRE((reinterpret_cast<uintptr_t>(src) & 15) == 0, "probe_hbm_read: src must be 16-byte aligned");
    if (non_temporal)
        probe_hbm_read_kernel<true><<<workgroups, 256, 0, as_stream(stream)>>>(static_cast<const i32x4*>(src), bytes / 16, sink);
    else
        probe_hbm_read_kernel<false><<<workgroups, 256, 0, as_stream(stream)>>>(static_cast<const i32x4*>(src), bytes / 16, sink);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"
