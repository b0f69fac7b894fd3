// int8 x int8 -> int32 GEMM for prefill on gfx950 matrix cores: C[m][n] = sum_k A[m][k]*W[n][k].
//
// Both operands are K-contiguous, which is exactly the per-lane operand shape of
// v_mfma_i32_32x32x32_i8 (lane l supplies 16 consecutive k-bytes of row/column l%32, k-group l/32), so
// tiles go global -> registers -> LDS (16-byte chunks, k-chunk-major planes) -> MFMA operands with plain
// 128-bit reads and no transposition.  Integer accumulation: exact in any order.
//
// Workgroup tile BM x BN x 64, 256 threads = 4 waves in a 2x2 grid, each wave (BM/2)x(BN/2) as 32x32 MFMA
// tiles, double-buffered LDS, four k-steps of global loads in flight in registers.
#pragma once
#include "common.h"
#include <stdlib.h>

namespace fx {

constexpr int kGemmBK = 64;        // k-bytes per stage
// LDS tile layout: [16-byte k-chunk (4 per stage)][row][16 B], i.e. for one k-chunk the rows are contiguous.
// A wave-wide 128-bit fragment read then touches two contiguous 512-byte runs; the +32 B on the plane pitch
// spreads the four chunks of one row, written by four neighbouring lanes, over all banks.
__host__ __device__ constexpr int gemm_plane(int rows) { return rows * 16 + 32; }

enum GemmEpi { kGemmRaw = 0, kGemmDequant = 1 };

template <int BM, int BN, int EPI, int D>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ w,
                                                      int32_t* __restrict__ c_out, const float* __restrict__ s_x,
                                                      const float* __restrict__ w_s, const float* __restrict__ residual,
                                                      float* __restrict__ y, int m, int k, int n, int tiles_m, int tiles_n) {
    constexpr int WM = BM / 2, WN = BN / 2;          // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 4 / 256;           // 16-byte chunks per thread per stage
    constexpr int B_CHUNKS = BN * 4 / 256;
    constexpr int PA = gemm_plane(BM), PB = gemm_plane(BN);
    __shared__ __attribute__((aligned(16))) int8_t lds_a[2][4 * PA];
    __shared__ __attribute__((aligned(16))) int8_t lds_b[2][4 * PB];

    // XCD-aware tile order.  Consecutive workgroup ids land on different XCDs (8 of them, each with its own
    // 4 MiB L2).  Give every XCD a contiguous range of weight columns and walk the token-row tiles fastest,
    // so that a weight block is fetched from HBM by one XCD only and is shared there by all token-row tiles
    // (the activations, M x K, are small and are read by every XCD).
    int tm, tn;
    if ((tiles_n & 7) == 0) {
        const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
        tn = xcd * (tiles_n >> 3) + idx / tiles_m;
        tm = idx % tiles_m;
    } else {
        tm = blockIdx.x / tiles_n;
        tn = blockIdx.x % tiles_n;
    }
    const int row0 = tm * BM, col0 = tn * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // global -> register staging: chunk id c = t + 256*i -> row c/4, 16-byte column c%4.  D k-steps of global
    // loads are kept in flight in registers (an L2/HBM round trip is several k-steps long).
    i32x4 ra[D][A_CHUNKS], rb[D][B_CHUNKS];
    const int8_t* a_ptr[A_CHUNKS];
    const int8_t* b_ptr[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) {
        const int c = t + 256 * i;
        a_ptr[i] = a + (size_t)min(row0 + (c >> 2), m - 1) * k + (c & 3) * 16;
    }
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
        const int c = t + 256 * i;
        b_ptr[i] = w + (size_t)min(col0 + (c >> 2), n - 1) * k + (c & 3) * 16;
    }
    auto load_global = [&](int k0, i32x4 (&xa)[A_CHUNKS], i32x4 (&xb)[B_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) xa[i] = *reinterpret_cast<const i32x4*>(a_ptr[i] + k0);
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) xb[i] = *reinterpret_cast<const i32x4*>(b_ptr[i] + k0);
    };
    auto store_lds = [&](int buf, const i32x4 (&xa)[A_CHUNKS], const i32x4 (&xb)[B_CHUNKS]) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_a[buf][(c & 3) * PA + (c >> 2) * 16]) = xa[i];
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_b[buf][(c & 3) * PB + (c >> 2) * 16]) = xb[i];
        }
    };

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int nk = k / kGemmBK;            // a multiple of D (checked by the launcher)
#pragma unroll
    for (int d = 0; d < D; d++)
        if (d < nk) load_global(d * kGemmBK, ra[d], rb[d]);
    store_lds(0, ra[0], rb[0]);
    __syncthreads();
    const int frag_row = (lane & 31) * 16, frag_g = lane >> 5;
    for (int kt0 = 0; kt0 < nk; kt0 += D) {
#pragma unroll
        for (int d = 0; d < D; d++) {
            const int kt = kt0 + d;
            const int buf = kt & 1;
            // slot d held k-step kt, which is already in LDS: refill it with k-step kt+D
            if (kt + D < nk) load_global((kt + D) * kGemmBK, ra[d], rb[d]);
#pragma unroll
            for (int ks = 0; ks < kGemmBK / 32; ks++) {
                i32x4 fa[TM], fb[TN];
#pragma unroll
                for (int i = 0; i < TM; i++)
                    fa[i] = *reinterpret_cast<const i32x4*>(&lds_a[buf][(ks * 2 + frag_g) * PA + (wm + i * 32) * 16 + frag_row]);
#pragma unroll
                for (int j = 0; j < TN; j++)
                    fb[j] = *reinterpret_cast<const i32x4*>(&lds_b[buf][(ks * 2 + frag_g) * PB + (wn + j * 32) * 16 + frag_row]);
#pragma unroll
                for (int i = 0; i < TM; i++)
#pragma unroll
                    for (int j = 0; j < TN; j++)
                        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
            if (kt + 1 < nk) {
                store_lds(buf ^ 1, ra[(d + 1) % D], rb[(d + 1) % D]);   // the other buffer was last read before the previous barrier
                __syncthreads();
            }
        }
    }

    // epilogue: 32x32 accumulator layout - lane l holds column l%32, register r holds row 8*(r/4) + 4*(l/32) + r%4
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
            const int col = col0 + wn + j * 32 + (lane & 31);
            if (col >= n) continue;
            float ws = 0.0f;
            if constexpr (EPI == kGemmDequant) ws = w_s[col];
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const int row = row0 + wm + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (row >= m) continue;
                if constexpr (EPI == kGemmDequant) {
                    float v = (float)acc[i][j][r] * s_x[row] * ws;
                    if (residual) v = v + residual[(size_t)row * n + col];
                    y[(size_t)row * n + col] = v;
                } else {
                    c_out[(size_t)row * n + col] = acc[i][j][r];
                }
            }
        }
}

template <int EPI>
inline int launch_gemm(const int8_t* a, const int8_t* w, int32_t* c, const float* s_x, const float* w_s,
                       const float* residual, float* y, int m, int k, int n, hipStream_t st) {
    // Measured on MI355X at M=1024: 128x128 tiles win once there are >= 4 workgroups per CU (gate/up), 64x64
    // tiles win for the narrow projections (more workgroups hide the per-k-step barrier better).
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    static const char* force = getenv("FLEXLLM_GEMM_TILE");
    int mode = tiles(128, 128) >= 1024 ? 0 : 2;
    if (force) mode = atoi(force);
    const int nk = k / kGemmBK;
#define FX_GEMM_LAUNCH(BM, BN, DD)                                                                                \
    do {                                                                                                          \
        const int tm = (m + BM - 1) / BM, tn = (n + BN - 1) / BN;                                                 \
        gemm_i8_kernel<BM, BN, EPI, DD><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn); \
    } while (0)
    const bool deep = nk % 4 == 0;      // prefetch depth 4 needs the k-steps in groups of 4 (K % 256 == 0)
    if (mode == 0) { if (deep) FX_GEMM_LAUNCH(128, 128, 4); else FX_GEMM_LAUNCH(128, 128, 1); }
    else if (mode == 1) { if (deep) FX_GEMM_LAUNCH(64, 128, 4); else FX_GEMM_LAUNCH(64, 128, 1); }
    else { if (deep) FX_GEMM_LAUNCH(64, 64, 4); else FX_GEMM_LAUNCH(64, 64, 1); }
#undef FX_GEMM_LAUNCH
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx
