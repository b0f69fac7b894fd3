// int8 x int8 -> int32 GEMM for prefill on gfx950 matrix cores: C[m][n] = sum_k A[m][k]*W[n][k].
//
// Both operands are K-contiguous, which is exactly the per-lane operand shape of
// v_mfma_i32_32x32x32_i8 (lane l supplies 16 consecutive k-bytes of row/column l%32, k-group l/32), so
// tiles go global -> registers -> LDS (16-byte chunks, rows padded to 80 B to spread LDS banks) -> MFMA
// operands with plain 128-bit reads and no transposition.  Integer accumulation: exact in any order.
//
// Workgroup tile BM x BN x 64, 256 threads = 4 waves in a 2x2 grid, each wave (BM/2)x(BN/2) as 32x32 MFMA
// tiles, double-buffered LDS, next tile's global loads in flight during the current tile's MFMAs.
#pragma once
#include "common.h"

namespace fx {

constexpr int kGemmBK = 64;        // k-bytes per stage
constexpr int kGemmLdsRow = 80;    // padded LDS row pitch in bytes

enum GemmEpi { kGemmRaw = 0, kGemmDequant = 1 };

template <int BM, int BN, int EPI>
__global__ __launch_bounds__(256) void gemm_i8_kernel(const int8_t* __restrict__ a, const int8_t* __restrict__ w,
                                                      int32_t* __restrict__ c_out, const float* __restrict__ s_x,
                                                      const float* __restrict__ w_s, const float* __restrict__ residual,
                                                      float* __restrict__ y, int m, int k, int n, int tiles_m, int tiles_n) {
    constexpr int WM = BM / 2, WN = BN / 2;          // wave tile
    constexpr int TM = WM / 32, TN = WN / 32;        // 32x32 MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 4 / 256;           // 16-byte chunks per thread per stage
    constexpr int B_CHUNKS = BN * 4 / 256;
    __shared__ __attribute__((aligned(16))) int8_t lds_a[2][BM * kGemmLdsRow];
    __shared__ __attribute__((aligned(16))) int8_t lds_b[2][BN * kGemmLdsRow];

    // XCD-aware tile order: consecutive workgroup ids land on different XCDs (8 of them, each with its own
    // L2); give every XCD a contiguous run of tiles so that neighbours share A row-blocks in one L2.
    const int ntiles = tiles_m * tiles_n;
    int tile = blockIdx.x;
    if ((ntiles & 7) == 0) tile = (blockIdx.x & 7) * (ntiles >> 3) + (blockIdx.x >> 3);
    const int tm = tile / tiles_n, tn = tile % tiles_n;
    const int row0 = tm * BM, col0 = tn * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = (wave >> 1) * WM, wn = (wave & 1) * WN;

    // global -> register staging: chunk id c = t + 256*i -> row c/4, 16-byte column c%4
    i32x4 ra[A_CHUNKS], rb[B_CHUNKS];
    auto load_global = [&](int k0) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int c = t + 256 * i;
            const int r = min(row0 + (c >> 2), m - 1);
            ra[i] = *reinterpret_cast<const i32x4*>(a + (size_t)r * k + k0 + (c & 3) * 16);
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int c = t + 256 * i;
            const int r = min(col0 + (c >> 2), n - 1);
            rb[i] = *reinterpret_cast<const i32x4*>(w + (size_t)r * k + k0 + (c & 3) * 16);
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_a[buf][(c >> 2) * kGemmLdsRow + (c & 3) * 16]) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_CHUNKS; i++) {
            const int c = t + 256 * i;
            *reinterpret_cast<i32x4*>(&lds_b[buf][(c >> 2) * kGemmLdsRow + (c & 3) * 16]) = rb[i];
        }
    };

    i32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0;

    const int nk = k / kGemmBK;
    load_global(0);
    store_lds(0);
    __syncthreads();
    const int frag_off = (lane & 31) * kGemmLdsRow + (lane >> 5) * 16;
    for (int kt = 0; kt < nk; kt++) {
        const int buf = kt & 1;
        if (kt + 1 < nk) load_global((kt + 1) * kGemmBK);
#pragma unroll
        for (int ks = 0; ks < kGemmBK / 32; ks++) {
            i32x4 fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; i++)
                fa[i] = *reinterpret_cast<const i32x4*>(&lds_a[buf][(wm + i * 32) * kGemmLdsRow + frag_off + ks * 32]);
#pragma unroll
            for (int j = 0; j < TN; j++)
                fb[j] = *reinterpret_cast<const i32x4*>(&lds_b[buf][(wn + j * 32) * kGemmLdsRow + frag_off + ks * 32]);
#pragma unroll
            for (int i = 0; i < TM; i++)
#pragma unroll
                for (int j = 0; j < TN; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < nk) {
            store_lds(buf ^ 1);      // the other buffer was last read before the previous barrier
            __syncthreads();
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
    // 128x128 tiles when they fill the chip (>= 256 workgroups), otherwise 64x128 / 64x64 for more workgroups
    auto tiles = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    if (tiles(128, 128) >= 512) {
        const int tm = (m + 127) / 128, tn = (n + 127) / 128;
        gemm_i8_kernel<128, 128, EPI><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn);
    } else if (tiles(64, 128) >= 256) {
        const int tm = (m + 63) / 64, tn = (n + 127) / 128;
        gemm_i8_kernel<64, 128, EPI><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn);
    } else {
        const int tm = (m + 63) / 64, tn = (n + 63) / 64;
        gemm_i8_kernel<64, 64, EPI><<<tm * tn, 256, 0, st>>>(a, w, c, s_x, w_s, residual, y, m, k, n, tm, tn);
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx
