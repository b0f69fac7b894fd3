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

}  // namespace fx
