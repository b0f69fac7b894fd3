// Decode linear layers: int8 GEMV entry points (raw int32 accumulators, and fused dequant/residual).
#include "gemv_i8.h"

namespace fx {

constexpr int kGemvBlock = 256;
constexpr int kGemvWaves = kGemvBlock / kWave;

// rows_per_wave consecutive rows per wave; grid covers ceil(n / (4*rows_per_wave)) blocks.
template <int NCH, int U, bool DEQUANT>
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
    if constexpr (DEQUANT) {
        const float sx = s_x[0];
        wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0, nrows, lane, [&](int row, int sum) {
            if (lane == 0) {
                float v = (float)sum * sx * w_s[row];
                if (residual) v = v + residual[row];
                y[row] = v;
            }
        });
    } else {
        wave_gemv_rows<NCH, U>(w, xr, k, nchunks, row0, nrows, lane, [&](int row, int sum) {
            if (lane == 0) acc_out[row] = sum;
        });
    }
}

// Picks rows per wave so that the grid has at least ~4 waves per SIMD-quarter of the chip while each wave
// still streams several KiB.
static inline int pick_rows_per_wave(int k, int n) {
    const int target_waves = 256 * 8;  // 256 CUs x 8 waves
    int rpw = (n + target_waves - 1) / target_waves;
    const int min_rows = k >= 8192 ? 1 : k >= 4096 ? 2 : 2;
    if (rpw < min_rows) rpw = min_rows;
    return rpw;
}

template <bool DEQUANT>
static int launch_gemv(const int8_t* x, const int8_t* w, int32_t* acc, const float* s_x, const float* w_s,
                       const float* residual, float* y, int k, int n, hipStream_t st) {
    const int nch = (k / 16 + 63) / 64;
    const int rpw = pick_rows_per_wave(k, n);
    const int waves = (n + rpw - 1) / rpw;
    const int grid = (waves + kGemvWaves - 1) / kGemvWaves;
#define FX_GEMV_CASE(NCH, U)                                                                                     \
    gemv_i8_kernel<NCH, U, DEQUANT><<<grid, kGemvBlock, 0, st>>>(x, w, acc, s_x, w_s, residual, y, k, n, rpw)
    if (nch <= 1) FX_GEMV_CASE(1, 4);
    else if (nch <= 2) FX_GEMV_CASE(2, 4);
    else if (nch <= 4) FX_GEMV_CASE(4, 2);
    else if (nch <= 8) FX_GEMV_CASE(8, 2);
    else FX_GEMV_CASE(16, 1);
#undef FX_GEMV_CASE
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_linear_i8_gemv(const int8_t* x, const int8_t* w, int32_t* acc, int k, int n, void* stream) {
    FX_REQUIRE(x && w && acc, "linear_i8_gemv: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<false>(x, w, acc, nullptr, nullptr, nullptr, nullptr, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemv_dequant(const int8_t* x, const float* s_x, const int8_t* w, const float* w_s,
                                   const float* residual, float* y, int k, int n, void* stream) {
    FX_REQUIRE(x && s_x && w && w_s && y, "linear_i8_gemv_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv_dequant: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv_dequant: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<true>(x, w, nullptr, s_x, w_s, residual, y, k, n, as_stream(stream));
}

}  // extern "C"
