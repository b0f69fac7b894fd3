// Decode linear layers: C ABI entry points of the int8 GEMV (kernels in gemv_i8.h).
#include "gemv_i8.h"


namespace fx {

// Unsigned 8-bit activations times signed int8 weights (the reference's is_uint_input / is_uint_A instantiation of its
// int8 PEs, used for the uint8 softmax probabilities): acc[m][n] = sum_k a[m][k] * w[n][k], a in 0..255.  gfx950's
// byte dot product is signed x signed, so (a - 128) . w + 128 * sum(w) is evaluated, both exact in int32.
// One wave per output element row-chunk: grid (ceil(n / 4), m), 4 waves per block, wave -> one column n.
static __global__ __launch_bounds__(256) void linear_u8i8_kernel(const uint8_t* __restrict__ a, const int8_t* __restrict__ w,
                                                                 int32_t* __restrict__ acc, int k, int n) {
    const int lane = threadIdx.x & 63, col = blockIdx.x * 4 + (threadIdx.x >> 6), row = blockIdx.y;
    if (col >= n) return;
    const i32x4* ar = reinterpret_cast<const i32x4*>(a + (size_t)row * k);
    const i32x4* wr = reinterpret_cast<const i32x4*>(w + (size_t)col * k);
    const i32x4 ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
    int dot = 0, wsum = 0;
    for (int c = lane; c < k / 16; c += 64) {
        i32x4 av = ar[c];
        const i32x4 wv = wr[c];
        av.x ^= 0x80808080; av.y ^= 0x80808080; av.z ^= 0x80808080; av.w ^= 0x80808080;     // a - 128 as signed bytes
        dot = dot16(av, wv, dot);
        wsum = dot16(ones, wv, wsum);
    }
    dot = wave_sum_i(dot + 128 * wsum);
    if (lane == 0) acc[(size_t)row * n + col] = dot;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_linear_u8i8_gemm(const uint8_t* a, const int8_t* w, int32_t* acc, int m, int k, int n, void* stream) {
    FX_REQUIRE(a && w && acc, "linear_u8i8_gemm: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0, "linear_u8i8_gemm: k=%d must be a positive multiple of 16", k);
    FX_REQUIRE(m >= 0 && n >= 0 && m <= 65535, "linear_u8i8_gemm: m=%d n=%d (m <= 65535)", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    linear_u8i8_kernel<<<dim3((n + 3) / 4, m), 256, 0, as_stream(stream)>>>(a, w, acc, k, n);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_linear_i8_gemv(const int8_t* x, const int8_t* w, int32_t* acc, int k, int n, void* stream) {
    FX_REQUIRE(x && w && acc, "linear_i8_gemv: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<kEpiRaw>(x, w, acc, nullptr, nullptr, nullptr, nullptr, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemv_dequant(const int8_t* x, const float* s_x, const int8_t* w, const float* w_s,
                                   const float* residual, float* y, int k, int n, void* stream) {
    FX_REQUIRE(x && s_x && w && w_s && y, "linear_i8_gemv_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv_dequant: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv_dequant: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<kEpiDequant>(x, w, nullptr, s_x, w_s, residual, y, k, n, as_stream(stream));
}

int flexllm_quant_linear_i8_gemv_dequant(const float* x, const int8_t* w, const float* w_s, const float* residual, float* y,
                                         float* s_x_out, int8_t* q_out, int k, int n, void* stream) {
    FX_REQUIRE(x && w && w_s && y, "quant_linear_i8_gemv_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 4096, "quant_linear_i8_gemv_dequant: k=%d must be a multiple of 16, <= 4096", k);
    FX_REQUIRE(n >= 0, "quant_linear_i8_gemv_dequant: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv_f32(x, w, w_s, residual, y, s_x_out, q_out, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemv_swiglu(const int8_t* x, const float* s_x, const int8_t* w_gu, const float* w_s_gu, float* y,
                                  int k, int n, void* stream) {
    FX_REQUIRE(x && s_x && w_gu && w_s_gu && y, "linear_i8_gemv_swiglu: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv_swiglu: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv_swiglu: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<kEpiSwiglu>(x, w_gu, nullptr, s_x, w_s_gu, nullptr, y, k, 2 * n, as_stream(stream));
}

}  // extern "C"
