// W4A4 linear layers: C ABI entry points (kernels in linear_w4a4.h and gemm_i8.h).
#include "linear_w4a4.h"
#include "gemm_i8.h"

using namespace fx;

extern "C" {

int flexllm_pack_nibbles(const uint8_t* values, uint8_t* packed, size_t n_values, void* stream) {
    FX_REQUIRE(values && packed, "pack_nibbles: null pointer");
    FX_REQUIRE(n_values % 2 == 0, "pack_nibbles: n_values=%zu must be even", n_values);
    if (n_values == 0) return FLEXLLM_OK;
    const size_t n_out = n_values / 2;
    const int grid = (int)((n_out + 255) / 256 < 4096 ? (n_out + 255) / 256 : 4096);
    pack_nibbles_kernel<<<grid, 256, 0, as_stream(stream)>>>(values, packed, n_out);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_linear_u4i4_gemv(const uint8_t* x4, const uint8_t* w4, int32_t* acc, int k, int n, void* stream) {
    FX_REQUIRE(x4 && w4 && acc, "linear_u4i4_gemv: null pointer");
    FX_REQUIRE(k > 0 && k % 32 == 0 && k <= 16384, "linear_u4i4_gemv: k=%d must be a multiple of 32, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_u4i4_gemv: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv_u4i4<kEpi4Raw>(x4, w4, acc, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, k, n, as_stream(stream));
}

int flexllm_linear_u4i4_gemv_dequant(const uint8_t* x4, const float* s_x, const float* b_x, const uint8_t* w4,
                                     const float* w_s, const float* w_sum, const float* residual, float* y, int k, int n,
                                     void* stream) {
    FX_REQUIRE(x4 && s_x && b_x && w4 && w_s && w_sum && y, "linear_u4i4_gemv_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % 32 == 0 && k <= 16384, "linear_u4i4_gemv_dequant: k=%d must be a multiple of 32, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_u4i4_gemv_dequant: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv_u4i4<kEpi4Dequant>(x4, w4, nullptr, s_x, b_x, w_s, w_sum, residual, y, k, n, as_stream(stream));
}

int flexllm_linear_u4i4_gemm(const uint8_t* a4, const uint8_t* w4, int32_t* acc, int m, int k, int n, void* stream) {
    FX_REQUIRE(a4 && w4 && acc, "linear_u4i4_gemm: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_u4i4_gemm: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0, "linear_u4i4_gemm: m=%d n=%d", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm_u4i4<kGemmRaw>(a4, w4, acc, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, m, k, n, as_stream(stream));
}

int flexllm_linear_u4i4_gemm_dequant(const uint8_t* a4, const float* s_x, const float* b_x, const uint8_t* w4,
                                     const float* w_s, const float* w_sum, const float* residual, float* y, int m, int k,
                                     int n, void* stream) {
    FX_REQUIRE(a4 && s_x && b_x && w4 && w_s && w_sum && y, "linear_u4i4_gemm_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_u4i4_gemm_dequant: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0, "linear_u4i4_gemm_dequant: m=%d n=%d", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm_u4i4<kGemmDequantAsym>(a4, w4, nullptr, s_x, b_x, w_s, w_sum, residual, y, m, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemm_dequant_asym(const int8_t* a, const float* s_x, const float* b_x, const int8_t* w, const float* w_s,
                                        const float* w_sum, const float* residual, float* y, int m, int k, int n, void* stream) {
    FX_REQUIRE(a && s_x && b_x && w && w_s && w_sum && y, "linear_i8_gemm_dequant_asym: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm_dequant_asym: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0 && n % 4 == 0, "linear_i8_gemm_dequant_asym: m=%d n=%d (n a multiple of 4)", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm_asym(a, w, s_x, b_x, w_s, w_sum, residual, y, m, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemm_swiglu_asym(const int8_t* a, const float* s_x, const float* b_x, const int8_t* w_gu, const float* w_s_gu,
                                       const float* w_sum_gu, float* h, int m, int k, int n, void* stream) {
    FX_REQUIRE(a && s_x && b_x && w_gu && w_s_gu && w_sum_gu && h, "linear_i8_gemm_swiglu_asym: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm_swiglu_asym: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0 && n % 2 == 0, "linear_i8_gemm_swiglu_asym: m=%d n=%d (n must be even)", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm_swiglu_asym(a, w_gu, s_x, b_x, w_s_gu, w_sum_gu, h, m, k, 2 * n, as_stream(stream));
}

}  // extern "C"
