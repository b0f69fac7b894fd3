// Prefill linear layers: C ABI entry points of the int8 MFMA GEMM (kernel in gemm_i8.h).
#include "gemm_i8.h"

using namespace fx;

extern "C" {

int flexllm_linear_i8_gemm(const int8_t* a, const int8_t* w, int32_t* acc, int m, int k, int n, void* stream) {
    FX_REQUIRE(a && w && acc, "linear_i8_gemm: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0, "linear_i8_gemm: m=%d n=%d", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm<kGemmRaw>(a, w, acc, nullptr, nullptr, nullptr, nullptr, m, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemm_dequant(const int8_t* a, const float* s_x, const int8_t* w, const float* w_s,
                                   const float* residual, float* y, int m, int k, int n, void* stream) {
    FX_REQUIRE(a && s_x && w && w_s && y, "linear_i8_gemm_dequant: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm_dequant: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0, "linear_i8_gemm_dequant: m=%d n=%d", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm<kGemmDequant>(a, w, nullptr, s_x, w_s, residual, y, m, k, n, as_stream(stream));
}

int flexllm_linear_i8_gemm_swiglu(const int8_t* a, const float* s_x, const int8_t* w_gu, const float* w_s_gu, float* h,
                                  int m, int k, int n, void* stream) {
    FX_REQUIRE(a && s_x && w_gu && w_s_gu && h, "linear_i8_gemm_swiglu: null pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm_swiglu: k=%d must be a multiple of 64", k);
    FX_REQUIRE(m >= 0 && n >= 0 && n % 2 == 0, "linear_i8_gemm_swiglu: m=%d n=%d (n must be even)", m, n);
    if (m == 0 || n == 0) return FLEXLLM_OK;
    return launch_gemm_swiglu(a, w_gu, s_x, w_s_gu, h, m, k, 2 * n, as_stream(stream));
}

}  // extern "C"
