// Decode linear layers: C ABI entry points of the int8 GEMV (kernels in gemv_i8.h).
#include "gemv_i8.h"


using namespace fx;

extern "C" {

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

int flexllm_linear_i8_gemv_swiglu(const int8_t* x, const float* s_x, const int8_t* w_gu, const float* w_s_gu, float* y,
                                  int k, int n, void* stream) {
    FX_REQUIRE(x && s_x && w_gu && w_s_gu && y, "linear_i8_gemv_swiglu: null pointer");
    FX_REQUIRE(k > 0 && k % 16 == 0 && k <= 16384, "linear_i8_gemv_swiglu: k=%d must be a multiple of 16, <= 16384", k);
    FX_REQUIRE(n >= 0, "linear_i8_gemv_swiglu: n=%d", n);
    if (n == 0) return FLEXLLM_OK;
    return launch_gemv<kEpiSwiglu>(x, w_gu, nullptr, s_x, w_s_gu, nullptr, y, k, 2 * n, as_stream(stream));
}

}  // extern "C"
