// C ABI entry points; the kernels live in fht_kernels.h.
#include "fht_kernels.h"

using namespace fx;

extern "C" {

int flexllm_fht_f32(const float* x, float* y, int rows, int n, float scale, void* stream) {
    FX_REQUIRE(x && y, "fht: null pointer");
    FX_REQUIRE(rows >= 0 && scale != 0.0f, "fht: rows=%d scale=%g", rows, (double)scale);
    if (rows == 0) return FLEXLLM_OK;
    return launch_fht<false>(x, y, nullptr, nullptr, rows, n, scale, as_stream(stream));
}

int flexllm_fht_quant_i8(const float* x, int8_t* q, float* s, int rows, int n, float scale, void* stream) {
    FX_REQUIRE(x && q && s, "fht_quant: null pointer");
    FX_REQUIRE(rows >= 0 && scale != 0.0f, "fht_quant: rows=%d scale=%g", rows, (double)scale);
    if (rows == 0) return FLEXLLM_OK;
    return launch_fht<true>(x, nullptr, q, s, rows, n, scale, as_stream(stream));
}

}  // extern "C"
