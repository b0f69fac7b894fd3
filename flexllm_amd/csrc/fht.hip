// C ABI entry points; the kernels live in fht_kernels.h.
#include "fht_kernels.h"

using namespace fx;

extern "C" {

int flexllm_fht_f32(const float* x, float* y, int rows, int n, float scale, void* stream) {
    FX_REQUIRE(x && y, "fht: null pointer");
    FX_REQUIRE(rows >= 0 && scale != 0.0f, "fht: rows=%d scale=%g", rows, (double)scale);
    if (rows == 0) return FLEXLLM_OK;
    return launch_fht<0>(x, y, nullptr, nullptr, rows, n, scale, as_stream(stream));
}

int flexllm_fht_quant_i8(const float* x, int8_t* q, float* s, int rows, int n, float scale, void* stream) {
    FX_REQUIRE(x && q && s, "fht_quant: null pointer");
    FX_REQUIRE(rows >= 0 && scale != 0.0f, "fht_quant: rows=%d scale=%g", rows, (double)scale);
    if (rows == 0) return FLEXLLM_OK;
    return launch_fht<1>(x, nullptr, q, s, rows, n, scale, as_stream(stream));
}

int flexllm_fht_quant_asym_u8(const float* x, uint8_t* q, float* s, float* b, int bits, int rows, int n, float scale, void* stream) {
    FX_REQUIRE(x && q && s && b, "fht_quant_asym: null pointer");
    FX_REQUIRE(bits >= 2 && bits <= 8, "fht_quant_asym: bits=%d", bits);
    FX_REQUIRE(rows >= 0 && scale != 0.0f, "fht_quant_asym: rows=%d scale=%g", rows, (double)scale);
    if (rows == 0) return FLEXLLM_OK;
    return launch_fht<2>(x, nullptr, reinterpret_cast<int8_t*>(q), s, rows, n, scale, as_stream(stream), b, (float)((1 << bits) - 1),
                         (1u << bits) - 1u);
}

}  // extern "C"
