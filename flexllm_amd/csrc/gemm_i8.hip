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

int flexllm_linear_i8_gemm_qkv_rope_cache(const int8_t* a, const float* s_x, const int8_t* w_qkv, const float* w_s,
                                          const float* sin_t, const float* cos_t, const flexllm_mha_scales* sc,
                                          int8_t* q8, int8_t* k_cache, int8_t* v_cache, int m, int k, int q_heads,
                                          int kv_heads, int max_pos, int pos0, void* stream) {
    FX_REQUIRE(a && s_x && w_qkv && w_s && sin_t && cos_t && sc && q8 && k_cache && v_cache, "linear_i8_gemm_qkv_rope_cache: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s, "linear_i8_gemm_qkv_rope_cache: null scale pointer");
    FX_REQUIRE(k > 0 && k % kGemmBK == 0, "linear_i8_gemm_qkv_rope_cache: k=%d must be a multiple of 64", k);
    FX_REQUIRE(q_heads > 0 && kv_heads > 0 && max_pos > 0 && max_pos % 64 == 0 && m >= 0 && pos0 >= 0,
               "linear_i8_gemm_qkv_rope_cache: q_heads=%d kv_heads=%d max_pos=%d m=%d pos0=%d", q_heads, kv_heads, max_pos, m, pos0);
    if (m == 0) return FLEXLLM_OK;
    QkvEpiArgs qa;
    qa.sin_t = sin_t; qa.cos_t = cos_t; qa.q_s = sc->q_s; qa.k_s = sc->k_s; qa.v_s = sc->v_s;
    qa.q8 = q8; qa.kc = k_cache; qa.vc = v_cache;
    qa.pos0 = pos0; qa.q_heads = q_heads; qa.kv_heads = kv_heads; qa.max_pos = max_pos;
    return launch_gemm_qkv(a, w_qkv, s_x, w_s, m, k, qa, as_stream(stream));
}

}  // extern "C"
