// C ABI entry points; the kernels live in elementwise_kernels.h.
#include "elementwise_kernels.h"

using namespace fx;

#define FX_DISPATCH_VPT(dim, CALL)                            \
    do {                                                      \
        const int nv_ = (dim) / 4;                            \
        if (nv_ <= kBlock) { constexpr int VPT = 1; CALL; }   \
        else if (nv_ <= 2 * kBlock) { constexpr int VPT = 2; CALL; } \
        else if (nv_ <= 4 * kBlock) { constexpr int VPT = 4; CALL; } \
        else if (nv_ <= 8 * kBlock) { constexpr int VPT = 8; CALL; } \
        else { constexpr int VPT = 16; CALL; }                \
    } while (0)

extern "C" {

int flexllm_quant_sym_i8(const float* x, int8_t* q, float* s, int rows, int dim, void* stream) {
    FX_REQUIRE(x && q && s, "quant_sym_i8: null pointer");
    FX_REQUIRE(rows >= 0 && dim > 0 && dim % 4 == 0 && dim <= 16384, "quant_sym_i8: dim=%d must be a multiple of 4, <= 16384", dim);
    if (rows == 0) return FLEXLLM_OK;
    FX_DISPATCH_VPT(dim, (quant_sym_kernel<VPT><<<rows, kBlock, 0, as_stream(stream)>>>(x, q, s, dim)));
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_quant_asym_u8(const float* x, uint8_t* q, float* s, float* b, int bits, int rows, int dim, void* stream) {
    FX_REQUIRE(x && q && s && b, "quant_asym_u8: null pointer");
    FX_REQUIRE(bits >= 2 && bits <= 8, "quant_asym_u8: bits=%d", bits);
    FX_REQUIRE(rows >= 0 && dim > 0 && dim % 4 == 0 && dim <= 16384, "quant_asym_u8: dim=%d must be a multiple of 4, <= 16384", dim);
    if (rows == 0) return FLEXLLM_OK;
    const float base = (float)((1 << bits) - 1);
    const unsigned mask = (1u << bits) - 1u;
    FX_DISPATCH_VPT(dim, (quant_asym_kernel<VPT><<<rows, kBlock, 0, as_stream(stream)>>>(x, q, s, b, dim, base, mask)));
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_dequant_i32_f32(const int32_t* acc, const float* s_x, const float* b_x, const float* w_s,
                            const float* w_sum, float* y, int rows, int n, void* stream) {
    FX_REQUIRE(acc && s_x && w_s && y, "dequant: null pointer");
    FX_REQUIRE((b_x == nullptr) == (w_sum == nullptr), "dequant: b_x and w_sum must both be set or both be null");
    FX_REQUIRE(rows >= 0 && rows <= 65535 && n > 0 && n % 4 == 0, "dequant: rows=%d n=%d (n %% 4 == 0, rows <= 65535)", rows, n);
    if (rows == 0) return FLEXLLM_OK;
    dim3 grid((unsigned)ew_grid((size_t)n / 4), (unsigned)rows);
    dequant_kernel<<<grid, kBlock, 0, as_stream(stream)>>>(acc, s_x, b_x, w_s, w_sum, y, n / 4);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_static_quant_i8(const float* x, int8_t* q, const float* scale, float factor, int is_signed, int rows,
                            int heads, int dim, void* stream) {
    FX_REQUIRE(x && q && scale, "static_quant: null pointer");
    FX_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && dim % 4 == 0, "static_quant: heads=%d dim=%d", heads, dim);
    const size_t nvec = (size_t)rows * heads * (dim / 4);
    if (nvec == 0) return FLEXLLM_OK;
    static_quant_kernel<<<ew_grid(nvec), kBlock, 0, as_stream(stream)>>>(x, q, scale, factor, is_signed, nvec, heads, dim / 4);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_static_dequant_i32_f32(const int32_t* acc, float* y, const float* a_s, const float* w_s, int rows,
                                   int act_heads, int w_heads, int dim, void* stream) {
    FX_REQUIRE(acc && y && a_s && w_s, "static_dequant: null pointer");
    FX_REQUIRE(rows >= 0 && act_heads > 0 && w_heads > 0 && act_heads % w_heads == 0 && dim > 0 && dim % 4 == 0,
               "static_dequant: act_heads=%d w_heads=%d dim=%d", act_heads, w_heads, dim);
    const size_t nvec = (size_t)rows * act_heads * (dim / 4);
    if (nvec == 0) return FLEXLLM_OK;
    static_dequant_kernel<<<ew_grid(nvec), kBlock, 0, as_stream(stream)>>>(acc, y, a_s, w_s, nvec, act_heads,
                                                                           act_heads / w_heads, dim / 4);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_head_quant_sym_i8(const float* x, int8_t* q, float* s, int rows, int heads, int dim, void* stream) {
    FX_REQUIRE(x && q && s, "head_quant: null pointer");
    FX_REQUIRE(rows >= 0 && heads > 0 && dim > 0 && dim % 4 == 0 && dim <= 256, "head_quant: dim=%d (multiple of 4, <= 256)", dim);
    const int nrows = rows * heads;
    if (nrows == 0) return FLEXLLM_OK;
    head_quant_kernel<<<(nrows + kNW - 1) / kNW, kBlock, 0, as_stream(stream)>>>(x, q, s, nrows, dim);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_rmsnorm_f32(const float* x, const float* gamma, float* y, int rows, int dim, float eps, void* stream) {
    FX_REQUIRE(x && gamma && y, "rmsnorm: null pointer");
    FX_REQUIRE(rows >= 0 && dim > 0 && dim % 4 == 0 && dim <= 16384, "rmsnorm: dim=%d must be a multiple of 4, <= 16384", dim);
    if (rows == 0) return FLEXLLM_OK;
    if (dim == 2048)      // the graphs' order of summation (see flexllm_rmsnorm_quant_i8)
        rmsnorm_kernel<1, false, 512><<<rows, 512, 0, as_stream(stream)>>>(x, gamma, y, nullptr, nullptr, dim, eps);
    else
        FX_DISPATCH_VPT(dim, (rmsnorm_kernel<VPT, false><<<rows, kBlock, 0, as_stream(stream)>>>(x, gamma, y, nullptr, nullptr, dim, eps)));
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_rmsnorm_quant_i8(const float* x, const float* gamma, int8_t* q, float* s, int rows, int dim, float eps,
                             void* stream) {
    FX_REQUIRE(x && gamma && q && s, "rmsnorm_quant: null pointer");
    FX_REQUIRE(rows >= 0 && dim > 0 && dim % 4 == 0 && dim <= 16384, "rmsnorm_quant: dim=%d must be a multiple of 4, <= 16384", dim);
    if (rows == 0) return FLEXLLM_OK;
    // Rows of 2048 values take the one-wave-per-row kernel of the layer graphs: one order of summation for the sum of
    // squares on every path (this entry point, the prefill graph, both decode schedules), so that a stage-by-stage
    // chain of entry points reproduces the graphs bit for bit.
    if (dim == 2048)
        rmsnorm_quant_2048_wave_kernel<<<(rows + kNormWaveRows - 1) / kNormWaveRows, 64 * kNormWaveRows, 0, as_stream(stream)>>>(x, gamma, q, s, rows, eps);
    else
        FX_DISPATCH_VPT(dim, (rmsnorm_kernel<VPT, true><<<rows, kBlock, 0, as_stream(stream)>>>(x, gamma, nullptr, q, s, dim, eps)));
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_rmsnorm_quant_asym_u8(const float* x, const float* gamma, uint8_t* q, float* s, float* b, int bits, int rows, int dim,
                                  float eps, void* stream) {
    FX_REQUIRE(x && gamma && q && s && b, "rmsnorm_quant_asym: null pointer");
    FX_REQUIRE(bits >= 2 && bits <= 8, "rmsnorm_quant_asym: bits=%d", bits);
    FX_REQUIRE(rows >= 0 && dim == 2048, "rmsnorm_quant_asym: dim=%d (instantiated for rows of 2048 values)", dim);
    if (rows == 0) return FLEXLLM_OK;
    rmsnorm_quant_asym_2048_wave_kernel<<<(rows + kNormWaveRows - 1) / kNormWaveRows, 64 * kNormWaveRows, 0, as_stream(stream)>>>(
        x, gamma, q, s, b, rows, eps, (float)((1 << bits) - 1), (1u << bits) - 1u);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_rope_f32(const float* x, float* y, const float* sin_t, const float* cos_t, int tokens, int heads,
                     int head_dim, int pos0, void* stream) {
    FX_REQUIRE(x && y && sin_t && cos_t, "rope: null pointer");
    FX_REQUIRE(tokens >= 0 && heads > 0 && head_dim > 0 && head_dim % 2 == 0 && pos0 >= 0, "rope: heads=%d head_dim=%d pos0=%d", heads, head_dim, pos0);
    const size_t npairs = (size_t)tokens * heads * (head_dim / 2);
    if (npairs == 0) return FLEXLLM_OK;
    rope_kernel<<<ew_grid(npairs), kBlock, 0, as_stream(stream)>>>(x, y, sin_t, cos_t, npairs, heads, head_dim / 2, pos0);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_rope_table_host(float* sin_t, float* cos_t, int max_pos, int head_dim, float theta, int factor,
                            int low_freq_factor, int high_freq_factor, int original_max_pe) {
    FX_REQUIRE(sin_t && cos_t && max_pos > 0 && head_dim > 0 && head_dim % 2 == 0, "rope_table: bad arguments");
    FX_REQUIRE(factor > 0 && low_freq_factor > 0 && high_freq_factor > low_freq_factor, "rope_table: bad scaling factors");
    const int half = head_dim / 2;
    const float high_wl = (float)(original_max_pe / high_freq_factor);
    const float low_wl = (float)(original_max_pe / low_freq_factor);
    for (int i = 0; i < half; i++) {
        const float inv_freq = powf(theta, (2.0f * (float)i) / (float)head_dim);
        const float freq = 1.0f / inv_freq;
        const float wavelength = (float)(2.0 * M_PI * (double)inv_freq);
        float f;
        if (wavelength < high_wl) f = freq;
        else if (wavelength > low_wl) f = freq / (float)factor;
        else {
            const float a = ((float)original_max_pe / wavelength - (float)low_freq_factor) /
                            (float)(high_freq_factor - low_freq_factor);
            f = (1.0f - a) * (freq / (float)factor) + a * freq;
        }
        for (int p = 0; p < max_pos; p++) {
            const float th = (float)p * f;
            sin_t[(size_t)p * half + i] = sinf(th);
            cos_t[(size_t)p * half + i] = cosf(th);
        }
    }
    return FLEXLLM_OK;
}

int flexllm_swish_f32(const float* x, float* y, size_t n, void* stream) {
    FX_REQUIRE(x && y, "swish: null pointer");
    if (n == 0) return FLEXLLM_OK;
    swish_kernel<<<ew_grid(n), kBlock, 0, as_stream(stream)>>>(x, y, n);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}
int flexllm_swiglu_f32(const float* gate, const float* up, float* y, size_t n, void* stream) {
    FX_REQUIRE(gate && up && y, "swiglu: null pointer");
    if (n == 0) return FLEXLLM_OK;
    swiglu_kernel<<<ew_grid(n), kBlock, 0, as_stream(stream)>>>(gate, up, y, n);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}
int flexllm_residual_add_f32(const float* a, const float* b, float* y, size_t n, void* stream) {
    FX_REQUIRE(a && b && y, "residual_add: null pointer");
    if (n == 0) return FLEXLLM_OK;
    add_kernel<<<ew_grid(n), kBlock, 0, as_stream(stream)>>>(a, b, y, n);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}
int flexllm_softmax_f32(const float* x, float* y, int rows, int dim, void* stream) {
    FX_REQUIRE(x && y, "softmax: null pointer");
    FX_REQUIRE(rows >= 0 && dim > 0, "softmax: dim=%d", dim);
    if (rows == 0) return FLEXLLM_OK;
    softmax_kernel<<<rows, kBlock, 0, as_stream(stream)>>>(x, y, dim);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"
