// Prefill path of the Llama graph: M tokens at once through int8 MFMA GEMMs and causal int8 attention,
// plus the C ABI entry point of the stand-alone prefill attention.
#include "prefill.h"
#include "attn_prefill.h"
#include "elementwise_kernels.h"
#include "fht_kernels.h"
#include "gemm_i8.h"

namespace fx {

struct PrefillBuffers {
    float *x, *x2, *att;    // residual stream before / after the attention block, attention output: [s][hidden]
    float* gu;              // SiLU(gate)*up [s][inter]
    int8_t *xq, *q8;        // quantised input of the current linear layer [s][inter at most]; quantised, rotated q [s][hidden]
    float *xs, *xb;         // per-token scales; per-token zero points (W4A4 graph)
};

static int prefill_workspace_get(PrefillWorkspace* ws, const flexllm_llama_config& c, int s, PrefillBuffers* b) {
    const size_t H = c.hidden, I = c.inter;
    auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
    const size_t sz_x = up(sizeof(float) * s * H), sz_gu = up(sizeof(float) * s * I), sz_xq = up((size_t)s * I), sz_q8 = up((size_t)s * H);
    const size_t sz_xs = up(sizeof(float) * s);
    const size_t total = 3 * sz_x + sz_gu + sz_xq + sz_q8 + 2 * sz_xs;
    if (ws->tokens < s) {
        FX_HIP(hipDeviceSynchronize());
        prefill_workspace_free(ws);
        hipError_t e = hipMalloc(&ws->base, total);
        if (e != hipSuccess) { set_error("prefill workspace hipMalloc(%zu) failed: %s", total, hipGetErrorString(e)); return FLEXLLM_ENOMEM; }
        ws->tokens = s;
    }
    char* p = (char*)ws->base;
    b->x = (float*)p; p += sz_x;
    b->x2 = (float*)p; p += sz_x;
    b->att = (float*)p; p += sz_x;
    b->gu = (float*)p; p += sz_gu;
    b->xq = (int8_t*)p; p += sz_xq;
    b->q8 = (int8_t*)p; p += sz_q8;
    b->xs = (float*)p; p += sz_xs;
    b->xb = (float*)p; p += sz_xs;
    return FLEXLLM_OK;
}

// RMSNorm + per-row quantisation of s rows of H = 2048 values: one wave per row (the same arithmetic as the
// one-workgroup-per-row kernel, to the bit, without its two workgroup barriers).
static inline void rmsnorm_quant_rows(const float* x, const float* gamma, int8_t* q, float* scale, int s, int H, float eps, hipStream_t st) {
    if (H == 2048)
        rmsnorm_quant_2048_wave_kernel<<<(s + kNormWaveRows - 1) / kNormWaveRows, 64 * kNormWaveRows, 0, st>>>(x, gamma, q, scale, s, eps);
    else
        rmsnorm_kernel<1, true, 512><<<s, 512, 0, st>>>(x, gamma, nullptr, q, scale, H, eps);
}

int llama_prefill_run(const flexllm_llama_config& c, const LayerW* layers, const float* gamma, const float* q_s_all,
                      const float* k_s_all, const float* v_s_all, const float* a_s_all, const float* rope_sin,
                      const float* rope_cos, int8_t* k_cache, int8_t* v_cache, size_t cache_layer_bytes,
                      PrefillWorkspace* ws, const float* x_in, int s, float* hidden_out, hipStream_t st) {
    FX_REQUIRE(s > 0 && s % kPfTile == 0 && s <= c.max_pos, "prefill: s=%d must be a positive multiple of 32, <= max_pos=%d", s, c.max_pos);
    PrefillBuffers b;
    int rc = prefill_workspace_get(ws, c, s, &b);
    if (rc) return rc;
    const int H = c.hidden, I = c.inter;
    // The first layer reads the caller's x_in and the last one writes the caller's hidden_out directly (x_in is last read
    // by the first layer's o projection, so the two may be one buffer): no copies in or out.
    const float* xin = x_in;
    for (int l = 0; l < c.layers; l++) {
        float* const xout = (l == c.layers - 1 && hidden_out) ? hidden_out : b.x;
        const LayerW& w = layers[l];
        const float* g0 = gamma + (size_t)(2 * l) * H;
        const float* g1 = gamma + (size_t)(2 * l + 1) * H;
        const float* q_s = q_s_all + (size_t)l * c.q_heads;
        const float* k_s = k_s_all + (size_t)l * c.kv_heads;
        const float* v_s = v_s_all + (size_t)l * c.kv_heads;
        const float* a_s = a_s_all + (size_t)l * c.q_heads;
        int8_t* kc = k_cache + (size_t)l * cache_layer_bytes;
        int8_t* vc = v_cache + (size_t)l * cache_layer_bytes;
        // attention block
        rmsnorm_quant_rows(xin, g0, b.xq, b.xs, s, H, c.eps, st);
        {   // q/k/v projection with RoPE, static quantisation and the cache stores in the GEMM epilogue
            QkvEpiArgs qa;
            qa.sin_t = rope_sin; qa.cos_t = rope_cos; qa.q_s = q_s; qa.k_s = k_s; qa.v_s = v_s;
            qa.q8 = b.q8; qa.kc = kc; qa.vc = vc;
            qa.pos0 = 0; qa.q_heads = c.q_heads; qa.kv_heads = c.kv_heads; qa.max_pos = c.max_pos;
            if ((rc = launch_gemm_qkv(b.xq, w.wqkv, b.xs, w.sqkv, s, H, qa, st))) return rc;
        }
        if ((rc = mha_prefill_launch(b.q8, kc, vc, q_s, k_s, v_s, a_s, b.att, nullptr, s, c.q_heads, c.kv_heads, c.max_pos, st))) return rc;
        quant_sym_kernel<2><<<s, kBlock, 0, st>>>(b.att, b.xq, b.xs, H);   // (one wave per row, as for the norm: measured no faster here)
        if ((rc = launch_gemm<kGemmDequant>(b.xq, w.wo, nullptr, b.xs, w.so, xin, b.x2, s, H, H, st))) return rc;
        // feed-forward block
        rmsnorm_quant_rows(b.x2, g1, b.xq, b.xs, s, H, c.eps, st);
        if ((rc = launch_gemm_swiglu(b.xq, w.wgu, b.xs, w.sgu, b.gu, s, H, 2 * I, st))) return rc;     // b.gu = SiLU(gate)*up [s][I]
        fht_kernel<13, true, false><<<s, kFhtBlock, 0, st>>>(b.gu, nullptr, b.xq, b.xs, c.fht_scale);
        if ((rc = launch_gemm<kGemmDequant>(b.xq, w.wd, nullptr, b.xs, w.sd, b.x2, xout, s, I, H, st))) return rc;
        xin = xout;
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

// The W4A4 configuration (asymmetric uint4 activations x int4 weights, the stage order of SpinQuant_Prefilling.h:807-1050)
// over the same kernels the module entry points use: the 4-bit values are held one per byte (layers: the matrices as
// flexllm_llama_create keeps them, sums: the row sums of the dequantised weights) and multiplied on the int8 direct-load
// MFMA kernel with the asymmetric dequantisation in its epilogue; RoPE, static quantisation and the cache stores run as
// one kernel per token row, SiLU(gate)*up is formed in the epilogue of the gate/up GEMM.
int llama_prefill_run_w4a4(const flexllm_llama_config& c, const LayerW* layers, const LayerW4* sums, const float* gamma,
                           const float* q_s_all, const float* k_s_all, const float* v_s_all, const float* a_s_all,
                           const float* rope_sin, const float* rope_cos, int8_t* k_cache, int8_t* v_cache,
                           size_t cache_layer_bytes, PrefillWorkspace* ws, const float* x_in, int s, float* hidden_out,
                           hipStream_t st) {
    FX_REQUIRE(s > 0 && s % kPfTile == 0 && s <= c.max_pos, "prefill: s=%d must be a positive multiple of 32, <= max_pos=%d", s, c.max_pos);
    FX_REQUIRE(c.hidden == 2048 && c.inter == 8192, "prefill (W4A4): hidden=%d inter=%d (instantiated for 2048/8192)", c.hidden, c.inter);
    PrefillBuffers b;
    int rc = prefill_workspace_get(ws, c, s, &b);
    if (rc) return rc;
    const int H = c.hidden, I = c.inter;
    uint8_t* xq = reinterpret_cast<uint8_t*>(b.xq);
    const float* xin = x_in;                                   // no copies in or out, as in llama_prefill_run
    for (int l = 0; l < c.layers; l++) {
        float* const xout = (l == c.layers - 1 && hidden_out) ? hidden_out : b.x;
        const LayerW& w = layers[l];
        const LayerW4& m4 = sums[l];
        const float* q_s = q_s_all + (size_t)l * c.q_heads;
        const float* k_s = k_s_all + (size_t)l * c.kv_heads;
        const float* v_s = v_s_all + (size_t)l * c.kv_heads;
        const float* a_s = a_s_all + (size_t)l * c.q_heads;
        int8_t* kc = k_cache + (size_t)l * cache_layer_bytes;
        int8_t* vc = v_cache + (size_t)l * cache_layer_bytes;
        // attention block
        rmsnorm_quant_asym_2048_wave_kernel<<<(s + kNormWaveRows - 1) / kNormWaveRows, 64 * kNormWaveRows, 0, st>>>(
            xin, gamma + (size_t)(2 * l) * H, xq, b.xs, b.xb, s, c.eps, 15.0f, 15u);
        {   // q/k/v projection with the asymmetric dequantisation, RoPE, static quantisation and the cache stores in the GEMM epilogue
            QkvEpiArgs qa;
            qa.sin_t = rope_sin; qa.cos_t = rope_cos; qa.q_s = q_s; qa.k_s = k_s; qa.v_s = v_s;
            qa.q8 = b.q8; qa.kc = kc; qa.vc = vc;
            qa.pos0 = 0; qa.q_heads = c.q_heads; qa.kv_heads = c.kv_heads; qa.max_pos = c.max_pos;
            qa.b_x = b.xb; qa.w_sum = m4.mqkv;
            if ((rc = launch_gemm_qkv(b.xq, w.wqkv, b.xs, w.sqkv, s, H, qa, st))) return rc;
        }
        if ((rc = mha_prefill_launch(b.q8, kc, vc, q_s, k_s, v_s, a_s, b.att, nullptr, s, c.q_heads, c.kv_heads, c.max_pos, st))) return rc;
        quant_asym_kernel<2><<<s, kBlock, 0, st>>>(b.att, xq, b.xs, b.xb, H, 15.0f, 15u);
        if ((rc = launch_gemm_asym(b.xq, w.wo, b.xs, b.xb, w.so, m4.mo, xin, b.x2, s, H, H, st))) return rc;
        // feed-forward block
        rmsnorm_quant_asym_2048_wave_kernel<<<(s + kNormWaveRows - 1) / kNormWaveRows, 64 * kNormWaveRows, 0, st>>>(
            b.x2, gamma + (size_t)(2 * l + 1) * H, xq, b.xs, b.xb, s, c.eps, 15.0f, 15u);
        // gate/up with SiLU(gate)*up in the GEMM epilogue: b.gu = [s][I]
        if ((rc = launch_gemm_swiglu_asym(b.xq, w.wgu, b.xs, b.xb, w.sgu, m4.mgu, b.gu, s, H, 2 * I, st))) return rc;
        fht_kernel<13, 2, false><<<s, kFhtBlock, 0, st>>>(b.gu, nullptr, b.xq, b.xs, c.fht_scale, b.xb, 15.0f, 15u);   // transform + uint4 quantisation
        if ((rc = launch_gemm_asym(b.xq, w.wd, b.xs, b.xb, w.sd, m4.md, b.x2, xout, s, I, H, st))) return rc;
        xin = xout;
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // namespace fx

using namespace fx;

extern "C" {

int flexllm_mha_i8_prefill(const int8_t* q8, const int8_t* k_cache, const int8_t* v_cache, const flexllm_mha_scales* sc,
                           float* o, uint8_t* p8_out, int s, int q_heads, int kv_heads, int head_dim, int max_pos,
                           void* stream) {
    FX_REQUIRE(q8 && k_cache && v_cache && sc && o, "mha_prefill: null pointer");
    FX_REQUIRE(sc->q_s && sc->k_s && sc->v_s && sc->a_s, "mha_prefill: null scale table");
    FX_REQUIRE(head_dim == kHd, "mha_prefill: head_dim=%d (only 64)", head_dim);
    FX_REQUIRE(kv_heads > 0 && q_heads % kv_heads == 0, "mha_prefill: q_heads=%d kv_heads=%d", q_heads, kv_heads);
    FX_REQUIRE(s > 0 && s % kPfTile == 0 && s <= max_pos && max_pos % kVBlock == 0,
               "mha_prefill: s=%d max_pos=%d (s a positive multiple of 32, s <= max_pos, max_pos %% 64 == 0)", s, max_pos);
    return mha_prefill_launch(q8, k_cache, v_cache, sc->q_s, sc->k_s, sc->v_s, sc->a_s, o, p8_out, s, q_heads, kv_heads,
                              max_pos, as_stream(stream));
}

}  // extern "C"
