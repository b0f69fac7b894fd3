// Prefill path of the Llama graph (M tokens at once): int8 MFMA GEMMs, causal int8 attention.
#pragma once
#include "common.h"

namespace fx {

struct LayerW {
    int8_t *wqkv, *wo, *wgu, *wd;      // [H+2KV][H], [H][H], [2I][H] (gate/up rows interleaved), [H][I]
    float *sqkv, *so, *sgu, *sd;
};

// Layer table of the W4A4 model: the same matrices with two 4-bit weights per byte along K (rows of K/2 bytes), and per
// output row the sum of its dequantised weights, which the asymmetric activations' zero point multiplies.
struct LayerW4 {
    int8_t *wqkv, *wo, *wgu, *wd;
    float *sqkv, *so, *sgu, *sd;
    float *mqkv, *mo, *mgu, *md;
};

struct PrefillWorkspace {
    int tokens = 0;
    void* base = nullptr;
};

inline void prefill_workspace_free(PrefillWorkspace* ws) {
    if (ws->base) (void)hipFree(ws->base);
    ws->base = nullptr;
    ws->tokens = 0;
}
inline void prefill_workspace_destroy(PrefillWorkspace* ws) {
    prefill_workspace_free(ws);
}

int llama_prefill_run(const flexllm_llama_config& cfg, const LayerW* layers, const float* gamma, const float* q_s,
                      const float* k_s, const float* v_s, const float* a_s, const float* rope_sin, const float* rope_cos,
                      int8_t* k_cache, int8_t* v_cache, size_t cache_layer_bytes, PrefillWorkspace* ws, const float* x_in,
                      int s, float* hidden_out, hipStream_t st);

int llama_prefill_run_w4a4(const flexllm_llama_config& cfg, const LayerW* layers, const LayerW4* sums, const float* gamma,
                           const float* q_s, const float* k_s, const float* v_s, const float* a_s, const float* rope_sin,
                           const float* rope_cos, int8_t* k_cache, int8_t* v_cache, size_t cache_layer_bytes,
                           PrefillWorkspace* ws, const float* x_in, int s, float* hidden_out, hipStream_t st);

}  // namespace fx
