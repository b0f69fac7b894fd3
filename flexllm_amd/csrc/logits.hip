// C ABI entry points; the kernels live in logits_kernels.h.
#include "logits_kernels.h"
#include <mutex>

using namespace fx;

static std::mutex g_logits_mu;      // guards the first-use allocation of the stand-alone entry points' scratch

extern "C" {

int flexllm_embed_f16(const uint16_t* embed, const int* token, float* y, int hidden, void* stream) {
    FX_REQUIRE(embed && token && y && hidden > 0, "embed: bad arguments");
    embed_kernel<<<(hidden + 255) / 256, 256, 0, as_stream(stream)>>>(reinterpret_cast<const __half*>(embed), token, y, hidden);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_lm_head_f16(const uint16_t* embed, const float* n, float* logits, int vocab, int hidden, void* stream) {
    FX_REQUIRE(embed && n && logits, "lm_head: null pointer");
    FX_REQUIRE(vocab >= 0 && hidden > 0 && hidden % 8 == 0 && hidden <= 4096, "lm_head: hidden=%d (multiple of 8, <= 4096)", hidden);
    if (vocab == 0) return FLEXLLM_OK;
    return lm_head_launch(embed, n, logits, vocab, hidden, as_stream(stream));
}

int flexllm_argmax_f32(const float* x, int n, int* result, void* stream) {
    FX_REQUIRE(x && result && n > 0, "argmax: bad arguments");
    {   // the first call allocates; concurrent first calls from several threads must not both do it
        std::lock_guard<std::mutex> lk(g_logits_mu);
        if (!g_pv) {
            FX_HIP(hipMalloc(&g_pv, kArgmaxParts * sizeof(float)));
            FX_HIP(hipMalloc(&g_pi, kArgmaxParts * sizeof(int)));
        }
    }
    return argmax_launch(x, n, result, g_pv, g_pi, as_stream(stream));
}

int flexllm_sample_topk_f32(const float* logits, int n, int top_k, const float* rand, int enable_sub_max, int* token,
                            int* top_idx, float* top_val, float* top_prob, void* stream) {
    FX_REQUIRE(logits && rand && token, "sample_topk: null pointer");
    FX_REQUIRE(n > 0 && top_k >= 1 && top_k <= kTopKMax && top_k <= n, "sample_topk: n=%d top_k=%d (1..%d)", n, top_k, kTopKMax);
    TopKOut out = {token, top_idx, top_val, top_prob, nullptr, nullptr, nullptr};
    if (n >= 4096) {
        {
            std::lock_guard<std::mutex> lk(g_logits_mu);
            if (!g_tv) {
                FX_HIP(hipMalloc(&g_tv, kTopKParts * kTopKMax * sizeof(float)));
                FX_HIP(hipMalloc(&g_ti, kTopKParts * kTopKMax * sizeof(int)));
            }
        }
        topk_partial_kernel<<<kTopKParts, kTopKPartThreads, 0, as_stream(stream)>>>(logits, n, top_k, g_tv, g_ti);
        topk_sample_kernel<256><<<1, 256, 0, as_stream(stream)>>>(g_tv, g_ti, kTopKParts * top_k, top_k, rand, 0, enable_sub_max, out);
    } else {
        topk_sample_kernel<kTopKThreads><<<1, kTopKThreads, 0, as_stream(stream)>>>(logits, nullptr, n, top_k, rand, 0, enable_sub_max, out);
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"
