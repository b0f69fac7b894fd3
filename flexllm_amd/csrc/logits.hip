// C ABI entry points; the kernels live in logits_kernels.h.
#include "logits_kernels.h"

using namespace fx;

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
    // per-workgroup candidates in the calling stream's scratch: [kArgmaxParts] values, then [kArgmaxParts] indices
    void* base = nullptr;
    int rc = stream_scratch(kScratchArgmax, as_stream(stream), kArgmaxParts * (sizeof(float) + sizeof(int)), &base);
    if (rc) return rc;
    float* pv = static_cast<float*>(base);
    return argmax_launch(x, n, result, pv, reinterpret_cast<int*>(pv + kArgmaxParts), as_stream(stream));
}

int flexllm_sample_topk_f32(const float* logits, int n, int top_k, const float* rand, int enable_sub_max, int* token,
                            int* top_idx, float* top_val, float* top_prob, void* stream) {
    FX_REQUIRE(logits && rand && token, "sample_topk: null pointer");
    FX_REQUIRE(n > 0 && top_k >= 1 && top_k <= kTopKMax && top_k <= n, "sample_topk: n=%d top_k=%d (1..%d)", n, top_k, kTopKMax);
    TopKOut out = {token, top_idx, top_val, top_prob, nullptr, nullptr, nullptr};
    if (n >= 4096) {
        void* base = nullptr;                      // the calling stream's scratch: candidate values, then their indices
        int rc = stream_scratch(kScratchTopK, as_stream(stream), (size_t)kTopKParts * kTopKMax * (sizeof(float) + sizeof(int)), &base);
        if (rc) return rc;
        float* tv = static_cast<float*>(base);
        int* ti = reinterpret_cast<int*>(tv + kTopKParts * kTopKMax);
        topk_partial_kernel<<<kTopKParts, kTopKPartThreads, 0, as_stream(stream)>>>(logits, n, top_k, tv, ti);
        topk_sample_kernel<256><<<1, 256, 0, as_stream(stream)>>>(tv, ti, kTopKParts * top_k, top_k, rand, 0, enable_sub_max, out);
    } else {
        topk_sample_kernel<kTopKThreads><<<1, kTopKThreads, 0, as_stream(stream)>>>(logits, nullptr, n, top_k, rand, 0, enable_sub_max, out);
    }
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"
