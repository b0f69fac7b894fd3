// C ABI entry points of the HMT plug-in; the kernels live in hmt_kernels.h.
#include "hmt_kernels.h"

using namespace fx;

extern "C" {

int flexllm_linear_f32_gemv(const float* x, const float* w, float* y, int k, int n, void* stream) {
    FX_REQUIRE(x && w && y, "linear_f32_gemv: null pointer");
    FX_REQUIRE(k > 0 && k % 4 == 0 && n > 0, "linear_f32_gemv: k=%d (multiple of 4) n=%d", k, n);
    linear_f32_gemv_kernel<<<(n + 3) / 4, 256, 0, as_stream(stream)>>>(x, w, y, k, n);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_hmt_retrieve(const float* q, const float* kmem, const float* mmem, float* a_sft, float* p_out, int mem_num,
                         int hidden, float scale, void* stream) {
    FX_REQUIRE(q && kmem && mmem && a_sft && p_out, "hmt_retrieve: null pointer");
    FX_REQUIRE(mem_num > 0 && mem_num <= kHmtMaxSlots && hidden > 0 && hidden % 4 == 0 && scale > 0.0f,
               "hmt_retrieve: mem_num=%d (1..%d) hidden=%d (multiple of 4) scale=%g", mem_num, kHmtMaxSlots, hidden, (double)scale);
    hmt_scores_softmax_kernel<<<1, 1024, 0, as_stream(stream)>>>(q, kmem, a_sft, mem_num, hidden, scale);
    hmt_weighted_sum_kernel<<<(hidden + 255) / 256, 256, 0, as_stream(stream)>>>(a_sft, mmem, p_out, mem_num, hidden);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

int flexllm_hmt_stage_input(const float* emb, const float* t_embed, const float* p_buf, float* x_out, int stage, int seq_off,
                            int cur_len, int cur_sum_len, int rec_len, int tail_p, int rows, int hidden, void* stream) {
    FX_REQUIRE(emb && t_embed && p_buf && x_out, "hmt_stage_input: null pointer");
    FX_REQUIRE((stage == 0 || stage == 1) && seq_off >= 0 && cur_len > 0 && cur_sum_len >= 0 && cur_sum_len <= cur_len && rec_len >= 0 &&
                   hidden > 0 && hidden % 4 == 0,
               "hmt_stage_input: stage=%d off=%d cur=%d sum=%d rec=%d hidden=%d", stage, seq_off, cur_len, cur_sum_len, rec_len, hidden);
    const int need = stage == 0 ? 1 + cur_sum_len + 1 : 1 + rec_len + cur_len + (tail_p ? 1 : 0);
    FX_REQUIRE(rows >= need, "hmt_stage_input: rows=%d < %d", rows, need);
    hmt_stage_input_kernel<<<rows, 256, 0, as_stream(stream)>>>(emb, t_embed, p_buf, x_out, stage, seq_off, cur_len, cur_sum_len, rec_len,
                                                            tail_p ? 1 : 0, hidden);
    FX_LAUNCH_CHECK();
    return FLEXLLM_OK;
}

}  // extern "C"
