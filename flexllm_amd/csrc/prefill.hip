// Prefill path (placeholder until the MFMA GEMM and the causal attention kernel land).
#include "prefill.h"

namespace fx {
int llama_prefill_run(const flexllm_llama_config&, const LayerW*, const float*, const float*, const float*, const float*,
                      const float*, const float*, const float*, int8_t*, int8_t*, size_t, PrefillWorkspace*, const float*,
                      int, float*, hipStream_t) {
    set_error("prefill: not built yet");
    return FLEXLLM_EINVAL;
}
}  // namespace fx
