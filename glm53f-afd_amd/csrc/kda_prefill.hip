// Placeholder until the MFMA prefill lands: the entry points exist and refuse to run.
#include "kda_common.h"

extern "C" int64_t glm53f_kda_prefill_workspace_bytes(int32_t, int32_t, int32_t) { return 0; }
#define UNUSED_PREFILL_ARGS                                                                                       \
    const glm53f_bf16*, int64_t, int64_t, const glm53f_bf16*, int64_t, const glm53f_bf16*, int64_t
extern "C" int glm53f_kda_prefill(int32_t, int32_t, UNUSED_PREFILL_ARGS, glm53f_bf16*, const glm53f_bf16*,
                                  const float*, float*, const float*, const float*, const glm53f_bf16*, float, float,
                                  glm53f_bf16*, int64_t, int32_t, float*, int64_t, glm53f_stream_t) {
    return (int)hipErrorNotSupported;
}
extern "C" int glm53f_kda_prefill_batch(int32_t, int32_t, const int32_t*, int32_t, UNUSED_PREFILL_ARGS, glm53f_bf16*,
                                        const int64_t*, const glm53f_bf16*, const float*, float*, const int64_t*,
                                        const float*, const float*, const glm53f_bf16*, float, float, glm53f_bf16*,
                                        int64_t, int32_t, float*, int64_t, glm53f_stream_t) {
    return (int)hipErrorNotSupported;
}
extern "C" int glm53f_kda_prefill_batch_bf16state(int32_t, int32_t, const int32_t*, int32_t, UNUSED_PREFILL_ARGS,
                                                  glm53f_bf16*, const int64_t*, const glm53f_bf16*,
                                                  const glm53f_bf16*, glm53f_bf16*, const int64_t*, const float*,
                                                  const float*, const glm53f_bf16*, float, float, glm53f_bf16*,
                                                  int64_t, int32_t, float*, int64_t, glm53f_stream_t) {
    return (int)hipErrorNotSupported;
}
