#include "hq_internal.h"
namespace hq {
int launch_quantize(hipStream_t, const float*, uint64_t, uint64_t, hq_ggml_type, void*) {
    return fail(HQ_ERR_UNSUPPORTED, "quantize: not built yet");
}
}
