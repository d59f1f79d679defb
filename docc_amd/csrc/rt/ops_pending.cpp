// Entry points whose kernels are not built yet report DOCC_ROCM_ERR_UNSUPPORTED.
#include "docc_rocm_ops.h"
#include "rt_state.h"
using namespace docc::rt::rocm;
extern "C" {
int docc_rocm_attention_bf16(docc_rocm_stream_t, int64_t, int64_t, int64_t, int64_t, int64_t, float, const uint16_t*, const uint16_t*, const uint16_t*, void*, int) { return fail(DOCC_ROCM_ERR_UNSUPPORTED, "attention: not built"); }
}
