// fp32 GEMM, asynchronous pipeline, 256x256 tile: 256 accumulator registers per lane, which only the AGPR half of
// the register file can hold (the other fp32 kernels are built with their accumulators in ordinary VGPRs, see
// gemm_f32.hip). One tile per compute unit at 4096^3: against the 128x256 tile a quarter less operand traffic per
// flop and no second round of work-groups (943 us against 970 for the 4096^3 product).
#include "gemm_async.h"

DOCC_AGEMM_CONFIG(sgemm, float, float, 256, 256, 32, 2, 2, 2)
