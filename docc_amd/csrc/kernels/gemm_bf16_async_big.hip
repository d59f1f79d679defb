// bf16 x bf16 -> fp32 GEMM, asynchronous pipeline, 256x256 tile: 256 accumulator registers per
// lane, which only the AGPR half of the register file can hold.
#include "gemm_async.h"

DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 256, 256, 64, 2, 2, 2)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 256, 256, 32, 2, 2, 4)
#endif
