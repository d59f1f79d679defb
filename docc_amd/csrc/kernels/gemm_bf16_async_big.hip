// bf16 x bf16 -> fp32 GEMM, asynchronous pipeline, 256x256 tile: 256 accumulator registers per
// lane, which only the AGPR half of the register file can hold.
#include "gemm_async16.h"

// Four stages of 32 k with the copies of a stage dealt over the MFMAs of a whole K-step: four waves that leave the
// barrier together and each issue their sixteen copies in one run queue up in the CU's one vector-memory pipe
// (a 4096^3 product: 91 us with two stages of 64 k and the copies in a run, 83 us this way, on operands that do
// not load the power limit; 117 and 113 us on N(0,1) operands).
DOCC_AGEMM_SPREAD_CONFIG(bgemm, uint16_t, float, 256, 256, 32, 2, 2, 4)
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 256, 256, 64, 2, 2, 2)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 256, 256, 32, 2, 2, 4)
#endif
// The same tile on the 16x16x32 MFMA (gemm_async16.h), for products with K a multiple of 32.
DOCC_AGEMM16_CONFIG(256, 256, 2, 2, 4)
