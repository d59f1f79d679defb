// bf16 x bf16 -> fp32 GEMM, asynchronous multi-stage pipeline (see gemm_async.h), tiles whose
// accumulators fit in ordinary VGPRs.
#include "gemm_async.h"

#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 128, 128, 64, 2, 2, 3)
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 128, 128, 64, 2, 2, 4)
#endif
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 128, 128, 32, 2, 2, 4)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(bgemm, uint16_t, float, 128, 256, 64, 2, 2, 3)
#endif
