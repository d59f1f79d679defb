// fp32 GEMM kernels (v_mfma_f32_32x32x2_f32), see gemm_mfma.h and gemm_async.h.
#include "gemm_async.h"

DOCC_GEMM_CONFIG(sgemm, float, 128, 128, 16, 2, 2)
DOCC_GEMM_CONFIG(sgemm, float, 64, 64, 16, 2, 2)

// asynchronous multi-stage variants (aligned operands). The two large tiles take 96 KB of LDS, so that one
// work-group owns a compute unit: two co-resident work-groups of these tiles run 6-9 % slower at 4096^3.
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 128, 32, 2, 2, 3)
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 256, 32, 2, 2, 2)
DOCC_AGEMM_CONFIG(sgemm, float, float, 64, 64, 16, 2, 2, 4)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternatives: no epilogue variants
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 128, 16, 2, 2, 3)
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 256, 16, 2, 2, 3)
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 256, 16, 2, 2, 4)
DOCC_AGEMM_CONFIG(sgemm, float, float, 128, 256, 32, 2, 2, 3)
DOCC_AGEMM_CONFIG(sgemm, float, float, 64, 64, 32, 2, 2, 3)
DOCC_AGEMM_SPREAD_CONFIG(sgemm, float, float, 128, 256, 32, 2, 2, 3)   // copies dealt over the K-step: 2-3 % slower here
#endif

#ifndef DOCC_GEMM_EPILOGUE
// C = beta * C (the k == 0 case); beta == 0 stores zeros without reading C.
extern "C" __global__ __launch_bounds__(256) void docc_sgemm_scale_c(float* C, long M, long N, long ldc, float beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        float* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.f) ? 0.f : beta * (*p);
    }
}
// The end of a product whose K extent was cut into `splits` parts (each part's product in P[z], an m x n matrix of its
// own): C = alpha * (P[0] + P[1] + ...) + beta * C, the parts added in order; beta == 0 does not read C.
extern "C" __global__ __launch_bounds__(256) void docc_splitk_combine_f32(const float* __restrict__ P, float* __restrict__ C, long M, long N,
                                                                         long ldc, int splits, float alpha, float beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        float sum = P[i];
        for (int z = 1; z < splits; z++) sum += P[(long) z * total + i];
        float* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.f) ? alpha * sum : alpha * sum + beta * (*p);
    }
}
#endif
