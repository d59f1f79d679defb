// fp64 GEMM kernels (v_mfma_f64_16x16x4_f64), see gemm_mfma.h.
#include "gemm_async.h"

DOCC_GEMM_CONFIG(dgemm, double, 64, 64, 16, 2, 2)
DOCC_GEMM_CONFIG(dgemm, double, 128, 128, 16, 2, 2)

// asynchronous multi-stage pipeline (aligned operands)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 64, 16, 2, 2, 2)
#endif
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 64, 16, 2, 2, 4)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 64, 16, 2, 2, 6)
#endif
DOCC_AGEMM_CONFIG(dgemm, double, double, 128, 128, 16, 2, 2, 3)
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 32, 16, 2, 2, 4)
#ifndef DOCC_GEMM_EPILOGUE   // tuning alternative: no epilogue variant
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 32, 32, 2, 2, 3)
DOCC_AGEMM_CONFIG(dgemm, double, double, 64, 64, 32, 2, 2, 3)
DOCC_AGEMM_SPREAD_CONFIG(dgemm, double, double, 64, 32, 16, 2, 2, 4)   // copies dealt over the K-step: no difference here
#endif

#ifndef DOCC_GEMM_EPILOGUE
extern "C" __global__ __launch_bounds__(256) void docc_dgemm_scale_c(double* C, long M, long N, long ldc, double beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        double* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.0) ? 0.0 : beta * (*p);
    }
}
// The end of a product whose K extent was cut into `splits` parts (each part's product in P[z], an m x n matrix of its
// own): C = alpha * (P[0] + P[1] + ...) + beta * C, the parts added in order; beta == 0 does not read C.
extern "C" __global__ __launch_bounds__(256) void docc_splitk_combine_f64(const double* __restrict__ P, double* __restrict__ C, long M, long N,
                                                                         long ldc, int splits, double alpha, double beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        double sum = P[i];
        for (int z = 1; z < splits; z++) sum += P[(long) z * total + i];
        double* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.0) ? alpha * sum : alpha * sum + beta * (*p);
    }
}
#endif
