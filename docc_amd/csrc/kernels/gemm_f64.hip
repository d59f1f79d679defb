// fp64 GEMM kernels (v_mfma_f64_16x16x4_f64), see gemm_mfma.h.
#include "gemm_mfma.h"

DOCC_GEMM_CONFIG(dgemm, double, 64, 64, 16, 2, 2)
DOCC_GEMM_CONFIG(dgemm, double, 128, 128, 16, 2, 2)
DOCC_GEMM_CONFIG(dgemm, double, 64, 64, 32, 2, 2)
DOCC_GEMM_CONFIG(dgemm, double, 64, 64, 64, 2, 2)

extern "C" __global__ __launch_bounds__(256) void docc_dgemm_scale_c(double* C, long M, long N, long ldc, double beta) {
    const long total = M * N;
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < total; i += stride) {
        double* p = C + (i / N) * ldc + (i % N);
        *p = (beta == 0.0) ? 0.0 : beta * (*p);
    }
}
