// The kernels of gemm_f32_big.hip with C = act(alpha A B + beta C + bias[column]) in their store
// (names with the suffix "_e"). Kept apart from the plain kernels so that those carry none of
// the activation code.
#define DOCC_GEMM_EPILOGUE 1
#include "gemm_f32_big.hip"
