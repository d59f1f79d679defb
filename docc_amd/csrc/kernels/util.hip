// Small utility kernels: calibration copy and fp32 <-> bf16 conversion.
#include "common.h"

using namespace docc_k;

// Plain 128-bit copy of n16 16-byte words: the known-size kernel used to
// calibrate the FETCH_SIZE / WRITE_SIZE counters.
extern "C" __global__ __launch_bounds__(256) void docc_copy_b128(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                   long n16) {
    long i = (long) blockIdx.x * 256 + threadIdx.x;
    const long stride = (long) gridDim.x * 256;
    for (; i < n16; i += stride) dst[i] = src[i];
}

extern "C" __global__ __launch_bounds__(256) void docc_f32_to_bf16(const float* __restrict__ src,
                                                                     uint16_t* __restrict__ dst, long n) {
    long i = (long) blockIdx.x * 256 + threadIdx.x;
    const long stride = (long) gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = f32_to_bf16_rne(src[i]);
}

extern "C" __global__ __launch_bounds__(256) void docc_bf16_to_f32(const uint16_t* __restrict__ src,
                                                                     float* __restrict__ dst, long n) {
    long i = (long) blockIdx.x * 256 + threadIdx.x;
    const long stride = (long) gridDim.x * 256;
    for (; i < n; i += stride) dst[i] = bf16_bits_to_f32(src[i]);
}
