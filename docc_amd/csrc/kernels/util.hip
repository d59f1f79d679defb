// Small utility kernels: calibration copy, MFMA rate probes and fp32 <-> bf16 conversion.
#include "common.h"

using namespace docc_k;

// 128-bit copy of n16 16-byte words: the known-size kernel used to calibrate the FETCH_SIZE / WRITE_SIZE
// counters and the streaming rate other HBM-bound kernels are held against. Non-temporal on both sides: on
// buffers that are not touched again (1 GiB walked in turn) a 128 MiB copy takes 42.3 us (6.35 TB/s) that way,
// 46.6 us with ordinary loads and stores, 44.0-44.8 us with ordinary loads and nt / sc1 stores.
// One work-group moves 16 KiB (four vectors per lane, all loaded before the first store).
extern "C" __global__ __launch_bounds__(256) void docc_copy_b128(const u32x4* __restrict__ src, u32x4* __restrict__ dst,
                                                                   long n16) {
    const long base = (long) blockIdx.x * 1024 + threadIdx.x;
    if (base + 768 < n16) {
        u32x4 v[4];
#pragma unroll
        for (int i = 0; i < 4; i++) v[i] = __builtin_nontemporal_load(src + base + 256 * i);
#pragma unroll
        for (int i = 0; i < 4; i++) __builtin_nontemporal_store(v[i], dst + base + 256 * i);
    } else {
        for (long i = base; i < n16 && i < base + 1024; i += 256) __builtin_nontemporal_store(__builtin_nontemporal_load(src + i), dst + i);
    }
}

// Byte fill, what hipMemsetAsync does, as a kernel: a memset recorded into a HIP graph is a node of its own kind,
// a kernel is a kernel. Bytes up to the first 16-byte boundary and after the last one are written singly (by the
// first work-group), the rest as 16-byte vectors.
extern "C" __global__ __launch_bounds__(256) void docc_fill_b8(uint8_t* __restrict__ dst, int value, long n) {
    const uint8_t b = (uint8_t) value;
    long head = (long) ((16 - ((uintptr_t) dst & 15)) & 15);
    if (head > n) head = n;
    const long n16 = (n - head) / 16;
    const long tail = head + n16 * 16;
    if (blockIdx.x == 0) {
        for (long i = threadIdx.x; i < head; i += 256) dst[i] = b;
        for (long i = tail + threadIdx.x; i < n; i += 256) dst[i] = b;
    }
    const uint32_t w = 0x01010101u * b;
    const u32x4 v = {w, w, w, w};
    u32x4* body = (u32x4*) (dst + head);
    const long stride = (long) gridDim.x * 256;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < n16; i += stride) body[i] = v;
}

// Rows of `d` 16-bit elements copied into rows of `dp` >= d (a multiple of 8), the rest of each row cleared: attention
// operands of a head dimension that is not built, widened to one that is. One 16-byte piece of the result per lane.
extern "C" __global__ __launch_bounds__(256) void docc_pad_rows_b16(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst,
                                                                      long rows, int d, int dp) {
    const int per_row = dp >> 3;
    const long pieces = rows * per_row;
    const long stride = (long) gridDim.x * 256;
    for (long p = (long) blockIdx.x * 256 + threadIdx.x; p < pieces; p += stride) {
        const long row = p / per_row;
        const int c0 = (int) (p % per_row) * 8;
        const uint16_t* from = src + row * d + c0;
        u32x4 out;
        if ((d & 7) == 0 && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {   // whole pieces on both sides
            out = c0 < d ? *reinterpret_cast<const u32x4*>(from) : u32x4{0u, 0u, 0u, 0u};
            *reinterpret_cast<u32x4*>(dst + row * dp + c0) = out;
            continue;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = c0 + 2 * i < d ? from[2 * i] : 0u;
            const uint32_t hi = c0 + 2 * i + 1 < d ? from[2 * i + 1] : 0u;
            out[i] = lo | (hi << 16);
        }
        *reinterpret_cast<u32x4*>(dst + row * dp + c0) = out;
    }
}

// The first `d` elements of rows of `dp` elements, packed: the result of the widened attention, narrowed again.
// WORD = uint16_t (bf16 result) or uint32_t (fp32 result).
template <typename WORD>
__device__ __forceinline__ void unpad_rows(const WORD* __restrict__ src, WORD* __restrict__ dst, long rows, int d, int dp) {
    const long stride = (long) gridDim.x * 256;
    constexpr int PER = 16 / sizeof(WORD);
    if (d % PER == 0 && dp % PER == 0 && ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 15) == 0) {
        // rows of whole 16-byte pieces on both sides
        const int per_row = d / PER;
        const long pieces = rows * per_row;
        for (long p = (long) blockIdx.x * 256 + threadIdx.x; p < pieces; p += stride)
            reinterpret_cast<u32x4*>(dst)[p] = *reinterpret_cast<const u32x4*>(src + (p / per_row) * dp + (p % per_row) * PER);
        return;
    }
    const long n = rows * d;
    for (long i = (long) blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = src[(i / d) * dp + i % d];
}
extern "C" __global__ __launch_bounds__(256) void docc_unpad_rows_b16(const uint16_t* src, uint16_t* dst, long rows, int d, int dp) {
    unpad_rows(src, dst, rows, d, dp);
}
extern "C" __global__ __launch_bounds__(256) void docc_unpad_rows_b32(const uint32_t* src, uint32_t* dst, long rows, int d, int dp) {
    unpad_rows(src, dst, rows, d, dp);
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

// Shader clock observed over `ticks` ticks of the constant 100 MHz counter (s_memrealtime) by one wave that does
// nothing but sleep and look at that counter: launched on a stream of its own next to a train of kernels, it
// gives the clock the device sustains under them. out[0] = MHz. The wait is bounded twice over (ticks, and a
// cap on the number of looks), so the wave always ends.
extern "C" __global__ __launch_bounds__(64) void docc_clock_probe(float* __restrict__ out, long ticks) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const long r0 = (long) __builtin_amdgcn_s_memrealtime();
    const long c0 = (long) __builtin_readcyclecounter();
    long r1 = r0;
    for (int looks = 0; looks < (1 << 20) && r1 - r0 < ticks; looks++) {
        __builtin_amdgcn_s_sleep(16);
        r1 = (long) __builtin_amdgcn_s_memrealtime();
    }
    const long c1 = (long) __builtin_readcyclecounter();
    out[0] = r1 > r0 ? (float) ((double) (c1 - c0) / (double) (r1 - r0) * 100.0) : 0.f;
}

// MFMA rate probes: `iters` rounds of 32 back-to-back MFMAs per wave on operands taken from
// `operands` (4096 floats; random values make the multipliers toggle as they do in a real GEMM,
// zeros do not), four accumulators, eight operand register sets in rotation. They measure what the
// power limit leaves of the nominal matrix peak on the device at hand - the ceiling a GEMM-shaped
// kernel can reach with that data. One wave per SIMD per work-group; launch 2 per CU for two.
typedef float probe_f32x16 __attribute__((ext_vector_type(16)));
typedef double probe_f64x4 __attribute__((ext_vector_type(4)));
typedef float probe_f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 probe_bf16x8 __attribute__((ext_vector_type(8)));

// Every index below is a compile-time constant once the loops are unrolled, so the operand sets live in
// registers and the set-up is sixteen loads: with run-time indices the compiler builds the sets one lane
// at a time, which costs as much as thousands of rounds and is then counted as matrix time. The MFMAs are
// written as asm with the accumulators held in VGPRs: left to itself the compiler keeps them in AGPRs and,
// for the fp64 loop, copies them across and back every round.
extern "C" __global__ __launch_bounds__(256) void docc_mfma_probe_f64(const float* __restrict__ operands, float* __restrict__ sink, int iters) {
    probe_f64x4 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = {0, 0, 0, 0};
    double a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = operands[(threadIdx.x * 8 + i) & 4095];
        b[i] = operands[(threadIdx.x * 8 + i + 2048) & 4095];
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("v_mfma_f64_16x16x4_f64 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[(s + i) & 7]), "v"(b[s]));
    }
    double r = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) r += acc[i][0] + acc[i][3];
    sink[blockIdx.x * 256 + threadIdx.x] = (float) r;
}

extern "C" __global__ __launch_bounds__(256) void docc_mfma_probe_f32(const float* __restrict__ operands, float* __restrict__ sink, int iters) {
    probe_f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    float a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = operands[(threadIdx.x * 8 + i) & 4095];
        b[i] = operands[(threadIdx.x * 8 + i + 2048) & 4095];
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("v_mfma_f32_32x32x2_f32 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[(s + i) & 7]), "v"(b[s]));
    }
    float r = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) r += acc[i][0] + acc[i][15];
    sink[blockIdx.x * 256 + threadIdx.x] = r;
}

extern "C" __global__ __launch_bounds__(256) void docc_mfma_probe_bf16(const float* __restrict__ operands, float* __restrict__ sink, int iters) {
    probe_f32x16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0;
    // each lane's eight operand sets: 64 consecutive table entries (a), the 64 of the lane 28 further on (b)
    const float4* row_a = reinterpret_cast<const float4*>(operands + ((threadIdx.x * 64) & 4095));
    const float4* row_b = reinterpret_cast<const float4*>(operands + ((threadIdx.x * 64 + 1792) & 4095));
    probe_bf16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 a0 = row_a[2 * i], a1 = row_a[2 * i + 1], b0 = row_b[2 * i], b1 = row_b[2 * i + 1];
        a[i] = probe_bf16x8{(__bf16) a0.x, (__bf16) a0.y, (__bf16) a0.z, (__bf16) a0.w, (__bf16) a1.x, (__bf16) a1.y, (__bf16) a1.z, (__bf16) a1.w};
        b[i] = probe_bf16x8{(__bf16) b0.x, (__bf16) b0.y, (__bf16) b0.z, (__bf16) b0.w, (__bf16) b1.x, (__bf16) b1.y, (__bf16) b1.z, (__bf16) b1.w};
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[(s + i) & 7]), "v"(b[s]));
    }
    float r = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) r += acc[i][0] + acc[i][15];
    sink[blockIdx.x * 256 + threadIdx.x] = r;
}

// the same on the other form of the bf16 instruction: a quarter of the output tile, twice the k
extern "C" __global__ __launch_bounds__(256) void docc_mfma_probe_bf16_16x16x32(const float* __restrict__ operands, float* __restrict__ sink, int iters) {
    probe_f32x4 acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = {0, 0, 0, 0};
    // each lane's eight operand sets: 64 consecutive table entries (a), the 64 of the lane 28 further on (b)
    const float4* row_a = reinterpret_cast<const float4*>(operands + ((threadIdx.x * 64) & 4095));
    const float4* row_b = reinterpret_cast<const float4*>(operands + ((threadIdx.x * 64 + 1792) & 4095));
    probe_bf16x8 a[8], b[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const float4 a0 = row_a[2 * i], a1 = row_a[2 * i + 1], b0 = row_b[2 * i], b1 = row_b[2 * i + 1];
        a[i] = probe_bf16x8{(__bf16) a0.x, (__bf16) a0.y, (__bf16) a0.z, (__bf16) a0.w, (__bf16) a1.x, (__bf16) a1.y, (__bf16) a1.z, (__bf16) a1.w};
        b[i] = probe_bf16x8{(__bf16) b0.x, (__bf16) b0.y, (__bf16) b0.z, (__bf16) b0.w, (__bf16) b1.x, (__bf16) b1.y, (__bf16) b1.z, (__bf16) b1.w};
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int s = 0; s < 8; s++)
#pragma unroll
            for (int i = 0; i < 4; i++) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a[(s + i) & 7]), "v"(b[s]));
    }
    float r = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) r += acc[i][0] + acc[i][3];
    sink[blockIdx.x * 256 + threadIdx.x] = r;
}
