// Row softmax over the last axis, fp32, for gfx950.
//
// Replaces the seven loop nests SoftmaxNode::expand produces (reference
// sdfg/src/data_flow/library_nodes/math/tensor/reduce_ops/softmax_node.cpp:142-252:
// Max -> Broadcast -> Sub -> Exp -> Sum -> Broadcast -> Div with six
// temporaries) by one kernel that reads X once and writes Y once.
//
// HBM-bound: algorithmic traffic is 8 bytes per element. Three shapes:
//   wave-per-row  (cols <= 1024, cols % 4 == 0; built up to 4096): a 64-lane wavefront
//       holds the whole row in registers (NV float4 per lane, 128-bit coalesced loads),
//       reduces max and sum with wave shuffles only - no LDS, no barrier;
//   block-per-row (cols <= 16384, cols % 4 == 0): 256 threads hold the row,
//       partial results cross the four waves through LDS; ahead of the wavefront
//       per row from 2048 columns on (more rows in flight per register); rows of
//       2049..4096 columns use 512 threads (two vectors per lane), the others 256;
//   streaming     (any cols): per-lane online max/sum over the row, then a
//       second read (served by L2 / Infinity Cache) to write the result.
#include "common.h"

using namespace docc_k;

namespace {

constexpr float kNegInf = -__builtin_huge_valf();

template <int NV>
__device__ __forceinline__ void softmax_row_wave(const float* __restrict__ x, float* __restrict__ y, int cols, int lane) {
    const int nvec = cols >> 2;
    const f32x4* xv = reinterpret_cast<const f32x4*>(x);
    f32x4* yv = reinterpret_cast<f32x4*>(y);
    f32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = lane + i * kWave;
        if (c < nvec) {
            v[i] = __builtin_nontemporal_load(xv + c);
        } else {
            v[i] = f32x4{kNegInf, kNegInf, kNegInf, kNegInf};
        }
    }
    float m = kNegInf;
#pragma unroll
    for (int i = 0; i < NV; i++) m = fmaxf(fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)), m);
    m = wave_max(m);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        v[i].x = exp_neg(v[i].x - m);
        v[i].y = exp_neg(v[i].y - m);
        v[i].z = exp_neg(v[i].z - m);
        v[i].w = exp_neg(v[i].w - m);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    s = wave_sum(s);
    // one IEEE division per row, then multiplies: within 1 ulp of the
    // element-wise division the reference's Div node performs
    const float inv = 1.0f / s;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = lane + i * kWave;
        if (c < nvec) {
            f32x4 o = v[i] * inv;
            __builtin_nontemporal_store(o, yv + c);
        }
    }
}

template <int NV>
__device__ __forceinline__ void softmax_wave_kernel(const float* X, float* Y, long rows, int cols) {
    const int lane = threadIdx.x & (kWave - 1);
    const long row = (long) blockIdx.x * (blockDim.x / kWave) + (threadIdx.x / kWave);
    if (row >= rows) return;
    softmax_row_wave<NV>(X + row * (long) cols, Y + row * (long) cols, cols, lane);
}

// block reductions across the NW waves of a work-group
template <int NW = 4>
__device__ __forceinline__ float block_max(float v, float* lds) {
    v = wave_max(v);
    const int w = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[w] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r = fmaxf(r, lds[i]);
    __syncthreads();
    return r;
}

template <int NW = 4>
__device__ __forceinline__ float block_sum(float v, float* lds) {
    v = wave_sum(v);
    const int w = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[w] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int i = 1; i < NW; i++) r += lds[i];
    __syncthreads();
    return r;
}

template <int NV, int NW = 4>
__device__ __forceinline__ void softmax_block_kernel(const float* X, float* Y, long rows, int cols) {
    constexpr int NT = NW * kWave;
    __shared__ float lds[NW];
    const long row = blockIdx.x;
    const int nvec = cols >> 2;
    const f32x4* xv = reinterpret_cast<const f32x4*>(X + row * (long) cols);
    f32x4* yv = reinterpret_cast<f32x4*>(Y + row * (long) cols);
    f32x4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = threadIdx.x + i * NT;
        if (c < nvec) {
            v[i] = __builtin_nontemporal_load(xv + c);
        } else {
            v[i] = f32x4{kNegInf, kNegInf, kNegInf, kNegInf};
        }
    }
    float m = kNegInf;
#pragma unroll
    for (int i = 0; i < NV; i++) m = fmaxf(fmaxf(fmaxf(v[i].x, v[i].y), fmaxf(v[i].z, v[i].w)), m);
    m = block_max<NW>(m, lds);
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        v[i].x = exp_neg(v[i].x - m);
        v[i].y = exp_neg(v[i].y - m);
        v[i].z = exp_neg(v[i].z - m);
        v[i].w = exp_neg(v[i].w - m);
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    s = block_sum<NW>(s, lds);
    const float inv = 1.0f / s;
#pragma unroll
    for (int i = 0; i < NV; i++) {
        int c = threadIdx.x + i * NT;
        if (c < nvec) {
            f32x4 o = v[i] * inv;
            __builtin_nontemporal_store(o, yv + c);
        }
    }
}

} // namespace

#define DOCC_SOFTMAX_WAVE(NV)                                                                             \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_f32_wave_v##NV(const float* X, float* Y, \
                                                                                  long rows, int cols) {  \
        softmax_wave_kernel<NV>(X, Y, rows, cols);                                                        \
    }
DOCC_SOFTMAX_WAVE(1)
DOCC_SOFTMAX_WAVE(2)
DOCC_SOFTMAX_WAVE(4)
DOCC_SOFTMAX_WAVE(8)
DOCC_SOFTMAX_WAVE(16)

#define DOCC_SOFTMAX_BLOCK(NV)                                                                             \
    extern "C" __global__ __launch_bounds__(256) void docc_softmax_f32_block_v##NV(const float* X, float* Y, \
                                                                                   long rows, int cols) {  \
        softmax_block_kernel<NV>(X, Y, rows, cols);                                                        \
    }
// eight wavefronts per row
#define DOCC_SOFTMAX_BLOCK8(NV)                                                                             \
    extern "C" __global__ __launch_bounds__(512) void docc_softmax_f32_block8_v##NV(const float* X, float* Y, \
                                                                                    long rows, int cols) {  \
        softmax_block_kernel<NV, 8>(X, Y, rows, cols);                                                      \
    }
DOCC_SOFTMAX_BLOCK8(2)
DOCC_SOFTMAX_BLOCK(1)
DOCC_SOFTMAX_BLOCK(2)
DOCC_SOFTMAX_BLOCK(4)
DOCC_SOFTMAX_BLOCK(8)
DOCC_SOFTMAX_BLOCK(16)

// Any cols, any alignment: one 256-thread block per row. Pass 1 keeps a
// per-thread running (max, sum) pair that is rescaled whenever the max moves
// (online softmax); the pairs are merged across the block; pass 2 re-reads the
// row and writes exp(x - max) / sum.
extern "C" __global__ __launch_bounds__(256) void docc_softmax_f32_stream(const float* X, float* Y, long rows,
                                                                            long cols) {
    __shared__ float lds[4];
    const long row = blockIdx.x;
    const float* x = X + row * cols;
    float* y = Y + row * cols;
    float m = kNegInf, s = 0.f;
    for (long c = threadIdx.x; c < cols; c += 256) {
        float v = x[c];
        if (v > m) {
            s = s * exp_neg(m - v) + 1.0f; // m == -inf: s is 0 and exp(-inf) is 0
            m = v;
        } else {
            s += exp_neg(v - m);
        }
    }
    float gm = block_max(m, lds);
    // a thread that saw no element has m = -inf, s = 0: contributes 0
    float contrib = (m == kNegInf) ? 0.f : s * exp_neg(m - gm);
    float gs = block_sum(contrib, lds);
    const float inv = 1.0f / gs;
    for (long c = threadIdx.x; c < cols; c += 256) y[c] = exp_neg(x[c] - gm) * inv;
}
