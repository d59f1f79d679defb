// The elementwise operations of the tensor nodes, shared by the elementwise kernels and by the
// GEMM epilogue. Semantics follow the reference's expansions:
//   ReLU     fmax(x, 0.0)            elementwise_ops/relu_node.cpp:40-43
//   Sigmoid  1.0 / (1.0 + exp(-x))   elementwise_ops/sigmoid_node.cpp:46-70
//   Maximum / Minimum  fmax / fmin   elementwise_ops/maximum_node.cpp:64, minimum_node.cpp
//   Abs, Exp, Sqrt, Tanh, Erf        the libm function of the element type (cmath_node.h)
//   Add, Sub, Mul, Div               the IEEE operation
//   Pow      pow(a, b)               elementwise_ops/pow_node.cpp:52-54 (CMathFunction::pow)
// Activations with scalar operands ("alpha", "beta" connectors; elu_node.cpp:21, leaky_relu_node.cpp:21,
// hard_sigmoid_node.cpp:21-22). The reference's expansions of these three are unfinished (Elu has no branch for
// x > 0, LeakyReLU's multiply has one operand, HardSigmoid's fma has one), so the semantics are the ONNX
// operators the nodes are named after:
//   Elu          x > 0 ? x : alpha * (exp(x) - 1)          (the reference's exp, subtract 1, times alpha for x <= 0)
//   LeakyReLU    x >= 0 ? x : alpha * x
//   HardSigmoid  fmax(0, fmin(1, alpha * x + beta))        (the reference's fma, fmin(.., 1), fmax(.., 0) order)
#pragma once

#include "common.h"

namespace docc_k {

enum UnaryOp : int { kAbs = 0, kExp = 1, kReLU = 2, kSigmoid = 3, kSqrt = 4, kTanh = 5, kErf = 6 };
enum ParamUnaryOp : int { kElu = 7, kLeakyReLU = 8, kHardSigmoid = 9 };
enum BinaryOp : int { kAdd = 0, kSub = 1, kMul = 2, kDiv = 3, kMaximum = 4, kMinimum = 5, kPow = 6 };

template <int OP>
__device__ __forceinline__ float unary(float x) {
    if (OP == kAbs) return fabsf(x);
    if (OP == kExp) return expf(x);
    if (OP == kReLU) return fmaxf(x, 0.0f);
    if (OP == kSigmoid) return 1.0f / (1.0f + expf(-x));
    if (OP == kSqrt) return sqrtf(x);
    if (OP == kTanh) return tanhf(x);
    return erff(x);
}
template <int OP>
__device__ __forceinline__ double unary(double x) {
    if (OP == kAbs) return fabs(x);
    if (OP == kExp) return exp(x);
    if (OP == kReLU) return fmax(x, 0.0);
    if (OP == kSigmoid) return 1.0 / (1.0 + exp(-x));
    if (OP == kSqrt) return sqrt(x);
    if (OP == kTanh) return tanh(x);
    return erf(x);
}
template <int OP>
__device__ __forceinline__ float binary(float a, float b) {
    if (OP == kAdd) return a + b;
    if (OP == kSub) return a - b;
    if (OP == kMul) return a * b;
    if (OP == kDiv) return a / b;
    if (OP == kMaximum) return fmaxf(a, b);
    if (OP == kPow) return powf(a, b);
    return fminf(a, b);
}
template <int OP>
__device__ __forceinline__ double binary(double a, double b) {
    if (OP == kAdd) return a + b;
    if (OP == kSub) return a - b;
    if (OP == kMul) return a * b;
    if (OP == kDiv) return a / b;
    if (OP == kMaximum) return fmax(a, b);
    if (OP == kPow) return pow(a, b);
    return fmin(a, b);
}

template <int OP>
__device__ __forceinline__ float param_unary(float x, float alpha, float beta) {
    if (OP == kElu) return x > 0.0f ? x : alpha * (expf(x) - 1.0f);
    if (OP == kLeakyReLU) return x >= 0.0f ? x : alpha * x;
    return fmaxf(fminf(__builtin_fmaf(alpha, x, beta), 1.0f), 0.0f);
}
template <int OP>
__device__ __forceinline__ double param_unary(double x, double alpha, double beta) {
    if (OP == kElu) return x > 0.0 ? x : alpha * (exp(x) - 1.0);
    if (OP == kLeakyReLU) return x >= 0.0 ? x : alpha * x;
    return fmax(fmin(__builtin_fma(alpha, x, beta), 1.0), 0.0);
}

// operation chosen at run time; the code is uniform over a launch, so this is a scalar branch
template <typename T>
__device__ __forceinline__ T apply_unary(int op, T x) {
    switch (op) {
        case kAbs: return unary<kAbs>(x);
        case kExp: return unary<kExp>(x);
        case kReLU: return unary<kReLU>(x);
        case kSigmoid: return unary<kSigmoid>(x);
        case kSqrt: return unary<kSqrt>(x);
        case kTanh: return unary<kTanh>(x);
        default: return unary<kErf>(x);
    }
}

template <typename T>
__device__ __forceinline__ T apply_binary(int op, T a, T b) {
    switch (op) {
        case kAdd: return binary<kAdd>(a, b);
        case kSub: return binary<kSub>(a, b);
        case kMul: return binary<kMul>(a, b);
        case kDiv: return binary<kDiv>(a, b);
        case kMaximum: return binary<kMaximum>(a, b);
        case kPow: return binary<kPow>(a, b);
        default: return binary<kMinimum>(a, b);
    }
}

} // namespace docc_k
