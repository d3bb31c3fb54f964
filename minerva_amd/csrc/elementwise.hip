// Elementwise, scalar, unary, activation, copy and fill entry points.
// All are single-pass HBM streams (stream_kernels.h); the functors below are the
// whole arithmetic.  add/sub/mul/div, the scalar ops, neg, relu and the relu
// gradient are one IEEE operation or a selection per element, so they reproduce
// the CPU implementation (reference minerva/op/impl/basic.cpp:23-148,406-448) bit
// for bit; exp/ln/sigmoid/tanh go through the device math library.
#include "stream_kernels.h"

namespace {

struct OpAdd { __device__ float operator()(float a, float b) const { return a + b; } };
struct OpSub { __device__ float operator()(float a, float b) const { return a - b; } };
struct OpMul { __device__ float operator()(float a, float b) const { return a * b; } };
struct OpDiv { __device__ float operator()(float a, float b) const { return a / b; } };

struct OpConstAdd  { float v; __device__ float operator()(float x, float) const { return x + v; } };
struct OpConstSub  { float v; __device__ float operator()(float x, float) const { return x - v; } };
struct OpConstRsub { float v; __device__ float operator()(float x, float) const { return v - x; } };
struct OpConstMul  { float v; __device__ float operator()(float x, float) const { return x * v; } };
struct OpConstDiv  { float v; __device__ float operator()(float x, float) const { return x / v; } };
struct OpConstRdiv { float v; __device__ float operator()(float x, float) const { return v / x; } };

struct OpExp { __device__ float operator()(float x, float) const { return expf(x); } };
struct OpLn  { __device__ float operator()(float x, float) const { return logf(x); } };
struct OpNeg { __device__ float operator()(float x, float) const { return -x; } };
// basic.cpp:116-122, the operations as written there (|x| / x is exactly +-1)
struct OpThresholdNorm {
  float t;
  __device__ float operator()(float x, float) const { return fabsf(x) > t ? fabsf(x) / x * t : x; }
};
struct OpCopy { __device__ float operator()(float x, float) const { return x; } };
struct OpFill { float v; __device__ float operator()(float, float) const { return v; } };

// basic.cpp:416 evaluates 1.0 / (1.0 + expf(-x)) in double and rounds once.
struct OpSigmoid {
  __device__ float operator()(float x, float) const {
    return (float)(1.0 / (1.0 + (double)expf(-x)));
  }
};
struct OpRelu { __device__ float operator()(float x, float) const { return x > 0.f ? x : 0.f; } };
struct OpTanh { __device__ float operator()(float x, float) const { return tanhf(x); } };

// Backward activations, cuDNN v2 semantics behind cuda_perform.cu:444-487.
// (y, dy) -> dy*y*(1-y)
struct OpSigmoidBwd {
  __device__ float operator()(float y, float dy) const { return dy * y * (1.0f - y); }
};
// (x, dy) -> x > 0 ? dy : 0
struct OpReluBwd {
  __device__ float operator()(float x, float dy) const { return x > 0.f ? dy : 0.f; }
};
// (y, dy) -> dy*(1-y*y)
struct OpTanhBwd {
  __device__ float operator()(float y, float dy) const { return dy * (1.0f - y * y); }
};

// (w, g) -> w - v*g: the product is rounded, then the difference, as the scalar multiply
// followed by the subtraction round (the library is built without contraction into fma)
struct OpSgd {
  float v;
  __device__ float operator()(float w, float g) const {
    const float step = g * v;
    return w - step;
  }
};

}  // namespace

extern "C" {

int mnv_add(const float* a, const float* b, float* c, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpAdd, 2>(a, b, c, n, OpAdd(), s);
}
int mnv_sub(const float* a, const float* b, float* c, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpSub, 2>(a, b, c, n, OpSub(), s);
}
int mnv_mul(const float* a, const float* b, float* c, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpMul, 2>(a, b, c, n, OpMul(), s);
}
int mnv_div(const float* a, const float* b, float* c, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpDiv, 2>(a, b, c, n, OpDiv(), s);
}

int mnv_const_add(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstAdd, 1>(x, nullptr, y, n, OpConstAdd{v}, s);
}
int mnv_const_sub(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstSub, 1>(x, nullptr, y, n, OpConstSub{v}, s);
}
int mnv_const_rsub(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstRsub, 1>(x, nullptr, y, n, OpConstRsub{v}, s);
}
int mnv_const_mul(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstMul, 1>(x, nullptr, y, n, OpConstMul{v}, s);
}
int mnv_const_div(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstDiv, 1>(x, nullptr, y, n, OpConstDiv{v}, s);
}
int mnv_const_rdiv(const float* x, float* y, float v, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpConstRdiv, 1>(x, nullptr, y, n, OpConstRdiv{v}, s);
}

int mnv_exp(const float* x, float* y, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpExp, 1>(x, nullptr, y, n, OpExp(), s);
}
int mnv_ln(const float* x, float* y, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpLn, 1>(x, nullptr, y, n, OpLn(), s);
}
int mnv_neg(const float* x, float* y, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpNeg, 1>(x, nullptr, y, n, OpNeg(), s);
}

int mnv_threshold_norm(const float* x, float* y, float threshold, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpThresholdNorm, 1>(x, nullptr, y, n, OpThresholdNorm{threshold}, s);
}
int mnv_copy(const float* in, float* out, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpCopy, 1>(in, nullptr, out, n, OpCopy(), s);
}
int mnv_fill(float* dst, size_t n, float v, mnv_stream_t s) {
  return mnv_stream_launch<OpFill, 0>(nullptr, nullptr, dst, n, OpFill{v}, s);
}

int mnv_sgd_update(const float* w, const float* g, float scale, float* w_out, size_t n,
                   mnv_stream_t s) {
  return mnv_stream_launch<OpSgd, 2>(w, g, w_out, n, OpSgd{scale}, s);
}

int mnv_sigmoid_fwd(const float* bottom, float* top, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpSigmoid, 1>(bottom, nullptr, top, n, OpSigmoid(), s);
}
int mnv_relu_fwd(const float* bottom, float* top, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpRelu, 1>(bottom, nullptr, top, n, OpRelu(), s);
}
int mnv_tanh_fwd(const float* bottom, float* top, size_t n, mnv_stream_t s) {
  return mnv_stream_launch<OpTanh, 1>(bottom, nullptr, top, n, OpTanh(), s);
}

int mnv_sigmoid_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, size_t n, mnv_stream_t s) {
  (void)bottom;  // the sigmoid gradient needs only the output
  return mnv_stream_launch<OpSigmoidBwd, 2>(top, top_diff, bottom_diff, n, OpSigmoidBwd(), s);
}
int mnv_relu_bwd(const float* bottom, const float* top, const float* top_diff,
                 float* bottom_diff, size_t n, mnv_stream_t s) {
  (void)top;  // cuDNN's relu gradient tests the input
  return mnv_stream_launch<OpReluBwd, 2>(bottom, top_diff, bottom_diff, n, OpReluBwd(), s);
}
int mnv_tanh_bwd(const float* bottom, const float* top, const float* top_diff,
                 float* bottom_diff, size_t n, mnv_stream_t s) {
  (void)bottom;
  return mnv_stream_launch<OpTanhBwd, 2>(top, top_diff, bottom_diff, n, OpTanhBwd(), s);
}

}  // extern "C"
