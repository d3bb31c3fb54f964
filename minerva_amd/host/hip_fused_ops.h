// Fused operators: an opt-in fast path beside the reference's operator set, never a
// replacement for it.  The reference launches every operator by itself: a convolution, then
// AddTensor for its bias (minerva/op/impl/cuda/cuda_perform.cu:227-264), and its
// applications follow each convolution / inner product with a ReLU, each gradient with the
// ReLU gradient, and update with a scalar multiply and a subtraction
// (owl/apps/imagenet_alexnet/alexnet.py:73-126, apps/mnist_common.h:185-197).  Each operator
// here performs one such pair in the store of the producing kernel and returns exactly the
// bits of the pair.  Closures and functions follow the conventions of the reference's
// (DataList inputs, DataList outputs, closure, context).
#pragma once
#include "minerva_types.h"

namespace minerva {

// top = relu(conv(bottom, filter) + bias); inputs {bottom, filter, bias}
struct ConvForwardReluClosure {
  int pad_height, pad_width, stride_vertical, stride_horizontal;
};
// bottom_diff = relu_backward(conv_backward_data(top_diff, filter), bottom);
// inputs {top_diff, filter, bottom}: `bottom` is the convolution's input, itself a ReLU output
struct ConvBackwardDataReluClosure {
  int pad_height, pad_width, stride_vertical, stride_horizontal;
};
// bottom_diff = relu_backward(max_pooling_backward(top_diff, top, bottom), bottom);
// inputs {top_diff, top, bottom}
struct PoolingBackwardReluClosure {
  int height, width, stride_vertical, stride_horizontal, pad_height, pad_width;
};
// out = [relu](a * b + bias), bias {m,1} replicated along dimension 1; inputs {a, b, bias}
struct MatMultBiasClosure {
  bool relu;
};
// out = relu_backward(a * b, bottom); inputs {a, b, bottom}
struct MatMultReluBackwardClosure {};
// out = a^T * b, a given as {k,m}; with three inputs {a, b, bottom} the product is gated like
// MatMultReluBackward: the pair Transpose(a), MatMult[ReluBackward] of an inner product's
// data gradient
struct MatMultTransAClosure {};
// out = a * b^T, b given as {n,k}: Transpose(b), MatMult -- an inner product's weight gradient
struct MatMultTransBClosure {};
// out = w - scale * g; inputs {w, g}
struct SgdUpdateClosure {
  float scale;
};
// out = w - scale * (a * b^T), b given as {n,k}; inputs {a, b, w}: MatMultTransB, then SgdUpdate,
// with the gradient never stored
struct MatMultTransBSgdClosure {
  float scale;
};
// out = filter - scale * conv_backward_filter(top_diff, bottom); inputs {top_diff, bottom, filter}
struct ConvBackwardFilterSgdClosure {
  int pad_height, pad_width, stride_vertical, stride_horizontal;
  float scale;
};

namespace hip {

void ConvForwardRelu(const DataList&, const DataList&, ConvForwardReluClosure&, const Context&);
void ConvBackwardDataRelu(const DataList&, const DataList&, ConvBackwardDataReluClosure&,
                          const Context&);
void PoolingBackwardRelu(const DataList&, const DataList&, PoolingBackwardReluClosure&,
                         const Context&);
void MatMultBias(const DataList&, const DataList&, MatMultBiasClosure&, const Context&);
void MatMultReluBackward(const DataList&, const DataList&, MatMultReluBackwardClosure&,
                         const Context&);
void MatMultTransA(const DataList&, const DataList&, MatMultTransAClosure&, const Context&);
void MatMultTransB(const DataList&, const DataList&, MatMultTransBClosure&, const Context&);
void SgdUpdate(const DataList&, const DataList&, SgdUpdateClosure&, const Context&);
void MatMultTransBSgd(const DataList&, const DataList&, MatMultTransBSgdClosure&, const Context&);
void ConvBackwardFilterSgd(const DataList&, const DataList&, ConvBackwardFilterSgdClosure&,
                           const Context&);

}  // namespace hip
}  // namespace minerva
