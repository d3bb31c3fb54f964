#include "hip_ops.h"
#include "staged_copy.h"

#include <cstring>

#include <atomic>

#include "mnv_hip.h"

namespace minerva {
namespace hip {

namespace {

void Ok(int status, const char* what) {
  MNV_CHECK(status == MNV_OK) << what << ": " << mnv_error_string(status);
}

// Collapses an N-d extent around one dimension into the {m, n} matrix the library
// reduces or broadcasts over.  Dimension 0 is the contiguous one ("col" kernels);
// the last dimension is the strided one ("row" kernels).  The reference's GPU path
// only accepts 2-D (minerva/op/impl/cuda.cpp:222-223,268-269); higher ranks are
// accepted here when the dimension is the first or the last, and rejected otherwise.
struct Collapsed {
  bool on_first;
  int m, n;
};

Collapsed Collapse(const Scale& size, int dim, const char* what) {
  const int nd = static_cast<int>(size.NumDims());
  MNV_CHECK(nd >= 1 && dim >= 0 && dim < nd) << what << ": dimension out of range";
  long long total = size.Prod();
  Collapsed c;
  if (dim == 0) {
    c.on_first = true;
    c.m = size[0];
    c.n = static_cast<int>(total / size[0]);
  } else {
    MNV_CHECK(dim == nd - 1) << what << ": only the first or the last dimension is supported";
    c.on_first = false;
    c.n = size[nd - 1];
    c.m = static_cast<int>(total / size[nd - 1]);
  }
  return c;
}

}  // namespace

void Arithmetic(const DataList& inputs, const DataList& outputs, ArithmeticClosure& closure,
                const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "Arithmetic takes 2 inputs";
  MNV_CHECK_EQ(outputs.size(), 1u) << "Arithmetic takes 1 output";
  const float* l = inputs[0].data_;
  const float* r = inputs[1].data_;
  float* o = outputs[0].data_;
  size_t n = outputs[0].size_.Prod();
  switch (closure.type) {
    case ArithmeticType::kAdd: Ok(mnv_add(l, r, o, n, ctx.stream), "add"); break;
    case ArithmeticType::kSub: Ok(mnv_sub(l, r, o, n, ctx.stream), "sub"); break;
    case ArithmeticType::kMult: Ok(mnv_mul(l, r, o, n, ctx.stream), "mul"); break;
    case ArithmeticType::kDiv: Ok(mnv_div(l, r, o, n, ctx.stream), "div"); break;
  }
}

void ArithmeticConst(const DataList& inputs, const DataList& outputs,
                     ArithmeticConstClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(arithmetic const) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(arithmetic const) #outputs is wrong!";
  const float* x = inputs[0].data_;
  float* y = outputs[0].data_;
  const float v = closure.val;
  size_t n = inputs[0].size_.Prod();
  const bool left = closure.side == 0;
  switch (closure.type) {
    case ArithmeticType::kAdd: Ok(mnv_const_add(x, y, v, n, ctx.stream), "const add"); break;
    case ArithmeticType::kSub:
      Ok(left ? mnv_const_rsub(x, y, v, n, ctx.stream) : mnv_const_sub(x, y, v, n, ctx.stream),
         "const sub");
      break;
    case ArithmeticType::kMult: Ok(mnv_const_mul(x, y, v, n, ctx.stream), "const mul"); break;
    case ArithmeticType::kDiv:
      // x / v is a true division here, as on the CPU (basic.cpp:99-103); the CUDA path
      // multiplies by 1/v instead (cuda.cpp:196), which is not the same rounding.
      Ok(left ? mnv_const_rdiv(x, y, v, n, ctx.stream) : mnv_const_div(x, y, v, n, ctx.stream),
         "const div");
      break;
  }
}

void Elewise(const DataList& inputs, const DataList& outputs, ElewiseClosure& closure,
             const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(elewise) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(elewise) #outputs is wrong!";
  const float* x = inputs[0].data_;
  float* y = outputs[0].data_;
  size_t n = outputs[0].size_.Prod();
  switch (closure.type) {
    case ElewiseType::kExp: Ok(mnv_exp(x, y, n, ctx.stream), "exp"); break;
    case ElewiseType::kLn: Ok(mnv_ln(x, y, n, ctx.stream), "ln"); break;
    case ElewiseType::kNegative: Ok(mnv_neg(x, y, n, ctx.stream), "neg"); break;
    default: MNV_FATAL() << "elewise algorithm not supported";
  }
}

void MatMult(const DataList& inputs, const DataList& outputs, MatMultClosure&,
             const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(matmult) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(matmult) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int k = inputs[0].size_[1];
  int n = outputs[0].size_[1];
  MNV_CHECK_EQ(inputs[1].size_[0], k) << "(matmult) inner dimensions differ";
  Ok(mnv_sgemm_nn(inputs[0].data_, inputs[1].data_, outputs[0].data_, m, n, k, ctx.workspace,
                  ctx.workspace_bytes, ctx.stream),
     "sgemm");
}

void Transpose(const DataList& inputs, const DataList& outputs, TransposeClosure&,
               const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(transpose) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(transpose) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int n = inputs[0].size_[1];
  Ok(mnv_transpose(inputs[0].data_, outputs[0].data_, m, n, ctx.stream), "transpose");
}

void NormArithmetic(const DataList& inputs, const DataList& outputs,
                    NormArithmeticClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "NormArithmetic kernel wrong #input";
  MNV_CHECK_EQ(outputs.size(), 1u) << "NormArithmetic kernel wrong #output";
  MNV_CHECK_EQ(closure.dims_to_replicate.NumDims(), 1u)
      << "currently do norm on one dimension only";
  Collapsed c = Collapse(inputs[0].size_, closure.dims_to_replicate[0], "NormArithmetic");
  const float* mat = inputs[0].data_;
  const float* vec = inputs[1].data_;
  float* res = outputs[0].data_;
  int (*fn)(const float*, const float*, float*, int, int, mnv_stream_t) = nullptr;
  // replicated along dim 0 => the vector has one entry per column ("OnCol")
  switch (closure.type) {
    case ArithmeticType::kAdd: fn = c.on_first ? mnv_norm_add_col : mnv_norm_add_row; break;
    case ArithmeticType::kSub: fn = c.on_first ? mnv_norm_sub_col : mnv_norm_sub_row; break;
    case ArithmeticType::kMult: fn = c.on_first ? mnv_norm_mul_col : mnv_norm_mul_row; break;
    case ArithmeticType::kDiv: fn = c.on_first ? mnv_norm_div_col : mnv_norm_div_row; break;
  }
  Ok(fn(mat, vec, res, c.m, c.n, ctx.stream), "norm arithmetic");
}

void Reduction(const DataList& inputs, const DataList& outputs, ReductionClosure& closure,
               const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "Reduction kernel wrong #input";
  MNV_CHECK_EQ(outputs.size(), 1u) << "Reduction kernel wrong #output";
  MNV_CHECK_EQ(closure.dims_to_reduce.NumDims(), 1u)
      << "currently do reduction on one dimension only";
  Collapsed c = Collapse(inputs[0].size_, closure.dims_to_reduce[0], "Reduction");
  const float* in = inputs[0].data_;
  float* out = outputs[0].data_;
  const bool sum = closure.type == ReductionType::kSum;
  int rc = c.on_first ? (sum ? mnv_reduce_sum_col(in, out, c.m, c.n, ctx.stream)
                             : mnv_reduce_max_col(in, out, c.m, c.n, ctx.stream))
                      : (sum ? mnv_reduce_sum_row(in, out, c.m, c.n, ctx.stream)
                             : mnv_reduce_max_row(in, out, c.m, c.n, ctx.stream));
  Ok(rc, "reduction");
}

void MaxIndex(const DataList& inputs, const DataList& outputs, MaxIndexClosure& closure,
              const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "MaxIndex kernel wrong #input";
  MNV_CHECK_EQ(outputs.size(), 1u) << "MaxIndex kernel wrong #output";
  Collapsed c = Collapse(inputs[0].size_, closure.dim, "MaxIndex");
  int rc = c.on_first
               ? mnv_maxindex_col(inputs[0].data_, outputs[0].data_, c.m, c.n, ctx.stream)
               : mnv_maxindex_row(inputs[0].data_, outputs[0].data_, c.m, c.n, ctx.stream);
  Ok(rc, "maxindex");
}

void Reshape(const DataList& inputs, const DataList& outputs, ReshapeClosure&,
             const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u);
  MNV_CHECK_EQ(outputs.size(), 1u);
  MNV_CHECK_EQ(inputs[0].size_.Prod(), outputs[0].size_.Prod()) << "reshape changes the size";
  Ok(mnv_copy(inputs[0].data_, outputs[0].data_, inputs[0].size_.Prod(), ctx.stream), "reshape");
}

#define MNV_ACT_FWD(Name, fn)                                                             \
  void Name(const DataList& inputs, const DataList& outputs, Name##Closure&,              \
            const Context& ctx) {                                                         \
    MNV_CHECK_EQ(inputs.size(), 1u) << #Name " #inputs wrong";                            \
    MNV_CHECK_EQ(outputs.size(), 1u) << #Name " #outputs wrong";                          \
    Ok(fn(inputs[0].data_, outputs[0].data_, inputs[0].size_.Prod(), ctx.stream), #Name); \
  }
MNV_ACT_FWD(SigmoidForward, mnv_sigmoid_fwd)
MNV_ACT_FWD(ReluForward, mnv_relu_fwd)
MNV_ACT_FWD(TanhForward, mnv_tanh_fwd)

// inputs: [top_diff, top, bottom] (cuda.cpp:348-392)
#define MNV_ACT_BWD(Name, fn)                                                              \
  void Name(const DataList& inputs, const DataList& outputs, Name##Closure&,               \
            const Context& ctx) {                                                          \
    MNV_CHECK_EQ(inputs.size(), 3u) << #Name " #inputs wrong";                             \
    MNV_CHECK_EQ(outputs.size(), 1u) << #Name " #outputs wrong";                           \
    Ok(fn(inputs[2].data_, inputs[1].data_, inputs[0].data_, outputs[0].data_,             \
          inputs[0].size_.Prod(), ctx.stream),                                             \
       #Name);                                                                             \
  }
MNV_ACT_BWD(SigmoidBackward, mnv_sigmoid_bwd)
MNV_ACT_BWD(ReluBackward, mnv_relu_bwd)
MNV_ACT_BWD(TanhBackward, mnv_tanh_bwd)

void ActivationForward(const DataList& inputs, const DataList& outputs,
                       ActivationForwardClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(activation forward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(activation forward) #outputs wrong";
  const float* b = inputs[0].data_;
  float* t = outputs[0].data_;
  size_t n = inputs[0].size_.Prod();
  switch (closure.algorithm) {
    case ActivationAlgorithm::kSigmoid: Ok(mnv_sigmoid_fwd(b, t, n, ctx.stream), "sigmoid"); break;
    case ActivationAlgorithm::kRelu: Ok(mnv_relu_fwd(b, t, n, ctx.stream), "relu"); break;
    case ActivationAlgorithm::kTanh: Ok(mnv_tanh_fwd(b, t, n, ctx.stream), "tanh"); break;
    default: MNV_FATAL() << "activation algorithm not supported";
  }
}

void ActivationBackward(const DataList& inputs, const DataList& outputs,
                        ActivationBackwardClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(activation backward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(activation backward) #outputs wrong";
  const float* td = inputs[0].data_;
  const float* top = inputs[1].data_;
  const float* bot = inputs[2].data_;
  float* bd = outputs[0].data_;
  size_t n = inputs[0].size_.Prod();
  switch (closure.algorithm) {
    case ActivationAlgorithm::kSigmoid:
      Ok(mnv_sigmoid_bwd(bot, top, td, bd, n, ctx.stream), "sigmoid bwd");
      break;
    case ActivationAlgorithm::kRelu: Ok(mnv_relu_bwd(bot, top, td, bd, n, ctx.stream), "relu bwd"); break;
    case ActivationAlgorithm::kTanh: Ok(mnv_tanh_bwd(bot, top, td, bd, n, ctx.stream), "tanh bwd"); break;
    default: MNV_FATAL() << "activation algorithm not supported";
  }
}

// Image batches are {W,H,C,N}; filters {S,R,Cin,Cout} (minerva/narray/image_batch.cpp:35-93)
void ConvForward(const DataList& inputs, const DataList& outputs, ConvForwardClosure& c,
                 const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(conv forward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv forward) #outputs wrong";
  auto& bottom = inputs[0];
  auto& filter = inputs[1];
  auto& bias = inputs[2];
  auto& top = outputs[0];
  MNV_CHECK_EQ(bottom.size_[2], filter.size_[2]) << "#input channels mismatch";
  Ok(mnv_conv_fwd(bottom.data_, filter.data_, bias.data_, top.data_, bottom.size_[3],
                  bottom.size_[2], top.size_[2], bottom.size_[1], bottom.size_[0], c.pad_height,
                  c.pad_width, c.stride_vertical, c.stride_horizontal, filter.size_[1],
                  filter.size_[0], ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "conv forward");
}

void ConvBackwardData(const DataList& inputs, const DataList& outputs,
                      ConvBackwardDataClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(conv backward data) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv backward data) #outputs wrong";
  auto& top_diff = inputs[0];
  auto& filter = inputs[1];
  auto& bottom_diff = outputs[0];
  // The extent of bottom_diff comes from the output shard (the forward bottom's size,
  // narray/convolution.cpp:47), not from a formula that only holds for exact fits.
  Ok(mnv_conv_bwd_data(top_diff.data_, filter.data_, bottom_diff.data_, top_diff.size_[3],
                       bottom_diff.size_[2], top_diff.size_[2], bottom_diff.size_[1],
                       bottom_diff.size_[0], c.pad_height, c.pad_width, c.stride_vertical,
                       c.stride_horizontal, filter.size_[1], filter.size_[0], ctx.workspace,
                       ctx.workspace_bytes, ctx.stream),
     "conv backward data");
}

void ConvBackwardFilter(const DataList& inputs, const DataList& outputs,
                        ConvBackwardFilterClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(conv backward filter) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv backward filter) #outputs wrong";
  auto& top_diff = inputs[0];
  auto& bottom = inputs[1];
  auto& filter_diff = outputs[0];
  Ok(mnv_conv_bwd_filter(bottom.data_, top_diff.data_, filter_diff.data_, top_diff.size_[3],
                         bottom.size_[2], top_diff.size_[2], bottom.size_[1], bottom.size_[0],
                         c.pad_height, c.pad_width, c.stride_vertical, c.stride_horizontal,
                         filter_diff.size_[1], filter_diff.size_[0], ctx.workspace,
                         ctx.workspace_bytes, ctx.stream),
     "conv backward filter");
}

void ConvBackwardBias(const DataList& inputs, const DataList& outputs, ConvBackwardBiasClosure&,
                      const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(conv backward bias) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv backward bias) #outputs wrong";
  auto& top_diff = inputs[0];
  Ok(mnv_conv_bwd_bias(top_diff.data_, outputs[0].data_, top_diff.size_[3], top_diff.size_[2],
                       top_diff.size_[1], top_diff.size_[0], ctx.workspace, ctx.workspace_bytes,
                       ctx.stream),
     "conv backward bias");
}

void SoftmaxForward(const DataList& inputs, const DataList& outputs,
                    SoftmaxForwardClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(softmax forward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(softmax forward) #outputs wrong";
  auto& b = inputs[0];
  MNV_CHECK_EQ(b.size_.NumDims(), 4u) << "softmax takes an image batch";
  switch (closure.algorithm) {
    case SoftmaxAlgorithm::kInstance:
      Ok(mnv_softmax_instance_fwd(b.data_, outputs[0].data_, b.size_[3], b.size_[2], b.size_[1],
                                  b.size_[0], ctx.stream), "softmax instance");
      break;
    case SoftmaxAlgorithm::kChannel:
      Ok(mnv_softmax_channel_fwd(b.data_, outputs[0].data_, b.size_[3], b.size_[2], b.size_[1],
                                 b.size_[0], ctx.stream), "softmax channel");
      break;
    default: MNV_FATAL() << "softmax algorithm not supported";
  }
}

void SoftmaxBackward(const DataList& inputs, const DataList& outputs,
                     SoftmaxBackwardClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(softmax backward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(softmax backward) #outputs wrong";
  auto& td = inputs[0];
  auto& top = inputs[1];
  MNV_CHECK_EQ(td.size_.NumDims(), 4u) << "softmax takes an image batch";
  switch (closure.algorithm) {
    case SoftmaxAlgorithm::kInstance:
      Ok(mnv_softmax_instance_bwd(td.data_, top.data_, outputs[0].data_, td.size_[3], td.size_[2],
                                  td.size_[1], td.size_[0], ctx.stream), "softmax instance bwd");
      break;
    case SoftmaxAlgorithm::kChannel:
      Ok(mnv_softmax_channel_bwd(td.data_, top.data_, outputs[0].data_, td.size_[3], td.size_[2],
                                 td.size_[1], td.size_[0], ctx.stream), "softmax channel bwd");
      break;
    default: MNV_FATAL() << "softmax algorithm not supported";
  }
}

void PoolingForward(const DataList& inputs, const DataList& outputs, PoolingForwardClosure& c,
                    const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(pooling forward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(pooling forward) #outputs wrong";
  auto& b = inputs[0];
  auto fn = c.algorithm == PoolingInfo::Algorithm::kMax ? mnv_maxpool_fwd : mnv_avgpool_fwd;
  Ok(fn(b.data_, outputs[0].data_, b.size_[3], b.size_[2], b.size_[1], b.size_[0],
        c.stride_vertical, c.stride_horizontal, c.height, c.width, c.pad_height, c.pad_width,
        ctx.stream),
     "pooling forward");
}

void PoolingBackward(const DataList& inputs, const DataList& outputs, PoolingBackwardClosure& c,
                     const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(pooling backward) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(pooling backward) #outputs wrong";
  auto& td = inputs[0];
  auto& top = inputs[1];
  auto& b = inputs[2];
  auto fn = c.algorithm == PoolingInfo::Algorithm::kMax ? mnv_maxpool_bwd : mnv_avgpool_bwd;
  Ok(fn(b.data_, top.data_, td.data_, outputs[0].data_, td.size_[3], td.size_[2], b.size_[1],
        b.size_[0], c.stride_vertical, c.stride_horizontal, c.height, c.width, c.pad_height,
        c.pad_width, ctx.stream),
     "pooling backward");
}

// inputs {bottom, scale}: `scale` arrives as an input and is filled by the operator, as in
// the reference (cuda.cpp:45-59); data_shape is the {W,H,C,N} extent of bottom.
void LRNForward(const DataList& inputs, const DataList& outputs, LRNForwardClosure& c,
                const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(LRNForward) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(LRNForward) #outputs is wrong!";
  MNV_CHECK_EQ(c.data_shape.NumDims(), 4u) << "(LRNForward) data shape must be {W,H,C,N}";
  Ok(mnv_lrn_fwd(inputs[0].data_, inputs[1].data_, outputs[0].data_, c.local_size, c.alpha, c.beta,
                 c.data_shape[3], c.data_shape[2], c.data_shape[1], c.data_shape[0], ctx.stream),
     "LRN forward");
}

// inputs {bottom, top, scale, top_diff} (cuda.cpp:61-77)
void LRNBackward(const DataList& inputs, const DataList& outputs, LRNBackwardClosure& c,
                 const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 4u) << "(LRNBackward) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(LRNBackward) #outputs is wrong!";
  MNV_CHECK_EQ(c.data_shape.NumDims(), 4u) << "(LRNBackward) data shape must be {W,H,C,N}";
  Ok(mnv_lrn_bwd(inputs[0].data_, inputs[1].data_, inputs[2].data_, inputs[3].data_,
                 outputs[0].data_, c.local_size, c.alpha, c.beta, c.data_shape[3], c.data_shape[2],
                 c.data_shape[1], c.data_shape[0], ctx.stream),
     "LRN backward");
}

namespace {
// product of the dimensions below / above d
size_t Inner(const Scale& s, size_t d) {
  size_t p = 1;
  for (size_t i = 0; i < d; ++i) p *= static_cast<size_t>(s[i]);
  return p;
}
size_t Outer(const Scale& s, size_t d) {
  size_t p = 1;
  for (size_t i = d + 1; i < s.NumDims(); ++i) p *= static_cast<size_t>(s[i]);
  return p;
}
}  // namespace

// CPU-only in the reference (bundle.h:31, basic.cpp:110-123)
void ThresholdNorm(const DataList& inputs, const DataList& outputs, ThresholdNormClosure& c,
                   const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(elewise) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(elewise) #outputs is wrong!";
  Ok(mnv_threshold_norm(inputs[0].data_, outputs[0].data_, c.threshold, outputs[0].size_.Prod(),
                        ctx.stream), "threshold norm");
}

// CPU-only in the reference (bundle.h:55, basic.cpp:473-488): the idx-th block of
// output-sized data
void Index(const DataList& inputs, const DataList& outputs, IndexClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(index) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(index) #outputs wrong";
  const size_t len = outputs[0].size_.Prod();
  MNV_CHECK(c.idx >= 0 && (static_cast<size_t>(c.idx) + 1) * len <= inputs[0].size_.Prod())
      << "(index) block " << c.idx << " outside the input";
  Ok(mnv_copy(inputs[0].data_ + static_cast<size_t>(c.idx) * len, outputs[0].data_, len, ctx.stream),
     "index");
}

// Any dimension is accepted (the reference CHECKs for the last three and then treats every
// dimension but the last as the second to last, cuda.cpp:83,97-118).
void Concat(const DataList& inputs, const DataList& outputs, ConcatClosure& c, const Context& ctx) {
  MNV_CHECK_GT(inputs.size(), 1u) << "(Concat) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(Concat) #outputs is wrong!";
  const Scale& os = outputs[0].size_;
  MNV_CHECK(c.catdim >= 0 && static_cast<size_t>(c.catdim) < os.NumDims()) << "(Concat) bad dimension";
  const size_t d = static_cast<size_t>(c.catdim);
  const size_t inner = Inner(os, d), outer = Outer(os, d);
  size_t offset = 0;
  for (auto& in : inputs) {
    MNV_CHECK_EQ(in.size_.NumDims(), os.NumDims()) << "(Concat) rank mismatch";
    for (size_t i = 0; i < os.NumDims(); ++i) {
      if (i != d) {
        MNV_CHECK_EQ(in.size_[i], os[i]) << "(Concat) extent mismatch in dimension " << i;
      }
    }
    const size_t e = static_cast<size_t>(in.size_[d]);
    MNV_CHECK_LE(offset + e, static_cast<size_t>(os[d])) << "(Concat) inputs exceed the output";
    Ok(mnv_copy_2d(in.data_, outputs[0].data_ + offset * inner, e * inner, outer, e * inner,
                   static_cast<size_t>(os[d]) * inner, ctx.stream), "concat");
    offset += e;
  }
  MNV_CHECK_EQ(offset, static_cast<size_t>(os[d])) << "(Concat) inputs do not fill the output";
}

void Slice(const DataList& inputs, const DataList& outputs, SliceClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u) << "(Slice) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(Slice) #outputs is wrong!";
  const Scale& is = inputs[0].size_;
  MNV_CHECK(c.slice_dim >= 0 && static_cast<size_t>(c.slice_dim) < is.NumDims()) << "(Slice) bad dimension";
  const size_t d = static_cast<size_t>(c.slice_dim);
  MNV_CHECK(c.st_off >= 0 && c.slice_count > 0 && c.st_off + c.slice_count <= is[d])
      << "(Slice) range outside the tensor";
  MNV_CHECK_EQ(outputs[0].size_[d], c.slice_count) << "(Slice) output extent";
  const size_t inner = Inner(is, d), outer = Outer(is, d);
  Ok(mnv_copy_2d(inputs[0].data_ + static_cast<size_t>(c.st_off) * inner, outputs[0].data_,
                 static_cast<size_t>(c.slice_count) * inner, outer,
                 static_cast<size_t>(is[d]) * inner, static_cast<size_t>(c.slice_count) * inner,
                 ctx.stream), "slice");
}

void Select(const DataList& inputs, const DataList& outputs, SelectClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 1u);
  MNV_CHECK_EQ(outputs.size(), 1u);
  MNV_CHECK_EQ(inputs[0].size_.NumDims(), 2u);
  MNV_CHECK_EQ(outputs[0].size_.NumDims(), 2u);
  MNV_CHECK_EQ(inputs[0].size_[0], outputs[0].size_[0]);
  MNV_CHECK_EQ(static_cast<size_t>(outputs[0].size_[1]), c.indices.size());
  for (auto i : c.indices) MNV_CHECK(i >= 0 && i < inputs[0].size_[1]) << "(Select) index " << i;
  Ok(mnv_select(inputs[0].data_, outputs[0].data_, c.indices.data(),
                static_cast<int>(c.indices.size()), inputs[0].size_[0], inputs[0].size_[1],
                ctx.workspace, ctx.workspace_bytes, ctx.stream), "select");
  // the index vector belongs to the closure: it must outlive the staging copy
  Ok(mnv_stream_sync(ctx.stream), "select sync");
}

void ArrayLoader(const DataList& outputs, ArrayLoaderClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(outputs.size(), 1u) << "(array loader) #outputs wrong";
  MNV_CHECK(closure.data) << "probably already executed";
  // on the operator's own stream (the reference uses the default stream, cuda.cpp:595); large
  // pageable buffers go through the stream's pinned staging area; synchronised, because the
  // host buffer must outlive the copy
  const size_t bytes = outputs[0].size_.Prod() * sizeof(float);
  Ok(StagedHostToDevice(outputs[0].data_, closure.data.get(), bytes, ctx.stream, ctx.staging,
                        ctx.staging_bytes),
     "array loader");
  closure.data.reset();
}

namespace {
std::atomic<uint64_t> g_seed_base{0x243F6A8885A308D3ull}, g_seed_count{0};
uint64_t NextSeed() {  // splitmix64 of (base + call number)
  uint64_t z = g_seed_base.load() + 0x9E3779B97F4A7C15ull * (g_seed_count.fetch_add(1) + 1);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}
}  // namespace

void SetRandomSeed(uint64_t seed) {
  g_seed_base.store(seed);
  g_seed_count.store(0);
}

void Randn(const DataList& outputs, RandnClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(outputs.size(), 1u) << "(normal) #outputs wrong";
  Ok(mnv_randn(outputs[0].data_, outputs[0].size_.Prod(), NextSeed(), closure.mu, closure.var,
               ctx.stream), "randn");
}

void RandBernoulli(const DataList& outputs, RandBernoulliClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(outputs.size(), 1u) << "(bernoulli) #outputs wrong";
  Ok(mnv_rand_bernoulli(outputs[0].data_, outputs[0].size_.Prod(), NextSeed(), closure.p,
                        ctx.stream), "rand bernoulli");
}

void Fill(const DataList& outputs, FillClosure& closure, const Context& ctx) {
  MNV_CHECK_EQ(outputs.size(), 1u) << "(fill) #outputs wrong";
  Ok(mnv_fill(outputs[0].data_, outputs[0].size_.Prod(), closure.val, ctx.stream), "fill");
}

}  // namespace hip
}  // namespace minerva
