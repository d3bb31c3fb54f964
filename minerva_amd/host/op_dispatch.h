// Operator objects and dispatch: what the engine stores in a task and calls.
// Mirrors the reference's ComputeFn / ComputeFnWithClosure / FnBundle / *Op layering
// (minerva/op/compute_fn.h:9-12, op/physical_fn.h:13-27, op/impl/impl.h:11-35,
// op/impl/bundle.h:19-56, op/physical_op.h:14-382) with one installed column: the HIP
// implementation.  Any other ImplType is "no implementation", as NO_IMPL is there.
#pragma once
#include <typeinfo>

#include "device.h"
#include "hip_fused_ops.h"
#include "hip_ops.h"
#include "minerva_types.h"

namespace minerva {

template <typename C> struct FnBundle;

template <typename C> [[noreturn]] void NoImpl(const Context& ctx) {
  MNV_FATAL() << "no implementation for " << typeid(C).name() << " on " << ctx.impl_type;
  throw Error("unreachable");
}

#define MNV_INSTALL_COMPUTE_FN(closure_name, hip_fn)                                        \
  template <> struct FnBundle<closure_name> {                                               \
    static void Call(const DataList& i, const DataList& o, closure_name& c, const Context& x) { \
      if (x.impl_type == ImplType::kHip) hip_fn(i, o, c, x);                                \
      else NoImpl<closure_name>(x);                                                         \
    }                                                                                       \
  };
#define MNV_INSTALL_DATAGEN_FN(closure_name, hip_fn)                           \
  template <> struct FnBundle<closure_name> {                                  \
    static void Call(const DataList& o, closure_name& c, const Context& x) {   \
      if (x.impl_type == ImplType::kHip) hip_fn(o, c, x);                      \
      else NoImpl<closure_name>(x);                                            \
    }                                                                          \
  };

MNV_INSTALL_COMPUTE_FN(ArithmeticClosure, hip::Arithmetic)
MNV_INSTALL_COMPUTE_FN(ArithmeticConstClosure, hip::ArithmeticConst)
MNV_INSTALL_COMPUTE_FN(MatMultClosure, hip::MatMult)
MNV_INSTALL_COMPUTE_FN(TransposeClosure, hip::Transpose)
MNV_INSTALL_COMPUTE_FN(ReductionClosure, hip::Reduction)
MNV_INSTALL_COMPUTE_FN(NormArithmeticClosure, hip::NormArithmetic)
MNV_INSTALL_COMPUTE_FN(MaxIndexClosure, hip::MaxIndex)
MNV_INSTALL_COMPUTE_FN(ReshapeClosure, hip::Reshape)
MNV_INSTALL_COMPUTE_FN(ElewiseClosure, hip::Elewise)
MNV_INSTALL_COMPUTE_FN(SigmoidForwardClosure, hip::SigmoidForward)
MNV_INSTALL_COMPUTE_FN(SigmoidBackwardClosure, hip::SigmoidBackward)
MNV_INSTALL_COMPUTE_FN(ReluForwardClosure, hip::ReluForward)
MNV_INSTALL_COMPUTE_FN(ReluBackwardClosure, hip::ReluBackward)
MNV_INSTALL_COMPUTE_FN(TanhForwardClosure, hip::TanhForward)
MNV_INSTALL_COMPUTE_FN(TanhBackwardClosure, hip::TanhBackward)
MNV_INSTALL_COMPUTE_FN(ConvForwardClosure, hip::ConvForward)
MNV_INSTALL_COMPUTE_FN(ConvBackwardDataClosure, hip::ConvBackwardData)
MNV_INSTALL_COMPUTE_FN(ConvBackwardFilterClosure, hip::ConvBackwardFilter)
MNV_INSTALL_COMPUTE_FN(ConvBackwardBiasClosure, hip::ConvBackwardBias)
MNV_INSTALL_COMPUTE_FN(SoftmaxForwardClosure, hip::SoftmaxForward)
MNV_INSTALL_COMPUTE_FN(SoftmaxBackwardClosure, hip::SoftmaxBackward)
MNV_INSTALL_COMPUTE_FN(ActivationForwardClosure, hip::ActivationForward)
MNV_INSTALL_COMPUTE_FN(ActivationBackwardClosure, hip::ActivationBackward)
MNV_INSTALL_COMPUTE_FN(PoolingForwardClosure, hip::PoolingForward)
MNV_INSTALL_COMPUTE_FN(PoolingBackwardClosure, hip::PoolingBackward)
MNV_INSTALL_COMPUTE_FN(LRNForwardClosure, hip::LRNForward)
MNV_INSTALL_COMPUTE_FN(LRNBackwardClosure, hip::LRNBackward)
MNV_INSTALL_COMPUTE_FN(ThresholdNormClosure, hip::ThresholdNorm)
MNV_INSTALL_COMPUTE_FN(IndexClosure, hip::Index)
MNV_INSTALL_COMPUTE_FN(ConcatClosure, hip::Concat)
MNV_INSTALL_COMPUTE_FN(SliceClosure, hip::Slice)
MNV_INSTALL_COMPUTE_FN(SelectClosure, hip::Select)
// the opt-in fused operators (hip_fused_ops.h): no counterpart in the reference's table
MNV_INSTALL_COMPUTE_FN(ConvForwardReluClosure, hip::ConvForwardRelu)
MNV_INSTALL_COMPUTE_FN(ConvBackwardDataReluClosure, hip::ConvBackwardDataRelu)
MNV_INSTALL_COMPUTE_FN(PoolingBackwardReluClosure, hip::PoolingBackwardRelu)
MNV_INSTALL_COMPUTE_FN(MatMultBiasClosure, hip::MatMultBias)
MNV_INSTALL_COMPUTE_FN(MatMultReluBackwardClosure, hip::MatMultReluBackward)
MNV_INSTALL_COMPUTE_FN(MatMultTransAClosure, hip::MatMultTransA)
MNV_INSTALL_COMPUTE_FN(MatMultTransBClosure, hip::MatMultTransB)
MNV_INSTALL_COMPUTE_FN(SgdUpdateClosure, hip::SgdUpdate)
MNV_INSTALL_COMPUTE_FN(MatMultTransBSgdClosure, hip::MatMultTransBSgd)
MNV_INSTALL_COMPUTE_FN(ConvBackwardFilterSgdClosure, hip::ConvBackwardFilterSgd)
MNV_INSTALL_DATAGEN_FN(ArrayLoaderClosure, hip::ArrayLoader)
MNV_INSTALL_DATAGEN_FN(FillClosure, hip::Fill)
MNV_INSTALL_DATAGEN_FN(RandnClosure, hip::Randn)
MNV_INSTALL_DATAGEN_FN(RandBernoulliClosure, hip::RandBernoulli)

template <typename C> class ComputeFnWithClosure : public ComputeFn {
 public:
  C closure;
  void Execute(const DataList& in, const DataList& out, const Context& ctx) override {
    FnBundle<C>::Call(in, out, closure, ctx);
  }
};

template <typename C> class PhyDataGenFnWithClosure : public ComputeFn {
 public:
  C closure;
  void Execute(const DataList&, const DataList& out, const Context& ctx) override {
    FnBundle<C>::Call(out, closure, ctx);
  }
};

inline const char* ArithSym(ArithmeticType t) {
  switch (t) {
    case ArithmeticType::kAdd: return "+";
    case ArithmeticType::kSub: return "-";
    case ArithmeticType::kMult: return ".*";
    case ArithmeticType::kDiv: return "./";
  }
  return "NA";
}

#define MNV_SIMPLE_OP(Cls, Base, Closure, name_str) \
  class Cls : public Base<Closure> {                \
   public:                                          \
    std::string Name() const override { return name_str; } \
  };

MNV_SIMPLE_OP(ArrayLoaderOp, PhyDataGenFnWithClosure, ArrayLoaderClosure, ":array loader")
MNV_SIMPLE_OP(RandnOp, PhyDataGenFnWithClosure, RandnClosure, ":normal")
MNV_SIMPLE_OP(RandBernoulliOp, PhyDataGenFnWithClosure, RandBernoulliClosure, ":bernoulli")
MNV_SIMPLE_OP(MatMultOp, ComputeFnWithClosure, MatMultClosure, "*")
MNV_SIMPLE_OP(TransOp, ComputeFnWithClosure, TransposeClosure, "trans")
MNV_SIMPLE_OP(MaxIndexOp, ComputeFnWithClosure, MaxIndexClosure, "max index")
MNV_SIMPLE_OP(ReshapeOp, ComputeFnWithClosure, ReshapeClosure, "reshape")
MNV_SIMPLE_OP(SigmoidForwardOp, ComputeFnWithClosure, SigmoidForwardClosure, "sigmoid forward")
MNV_SIMPLE_OP(SigmoidBackwardOp, ComputeFnWithClosure, SigmoidBackwardClosure, "sigmoid backward")
MNV_SIMPLE_OP(ReluForwardOp, ComputeFnWithClosure, ReluForwardClosure, "relu forward")
MNV_SIMPLE_OP(ReluBackwardOp, ComputeFnWithClosure, ReluBackwardClosure, "relu backward")
MNV_SIMPLE_OP(TanhForwardOp, ComputeFnWithClosure, TanhForwardClosure, "tanh forward")
MNV_SIMPLE_OP(TanhBackwardOp, ComputeFnWithClosure, TanhBackwardClosure, "tanh backward")
MNV_SIMPLE_OP(ConvBackwardBiasOp, ComputeFnWithClosure, ConvBackwardBiasClosure, "conv bp bias")
class LRNForwardOp : public ComputeFnWithClosure<LRNForwardClosure> {
 public:
  std::string Name() const override { return "LRN Forward"; }
  int MutatedInput() const override { return 1; }
};
MNV_SIMPLE_OP(LRNBackwardOp, ComputeFnWithClosure, LRNBackwardClosure, "LRN Backward")
MNV_SIMPLE_OP(ThresholdNormOp, ComputeFnWithClosure, ThresholdNormClosure, "threshold norm")
MNV_SIMPLE_OP(IndexOp, ComputeFnWithClosure, IndexClosure, "index")
MNV_SIMPLE_OP(ConcatOp, ComputeFnWithClosure, ConcatClosure, "Concat")
MNV_SIMPLE_OP(SliceOp, ComputeFnWithClosure, SliceClosure, "Slice")
MNV_SIMPLE_OP(SelectOp, ComputeFnWithClosure, SelectClosure, "select")
MNV_SIMPLE_OP(PoolingBackwardReluOp, ComputeFnWithClosure, PoolingBackwardReluClosure,
              "max pooling bp + relu bp")
MNV_SIMPLE_OP(MatMultReluBackwardOp, ComputeFnWithClosure, MatMultReluBackwardClosure, "* + relu bp")
MNV_SIMPLE_OP(MatMultTransAOp, ComputeFnWithClosure, MatMultTransAClosure, "trans * [+ relu bp]")
MNV_SIMPLE_OP(MatMultTransBOp, ComputeFnWithClosure, MatMultTransBClosure, "* trans")
MNV_SIMPLE_OP(SgdUpdateOp, ComputeFnWithClosure, SgdUpdateClosure, "sgd update")
MNV_SIMPLE_OP(MatMultTransBSgdOp, ComputeFnWithClosure, MatMultTransBSgdClosure, "* trans + sgd update")

class MatMultBiasOp : public ComputeFnWithClosure<MatMultBiasClosure> {
 public:
  std::string Name() const override { return closure.relu ? "* + bias + relu" : "* + bias"; }
};

class FillOp : public PhyDataGenFnWithClosure<FillClosure> {
 public:
  std::string Name() const override {
    std::ostringstream ss;
    ss << ":const=" << closure.val;
    return ss.str();
  }
};

class ReductionOp : public ComputeFnWithClosure<ReductionClosure> {
 public:
  std::string Name() const override { return closure.type == ReductionType::kSum ? "sum" : "max"; }
};

class ElewiseOp : public ComputeFnWithClosure<ElewiseClosure> {
 public:
  std::string Name() const override {
    switch (closure.type) {
      case ElewiseType::kExp: return "exp";
      case ElewiseType::kLn: return "ln";
      case ElewiseType::kNegative: return "-";
    }
    return "NA";
  }
};

class ArithmeticOp : public ComputeFnWithClosure<ArithmeticClosure> {
 public:
  std::string Name() const override { return ArithSym(closure.type); }
};

class ArithmeticConstOp : public ComputeFnWithClosure<ArithmeticConstClosure> {
 public:
  std::string Name() const override {
    std::ostringstream ss;
    if (closure.side == 0) ss << closure.val;
    ss << (closure.type == ArithmeticType::kAdd ? "+." : closure.type == ArithmeticType::kSub ? "-."
                                                                                             : ArithSym(closure.type));
    if (closure.side == 1) ss << closure.val;
    return ss.str();
  }
};

class NormArithmeticOp : public ComputeFnWithClosure<NormArithmeticClosure> {
 public:
  std::string Name() const override { return std::string(ArithSym(closure.type)) + " norm"; }
};

template <class Base, int kind> class ConvNamed : public Base {
 public:
  std::string Name() const override {
    std::ostringstream ss;
    ss << "pad:" << this->closure.pad_height << "*" << this->closure.pad_width
       << " stride:" << this->closure.stride_vertical << "*" << this->closure.stride_horizontal
       << (kind == 0 ? " conv ff" : kind == 1 ? " conv bp data" : kind == 2 ? " conv bp filter"
           : kind == 3 ? " conv ff + relu" : kind == 4 ? " conv bp data + relu bp"
                                           : " conv bp filter + sgd update");
    return ss.str();
  }
};
typedef ConvNamed<ComputeFnWithClosure<ConvForwardClosure>, 0> ConvForwardOp;
typedef ConvNamed<ComputeFnWithClosure<ConvBackwardDataClosure>, 1> ConvBackwardDataOp;
typedef ConvNamed<ComputeFnWithClosure<ConvBackwardFilterClosure>, 2> ConvBackwardFilterOp;
typedef ConvNamed<ComputeFnWithClosure<ConvForwardReluClosure>, 3> ConvForwardReluOp;
typedef ConvNamed<ComputeFnWithClosure<ConvBackwardDataReluClosure>, 4> ConvBackwardDataReluOp;
typedef ConvNamed<ComputeFnWithClosure<ConvBackwardFilterSgdClosure>, 5> ConvBackwardFilterSgdOp;

template <class Base, bool fwd> class SoftmaxNamed : public Base {
 public:
  std::string Name() const override {
    return std::string(this->closure.algorithm == SoftmaxAlgorithm::kInstance ? "instance" : "channel") +
           (fwd ? " softmax ff" : " softmax bp");
  }
};
typedef SoftmaxNamed<ComputeFnWithClosure<SoftmaxForwardClosure>, true> SoftmaxForwardOp;
typedef SoftmaxNamed<ComputeFnWithClosure<SoftmaxBackwardClosure>, false> SoftmaxBackwardOp;

template <class Base, bool fwd> class ActivationNamed : public Base {
 public:
  std::string Name() const override {
    const char* a = this->closure.algorithm == ActivationAlgorithm::kSigmoid ? "sigmoid"
                    : this->closure.algorithm == ActivationAlgorithm::kRelu  ? "relu"
                                                                             : "tanh";
    return std::string(a) + (fwd ? " ff" : " bp");
  }
};
typedef ActivationNamed<ComputeFnWithClosure<ActivationForwardClosure>, true> ActivationForwardOp;
typedef ActivationNamed<ComputeFnWithClosure<ActivationBackwardClosure>, false> ActivationBackwardOp;

template <class Base, bool fwd> class PoolingNamed : public Base {
 public:
  std::string Name() const override {
    std::ostringstream ss;
    ss << (this->closure.algorithm == PoolingInfo::Algorithm::kMax ? "max" : "average")
       << (fwd ? " pooling ff " : " pooling bp ") << this->closure.height << "*"
       << this->closure.width << " stride:" << this->closure.stride_horizontal << "*"
       << this->closure.stride_vertical;
    return ss.str();
  }
};
typedef PoolingNamed<ComputeFnWithClosure<PoolingForwardClosure>, true> PoolingForwardOp;
typedef PoolingNamed<ComputeFnWithClosure<PoolingBackwardClosure>, false> PoolingBackwardOp;

}  // namespace minerva
