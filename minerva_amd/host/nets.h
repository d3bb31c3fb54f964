// The three training graphs of the benchmark configurations, written against the
// Runner exactly as the reference applications write them against NArray:
//   MLP 784-256-10          apps/mnist_common.h:213-288 (MnistMlpAlgo)
//   MNIST CNN               apps/mnist_common.h:123-211 (MnistCnnAlgo)
//   AlexNet-shaped network  owl/apps/imagenet_alexnet/alexnet.py:7-133 (no dropout / LRN,
//                           single group), plain SGD w -= lr/batch * grad
// One Step = forward + backward + parameter update, one operator at a time; nothing is
// fused across operator boundaries unless `fused` is set, which swaps every
// (producer, ReLU / ReLU gradient / bias add) pair and the two-operator SGD update for the
// fused operator that returns the same bits (hip_fused_ops.h).
#pragma once
#include <map>

#include "runner.h"

namespace minerva {

class Net {
 public:
  Net(Runner* r, int batch) : rt(r), batch_(batch) {}
  virtual ~Net() {}
  virtual void Step(const Tensor& data, const Tensor& label, float lr) = 0;
  virtual Scale DataSize() const = 0;
  virtual Scale LabelSize() const = 0;
  int batch() const { return batch_; }
  // Whether replaying a recording of one Step equals calling Step again.  Not so when the
  // step draws fresh random seeds on the host (dropout): a recording would repeat them.
  virtual bool Capturable() const { return true; }

  std::vector<std::string> param_names;   // "w0", "b0", ...
  std::map<std::string, Tensor> params;   // current parameters
  std::map<std::string, Tensor> results;  // "prob" and "g_<param>" of the last Step
  // Tests only: the step also leaves its activations in `results` ("act1", "act2", ...),
  // which keeps their device blocks alive until the next step.
  bool keep_activations = false;
  // Opt-in fast path: fused epilogues instead of separate ReLU / bias / update operators.
  bool fused = false;
  // With `fused`: the weight updates of convolutions and inner products are applied in the
  // store of the kernel that produces the gradient.  Same parameters bit for bit, but the
  // weight gradients are never stored, so `results` holds no "g_w<i>".
  bool fuse_update = false;

 protected:
  // w <- w - (lr / batch) * g : ArithmeticConst(mult, const on the left) + Arithmetic(sub)
  void Sgd(const std::string& name, const Tensor& grad, float lr);
  void AddParam(const std::string& name, const Scale& size);
  // The operator pairs of the graphs, separate or fused according to `fused`.
  Tensor ConvRelu(const Tensor& x, const Tensor& w, const Tensor& b, ConvInfo info);
  Tensor ConvBackwardDataRelu(const Tensor& diff, const Tensor& bottom, const Tensor& w, ConvInfo info);
  Tensor PoolBackwardRelu(const Tensor& diff, const Tensor& top, const Tensor& bottom, PoolingInfo info);
  Tensor Fc(const Tensor& w, const Tensor& x, const Tensor& b, bool relu);
  Tensor MatMultReluBackward(const Tensor& a, const Tensor& b, const Tensor& act);
  Tensor TransMatMult(const Tensor& at, const Tensor& b);
  Tensor TransMatMultReluBackward(const Tensor& at, const Tensor& b, const Tensor& act);
  Tensor MatMultTrans(const Tensor& a, const Tensor& bt);
  // gradient + update of an inner product's weights (sens * act^T) and of a filter
  void SgdFc(const std::string& name, const Tensor& sens, const Tensor& act, float lr);
  void SgdConv(const std::string& name, const Tensor& diff, const Tensor& bottom, ConvInfo info, float lr);
  Runner* rt;
  int batch_;
};

class MlpNet : public Net {
 public:
  MlpNet(Runner* r, int batch, int in = 784, int hidden = 256, int out = 10);
  void Step(const Tensor& data, const Tensor& label, float lr) override;
  Scale DataSize() const override { return Scale{in_, batch_}; }
  Scale LabelSize() const override { return Scale{out_, batch_}; }

 private:
  int in_, hidden_, out_;
};

class CnnNet : public Net {
 public:
  // pad2 / pool2: 0 and 2x2/2 (benchmark configuration) or 2 and 3x3/3 (reference app)
  CnnNet(Runner* r, int batch, int pad2 = 0, int pool2 = 2);
  void Step(const Tensor& data, const Tensor& label, float lr) override;
  Scale DataSize() const override { return Scale{28, 28, 1, batch_}; }
  Scale LabelSize() const override { return Scale{10, 1, 1, batch_}; }

 private:
  ConvInfo conv_info[2];
  PoolingInfo pool_info[2];
};

class AlexNet : public Net {
 public:
  // dropout_rate > 0: the reference application's drop6 / drop7 (owl/apps/imagenet_alexnet/
  // alexnet.py:86-89,97-101): activations times a Bernoulli(dropout_rate) mask, no rescaling
  AlexNet(Runner* r, int batch, int num_classes = 1000, float dropout_rate = 0.f);
  void Step(const Tensor& data, const Tensor& label, float lr) override;
  Scale DataSize() const override { return Scale{227, 227, 3, batch_}; }
  Scale LabelSize() const override { return Scale{classes_, batch_}; }
  bool Capturable() const override { return dropout_rate_ == 0.f; }

 private:
  int classes_;
  float dropout_rate_;
  ConvInfo convs[5];
  PoolingInfo poolings[3];
};

}  // namespace minerva
