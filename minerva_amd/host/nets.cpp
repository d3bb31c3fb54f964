#include "nets.h"

namespace minerva {

void Net::AddParam(const std::string& name, const Scale& size) {
  param_names.push_back(name);
  params[name] = rt->Zeros(size);
}

void Net::Sgd(const std::string& name, const Tensor& grad, float lr) {
  results["g_" + name] = grad;
  const float scale = lr / static_cast<float>(batch_);
  if (fused) {
    params[name] = rt->SgdUpdate(params[name], grad, scale);
    return;
  }
  Tensor step = rt->ArithmeticConst(grad, scale, ArithmeticType::kMult, 0);
  params[name] = rt->Sub(params[name], step);
}

Tensor Net::ConvRelu(const Tensor& x, const Tensor& w, const Tensor& b, ConvInfo info) {
  if (fused) return rt->ConvForwardRelu(x, w, b, info);
  return rt->ReluForward(rt->ConvForward(x, w, b, info));
}

Tensor Net::ConvBackwardDataRelu(const Tensor& diff, const Tensor& bottom, const Tensor& w,
                                 ConvInfo info) {
  if (fused) return rt->ConvBackwardDataRelu(diff, bottom, w, info);
  return rt->ReluBackward(rt->ConvBackwardData(diff, bottom, w, info), bottom, bottom);
}

Tensor Net::PoolBackwardRelu(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                             PoolingInfo info) {
  if (fused) return rt->PoolingBackwardRelu(diff, top, bottom, info);
  return rt->ReluBackward(rt->PoolingBackward(diff, top, bottom, info), bottom, bottom);
}

Tensor Net::Fc(const Tensor& w, const Tensor& x, const Tensor& b, bool relu) {
  if (fused) return rt->MatMultBias(w, x, b, relu);
  Tensor y = rt->NormArithmetic(rt->MatMult(w, x), b, ArithmeticType::kAdd);
  return relu ? rt->ReluForward(y) : y;
}

Tensor Net::MatMultReluBackward(const Tensor& a, const Tensor& b, const Tensor& act) {
  if (fused) return rt->MatMultReluBackward(a, b, act);
  return rt->ReluBackward(rt->MatMult(a, b), act, act);
}

// The products of an inner product's backward pass, which the reference's applications write
// as Transpose + MatMult (apps/mnist_common.h:258-262): fused, the transposed operand is read
// in place.
Tensor Net::TransMatMult(const Tensor& at, const Tensor& b) {
  if (fused) return rt->MatMultTransA(at, b);
  return rt->MatMult(rt->Trans(at), b);
}

Tensor Net::TransMatMultReluBackward(const Tensor& at, const Tensor& b, const Tensor& act) {
  if (fused) return rt->MatMultTransA(at, b, act);
  return rt->ReluBackward(rt->MatMult(rt->Trans(at), b), act, act);
}

Tensor Net::MatMultTrans(const Tensor& a, const Tensor& bt) {
  if (fused) return rt->MatMultTransB(a, bt);
  return rt->MatMult(a, rt->Trans(bt));
}

void Net::SgdFc(const std::string& name, const Tensor& sens, const Tensor& act, float lr) {
  if (fused && fuse_update) {
    results.erase("g_" + name);
    params[name] = rt->MatMultTransBSgd(sens, act, params[name], lr / static_cast<float>(batch_));
    return;
  }
  Sgd(name, MatMultTrans(sens, act), lr);
}

void Net::SgdConv(const std::string& name, const Tensor& diff, const Tensor& bottom, ConvInfo info,
                  float lr) {
  if (fused && fuse_update) {
    results.erase("g_" + name);
    params[name] = rt->ConvBackwardFilterSgd(diff, bottom, params[name], info,
                                             lr / static_cast<float>(batch_));
    return;
  }
  Sgd(name, rt->ConvBackwardFilter(diff, bottom, params[name], info), lr);
}

// ------------------------------------------------------------------------- MLP

MlpNet::MlpNet(Runner* r, int batch, int in, int hidden, int out)
    : Net(r, batch), in_(in), hidden_(hidden), out_(out) {
  AddParam("w0", Scale{hidden, in});
  AddParam("b0", Scale{hidden, 1});
  AddParam("w1", Scale{out, hidden});
  AddParam("b1", Scale{out, 1});
}

void MlpNet::Step(const Tensor& data, const Tensor& label, float lr) {
  Tensor& w0 = params["w0"]; Tensor& b0 = params["b0"];
  Tensor& w1 = params["w1"]; Tensor& b1 = params["b1"];
  // FF
  Tensor a1 = Fc(w0, data, b0, true);
  Tensor a2 = Fc(w1, a1, b1, false);
  Tensor a3 = rt->Reshape(
      rt->SoftmaxForward(rt->Reshape(a2, Scale{out_, 1, 1, batch_}), SoftmaxAlgorithm::kInstance),
      Scale{out_, batch_});
  results["prob"] = a3;
  // BP
  Tensor s2 = rt->Sub(a3, label);
  Tensor s1 = TransMatMultReluBackward(w1, s2, a1);
  Tensor gb0 = rt->Sum(s1, 1);
  Tensor gb1 = rt->Sum(s2, 1);
  // weight gradients and update
  SgdFc("w0", s1, data, lr); Sgd("b0", gb0, lr); SgdFc("w1", s2, a1, lr); Sgd("b1", gb1, lr);
}

// ------------------------------------------------------------------------- CNN

CnnNet::CnnNet(Runner* r, int batch, int pad2, int pool2) : Net(r, batch) {
  conv_info[0] = ConvInfo(0, 0, 1, 1);
  conv_info[1] = ConvInfo(pad2, pad2, 1, 1);
  pool_info[0] = PoolingInfo(PoolingInfo::Algorithm::kMax, 2, 2, 2, 2);
  pool_info[1] = PoolingInfo(PoolingInfo::Algorithm::kMax, pool2, pool2, pool2, pool2);
  AddParam("w0", Scale{5, 5, 1, 16});
  AddParam("b0", Scale{16});
  AddParam("w1", Scale{5, 5, 16, 32});
  AddParam("b1", Scale{32});
  AddParam("w2", Scale{10, 512});
  AddParam("b2", Scale{10, 1});
}

void CnnNet::Step(const Tensor& data, const Tensor& label, float lr) {
  const int b = batch_;
  Tensor a0 = data;
  // fused: the pre-activations a1 / a4 are never stored, and the ReLU gradients below test
  // the activations a2 / a5 instead (x > 0 exactly when relu(x) > 0)
  Tensor a1, a2, a4, a5;
  if (fused) {
    a2 = rt->ConvForwardRelu(a0, params["w0"], params["b0"], conv_info[0]);
  } else {
    a1 = rt->ConvForward(a0, params["w0"], params["b0"], conv_info[0]);
    a2 = rt->ActivationForward(a1, ActivationAlgorithm::kRelu);
  }
  Tensor a3 = rt->PoolingForward(a2, pool_info[0]);
  if (fused) {
    a5 = rt->ConvForwardRelu(a3, params["w1"], params["b1"], conv_info[1]);
  } else {
    a4 = rt->ConvForward(a3, params["w1"], params["b1"], conv_info[1]);
    a5 = rt->ActivationForward(a4, ActivationAlgorithm::kRelu);
  }
  Tensor a6 = rt->PoolingForward(a5, pool_info[1]);
  Tensor re6 = rt->Reshape(a6, Scale{a6->size.Prod() / b, b});
  MNV_CHECK_EQ(re6->size[0], 512) << "the classifier expects 512 features";
  Tensor a7 = Fc(params["w2"], re6, params["b2"], false);
  Tensor a8 = rt->SoftmaxForward(rt->Reshape(a7, Scale{10, 1, 1, b}), SoftmaxAlgorithm::kInstance);
  results["prob"] = a8;
  // BP
  Tensor s8 = rt->Sub(a8, label);
  Tensor s7 = rt->Reshape(s8, Scale{10, b});
  Tensor s6 = rt->Reshape(TransMatMult(params["w2"], s7), a6->size);
  Tensor s4, s1;
  if (fused) {
    s4 = rt->PoolingBackwardRelu(s6, a6, a5, pool_info[1]);
  } else {
    Tensor s5 = rt->PoolingBackward(s6, a6, a5, pool_info[1]);
    s4 = rt->ActivationBackward(s5, a5, a4, ActivationAlgorithm::kRelu);
  }
  Tensor s3 = rt->ConvBackwardData(s4, a3, params["w1"], conv_info[1]);
  if (fused) {
    s1 = rt->PoolingBackwardRelu(s3, a3, a2, pool_info[0]);
  } else {
    Tensor s2 = rt->PoolingBackward(s3, a3, a2, pool_info[0]);
    s1 = rt->ActivationBackward(s2, a2, a1, ActivationAlgorithm::kRelu);
  }
  Tensor gb0 = rt->ConvBackwardBias(s1);
  Tensor gb1 = rt->ConvBackwardBias(s4);
  Tensor gb2 = rt->Sum(s7, 1);
  SgdConv("w0", s1, a0, conv_info[0], lr); Sgd("b0", gb0, lr);
  SgdConv("w1", s4, a3, conv_info[1], lr); Sgd("b1", gb1, lr);
  SgdFc("w2", s7, re6, lr); Sgd("b2", gb2, lr);
}

// --------------------------------------------------------------------- AlexNet

AlexNet::AlexNet(Runner* r, int batch, int num_classes, float dropout_rate)
    : Net(r, batch), classes_(num_classes), dropout_rate_(dropout_rate) {
  convs[0] = ConvInfo(0, 0, 4, 4);
  convs[1] = ConvInfo(2, 2, 1, 1);
  convs[2] = convs[3] = convs[4] = ConvInfo(1, 1, 1, 1);
  for (auto& p : poolings) p = PoolingInfo(PoolingInfo::Algorithm::kMax, 3, 3, 2, 2);
  AddParam("w0", Scale{11, 11, 3, 96});
  AddParam("w1", Scale{5, 5, 96, 256});
  AddParam("w2", Scale{3, 3, 256, 384});
  AddParam("w3", Scale{3, 3, 384, 384});
  AddParam("w4", Scale{3, 3, 384, 256});
  AddParam("w5", Scale{4096, 9216});
  AddParam("w6", Scale{4096, 4096});
  AddParam("w7", Scale{num_classes, 4096});
  AddParam("b0", Scale{96});
  AddParam("b1", Scale{256});
  AddParam("b2", Scale{384});
  AddParam("b3", Scale{384});
  AddParam("b4", Scale{256});
  AddParam("b5", Scale{4096, 1});
  AddParam("b6", Scale{4096, 1});
  AddParam("b7", Scale{num_classes, 1});
}

void AlexNet::Step(const Tensor& data, const Tensor& label, float lr) {
  const int n = batch_;
  auto W = [&](int i) -> Tensor& { return params["w" + std::to_string(i)]; };
  auto B = [&](int i) -> Tensor& { return params["b" + std::to_string(i)]; };
  Tensor acts[12], sens[12];
  // FF
  acts[0] = data;
  acts[1] = ConvRelu(acts[0], W(0), B(0), convs[0]);   // conv1
  acts[2] = rt->PoolingForward(acts[1], poolings[0]);                           // pool1
  acts[3] = ConvRelu(acts[2], W(1), B(1), convs[1]);   // conv2
  acts[4] = rt->PoolingForward(acts[3], poolings[1]);                           // pool2
  acts[5] = ConvRelu(acts[4], W(2), B(2), convs[2]);   // conv3
  acts[6] = ConvRelu(acts[5], W(3), B(3), convs[3]);   // conv4
  acts[7] = ConvRelu(acts[6], W(4), B(4), convs[4]);   // conv5
  acts[8] = rt->PoolingForward(acts[7], poolings[2]);                           // pool5
  Tensor re8 = rt->Reshape(acts[8], Scale{acts[8]->size.Prod() / n, n});
  const bool drop = dropout_rate_ > 0.f;
  Tensor mask6, mask7;
  acts[9] = Fc(W(5), re8, B(5), true);                                        // fc6
  if (drop) {
    mask6 = rt->RandBernoulli(acts[9]->size, dropout_rate_);
    acts[9] = rt->Mult(acts[9], mask6);                                         // drop6
  }
  acts[10] = Fc(W(6), acts[9], B(6), true);                                   // fc7
  if (drop) {
    mask7 = rt->RandBernoulli(acts[10]->size, dropout_rate_);
    acts[10] = rt->Mult(acts[10], mask7);                                       // drop7
  }
  acts[11] = Fc(W(7), acts[10], B(7), false);                                                   // fc8
  Tensor out = rt->Reshape(
      rt->SoftmaxForward(rt->Reshape(acts[11], Scale{classes_, 1, 1, n}), SoftmaxAlgorithm::kInstance),
      Scale{classes_, n});
  results["prob"] = out;
  if (keep_activations)
    for (int i = 1; i <= 10; ++i) results["act" + std::to_string(i)] = acts[i];
  // BP
  sens[11] = rt->Sub(out, label);
  if (drop) {
    sens[10] = rt->Mult(TransMatMult(W(7), sens[11]), mask7);         // fc8, drop7
    sens[10] = rt->ReluBackward(sens[10], acts[10], acts[10]);                  // relu7
    sens[9] = rt->Mult(TransMatMult(W(6), sens[10]), mask6);          // fc7, drop6
    sens[9] = rt->ReluBackward(sens[9], acts[9], acts[9]);                      // relu6
  } else {
    sens[10] = TransMatMultReluBackward(W(7), sens[11], acts[10]);        // fc8, relu7
    sens[9] = TransMatMultReluBackward(W(6), sens[10], acts[9]);          // fc7, relu6
  }
  sens[8] = rt->Reshape(TransMatMult(W(5), sens[9]), acts[8]->size);
  sens[7] = PoolBackwardRelu(sens[8], acts[8], acts[7], poolings[2]);
  sens[6] = ConvBackwardDataRelu(sens[7], acts[6], W(4), convs[4]);
  sens[5] = ConvBackwardDataRelu(sens[6], acts[5], W(3), convs[3]);
  sens[4] = rt->ConvBackwardData(sens[5], acts[4], W(2), convs[2]);
  sens[3] = PoolBackwardRelu(sens[4], acts[4], acts[3], poolings[1]);
  sens[2] = rt->ConvBackwardData(sens[3], acts[2], W(1), convs[1]);
  sens[1] = PoolBackwardRelu(sens[2], acts[2], acts[1], poolings[0]);
  Tensor gb[8];
  gb[7] = rt->Sum(sens[11], 1);
  gb[6] = rt->Sum(sens[10], 1);
  gb[5] = rt->Sum(sens[9], 1);
  gb[4] = rt->ConvBackwardBias(sens[7]);
  gb[3] = rt->ConvBackwardBias(sens[6]);
  gb[2] = rt->ConvBackwardBias(sens[5]);
  gb[1] = rt->ConvBackwardBias(sens[3]);
  gb[0] = rt->ConvBackwardBias(sens[1]);
  // weight gradients and updates
  SgdFc("w7", sens[11], acts[10], lr);
  SgdFc("w6", sens[10], acts[9], lr);
  SgdFc("w5", sens[9], re8, lr);
  SgdConv("w4", sens[7], acts[6], convs[4], lr);
  SgdConv("w3", sens[6], acts[5], convs[3], lr);
  SgdConv("w2", sens[5], acts[4], convs[2], lr);
  SgdConv("w1", sens[3], acts[2], convs[1], lr);
  SgdConv("w0", sens[1], acts[0], convs[0], lr);
  for (int i = 0; i < 8; ++i) Sgd("b" + std::to_string(i), gb[i], lr);
}

}  // namespace minerva
