#include "hip_fused_ops.h"

#include "mnv_hip.h"

namespace minerva {
namespace hip {

namespace {
void Ok(int status, const char* what) {
  MNV_CHECK(status == MNV_OK) << what << ": " << mnv_error_string(status);
}
}  // namespace

void ConvForwardRelu(const DataList& inputs, const DataList& outputs, ConvForwardReluClosure& c,
                     const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(conv forward + relu) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv forward + relu) #outputs wrong";
  auto& bottom = inputs[0];
  auto& filter = inputs[1];
  auto& bias = inputs[2];
  auto& top = outputs[0];
  MNV_CHECK_EQ(bottom.size_[2], filter.size_[2]) << "#input channels mismatch";
  Ok(mnv_conv_fwd_relu(bottom.data_, filter.data_, bias.data_, top.data_, bottom.size_[3],
                       bottom.size_[2], top.size_[2], bottom.size_[1], bottom.size_[0],
                       c.pad_height, c.pad_width, c.stride_vertical, c.stride_horizontal,
                       filter.size_[1], filter.size_[0], ctx.workspace, ctx.workspace_bytes,
                       ctx.stream),
     "conv forward + relu");
}

void ConvBackwardDataRelu(const DataList& inputs, const DataList& outputs,
                          ConvBackwardDataReluClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(conv backward data + relu) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv backward data + relu) #outputs wrong";
  auto& top_diff = inputs[0];
  auto& filter = inputs[1];
  auto& bottom = inputs[2];
  auto& bottom_diff = outputs[0];
  MNV_CHECK(bottom.size_ == bottom_diff.size_) << "gate and gradient extents differ";
  Ok(mnv_conv_bwd_data_relu(top_diff.data_, filter.data_, bottom.data_, bottom_diff.data_,
                            top_diff.size_[3], bottom_diff.size_[2], top_diff.size_[2],
                            bottom_diff.size_[1], bottom_diff.size_[0], c.pad_height, c.pad_width,
                            c.stride_vertical, c.stride_horizontal, filter.size_[1],
                            filter.size_[0], ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "conv backward data + relu");
}

void PoolingBackwardRelu(const DataList& inputs, const DataList& outputs,
                         PoolingBackwardReluClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(pooling backward + relu) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(pooling backward + relu) #outputs wrong";
  auto& td = inputs[0];
  auto& top = inputs[1];
  auto& b = inputs[2];
  Ok(mnv_maxpool_bwd_relu(b.data_, top.data_, td.data_, outputs[0].data_, td.size_[3], td.size_[2],
                          b.size_[1], b.size_[0], c.stride_vertical, c.stride_horizontal, c.height,
                          c.width, c.pad_height, c.pad_width, ctx.stream),
     "pooling backward + relu");
}

void MatMultBias(const DataList& inputs, const DataList& outputs, MatMultBiasClosure& c,
                 const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(matmult + bias) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(matmult + bias) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int k = inputs[0].size_[1];
  int n = outputs[0].size_[1];
  MNV_CHECK_EQ(inputs[1].size_[0], k) << "(matmult + bias) inner dimensions differ";
  MNV_CHECK_EQ(inputs[2].size_.Prod(), m) << "(matmult + bias) bias must have one entry per row";
  Ok(mnv_sgemm_nn_bias(inputs[0].data_, inputs[1].data_, inputs[2].data_, outputs[0].data_, m, n, k,
                       c.relu ? 1 : 0, ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "sgemm + bias");
}

void MatMultReluBackward(const DataList& inputs, const DataList& outputs,
                         MatMultReluBackwardClosure&, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(matmult + relu backward) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(matmult + relu backward) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int k = inputs[0].size_[1];
  int n = outputs[0].size_[1];
  MNV_CHECK_EQ(inputs[1].size_[0], k) << "(matmult + relu backward) inner dimensions differ";
  MNV_CHECK(inputs[2].size_ == outputs[0].size_) << "gate and product extents differ";
  Ok(mnv_sgemm_nn_relu_bwd(inputs[0].data_, inputs[1].data_, inputs[2].data_, outputs[0].data_, m,
                           n, k, ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "sgemm + relu backward");
}

void MatMultTransA(const DataList& inputs, const DataList& outputs, MatMultTransAClosure&,
                   const Context& ctx) {
  MNV_CHECK(inputs.size() == 2u || inputs.size() == 3u) << "(transposed matmult) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(transposed matmult) #outputs is wrong!";
  int k = inputs[0].size_[0];
  int m = inputs[0].size_[1];
  int n = outputs[0].size_[1];
  MNV_CHECK_EQ(inputs[1].size_[0], k) << "(transposed matmult) inner dimensions differ";
  const float* gate = nullptr;
  if (inputs.size() == 3u) {
    MNV_CHECK(inputs[2].size_ == outputs[0].size_) << "gate and product extents differ";
    gate = inputs[2].data_;
  }
  Ok(mnv_sgemm_tn(inputs[0].data_, inputs[1].data_, gate, outputs[0].data_, m, n, k, ctx.workspace,
                  ctx.workspace_bytes, ctx.stream),
     "sgemm, left operand transposed");
}

void MatMultTransB(const DataList& inputs, const DataList& outputs, MatMultTransBClosure&,
                   const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(matmult transposed) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(matmult transposed) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int k = inputs[0].size_[1];
  int n = inputs[1].size_[0];
  MNV_CHECK_EQ(inputs[1].size_[1], k) << "(matmult transposed) inner dimensions differ";
  Ok(mnv_sgemm_nt(inputs[0].data_, inputs[1].data_, outputs[0].data_, m, n, k, ctx.workspace,
                  ctx.workspace_bytes, ctx.stream),
     "sgemm, right operand transposed");
}

void SgdUpdate(const DataList& inputs, const DataList& outputs, SgdUpdateClosure& c,
               const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 2u) << "(sgd update) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(sgd update) #outputs is wrong!";
  MNV_CHECK_EQ(inputs[0].size_.Prod(), inputs[1].size_.Prod()) << "parameter and gradient differ";
  Ok(mnv_sgd_update(inputs[0].data_, inputs[1].data_, c.scale, outputs[0].data_,
                    outputs[0].size_.Prod(), ctx.stream),
     "sgd update");
}

void MatMultTransBSgd(const DataList& inputs, const DataList& outputs, MatMultTransBSgdClosure& c,
                      const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(matmult transposed + sgd) #inputs is wrong!";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(matmult transposed + sgd) #outputs is wrong!";
  int m = inputs[0].size_[0];
  int k = inputs[0].size_[1];
  int n = inputs[1].size_[0];
  MNV_CHECK_EQ(inputs[1].size_[1], k) << "(matmult transposed + sgd) inner dimensions differ";
  MNV_CHECK(inputs[2].size_ == (Scale{m, n})) << "parameter and gradient differ";
  Ok(mnv_sgemm_nt_sgd(inputs[0].data_, inputs[1].data_, inputs[2].data_, c.scale, outputs[0].data_,
                      m, n, k, ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "sgemm, right operand transposed, + sgd update");
}

void ConvBackwardFilterSgd(const DataList& inputs, const DataList& outputs,
                           ConvBackwardFilterSgdClosure& c, const Context& ctx) {
  MNV_CHECK_EQ(inputs.size(), 3u) << "(conv backward filter + sgd) #inputs wrong";
  MNV_CHECK_EQ(outputs.size(), 1u) << "(conv backward filter + sgd) #outputs wrong";
  auto& top_diff = inputs[0];
  auto& bottom = inputs[1];
  auto& filter = inputs[2];
  MNV_CHECK(filter.size_ == outputs[0].size_) << "parameter and result differ";
  Ok(mnv_conv_bwd_filter_sgd(bottom.data_, top_diff.data_, filter.data_, c.scale, outputs[0].data_,
                             top_diff.size_[3], bottom.size_[2], top_diff.size_[2],
                             bottom.size_[1], bottom.size_[0], c.pad_height, c.pad_width,
                             c.stride_vertical, c.stride_horizontal, filter.size_[1],
                             filter.size_[0], ctx.workspace, ctx.workspace_bytes, ctx.stream),
     "conv backward filter + sgd update");
}

}  // namespace hip
}  // namespace minerva
