#include "runner.h"

#include <cstring>

namespace minerva {

TensorNode::~TensorNode() {
  if (runner && runner->manager_) runner->manager_->FreeData(id);
}

Runner::Runner(int gpu_id, bool sync_each_op, bool dataflow, size_t pool_bytes)
    : dataflow_(dataflow) {
  manager_.reset(new DeviceManager(pool_bytes));
  manager_->RegisterListener(this);
  device_ = static_cast<HipDevice*>(manager_->GetDevice(manager_->CreateGpuDevice(gpu_id)));
  device_->set_sync_each_op(sync_each_op);
  if (dataflow) device_->set_dataflow(true);
}

void Runner::Sync() {
  device_->Barrier(0);
  for (auto& q : queued_) q = 0;
  ++epoch_;
}

void Runner::SetDataflow(bool on) {
  Sync();
  device_->set_dataflow(on);
  if (!on) device_->set_sync_each_op(false);
  if (!on) forced_stream_ = -1;
  dataflow_ = on;
}

int Runner::PickStream(const std::vector<Tensor>& inputs, const Scale& out_size) {
  if (forced_stream_ >= 0) return forced_stream_;
  const TensorNode* newest = nullptr;
  for (auto& t : inputs)
    if (t->epoch == epoch_ && (!newest || t->id > newest->id)) newest = t.get();
  if (newest) return newest->stream;
  // inputs, but none in flight (weights of the last step, a resident batch): what this
  // operator makes is most likely for the chain that is being queued right now
  if (!inputs.empty()) return last_stream_;
  // no inputs: a load or a fill.  A large one depends on nothing that is queued and goes
  // where the least is queued; a small one is not worth an event and a wait later on
  if (static_cast<size_t>(out_size.Prod()) * sizeof(float) < kForkBytes) return last_stream_;
  int pick = 0;
  for (int s = 1; s < static_cast<int>(HipDevice::kParallelism); ++s)
    if (queued_[s] < queued_[pick]) pick = s;
  return pick;
}

void Runner::SetStream(int stream) {
  MNV_CHECK(stream >= -1 && stream < static_cast<int>(HipDevice::kParallelism)) << "bad stream";
  MNV_CHECK(stream < 0 || dataflow_) << "operators are placed on streams in dataflow mode only";
  forced_stream_ = stream;
}

Runner::~Runner() {
  device_->WaitForAllFinished();
}

Tensor Runner::Compute(const std::vector<Tensor>& inputs, const Scale& out_size,
                       std::shared_ptr<ComputeFn> fn) {
  Task task;
  for (auto& t : inputs) {
    MNV_CHECK(t) << "null tensor";
    task.inputs.emplace_back(PhysicalData(t->size, device_->device_id(), t->id), t->id);
  }
  Tensor out = std::make_shared<TensorNode>(this, next_id_++, out_size);
  task.outputs.emplace_back(PhysicalData(out_size, device_->device_id(), out->id), out->id);
  task.op.compute_fn = std::move(fn);
  task.op.device_id = device_->device_id();
  task.id = ops_issued_++;
  task.light = true;  // issued in program order from the caller's thread
  if (dataflow_) {
    task.stream = out->stream = PickStream(inputs, out_size);
    last_stream_ = task.stream;
    out->seq = ++issued_[task.stream];
    out->epoch = epoch_;
    ++queued_[task.stream];
  }
  device_->PushTask(&task);
  if (retain_) retained_.push_back(out);
  return out;
}

void Runner::Upload(const Tensor& t, const float* host) {
  MNV_CHECK(t && host) << "null argument";
  device_->Barrier(0);
  device_->CopyFromHost(t->id, host, t->size.Prod());
}

void Runner::UploadOn(int stream, const Tensor& t, const float* host) {
  MNV_CHECK(t && host) << "null argument";
  device_->CopyFromHostOn(stream, t->id, host, t->size.Prod());
}

void Runner::CopyInto(const Tensor& dst, const Tensor& src) {
  MNV_CHECK(dst && src && dst->size == src->size) << "extents differ";
  device_->CopyOnDevice(dst->id, src->id, src->size.Prod());
}

void Runner::BeginRetain() {
  MNV_CHECK(!retain_) << "already retaining";
  retain_ = true;
}

std::vector<Tensor> Runner::EndRetain() {
  retain_ = false;
  std::vector<Tensor> kept;
  kept.swap(retained_);
  return kept;
}

std::vector<float> Runner::Get(const Tensor& t) {
  std::vector<float> host(t->size.Prod());
  Read(t, host.data());
  return host;
}

void Runner::Read(const Tensor& t, float* host) {
  MNV_CHECK(t && host) << "null argument";
  device_->Barrier(0);
  device_->CopyToHost(host, t->id, t->size.Prod());
}

Tensor Runner::MakeNArray(const Scale& size, std::shared_ptr<float> host) {
  auto op = std::make_shared<ArrayLoaderOp>();
  op->closure.data = std::move(host);
  return Compute({}, size, op);
}

Tensor Runner::MakeNArray(const Scale& size, const float* host) {
  MNV_CHECK(host) << "null host data";
  std::shared_ptr<float> borrowed(const_cast<float*>(host), [](float*) {});
  return MakeNArray(size, borrowed);
}

Tensor Runner::Constant(const Scale& size, float v) {
  auto op = std::make_shared<FillOp>();
  op->closure.val = v;
  return Compute({}, size, op);
}

Tensor Runner::Randn(const Scale& size, float mu, float var) {
  auto op = std::make_shared<RandnOp>();
  op->closure = {mu, var};
  return Compute({}, size, op);
}

Tensor Runner::RandBernoulli(const Scale& size, float p) {
  MNV_CHECK(p >= 0.f && p <= 1.f) << "probability out of range: " << p;
  auto op = std::make_shared<RandBernoulliOp>();
  op->closure = {p};
  return Compute({}, size, op);
}

Tensor Runner::Arithmetic(const Tensor& a, const Tensor& b, ArithmeticType t) {
  MNV_CHECK(a->size == b->size) << "size must match " << a->size << " " << b->size;
  auto op = std::make_shared<ArithmeticOp>();
  op->closure.type = t;
  return Compute({a, b}, a->size, op);
}

Tensor Runner::ArithmeticConst(const Tensor& a, float v, ArithmeticType t, int side) {
  auto op = std::make_shared<ArithmeticConstOp>();
  op->closure = {t, v, side};
  return Compute({a}, a->size, op);
}

Tensor Runner::Elewise(const Tensor& a, ElewiseType t) {
  auto op = std::make_shared<ElewiseOp>();
  op->closure.type = t;
  return Compute({a}, a->size, op);
}

Tensor Runner::NormArithmetic(const Tensor& lhs, const Tensor& rhs, ArithmeticType t) {
  MNV_CHECK_EQ(lhs->size.NumDims(), rhs->size.NumDims()) << "#dimension mismatch";
  std::vector<int> rep;
  for (size_t i = 0; i < lhs->size.NumDims(); ++i) {
    if (lhs->size[i] == rhs->size[i]) continue;
    MNV_CHECK_EQ(rhs->size[i], 1) << "NormArithmetic cannot replicate a dimension that is not 1";
    rep.push_back(static_cast<int>(i));
  }
  MNV_CHECK(!rep.empty()) << "nothing to replicate";
  auto op = std::make_shared<NormArithmeticOp>();
  op->closure.type = t;
  op->closure.dims_to_replicate = Scale(rep);
  return Compute({lhs, rhs}, lhs->size, op);
}

Tensor Runner::MatMult(const Tensor& a, const Tensor& b) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(b->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(a->size[1], b->size[0]) << "size must match";
  return Compute({a, b}, Scale{a->size[0], b->size[1]}, std::make_shared<MatMultOp>());
}

Tensor Runner::Trans(const Tensor& a) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  return Compute({a}, Scale{a->size[1], a->size[0]}, std::make_shared<TransOp>());
}

Tensor Runner::Reshape(const Tensor& a, const Scale& size) {
  MNV_CHECK_EQ(a->size.Prod(), size.Prod()) << "reshape must keep the element count";
  return Compute({a}, size, std::make_shared<ReshapeOp>());
}

Tensor Runner::Reduce(const Tensor& a, int dim, ReductionType t) {
  MNV_CHECK(0 <= dim && dim < static_cast<int>(a->size.NumDims())) << "dim out of bound";
  Scale size = a->size;
  size[dim] = 1;
  auto op = std::make_shared<ReductionOp>();
  op->closure.type = t;
  op->closure.dims_to_reduce = Scale{dim};
  return Compute({a}, size, op);
}

Tensor Runner::MaxIndex(const Tensor& a, int dim) {
  MNV_CHECK(0 <= dim && dim < static_cast<int>(a->size.NumDims())) << "dim out of bound";
  Scale size = a->size;
  size[dim] = 1;
  auto op = std::make_shared<MaxIndexOp>();
  op->closure.dim = dim;
  return Compute({a}, size, op);
}

Tensor Runner::SigmoidForward(const Tensor& a) { return Compute({a}, a->size, std::make_shared<SigmoidForwardOp>()); }
Tensor Runner::ReluForward(const Tensor& a) { return Compute({a}, a->size, std::make_shared<ReluForwardOp>()); }
Tensor Runner::TanhForward(const Tensor& a) { return Compute({a}, a->size, std::make_shared<TanhForwardOp>()); }

static void CheckSame(const Tensor& a, const Tensor& b) {
  MNV_CHECK(a->size == b->size) << "inputs sizes mismatch";
}

Tensor Runner::SigmoidBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom) {
  CheckSame(diff, top); CheckSame(diff, bottom);
  return Compute({diff, top, bottom}, diff->size, std::make_shared<SigmoidBackwardOp>());
}
Tensor Runner::ReluBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom) {
  CheckSame(diff, top); CheckSame(diff, bottom);
  return Compute({diff, top, bottom}, diff->size, std::make_shared<ReluBackwardOp>());
}
Tensor Runner::TanhBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom) {
  CheckSame(diff, top); CheckSame(diff, bottom);
  return Compute({diff, top, bottom}, diff->size, std::make_shared<TanhBackwardOp>());
}

Tensor Runner::ActivationForward(const Tensor& a, ActivationAlgorithm alg) {
  auto op = std::make_shared<ActivationForwardOp>();
  op->closure.algorithm = alg;
  return Compute({a}, a->size, op);
}

Tensor Runner::ActivationBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                                  ActivationAlgorithm alg) {
  CheckSame(diff, top); CheckSame(diff, bottom);
  auto op = std::make_shared<ActivationBackwardOp>();
  op->closure.algorithm = alg;
  return Compute({diff, top, bottom}, diff->size, op);
}

Tensor Runner::SoftmaxForward(const Tensor& a, SoftmaxAlgorithm alg) {
  auto op = std::make_shared<SoftmaxForwardOp>();
  op->closure.algorithm = alg;
  return Compute({a}, a->size, op);
}

Tensor Runner::SoftmaxBackward(const Tensor& diff, const Tensor& top, SoftmaxAlgorithm alg) {
  CheckSame(diff, top);
  auto op = std::make_shared<SoftmaxBackwardOp>();
  op->closure.algorithm = alg;
  return Compute({diff, top}, diff->size, op);
}

Tensor Runner::ConvForward(const Tensor& src, const Tensor& filter, const Tensor& bias,
                           ConvInfo info) {
  MNV_CHECK_EQ(src->size.NumDims(), 4u);
  MNV_CHECK_EQ(filter->size.NumDims(), 4u);
  MNV_CHECK_EQ(src->size[2], filter->size[2]) << "#input channels mismatch";
  MNV_CHECK_EQ(bias->size.NumDims(), 1u) << "bias dimension mismatch";
  MNV_CHECK_EQ(bias->size[0], filter->size[3]) << "bias size mismatch";
  Scale out{(src->size[0] + 2 * info.pad_width - filter->size[0]) / info.stride_horizontal + 1,
            (src->size[1] + 2 * info.pad_height - filter->size[1]) / info.stride_vertical + 1,
            filter->size[3], src->size[3]};
  auto op = std::make_shared<ConvForwardOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal};
  return Compute({src, filter, bias}, out, op);
}

Tensor Runner::ConvBackwardData(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                                ConvInfo info) {
  MNV_CHECK_EQ(diff->size[2], filter->size[3]) << "#output channels mismatch";
  auto op = std::make_shared<ConvBackwardDataOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal};
  return Compute({diff, filter}, bottom->size, op);
}

Tensor Runner::ConvBackwardFilter(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                                  ConvInfo info) {
  MNV_CHECK_EQ(diff->size[3], bottom->size[3]) << "#images mismatch";
  auto op = std::make_shared<ConvBackwardFilterOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal};
  return Compute({diff, bottom}, filter->size, op);
}

Tensor Runner::ConvBackwardBias(const Tensor& diff) {
  return Compute({diff}, Scale{diff->size[2]}, std::make_shared<ConvBackwardBiasOp>());
}

static int PooledSize(int in, int win, int stride, int pad) {
  int p = (in + 2 * pad - win + stride - 1) / stride + 1;
  if (0 <= (p - 1) * stride - in - pad) --p;
  return p;
}

Tensor Runner::PoolingForward(const Tensor& src, PoolingInfo info) {
  MNV_CHECK_EQ(src->size.NumDims(), 4u);
  Scale out{PooledSize(src->size[0], info.width, info.stride_horizontal, info.pad_width),
            PooledSize(src->size[1], info.height, info.stride_vertical, info.pad_height),
            src->size[2], src->size[3]};
  auto op = std::make_shared<PoolingForwardOp>();
  op->closure = {info.algorithm, info.height, info.width, info.stride_vertical,
                 info.stride_horizontal, info.pad_height, info.pad_width};
  return Compute({src}, out, op);
}

Tensor Runner::PoolingBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                               PoolingInfo info) {
  CheckSame(diff, top);
  auto op = std::make_shared<PoolingBackwardOp>();
  op->closure = {info.algorithm, info.height, info.width, info.stride_vertical,
                 info.stride_horizontal, info.pad_height, info.pad_width};
  return Compute({diff, top, bottom}, bottom->size, op);
}

Tensor Runner::ThresholdNorm(const Tensor& a, float threshold) {
  auto op = std::make_shared<ThresholdNormOp>();
  op->closure = {threshold};
  return Compute({a}, a->size, op);
}

Tensor Runner::Index(const Tensor& a, int idx, const Scale& block) {
  auto op = std::make_shared<IndexOp>();
  op->closure = {idx};
  return Compute({a}, block, op);
}

Tensor Runner::Concat(const std::vector<Tensor>& arrays, int catdim) {
  MNV_CHECK_GT(arrays.size(), 1u) << "Concat more than one narray";
  MNV_CHECK(catdim >= 0 && arrays[0]->size.NumDims() > static_cast<size_t>(catdim))
      << "can't concat on non-sense dim";
  std::vector<int> dims(arrays[0]->size.NumDims());
  int target = 0;
  for (auto& a : arrays) {
    MNV_CHECK_EQ(a->size.NumDims(), dims.size()) << "rank mismatch";
    target += a->size[catdim];
  }
  for (size_t i = 0; i < dims.size(); ++i)
    dims[i] = i == static_cast<size_t>(catdim) ? target : arrays[0]->size[i];
  auto op = std::make_shared<ConcatOp>();
  op->closure = {catdim};
  return Compute(arrays, Scale(dims), op);
}

Tensor Runner::Slice(const Tensor& src, int slice_dim, int st_off, int slice_count) {
  MNV_CHECK(slice_dim >= 0 && src->size.NumDims() > static_cast<size_t>(slice_dim))
      << "can't slice on non-sense dim";
  std::vector<int> dims(src->size.NumDims());
  for (size_t i = 0; i < dims.size(); ++i)
    dims[i] = i == static_cast<size_t>(slice_dim) ? slice_count : src->size[i];
  auto op = std::make_shared<SliceOp>();
  op->closure = {slice_dim, st_off, slice_count};
  return Compute({src}, Scale(dims), op);
}

// The reference's NArray::Select never hands its indices to the operator (narray.cpp:190
// leaves the closure empty); here they are.
Tensor Runner::Select(const Tensor& src, const std::vector<int>& indices) {
  MNV_CHECK_EQ(src->size.NumDims(), 2u);
  MNV_CHECK_LT(0u, indices.size());
  for (auto i : indices) MNV_CHECK(i >= 0 && i < src->size[1]) << "index " << i << " out of range";
  auto op = std::make_shared<SelectOp>();
  op->closure = {indices};
  return Compute({src}, Scale{src->size[0], static_cast<int>(indices.size())}, op);
}

Tensor Runner::LRNForward(const Tensor& src, const Tensor& scale, int local_size, float alpha,
                          float beta) {
  MNV_CHECK_EQ(src->size.NumDims(), 4u);
  CheckSame(src, scale);
  auto op = std::make_shared<LRNForwardOp>();
  op->closure = {local_size, alpha, beta, src->size};
  return Compute({src, scale}, src->size, op);
}

Tensor Runner::LRNBackward(const Tensor& bottom, const Tensor& top, const Tensor& scale,
                           const Tensor& top_diff, int local_size, float alpha, float beta) {
  MNV_CHECK_EQ(bottom->size.NumDims(), 4u);
  CheckSame(bottom, top);
  CheckSame(bottom, scale);
  CheckSame(bottom, top_diff);
  auto op = std::make_shared<LRNBackwardOp>();
  op->closure = {local_size, alpha, beta, bottom->size};
  return Compute({bottom, top, scale, top_diff}, bottom->size, op);
}

// ---------------------------------------------------------------- fused operators

Tensor Runner::ConvForwardRelu(const Tensor& src, const Tensor& filter, const Tensor& bias,
                               ConvInfo info) {
  MNV_CHECK_EQ(src->size.NumDims(), 4u);
  MNV_CHECK_EQ(filter->size.NumDims(), 4u);
  MNV_CHECK_EQ(src->size[2], filter->size[2]) << "#input channels mismatch";
  MNV_CHECK_EQ(bias->size.NumDims(), 1u) << "bias dimension mismatch";
  MNV_CHECK_EQ(bias->size[0], filter->size[3]) << "bias size mismatch";
  Scale out{(src->size[0] + 2 * info.pad_width - filter->size[0]) / info.stride_horizontal + 1,
            (src->size[1] + 2 * info.pad_height - filter->size[1]) / info.stride_vertical + 1,
            filter->size[3], src->size[3]};
  auto op = std::make_shared<ConvForwardReluOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal};
  return Compute({src, filter, bias}, out, op);
}

Tensor Runner::ConvBackwardDataRelu(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                                    ConvInfo info) {
  MNV_CHECK_EQ(diff->size[2], filter->size[3]) << "#output channels mismatch";
  auto op = std::make_shared<ConvBackwardDataReluOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal};
  return Compute({diff, filter, bottom}, bottom->size, op);
}

Tensor Runner::PoolingBackwardRelu(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                                   PoolingInfo info) {
  CheckSame(diff, top);
  MNV_CHECK(info.algorithm == PoolingInfo::Algorithm::kMax) << "fused only for max pooling";
  auto op = std::make_shared<PoolingBackwardReluOp>();
  op->closure = {info.height, info.width, info.stride_vertical, info.stride_horizontal,
                 info.pad_height, info.pad_width};
  return Compute({diff, top, bottom}, bottom->size, op);
}

Tensor Runner::MatMultBias(const Tensor& a, const Tensor& b, const Tensor& bias, bool relu) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(b->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(a->size[1], b->size[0]) << "size must match";
  MNV_CHECK(bias->size == (Scale{a->size[0], 1})) << "bias must be {m,1}";
  auto op = std::make_shared<MatMultBiasOp>();
  op->closure = {relu};
  return Compute({a, b, bias}, Scale{a->size[0], b->size[1]}, op);
}

Tensor Runner::MatMultReluBackward(const Tensor& a, const Tensor& b, const Tensor& bottom) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(b->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(a->size[1], b->size[0]) << "size must match";
  MNV_CHECK(bottom->size == (Scale{a->size[0], b->size[1]})) << "gate extent must match the product";
  return Compute({a, b, bottom}, bottom->size, std::make_shared<MatMultReluBackwardOp>());
}

Tensor Runner::MatMultTransA(const Tensor& at, const Tensor& b, const Tensor& bottom) {
  MNV_CHECK_EQ(at->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(b->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(at->size[0], b->size[0]) << "size must match";
  const Scale out{at->size[1], b->size[1]};
  if (!bottom) return Compute({at, b}, out, std::make_shared<MatMultTransAOp>());
  MNV_CHECK(bottom->size == out) << "gate extent must match the product";
  return Compute({at, b, bottom}, out, std::make_shared<MatMultTransAOp>());
}

Tensor Runner::MatMultTransB(const Tensor& a, const Tensor& bt) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(bt->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(a->size[1], bt->size[1]) << "size must match";
  return Compute({a, bt}, Scale{a->size[0], bt->size[0]}, std::make_shared<MatMultTransBOp>());
}

Tensor Runner::SgdUpdate(const Tensor& w, const Tensor& g, float scale) {
  MNV_CHECK_EQ(w->size.Prod(), g->size.Prod()) << "parameter and gradient differ in size";
  auto op = std::make_shared<SgdUpdateOp>();
  op->closure = {scale};
  return Compute({w, g}, w->size, op);
}

Tensor Runner::MatMultTransBSgd(const Tensor& a, const Tensor& bt, const Tensor& w, float scale) {
  MNV_CHECK_EQ(a->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(bt->size.NumDims(), 2u) << "eligible only for 2D";
  MNV_CHECK_EQ(a->size[1], bt->size[1]) << "size must match";
  MNV_CHECK(w->size == (Scale{a->size[0], bt->size[0]})) << "parameter extent must match the product";
  auto op = std::make_shared<MatMultTransBSgdOp>();
  op->closure = {scale};
  return Compute({a, bt, w}, w->size, op);
}

Tensor Runner::ConvBackwardFilterSgd(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                                     ConvInfo info, float scale) {
  MNV_CHECK_EQ(diff->size[3], bottom->size[3]) << "#images mismatch";
  auto op = std::make_shared<ConvBackwardFilterSgdOp>();
  op->closure = {info.pad_height, info.pad_width, info.stride_vertical, info.stride_horizontal, scale};
  return Compute({diff, bottom, filter}, filter->size, op);
}

}  // namespace minerva
