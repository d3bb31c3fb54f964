// A small sequential graph runner: the eager stand-in for Minerva's NArray front end
// and DAG scheduler, enough to drive the operator layer exactly the way the reference
// applications do.  Every call builds the same closure the reference's NArray method
// builds, derives the output extent with the same rule, wraps it in a Task and hands it
// to the HipDevice; a tensor frees its device data when its last handle dies, which is
// what the DAG's reference counting does.  Output-extent rules follow
//   convolution floor formula   minerva/narray/convolution.cpp:13-18
//   pooling ceil + clip         minerva/narray/convolution.cpp:107-114
//   broadcast dim detection     minerva/narray/narray.cpp:195-214
//   reductions                  minerva/narray/narray_reduction.cpp:14-51
#pragma once
#include <atomic>

#include "device_manager.h"
#include "hip_device.h"

namespace minerva {

class Runner;

struct TensorNode {
  TensorNode(Runner* r, uint64_t i, const Scale& s) : runner(r), id(i), size(s) {}
  ~TensorNode();
  Runner* runner;
  uint64_t id;
  Scale size;
  int stream = 0;      // the worker stream its producer ran on
  uint64_t seq = 0;    // how many operators that stream had been given when the producer was queued
  uint64_t epoch = 0;  // Sync count at that time: a tensor of an earlier epoch is complete
};
using Tensor = std::shared_ptr<TensorNode>;

class Runner : public DeviceListener {
 public:
  // dataflow: operators are spread over the device's four streams and ordered by events
  // (see PickStream); otherwise everything runs on stream 0 in program order.
  explicit Runner(int gpu_id, bool sync_each_op = true, bool dataflow = false,
                  size_t pool_bytes = HipDevice::kDefaultPoolBytes);
  ~Runner() override;
  void OnOperationComplete(Task*) override { ++ops_completed_; }

  HipDevice& device() { return *device_; }
  uint64_t ops_issued() const { return ops_issued_; }
  void Sync();
  // Overwrites `t` from host memory on worker stream `stream` while the other streams keep
  // running (HipDevice::CopyFromHostOn); the caller vouches that no queued work touches `t`.
  void UploadOn(int stream, const Tensor& t, const float* host);
  // Dataflow mode: the following operators go to worker stream `stream` (-1: placed
  // automatically again).  Dependencies on tensors of other streams are kept by events.
  void SetStream(int stream);
  // Switches between the one-stream order and dataflow placement; tensors stay valid.
  void SetDataflow(bool on);

  Tensor Compute(const std::vector<Tensor>& inputs, const Scale& out_size,
                 std::shared_ptr<ComputeFn> fn);
  std::vector<float> Get(const Tensor& t);
  void Read(const Tensor& t, float* host);  // the same into the caller's buffer
  // Overwrites a tensor's device data in place (synchronous); its address is kept, which
  // is what a recorded graph that reads it needs.
  void Upload(const Tensor& t, const float* host);
  // dst <- src, both alive, same extent; ordered after everything issued so far.
  void CopyInto(const Tensor& dst, const Tensor& src);
  // While retaining, every tensor Compute creates is kept alive by the runner, so no
  // device block is released or reused; EndRetain hands the kept tensors to the caller.
  // A recorded graph owns them for as long as it may be replayed.
  void BeginRetain();
  std::vector<Tensor> EndRetain();

  // data generators
  Tensor MakeNArray(const Scale& size, std::shared_ptr<float> host);
  // The loader runs before this returns (operators are issued from the caller's thread and
  // the loader waits for its copy), so the caller's buffer is read in place, not copied.
  Tensor MakeNArray(const Scale& size, const float* host);
  Tensor Constant(const Scale& size, float v);
  Tensor Zeros(const Scale& size) { return Constant(size, 0.f); }
  // reference minerva/narray/narray.cpp:21-33
  Tensor Randn(const Scale& size, float mu, float var);
  Tensor RandBernoulli(const Scale& size, float p);

  // NArray arithmetic
  Tensor Arithmetic(const Tensor& a, const Tensor& b, ArithmeticType t);
  Tensor Add(const Tensor& a, const Tensor& b) { return Arithmetic(a, b, ArithmeticType::kAdd); }
  Tensor Sub(const Tensor& a, const Tensor& b) { return Arithmetic(a, b, ArithmeticType::kSub); }
  Tensor Mult(const Tensor& a, const Tensor& b) { return Arithmetic(a, b, ArithmeticType::kMult); }
  Tensor Div(const Tensor& a, const Tensor& b) { return Arithmetic(a, b, ArithmeticType::kDiv); }
  Tensor ArithmeticConst(const Tensor& a, float v, ArithmeticType t, int side);
  Tensor Elewise(const Tensor& a, ElewiseType t);
  Tensor NormArithmetic(const Tensor& lhs, const Tensor& rhs, ArithmeticType t);
  Tensor MatMult(const Tensor& a, const Tensor& b);
  Tensor Trans(const Tensor& a);
  Tensor Reshape(const Tensor& a, const Scale& size);
  Tensor Reduce(const Tensor& a, int dim, ReductionType t);
  Tensor Sum(const Tensor& a, int dim) { return Reduce(a, dim, ReductionType::kSum); }
  Tensor Max(const Tensor& a, int dim) { return Reduce(a, dim, ReductionType::kMax); }
  Tensor MaxIndex(const Tensor& a, int dim);

  // Elewise:: and Convolution::
  Tensor SigmoidForward(const Tensor& a);
  Tensor ReluForward(const Tensor& a);
  Tensor TanhForward(const Tensor& a);
  Tensor SigmoidBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom);
  Tensor ReluBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom);
  Tensor TanhBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom);
  Tensor ActivationForward(const Tensor& a, ActivationAlgorithm alg);
  Tensor ActivationBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                            ActivationAlgorithm alg);
  Tensor SoftmaxForward(const Tensor& a, SoftmaxAlgorithm alg);
  Tensor SoftmaxBackward(const Tensor& diff, const Tensor& top, SoftmaxAlgorithm alg);
  Tensor ConvForward(const Tensor& src, const Tensor& filter, const Tensor& bias, ConvInfo info);
  Tensor ConvBackwardData(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                          ConvInfo info);
  Tensor ConvBackwardFilter(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                            ConvInfo info);
  Tensor ConvBackwardBias(const Tensor& diff);
  Tensor PoolingForward(const Tensor& src, PoolingInfo info);
  Tensor PoolingBackward(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                         PoolingInfo info);
  // reference minerva/narray/narray.cpp:129-160, 183-192
  Tensor ThresholdNorm(const Tensor& a, float threshold);
  Tensor Index(const Tensor& a, int idx, const Scale& block);  // the idx-th `block`-sized piece
  Tensor Concat(const std::vector<Tensor>& arrays, int catdim);
  Tensor Slice(const Tensor& src, int slice_dim, int st_off, int slice_count);
  Tensor Select(const Tensor& src, const std::vector<int>& indices);
  // reference minerva/narray/convolution.cpp:165-175; `scale` is filled by the forward pass
  Tensor LRNForward(const Tensor& src, const Tensor& scale, int local_size, float alpha,
                    float beta);
  Tensor LRNBackward(const Tensor& bottom, const Tensor& top, const Tensor& scale,
                     const Tensor& top_diff, int local_size, float alpha, float beta);

  // The opt-in fused operators (hip_fused_ops.h).  Each returns the bits of the pair of calls
  // named in its comment.
  // ReluForward(ConvForward(src, filter, bias, info))
  Tensor ConvForwardRelu(const Tensor& src, const Tensor& filter, const Tensor& bias, ConvInfo info);
  // ReluBackward(ConvBackwardData(diff, bottom, filter, info), bottom, bottom)
  Tensor ConvBackwardDataRelu(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                              ConvInfo info);
  // ReluBackward(PoolingBackward(diff, top, bottom, info), bottom, bottom); max pooling only
  Tensor PoolingBackwardRelu(const Tensor& diff, const Tensor& top, const Tensor& bottom,
                             PoolingInfo info);
  // [ReluForward](NormArithmetic(MatMult(a, b), bias{m,1}, add))
  Tensor MatMultBias(const Tensor& a, const Tensor& b, const Tensor& bias, bool relu);
  // ReluBackward(MatMult(a, b), bottom, bottom)
  Tensor MatMultReluBackward(const Tensor& a, const Tensor& b, const Tensor& bottom);
  // MatMult(Trans(at), b), or with a gate ReluBackward(MatMult(Trans(at), b), bottom, bottom)
  Tensor MatMultTransA(const Tensor& at, const Tensor& b, const Tensor& bottom = Tensor());
  // MatMult(a, Trans(bt))
  Tensor MatMultTransB(const Tensor& a, const Tensor& bt);
  // Sub(w, ArithmeticConst(g, scale, mult))
  Tensor SgdUpdate(const Tensor& w, const Tensor& g, float scale);
  // w - scale * (a * bt^T) and filter - scale * ConvBackwardFilter(diff, bottom): the update
  // applied where the gradient is produced
  Tensor MatMultTransBSgd(const Tensor& a, const Tensor& bt, const Tensor& w, float scale);
  Tensor ConvBackwardFilterSgd(const Tensor& diff, const Tensor& bottom, const Tensor& filter,
                               ConvInfo info, float scale);

 private:
  friend struct TensorNode;
  // the devices live in a manager, as in the reference's MinervaSystem (system/minerva_system.cpp:84);
  // this runner drives the one GPU device it created there
  std::unique_ptr<DeviceManager> manager_;
  HipDevice* device_ = nullptr;
  std::atomic<uint64_t> next_id_{1};
  std::atomic<uint64_t> ops_issued_{0}, ops_completed_{0};
  bool retain_ = false;
  std::vector<Tensor> retained_;
  // Dataflow placement.  An operator follows its newest input that is still in flight onto
  // that input's stream, so a chain and its side branches stay together and stream order does
  // the waiting (on one GPU the branches of a training graph compete for the same CUs: spread
  // over streams they gained nothing and every cross-stream edge cost an event and a wait).
  // An operator whose inputs are all complete (weights of the last step, a resident batch)
  // joins the stream that was given the operator before it.  Only a large operator without
  // inputs (the load of the next batch) goes to the stream with the least queued since the last
  // Sync.  A caller that knows two chains to be independent says so with SetStream, the
  // counterpart on one device of the reference's owl.set_device (owl/owl/__init__.py).
  static constexpr size_t kForkBytes = (size_t)32 << 20;
  int PickStream(const std::vector<Tensor>& inputs, const Scale& out_size);
  bool dataflow_ = false;
  uint64_t issued_[HipDevice::kParallelism] = {};  // operators ever queued per stream
  uint64_t queued_[HipDevice::kParallelism] = {};  // operators queued per stream since Sync
  uint64_t epoch_ = 1;                             // Syncs so far + 1
  int last_stream_ = 0;                            // stream of the operator queued last
  int forced_stream_ = -1;                         // SetStream: where the caller wants the next operators
};

}  // namespace minerva
