// C entry points of the host layer (include/mnv_host.h).
#include <cstring>
#include <string>

#include "mnv_hip.h"
#include "mnv_host.h"
#include "nets.h"

using namespace minerva;

namespace {

thread_local std::string g_error;

struct NetHandle {
  Runner* rt;
  std::unique_ptr<Net> net;
  Tensor data, label;
  // the batch being loaded while a step runs (mnvh_net_prefetch_batch): a second pair of
  // tensors, and a marker behind the last step that read them
  Tensor next_data, next_label;
  bool next_ready = false;
  void* spare_last_use = nullptr;
  // a recorded Step: the instantiated graph and every tensor its kernels read or write
  void* graph = nullptr;
  std::vector<Tensor> graph_tensors;
  void ReleaseGraph() {
    if (!graph) return;
    rt->Sync();
    mnv_graph_destroy(graph);
    graph = nullptr;
    graph_tensors.clear();
    net->results.clear();
  }
  ~NetHandle() {
    try {
      ReleaseGraph();
    } catch (...) {
    }
  }
};

template <class F> int Guard(F&& f) {
  try {
    f();
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
  } catch (...) {
    g_error = "unknown exception";
  }
  return -1;
}

Scale ToScale(const mnvh_tensor& t) {
  MNV_CHECK(t.ndims >= 1 && t.ndims <= MNVH_MAX_DIMS) << "bad tensor rank";
  return Scale(std::vector<int>(t.dims, t.dims + t.ndims));
}

int P(const double* p, int n, int i) {
  MNV_CHECK(i < n) << "missing operator parameter " << i;
  return static_cast<int>(p[i]);
}

// One operator by name on device tensors: the NArray call the name stands for.
Tensor RunNamedOp(Runner* rt, const std::string& op, const std::vector<Tensor>& in,
                  const double* params, int n_params) {
  const int n_inputs = static_cast<int>(in.size());
  auto need = [&](int n) { MNV_CHECK_EQ(n_inputs, n) << op << " takes " << n << " inputs"; };
  auto conv_info = [&] {
    return ConvInfo(P(params, n_params, 0), P(params, n_params, 1), P(params, n_params, 2),
                    P(params, n_params, 3));
  };
  auto pool_info = [&] {
    return PoolingInfo(static_cast<PoolingInfo::Algorithm>(P(params, n_params, 0)),
                       P(params, n_params, 1), P(params, n_params, 2), P(params, n_params, 3),
                       P(params, n_params, 4), P(params, n_params, 5), P(params, n_params, 6));
  };
  Tensor r;
  if (op == "arithmetic") {
    need(2);
    r = rt->Arithmetic(in[0], in[1], static_cast<ArithmeticType>(P(params, n_params, 0)));
  } else if (op == "arithmetic_const") {
    need(1);
    MNV_CHECK(n_params >= 3) << "arithmetic_const takes type, val, side";
    r = rt->ArithmeticConst(in[0], static_cast<float>(params[1]),
                            static_cast<ArithmeticType>(P(params, n_params, 0)),
                            P(params, n_params, 2));
  } else if (op == "elewise") {
    need(1);
    r = rt->Elewise(in[0], static_cast<ElewiseType>(P(params, n_params, 0)));
  } else if (op == "norm_arithmetic") {
    need(2);
    r = rt->NormArithmetic(in[0], in[1], static_cast<ArithmeticType>(P(params, n_params, 0)));
  } else if (op == "matmult") {
    need(2);
    r = rt->MatMult(in[0], in[1]);
  } else if (op == "trans") {
    need(1);
    r = rt->Trans(in[0]);
  } else if (op == "reshape") {
    need(1);
    std::vector<int> d;
    for (int i = 0; i < n_params; ++i) d.push_back(static_cast<int>(params[i]));
    r = rt->Reshape(in[0], Scale(d));
  } else if (op == "reduction") {
    need(1);
    r = rt->Reduce(in[0], P(params, n_params, 1),
                   static_cast<ReductionType>(P(params, n_params, 0)));
  } else if (op == "maxindex") {
    need(1);
    r = rt->MaxIndex(in[0], P(params, n_params, 0));
  } else if (op == "sigmoid_forward") {
    need(1);
    r = rt->SigmoidForward(in[0]);
  } else if (op == "relu_forward") {
    need(1);
    r = rt->ReluForward(in[0]);
  } else if (op == "tanh_forward") {
    need(1);
    r = rt->TanhForward(in[0]);
  } else if (op == "sigmoid_backward") {
    need(3);
    r = rt->SigmoidBackward(in[0], in[1], in[2]);
  } else if (op == "relu_backward") {
    need(3);
    r = rt->ReluBackward(in[0], in[1], in[2]);
  } else if (op == "tanh_backward") {
    need(3);
    r = rt->TanhBackward(in[0], in[1], in[2]);
  } else if (op == "activation_forward") {
    need(1);
    r = rt->ActivationForward(in[0], static_cast<ActivationAlgorithm>(P(params, n_params, 0)));
  } else if (op == "activation_backward") {
    need(3);
    r = rt->ActivationBackward(in[0], in[1], in[2],
                               static_cast<ActivationAlgorithm>(P(params, n_params, 0)));
  } else if (op == "softmax_forward") {
    need(1);
    r = rt->SoftmaxForward(in[0], static_cast<SoftmaxAlgorithm>(P(params, n_params, 0)));
  } else if (op == "softmax_backward") {
    need(2);
    r = rt->SoftmaxBackward(in[0], in[1], static_cast<SoftmaxAlgorithm>(P(params, n_params, 0)));
  } else if (op == "conv_forward") {
    need(3);
    r = rt->ConvForward(in[0], in[1], in[2], conv_info());
  } else if (op == "conv_backward_data") {
    need(3);
    r = rt->ConvBackwardData(in[0], in[1], in[2], conv_info());
  } else if (op == "conv_backward_filter") {
    need(3);
    r = rt->ConvBackwardFilter(in[0], in[1], in[2], conv_info());
  } else if (op == "conv_backward_bias") {
    need(1);
    r = rt->ConvBackwardBias(in[0]);
  } else if (op == "pooling_forward") {
    need(1);
    r = rt->PoolingForward(in[0], pool_info());
  } else if (op == "pooling_backward") {
    need(3);
    r = rt->PoolingBackward(in[0], in[1], in[2], pool_info());
  } else if (op == "conv_forward_relu") {
    need(3);
    r = rt->ConvForwardRelu(in[0], in[1], in[2], conv_info());
  } else if (op == "conv_backward_data_relu") {  // inputs: diff, bottom, filter
    need(3);
    r = rt->ConvBackwardDataRelu(in[0], in[1], in[2], conv_info());
  } else if (op == "pooling_backward_relu") {  // params: h, w, sv, sh, ph, pw (max pooling)
    need(3);
    r = rt->PoolingBackwardRelu(in[0], in[1], in[2],
                                PoolingInfo(PoolingInfo::Algorithm::kMax, P(params, n_params, 0),
                                            P(params, n_params, 1), P(params, n_params, 2),
                                            P(params, n_params, 3), P(params, n_params, 4),
                                            P(params, n_params, 5)));
  } else if (op == "matmult_bias") {  // params: relu (0 / 1); inputs: a, b, bias {m,1}
    need(3);
    r = rt->MatMultBias(in[0], in[1], in[2], P(params, n_params, 0) != 0);
  } else if (op == "matmult_relu_backward") {  // inputs: a, b, bottom
    need(3);
    r = rt->MatMultReluBackward(in[0], in[1], in[2]);
  } else if (op == "matmult_trans_a") {  // inputs: at {k,m}, b {k,n} [, bottom {m,n}]
    MNV_CHECK(n_inputs == 2 || n_inputs == 3) << "matmult_trans_a takes 2 or 3 inputs";
    r = n_inputs == 3 ? rt->MatMultTransA(in[0], in[1], in[2]) : rt->MatMultTransA(in[0], in[1]);
  } else if (op == "matmult_trans_b") {  // inputs: a {m,k}, bt {n,k}
    need(2);
    r = rt->MatMultTransB(in[0], in[1]);
  } else if (op == "sgd_update") {  // params: scale; inputs: w, g
    need(2);
    MNV_CHECK(n_params >= 1) << "sgd_update takes the scale";
    r = rt->SgdUpdate(in[0], in[1], static_cast<float>(params[0]));
  } else if (op == "matmult_trans_b_sgd") {  // params: scale; inputs: a {m,k}, bt {n,k}, w {m,n}
    need(3);
    MNV_CHECK(n_params >= 1) << "matmult_trans_b_sgd takes the scale";
    r = rt->MatMultTransBSgd(in[0], in[1], in[2], static_cast<float>(params[0]));
  } else if (op == "conv_backward_filter_sgd") {  // params: conv info, scale; inputs: diff, bottom, filter
    need(3);
    MNV_CHECK(n_params >= 5) << "conv_backward_filter_sgd takes the convolution and the scale";
    r = rt->ConvBackwardFilterSgd(in[0], in[1], in[2], conv_info(),
                                  static_cast<float>(params[4]));
  } else if (op == "threshold_norm") {  // params: threshold
    need(1);
    MNV_CHECK(n_params >= 1) << "threshold_norm takes the threshold";
    r = rt->ThresholdNorm(in[0], static_cast<float>(params[0]));
  } else if (op == "index") {  // params: idx, then the extents of one block
    need(1);
    std::vector<int> d;
    for (int i = 1; i < n_params; ++i) d.push_back(static_cast<int>(params[i]));
    MNV_CHECK(!d.empty()) << "index takes idx, d0, ...";
    r = rt->Index(in[0], P(params, n_params, 0), Scale(d));
  } else if (op == "concat") {  // params: catdim; any number (> 1) of inputs
    r = rt->Concat(in, P(params, n_params, 0));
  } else if (op == "slice") {  // params: slice_dim, st_off, slice_count
    need(1);
    r = rt->Slice(in[0], P(params, n_params, 0), P(params, n_params, 1), P(params, n_params, 2));
  } else if (op == "select") {  // params: the column indices
    need(1);
    std::vector<int> idx;
    for (int i = 0; i < n_params; ++i) idx.push_back(static_cast<int>(params[i]));
    r = rt->Select(in[0], idx);
  } else if (op == "lrn_forward") {  // params: local_size, alpha, beta; inputs: bottom, scale
    need(2);
    MNV_CHECK(n_params >= 3) << "lrn_forward takes local_size, alpha, beta";
    r = rt->LRNForward(in[0], in[1], static_cast<int>(params[0]), static_cast<float>(params[1]),
                       static_cast<float>(params[2]));
  } else if (op == "lrn_backward") {  // inputs: bottom, top, scale, top_diff
    need(4);
    MNV_CHECK(n_params >= 3) << "lrn_backward takes local_size, alpha, beta";
    r = rt->LRNBackward(in[0], in[1], in[2], in[3], static_cast<int>(params[0]),
                        static_cast<float>(params[1]), static_cast<float>(params[2]));
  } else if (op == "randn" || op == "rand_bernoulli") {  // params: mu, var | p ; then d0, d1, ...
    need(0);
    const int lead = op == "randn" ? 2 : 1;
    MNV_CHECK(n_params > lead) << op << " takes its parameters, then the extents";
    std::vector<int> d;
    for (int i = lead; i < n_params; ++i) d.push_back(static_cast<int>(params[i]));
    r = op == "randn" ? rt->Randn(Scale(d), static_cast<float>(params[0]), static_cast<float>(params[1]))
                      : rt->RandBernoulli(Scale(d), static_cast<float>(params[0]));
  } else if (op == "fill") {
    need(0);
    std::vector<int> d;
    for (int i = 1; i < n_params; ++i) d.push_back(static_cast<int>(params[i]));
    MNV_CHECK(n_params >= 2) << "fill takes val, d0, ...";
    r = rt->Constant(Scale(d), static_cast<float>(params[0]));
  } else {
    MNV_FATAL() << "unknown operator '" << op << "'";
  }
  return r;
}

}  // namespace

extern "C" {

const char* mnvh_last_error(void) { return g_error.c_str(); }

int mnvh_runtime_create(int gpu_id, int sync_each_op, void** runtime) {
  return Guard([&] {
    MNV_CHECK(runtime) << "null out pointer";
    MNV_CHECK(sync_each_op >= 0 && sync_each_op <= 2) << "mode must be 0, 1 or 2";
    *runtime = new Runner(gpu_id, sync_each_op == 1, sync_each_op == 2);
  });
}

int mnvh_runtime_create_pool(int gpu_id, int sync_each_op, size_t pool_bytes, void** runtime) {
  return Guard([&] {
    MNV_CHECK(runtime && pool_bytes > 0) << "bad argument";
    MNV_CHECK(sync_each_op >= 0 && sync_each_op <= 2) << "mode must be 0, 1 or 2";
    *runtime = new Runner(gpu_id, sync_each_op == 1, sync_each_op == 2, pool_bytes);
  });
}

int mnvh_runtime_destroy(void* runtime) {
  return Guard([&] { delete static_cast<Runner*>(runtime); });
}

int mnvh_runtime_sync(void* runtime) {
  return Guard([&] { static_cast<Runner*>(runtime)->Sync(); });
}

int mnvh_runtime_ops_issued(void* runtime, unsigned long long* count) {
  return Guard([&] { *count = static_cast<Runner*>(runtime)->ops_issued(); });
}

int mnvh_runtime_pool_stats(void* runtime, size_t* total_bytes, size_t* cached_blocks) {
  return Guard([&] {
    auto& ds = static_cast<Runner*>(runtime)->device().data_store();
    if (total_bytes) *total_bytes = ds.GetTotalBytes();
    if (cached_blocks) *cached_blocks = ds.NumCachedBlocks();
  });
}

int mnvh_runtime_dataflow_stats(void* runtime, unsigned long long* producer_waits,
                                unsigned long long* recycle_waits) {
  return Guard([&] {
    HipDevice& d = static_cast<Runner*>(runtime)->device();
    if (producer_waits) *producer_waits = d.producer_waits();
    if (recycle_waits) *recycle_waits = d.recycle_waits();
  });
}

int mnvh_runtime_set_stream(void* runtime, int stream) {
  return Guard([&] { static_cast<Runner*>(runtime)->SetStream(stream); });
}

int mnvh_runtime_set_dataflow(void* runtime, int enable) {
  return Guard([&] { static_cast<Runner*>(runtime)->SetDataflow(enable != 0); });
}

int mnvh_runtime_profile(void* runtime, int enable) {
  return Guard([&] { static_cast<Runner*>(runtime)->device().set_profile(enable != 0); });
}

int mnvh_runtime_profile_filter(void* runtime, const char* name_part) {
  return Guard([&] {
    static_cast<Runner*>(runtime)->device().set_profile_filter(name_part ? name_part : "");
  });
}

int mnvh_runtime_profile_read(void* runtime, char* text_out, size_t capacity) {
  return Guard([&] {
    auto prof = static_cast<Runner*>(runtime)->device().CollectProfile();
    std::ostringstream ss;
    for (auto& kv : prof) ss << kv.first << "\t" << kv.second.first << "\t" << kv.second.second << "\n";
    std::string s = ss.str();
    MNV_CHECK(text_out && s.size() + 1 <= capacity) << "profile text needs " << s.size() + 1 << " bytes";
    std::memcpy(text_out, s.c_str(), s.size() + 1);
  });
}

int mnvh_op(void* runtime, const char* op_name, const mnvh_tensor* inputs, int n_inputs,
            const double* params, int n_params, float* out, size_t out_capacity,
            int* out_ndims, int* out_dims) {
  return Guard([&] {
    Runner* rt = static_cast<Runner*>(runtime);
    MNV_CHECK(rt && op_name && out) << "null argument";
    std::vector<Tensor> in;
    for (int i = 0; i < n_inputs; ++i) {
      MNV_CHECK(inputs[i].data) << "null input data";
      in.push_back(rt->MakeNArray(ToScale(inputs[i]), inputs[i].data));
    }
    Tensor r = RunNamedOp(rt, op_name, in, params, n_params);
    size_t n = r->size.Prod();
    MNV_CHECK(n <= out_capacity) << "output needs " << n << " floats, capacity " << out_capacity;
    rt->Read(r, out);
    if (out_ndims) *out_ndims = static_cast<int>(r->size.NumDims());
    if (out_dims)
      for (size_t i = 0; i < r->size.NumDims(); ++i) out_dims[i] = r->size[i];
  });
}

// ---- device-resident tensors: graphs of operators without a round trip to the host

int mnvh_tensor_create(void* runtime, const mnvh_tensor* host, void** tensor) {
  return Guard([&] {
    Runner* rt = static_cast<Runner*>(runtime);
    MNV_CHECK(rt && host && host->data && tensor) << "null argument";
    *tensor = new Tensor(rt->MakeNArray(ToScale(*host), host->data));
  });
}

int mnvh_tensor_op(void* runtime, const char* op_name, void* const* inputs, int n_inputs,
                   const double* params, int n_params, void** out) {
  return Guard([&] {
    Runner* rt = static_cast<Runner*>(runtime);
    MNV_CHECK(rt && op_name && out) << "null argument";
    std::vector<Tensor> in;
    for (int i = 0; i < n_inputs; ++i) {
      MNV_CHECK(inputs && inputs[i]) << "null input tensor";
      in.push_back(*static_cast<Tensor*>(inputs[i]));
    }
    *out = new Tensor(RunNamedOp(rt, op_name, in, params, n_params));
  });
}

int mnvh_tensor_info(void* tensor, int* ndims, int* dims, int* stream) {
  return Guard([&] {
    MNV_CHECK(tensor) << "null tensor";
    const Tensor& t = *static_cast<Tensor*>(tensor);
    if (ndims) *ndims = static_cast<int>(t->size.NumDims());
    if (dims)
      for (size_t i = 0; i < t->size.NumDims(); ++i) dims[i] = t->size[i];
    if (stream) *stream = t->stream;
  });
}

int mnvh_tensor_read(void* runtime, void* tensor, float* out, size_t out_capacity) {
  return Guard([&] {
    MNV_CHECK(runtime && tensor && out) << "null argument";
    const Tensor& t = *static_cast<Tensor*>(tensor);
    size_t n = t->size.Prod();
    MNV_CHECK(n <= out_capacity) << "tensor has " << n << " floats, capacity " << out_capacity;
    static_cast<Runner*>(runtime)->Read(t, out);
  });
}

int mnvh_tensor_free(void* tensor) {
  return Guard([&] { delete static_cast<Tensor*>(tensor); });
}

int mnvh_set_random_seed(unsigned long long seed) {
  minerva::hip::SetRandomSeed(seed);
  return 0;
}

int mnvh_concurrent_adds(void* runtime, const float* a, const float* b, size_t n, int count,
                         float* out) {
  return Guard([&] {
    Runner* rt = static_cast<Runner*>(runtime);
    HipDevice& dev = rt->device();
    Scale size{static_cast<int>(n)};
    Tensor ta = rt->MakeNArray(size, a), tb = rt->MakeNArray(size, b);
    // tasks and their output ids live until every worker is done
    std::vector<Task> tasks(count);
    const uint64_t base_id = (1ull << 40);
    for (int i = 0; i < count; ++i) {
      auto op = std::make_shared<ArithmeticOp>();
      op->closure.type = ArithmeticType::kAdd;
      Task& t = tasks[i];
      t.inputs.emplace_back(PhysicalData(size, dev.device_id(), ta->id), ta->id);
      t.inputs.emplace_back(PhysicalData(size, dev.device_id(), tb->id), tb->id);
      t.outputs.emplace_back(PhysicalData(size, dev.device_id(), base_id + i), base_id + i);
      t.op.compute_fn = op;
      t.id = i;
      t.light = false;
    }
    for (int i = 0; i < count; ++i) dev.PushTask(&tasks[i]);
    dev.WaitForAllFinished();
    // the host threads are done; in dataflow mode their kernels may still be in flight on
    // the four streams, and the copies below run on stream 0
    dev.Barrier(0);
    std::string err = dev.TakeAsyncError();
    for (int i = 0; i < count; ++i) {
      if (err.empty()) dev.CopyToHost(out + (size_t)i * n, base_id + i, n);
      dev.FreeDataIfExist(base_id + i);
    }
    MNV_CHECK(err.empty()) << err;
  });
}

int mnvh_net_create(void* runtime, const char* kind, int batch, int variant, void** net) {
  return Guard([&] {
    Runner* rt = static_cast<Runner*>(runtime);
    MNV_CHECK(rt && kind && net && batch > 0) << "bad argument";
    std::unique_ptr<NetHandle> h(new NetHandle);
    h->rt = rt;
    std::string k(kind);
    if (k == "mlp") h->net.reset(new MlpNet(rt, batch));
    else if (k == "cnn") h->net.reset(variant == 1 ? new CnnNet(rt, batch, 2, 3) : new CnnNet(rt, batch));
    else if (k == "alexnet") h->net.reset(new AlexNet(rt, batch, 1000, variant == 1 ? 0.5f : 0.f));
    else MNV_FATAL() << "unknown net '" << k << "'";
    *net = h.release();
  });
}

int mnvh_net_destroy(void* net) {
  return Guard([&] { delete static_cast<NetHandle*>(net); });
}

int mnvh_net_num_params(void* net, int* count) {
  return Guard([&] { *count = static_cast<int>(static_cast<NetHandle*>(net)->net->param_names.size()); });
}

int mnvh_net_param_info(void* net, int index, char* name_out, size_t* floats) {
  return Guard([&] {
    Net& n = *static_cast<NetHandle*>(net)->net;
    MNV_CHECK(index >= 0 && index < static_cast<int>(n.param_names.size())) << "bad index";
    const std::string& name = n.param_names[index];
    if (name_out) {
      std::strncpy(name_out, name.c_str(), 15);
      name_out[15] = 0;
    }
    if (floats) *floats = n.params[name]->size.Prod();
  });
}

int mnvh_net_set_param(void* net, const char* name, const float* host, size_t floats) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    auto it = h->net->params.find(name);
    MNV_CHECK(it != h->net->params.end()) << "no parameter '" << name << "'";
    Scale size = it->second->size;
    MNV_CHECK_EQ(static_cast<size_t>(size.Prod()), floats) << "size of '" << name << "'";
    if (h->graph) h->rt->Upload(it->second, host);  // the recording reads this address
    else it->second = h->rt->MakeNArray(size, host);
  });
}

int mnvh_net_read(void* net, const char* name, float* host_out, size_t floats) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    Tensor t;
    auto it = h->net->params.find(name);
    if (it != h->net->params.end()) t = it->second;
    else {
      auto jt = h->net->results.find(name);
      MNV_CHECK(jt != h->net->results.end()) << "no tensor '" << name << "'";
      t = jt->second;
    }
    MNV_CHECK_EQ(static_cast<size_t>(t->size.Prod()), floats) << "size of '" << name << "'";
    h->rt->Read(t, host_out);
  });
}

int mnvh_net_set_fused(void* net, int on) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    MNV_CHECK(!h->graph) << "release the recorded step before switching operator sets";
    h->net->fused = on != 0;
    h->net->fuse_update = on == 2;
  });
}

int mnvh_net_keep_activations(void* net, int on) {
  return Guard([&] { static_cast<NetHandle*>(net)->net->keep_activations = on != 0; });
}

int mnvh_net_load_batch(void* net, const float* data, size_t data_floats, const float* label,
                        size_t label_floats) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    Scale ds = h->net->DataSize(), ls = h->net->LabelSize();
    MNV_CHECK_EQ(static_cast<size_t>(ds.Prod()), data_floats) << "data size";
    MNV_CHECK_EQ(static_cast<size_t>(ls.Prod()), label_floats) << "label size";
    if (h->graph) {  // the recording reads these addresses
      h->rt->Upload(h->data, data);
      h->rt->Upload(h->label, label);
    } else {
      h->data = h->rt->MakeNArray(ds, data);
      h->label = h->rt->MakeNArray(ls, label);
    }
  });
}

int mnvh_net_prefetch_batch(void* net, const float* data, size_t data_floats, const float* label,
                            size_t label_floats) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    Scale ds = h->net->DataSize(), ls = h->net->LabelSize();
    MNV_CHECK_EQ(static_cast<size_t>(ds.Prod()), data_floats) << "data size";
    MNV_CHECK_EQ(static_cast<size_t>(ls.Prod()), label_floats) << "label size";
    MNV_CHECK(!h->graph) << "a recorded step reads one pair of tensors: use mnvh_net_load_batch";
    MNV_CHECK(!h->rt->device().dataflow()) << "in dataflow mode mnvh_net_load_batch is placed on a "
                                           << "stream of its own already";
    HipDevice& dev = h->rt->device();
    if (!h->next_data) {  // first use: the second pair, created in stream order
      h->next_data = h->rt->Constant(ds, 0.f);
      h->next_label = h->rt->Constant(ls, 0.f);
      h->spare_last_use = dev.StreamMarker(0);
    }
    // the step that last read the spare pair must have left the GPU
    dev.WaitMarker(h->spare_last_use);
    h->spare_last_use = nullptr;
    // worker stream 1 carries the copy; stream 0 keeps computing the step in flight
    h->rt->UploadOn(1, h->next_data, data);
    h->rt->UploadOn(1, h->next_label, label);
    h->next_ready = true;
  });
}

int mnvh_net_step(void* net, float lr) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    MNV_CHECK(!h->graph) << "the step is recorded: replay it or release the recording first";
    if (h->next_ready) {  // the prefetched batch becomes the current one
      std::swap(h->data, h->next_data);
      std::swap(h->label, h->next_label);
      h->next_ready = false;
      // the pair that just became spare was read by the previous step, which may still run
      if (h->next_data) h->spare_last_use = h->rt->device().StreamMarker(0);
    }
    MNV_CHECK(h->data && h->label) << "load a batch first";
    h->net->Step(h->data, h->label, lr);
  });
}

int mnvh_net_capture_step(void* net, float lr, size_t* num_nodes) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    MNV_CHECK(h->data && h->label) << "load a batch first";
    MNV_CHECK(!h->graph) << "the step is already recorded";
    MNV_CHECK(!h->rt->device().dataflow()) << "recording needs the one-stream order, not dataflow mode";
    MNV_CHECK(h->net->Capturable()) << "this network draws random seeds on the host in every "
                                    << "step; a recording would repeat them";
    Runner* rt = h->rt;
    Net& n = *h->net;
    const std::map<std::string, Tensor> saved = n.params;
    auto pass = [&](bool record) {
      rt->BeginRetain();
      try {
        if (record) rt->device().BeginCapture();
        n.Step(h->data, h->label, lr);
        // The step leaves the new parameters in new tensors; a replay must find them
        // where it reads them, so they are copied back over the old ones.
        if (record)
          for (auto& name : n.param_names) rt->CopyInto(saved.at(name), n.params[name]);
        n.params = saved;
        if (record) {
          h->graph = rt->device().EndCapture(num_nodes);
          h->graph_tensors = rt->EndRetain();
        } else {
          rt->Sync();
          n.results.clear();
          rt->EndRetain();  // every block of the step goes back to the pool's free lists
        }
      } catch (...) {
        rt->device().AbortCapture();
        n.params = saved;
        n.results.clear();
        rt->EndRetain();
        throw;
      }
    };
    // First an eager pass that changes nothing (the new parameters are dropped): it runs
    // the kernels' one-time set-up and leaves one cached block per tensor of the step, so
    // that the recording pass allocates nothing.
    pass(false);
    pass(true);
  });
}

int mnvh_net_replay(void* net, int steps, int sync_each_step) {
  return Guard([&] {
    NetHandle* h = static_cast<NetHandle*>(net);
    MNV_CHECK(h->graph) << "record a step first";
    for (int i = 0; i < steps; ++i) {
      h->rt->device().LaunchGraph(h->graph);
      if (sync_each_step) h->rt->Sync();
    }
    h->rt->Sync();
  });
}

int mnvh_net_release_graph(void* net) {
  return Guard([&] { static_cast<NetHandle*>(net)->ReleaseGraph(); });
}

}  // extern "C"
