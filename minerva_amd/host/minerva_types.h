// Operator-interface types of the host layer.  Names, fields and meaning follow the
// reference so that operator code written against Minerva compiles against these:
//   Scale                      minerva/common/scale.h:14-128 (column-major, dim 0 fastest)
//   DataShard / DataList       minerva/op/data_shard.h:7-14
//   ImplType / Context         minerva/op/context.h:11-37 (kHip added; the three CUDA
//                              handles become one stream plus a scratch arena)
//   closures and enums         minerva/op/closure.h:8-176, minerva/narray/convolution_info.h:5-57
// Errors: the reference aborts through CHECK / LOG(FATAL) (which dmlc-core raises as an
// exception); here every failed check throws minerva::Error.
#pragma once
#include <cstddef>
#include <cstdint>
#include <initializer_list>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace minerva {

class Error : public std::runtime_error {
 public:
  explicit Error(const std::string& what) : std::runtime_error(what) {}
};

namespace detail {
struct Thrower {
  std::ostringstream os;
  Thrower(const char* file, int line, const char* cond) {
    os << file << ":" << line << ": check failed: " << cond << " ";
  }
  [[noreturn]] ~Thrower() noexcept(false) { throw Error(os.str()); }
};
}  // namespace detail

#define MNV_CHECK(cond) \
  if (cond) {           \
  } else                \
    ::minerva::detail::Thrower(__FILE__, __LINE__, #cond).os
#define MNV_CHECK_EQ(a, b) MNV_CHECK((a) == (b)) << "(" << (a) << " vs " << (b) << ") "
#define MNV_CHECK_GT(a, b) MNV_CHECK((a) > (b)) << "(" << (a) << " vs " << (b) << ") "
#define MNV_CHECK_LT(a, b) MNV_CHECK((a) < (b)) << "(" << (a) << " vs " << (b) << ") "
#define MNV_CHECK_LE(a, b) MNV_CHECK((a) <= (b)) << "(" << (a) << " vs " << (b) << ") "
#define MNV_FATAL() ::minerva::detail::Thrower(__FILE__, __LINE__, "fatal").os

// ---- Scale: an N-d extent or index; dimension 0 is the fastest in memory.
class Scale {
 public:
  Scale() = default;
  Scale(std::initializer_list<int> l) : vec_(l) {}
  explicit Scale(std::vector<int> v) : vec_(std::move(v)) {}
  static Scale Origin(size_t nd) { return Scale(std::vector<int>(nd, 0)); }
  static Scale Constant(size_t nd, int v) { return Scale(std::vector<int>(nd, v)); }
  int operator[](size_t i) const { return vec_[i]; }
  int& operator[](size_t i) { return vec_[i]; }
  bool operator==(const Scale& o) const { return vec_ == o.vec_; }
  bool operator!=(const Scale& o) const { return vec_ != o.vec_; }
  size_t NumDims() const { return vec_.size(); }
  // The reference returns int (scale.h:105-111); the wider type only matters past 2^31.
  int Prod() const {
    long long p = vec_.empty() ? 0 : 1;
    for (int d : vec_) p *= d;
    MNV_CHECK(p <= 0x7fffffffLL) << "tensor larger than 2^31-1 elements";
    return static_cast<int>(p);
  }
  bool Contains(int v) const {
    for (int d : vec_)
      if (d == v) return true;
    return false;
  }
  Scale Concat(int v) const {
    Scale r(*this);
    r.vec_.push_back(v);
    return r;
  }
  std::vector<int>::const_iterator begin() const { return vec_.begin(); }
  std::vector<int>::const_iterator end() const { return vec_.end(); }
  const std::vector<int>& ToVector() const { return vec_; }
  std::string ToString() const {
    std::ostringstream ss;
    ss << "[ ";
    for (int d : vec_) ss << d << " ";
    ss << "]";
    return ss.str();
  }

 private:
  std::vector<int> vec_;
};

inline std::ostream& operator<<(std::ostream& os, const Scale& s) { return os << s.ToString(); }

// ---- one tensor handed to an operator: raw device pointer + extent (not owned)
struct DataShard {
  DataShard(float* data, Scale const& size) : data_(data), size_(size) {}
  float* const data_;
  Scale const& size_;
};
using DataList = std::vector<DataShard>;

enum class ImplType { kNA = 0, kBasic, kMkl, kCuda, kHip };

inline std::ostream& operator<<(std::ostream& os, ImplType t) {
  switch (t) {
    case ImplType::kNA: return os << "N/A";
    case ImplType::kBasic: return os << "Basic";
    case ImplType::kMkl: return os << "Mkl";
    case ImplType::kCuda: return os << "Cuda";
    case ImplType::kHip: return os << "Hip";
  }
  return os << "Unknown impl type";
}

// What a device hands to an operator.  `stream` is a hipStream_t; `workspace` is the
// per-stream scratch arena the device owns (operators never allocate).
struct Context {
  ImplType impl_type = ImplType::kNA;
  void* stream = nullptr;
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  // pinned host memory of the stream, for staging copies from pageable host buffers
  void* staging = nullptr;
  size_t staging_bytes = 0;
  virtual ~Context() {}
};

// ---- enums and closures (one per operator; the op's only parameters)
enum class ArithmeticType { kAdd = 0, kSub, kMult, kDiv };
enum class ElewiseType { kExp = 0, kLn, kNegative };
enum class ReductionType { kSum = 0, kMax };
enum class SoftmaxAlgorithm { kInstance, kChannel };
enum class ActivationAlgorithm { kSigmoid, kRelu, kTanh };

struct ConvInfo {
  ConvInfo(int ph = 0, int pw = 0, int sv = 1, int sh = 1)
      : pad_height(ph), pad_width(pw), stride_vertical(sv), stride_horizontal(sh) {}
  int pad_height, pad_width, stride_vertical, stride_horizontal;
};

struct PoolingInfo {
  enum class Algorithm { kMax, kAverage };
  PoolingInfo(Algorithm alg = Algorithm::kMax, int h = 0, int w = 0, int sv = 1, int sh = 1,
              int ph = 0, int pw = 0)
      : algorithm(alg), height(h), width(w), stride_vertical(sv), stride_horizontal(sh),
        pad_height(ph), pad_width(pw) {}
  Algorithm algorithm;
  int height, width, stride_vertical, stride_horizontal, pad_height, pad_width;
};

struct ArrayLoaderClosure { std::shared_ptr<float> data; };
struct FillClosure { float val; };
// reference minerva/op/closure.h:30-36; `var` is handed to the generator as the standard
// deviation, as the reference does (cuda_perform.cu:621, basic.cpp:275)
struct RandnClosure { float mu, var; };
struct RandBernoulliClosure { float p; };
struct MatMultClosure {};
struct TransposeClosure {};
struct ReshapeClosure {};
struct ReductionClosure { ReductionType type; Scale dims_to_reduce; };
struct MaxIndexClosure { int dim; };
struct ElewiseClosure { ElewiseType type; };
struct SigmoidForwardClosure {};
struct SigmoidBackwardClosure {};
struct ReluForwardClosure {};
struct ReluBackwardClosure {};
struct TanhForwardClosure {};
struct TanhBackwardClosure {};
struct ArithmeticClosure { ArithmeticType type; };
struct ArithmeticConstClosure {
  ArithmeticType type;
  float val;
  int side;  // 0: the constant is the left operand, 1: the right operand
};
struct NormArithmeticClosure { ArithmeticType type; Scale dims_to_replicate; };

template <int i> struct ConvClosure {
  int pad_height, pad_width, stride_vertical, stride_horizontal;
};
typedef ConvClosure<0> ConvForwardClosure;
typedef ConvClosure<1> ConvBackwardDataClosure;
typedef ConvClosure<2> ConvBackwardFilterClosure;
struct ConvBackwardBiasClosure {};

template <int i> struct SoftmaxClosure { SoftmaxAlgorithm algorithm; };
typedef SoftmaxClosure<0> SoftmaxForwardClosure;
typedef SoftmaxClosure<1> SoftmaxBackwardClosure;

template <int i> struct ActivationClosure { ActivationAlgorithm algorithm; };
typedef ActivationClosure<0> ActivationForwardClosure;
typedef ActivationClosure<1> ActivationBackwardClosure;

template <int i> struct PoolingClosure {
  PoolingInfo::Algorithm algorithm;
  int height, width, stride_vertical, stride_horizontal, pad_height, pad_width;
};
typedef PoolingClosure<0> PoolingForwardClosure;
typedef PoolingClosure<1> PoolingBackwardClosure;

// reference minerva/op/closure.h:151-158
template <int i> struct LRNClosure {
  int local_size;
  float alpha, beta;
  Scale data_shape;
};
typedef LRNClosure<0> LRNForwardClosure;
typedef LRNClosure<1> LRNBackwardClosure;

// reference minerva/op/closure.h:74-76, 160-176
struct ThresholdNormClosure { float threshold; };
struct IndexClosure { int idx; };
struct ConcatClosure { int catdim; };
struct SliceClosure { int slice_dim, st_off, slice_count; };
struct SelectClosure { std::vector<int> indices; };

}  // namespace minerva
