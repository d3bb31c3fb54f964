// SGEMM C{m,n} = A{m,k} * B{k,n}, column-major, no transposes, alpha 1 / beta 0:
// the product Minerva's MatMult asks for (reference minerva/op/impl/basic.cpp:150-173;
// cublasSgemm call at minerva/op/impl/cuda/cuda_perform.cu:66-70).
// Built on the fp32 MFMA core in gemm_core.h; A is fetched x-fast (m contiguous),
// B k-fast (k contiguous).  Products with too few output tiles to fill 256 CUs split
// the k range over blockIdx.z when the caller lends a workspace.
#include <mutex>

#include "gemm_core.h"

// Split-k partial sums of mnv_sgemm_nn_static: one array per GPU the library is loaded on,
// held until the process ends.  In host code the name `scratch` is only a handle for
// hipGetSymbolAddress; kernels and every other use take the address it returns.
#define MNV_SGEMM_STATIC_SCRATCH_FLOATS ((size_t)MNV_SGEMM_STATIC_SCRATCH_BYTES / sizeof(float))
static __device__ __align__(256) float scratch[MNV_SGEMM_STATIC_SCRATCH_FLOATS];

namespace {

// Period 0 holds every full 16-deep slab: the per-thread byte offsets are fixed and only
// the uniform slab offset moves.  A k extent that is not a multiple of 16 leaves one
// partial slab, which is period 1 and gets its own masked offsets.
// TA / TB: the operand is given transposed -- A as {k,m} (element (m,k) at k + m*lda), B as
// {n,k} (element (k,n) at n + k*ldb) -- which only swaps its fetch direction: a transposed A
// is k-fast, a transposed B x-fast.  The values multiplied and the order they are added in
// are those of the product of the explicitly transposed matrices.
template <bool VEC, bool TA = false, bool TB = false>
struct SgemmNN {
  static constexpr bool A_KFAST = TA, B_KFAST = !TB;
  static constexpr int A_NOFF = VEC ? 1 : 4, B_NOFF = VEC ? 1 : 4;
  const float* __restrict__ A;
  const float* __restrict__ B;
  float* __restrict__ C;
  int M, N, K, total_slabs, spp, bk;
  // Leading dimensions (floats between consecutive columns as stored): m, k, m for whole
  // untransposed matrices (k for a transposed A, n for a transposed B); larger when the
  // operands are panels of matrices too large for 32-bit byte offsets.
  // accumulate: C += A*B (the k panels after the first).
  int lda, ldb, ldc, accumulate;
  // Fused epilogues (all off for the plain product), applied in this order to the value
  // stored, each the single operation the separate operator performs:
  //   bias: + bias[m] (the broadcast add of an {m,1} vector); relu: max(., 0);
  //   gate: gate[m,n] > 0 ? . : 0 (the ReLU gradient's selection)
  //   sgd_w (B transposed only, the weight gradient of an inner product): the value stored
  //   is sgd_w[m,n] - sgd_scale * ., the parameter update; C may be sgd_w itself
  const float* __restrict__ bias;
  const float* __restrict__ gate;
  int relu;
  const float* sgd_w;
  float sgd_scale;
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {};
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(A, TA ? ((unsigned)(M - 1) * (unsigned)lda + (unsigned)K) * 4u
                              : ((unsigned)(K - 1) * (unsigned)lda + (unsigned)M) * 4u);
    r.b = mnv_make_rsrc(B, TB ? ((unsigned)(K - 1) * (unsigned)ldb + (unsigned)N) * 4u
                              : ((unsigned)(N - 1) * (unsigned)ldb + (unsigned)K) * 4u);
  }
  __device__ void a_init(const Res&, AState&, int) const {}
  __device__ void b_init(const Res&, BState&, int) const {}
  // A[m..m+3, k] (x-fast) or, transposed, A[m, k..k+3] (k-fast)
  __device__ void a_period(const AState&, unsigned (&off)[A_NOFF], int m, int kl, int period) const {
    const int k = period * spp * bk + kl;
    if (TA) {
      const unsigned base = ((unsigned)m * (unsigned)lda + (unsigned)k) * 4u;
#pragma unroll
      for (int q = 0; q < A_NOFF; ++q) off[q] = ((m < M) & (k + q < K)) ? base + 4u * q : MNV_OOB;
    } else {
      const unsigned base = ((unsigned)k * (unsigned)lda + (unsigned)m) * 4u;
#pragma unroll
      for (int q = 0; q < A_NOFF; ++q) off[q] = ((m + q < M) & (k < K)) ? base + 4u * q : MNV_OOB;
    }
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[A_NOFF], int, int s,
                         int, float (&v)[4]) const {
    mnv_fetch_vec<A_NOFF>(r.a, off, (unsigned)s * (unsigned)bk * (TA ? 1u : (unsigned)lda) * 4u, v);
  }
  // B[k..k+3, n] (k-fast) or, transposed, B[k, n..n+3] (x-fast)
  __device__ void b_period(const BState&, unsigned (&off)[B_NOFF], int n, int kl, int period) const {
    const int k = period * spp * bk + kl;
    if (TB) {
      const unsigned base = ((unsigned)k * (unsigned)ldb + (unsigned)n) * 4u;
#pragma unroll
      for (int q = 0; q < B_NOFF; ++q) off[q] = ((n + q < N) & (k < K)) ? base + 4u * q : MNV_OOB;
    } else {
      const unsigned base = ((unsigned)n * (unsigned)ldb + (unsigned)k) * 4u;
#pragma unroll
      for (int q = 0; q < B_NOFF; ++q) off[q] = ((n < N) & (k + q < K)) ? base + 4u * q : MNV_OOB;
    }
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[B_NOFF], int, int s,
                         int, float (&v)[4]) const {
    mnv_fetch_vec<B_NOFF>(r.b, off, (unsigned)s * (unsigned)bk * (TB ? (unsigned)ldb : 1u) * 4u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  void set_bk(int b) {
    bk = b;
    spp = K >= b ? K / b : 1;
    total_slabs = (K + b - 1) / b;
  }
  __device__ void block_init(Res&, float*, int, int) const {}
  __device__ void c_store(int m, int n, float x) const {
    const size_t at = (size_t)n * ldc + m;
    if (accumulate) x = C[at] + x;
    if (bias) x = x + bias[m];
    if (relu) x = x > 0.f ? x : 0.f;
    if (gate) x = gate[at] > 0.f ? x : 0.f;
    if (TB) {
      if (sgd_w) x = sgd_w[at] - sgd_scale * x;
    }
    C[at] = x;
  }
  // four consecutive rows of one column: one 16-byte store for the plain product, element by
  // element when an epilogue is on
  static constexpr bool C_STORE4 = true;
  __device__ void c_store4(int m, int n, const float (&x)[4]) const {
    if (m + 3 < M && !accumulate && !bias && !relu && !gate && !sgd_w) {
      const mnv_f4u v = {x[0], x[1], x[2], x[3]};
      *reinterpret_cast<mnv_f4u*>(C + (size_t)n * ldc + m) = v;
    } else {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        if (m + q < M) c_store(m + q, n, x[q]);
    }
  }
  // the update read ahead of the block's stores (only bias / relu / gate / accumulate off)
  static constexpr bool C_PRELOAD = TB;
  __device__ bool c_preload_on() const { return sgd_w != nullptr; }
  __device__ float c_preload(int m, int n) const { return sgd_w[(size_t)n * ldc + m]; }
  __device__ void c_store_with(int m, int n, float x, float w) const {
    C[(size_t)n * ldc + m] = w - sgd_scale * x;
  }
};

struct SgemmEpilogue {
  const float* bias;
  const float* gate;
  int relu;
  int lda = 0, ldb = 0, ldc = 0, accumulate = 0;  // 0: the matrices' own m, k, m
  const float* sgd_w = nullptr;
  float sgd_scale = 0.f;
};

template <bool VEC, bool TA = false, bool TB = false>
SgemmNN<VEC, TA, TB> make_sgemm(const float* a, const float* b, float* c, int m, int n, int k,
                                const SgemmEpilogue& e) {
  SgemmNN<VEC, TA, TB> p;
  p.A = a; p.B = b; p.C = c; p.M = m; p.N = n; p.K = k;
  p.bias = e.bias; p.gate = e.gate; p.relu = e.relu;
  p.lda = e.lda ? e.lda : (TA ? k : m); p.ldb = e.ldb ? e.ldb : (TB ? n : k); p.ldc = e.ldc ? e.ldc : m;
  p.accumulate = e.accumulate;
  p.sgd_w = e.sgd_w; p.sgd_scale = e.sgd_scale;
  p.set_bk(16);
  return p;
}

typedef MnvGemmTile<128, 128, 16, 2, 2> TileBig;
typedef MnvGemmTile<64, 64, 16, 2, 2> TileSmall;
// Eight wavefronts of 64 x 64 (512 threads, two workgroups per CU): a quarter fewer bytes
// fetched and staged per multiply than TileBig, the same reads from LDS.
typedef MnvGemmTile<256, 128, 16, 4, 2> TileTall;
#define MNV_SGEMM_MAX_SPLITS 16

// Tile shape and number of k ranges for an (m,n,k) product given `ws_floats` floats of
// scratch.  Both shapes are priced with the occupancy model of mnv_pick_splits, in units of
// one 128x128x16 slab: a 64x64 slab is a quarter of the arithmetic at about 80% of the
// efficiency, and every extra k range writes and re-reads m*n floats (about 1.2 us per
// slab unit, 6 TB/s for the partial sums).
struct SgemmPlan {
  bool small;
  int splits;
  int groups = 1;  // 4: workgroups of four wavefront groups that share a tile's k range
  bool tall = false;  // 256 x 128 tiles (no k ranges, one wavefront group)
};

SgemmPlan plan_sgemm(int m, int n, int k, size_t ws_floats) {
  const int slabs = (k + 15) / 16;
  const size_t mn = (size_t)m * n;
  const double per_split = 8.0 * (double)mn / 6e6 / 1.2;
  SgemmPlan best{false, 1};
  double best_cost = 0;
  for (int small = 0; small < 2; ++small) {
    const int bm = small ? 64 : 128;
    const long long tiles = (long long)((m + bm - 1) / bm) * ((n + bm - 1) / bm);
    int max_splits = MNV_SGEMM_MAX_SPLITS;
    if (max_splits > slabs / 4) max_splits = slabs / 4;
    const size_t fit = mn ? ws_floats / mn : 0;
    if ((size_t)max_splits > fit) max_splits = (int)fit;
    if (tiles >= 4LL * mnv_cu_count() || slabs < 8) max_splits = 1;  // one per resident workgroup
    const double unit = small ? 0.31 : 1.0;
    double cost;
    const int splits = mnv_pick_splits(tiles, slabs, max_splits, per_split / unit, &cost);
    cost *= unit;
    const bool forced = small ? (m <= 64 || n <= 64) : false;
    if (small == 0 || forced || cost < best_cost) {
      best = SgemmPlan{small != 0, splits};
      best_cost = cost;
    }
  }
  // Workgroups of four wavefront groups (one per CU for the large tile, two for the small
  // one): a step multiplies four slabs, one per group, and ends in about five slab times
  // for the prologue and the addition through LDS.  Measured on the inner products of the
  // AlexNet shape, back to back at sustained clocks: 4096x256x9216 0.190 -> 0.180 ms,
  // 4096x256x4096 0.100 -> 0.092 ms (64x64 tiles, no k ranges in memory at all),
  // 1000x256x4096 0.0304 -> 0.0278 ms, 4096x256x1000 0.031 -> 0.025 ms; 9216x256x4096, whose
  // 144 large tiles do not divide the 256 CUs, stays with single groups.
  // The launch of the reduction kernel itself (about six slab times) only matters in this
  // comparison, where a plan without k ranges in memory competes.
  const double reduce_launch = 6.0;
  if (best.splits > 1) best_cost += reduce_launch;
  for (int small = 0; small < 2; ++small) {
    if (!small && (m <= 64 || n <= 64)) continue;
    const int bm = small ? 64 : 128;
    const long long tiles = (long long)((m + bm - 1) / bm) * ((n + bm - 1) / bm);
    const double unit = small ? 0.27 : 1.0, overhead = small ? 4.0 : 5.0;
    const size_t fit = mn ? ws_floats / mn : 0;
    for (int z = 1; z <= MNV_SGEMM_MAX_SPLITS; ++z) {
      if (z > 1 && (size_t)z > fit) break;
      const int len4 = ((slabs + z - 1) / z + 3) / 4;
      if (len4 < 8) break;  // shorter loops do not repay the prologue and the addition
      // The sixteen wavefronts of such a workgroup share every barrier, so each step waits
      // out a trip to memory that separate workgroups would overlap: worth it only when the
      // workgroups cover most of the chip (MLP 784-256-10 at batch 256, 16 tiles: 0.111 ms
      // per step with single groups, 0.158 ms with grouped ones).
      if (tiles * z < 192) continue;
      const long long per_cu = (tiles * z + 255) / 256;
      const double cost = (double)per_cu * (4.0 * len4 * unit + overhead) +
                          (z > 1 ? per_split * z + reduce_launch : 0.0);
      if (cost < best_cost * 0.95) {
        best = SgemmPlan{small != 0, z, 4};
        best_cost = cost;
      }
    }
  }
  // Large products whose 256 x 128 tiles fill the chip's two-per-CU slots in whole rounds
  // (at least 95% of the multiplies of all rounds are the product's own): measured back to
  // back, 4096^3 0.956 -> 0.940 ms, 8192 x 4096 x 8192 3.85 -> 3.74 ms.  Every element is summed
  // over k in the same order as on the 128 x 128 tile: the same bits.
  if (!best.small && best.splits == 1 && best.groups == 1 && m >= 256 && slabs >= 32) {
    const long long tiles = (long long)((m + 255) / 256) * ((n + 127) / 128);
    const long long slots = 2LL * mnv_cu_count(), rounds = (tiles + slots - 1) / slots;
    if ((double)m * n >= 0.95 * (double)(rounds * slots) * 256.0 * 128.0) best.tall = true;
  }
  return best;
}

// A launch without k ranges may use the workspace for the partial tiles of a cut tail.
template <class P>
int launch_plan(const SgemmPlan& plan, const P& p, void* workspace, size_t workspace_bytes,
                hipStream_t s) {
  if (plan.tall) return mnv_gemm_launch<TileTall>(p, 1, workspace, s);
  if (plan.groups == 4)
    return plan.small ? mnv_gemm_launch<TileSmall, 4>(p, plan.splits, workspace, s)
                      : mnv_gemm_launch<TileBig, 4>(p, plan.splits, workspace, s);
  const size_t tail_bytes = plan.splits == 1 && workspace ? workspace_bytes : 0;
  return plan.small ? mnv_gemm_launch<TileSmall>(p, plan.splits, workspace, s, tail_bytes)
                    : mnv_gemm_launch<TileBig>(p, plan.splits, workspace, s, tail_bytes);
}

// Bytes a product without k ranges wants for the partial tiles of its cut tail.
size_t sgemm_tail_bytes(const SgemmPlan& plan, int m, int n, int k) {
  if (plan.splits != 1 || plan.groups != 1 || plan.tall) return 0;
  const int bm = plan.small ? 64 : 128;
  const long long tiles = (long long)((m + bm - 1) / bm) * ((n + bm - 1) / bm);
  const MnvTailPlan t = mnv_tail_plan(tiles, (k + 15) / 16, (size_t)bm * bm, (size_t)-1 / sizeof(float));
  return t.z > 1 ? (size_t)(tiles - t.begin) * t.z * bm * bm * sizeof(float) : 0;
}

#define MNV_MAX_DEVICES 64
std::mutex g_scratch_mutex;
float* g_scratch_ptr[MNV_MAX_DEVICES];  // device address of `scratch` on each GPU

// The address of the current device's copy of `scratch`, looked up once per device.
int scratch_address(float** out) {
  int dev = -1;
  MNV_HIP_TRY(hipGetDevice(&dev));
  if (dev < 0 || dev >= MNV_MAX_DEVICES) return MNV_ERR_INVALID;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    MNV_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return MNV_ERR_INVALID;
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *out = g_scratch_ptr[dev];
  return MNV_OK;
}

int sgemm_nn_impl(const float* a, const float* b, float* c, int m, int n, int k, void* workspace,
                  size_t workspace_bytes, hipStream_t s,
                  const SgemmEpilogue& e = SgemmEpilogue{nullptr, nullptr, 0}) {
  bool vec = (m % 4 == 0) && (k % 4 == 0) && mnv_aligned16(a) && mnv_aligned16(b) &&
             e.lda % 4 == 0 && e.ldb % 4 == 0;
  const SgemmPlan plan = plan_sgemm(m, n, k, workspace ? workspace_bytes / sizeof(float) : 0);
  if (vec) return launch_plan(plan, make_sgemm<true>(a, b, c, m, n, k, e), workspace, workspace_bytes, s);
  return launch_plan(plan, make_sgemm<false>(a, b, c, m, n, k, e), workspace, workspace_bytes, s);
}

// Products with one operand given transposed: same plan (tile shape, k ranges) as the plain
// product of the same extents, so that the result has the bits of transposing first.
template <bool TA, bool TB>
int sgemm_t_impl(const float* a, const float* b, float* c, int m, int n, int k, void* workspace,
                 size_t workspace_bytes, hipStream_t s, const SgemmEpilogue& e) {
  const bool vec = mnv_aligned16(a) && mnv_aligned16(b) && (TA ? k % 4 == 0 : m % 4 == 0) &&
                   (TB ? n % 4 == 0 : k % 4 == 0);
  SgemmPlan plan = plan_sgemm(m, n, k, workspace ? workspace_bytes / sizeof(float) : 0);
  // a B given transposed is fetched along n: measured on 4096^3, 0.987 ms on the 256 x 128
  // tile against 0.951 on 128 x 128 (the bits are the same on either)
  if (TB) plan.tall = false;
  if (vec) return launch_plan(plan, make_sgemm<true, TA, TB>(a, b, c, m, n, k, e), workspace, workspace_bytes, s);
  return launch_plan(plan, make_sgemm<false, TA, TB>(a, b, c, m, n, k, e), workspace, workspace_bytes, s);
}

// Operands of 2^29 elements and more (up to the reference's limit, int element counts): the
// product is cut into panels whose spans fit 32-bit byte offsets -- columns of B and C, rows
// of A and C, and ranges of k, the later k ranges accumulating into C -- each panel one launch
// with the whole matrices' leading dimensions.  Slower than one launch (C is re-read per k
// range, no k ranges over workgroups), and the sum over k is taken range by range.
const long long kOperandLimit = (1LL << 29) - 1;  // elements a launch can address per operand

bool sgemm_is_large(int m, int n, int k) {
  return (long long)m * k > kOperandLimit || (long long)k * n > kOperandLimit;
}

int sgemm_nn_large(const float* a, const float* b, float* c, int m, int n, int k, hipStream_t s) {
  const long long mc = m < (1 << 28) ? m : (1 << 28);
  long long kc = (kOperandLimit - mc) / m + 1;          // ((kc-1)*m + mc) <= limit
  if (kc > k) kc = k;
  if (kc >= 16) kc -= kc % 16;
  long long nc = (kOperandLimit - kc) / k + 1;          // ((nc-1)*k + kc) <= limit
  if (nc > n) nc = n;
  if (kc < 1 || nc < 1) return MNV_ERR_INVALID;
  for (long long n0 = 0; n0 < n; n0 += nc)
    for (long long m0 = 0; m0 < m; m0 += mc)
      for (long long k0 = 0; k0 < k; k0 += kc) {
        const int mm = (int)(m - m0 < mc ? m - m0 : mc), nn = (int)(n - n0 < nc ? n - n0 : nc);
        const int kk = (int)(k - k0 < kc ? k - k0 : kc);
        SgemmEpilogue e{nullptr, nullptr, 0, m, k, m, k0 > 0};
        int rc = sgemm_nn_impl(a + (size_t)k0 * m + m0, b + (size_t)n0 * k + k0,
                               c + (size_t)n0 * m + m0, mm, nn, kk, nullptr, 0, s, e);
        if (rc) return rc;
      }
  return MNV_OK;
}

}  // namespace

extern "C" {

size_t mnv_sgemm_nn_workspace_bytes(int m, int n, int k) {
  if (m <= 0 || n <= 0 || k <= 0) return 0;
  const SgemmPlan plan = plan_sgemm(m, n, k, (size_t)-1);
  return plan.splits > 1 ? (size_t)plan.splits * m * n * sizeof(float) : sgemm_tail_bytes(plan, m, n, k);
}

int mnv_sgemm_nn_plan(int m, int n, int k, size_t workspace_bytes, int* tile_rows, int* k_ranges,
                      int* groups) {
  if (m <= 0 || n <= 0 || k <= 0 || !tile_rows || !k_ranges || !groups) return MNV_ERR_INVALID;
  const SgemmPlan plan = plan_sgemm(m, n, k, workspace_bytes / sizeof(float));
  *tile_rows = plan.tall ? 256 : plan.small ? 64 : 128;
  const int slabs = (k + 15) / 16, per = (slabs + plan.splits - 1) / plan.splits;
  *k_ranges = (slabs + per - 1) / per;  // as the launch rounds it: ranges of equal length
  *groups = plan.groups;
  return MNV_OK;
}

int mnv_sgemm_nn(const float* a, const float* b, float* c, int m, int n, int k, void* workspace,
                 size_t workspace_bytes, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !b || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  // every operand is at most 2^31 - 1 elements (the reference's int element counts)
  if ((long long)m * k > 0x7fffffffLL || (long long)k * n > 0x7fffffffLL ||
      (long long)m * n > 0x7fffffffLL)
    return MNV_ERR_INVALID;
  if (sgemm_is_large(m, n, k)) return sgemm_nn_large(a, b, c, m, n, k, mnv_stream(stream));
  return sgemm_nn_impl(a, b, c, m, n, k, workspace, workspace_bytes, mnv_stream(stream));
}

int mnv_sgemm_nn_bias(const float* a, const float* b, const float* bias, float* c, int m, int n,
                      int k, int relu, void* workspace, size_t workspace_bytes,
                      mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !b || !bias || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  return sgemm_nn_impl(a, b, c, m, n, k, workspace, workspace_bytes, mnv_stream(stream),
                       SgemmEpilogue{bias, nullptr, relu != 0});
}

int mnv_sgemm_nn_relu_bwd(const float* a, const float* b, const float* bottom, float* c, int m,
                          int n, int k, void* workspace, size_t workspace_bytes,
                          mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !b || !bottom || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  return sgemm_nn_impl(a, b, c, m, n, k, workspace, workspace_bytes, mnv_stream(stream),
                       SgemmEpilogue{nullptr, bottom, 0});
}

int mnv_sgemm_tn(const float* at, const float* b, const float* gate, float* c, int m, int n, int k,
                 void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!at || !b || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  return sgemm_t_impl<true, false>(at, b, c, m, n, k, workspace, workspace_bytes, mnv_stream(stream),
                                   SgemmEpilogue{nullptr, gate, 0});
}

int mnv_sgemm_nt(const float* a, const float* bt, float* c, int m, int n, int k, void* workspace,
                 size_t workspace_bytes, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !bt || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  return sgemm_t_impl<false, true>(a, bt, c, m, n, k, workspace, workspace_bytes, mnv_stream(stream),
                                   SgemmEpilogue{nullptr, nullptr, 0});
}

int mnv_sgemm_nt_sgd(const float* a, const float* bt, const float* w, float scale, float* w_out,
                     int m, int n, int k, void* workspace, size_t workspace_bytes,
                     mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !bt || !w || !w_out || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  SgemmEpilogue e{nullptr, nullptr, 0};
  e.sgd_w = w;
  e.sgd_scale = scale;
  return sgemm_t_impl<false, true>(a, bt, w_out, m, n, k, workspace, workspace_bytes,
                                   mnv_stream(stream), e);
}

int mnv_sgemm_nn_static(const float* a, const float* b, float* c, int m, int n, int k,
                        mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !b || !c || m < 0 || n < 0 || k <= 0) return MNV_ERR_INVALID;
  if ((long long)m * k >= (1LL << 29) || (long long)k * n >= (1LL << 29)) return MNV_ERR_INVALID;
  // at least two k ranges of partial sums must fit the static array
  if ((unsigned long long)m * (unsigned long long)n * 2ull > MNV_SGEMM_STATIC_SCRATCH_FLOATS)
    return MNV_ERR_TOO_LARGE;
  float* ws = nullptr;
  int rc = scratch_address(&ws);
  if (rc) return rc;
  return sgemm_nn_impl(a, b, c, m, n, k, ws, MNV_SGEMM_STATIC_SCRATCH_BYTES, mnv_stream(stream));
}

}  // extern "C"
