// fp32 MFMA GEMM core for gfx950, shared by SGEMM and the implicit-GEMM convolutions.
//
// Computes C[m,n] = sum_k A[m,k] * B[k,n] for one BM x BN tile per workgroup (and one
// k range per blockIdx.z when the k dimension is split).  The operands are described
// by a Problem policy: it knows how to fetch four values of A or B at once, either
// four consecutive m/n at one k ("x-fast", the natural direction of a column-major
// left operand or of an im2col gather) or four consecutive k at one m/n ("k-fast", a
// column-major right operand or a filter), and how to store an element of C.  So a
// convolution never materialises its im2col matrix: the gather happens on the way
// from HBM to LDS.
//
// Data path: HBM -> registers (policy fetch, issued one k-slab ahead) -> LDS, two
// slabs deep (double buffered, one barrier per slab) -> one fp32 value per lane per
// operand -> v_mfma_f32_32x32x2_f32.  Each wavefront owns a (TM*32) x (TN*32) block of
// accumulators.  The MFMA is issued with the operands swapped (B as the "A" input) so
// that the 64 lanes of an accumulator register hold 32 consecutive m: the C store of
// a column-major result is then 128 contiguous bytes per half wavefront.
//
// Roofline: fp32 MFMA, 2*M*N*K algorithmic flops; 256 flop/clk/CU.
#pragma once
#include "mnv_common.h"

typedef float mnv_f16v __attribute__((ext_vector_type(16)));

// Division by a run-time constant, prepared on the host (valid for 0 <= n < 2^31).
struct MnvFastDiv {
  unsigned mul, shift;
  int d;
};

static inline MnvFastDiv mnv_fastdiv_make(int d) {
  MnvFastDiv f;
  f.d = d;
  if (d <= 1) {
    f.mul = 0;
    f.shift = 0;
    return f;
  }
  unsigned lg = 0;
  while ((1ull << lg) < (unsigned long long)d) ++lg;  // ceil(log2 d)
  unsigned p = 31 + lg;
  f.mul = (unsigned)(((1ull << p) + (unsigned)d - 1) / (unsigned)d);
  f.shift = p - 32;
  return f;
}

#ifdef __HIPCC__
__device__ __forceinline__ int mnv_fastdiv(int n, const MnvFastDiv& f) {
  return f.d == 1 ? n : (int)(__umulhi((unsigned)n, f.mul) >> f.shift);
}

template <int BM_, int BN_, int BK_, int WGM_, int WGN_, int PAD_ = 0>
struct MnvGemmTile {
  static constexpr int BM = BM_, BN = BN_, BK = BK_, WGM = WGM_, WGN = WGN_;
  static constexpr int NT = MNV_WAVE * WGM * WGN;
  static constexpr int WM = BM / WGM, WN = BN / WGN;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int LDA = BM + PAD_, LDB = BN + PAD_;
  static constexpr int AV = BM * BK / (4 * NT);  // 4-vectors of A per thread per slab
  static constexpr int BV = BN * BK / (4 * NT);
  static constexpr size_t LDS_BYTES = (size_t)2 * BK * (LDA + LDB) * sizeof(float);
  static_assert(WM % 32 == 0 && WN % 32 == 0, "wave tile must be a multiple of 32x32");
  static_assert(BK % 4 == 0 && (BM * BK) % (4 * NT) == 0 && (BN * BK) % (4 * NT) == 0, "tile/thread mismatch");
};

// Per-thread position of its fetches inside an operand tile (BX x BK).
//  x-fast: vector p covers x = xg*4..+3 at k = kr + p*RP
//  k-fast: vector p covers k = kg*4..+3 at x = xc + p*CP
template <int BX, int BK, int NT, bool KFAST>
struct MnvFetchMap {
  static constexpr int GX = BX / 4, RP = NT / GX;  // x-fast
  static constexpr int GK = BK / 4, CP = NT / GK;  // k-fast
  static_assert(KFAST || (NT % GX == 0 && RP >= 1 && (BK % RP == 0 || RP > BK)), "x-fast map");
  static_assert(!KFAST || (NT % GK == 0 && BX % CP == 0), "k-fast map");
  __device__ static int x(int tid, int p) { return KFAST ? (tid / GK + p * CP) : (tid % GX) * 4; }
  __device__ static int k(int tid, int p) { return KFAST ? (tid % GK) * 4 : (tid / GX + p * RP); }
};

// Problem policy contract (all __device__):
//   static constexpr bool A_KFAST, B_KFAST;
//   struct AState / BState;                          per-thread, per-fetch-vector state
//   void a_init(AState&, int x /*m, global*/) const;   called once per vector slot
//   void a_fetch(const AState&, int m, int k, float (&v)[4]) const;   zero-fills out of range
//   (same for b with n)
//   void c_store(int m, int n, float v) const;         only called for m < M, n < N
//   int M, N, K;
template <class T, class P>
__global__ __launch_bounds__(T::NT) void mnv_gemm_kernel(P prob, int tiles_m, int tiles_n,
                                                         int slabs_per_split,
                                                         float* __restrict__ partial) {
  extern __shared__ float mnv_gemm_lds[];
  float* As = mnv_gemm_lds;                       // [2][BK][LDA]
  float* Bs = mnv_gemm_lds + 2 * T::BK * T::LDA;  // [2][BK][LDB]
  typedef MnvFetchMap<T::BM, T::BK, T::NT, P::A_KFAST> MapA;
  typedef MnvFetchMap<T::BN, T::BK, T::NT, P::B_KFAST> MapB;

  const int tid = threadIdx.x;
  // Workgroups are dealt round-robin to the 8 XCDs; remap so that each XCD (one L2)
  // works on a contiguous run of tiles that share B panels.
  int b = blockIdx.x;
  const int total = tiles_m * tiles_n;
  const int per_xcd = total / 8;
  if (b < per_xcd * 8) b = (b % 8) * per_xcd + b / 8;
  const int tile_m = b % tiles_m, tile_n = b / tiles_m;
  const int m0 = tile_m * T::BM, n0 = tile_n * T::BN;

  const int total_slabs = (prob.K + T::BK - 1) / T::BK;
  const int slab_begin = blockIdx.z * slabs_per_split;
  int slab_end = slab_begin + slabs_per_split;
  if (slab_end > total_slabs) slab_end = total_slabs;

  typename P::AState ast[T::AV];
  typename P::BState bst[T::BV];
#pragma unroll
  for (int p = 0; p < T::AV; ++p) prob.a_init(ast[p], m0 + MapA::x(tid, p));
#pragma unroll
  for (int p = 0; p < T::BV; ++p) prob.b_init(bst[p], n0 + MapB::x(tid, p));

  float ra[T::AV][4], rb[T::BV][4];

  auto fetch = [&](int slab) {
    const int k0 = slab * T::BK;
#pragma unroll
    for (int p = 0; p < T::AV; ++p)
      prob.a_fetch(ast[p], m0 + MapA::x(tid, p), k0 + MapA::k(tid, p), ra[p]);
#pragma unroll
    for (int p = 0; p < T::BV; ++p)
      prob.b_fetch(bst[p], n0 + MapB::x(tid, p), k0 + MapB::k(tid, p), rb[p]);
  };
  auto stash = [&](int buf) {
    float* a = As + buf * T::BK * T::LDA;
    float* bb = Bs + buf * T::BK * T::LDB;
#pragma unroll
    for (int p = 0; p < T::AV; ++p) {
      const int x = MapA::x(tid, p), k = MapA::k(tid, p);
      if (P::A_KFAST) {
#pragma unroll
        for (int q = 0; q < 4; ++q) a[(k + q) * T::LDA + x] = ra[p][q];
      } else {
        mnv_f4 v = {ra[p][0], ra[p][1], ra[p][2], ra[p][3]};
        *reinterpret_cast<mnv_f4*>(a + k * T::LDA + x) = v;
      }
    }
#pragma unroll
    for (int p = 0; p < T::BV; ++p) {
      const int x = MapB::x(tid, p), k = MapB::k(tid, p);
      if (P::B_KFAST) {
#pragma unroll
        for (int q = 0; q < 4; ++q) bb[(k + q) * T::LDB + x] = rb[p][q];
      } else {
        mnv_f4 v = {rb[p][0], rb[p][1], rb[p][2], rb[p][3]};
        *reinterpret_cast<mnv_f4*>(bb + k * T::LDB + x) = v;
      }
    }
  };

  mnv_f16v acc[T::TM][T::TN];
#pragma unroll
  for (int i = 0; i < T::TM; ++i)
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int wave = tid / MNV_WAVE, lane = tid % MNV_WAVE;
  const int wm = (wave % T::WGM) * T::WM, wn = (wave / T::WGM) * T::WN;
  const int lm = lane % 32, lk = lane / 32;

  if (slab_begin < slab_end) {
    fetch(slab_begin);
    stash(0);
  }
  __syncthreads();

  for (int slab = slab_begin; slab < slab_end; ++slab) {
    const int buf = (slab - slab_begin) & 1;
    const bool more = slab + 1 < slab_end;
    if (more) fetch(slab + 1);  // global loads in flight while this slab is multiplied
    const float* a = As + buf * T::BK * T::LDA + wm + lm;
    const float* bb = Bs + buf * T::BK * T::LDB + wn + lm;
#pragma unroll
    for (int kk = 0; kk < T::BK / 2; ++kk) {
      float av[T::TM], bv[T::TN];
#pragma unroll
      for (int i = 0; i < T::TM; ++i) av[i] = a[(kk * 2 + lk) * T::LDA + i * 32];
#pragma unroll
      for (int j = 0; j < T::TN; ++j) bv[j] = bb[(kk * 2 + lk) * T::LDB + j * 32];
#pragma unroll
      for (int i = 0; i < T::TM; ++i)
#pragma unroll
        for (int j = 0; j < T::TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j], av[i], acc[i][j], 0, 0, 0);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
  }

  // Accumulator register r of lane (lm, lk) holds C[m = lm, n = lk*4 + r%4 + 8*(r/4)]
  // of its 32x32 block.
  const bool split = gridDim.z > 1;
  float* part = split ? partial + (size_t)blockIdx.z * prob.M * prob.N : nullptr;
#pragma unroll
  for (int i = 0; i < T::TM; ++i) {
    const int m = m0 + wm + i * 32 + lm;
    if (m >= prob.M) continue;
#pragma unroll
    for (int j = 0; j < T::TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int n = n0 + wn + j * 32 + lk * 4 + (r & 3) + 8 * (r >> 2);
        if (n < prob.N) {
          if (split) part[(size_t)n * prob.M + m] = acc[i][j][r];
          else prob.c_store(m, n, acc[i][j][r]);
        }
      }
  }
}

// Sums the per-split partial results in split order (deterministic) and hands each
// element to the policy's store.
template <class P>
__global__ __launch_bounds__(256) void mnv_gemm_splitk_reduce_kernel(P prob,
                                                                    const float* __restrict__ partial,
                                                                    int splits) {
  const size_t mn = (size_t)prob.M * prob.N;
  for (size_t q = (size_t)blockIdx.x * 256 + threadIdx.x; q < mn; q += (size_t)gridDim.x * 256) {
    float s = partial[q];
    for (int z = 1; z < splits; ++z) s += partial[(size_t)z * mn + q];
    prob.c_store((int)(q % prob.M), (int)(q / prob.M), s);
  }
}

// Host-side launch of one tile configuration.  `splits` > 1 needs
// splits*M*N*sizeof(float) bytes at `workspace`.
template <class T, class P>
static int mnv_gemm_launch(const P& prob, int splits, void* workspace, hipStream_t s) {
  const int tiles_m = (prob.M + T::BM - 1) / T::BM, tiles_n = (prob.N + T::BN - 1) / T::BN;
  const int total_slabs = (prob.K + T::BK - 1) / T::BK;
  if (splits < 1) splits = 1;
  if (splits > total_slabs) splits = total_slabs > 0 ? total_slabs : 1;
  int per = (total_slabs + splits - 1) / splits;
  if (per < 1) per = 1;
  splits = total_slabs > 0 ? (total_slabs + per - 1) / per : 1;
  if ((long long)tiles_m * tiles_n > 0x7fffffffLL || splits > 65535) return MNV_ERR_INVALID;
  static bool attr_set = false;  // idempotent; a race only repeats the same call
  if (!attr_set && T::LDS_BYTES > 48 * 1024) {
    MNV_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void*>(&mnv_gemm_kernel<T, P>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)T::LDS_BYTES));
    attr_set = true;
  }
  hipLaunchKernelGGL((mnv_gemm_kernel<T, P>), dim3(tiles_m * tiles_n, 1, splits), dim3(T::NT),
                     T::LDS_BYTES, s, prob, tiles_m, tiles_n, per,
                     reinterpret_cast<float*>(workspace));
  int rc = MNV_LAUNCH_STATUS();
  if (rc) return rc;
  if (splits > 1) {
    size_t mn = (size_t)prob.M * prob.N;
    size_t blocks = mnv_ceil_div(mn, 256);
    if (blocks > MNV_MAX_STREAM_BLOCKS) blocks = MNV_MAX_STREAM_BLOCKS;
    hipLaunchKernelGGL((mnv_gemm_splitk_reduce_kernel<P>), dim3((unsigned)blocks), dim3(256), 0, s,
                       prob, reinterpret_cast<const float*>(workspace), splits);
    rc = MNV_LAUNCH_STATUS();
  }
  return rc;
}
#endif  // __HIPCC__
