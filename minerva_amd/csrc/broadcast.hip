// Broadcast ("norm") arithmetic on a column-major {m,n} matrix: the matrix is
// combined with a vector that is replicated along one dimension (reference
// minerva/op/impl/basic.cpp:319-367; CUDA kernels cuda_kernel.h:107-130).
// HBM stream, 8 bytes per element (+ the vector, which stays in cache).
//   col variant: vec has n entries, one per column  -> res[r + c*m] = M[r + c*m] (op) vec[c]
//   row variant: vec has m entries, one per row     -> res[r + c*m] = M[r + c*m] (op) vec[r]
// Work is laid out as (column, 1 KiB row segment) tiles so every wavefront access is
// contiguous and no thread divides by m.
#include "mnv_common.h"

namespace {

struct OpAdd { __device__ float operator()(float a, float b) const { return a + b; } };
struct OpSub { __device__ float operator()(float a, float b) const { return a - b; } };
struct OpMul { __device__ float operator()(float a, float b) const { return a * b; } };
struct OpDiv { __device__ float operator()(float a, float b) const { return a / b; } };

#define MNV_BC_THREADS 256
#define MNV_BC_COLS 4  // columns per workgroup iteration: 4 independent 16-byte loads in flight

// ROWVEC = true: vector indexed by row (shape {m,1}); false: by column ({1,n}).
template <class Op, bool ROWVEC, bool VEC4, bool NT>
__global__ __launch_bounds__(MNV_BC_THREADS) void mnv_norm_kernel(
    const float* __restrict__ mat, const float* __restrict__ vec, float* __restrict__ res, int m,
    int n, Op op) {
  constexpr int W = VEC4 ? 4 : 1;
  const int rows_per_block = MNV_BC_THREADS * W;
  const int r0 = blockIdx.x * rows_per_block + threadIdx.x * W;
  if (r0 >= m) return;
  float rv[W];
  if (ROWVEC) {
#pragma unroll
    for (int q = 0; q < W; ++q) rv[q] = (r0 + q < m) ? vec[r0 + q] : 0.f;
  }
  for (int c0 = blockIdx.y * MNV_BC_COLS; c0 < n; c0 += gridDim.y * MNV_BC_COLS) {
    if (VEC4) {
      mnv_f4 v[MNV_BC_COLS];
#pragma unroll
      for (int u = 0; u < MNV_BC_COLS; ++u)
        if (c0 + u < n)
          v[u] = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(mat + (size_t)(c0 + u) * m + r0));
#pragma unroll
      for (int u = 0; u < MNV_BC_COLS; ++u)
        if (c0 + u < n) {
          float cv = ROWVEC ? 0.f : vec[c0 + u];
          mnv_f4 o;
          o.x = op(v[u].x, ROWVEC ? rv[0] : cv);
          o.y = op(v[u].y, ROWVEC ? rv[1 % W] : cv);
          o.z = op(v[u].z, ROWVEC ? rv[2 % W] : cv);
          o.w = op(v[u].w, ROWVEC ? rv[3 % W] : cv);
          if (NT) __builtin_nontemporal_store(o, reinterpret_cast<mnv_f4*>(res + (size_t)(c0 + u) * m + r0));
          else *reinterpret_cast<mnv_f4*>(res + (size_t)(c0 + u) * m + r0) = o;
        }
    } else {
#pragma unroll
      for (int u = 0; u < MNV_BC_COLS; ++u)
        if (c0 + u < n) {
          size_t i = (size_t)(c0 + u) * m + r0;
          res[i] = op(mat[i], ROWVEC ? rv[0] : vec[c0 + u]);
        }
    }
  }
}

template <class Op, bool ROWVEC>
int launch_norm(const float* mat, const float* vec, float* res, int m, int n, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!mat || !vec || !res || m < 0 || n < 0) return MNV_ERR_INVALID;
  bool vec4 = (m % 4 == 0) && mnv_aligned16(mat) && mnv_aligned16(res);
  int rows_per_block = MNV_BC_THREADS * (vec4 ? 4 : 1);
  unsigned gx = (unsigned)mnv_ceil_div((size_t)m, rows_per_block);
  // enough column groups to give ~8192 workgroups in total, at most one per column group
  unsigned want = 8192u / (gx ? gx : 1u);
  unsigned gy = (unsigned)mnv_ceil_div((size_t)n, MNV_BC_COLS);
  if (gy > want) gy = want ? want : 1u;
  if (gy > 65535u) gy = 65535u;
  dim3 grid(gx, gy);
  // past the 256 MB last-level cache the matrix streams with non-temporal accesses
  const bool nt = (size_t)m * n * 8 >= ((size_t)512 << 20);
  if (vec4 && nt)
    hipLaunchKernelGGL((mnv_norm_kernel<Op, ROWVEC, true, true>), grid, dim3(MNV_BC_THREADS), 0,
                       mnv_stream(stream), mat, vec, res, m, n, Op());
  else if (vec4)
    hipLaunchKernelGGL((mnv_norm_kernel<Op, ROWVEC, true, false>), grid, dim3(MNV_BC_THREADS), 0,
                       mnv_stream(stream), mat, vec, res, m, n, Op());
  else
    hipLaunchKernelGGL((mnv_norm_kernel<Op, ROWVEC, false, false>), grid, dim3(MNV_BC_THREADS), 0,
                       mnv_stream(stream), mat, vec, res, m, n, Op());
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" {
#define MNV_NORM_ENTRY(name, OP, ROWVEC)                                                   \
  int name(const float* matrix, const float* vec, float* res, int m, int n, mnv_stream_t s) { \
    return launch_norm<OP, ROWVEC>(matrix, vec, res, m, n, s);                             \
  }
MNV_NORM_ENTRY(mnv_norm_add_col, OpAdd, false)
MNV_NORM_ENTRY(mnv_norm_sub_col, OpSub, false)
MNV_NORM_ENTRY(mnv_norm_mul_col, OpMul, false)
MNV_NORM_ENTRY(mnv_norm_div_col, OpDiv, false)
MNV_NORM_ENTRY(mnv_norm_add_row, OpAdd, true)
MNV_NORM_ENTRY(mnv_norm_sub_row, OpSub, true)
MNV_NORM_ENTRY(mnv_norm_mul_row, OpMul, true)
MNV_NORM_ENTRY(mnv_norm_div_row, OpDiv, true)
}  // extern "C"
