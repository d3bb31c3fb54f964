// Matrix transpose (reference minerva/op/impl/basic.cpp:175-187; cublasSgeam call at
// minerva/op/impl/cuda/cuda_perform.cu:77-81).  a is column-major {m,n}; c is {n,m}:
// c[j + i*n] = a[i + j*m].  Roofline: HBM bandwidth, 8 bytes per element.  A 64x64
// tile goes through LDS so that both the read (along i) and the write (along j) are
// contiguous 256-byte runs per 64 threads; the LDS row pitch of 65 floats keeps the
// transposed reads off a single bank.
#include "mnv_common.h"

namespace {

#define MNV_TR_TILE 64
#define MNV_TR_THREADS 256

__global__ __launch_bounds__(MNV_TR_THREADS) void mnv_transpose_kernel(
    const float* __restrict__ a, float* __restrict__ c, int m, int n, int tiles_i) {
  __shared__ float tile[MNV_TR_TILE][MNV_TR_TILE + 1];
  const int ti = blockIdx.x % tiles_i, tj = blockIdx.x / tiles_i;
  const int i0 = ti * MNV_TR_TILE, j0 = tj * MNV_TR_TILE;
  const int tx = threadIdx.x % MNV_TR_TILE, ty = threadIdx.x / MNV_TR_TILE;
  // read: tx runs along i (contiguous in a)
#pragma unroll
  for (int p = 0; p < MNV_TR_TILE; p += MNV_TR_THREADS / MNV_TR_TILE) {
    int i = i0 + tx, j = j0 + ty + p;
    if (i < m && j < n) tile[ty + p][tx] = a[(size_t)j * m + i];
  }
  __syncthreads();
  // write: tx runs along j (contiguous in c)
#pragma unroll
  for (int p = 0; p < MNV_TR_TILE; p += MNV_TR_THREADS / MNV_TR_TILE) {
    int j = j0 + tx, i = i0 + ty + p;
    if (i < m && j < n) c[(size_t)i * n + j] = tile[tx][ty + p];
  }
}

}  // namespace

extern "C" int mnv_transpose(const float* a, float* c, int m, int n, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !c || m < 0 || n < 0) return MNV_ERR_INVALID;
  size_t tiles_i = mnv_ceil_div((size_t)m, MNV_TR_TILE), tiles_j = mnv_ceil_div((size_t)n, MNV_TR_TILE);
  if (tiles_i * tiles_j > 0x7fffffffULL) return MNV_ERR_INVALID;
  hipLaunchKernelGGL(mnv_transpose_kernel, dim3((unsigned)(tiles_i * tiles_j)),
                     dim3(MNV_TR_THREADS), 0, mnv_stream(stream), a, c, m, n, (int)tiles_i);
  return MNV_LAUNCH_STATUS();
}
