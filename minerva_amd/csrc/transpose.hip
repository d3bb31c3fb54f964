// Matrix transpose (reference minerva/op/impl/basic.cpp:175-187; cublasSgeam call at
// minerva/op/impl/cuda/cuda_perform.cu:77-81).  a is column-major {m,n}; c is {n,m}:
// c[j + i*n] = a[i + j*m].  Roofline: HBM bandwidth, 8 bytes per element.  A 64x64
// tile goes through LDS so that both the read (along i) and the write (along j) are
// contiguous 256-byte runs per 64 threads; the LDS row pitch of 65 floats keeps the
// transposed reads off a single bank.  Tiles are visited along diagonals: workgroups that
// run together then differ in both their row and their column offset, so neither their
// reads nor their writes (whose addresses would otherwise differ by multiples of 64 rows
// of a power-of-two pitch) pile onto a few memory channels.
#include "mnv_common.h"

namespace {

#define MNV_TR_TILE 64
#define MNV_TR_THREADS 256

__global__ __launch_bounds__(MNV_TR_THREADS) void mnv_transpose_kernel(
    const float* __restrict__ a, float* __restrict__ c, int m, int n, int tiles_i, int tiles_j) {
  __shared__ float tile[MNV_TR_TILE][MNV_TR_TILE + 1];
  const int ti = blockIdx.x % tiles_i, tj = (blockIdx.x / tiles_i + ti) % tiles_j;
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

// 16-byte global accesses on both sides: a thread reads four consecutive i of one column
// and writes four consecutive j of one output column; the 64x64 tile is transposed
// through LDS with 4-byte accesses.  Needs m % 4 == 0, n % 4 == 0 and aligned pointers.
template <bool NT>
__global__ __launch_bounds__(MNV_TR_THREADS) void mnv_transpose_vec4_kernel(
    const float* __restrict__ a, float* __restrict__ c, int m, int n, int tiles_i, int tiles_j) {
  __shared__ float tile[MNV_TR_TILE][MNV_TR_TILE + 1];
  const int ti = blockIdx.x % tiles_i, tj = (blockIdx.x / tiles_i + ti) % tiles_j;
  const int i0 = ti * MNV_TR_TILE, j0 = tj * MNV_TR_TILE;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  mnv_f4 v[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    int i = i0 + tx * 4, j = j0 + ty + 16 * p;
    if (i < m && j < n) v[p] = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(a + (size_t)j * m + i));
  }
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    float* t = &tile[ty + 16 * p][tx * 4];
    t[0] = v[p].x; t[1] = v[p].y; t[2] = v[p].z; t[3] = v[p].w;
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    int j = j0 + tx * 4, i = i0 + ty + 16 * p;
    if (i < m && j < n) {
      mnv_f4 o;
      o.x = tile[tx * 4 + 0][ty + 16 * p];
      o.y = tile[tx * 4 + 1][ty + 16 * p];
      o.z = tile[tx * 4 + 2][ty + 16 * p];
      o.w = tile[tx * 4 + 3][ty + 16 * p];
      __builtin_nontemporal_store(o, reinterpret_cast<mnv_f4*>(c + (size_t)i * n + j));
    }
  }
}

}  // namespace

extern "C" int mnv_transpose(const float* a, float* c, int m, int n, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !c || m < 0 || n < 0) return MNV_ERR_INVALID;
  size_t tiles_i = mnv_ceil_div((size_t)m, MNV_TR_TILE), tiles_j = mnv_ceil_div((size_t)n, MNV_TR_TILE);
  if (tiles_i * tiles_j > 0x7fffffffULL) return MNV_ERR_INVALID;
  const bool vec = m % 4 == 0 && n % 4 == 0 && mnv_aligned16(a) && mnv_aligned16(c);
  if (vec && (size_t)m * n * sizeof(float) >= MNV_PAST_CACHE_BYTES)
    hipLaunchKernelGGL(mnv_transpose_vec4_kernel<true>, dim3((unsigned)(tiles_i * tiles_j)),
                       dim3(MNV_TR_THREADS), 0, mnv_stream(stream), a, c, m, n, (int)tiles_i, (int)tiles_j);
  else if (vec)
    hipLaunchKernelGGL(mnv_transpose_vec4_kernel<false>, dim3((unsigned)(tiles_i * tiles_j)),
                       dim3(MNV_TR_THREADS), 0, mnv_stream(stream), a, c, m, n, (int)tiles_i, (int)tiles_j);
  else
    hipLaunchKernelGGL(mnv_transpose_kernel, dim3((unsigned)(tiles_i * tiles_j)),
                       dim3(MNV_TR_THREADS), 0, mnv_stream(stream), a, c, m, n, (int)tiles_i, (int)tiles_j);
  return MNV_LAUNCH_STATUS();
}
