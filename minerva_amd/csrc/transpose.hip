// Matrix transpose (reference minerva/op/impl/basic.cpp:175-187; cublasSgeam call at
// minerva/op/impl/cuda/cuda_perform.cu:77-81).  a is column-major {m,n}; c is {n,m}:
// c[j + i*n] = a[i + j*m].  Roofline: HBM bandwidth, 8 bytes per element.  A square
// tile goes through LDS so that both the read (along i) and the write (along j) are
// contiguous runs of a whole tile edge; the odd LDS row pitch keeps the transposed
// reads off a single bank.  Tiles are visited along diagonals: workgroups that
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
// and writes four consecutive j of one output column; the TI x TJ tile is transposed
// through LDS with 4-byte accesses.  Needs m % 4 == 0, n % 4 == 0 and aligned pointers.
// Two shapes: 64x64 with 256 threads (16 KB of LDS, many small workgroups: matrices of a
// few hundred tiles) and 128x128 with 1024 threads (66 KB), whose 512-byte runs on both
// sides are what HBM wants: 6.4 TB/s against 5.7 TB/s for the small tile at 8192 x 8192.
template <int TI, int TJ, int NTH, bool NT>
__global__ __launch_bounds__(NTH) void mnv_transpose_vec4_kernel(
    const float* __restrict__ a, float* __restrict__ c, int m, int n, int tiles_i, int tiles_j) {
  __shared__ float tile[TJ][TI + 1];
  constexpr int LI = TI / 4, CP = NTH / LI, RP = TJ / CP;  // read: lanes per column, columns per pass, passes
  constexpr int LJ = TJ / 4, IP = NTH / LJ, WP = TI / IP;  // write: lanes per row, rows per pass, passes
  static_assert(NTH % LI == 0 && NTH % LJ == 0 && TJ % CP == 0 && TI % IP == 0, "tile/thread mismatch");
  const int ti = blockIdx.x % tiles_i, tj = (blockIdx.x / tiles_i + ti) % tiles_j;
  const int i0 = ti * TI, j0 = tj * TJ;
  {
    const int tx = threadIdx.x % LI, ty = threadIdx.x / LI;
    mnv_f4 v[RP];
#pragma unroll
    for (int p = 0; p < RP; ++p) {
      int i = i0 + tx * 4, j = j0 + ty + CP * p;
      if (i < m && j < n) v[p] = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(a + (size_t)j * m + i));
    }
#pragma unroll
    for (int p = 0; p < RP; ++p) {
      float* t = &tile[ty + CP * p][tx * 4];
      t[0] = v[p].x; t[1] = v[p].y; t[2] = v[p].z; t[3] = v[p].w;
    }
  }
  __syncthreads();
  const int tx = threadIdx.x % LJ, ty = threadIdx.x / LJ;
#pragma unroll
  for (int p = 0; p < WP; ++p) {
    int j = j0 + tx * 4, i = i0 + ty + IP * p;
    if (i < m && j < n) {
      mnv_f4 o;
      o.x = tile[tx * 4 + 0][ty + IP * p];
      o.y = tile[tx * 4 + 1][ty + IP * p];
      o.z = tile[tx * 4 + 2][ty + IP * p];
      o.w = tile[tx * 4 + 3][ty + IP * p];
      __builtin_nontemporal_store(o, reinterpret_cast<mnv_f4*>(c + (size_t)i * n + j));
    }
  }
}

template <int TI, int TJ, int NTH>
int launch_vec4(const float* a, float* c, int m, int n, bool nt, hipStream_t s) {
  const size_t tiles_i = mnv_ceil_div((size_t)m, TI), tiles_j = mnv_ceil_div((size_t)n, TJ);
  if (tiles_i * tiles_j > 0x7fffffffULL) return MNV_ERR_INVALID;
  const dim3 grid((unsigned)(tiles_i * tiles_j)), block(NTH);
  if (nt)
    hipLaunchKernelGGL((mnv_transpose_vec4_kernel<TI, TJ, NTH, true>), grid, block, 0, s, a, c, m, n,
                       (int)tiles_i, (int)tiles_j);
  else
    hipLaunchKernelGGL((mnv_transpose_vec4_kernel<TI, TJ, NTH, false>), grid, block, 0, s, a, c, m, n,
                       (int)tiles_i, (int)tiles_j);
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" int mnv_transpose(const float* a, float* c, int m, int n, mnv_stream_t stream) {
  if (m == 0 || n == 0) return MNV_OK;
  if (!a || !c || m < 0 || n < 0) return MNV_ERR_INVALID;
  const bool vec = m % 4 == 0 && n % 4 == 0 && mnv_aligned16(a) && mnv_aligned16(c);
  if (vec) {
    // past the last-level cache the source streams with non-temporal loads
    const bool nt = (size_t)m * n * sizeof(float) >= MNV_PAST_CACHE_BYTES;
    // the large tile from 128 of them on; below that the small tile's four times as many
    // workgroups fill the chip better
    const size_t big_tiles = mnv_ceil_div((size_t)m, 128) * mnv_ceil_div((size_t)n, 128);
    if (big_tiles >= 128) return launch_vec4<128, 128, 1024>(a, c, m, n, nt, mnv_stream(stream));
    return launch_vec4<64, 64, 256>(a, c, m, n, nt, mnv_stream(stream));
  }
  size_t tiles_i = mnv_ceil_div((size_t)m, MNV_TR_TILE), tiles_j = mnv_ceil_div((size_t)n, MNV_TR_TILE);
  if (tiles_i * tiles_j > 0x7fffffffULL) return MNV_ERR_INVALID;
  hipLaunchKernelGGL(mnv_transpose_kernel, dim3((unsigned)(tiles_i * tiles_j)),
                     dim3(MNV_TR_THREADS), 0, mnv_stream(stream), a, c, m, n, (int)tiles_i, (int)tiles_j);
  return MNV_LAUNCH_STATUS();
}
