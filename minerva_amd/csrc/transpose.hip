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
//
// SHIFT: when the rows of the result do not lie on 64-byte boundaries (n % 16 != 0 or c off
// such a boundary), a 4*TJ-byte run written at a fixed j0 would begin and end inside a 64-byte
// sector that the neighbouring tile completes later, and the memory side pays a
// read-modify-write for each of the two partial writes (8000 x 8200: 55% of HBM peak against
// 80% at 8192 x 8192).  Each output row i therefore moves its run to the left by
// s_i = (address of c[i*n + j0] in floats) mod 16, so that every run starts and ends on a
// sector boundary; the tile reads 16 more columns on its left to have those values.
template <int TI, int TJ, int NTH, bool NT, bool SHIFT>
__global__ __launch_bounds__(NTH) void mnv_transpose_vec4_kernel(
    const float* __restrict__ a, float* __restrict__ c, int m, int n, int tiles_i, int tiles_j, int diagonal) {
  constexpr int HALO = SHIFT ? 16 : 0;
  __shared__ float tile[TJ + HALO][TI + 1];
  constexpr int LI = TI / 4, CP = NTH / LI, RP = TJ / CP;  // read: lanes per column, columns per pass, passes
  constexpr int LJ = TJ / 4, IP = NTH / LJ, WP = TI / IP;  // write: lanes per row, rows per pass, passes
  static_assert(NTH % LI == 0 && NTH % LJ == 0 && TJ % CP == 0 && TI % IP == 0, "tile/thread mismatch");
  // Tiles along diagonals (see the head of the file) only when both pitches are multiples of
  // 16 KB; otherwise consecutive workgroups take consecutive tiles of a column of tiles
  // (8000 x 8200: 67% against 63% of HBM peak, 8064 x 8192: 71% against 65%; 8192 x 8192:
  // 69% against 81%).
  const int ti = blockIdx.x % tiles_i;
  const int tj = diagonal ? (blockIdx.x / tiles_i + ti) % tiles_j : blockIdx.x / tiles_i;
  const int i0 = ti * TI, j0 = tj * TJ;
  {
    const int tx = threadIdx.x % LI, ty = threadIdx.x / LI;
    constexpr int RPH = (TJ + HALO + CP - 1) / CP;  // passes over the columns incl. the halo
    mnv_f4 v[RPH];
#pragma unroll
    for (int p = 0; p < RPH; ++p) {
      const int jj = ty + CP * p;  // column of the tile in LDS
      int i = i0 + tx * 4, j = j0 - HALO + jj;
      if (jj < TJ + HALO && i < m && j >= 0 && j < n)
        v[p] = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(a + (size_t)j * m + i));
    }
#pragma unroll
    for (int p = 0; p < RPH; ++p) {
      const int jj = ty + CP * p;
      if (jj < TJ + HALO) {
        float* t = &tile[jj][tx * 4];
        t[0] = v[p].x; t[1] = v[p].y; t[2] = v[p].z; t[3] = v[p].w;
      }
    }
  }
  __syncthreads();
  const int tx = threadIdx.x % LJ, ty = threadIdx.x / LJ;
  const int phase = (int)((reinterpret_cast<uintptr_t>(c) >> 2) & 15u);
#pragma unroll
  for (int p = 0; p < WP; ++p) {
    const int r = ty + IP * p, i = i0 + r;
    // floats from the sector boundary at or below c[i*n + j0] to that element (j0 % 16 == 0)
    const int sft = SHIFT ? (((i & 15) * (n & 15) + phase) & 15) : 0;
    const int jj = HALO - sft + tx * 4, j = j0 - HALO + jj;
    if (i < m && j >= 0 && j < n) {
      mnv_f4 o;
      o.x = tile[jj + 0][r];
      o.y = tile[jj + 1][r];
      o.z = tile[jj + 2][r];
      o.w = tile[jj + 3][r];
      __builtin_nontemporal_store(o, reinterpret_cast<mnv_f4*>(c + (size_t)i * n + j));
    }
  }
}

template <int TI, int TJ, int NTH>
int launch_vec4(const float* a, float* c, int m, int n, bool nt, hipStream_t s) {
  // rows of the result off the 64-byte grid: shifted runs (the shift is a multiple of four
  // floats because n % 4 == 0 and c is 16-byte aligned); the last tile then has to reach
  // 12 columns further
  const bool shift = n % 16 != 0 || (reinterpret_cast<uintptr_t>(c) & 63u) != 0;
  const size_t tiles_i = mnv_ceil_div((size_t)m, TI), tiles_j = mnv_ceil_div((size_t)n + (shift ? 12 : 0), TJ);
  if (tiles_i * tiles_j > 0x7fffffffULL) return MNV_ERR_INVALID;
  const int diagonal = m % 4096 == 0 && n % 4096 == 0;
  const dim3 grid((unsigned)(tiles_i * tiles_j)), block(NTH);
#define MNV_TR_LAUNCH(NT, SHIFT)                                                                    \
  hipLaunchKernelGGL((mnv_transpose_vec4_kernel<TI, TJ, NTH, NT, SHIFT>), grid, block, 0, s, a, c, \
                     m, n, (int)tiles_i, (int)tiles_j, diagonal)
  if (shift) {
    if (nt) MNV_TR_LAUNCH(true, true); else MNV_TR_LAUNCH(false, true);
  } else {
    if (nt) MNV_TR_LAUNCH(true, false); else MNV_TR_LAUNCH(false, false);
  }
#undef MNV_TR_LAUNCH
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
