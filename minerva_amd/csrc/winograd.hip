// 3 x 3 and 5 x 5 unit-stride convolutions by minimal filtering (Winograd / Toom-Cook): an
// m x m block of outputs of one channel pair costs (m + r - 1)^2 multiplies instead of r^2 m^2.
//   F(2 x 2, 3 x 3): 4 x 4 input tiles at stride 2, 16 points, 16 multiplies per 4 outputs;
//   F(4 x 4, 3 x 3): 6 x 6 input tiles at stride 4, 36 points, 36 multiplies per 16 outputs, taken
//                    when it needs clearly fewer products for the plane at hand (13 x 13
//                    outputs: 4 x 4 tiles x 36 = 576 against 7 x 7 x 16 = 784);
//   F(5 x 5, 3 x 3): 7 x 7 input tiles at stride 5, 49 points, 49 multiplies per 25 outputs (13 x 13
//                    outputs: 3 x 3 tiles x 49 = 441);
//   F(4 x 4, 5 x 5): 8 x 8 input tiles at stride 4, 64 points, 64 multiplies per 16 outputs
//                    instead of 400.
// The work becomes al^2 independent matrix products, one per point (xi, nu) of the transformed
// al x al tile (al = m + r - 1),
//     M[xi,nu][co][p] = sum_ci U[xi,nu][co][ci] * V[xi,nu][ci][p],      p = (image, tile row, tile col)
// with U = G g G^T (filters), V = B^T d B (input tiles) and the outputs Y = A^T M A.  The
// products run as ONE launch of the fp32 MFMA core (gemm_core.h): the point is folded into the
// column index, n = point * Coutp + co, and a workgroup picks the V panel of its point once, in
// block_init.  Semantics are those of conv.hip: the forward pass correlates with the flipped
// filter (cuDNN's CUDNN_CONVOLUTION as selected at minerva/op/impl/cuda/cuda_perform.cu:227-264),
// the data gradient (cuda_perform.cu:266-291) is the same correlation of top_diff with the
// unflipped filter, channels exchanged, under a padding of r - 1 - pad.  The filter gradient
// (cuda_perform.cu:293-318) is F(r x r, m x m) on the same points: the m x m tiles of top_diff
// take the filter's place, Yt = G' dy G'^T, the sum over images and tiles is the reduction
// dimension of the products Q[xi,nu][k][c] = sum_p Yt[xi,nu][k][p] V[xi,nu][c][p], and the
// gradient is A'^T Q A'.
//
// The matrices are those of the Toom-Cook construction (evaluation at the points, interpolation
// by the transposed inverse Vandermonde matrix) on {0, 1, -1, inf} (al = 4), {0, 1, -1, 2, -1/2,
// inf} (al = 6), {0, 1, -1, 2, -2, -1/2, inf} (al = 7) and {0, 1, -1, 2, -2, 1/2, -1/2, inf} (al = 8): B^T depends on the points alone
// and serves all three passes.  al = 4 (G and G' carry the halves):
//   B^T = | 1  0 -1  0 |   G = | 1    0    0  |   A^T = | 1  1  1  0 |   G' = | 1    0  |   A'^T = | 1  1  1  0 |
//         | 0  1  1  0 |       | 1/2  1/2  1/2|         | 0  1 -1 -1 |        | 1/2  1/2|          | 0  1 -1  0 |
//         | 0 -1  1  0 |       | 1/2 -1/2  1/2|                              | 1/2 -1/2|          | 0  1  1 -1 |
//         | 0  1  0 -1 |       | 0    0    1  |                              | 0    1  |
// al = 6 and 8: see WinoF below (G, G', A^T, A'^T are powers of the points, exact in fp32; B^T
// carries the fractions).  The point sets were chosen by an fp32 emulation of the whole pass:
// for al = 6 the customary {0, +-1, +-2} gave 2.6 times the error of the set above.
//
// Rounding: the transforms are short sums with small constants, the products are summed in
// fp32 in k order; against the direct sum the results differ by a few 1e-6 of the output's
// largest element (al = 4), up to about 6e-6 (al = 6) and up to about 2.5e-5 (al = 7 and 8);
// the bound of the convolutions is 1e-4.  A whole AlexNet-shaped backward pass at batch 256 is
// 2e-5 from the oracle's with the larger tiles (set by the 8 x 8 tiles of the 5 x 5 layer; the
// tile of the 3 x 3 layers does not move it), 4e-6 on the direct kernels.
// Roofline: the matrix products are MFMA-bound (2 * al^2 * Cout * Cin * tiles flops; with few
// input channels they approach the bandwidth bound of their al^2 * (Cin + Cout) * tiles * 4
// bytes); the transform kernels stream al^2 * 4 bytes per (channel, tile) and are HBM-bound.

#include <mutex>
#include <vector>

#include "gemm_core.h"
#include "winograd.h"

namespace {

struct WinoGeom {
  int N, Cin, Cout, Coutp;  // Coutp: Cout rounded up to the tile width of the product
  int Hs, Ws, Hd, Wd;       // source and destination planes
  int pad_h, pad_w;         // of the correlation: d[a][b] = src[m th - pad_h + a][m tw - pad_w + b]
  int al, r, m;             // points per dimension, filter extent, outputs per tile and dimension (al - r + 1)
  int TH, TW, P, Pp;        // tiles per plane, tiles in all, P rounded up to 4
  MnvFastDiv d_T, d_TW, d_Cin;
};

// The matrices of one tile size as compile-time functions, so that the unrolled transforms
// below fold every coefficient (zeros cost nothing, +-1 no multiply).
template <int AL, int R>
struct WinoF;
template <>
struct WinoF<4, 3> {
  struct BT { static constexpr int R = 4, C = 4;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[4][4] = {{1, 0, -1, 0}, {0, 1, 1, 0}, {0, -1, 1, 0}, {0, 1, 0, -1}};
      return t[i][j]; } };
  struct G { static constexpr int R = 4, C = 3;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[4][3] = {{1, 0, 0}, {.5f, .5f, .5f}, {.5f, -.5f, .5f}, {0, 0, 1}};
      return t[i][j]; } };
  struct AT { static constexpr int R = 2, C = 4;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[2][4] = {{1, 1, 1, 0}, {0, 1, -1, -1}};
      return t[i][j]; } };
  struct GG { static constexpr int R = 4, C = 2;  // G'
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[4][2] = {{1, 0}, {.5f, .5f}, {.5f, -.5f}, {0, 1}};
      return t[i][j]; } };
  struct AAT { static constexpr int R = 3, C = 4;  // A'^T
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[3][4] = {{1, 1, 1, 0}, {0, 1, -1, 0}, {0, 1, 1, -1}};
      return t[i][j]; } };
};
template <>
struct WinoF<6, 3> {
  struct BT { static constexpr int R = 6, C = 6;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[6][6] = {{1, 1.5f, -2, -1.5f, 1, 0},
                                 {0, 1.f / 3, 5.f / 6, 1.f / 6, -1.f / 3, 0},
                                 {0, 1.f / 3, 1.f / 6, -5.f / 6, 1.f / 3, 0},
                                 {0, -1.f / 30, -1.f / 15, 1.f / 30, 1.f / 15, 0},
                                 {0, -32.f / 15, 16.f / 15, 32.f / 15, -16.f / 15, 0},
                                 {0, 1, 1.5f, -2, -1.5f, 1}};
      return t[i][j]; } };
  struct G { static constexpr int R = 6, C = 3;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[6][3] = {{1, 0, 0}, {1, 1, 1}, {1, -1, 1}, {1, 2, 4}, {1, -.5f, .25f}, {0, 0, 1}};
      return t[i][j]; } };
  struct AT { static constexpr int R = 4, C = 6;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[4][6] = {{1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -.5f, 0}, {0, 1, 1, 4, .25f, 0},
                                 {0, 1, -1, 8, -.125f, 1}};
      return t[i][j]; } };
  struct GG { static constexpr int R = 6, C = 4;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[6][4] = {{1, 0, 0, 0}, {1, 1, 1, 1}, {1, -1, 1, -1}, {1, 2, 4, 8},
                                 {1, -.5f, .25f, -.125f}, {0, 0, 0, 1}};
      return t[i][j]; } };
  struct AAT { static constexpr int R = 3, C = 6;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[3][6] = {{1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -.5f, 0}, {0, 1, 1, 4, .25f, 1}};
      return t[i][j]; } };
};
// 3 x 3 filters, 5 x 5 outputs per tile: the points {0, 1, -1, 2, -2, -1/2, inf}
template <>
struct WinoF<7, 3> {
  struct BT { static constexpr int R = 7, C = 7;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[7][7] = {{1, 2, -5.f / 4, -5.f / 2, 1.f / 4, 1.f / 2, 0},
                                 {0, 2.f / 9, 2.f / 3, 7.f / 18, -1.f / 6, -1.f / 9, 0},
                                 {0, 2.f / 3, 2.f / 3, -3.f / 2, -1.f / 6, 1.f / 3, 0},
                                 {0, -1.f / 60, -1.f / 24, 0, 1.f / 24, 1.f / 60, 0},
                                 {0, -1.f / 36, -1.f / 24, 1.f / 18, 1.f / 24, -1.f / 36, 0},
                                 {0, -128.f / 45, 0, 32.f / 9, 0, -32.f / 45, 0},
                                 {0, 2, 4, -5.f / 2, -5, 1.f / 2, 1}};
      return t[i][j]; } };
  struct G { static constexpr int R = 7, C = 3;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[7][3] = {{1, 0, 0}, {1, 1, 1}, {1, -1, 1}, {1, 2, 4}, {1, -2, 4}, {1, -.5f, .25f}, {0, 0, 1}};
      return t[i][j]; } };
  struct AT { static constexpr int R = 5, C = 7;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[5][7] = {{1, 1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, -.5f, 0}, {0, 1, 1, 4, 4, .25f, 0},
                                 {0, 1, -1, 8, -8, -.125f, 0}, {0, 1, 1, 16, 16, .0625f, 1}};
      return t[i][j]; } };
  struct GG { static constexpr int R = 7, C = 5;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[7][5] = {{1, 0, 0, 0, 0}, {1, 1, 1, 1, 1}, {1, -1, 1, -1, 1}, {1, 2, 4, 8, 16},
                                 {1, -2, 4, -8, 16}, {1, -.5f, .25f, -.125f, .0625f}, {0, 0, 0, 0, 1}};
      return t[i][j]; } };
  struct AAT { static constexpr int R = 3, C = 7;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[3][7] = {{1, 1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, -.5f, 0}, {0, 1, 1, 4, 4, .25f, 1}};
      return t[i][j]; } };
};
// 5 x 5 filters, 4 x 4 outputs per tile: the points {0, 1, -1, 2, -2, 1/2, -1/2, inf}
template <>
struct WinoF<8, 5> {
  struct BT { static constexpr int R = 8, C = 8;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[8][8] = {
          {1, 0, -21.f / 4, 0, 21.f / 4, 0, -1, 0},
          {0, -2.f / 9, -2.f / 9, 17.f / 18, 17.f / 18, -2.f / 9, -2.f / 9, 0},
          {0, 2.f / 9, -2.f / 9, -17.f / 18, 17.f / 18, 2.f / 9, -2.f / 9, 0},
          {0, 1.f / 180, 1.f / 360, -1.f / 36, -1.f / 72, 1.f / 45, 1.f / 90, 0},
          {0, -1.f / 180, 1.f / 360, 1.f / 36, -1.f / 72, -1.f / 45, 1.f / 90, 0},
          {0, 64.f / 45, 128.f / 45, -16.f / 9, -32.f / 9, 16.f / 45, 32.f / 45, 0},
          {0, -64.f / 45, 128.f / 45, 16.f / 9, -32.f / 9, -16.f / 45, 32.f / 45, 0},
          {0, -1, 0, 21.f / 4, 0, -21.f / 4, 0, 1}};
      return t[i][j]; } };
  struct G { static constexpr int R = 8, C = 5;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[8][5] = {{1, 0, 0, 0, 0}, {1, 1, 1, 1, 1}, {1, -1, 1, -1, 1}, {1, 2, 4, 8, 16},
                                 {1, -2, 4, -8, 16}, {1, .5f, .25f, .125f, .0625f},
                                 {1, -.5f, .25f, -.125f, .0625f}, {0, 0, 0, 0, 1}};
      return t[i][j]; } };
  struct AT { static constexpr int R = 4, C = 8;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[4][8] = {{1, 1, 1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, .5f, -.5f, 0},
                                 {0, 1, 1, 4, 4, .25f, .25f, 0}, {0, 1, -1, 8, -8, .125f, -.125f, 1}};
      return t[i][j]; } };
  struct GG { static constexpr int R = 8, C = 4;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[8][4] = {{1, 0, 0, 0}, {1, 1, 1, 1}, {1, -1, 1, -1}, {1, 2, 4, 8}, {1, -2, 4, -8},
                                 {1, .5f, .25f, .125f}, {1, -.5f, .25f, -.125f}, {0, 0, 0, 1}};
      return t[i][j]; } };
  struct AAT { static constexpr int R = 5, C = 8;
    __host__ __device__ static constexpr float at(int i, int j) {
      constexpr float t[5][8] = {{1, 1, 1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, .5f, -.5f, 0},
                                 {0, 1, 1, 4, 4, .25f, .25f, 0}, {0, 1, -1, 8, -8, .125f, -.125f, 0},
                                 {0, 1, 1, 16, 16, .0625f, .0625f, 1}};
      return t[i][j]; } };
};

// Points come in pairs +-p.  In B^T, G and G' (one row per point) the rows of such a pair agree
// in their even columns and differ in sign in the odd ones: both are e + o and e - o of one
// even and one odd partial sum.  In A^T and A'^T (one column per point) the columns of a pair
// agree in the even rows and differ in sign in the odd ones: a row needs one product with
// in[j] + in[j+1] or in[j] - in[j+1] instead of two.  Either way the pair costs about half the
// multiplies; which rows / columns pair up is read off the matrix at compile time.
template <class L>
__host__ __device__ constexpr bool wino_row_pair(int i) {
  if (i < 0 || i + 1 >= L::R) return false;
  bool any = false;
  for (int j = 0; j < L::C; ++j) {
    const float a = L::at(i, j), b = L::at(i + 1, j);
    if ((j & 1) ? (b != -a) : (b != a)) return false;
    if (a != 0.f) any = true;
  }
  return any;
}
template <class L>
__host__ __device__ constexpr bool wino_col_pair(int j) {
  if (j < 0 || j + 1 >= L::C) return false;
  bool any = false;
  for (int i = 0; i < L::R; ++i) {
    const float a = L::at(i, j), b = L::at(i, j + 1);
    if ((i & 1) ? (b != -a) : (b != a)) return false;
    if (a != 0.f) any = true;
  }
  return any;
}
// the first row / column of a pair (pairs are taken greedily from the top / left)
template <class L>
__host__ __device__ constexpr bool wino_row_first(int i) {
  return i >= 0 && wino_row_pair<L>(i) && !wino_row_first<L>(i - 1);
}
template <class L>
__host__ __device__ constexpr bool wino_col_first(int j) {
  return j >= 0 && wino_col_pair<L>(j) && !wino_col_first<L>(j - 1);
}
template <class L>
__host__ __device__ constexpr bool wino_has_row_pairs() {
  for (int i = 0; i < L::R; ++i)
    if (wino_row_first<L>(i)) return true;
  return false;
}

__device__ __forceinline__ float wino_term(float c, float x) { return c == 1.f ? x : c == -1.f ? -x : c * x; }

// out = L in for one vector, fully unrolled with the coefficients folded (zeros cost nothing,
// +-1 no multiply).
template <class L>
__device__ __forceinline__ void wino_apply(const float (&in)[L::C], float (&out)[L::R]) {
  if constexpr (wino_has_row_pairs<L>()) {
#pragma unroll
    for (int i = 0; i < L::R; ++i) {
      if (wino_row_first<L>(i - 1)) continue;  // written with its partner
      const bool pair = wino_row_first<L>(i);
      float part[2] = {0.f, 0.f};  // pair: even- and odd-column sums; otherwise all in part[0]
      bool any[2] = {false, false};
#pragma unroll
      for (int j = 0; j < L::C; ++j) {
        const float c = L::at(i, j);
        if (c != 0.f) {
          const int w = pair ? (j & 1) : 0;
          const float t = wino_term(c, in[j]);
          part[w] = any[w] ? part[w] + t : t;
          any[w] = true;
        }
      }
      if (pair) {
        out[i] = part[0] + part[1];
        out[i + 1] = part[0] - part[1];
      } else {
        out[i] = part[0];
      }
    }
  } else {
    float sum[L::C], dif[L::C];
#pragma unroll
    for (int j = 0; j < L::C; ++j) {
      sum[j] = dif[j] = 0.f;
      if (wino_col_first<L>(j)) {
        sum[j] = in[j] + in[j + 1];
        dif[j] = in[j] - in[j + 1];
      }
    }
#pragma unroll
    for (int i = 0; i < L::R; ++i) {
      float acc = 0.f;
      bool any = false;
#pragma unroll
      for (int j = 0; j < L::C; ++j) {
        if (wino_col_first<L>(j - 1)) continue;  // taken with its partner
        const float c = L::at(i, j);
        if (c != 0.f) {
          const float x = wino_col_first<L>(j) ? ((i & 1) ? dif[j] : sum[j]) : in[j];
          const float t = wino_term(c, x);
          acc = any ? acc + t : t;
          any = true;
        }
      }
      out[i] = acc;
    }
  }
}

// out = L in along the rows of a block, out = in L^T along its columns
template <class L, int K>
__device__ __forceinline__ void wino_rows(const float (&in)[L::C][K], float (&out)[L::R][K]) {
#pragma unroll
  for (int k = 0; k < K; ++k) {
    float a[L::C], b[L::R];
#pragma unroll
    for (int j = 0; j < L::C; ++j) a[j] = in[j][k];
    wino_apply<L>(a, b);
#pragma unroll
    for (int i = 0; i < L::R; ++i) out[i][k] = b[i];
  }
}
template <class L, int K>
__device__ __forceinline__ void wino_cols(const float (&in)[K][L::C], float (&out)[K][L::R]) {
#pragma unroll
  for (int k = 0; k < K; ++k) wino_apply<L>(in[k], out[k]);
}

// U[point][co][ci] from filter[k][c][R][R].  Forward: co = k, ci = c, g[r][s] = f[R-1-r][R-1-s];
// data gradient (`transposed`): co = c, ci = k, g = f.  Rows co >= Cout are zero.
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_filter_kernel(const float* __restrict__ filter,
                                                              float* __restrict__ U, WinoGeom g,
                                                              int K, int C, bool transposed) {
  typedef WinoF<AL, R> F;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.Coutp * g.Cin) return;
  const int co = mnv_fastdiv(t, g.d_Cin), ci = t - co * g.Cin;
  float f[R][R];
  if (co < g.Cout) {
    const float* src = transposed ? filter + ((size_t)ci * C + co) * (R * R) : filter + ((size_t)co * C + ci) * (R * R);
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int s = 0; s < R; ++s) f[r][s] = transposed ? src[r * R + s] : src[(R - 1 - r) * R + (R - 1 - s)];
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int s = 0; s < R; ++s) f[r][s] = 0.f;
  }
  float h[AL][R], u[AL][AL];
  wino_rows<typename F::G, R>(f, h);
  wino_cols<typename F::G, AL>(h, u);
  const size_t plane = (size_t)g.Coutp * g.Cin;
  float* out = U + (size_t)co * g.Cin + ci;
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) out[(xi * AL + nu) * plane] = u[xi][nu];
}

// V[point][ci][p] = (B^T d B)[point] of the al x al tile p of channel ci; p >= P writes zeros.
template <int AL, int R>
__device__ __forceinline__ void wino_store_v(float (&d)[AL][AL], float* __restrict__ out, size_t plane) {
  typedef WinoF<AL, R> F;
  float h[AL][AL], v[AL][AL];
  wino_rows<typename F::BT, AL>(d, h);
  wino_cols<typename F::BT, AL>(h, v);
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) out[(xi * AL + nu) * plane] = v[xi][nu];
}

template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_input_kernel(const float* __restrict__ src,
                                                             float* __restrict__ V, WinoGeom g) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int ci = blockIdx.y;
  if (p >= g.Pp) return;
  float d[AL][AL];
#pragma unroll
  for (int a = 0; a < AL; ++a)
#pragma unroll
    for (int b = 0; b < AL; ++b) d[a][b] = 0.f;
  if (p < g.P) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const int y0 = (AL - R + 1) * th - g.pad_h, x0 = (AL - R + 1) * tw - g.pad_w;
    const float* plane = src + ((size_t)img * g.Cin + ci) * (g.Hs * g.Ws);
#pragma unroll
    for (int a = 0; a < AL; ++a)
#pragma unroll
      for (int b = 0; b < AL; ++b) {
        const int y = y0 + a, x = x0 + b;
        if ((unsigned)y < (unsigned)g.Hs && (unsigned)x < (unsigned)g.Ws) d[a][b] = plane[y * g.Ws + x];
      }
  }
  wino_store_v<AL, R>(d, V + (size_t)ci * g.Pp + p, (size_t)g.Cin * g.Pp);
}

// The same through LDS, for planes small enough that the planes of the images a workgroup's
// 256 tiles belong to fit there: they are fetched whole, in runs of contiguous floats (a
// plane of 13 x 13 is 676 contiguous bytes), where the kernel above gathers al^2 values per
// thread at a stride of a few bytes between neighbouring tiles (F(2 x 2) on 384 channels of
// 256 x 13 x 13: 107 -> 80 us).  One channel per workgroup: four (the tile arithmetic done once
// for four) measured 84.7 against 79.6 us.
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_input_lds_kernel(const float* __restrict__ src,
                                                                 float* __restrict__ V, WinoGeom g,
                                                                 MnvFastDiv d_HW) {
  extern __shared__ float planes[];
  const int p0 = blockIdx.x * 256, p = p0 + threadIdx.x;
  const int ci = blockIdx.y;
  const int HW = g.Hs * g.Ws;
  const int img0 = mnv_fastdiv(p0, g.d_T);
  const int last = p0 + 255 < g.P ? p0 + 255 : g.P - 1;
  const int count = (last >= p0 ? mnv_fastdiv(last, g.d_T) - img0 + 1 : 0) * HW;
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pl = mnv_fastdiv(i, d_HW);
    planes[i] = src[((size_t)(img0 + pl) * g.Cin + ci) * HW + (i - pl * HW)];
  }
  __syncthreads();
  if (p >= g.Pp) return;
  float d[AL][AL];
#pragma unroll
  for (int a = 0; a < AL; ++a)
#pragma unroll
    for (int b = 0; b < AL; ++b) d[a][b] = 0.f;
  if (p < g.P) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const int y0 = (AL - R + 1) * th - g.pad_h, x0 = (AL - R + 1) * tw - g.pad_w;
    const float* plane = planes + (img - img0) * HW;
#pragma unroll
    for (int a = 0; a < AL; ++a)
#pragma unroll
      for (int b = 0; b < AL; ++b) {
        const int y = y0 + a, x = x0 + b;
        if ((unsigned)y < (unsigned)g.Hs && (unsigned)x < (unsigned)g.Ws) d[a][b] = plane[y * g.Ws + x];
      }
  }
  wino_store_v<AL, R>(d, V + (size_t)ci * g.Pp + p, (size_t)g.Cin * g.Pp);
}

// dst[img][co][m th + a][m tw + b] = (A^T M A)[a][b] (+ bias[co]) (then max(., 0)) (then kept
// only where gate > 0): the epilogues of the direct kernels, each the single operation of the
// separate operator.
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_output_kernel(const float* __restrict__ Mx,
                                                              const float* __restrict__ bias,
                                                              const float* __restrict__ gate,
                                                              float* __restrict__ dst, WinoGeom g,
                                                              int relu) {
  typedef WinoF<AL, R> F;
  constexpr int MO = AL - R + 1;
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int co = blockIdx.y;
  if (p >= g.P) return;
  const size_t plane = (size_t)g.Coutp * g.Pp;
  const float* in = Mx + (size_t)co * g.Pp + p;
  float mm[AL][AL];
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) mm[xi][nu] = in[(xi * AL + nu) * plane];
  float h[MO][AL], y[MO][MO];
  wino_rows<typename F::AT, AL>(mm, h);
  wino_cols<typename F::AT, MO>(h, y);
  const int img = mnv_fastdiv(p, g.d_T);
  const int t = p - img * (g.TH * g.TW);
  const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
  const float b = bias ? bias[co] : 0.f;
  const size_t base = ((size_t)img * g.Cout + co) * (g.Hd * g.Wd);
#pragma unroll
  for (int a = 0; a < MO; ++a)
#pragma unroll
    for (int c = 0; c < MO; ++c) {
      const int yy = MO * th + a, xx = MO * tw + c;
      if (yy < g.Hd && xx < g.Wd) {
        float v = y[a][c];
        if (bias) v = v + b;
        if (relu) v = v > 0.f ? v : 0.f;
        const size_t at = base + yy * g.Wd + xx;
        if (gate) v = gate[at] > 0.f ? v : 0.f;
        dst[at] = v;
      }
    }
}

// The same through LDS, for planes small enough that the output planes a workgroup's 256
// tiles belong to fit there: a thread leaves its m x m outputs in LDS and the workgroup then
// stores every plane in runs of contiguous floats, where the kernel above stores m floats per
// row and thread, neighbouring threads m floats apart (4 x 4 tiles on 384 channels of
// 256 x 13 x 13: 95 us).  A pixel is stored by the workgroup that holds its tile.
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_output_lds_kernel(const float* __restrict__ Mx,
                                                                  const float* __restrict__ bias,
                                                                  const float* __restrict__ gate,
                                                                  float* __restrict__ dst, WinoGeom g,
                                                                  int relu, MnvFastDiv d_HW, MnvFastDiv d_W) {
  typedef WinoF<AL, R> F;
  constexpr int MO = AL - R + 1;
  extern __shared__ float planes[];
  const int p0 = blockIdx.x * 256, p = p0 + threadIdx.x;
  const int co = blockIdx.y;
  const int HW = g.Hd * g.Wd, T = g.TH * g.TW;
  const int img0 = mnv_fastdiv(p0, g.d_T);
  const int last = p0 + 255 < g.P ? p0 + 255 : g.P - 1;  // p0 < P: the grid covers P
  const int count = (mnv_fastdiv(last, g.d_T) - img0 + 1) * HW;
  if (p < g.P) {
    const size_t plane = (size_t)g.Coutp * g.Pp;
    const float* in = Mx + (size_t)co * g.Pp + p;
    float mm[AL][AL];
#pragma unroll
    for (int xi = 0; xi < AL; ++xi)
#pragma unroll
      for (int nu = 0; nu < AL; ++nu) mm[xi][nu] = in[(xi * AL + nu) * plane];
    float h[MO][AL], y[MO][MO];
    wino_rows<typename F::AT, AL>(mm, h);
    wino_cols<typename F::AT, MO>(h, y);
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * T;
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const float b = bias ? bias[co] : 0.f;
    float* out = planes + (img - img0) * HW;
#pragma unroll
    for (int a = 0; a < MO; ++a)
#pragma unroll
      for (int c = 0; c < MO; ++c) {
        const int yy = MO * th + a, xx = MO * tw + c;
        if (yy < g.Hd && xx < g.Wd) {
          float v = y[a][c];
          if (bias) v = v + b;
          if (relu) v = v > 0.f ? v : 0.f;
          out[yy * g.Wd + xx] = v;
        }
      }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pl = mnv_fastdiv(i, d_HW);
    const int r = i - pl * HW;
    const int yy = mnv_fastdiv(r, d_W), xx = r - yy * g.Wd;
    const int owner = (img0 + pl) * T + (yy / MO) * g.TW + xx / MO;
    if (owner >= p0 && owner <= last) {
      const size_t at = ((size_t)(img0 + pl) * g.Cout + co) * HW + r;
      float v = planes[i];
      if (gate) v = gate[at] > 0.f ? v : 0.f;
      dst[at] = v;
    }
  }
}

// The products of all points as one: C{Pp, points Coutp} = A{Pp, Cin} B{Cin, points Coutp}, column-major, where the
// A of a column tile is the V panel of the tile's transform point.
struct WinoGemm {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  static constexpr int A_NOFF = 1, B_NOFF = 1;
  const float* __restrict__ V;
  const float* __restrict__ U;
  float* __restrict__ Mx;
  int M, N, K, total_slabs, spp;  // Pp, points * Coutp, Cin
  int coutp;
  int n_group;  // column tiles per transform point: they read the same V panel
  static constexpr bool N_GROUPED = true;
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {};
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(V, (unsigned)K * (unsigned)M * 4u);
    r.b = mnv_make_rsrc(U, (unsigned)N * (unsigned)K * 4u);
  }
  __device__ void block_init(Res& r, float*, int, int n0) const {
    r.a = mnv_make_rsrc(V + (size_t)(n0 / coutp) * K * M, (unsigned)K * (unsigned)M * 4u);
  }
  __device__ void a_init(const Res&, AState&, int) const {}
  __device__ void b_init(const Res&, BState&, int) const {}
  __device__ void a_period(const AState&, unsigned (&off)[1], int m, int kl, int period) const {
    const int k = period * spp * 16 + kl;
    off[0] = ((m < M) & (k < K)) ? ((unsigned)k * (unsigned)M + (unsigned)m) * 4u : MNV_OOB;
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[1], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<1>(r.a, off, (unsigned)s * 16u * (unsigned)M * 4u, v);
  }
  __device__ void b_period(const BState&, unsigned (&off)[1], int n, int kl, int period) const {
    const int k = period * spp * 16 + kl;
    off[0] = ((n < N) & (k < K)) ? ((unsigned)n * (unsigned)K + (unsigned)k) * 4u : MNV_OOB;
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[1], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<1>(r.b, off, (unsigned)s * 64u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  __device__ void c_store(int m, int n, float x) const { Mx[(size_t)n * M + m] = x; }
  static constexpr bool C_STORE4 = true;
  __device__ void c_store4(int m, int n, const float (&x)[4]) const {
    const mnv_f4 v = {x[0], x[1], x[2], x[3]};  // M is a multiple of 4: whole and aligned
    *reinterpret_cast<mnv_f4*>(Mx + (size_t)n * M + m) = v;
  }
};

// ---- filter gradient
// Yt[point][k][p] = (G' dy G'^T)[point] of the m x m tile p of channel k of top_diff; zeros
// for p >= P and for the rows k >= Cout.
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_grad_kernel(const float* __restrict__ top_diff,
                                                            float* __restrict__ Yt, WinoGeom g) {
  typedef WinoF<AL, R> F;
  constexpr int MO = AL - R + 1;
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (p >= g.Pp) return;
  float d[MO][MO];
#pragma unroll
  for (int a = 0; a < MO; ++a)
#pragma unroll
    for (int b = 0; b < MO; ++b) d[a][b] = 0.f;
  if (p < g.P && k < g.Cout) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const float* plane = top_diff + ((size_t)img * g.Cout + k) * (g.Hd * g.Wd);
#pragma unroll
    for (int a = 0; a < MO; ++a)
#pragma unroll
      for (int b = 0; b < MO; ++b) {
        const int y = MO * th + a, x = MO * tw + b;
        if (y < g.Hd && x < g.Wd) d[a][b] = plane[y * g.Wd + x];
      }
  }
  float h[AL][MO], v[AL][AL];
  wino_rows<typename F::GG, MO>(d, h);
  wino_cols<typename F::GG, AL>(h, v);
  const size_t plane = (size_t)g.Coutp * g.Pp;
  float* out = Yt + (size_t)k * g.Pp + p;
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) out[(xi * AL + nu) * plane] = v[xi][nu];
}

// The same with the planes of top_diff fetched whole into LDS (see mnv_wino_input_lds_kernel).
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_grad_lds_kernel(const float* __restrict__ top_diff,
                                                                float* __restrict__ Yt, WinoGeom g,
                                                                MnvFastDiv d_HW) {
  typedef WinoF<AL, R> F;
  constexpr int MO = AL - R + 1;
  extern __shared__ float planes[];
  const int p0 = blockIdx.x * 256, p = p0 + threadIdx.x;
  const int k = blockIdx.y;
  const int HW = g.Hd * g.Wd;
  const int img0 = mnv_fastdiv(p0, g.d_T);
  const int last = p0 + 255 < g.P ? p0 + 255 : g.P - 1;
  const int count = (last >= p0 && k < g.Cout ? mnv_fastdiv(last, g.d_T) - img0 + 1 : 0) * HW;
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pl = mnv_fastdiv(i, d_HW);
    planes[i] = top_diff[((size_t)(img0 + pl) * g.Cout + k) * HW + (i - pl * HW)];
  }
  __syncthreads();
  if (p >= g.Pp) return;
  float d[MO][MO];
#pragma unroll
  for (int a = 0; a < MO; ++a)
#pragma unroll
    for (int b = 0; b < MO; ++b) d[a][b] = 0.f;
  if (p < g.P && k < g.Cout) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const float* plane = planes + (img - img0) * HW;
#pragma unroll
    for (int a = 0; a < MO; ++a)
#pragma unroll
      for (int b = 0; b < MO; ++b) {
        const int y = MO * th + a, x = MO * tw + b;
        if (y < g.Hd && x < g.Wd) d[a][b] = plane[y * g.Wd + x];
      }
  }
  float h[AL][MO], v[AL][AL];
  wino_rows<typename F::GG, MO>(d, h);
  wino_cols<typename F::GG, AL>(h, v);
  const size_t plane = (size_t)g.Coutp * g.Pp;
  float* out = Yt + (size_t)k * g.Pp + p;
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) out[(xi * AL + nu) * plane] = v[xi][nu];
}

// filter_diff[k][c][R-1-r][R-1-s] = (A'^T Q A')[r][s] with the epilogues of the direct kernel's
// store: the parameter update sgd_w - sgd_scale * ., or the sum with what is there.
// (filter_diff may be sgd_w itself: a thread reads the R x R parameters it then writes.)
template <int AL, int R>
__global__ __launch_bounds__(256) void mnv_wino_grad_output_kernel(const float* __restrict__ Q,
                                                                   float* filter_diff, WinoGeom g,
                                                                   int accumulate, const float* sgd_w,
                                                                   float sgd_scale) {
  typedef WinoF<AL, R> F;
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.Cout * g.Cin) return;
  const int k = mnv_fastdiv(t, g.d_Cin), c = t - k * g.Cin;
  const size_t plane = (size_t)g.Coutp * g.Cin;
  const float* in = Q + (size_t)k * g.Cin + c;
  float q[AL][AL];
#pragma unroll
  for (int xi = 0; xi < AL; ++xi)
#pragma unroll
    for (int nu = 0; nu < AL; ++nu) q[xi][nu] = in[(xi * AL + nu) * plane];
  float h[R][AL], dg[R][R];
  wino_rows<typename F::AAT, AL>(q, h);
  wino_cols<typename F::AAT, R>(h, dg);
  float* out = filter_diff + (size_t)t * (R * R);
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int s = 0; s < R; ++s) {
      const int at = (R - 1 - r) * R + (R - 1 - s);
      float x = dg[r][s];
      if (sgd_w) x = sgd_w[(size_t)t * (R * R) + at] - sgd_scale * x;
      else if (accumulate) x = out[at] + x;
      out[at] = x;
    }
}

// The products of the filter gradient as one: C{Cin, points Coutp} = A{Cin, Pp} B{Pp, points Coutp},
// both operands with the reduction index p contiguous; the A of a column tile is the V panel
// of the tile's transform point.
struct WinoGradGemm {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  static constexpr int A_NOFF = 1, B_NOFF = 1;
  const float* __restrict__ V;
  const float* __restrict__ Yt;
  float* __restrict__ Q;
  int M, N, K, total_slabs, spp;  // Cin, points * Coutp, Pp
  int coutp, accumulate;
  struct Res {
    mnv_rsrc a, b;
  };
  struct AState {};
  struct BState {};
  __device__ void make_res(Res& r) const {
    r.a = mnv_make_rsrc(V, (unsigned)M * (unsigned)K * 4u);
    r.b = mnv_make_rsrc(Yt, (unsigned)N * (unsigned)K * 4u);
  }
  __device__ void block_init(Res& r, float*, int, int n0) const {
    r.a = mnv_make_rsrc(V + (size_t)(n0 / coutp) * M * K, (unsigned)M * (unsigned)K * 4u);
  }
  __device__ void a_init(const Res&, AState&, int) const {}
  __device__ void b_init(const Res&, BState&, int) const {}
  __device__ void a_period(const AState&, unsigned (&off)[1], int m, int kl, int period) const {
    const int k = period * spp * 16 + kl;  // K is a multiple of 4: a vector is whole or absent
    off[0] = ((m < M) & (k < K)) ? ((unsigned)m * (unsigned)K + (unsigned)k) * 4u : MNV_OOB;
  }
  __device__ void a_load(const Res& r, const AState&, const unsigned (&off)[1], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<1>(r.a, off, (unsigned)s * 64u, v);
  }
  __device__ void b_period(const BState&, unsigned (&off)[1], int n, int kl, int period) const {
    const int k = period * spp * 16 + kl;
    off[0] = ((n < N) & (k < K)) ? ((unsigned)n * (unsigned)K + (unsigned)k) * 4u : MNV_OOB;
  }
  __device__ void b_load(const Res& r, const BState&, const unsigned (&off)[1], int, int s, int,
                         float (&v)[4]) const {
    mnv_fetch_vec<1>(r.b, off, (unsigned)s * 64u, v);
  }
  size_t extra_lds_bytes() const { return 0; }
  __device__ void c_store(int m, int n, float x) const {
    const size_t at = (size_t)n * M + m;
    Q[at] = accumulate ? Q[at] + x : x;
  }
};

typedef MnvGemmTile<128, 128, 16, 2, 2> TileBig;

// Measurement aid (mnv_conv_winograd_profile): while it is on, every launch of the products
// is bracketed by an event pair on its stream, so that a benchmark can time the MFMA kernel of
// a pass apart from the transform kernels around it.
struct ProductProfile {
  struct Rec {
    hipEvent_t begin, end;
    double flops;
    int kind;  // 0: forward / data gradient, 1: filter gradient (with the reduction of its shares)
  };
  std::mutex mu;
  bool on = false;
  std::vector<Rec> recs;
  void drop() {
    for (auto& r : recs) {
      (void)hipEventDestroy(r.begin);
      (void)hipEventDestroy(r.end);
    }
    recs.clear();
  }
};
ProductProfile g_profile;

// the event pair of one launch, or false when the profile is off
bool profile_begin(hipEvent_t* begin, hipEvent_t* end, hipStream_t s) {
  std::lock_guard<std::mutex> lock(g_profile.mu);
  if (!g_profile.on) return false;
  if (hipEventCreate(begin) != hipSuccess) return false;
  if (hipEventCreate(end) != hipSuccess) {
    (void)hipEventDestroy(*begin);
    return false;
  }
  (void)hipEventRecord(*begin, s);
  return true;
}
void profile_end(hipEvent_t begin, hipEvent_t end, hipStream_t s, int kind, double flops) {
  (void)hipEventRecord(end, s);
  std::lock_guard<std::mutex> lock(g_profile.mu);
  g_profile.recs.push_back({begin, end, flops, kind});
}

inline size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

// Mode of mnv_conv_winograd_mode: 0 never, 1 where it pays, 2 wherever it applies, 3 / 4 / 5 as 2
// with the tile size pinned to 2 x 2 / 4 x 4 / 5 x 5 outputs.
std::atomic<int> g_mode{1};

// Points per dimension for an Hd x Wd output plane under r x r filters.  3 x 3: 4, 6 or 7 (2 x 2,
// 4 x 4 or 5 x 5 outputs per tile): a larger tile is taken when it needs at most 85% of the
// products of the best smaller one; its results are a few times further from the direct sum,
// so a near tie goes to the smaller tile.  5 x 5: 8 (4 x 4 outputs per tile) or not at all.
int pick_points(int Hd, int Wd, int R, int mode) {
  if (R == 5) return mode == 3 ? 0 : 8;
  if (mode == 3) return 4;
  if (mode == 4) return 6;
  if (mode == 5) return 7;
  long long best = 16LL * ((Hd + 1) / 2) * ((Wd + 1) / 2);
  int al = 4;
  const long long six = 36LL * ((Hd + 3) / 4) * ((Wd + 3) / 4);
  if (six * 100 <= best * 85) {
    best = six;
    al = 6;
  }
  const long long seven = 49LL * ((Hd + 4) / 5) * ((Wd + 4) / 5);
  if (seven * 100 <= best * 85) al = 7;
  return al;
}

int make_wino_geom(WinoGeom* g, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w,
                   int al, int r) {
  // (channel counts are grid extents of the transform kernels)
  if (N <= 0 || Cin <= 0 || Cout <= 0 || Cin > 65535 || Cout > 65535 - 127 || Hs <= 0 || Ws <= 0 ||
      pad_h < 0 || pad_w < 0 || pad_h > r - 1 || pad_w > r - 1 || Hs + 2 * pad_h < r || Ws + 2 * pad_w < r ||
      !((r == 3 && (al == 4 || al == 6 || al == 7)) || (r == 5 && al == 8)))
    return MNV_ERR_INVALID;
  g->N = N; g->Cin = Cin; g->Cout = Cout; g->Coutp = (Cout + 127) / 128 * 128;
  g->Hs = Hs; g->Ws = Ws; g->Hd = Hs + 2 * pad_h - (r - 1); g->Wd = Ws + 2 * pad_w - (r - 1);
  g->pad_h = pad_h; g->pad_w = pad_w;
  g->al = al; g->r = r; g->m = al - r + 1;
  g->TH = (g->Hd + g->m - 1) / g->m; g->TW = (g->Wd + g->m - 1) / g->m;
  const long long P = (long long)N * g->TH * g->TW;
  if (P > (1LL << 28)) return MNV_ERR_INVALID;
  g->P = (int)P; g->Pp = (int)((P + 3) / 4 * 4);
  // a V panel and U are read through 32-bit byte offsets
  if ((long long)Cin * g->Pp > (1LL << 29) - 1 || (long long)al * al * g->Coutp * Cin > (1LL << 29) - 1)
    return MNV_ERR_INVALID;
  g->d_T = mnv_fastdiv_make(g->TH * g->TW);
  g->d_TW = mnv_fastdiv_make(g->TW);
  g->d_Cin = mnv_fastdiv_make(Cin);
  return MNV_OK;
}

// V of the group of images that `g` describes
template <int AL, int R>
int launch_input_transform(const float* src, float* V, const WinoGeom& g, hipStream_t s) {
  const int T = g.TH * g.TW, HW = g.Hs * g.Ws;
  // planes a workgroup's 256 consecutive tiles can touch
  const size_t lds = (size_t)(255 / T + 2) * HW * sizeof(float);
  if (lds <= 48 * 1024)
    hipLaunchKernelGGL((mnv_wino_input_lds_kernel<AL, R>), dim3((g.Pp + 255) / 256, g.Cin), dim3(256), lds,
                       s, src, V, g, mnv_fastdiv_make(HW));
  else
    hipLaunchKernelGGL((mnv_wino_input_kernel<AL, R>), dim3((g.Pp + 255) / 256, g.Cin), dim3(256), 0, s, src,
                       V, g);
  return MNV_LAUNCH_STATUS();
}

size_t u_bytes(const WinoGeom& g) {
  return align256((size_t)g.al * g.al * g.Coutp * g.Cin * sizeof(float));
}
// V and M of `images` images
size_t vm_bytes(const WinoGeom& g, int images) {
  const size_t pp = ((size_t)images * g.TH * g.TW + 3) / 4 * 4, points = (size_t)g.al * g.al;
  return align256(points * pp * g.Cin * sizeof(float)) + align256(points * pp * g.Coutp * sizeof(float));
}
// partial tiles of the filter gradient's equal-shares launch: at most four workgroups per CU,
// a partial tile each and one more per output tile
size_t grad_sk_bytes(const WinoGeom& g) {
  const long long tiles = (long long)((g.Cin + 127) / 128) * (g.al * g.al * g.Coutp / 128);
  return (size_t)(4 * mnv_cu_count() + tiles) * 128 * 128 * sizeof(float);
}

// the largest group of images whose transformed tensors fit `avail` bytes, then groups of
// equal size; 0 when not even one image fits
int images_that_fit(const WinoGeom& g, int N, size_t avail) {
  if (avail < vm_bytes(g, 1)) return 0;
  if (avail >= vm_bytes(g, N)) return N;
  int lo = 1, hi = N;
  while (lo < hi) {
    const int mid = (lo + hi + 1) / 2;
    if (vm_bytes(g, mid) <= avail) lo = mid;
    else hi = mid - 1;
  }
  const int groups = (N + lo - 1) / lo;
  return (N + groups - 1) / groups;
}

// the geometry of a pass under the current mode; false: the pass does not run this way
bool plan_geom(WinoGeom* g, int* mode_out, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w,
               int R, int S, int sv, int sh) {
  const int mode = g_mode.load(std::memory_order_relaxed);
  *mode_out = mode;
  if (mode == 0 || R != S || (R != 3 && R != 5) || sv != 1 || sh != 1 || pad_h < 0 || pad_w < 0 ||
      pad_h > R - 1 || pad_w > R - 1 || Hs + 2 * pad_h < R || Ws + 2 * pad_w < R)
    return false;
  const int al = pick_points(Hs + 2 * pad_h - (R - 1), Ws + 2 * pad_w - (R - 1), R, mode);
  return al && make_wino_geom(g, N, Cin, Cout, Hs, Ws, pad_h, pad_w, al, R) == MNV_OK;
}

// Mode 1: the path is taken where a cost estimate puts it at 80% of the direct kernel's time
// or less, and the direct kernel's estimate is at least 100 us (four or five launches instead
// of one).  Per output pixel and image, with pts = transformed values per output (al^2 / m^2,
// times the waste of rounding the plane up to whole tiles):
//   direct   2 r^2 Cin Cout flops at 130 TFLOP/s (what the direct kernels sustain);
//   filtered pts (Cin + Coutp) values written and read once, 8 bytes each way, at 5 TB/s (the
//            transform kernels), plus 2 pts Cin' Coutp flops at the rate this core reaches on
//            the products: 157 TFLOP/s x k / (k + 64 slab-equivalents of prologue and store),
//            k = Cin for forward / data gradient, 0.85 for the filter gradient's long k
//            (Cin' = Cin rounded up to the 128-row tile there).
// Checked against the batch-256 layers: 96 -> 256 channels under 5 x 5 filters 0.46 estimated,
// 0.43 measured; 256 -> 384 under 3 x 3 on 13 x 13 planes 0.65 / 0.63.  Layers of 128 channels
// and fewer stay direct: the transforms alone cost what the multiplies save.
bool pays(const WinoGeom& g, int images, bool filter_gradient) {
  const double px = (double)g.Hd * g.Wd;
  const double pts = (double)g.al * g.al * g.TH * g.TW / px;
  const double direct = 2.0 * g.r * g.r * g.Cin * g.Cout / 130e12;
  const double rate = filter_gradient ? 0.85 : (double)g.Cin / (g.Cin + 64.0);
  const double rows = filter_gradient ? (g.Cin + 127) / 128 * 128 : g.Cin;
  const double filtered = pts * (g.Cin + g.Coutp) * 8.0 / 5e12 + 2.0 * pts * rows * g.Coutp / (rate * 157.3e12);
  return filtered <= 0.8 * direct && direct * px * images >= 100e-6;
}

template <int AL, int R>
int wino_conv(const WinoGeom& g0, const float* src, const float* filter, const float* bias,
              const float* gate, float* dst, int N, int transposed, int relu, int images,
              void* workspace, hipStream_t s) {
  WinoGeom g = g0;
  const int Cin = g.Cin, Cout = g.Cout;
  char* w = static_cast<char*>(workspace);
  float* U = reinterpret_cast<float*>(w);
  w += u_bytes(g);
  float* V = reinterpret_cast<float*>(w);
  w += align256((size_t)AL * AL * g.Pp * Cin * sizeof(float));
  float* Mx = reinterpret_cast<float*>(w);
  const int K = transposed ? Cin : Cout, C = transposed ? Cout : Cin;
  hipLaunchKernelGGL((mnv_wino_filter_kernel<AL, R>), dim3((g.Coutp * Cin + 255) / 256), dim3(256), 0, s,
                     filter, U, g, K, C, transposed != 0);
  int rc = MNV_LAUNCH_STATUS();
  if (rc) return rc;
  const size_t per_src = (size_t)Cin * g.Hs * g.Ws, per_dst = (size_t)Cout * g.Hd * g.Wd;
  for (int n0 = 0; n0 < N; n0 += images) {
    const int nn = N - n0 < images ? N - n0 : images;
    if (nn != g.N && (rc = make_wino_geom(&g, nn, Cin, Cout, g.Hs, g.Ws, g.pad_h, g.pad_w, AL, R))) return rc;
    if ((rc = launch_input_transform<AL, R>(src + n0 * per_src, V, g, s))) return rc;
    WinoGemm p{V, U, Mx, g.Pp, AL * AL * g.Coutp, Cin, Cin / 16, Cin / 16, g.Coutp, g.Coutp / 128};
    hipEvent_t e0, e1;
    const bool timed = profile_begin(&e0, &e1, s);
    rc = mnv_gemm_launch<TileBig>(p, 1, nullptr, s);
    if (timed) profile_end(e0, e1, s, 0, 2.0 * AL * AL * Cout * Cin * g.P);
    if (rc) return rc;
    const size_t lds = (size_t)(255 / (g.TH * g.TW) + 2) * g.Hd * g.Wd * sizeof(float);
    if (lds <= 48 * 1024)
      hipLaunchKernelGGL((mnv_wino_output_lds_kernel<AL, R>), dim3((g.P + 255) / 256, Cout), dim3(256), lds, s,
                         Mx, bias, gate ? gate + n0 * per_dst : nullptr, dst + n0 * per_dst, g, relu,
                         mnv_fastdiv_make(g.Hd * g.Wd), mnv_fastdiv_make(g.Wd));
    else
      hipLaunchKernelGGL((mnv_wino_output_kernel<AL, R>), dim3((g.P + 255) / 256, Cout), dim3(256), 0, s, Mx,
                         bias, gate ? gate + n0 * per_dst : nullptr, dst + n0 * per_dst, g, relu);
    if ((rc = MNV_LAUNCH_STATUS())) return rc;
  }
  return MNV_OK;
}

// Slabs the filter-gradient products' loads run ahead (see mnv_gemm_kernel): two; the kernel
// still holds four workgroups per CU (conv2 / conv4 at batch 256: 387 -> 377 us on average).
#ifndef MNV_WINO_SK_PF
#define MNV_WINO_SK_PF 2
#endif
// (the forward / data-gradient products gain nothing from it: 388 / 474 / 435 against 388 / 474 /
// 426 us.)
template <int AL, int R>
int wino_filter_grad(const WinoGeom& g0, const float* bottom, const float* top_diff, float* filter_diff,
                     int N, int images, int accumulate, const float* sgd_w, float sgd_scale,
                     void* workspace, hipStream_t s, int* plan) {
  WinoGeom g = g0;
  const int C = g.Cin, K = g.Cout;
  const size_t sk_bytes = grad_sk_bytes(g);
  char* w = static_cast<char*>(workspace);
  float* Q = reinterpret_cast<float*>(w);
  w += u_bytes(g);
  float* V = reinterpret_cast<float*>(w);
  w += align256((size_t)AL * AL * g.Pp * C * sizeof(float));
  float* Yt = reinterpret_cast<float*>(w);
  w += align256((size_t)AL * AL * g.Pp * g.Coutp * sizeof(float));
  if (plan) {
    WinoGradGemm p{V, Yt, Q, C, AL * AL * g.Coutp, g.Pp, (g.Pp + 15) / 16, g.Pp >= 16 ? g.Pp / 16 : 1,
                   g.Coutp, 0};
    bool done = false;
    plan[0] = 128;
    plan[1] = 1;
    plan[2] = 0;
    return mnv_gemm_streamk_launch<TileBig, MNV_WINO_SK_PF>(p, w, sk_bytes, s, &done, plan + 2);
  }
  int rc;
  const size_t per_bottom = (size_t)C * g.Hs * g.Ws, per_top = (size_t)K * g.Hd * g.Wd;
  for (int n0 = 0; n0 < N; n0 += images) {
    const int nn = N - n0 < images ? N - n0 : images;
    if (nn != g.N && (rc = make_wino_geom(&g, nn, C, K, g.Hs, g.Ws, g.pad_h, g.pad_w, AL, R))) return rc;
    if ((rc = launch_input_transform<AL, R>(bottom + n0 * per_bottom, V, g, s))) return rc;
    const size_t lds = (size_t)(255 / (g.TH * g.TW) + 2) * g.Hd * g.Wd * sizeof(float);
    if (lds <= 48 * 1024)
      hipLaunchKernelGGL((mnv_wino_grad_lds_kernel<AL, R>), dim3((g.Pp + 255) / 256, g.Coutp), dim3(256), lds, s,
                         top_diff + n0 * per_top, Yt, g, mnv_fastdiv_make(g.Hd * g.Wd));
    else
      hipLaunchKernelGGL((mnv_wino_grad_kernel<AL, R>), dim3((g.Pp + 255) / 256, g.Coutp), dim3(256), 0, s,
                         top_diff + n0 * per_top, Yt, g);
    if ((rc = MNV_LAUNCH_STATUS())) return rc;
    WinoGradGemm p{V, Yt, Q, C, AL * AL * g.Coutp, g.Pp, (g.Pp + 15) / 16, g.Pp >= 16 ? g.Pp / 16 : 1,
                   g.Coutp, n0 > 0};
    bool done = false;
    hipEvent_t e0, e1;
    const bool timed = profile_begin(&e0, &e1, s);
    rc = mnv_gemm_streamk_launch<TileBig, MNV_WINO_SK_PF>(p, w, sk_bytes, s, &done);
    if (!rc && !done) rc = mnv_gemm_launch<TileBig>(p, 1, nullptr, s);
    if (timed) profile_end(e0, e1, s, 1, 2.0 * AL * AL * K * C * g.P);
    if (rc) return rc;
  }
  hipLaunchKernelGGL((mnv_wino_grad_output_kernel<AL, R>), dim3((K * C + 255) / 256), dim3(256), 0, s, Q,
                     filter_diff, g, accumulate, sgd_w, sgd_scale);
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" int mnv_conv_winograd_mode(int mode) {
  if (mode < 0 || mode > 5) return g_mode.load(std::memory_order_relaxed);
  return g_mode.exchange(mode, std::memory_order_relaxed);
}

extern "C" int mnv_conv_winograd_profile(int enable) {
  std::lock_guard<std::mutex> lock(g_profile.mu);
  if (enable) g_profile.drop();
  g_profile.on = enable != 0;
  return MNV_OK;
}

extern "C" int mnv_conv_winograd_profile_read(int kind, int* launches, double* milliseconds,
                                              double* gflop) {
  std::lock_guard<std::mutex> lock(g_profile.mu);
  int n = 0;
  double ms = 0, fl = 0;
  for (auto& r : g_profile.recs) {
    if (r.kind != kind) continue;
    MNV_HIP_TRY(hipEventSynchronize(r.end));
    float t = 0;
    MNV_HIP_TRY(hipEventElapsedTime(&t, r.begin, r.end));
    ++n;
    ms += t;
    fl += r.flops;
  }
  if (launches) *launches = n;
  if (milliseconds) *milliseconds = ms;
  if (gflop) *gflop = fl / 1e9;
  return MNV_OK;
}

size_t mnv_wino_workspace_bytes(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R) {
  WinoGeom g;
  int mode;
  if (!plan_geom(&g, &mode, N, Cin, Cout, Hs, Ws, pad_h, pad_w, R, R, 1, 1)) return 0;
  return u_bytes(g) + vm_bytes(g, N);
}

int mnv_wino_images(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R, int S,
                    int sv, int sh, size_t workspace_bytes) {
  WinoGeom g;
  int mode;
  if (Cin % 16 != 0 || !plan_geom(&g, &mode, N, Cin, Cout, Hs, Ws, pad_h, pad_w, R, S, sv, sh)) return 0;
  if (workspace_bytes < u_bytes(g)) return 0;
  const int images = images_that_fit(g, N, workspace_bytes - u_bytes(g));
  if (mode != 1 || images == 0) return images;
  return pays(g, images, false) ? images : 0;
}

int mnv_wino_conv(const float* src, const float* filter, const float* bias, const float* gate,
                  float* dst, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R,
                  int transposed, int relu, int images, void* workspace, size_t workspace_bytes,
                  hipStream_t s) {
  WinoGeom g;
  int mode;
  if (!src || !filter || !dst || images <= 0 || Cin % 16 != 0) return MNV_ERR_INVALID;
  if (images > N) images = N;
  if (!plan_geom(&g, &mode, images, Cin, Cout, Hs, Ws, pad_h, pad_w, R, R, 1, 1)) return MNV_ERR_INVALID;
  if (!workspace || workspace_bytes < u_bytes(g) + vm_bytes(g, images)) return MNV_ERR_INVALID;
  if (g.al == 8)
    return wino_conv<8, 5>(g, src, filter, bias, gate, dst, N, transposed, relu, images, workspace, s);
  if (g.al == 7)
    return wino_conv<7, 3>(g, src, filter, bias, gate, dst, N, transposed, relu, images, workspace, s);
  return g.al == 6 ? wino_conv<6, 3>(g, src, filter, bias, gate, dst, N, transposed, relu, images, workspace, s)
                   : wino_conv<4, 3>(g, src, filter, bias, gate, dst, N, transposed, relu, images, workspace, s);
}

size_t mnv_wino_grad_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw, int R) {
  WinoGeom g;
  int mode;
  if (!plan_geom(&g, &mode, N, C, K, H, W, ph, pw, R, R, 1, 1)) return 0;
  return u_bytes(g) + vm_bytes(g, N) + grad_sk_bytes(g);
}

int mnv_wino_grad_images(int N, int C, int K, int H, int W, int ph, int pw, int R, int S, int sv,
                         int sh, size_t workspace_bytes) {
  WinoGeom g;
  int mode;
  if (!plan_geom(&g, &mode, N, C, K, H, W, ph, pw, R, S, sv, sh)) return 0;
  if (workspace_bytes < u_bytes(g) + grad_sk_bytes(g)) return 0;
  int images = images_that_fit(g, N, workspace_bytes - u_bytes(g) - grad_sk_bytes(g));
  // Yt of a group is read through 32-bit byte offsets
  const long long per_image = (long long)g.TH * g.TW;
  const long long most = ((1LL << 29) - 1) / ((long long)g.al * g.al * g.Coutp) / per_image;
  if (images > most) images = (int)most;
  if (mode != 1 || images == 0) return images;
  return pays(g, images, true) ? images : 0;
}

int mnv_wino_filter_grad(const float* bottom, const float* top_diff, float* filter_diff, int N, int C,
                         int K, int H, int W, int ph, int pw, int R, int images, int accumulate,
                         const float* sgd_w, float sgd_scale, void* workspace,
                         size_t workspace_bytes, hipStream_t s, int* plan) {
  WinoGeom g;
  int mode;
  if (images <= 0) return MNV_ERR_INVALID;
  if (images > N) images = N;
  if (!plan_geom(&g, &mode, images, C, K, H, W, ph, pw, R, R, 1, 1)) return MNV_ERR_INVALID;
  if (!workspace || workspace_bytes < u_bytes(g) + vm_bytes(g, images) + grad_sk_bytes(g))
    return MNV_ERR_INVALID;
  if (!plan && (!bottom || !top_diff || !filter_diff)) return MNV_ERR_INVALID;
  if (g.al == 8)
    return wino_filter_grad<8, 5>(g, bottom, top_diff, filter_diff, N, images, accumulate, sgd_w, sgd_scale,
                                  workspace, s, plan);
  if (g.al == 7)
    return wino_filter_grad<7, 3>(g, bottom, top_diff, filter_diff, N, images, accumulate, sgd_w, sgd_scale,
                                  workspace, s, plan);
  return g.al == 6 ? wino_filter_grad<6, 3>(g, bottom, top_diff, filter_diff, N, images, accumulate, sgd_w,
                                            sgd_scale, workspace, s, plan)
                   : wino_filter_grad<4, 3>(g, bottom, top_diff, filter_diff, N, images, accumulate, sgd_w,
                                            sgd_scale, workspace, s, plan);
}
