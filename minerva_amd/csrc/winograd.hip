// 3 x 3, unit-stride convolutions by the minimal-filtering algorithm F(2 x 2, 3 x 3)
// (Winograd): every 2 x 2 block of outputs of one channel pair costs 16 multiplies instead
// of 36.  The work becomes 16 independent matrix products, one per point (xi, nu) of the
// transformed 4 x 4 tile,
//     M[xi,nu][co][p] = sum_ci U[xi,nu][co][ci] * V[xi,nu][ci][p],      p = (image, tile row, tile col)
// with U = G g G^T (filters), V = B^T d B (4 x 4 input tiles, stride 2) and the outputs
// Y = A^T M A.  The 16 products run as ONE launch of the fp32 MFMA core (gemm_core.h): the
// transform point is folded into the column index, n = point * Coutp + co, and a workgroup
// picks the V panel of its point once, in block_init.  Semantics are those of conv.hip: the
// forward pass correlates with the flipped filter (cuDNN's CUDNN_CONVOLUTION as selected at
// minerva/op/impl/cuda/cuda_perform.cu:227-264), the data gradient (cuda_perform.cu:266-291)
// is the same correlation of top_diff with the unflipped filter, channels exchanged, under a
// padding of 2 - pad.
//
//   B^T = | 1  0 -1  0 |   G = | 1    0    0  |   A^T = | 1  1  1  0 |
//         | 0  1  1  0 |       | 1/2  1/2  1/2|         | 0  1 -1 -1 |
//         | 0 -1  1  0 |       | 1/2 -1/2  1/2|
//         | 0  1  0 -1 |       | 0    0    1  |
//
// Rounding: the transforms add and halve, the products are summed in fp32 over Cin; the
// result differs from the direct sum by a few 1e-7 of the output's norm.
// Roofline: the matrix products are MFMA-bound (2 * 16 * Cout * Cin * tiles flops, 4 / 9 of
// the direct flops when the output extents are even); the three transform kernels stream
// 16 * 4 bytes per (channel, tile) and are HBM-bound.

#include "gemm_core.h"
#include "winograd.h"

namespace {

// Channels per workgroup of the LDS-staged input transform.  Four channels per workgroup (the
// tile arithmetic done once for four) measured no faster than one: 84.7 against 79.6 us for
// 384 channels of 256 x 13 x 13.
#define WINO_CH 1

struct WinoGeom {
  int N, Cin, Cout, Coutp;  // Coutp: Cout rounded up to the tile width of the product
  int Hs, Ws, Hd, Wd;       // source and destination planes
  int pad_h, pad_w;         // of the correlation: d[a][b] = src[2 th - pad_h + a][2 tw - pad_w + b]
  int TH, TW, P, Pp;        // tiles per plane, tiles in all, P rounded up to 4
  MnvFastDiv d_T, d_TW, d_Cin;
};

// U[point][co][ci] from filter[k][c][3][3].  Forward: co = k, ci = c, g[r][s] = f[2-r][2-s];
// data gradient (`transposed`): co = c, ci = k, g = f.  Rows co >= Cout are zero.
__global__ __launch_bounds__(256) void mnv_wino_filter_kernel(const float* __restrict__ filter,
                                                              float* __restrict__ U, WinoGeom g,
                                                              int K, int C, bool transposed) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.Coutp * g.Cin) return;
  const int co = mnv_fastdiv(t, g.d_Cin), ci = t - co * g.Cin;
  float f[3][3];
  if (co < g.Cout) {
    const float* src = transposed ? filter + ((size_t)ci * C + co) * 9 : filter + ((size_t)co * C + ci) * 9;
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int s = 0; s < 3; ++s) f[r][s] = transposed ? src[r * 3 + s] : src[(2 - r) * 3 + (2 - s)];
  } else {
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int s = 0; s < 3; ++s) f[r][s] = 0.f;
  }
  float h[4][3];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    h[0][s] = f[0][s];
    h[1][s] = 0.5f * (f[0][s] + f[1][s] + f[2][s]);
    h[2][s] = 0.5f * (f[0][s] - f[1][s] + f[2][s]);
    h[3][s] = f[2][s];
  }
  const size_t plane = (size_t)g.Coutp * g.Cin;
  float* out = U + (size_t)co * g.Cin + ci;
#pragma unroll
  for (int xi = 0; xi < 4; ++xi) {
    out[(xi * 4 + 0) * plane] = h[xi][0];
    out[(xi * 4 + 1) * plane] = 0.5f * (h[xi][0] + h[xi][1] + h[xi][2]);
    out[(xi * 4 + 2) * plane] = 0.5f * (h[xi][0] - h[xi][1] + h[xi][2]);
    out[(xi * 4 + 3) * plane] = h[xi][2];
  }
}

// V[point][ci][p] = (B^T d B)[point] of the 4 x 4 tile p of channel ci; p >= P writes zeros.
__global__ __launch_bounds__(256) void mnv_wino_input_kernel(const float* __restrict__ src,
                                                             float* __restrict__ V, WinoGeom g) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int ci = blockIdx.y;
  if (p >= g.Pp) return;
  float d[4][4];
  if (p < g.P) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const int y0 = 2 * th - g.pad_h, x0 = 2 * tw - g.pad_w;
    const float* plane = src + ((size_t)img * g.Cin + ci) * (g.Hs * g.Ws);
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int y = y0 + a, x = x0 + b;
        d[a][b] = ((unsigned)y < (unsigned)g.Hs && (unsigned)x < (unsigned)g.Ws) ? plane[y * g.Ws + x] : 0.f;
      }
  } else {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) d[a][b] = 0.f;
  }
  float h[4][4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    h[0][b] = d[0][b] - d[2][b];
    h[1][b] = d[1][b] + d[2][b];
    h[2][b] = d[2][b] - d[1][b];
    h[3][b] = d[1][b] - d[3][b];
  }
  const size_t plane = (size_t)g.Cin * g.Pp;
  float* out = V + (size_t)ci * g.Pp + p;
#pragma unroll
  for (int xi = 0; xi < 4; ++xi) {
    out[(xi * 4 + 0) * plane] = h[xi][0] - h[xi][2];
    out[(xi * 4 + 1) * plane] = h[xi][1] + h[xi][2];
    out[(xi * 4 + 2) * plane] = h[xi][2] - h[xi][1];
    out[(xi * 4 + 3) * plane] = h[xi][1] - h[xi][3];
  }
}

// The same through LDS, for planes small enough that the planes of the images a workgroup's
// 256 tiles belong to fit there: they are fetched whole, in runs of contiguous floats (a
// plane of 13 x 13 is 676 contiguous bytes), where the kernel above gathers 16 values per
// thread at a stride of 8 bytes between neighbouring tiles.
__global__ __launch_bounds__(256) void mnv_wino_input_lds_kernel(const float* __restrict__ src,
                                                                 float* __restrict__ V, WinoGeom g,
                                                                 MnvFastDiv d_HW) {
  extern __shared__ float planes[];
  const int p0 = blockIdx.x * 256, p = p0 + threadIdx.x;
  const int c0 = blockIdx.y * WINO_CH;
  const int nch = g.Cin - c0 < WINO_CH ? g.Cin - c0 : WINO_CH;
  const int HW = g.Hs * g.Ws;
  const int img0 = mnv_fastdiv(p0, g.d_T);
  const int last = p0 + 255 < g.P ? p0 + 255 : g.P - 1;
  const int count = (last >= p0 ? mnv_fastdiv(last, g.d_T) - img0 + 1 : 0) * HW;  // per channel
  for (int i = threadIdx.x; i < count; i += 256) {
    const int pl = mnv_fastdiv(i, d_HW);
    const float* at = src + ((size_t)(img0 + pl) * g.Cin + c0) * HW + (i - pl * HW);
#pragma unroll
    for (int cc = 0; cc < WINO_CH; ++cc)
      if (cc < nch) planes[cc * count + i] = at[(size_t)cc * HW];
  }
  __syncthreads();
  if (p >= g.Pp) return;
  int at[4][4];  // LDS index of every tile element of this thread's tile, -1: reads as zero
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) at[a][b] = -1;
  if (p < g.P) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const int y0 = 2 * th - g.pad_h, x0 = 2 * tw - g.pad_w;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int y = y0 + a, x = x0 + b;
        if ((unsigned)y < (unsigned)g.Hs && (unsigned)x < (unsigned)g.Ws)
          at[a][b] = (img - img0) * HW + y * g.Ws + x;
      }
  }
  const size_t plane = (size_t)g.Cin * g.Pp;
  for (int cc = 0; cc < nch; ++cc) {
    const float* pl = planes + cc * count;
    float h[4][4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      float d[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) d[a] = at[a][b] >= 0 ? pl[at[a][b]] : 0.f;
      h[0][b] = d[0] - d[2];
      h[1][b] = d[1] + d[2];
      h[2][b] = d[2] - d[1];
      h[3][b] = d[1] - d[3];
    }
    float* out = V + (size_t)(c0 + cc) * g.Pp + p;
#pragma unroll
    for (int xi = 0; xi < 4; ++xi) {
      out[(xi * 4 + 0) * plane] = h[xi][0] - h[xi][2];
      out[(xi * 4 + 1) * plane] = h[xi][1] + h[xi][2];
      out[(xi * 4 + 2) * plane] = h[xi][2] - h[xi][1];
      out[(xi * 4 + 3) * plane] = h[xi][1] - h[xi][3];
    }
  }
}

// dst[img][co][2 th + a][2 tw + b] = (A^T M A)[a][b] (+ bias[co]) (then max(., 0)) (then kept
// only where gate > 0): the epilogues of the direct kernels, each the single operation of the
// separate operator.
__global__ __launch_bounds__(256) void mnv_wino_output_kernel(const float* __restrict__ Mx,
                                                              const float* __restrict__ bias,
                                                              const float* __restrict__ gate,
                                                              float* __restrict__ dst, WinoGeom g,
                                                              int relu) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int co = blockIdx.y;
  if (p >= g.P) return;
  const size_t plane = (size_t)g.Coutp * g.Pp;
  const float* in = Mx + (size_t)co * g.Pp + p;
  float m[4][4];
#pragma unroll
  for (int xi = 0; xi < 4; ++xi)
#pragma unroll
    for (int nu = 0; nu < 4; ++nu) m[xi][nu] = in[(xi * 4 + nu) * plane];
  float h[2][4];
#pragma unroll
  for (int nu = 0; nu < 4; ++nu) {
    h[0][nu] = m[0][nu] + m[1][nu] + m[2][nu];
    h[1][nu] = m[1][nu] - m[2][nu] - m[3][nu];
  }
  float y[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    y[a][0] = h[a][0] + h[a][1] + h[a][2];
    y[a][1] = h[a][1] - h[a][2] - h[a][3];
  }
  const int img = mnv_fastdiv(p, g.d_T);
  const int t = p - img * (g.TH * g.TW);
  const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
  const float b = bias ? bias[co] : 0.f;
  const size_t base = ((size_t)img * g.Cout + co) * (g.Hd * g.Wd);
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int yy = 2 * th + a, xx = 2 * tw + c;
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

// The 16 products as one: C{Pp, 16 Coutp} = A{Pp, Cin} B{Cin, 16 Coutp}, column-major, where the
// A of a column tile is the V panel of the tile's transform point.
struct WinoGemm {
  static constexpr bool A_KFAST = false, B_KFAST = true;
  static constexpr int A_NOFF = 1, B_NOFF = 1;
  const float* __restrict__ V;
  const float* __restrict__ U;
  float* __restrict__ Mx;
  int M, N, K, total_slabs, spp;  // Pp, 16 Coutp, Cin
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

// ---- filter gradient: F(3 x 3, 2 x 2), the same four points
//   dg[k][c] = sum_p A'^T [ (G' dy_p G'^T) (.) (B^T d_p B) ] A'      dy_p: the 2 x 2 tile p of top_diff
//   A'^T = | 1  1  1  0 |   G' = | 1    0  |
//          | 0  1 -1  0 |        | 1/2  1/2|
//          | 0  1  1 -1 |        | 1/2 -1/2|
//                                | 0    1  |
// The sum over the tiles is the k dimension of the 16 products Q[point][k][c] =
// sum_p Yt[point][k][p] V[point][c][p].

// Yt[point][k][p] = (G' dy G'^T)[point] of the 2 x 2 tile p of channel k of top_diff; zeros
// for p >= P and for the rows k >= Cout.
__global__ __launch_bounds__(256) void mnv_wino_grad_kernel(const float* __restrict__ top_diff,
                                                            float* __restrict__ Yt, WinoGeom g) {
  const int p = blockIdx.x * 256 + threadIdx.x;
  const int k = blockIdx.y;
  if (p >= g.Pp) return;
  float d[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
  if (p < g.P && k < g.Cout) {
    const int img = mnv_fastdiv(p, g.d_T);
    const int t = p - img * (g.TH * g.TW);
    const int th = mnv_fastdiv(t, g.d_TW), tw = t - th * g.TW;
    const float* plane = top_diff + ((size_t)img * g.Cout + k) * (g.Hd * g.Wd);
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int y = 2 * th + a, x = 2 * tw + b;
        if (y < g.Hd && x < g.Wd) d[a][b] = plane[y * g.Wd + x];
      }
  }
  float h[4][2];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    h[0][b] = d[0][b];
    h[1][b] = 0.5f * (d[0][b] + d[1][b]);
    h[2][b] = 0.5f * (d[0][b] - d[1][b]);
    h[3][b] = d[1][b];
  }
  const size_t plane = (size_t)g.Coutp * g.Pp;
  float* out = Yt + (size_t)k * g.Pp + p;
#pragma unroll
  for (int xi = 0; xi < 4; ++xi) {
    out[(xi * 4 + 0) * plane] = h[xi][0];
    out[(xi * 4 + 1) * plane] = 0.5f * (h[xi][0] + h[xi][1]);
    out[(xi * 4 + 2) * plane] = 0.5f * (h[xi][0] - h[xi][1]);
    out[(xi * 4 + 3) * plane] = h[xi][1];
  }
}

// filter_diff[k][c][2-r][2-s] = (A'^T Q A')[r][s] with the epilogues of the direct kernel's
// store: the parameter update sgd_w - sgd_scale * ., or the sum with what is there.
// (filter_diff may be sgd_w itself: a thread reads the nine parameters it then writes.)
__global__ __launch_bounds__(256) void mnv_wino_grad_output_kernel(const float* __restrict__ Q,
                                                                   float* filter_diff, WinoGeom g,
                                                                   int accumulate, const float* sgd_w,
                                                                   float sgd_scale) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= g.Cout * g.Cin) return;
  const int k = mnv_fastdiv(t, g.d_Cin), c = t - k * g.Cin;
  const size_t plane = (size_t)g.Coutp * g.Cin;
  const float* in = Q + (size_t)k * g.Cin + c;
  float q[4][4];
#pragma unroll
  for (int xi = 0; xi < 4; ++xi)
#pragma unroll
    for (int nu = 0; nu < 4; ++nu) q[xi][nu] = in[(xi * 4 + nu) * plane];
  float h[3][4];
#pragma unroll
  for (int nu = 0; nu < 4; ++nu) {
    h[0][nu] = q[0][nu] + q[1][nu] + q[2][nu];
    h[1][nu] = q[1][nu] - q[2][nu];
    h[2][nu] = q[1][nu] + q[2][nu] - q[3][nu];
  }
  float* out = filter_diff + (size_t)t * 9;
#pragma unroll
  for (int r = 0; r < 3; ++r) {
    const float dg[3] = {h[r][0] + h[r][1] + h[r][2], h[r][1] - h[r][2], h[r][1] + h[r][2] - h[r][3]};
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      const int at = (2 - r) * 3 + (2 - s);
      float x = dg[s];
      if (sgd_w) x = sgd_w[(size_t)t * 9 + at] - sgd_scale * x;
      else if (accumulate) x = out[at] + x;
      out[at] = x;
    }
  }
}

// The 16 products of the filter gradient as one: C{Cin, 16 Coutp} = A{Cin, Pp} B{Pp, 16 Coutp},
// both operands with the reduction index p contiguous; the A of a column tile is the V panel
// of the tile's transform point.
struct WinoGradGemm {
  static constexpr bool A_KFAST = true, B_KFAST = true;
  static constexpr int A_NOFF = 1, B_NOFF = 1;
  const float* __restrict__ V;
  const float* __restrict__ Yt;
  float* __restrict__ Q;
  int M, N, K, total_slabs, spp;  // Cin, 16 Coutp, Pp
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

inline size_t align256(size_t b) { return (b + 255) & ~(size_t)255; }

int make_wino_geom(WinoGeom* g, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w) {
  if (N <= 0 || Cin <= 0 || Cout <= 0 || Hs <= 0 || Ws <= 0 || pad_h < 0 || pad_w < 0 || pad_h > 2 ||
      pad_w > 2 || Hs + 2 * pad_h < 3 || Ws + 2 * pad_w < 3)
    return MNV_ERR_INVALID;
  g->N = N; g->Cin = Cin; g->Cout = Cout; g->Coutp = (Cout + 127) / 128 * 128;
  g->Hs = Hs; g->Ws = Ws; g->Hd = Hs + 2 * pad_h - 2; g->Wd = Ws + 2 * pad_w - 2;
  g->pad_h = pad_h; g->pad_w = pad_w;
  g->TH = (g->Hd + 1) / 2; g->TW = (g->Wd + 1) / 2;
  const long long P = (long long)N * g->TH * g->TW;
  if (P > (1LL << 28)) return MNV_ERR_INVALID;
  g->P = (int)P; g->Pp = (int)((P + 3) / 4 * 4);
  // a V panel and U are read through 32-bit byte offsets
  if ((long long)Cin * g->Pp > (1LL << 29) - 1 || 16LL * g->Coutp * Cin > (1LL << 29) - 1)
    return MNV_ERR_INVALID;
  g->d_T = mnv_fastdiv_make(g->TH * g->TW);
  g->d_TW = mnv_fastdiv_make(g->TW);
  g->d_Cin = mnv_fastdiv_make(Cin);
  return MNV_OK;
}

// V of the group of images that `g` describes
int launch_input_transform(const float* src, float* V, const WinoGeom& g, hipStream_t s) {
  const int T = g.TH * g.TW, HW = g.Hs * g.Ws;
  // planes a workgroup's 256 consecutive tiles can touch
  const size_t lds = (size_t)WINO_CH * (255 / T + 2) * HW * sizeof(float);
  if (lds <= 32 * 1024)
    hipLaunchKernelGGL(mnv_wino_input_lds_kernel, dim3((g.Pp + 255) / 256, (g.Cin + WINO_CH - 1) / WINO_CH),
                       dim3(256), lds, s, src, V, g, mnv_fastdiv_make(HW));
  else
    hipLaunchKernelGGL(mnv_wino_input_kernel, dim3((g.Pp + 255) / 256, g.Cin), dim3(256), 0, s, src, V, g);
  return MNV_LAUNCH_STATUS();
}

size_t u_bytes(const WinoGeom& g) { return align256((size_t)16 * g.Coutp * g.Cin * sizeof(float)); }
// V and M of `images` images
size_t vm_bytes(const WinoGeom& g, int images) {
  const size_t pp = ((size_t)images * g.TH * g.TW + 3) / 4 * 4;
  return align256(16 * pp * g.Cin * sizeof(float)) + align256(16 * pp * g.Coutp * sizeof(float));
}

// partial tiles of the filter gradient's equal-shares launch: at most four workgroups per CU,
// a partial tile each and one more per output tile
size_t grad_sk_bytes(const WinoGeom& g) {
  const long long tiles = (long long)((g.Cin + 127) / 128) * (16 * g.Coutp / 128);
  return (size_t)(4 * mnv_cu_count() + tiles) * 128 * 128 * sizeof(float);
}

std::atomic<int> g_mode{1};

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

}  // namespace

extern "C" int mnv_conv_winograd_mode(int mode) {
  if (mode < 0 || mode > 2) return g_mode.load(std::memory_order_relaxed);
  return g_mode.exchange(mode, std::memory_order_relaxed);
}

size_t mnv_wino_workspace_bytes(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w) {
  WinoGeom g;
  if (make_wino_geom(&g, N, Cin, Cout, Hs, Ws, pad_h, pad_w)) return 0;
  return u_bytes(g) + vm_bytes(g, N);
}

int mnv_wino_images(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R, int S,
                    int sv, int sh, size_t workspace_bytes) {
  const int mode = g_mode.load(std::memory_order_relaxed);
  WinoGeom g;
  if (mode == 0 || R != 3 || S != 3 || sv != 1 || sh != 1 || Cin % 16 != 0 ||
      make_wino_geom(&g, N, Cin, Cout, Hs, Ws, pad_h, pad_w))
    return 0;
  if (workspace_bytes < u_bytes(g)) return 0;
  const int images = images_that_fit(g, N, workspace_bytes - u_bytes(g));
  if (mode == 2 || images == 0) return images;
  const long long tiles = (long long)images * g.TH * g.TW;
  const bool pays = Cin >= 32 && Cout * 4 >= g.Coutp * 3 && tiles >= 1024 &&
                    4LL * g.TH * g.TW * 5 <= 7LL * g.Hd * g.Wd;
  return pays ? images : 0;
}

int mnv_wino_conv(const float* src, const float* filter, const float* bias, const float* gate,
                  float* dst, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w,
                  int transposed, int relu, int images, void* workspace, size_t workspace_bytes,
                  hipStream_t s) {
  WinoGeom g;
  if (!src || !filter || !dst || images <= 0 || Cin % 16 != 0) return MNV_ERR_INVALID;
  if (images > N) images = N;
  int rc = make_wino_geom(&g, images, Cin, Cout, Hs, Ws, pad_h, pad_w);
  if (rc) return rc;
  if (!workspace || workspace_bytes < u_bytes(g) + vm_bytes(g, images)) return MNV_ERR_INVALID;
  char* w = static_cast<char*>(workspace);
  float* U = reinterpret_cast<float*>(w);
  w += u_bytes(g);
  float* V = reinterpret_cast<float*>(w);
  w += align256((size_t)16 * g.Pp * Cin * sizeof(float));
  float* Mx = reinterpret_cast<float*>(w);
  const int K = transposed ? Cin : Cout, C = transposed ? Cout : Cin;
  hipLaunchKernelGGL(mnv_wino_filter_kernel, dim3((g.Coutp * Cin + 255) / 256), dim3(256), 0, s,
                     filter, U, g, K, C, transposed != 0);
  if ((rc = MNV_LAUNCH_STATUS())) return rc;
  const size_t per_src = (size_t)Cin * Hs * Ws, per_dst = (size_t)Cout * g.Hd * g.Wd;
  for (int n0 = 0; n0 < N; n0 += images) {
    const int nn = N - n0 < images ? N - n0 : images;
    if (nn != g.N && (rc = make_wino_geom(&g, nn, Cin, Cout, Hs, Ws, pad_h, pad_w))) return rc;
    if ((rc = launch_input_transform(src + n0 * per_src, V, g, s))) return rc;
    WinoGemm p{V, U, Mx, g.Pp, 16 * g.Coutp, Cin, Cin / 16, Cin / 16, g.Coutp, g.Coutp / 128};
    if ((rc = mnv_gemm_launch<TileBig>(p, 1, nullptr, s))) return rc;
    hipLaunchKernelGGL(mnv_wino_output_kernel, dim3((g.P + 255) / 256, Cout), dim3(256), 0, s, Mx,
                       bias, gate ? gate + n0 * per_dst : nullptr, dst + n0 * per_dst, g, relu);
    if ((rc = MNV_LAUNCH_STATUS())) return rc;
  }
  return MNV_OK;
}

size_t mnv_wino_grad_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw) {
  WinoGeom g;
  if (make_wino_geom(&g, N, C, K, H, W, ph, pw)) return 0;
  return u_bytes(g) + vm_bytes(g, N) + grad_sk_bytes(g);
}

int mnv_wino_grad_images(int N, int C, int K, int H, int W, int ph, int pw, int R, int S, int sv,
                         int sh, size_t workspace_bytes) {
  const int mode = g_mode.load(std::memory_order_relaxed);
  WinoGeom g;
  if (mode == 0 || R != 3 || S != 3 || sv != 1 || sh != 1 || make_wino_geom(&g, N, C, K, H, W, ph, pw))
    return 0;
  if (workspace_bytes < u_bytes(g) + grad_sk_bytes(g)) return 0;
  int images = images_that_fit(g, N, workspace_bytes - u_bytes(g) - grad_sk_bytes(g));
  // Yt of a group is read through 32-bit byte offsets
  const long long per_image = (long long)g.TH * g.TW;
  const long long most = ((1LL << 29) - 1) / (16LL * g.Coutp) / per_image;
  if (images > most) images = (int)most;
  if (mode == 2 || images == 0) return images;
  const long long tiles = (long long)images * per_image;
  const bool pays = C >= 32 && C * 4 >= (C + 127) / 128 * 128 * 3 && K * 4 >= g.Coutp * 3 &&
                    tiles >= 1024 && 4LL * g.TH * g.TW * 5 <= 7LL * g.Hd * g.Wd;
  return pays ? images : 0;
}

#ifndef MNV_WINO_SK_PF
#define MNV_WINO_SK_PF 1
#endif
int mnv_wino_filter_grad(const float* bottom, const float* top_diff, float* filter_diff, int N, int C,
                         int K, int H, int W, int ph, int pw, int images, int accumulate,
                         const float* sgd_w, float sgd_scale, void* workspace,
                         size_t workspace_bytes, hipStream_t s, int* plan) {
  WinoGeom g;
  if (images <= 0) return MNV_ERR_INVALID;
  if (images > N) images = N;
  int rc = make_wino_geom(&g, images, C, K, H, W, ph, pw);
  if (rc) return rc;
  const size_t sk_bytes = grad_sk_bytes(g);
  if (!workspace || workspace_bytes < u_bytes(g) + vm_bytes(g, images) + sk_bytes) return MNV_ERR_INVALID;
  char* w = static_cast<char*>(workspace);
  float* Q = reinterpret_cast<float*>(w);
  w += u_bytes(g);
  float* V = reinterpret_cast<float*>(w);
  w += align256((size_t)16 * g.Pp * C * sizeof(float));
  float* Yt = reinterpret_cast<float*>(w);
  w += align256((size_t)16 * g.Pp * g.Coutp * sizeof(float));
  if (plan) {
    WinoGradGemm p{V, Yt, Q, C, 16 * g.Coutp, g.Pp, (g.Pp + 15) / 16, g.Pp >= 16 ? g.Pp / 16 : 1, g.Coutp, 0};
    bool done = false;
    plan[0] = 128;
    plan[1] = 1;
    plan[2] = 0;
    return mnv_gemm_streamk_launch<TileBig, MNV_WINO_SK_PF>(p, w, sk_bytes, s, &done, plan + 2);
  }
  if (!bottom || !top_diff || !filter_diff) return MNV_ERR_INVALID;
  const size_t per_bottom = (size_t)C * H * W, per_top = (size_t)K * g.Hd * g.Wd;
  for (int n0 = 0; n0 < N; n0 += images) {
    const int nn = N - n0 < images ? N - n0 : images;
    if (nn != g.N && (rc = make_wino_geom(&g, nn, C, K, H, W, ph, pw))) return rc;
    if ((rc = launch_input_transform(bottom + n0 * per_bottom, V, g, s))) return rc;
    hipLaunchKernelGGL(mnv_wino_grad_kernel, dim3((g.Pp + 255) / 256, g.Coutp), dim3(256), 0, s,
                       top_diff + n0 * per_top, Yt, g);
    if ((rc = MNV_LAUNCH_STATUS())) return rc;
    WinoGradGemm p{V, Yt, Q, C, 16 * g.Coutp, g.Pp, (g.Pp + 15) / 16, g.Pp >= 16 ? g.Pp / 16 : 1,
                   g.Coutp, n0 > 0};
    bool done = false;
    if ((rc = mnv_gemm_streamk_launch<TileBig, MNV_WINO_SK_PF>(p, w, sk_bytes, s, &done))) return rc;
    if (!done && (rc = mnv_gemm_launch<TileBig>(p, 1, nullptr, s))) return rc;
  }
  hipLaunchKernelGGL(mnv_wino_grad_output_kernel, dim3((K * C + 255) / 256), dim3(256), 0, s, Q,
                     filter_diff, g, accumulate, sgd_w, sgd_scale);
  return MNV_LAUNCH_STATUS();
}
