// Max / average pooling, forward and backward, on an image batch {W,H,C,N}
// (cuDNN v2 modes selected at reference minerva/op/impl/cuda/cuda_perform.cu:489-615;
// output extent rule minerva/narray/convolution.cpp:107-114).
// Roofline: HBM bandwidth; forward moves 4*(in + out) bytes, backward
// 4*(top_diff + bottom + bottom_diff) (the overlapping window re-reads hit in cache).
//
// Window o covers rows [o*stride - pad, o*stride - pad + window) clipped to the
// tensor.  max: padding never wins.  average: divisor is the full window area.
// max backward is a gather: every bottom position revisits the (few) windows that
// contain it, recomputes each window's first maximum in (row, column) scan order and
// adds that window's gradient if the maximum is itself; windows are visited in
// ascending order so overlapping contributions add up in the same order as a
// sequential scatter, and no atomics are needed.
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_POOL_THREADS 256

struct PoolGeom {
  int H, W, Ho, Wo, sv, sh, kh, kw, ph, pw;
};

template <bool MAX>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_fwd_kernel(
    const float* __restrict__ bottom, float* __restrict__ top, size_t planes, PoolGeom g) {
  const size_t per_plane = (size_t)g.Ho * g.Wo;
  const size_t total = planes * per_plane;
  for (size_t q = (size_t)blockIdx.x * MNV_POOL_THREADS + threadIdx.x; q < total;
       q += (size_t)gridDim.x * MNV_POOL_THREADS) {
    size_t plane = q / per_plane;
    int o = (int)(q - plane * per_plane);
    int i = o / g.Wo, j = o - i * g.Wo;
    int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
    int ys = max(y0, 0), xs = max(x0, 0);
    int ye = min(y0 + g.kh, g.H), xe = min(x0 + g.kw, g.W);
    const float* b = bottom + plane * (size_t)g.H * g.W;
    if (MAX) {
      float mx = -INFINITY;
      for (int y = ys; y < ye; ++y)
        for (int x = xs; x < xe; ++x) {
          float v = b[y * g.W + x];
          if (mx < v) mx = v;
        }
      top[q] = mx;
    } else {
      float s = 0.f;
      for (int y = ys; y < ye; ++y)
        for (int x = xs; x < xe; ++x) s += b[y * g.W + x];
      top[q] = s / (float)(g.kh * g.kw);
    }
  }
}

__device__ __forceinline__ int ceil_div_pos(int a, int b) {  // b > 0, any a
  return a >= 0 ? (a + b - 1) / b : -((-a) / b);
}

template <bool MAX>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_bwd_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, size_t planes, PoolGeom g) {
  const size_t per_plane = (size_t)g.H * g.W;
  const size_t total = planes * per_plane;
  for (size_t q = (size_t)blockIdx.x * MNV_POOL_THREADS + threadIdx.x; q < total;
       q += (size_t)gridDim.x * MNV_POOL_THREADS) {
    size_t plane = q / per_plane;
    int pos = (int)(q - plane * per_plane);
    int y = pos / g.W, x = pos - y * g.W;
    // windows i with i*sv - ph <= y < i*sv - ph + kh
    int i_lo = max(ceil_div_pos(y + g.ph - g.kh + 1, g.sv), 0);
    int i_hi = min((y + g.ph) / g.sv, g.Ho - 1);
    int j_lo = max(ceil_div_pos(x + g.pw - g.kw + 1, g.sh), 0);
    int j_hi = min((x + g.pw) / g.sh, g.Wo - 1);
    const float* b = bottom + plane * per_plane;
    const float* dt = top_diff + plane * (size_t)g.Ho * g.Wo;
    float acc = 0.f;
    const float mine = MAX ? b[pos] : 0.f;
    for (int i = i_lo; i <= i_hi; ++i)
      for (int j = j_lo; j <= j_hi; ++j) {
        if (MAX) {
          int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
          int ys = max(y0, 0), xs = max(x0, 0);
          int ye = min(y0 + g.kh, g.H), xe = min(x0 + g.kw, g.W);
          // first maximum in scan order (strict '<'), as a flat position
          float mx = -INFINITY;
          int arg = ys * g.W + xs;
          for (int yy = ys; yy < ye; ++yy)
            for (int xx = xs; xx < xe; ++xx) {
              float v = b[yy * g.W + xx];
              if (mx < v) {
                mx = v;
                arg = yy * g.W + xx;
              }
            }
          (void)mine;
          if (arg == pos) acc += dt[i * g.Wo + j];
        } else {
          acc += dt[i * g.Wo + j] / (float)(g.kh * g.kw);
        }
      }
    bottom_diff[q] = acc;
  }
}

int make_geom(PoolGeom* g, int n, int c, int h, int w, int sv, int sh, int kh, int kw, int ph,
              int pw) {
  if (n <= 0 || c <= 0 || h <= 0 || w <= 0 || sv <= 0 || sh <= 0 || kh <= 0 || kw <= 0 ||
      ph < 0 || pw < 0)
    return MNV_ERR_INVALID;
  if ((long long)h * w > 0x7fffffffLL) return MNV_ERR_INVALID;
  g->H = h; g->W = w; g->sv = sv; g->sh = sh; g->kh = kh; g->kw = kw; g->ph = ph; g->pw = pw;
  g->Ho = mnv_pooled_size(h, kh, sv, ph);
  g->Wo = mnv_pooled_size(w, kw, sh, pw);
  if (g->Ho <= 0 || g->Wo <= 0) return MNV_ERR_INVALID;
  return MNV_OK;
}

unsigned pool_grid(size_t total) {
  size_t blocks = mnv_ceil_div(total, MNV_POOL_THREADS);
  if (blocks > 4 * MNV_MAX_STREAM_BLOCKS) blocks = 4 * MNV_MAX_STREAM_BLOCKS;
  return (unsigned)blocks;
}

template <bool MAX>
int pool_fwd(const float* bottom, float* top, int n, int c, int h, int w, int sv, int sh, int kh,
             int kw, int ph, int pw, mnv_stream_t stream) {
  PoolGeom g;
  if (!bottom || !top) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  size_t planes = (size_t)n * c;
  hipLaunchKernelGGL((mnv_pool_fwd_kernel<MAX>), dim3(pool_grid(planes * g.Ho * g.Wo)),
                     dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top, planes, g);
  return MNV_LAUNCH_STATUS();
}

template <bool MAX>
int pool_bwd(const float* bottom, const float* top_diff, float* bottom_diff, int n, int c, int h,
             int w, int sv, int sh, int kh, int kw, int ph, int pw, mnv_stream_t stream) {
  PoolGeom g;
  if (!bottom || !top_diff || !bottom_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  size_t planes = (size_t)n * c;
  hipLaunchKernelGGL((mnv_pool_bwd_kernel<MAX>), dim3(pool_grid(planes * h * w)),
                     dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top_diff, bottom_diff,
                     planes, g);
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" {

int mnv_pooled_size(int in, int window, int stride, int pad) {
  if (stride <= 0) return 0;
  int p = (in + 2 * pad - window + stride - 1) / stride + 1;
  if (0 <= (p - 1) * stride - in - pad) --p;
  return p;
}

int mnv_maxpool_fwd(const float* bottom, float* top, int n, int c, int h, int w, int sv, int sh,
                    int kh, int kw, int ph, int pw, mnv_stream_t s) {
  return pool_fwd<true>(bottom, top, n, c, h, w, sv, sh, kh, kw, ph, pw, s);
}
int mnv_avgpool_fwd(const float* bottom, float* top, int n, int c, int h, int w, int sv, int sh,
                    int kh, int kw, int ph, int pw, mnv_stream_t s) {
  return pool_fwd<false>(bottom, top, n, c, h, w, sv, sh, kh, kw, ph, pw, s);
}
int mnv_maxpool_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, int n, int c, int h, int w, int sv, int sh, int kh,
                    int kw, int ph, int pw, mnv_stream_t s) {
  (void)top;  // the first-maximum rule is evaluated on bottom itself
  return pool_bwd<true>(bottom, top_diff, bottom_diff, n, c, h, w, sv, sh, kh, kw, ph, pw, s);
}
int mnv_avgpool_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, int n, int c, int h, int w, int sv, int sh, int kh,
                    int kw, int ph, int pw, mnv_stream_t s) {
  (void)top;
  if (!bottom) return MNV_ERR_INVALID;
  return pool_bwd<false>(bottom, top_diff, bottom_diff, n, c, h, w, sv, sh, kh, kw, ph, pw, s);
}

}  // extern "C"
