// Max / average pooling, forward and backward, on an image batch {W,H,C,N}
// (cuDNN v2 modes selected at reference minerva/op/impl/cuda/cuda_perform.cu:489-615;
// output extent rule minerva/narray/convolution.cpp:107-114).
// Roofline: HBM bandwidth; forward moves 4*(in + out) bytes, backward
// 4*(top_diff + bottom + bottom_diff).
//
// Window o covers rows [o*stride - pad, o*stride - pad + window) clipped to the
// tensor.  max: padding never wins.  average: divisor is the full window area.
// max backward sends each top_diff to the first maximum of its window in (row, column)
// scan order; a position that wins several overlapping windows adds their gradients in
// ascending window order, which is the order a sequential scatter would use, so the
// result is bit-identical to it and no atomics are needed.
//
// Main path: a workgroup stages whole (n,c) planes in LDS with contiguous 16-byte loads,
// finds every window's arg-max once from LDS, then walks the plane's positions and
// gathers the gradients of the (at most ceil(k/s)^2) windows each one can win.  HBM sees
// every tensor exactly once.  Planes too large for LDS take the direct kernels below.
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_POOL_THREADS 256
#define MNV_POOL_LDS_FLOATS 8192  // plane data staged per workgroup (32 KiB)

struct PoolGeom {
  int H, W, Ho, Wo, sv, sh, kh, kw, ph, pw;
  MnvFastDiv d_hw, d_howo, d_W, d_Wo, d_sv, d_sh;  // run-time integer division is ~40 instructions
};

__device__ __forceinline__ int ceil_div_pos(int a, int b) {  // b > 0, any a
  return a >= 0 ? (a + b - 1) / b : -((-a) / b);
}

// a / stride for a >= 0; ST = 1 or 2 when both strides are that constant, 0 otherwise
template <int ST>
__device__ __forceinline__ int div_stride(int a, const MnvFastDiv& d) {
  return ST == 1 ? a : ST == 2 ? (a >> 1) : mnv_fastdiv(a, d);
}

// Loads `count` floats starting at src (any alignment) into LDS.
__device__ __forceinline__ void stage(const float* __restrict__ src, float* dst, int count) {
  // align the global side to 16 bytes, then copy vectors
  int head = (int)(((16 - (reinterpret_cast<uintptr_t>(src) & 15)) & 15) >> 2);
  if (head > count) head = count;
  for (int i = threadIdx.x; i < head; i += MNV_POOL_THREADS) dst[i] = src[i];
  const int n4 = (count - head) >> 2;
  const mnv_f4* s4 = reinterpret_cast<const mnv_f4*>(src + head);
  for (int i = threadIdx.x; i < n4; i += MNV_POOL_THREADS) {
    mnv_f4 v = s4[i];
    float* d = dst + head + 4 * i;
    d[0] = v.x; d[1] = v.y; d[2] = v.z; d[3] = v.w;
  }
  for (int i = head + 4 * n4 + threadIdx.x; i < count; i += MNV_POOL_THREADS) dst[i] = src[i];
}

// ---- LDS-staged kernels: `ppb` planes per workgroup --------------------------------
template <bool MAX>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_fwd_lds_kernel(
    const float* __restrict__ bottom, float* __restrict__ top, int planes, int ppb, PoolGeom g) {
  extern __shared__ float lds[];
  const int hw = g.H * g.W, howo = g.Ho * g.Wo;
  for (int p0 = blockIdx.x * ppb; p0 < planes; p0 += gridDim.x * ppb) {
    const int np = min(ppb, planes - p0);
    __syncthreads();
    stage(bottom + (size_t)p0 * hw, lds, np * hw);
    __syncthreads();
    for (int q = threadIdx.x; q < np * howo; q += MNV_POOL_THREADS) {
      int pl = mnv_fastdiv(q, g.d_howo), o = q - pl * howo;
      int i = mnv_fastdiv(o, g.d_Wo), j = o - i * g.Wo;
      int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
      int ys = max(y0, 0), xs = max(x0, 0);
      int ye = min(y0 + g.kh, g.H), xe = min(x0 + g.kw, g.W);
      const float* b = lds + pl * hw;
      float r;
      if (MAX) {
        r = -INFINITY;
        for (int y = ys; y < ye; ++y)
          for (int x = xs; x < xe; ++x) {
            float v = b[y * g.W + x];
            if (r < v) r = v;
          }
      } else {
        float s = 0.f;
        for (int y = ys; y < ye; ++y)
          for (int x = xs; x < xe; ++x) s += b[y * g.W + x];
        r = s / (float)(g.kh * g.kw);
      }
      top[(size_t)p0 * howo + q] = r;
    }
  }
}

// LDS: [ppb*hw] plane data, then [ppb*howo] top_diff, then [ppb*howo] arg-max positions.
template <bool MAX, int ST>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_bwd_lds_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, int planes, int ppb, PoolGeom g) {
  extern __shared__ float lds[];
  const int hw = g.H * g.W, howo = g.Ho * g.Wo;
  float* sx = lds;
  float* sd = lds + ppb * hw;
  int* sarg = reinterpret_cast<int*>(sd + ppb * howo);
  for (int p0 = blockIdx.x * ppb; p0 < planes; p0 += gridDim.x * ppb) {
    const int np = min(ppb, planes - p0);
    __syncthreads();
    if (MAX) stage(bottom + (size_t)p0 * hw, sx, np * hw);
    stage(top_diff + (size_t)p0 * howo, sd, np * howo);
    __syncthreads();
    if (MAX) {
      // first maximum of every window in scan order (strict '<'), as a flat position
      for (int q = threadIdx.x; q < np * howo; q += MNV_POOL_THREADS) {
        int pl = mnv_fastdiv(q, g.d_howo), o = q - pl * howo;
        int i = mnv_fastdiv(o, g.d_Wo), j = o - i * g.Wo;
        int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
        int ys = max(y0, 0), xs = max(x0, 0);
        int ye = min(y0 + g.kh, g.H), xe = min(x0 + g.kw, g.W);
        const float* b = sx + pl * hw;
        float mx = -INFINITY;
        int arg = ys * g.W + xs;
        for (int y = ys; y < ye; ++y)
          for (int x = xs; x < xe; ++x) {
            float v = b[y * g.W + x];
            if (mx < v) {
              mx = v;
              arg = y * g.W + x;
            }
          }
        sarg[q] = arg;
      }
      __syncthreads();
    }
    for (int q = threadIdx.x; q < np * hw; q += MNV_POOL_THREADS) {
      int pl = mnv_fastdiv(q, g.d_hw), pos = q - pl * hw;
      int y = mnv_fastdiv(pos, g.d_W), x = pos - y * g.W;
      // windows i with i*sv - ph <= y < i*sv - ph + kh, clipped to [0, Ho)
      int ay = y + g.ph - g.kh + g.sv, ax = x + g.pw - g.kw + g.sh;  // ceil((y+ph-kh+1)/sv)
      int i_lo = ay > 0 ? div_stride<ST>(ay, g.d_sv) : 0;
      int i_hi = min(div_stride<ST>(y + g.ph, g.d_sv), g.Ho - 1);
      int j_lo = ax > 0 ? div_stride<ST>(ax, g.d_sh) : 0;
      int j_hi = min(div_stride<ST>(x + g.pw, g.d_sh), g.Wo - 1);
      float acc = 0.f;
      for (int i = i_lo; i <= i_hi; ++i)
        for (int j = j_lo; j <= j_hi; ++j) {
          int o = pl * howo + i * g.Wo + j;
          if (MAX) {
            if (sarg[o] == pos) acc += sd[o];
          } else {
            acc += sd[o] / (float)(g.kh * g.kw);
          }
        }
      bottom_diff[(size_t)p0 * hw + q] = acc;
    }
  }
}

// ---- direct kernels for planes that do not fit in LDS -------------------------------
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
    for (int i = i_lo; i <= i_hi; ++i)
      for (int j = j_lo; j <= j_hi; ++j) {
        if (MAX) {
          int y0 = i * g.sv - g.ph, x0 = j * g.sh - g.pw;
          int ys = max(y0, 0), xs = max(x0, 0);
          int ye = min(y0 + g.kh, g.H), xe = min(x0 + g.kw, g.W);
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
  if ((long long)h * w > 0x7fffffffLL || (long long)n * c > 0x7fffffffLL) return MNV_ERR_INVALID;
  g->H = h; g->W = w; g->sv = sv; g->sh = sh; g->kh = kh; g->kw = kw; g->ph = ph; g->pw = pw;
  g->Ho = mnv_pooled_size(h, kh, sv, ph);
  g->Wo = mnv_pooled_size(w, kw, sh, pw);
  if (g->Ho <= 0 || g->Wo <= 0) return MNV_ERR_INVALID;
  g->d_hw = mnv_fastdiv_make(h * w);
  g->d_howo = mnv_fastdiv_make(g->Ho * g->Wo);
  g->d_W = mnv_fastdiv_make(w);
  g->d_Wo = mnv_fastdiv_make(g->Wo);
  g->d_sv = mnv_fastdiv_make(sv);
  g->d_sh = mnv_fastdiv_make(sh);
  return MNV_OK;
}

unsigned pool_grid(size_t total) {
  size_t blocks = mnv_ceil_div(total, MNV_POOL_THREADS);
  if (blocks > 4 * MNV_MAX_STREAM_BLOCKS) blocks = 4 * MNV_MAX_STREAM_BLOCKS;
  return (unsigned)blocks;
}

// Planes per workgroup for the LDS path: as many as fit the staging area, but no more
// than leaves every CU several workgroups.  0 = plane too large, use the direct kernels.
int planes_per_block(const PoolGeom& g, long long planes, bool bwd) {
  long long per_plane = (long long)g.H * g.W + (bwd ? 2LL * g.Ho * g.Wo : 0);
  if (per_plane > MNV_POOL_LDS_FLOATS) return 0;
  long long ppb = MNV_POOL_LDS_FLOATS / per_plane;
  long long cap = planes / 2048;  // keep at least ~2048 workgroups
  if (cap < 1) cap = 1;
  if (ppb > cap) ppb = cap;
  if (ppb > 64) ppb = 64;
  return (int)ppb;
}

template <bool MAX>
int pool_fwd(const float* bottom, float* top, int n, int c, int h, int w, int sv, int sh, int kh,
             int kw, int ph, int pw, mnv_stream_t stream) {
  PoolGeom g;
  if (!bottom || !top) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  long long planes = (long long)n * c;
  int ppb = planes_per_block(g, planes, false);
  if (ppb > 0) {
    size_t lds = (size_t)ppb * h * w * sizeof(float);
    long long blocks = (planes + ppb - 1) / ppb;
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL((mnv_pool_fwd_lds_kernel<MAX>), dim3((unsigned)blocks),
                       dim3(MNV_POOL_THREADS), lds, mnv_stream(stream), bottom, top, (int)planes,
                       ppb, g);
  } else {
    hipLaunchKernelGGL((mnv_pool_fwd_kernel<MAX>), dim3(pool_grid((size_t)planes * g.Ho * g.Wo)),
                       dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top, (size_t)planes,
                       g);
  }
  return MNV_LAUNCH_STATUS();
}

template <bool MAX>
int pool_bwd(const float* bottom, const float* top_diff, float* bottom_diff, int n, int c, int h,
             int w, int sv, int sh, int kh, int kw, int ph, int pw, mnv_stream_t stream) {
  PoolGeom g;
  if (!bottom || !top_diff || !bottom_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  long long planes = (long long)n * c;
  int ppb = planes_per_block(g, planes, true);
  if (ppb > 0) {
    size_t lds = (size_t)ppb * ((size_t)h * w + 2 * (size_t)g.Ho * g.Wo) * sizeof(float);
    long long blocks = (planes + ppb - 1) / ppb;
    if (blocks > 65536) blocks = 65536;
    const int st = (sv == sh && (sv == 1 || sv == 2)) ? sv : 0;
    auto kernel = st == 1   ? mnv_pool_bwd_lds_kernel<MAX, 1>
                  : st == 2 ? mnv_pool_bwd_lds_kernel<MAX, 2>
                            : mnv_pool_bwd_lds_kernel<MAX, 0>;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(MNV_POOL_THREADS), lds,
                       mnv_stream(stream), bottom, top_diff, bottom_diff, (int)planes, ppb, g);
  } else {
    hipLaunchKernelGGL((mnv_pool_bwd_kernel<MAX>), dim3(pool_grid((size_t)planes * h * w)),
                       dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top_diff,
                       bottom_diff, (size_t)planes, g);
  }
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
