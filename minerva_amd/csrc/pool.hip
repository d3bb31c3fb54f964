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
// Main path: a workgroup stages groups of whole (n,c) planes in LDS with aligned 16-byte
// loads, finds every window's arg-max once from LDS, then walks the planes' positions and
// gathers the gradients of the (at most ceil(k/s)^2) windows each one can win.  HBM sees
// every tensor exactly once.  The workgroups are persistent and keep the next group's
// loads in flight (in registers) while they work on the current one; 3x3/2 and 2x2/2
// windows are unrolled at compile time.  Planes too large for LDS take the direct kernels.
#include <math.h>
#include <stdlib.h>

#include <algorithm>

#include "mnv_common.h"

namespace {

#ifndef MNV_POOL_THREADS
#define MNV_POOL_THREADS 256
#endif
#define MNV_POOL_XV 8  // 16-byte vectors of plane data a thread holds for the next group
#define MNV_POOL_DV 4  // ... of top_diff
#define MNV_POOL_X_FLOATS (MNV_POOL_THREADS * 4 * MNV_POOL_XV)
#define MNV_POOL_D_FLOATS (MNV_POOL_THREADS * 4 * MNV_POOL_DV)

struct PoolGeom {
  int H, W, Ho, Wo, sv, sh, kh, kw, ph, pw;
  MnvFastDiv d_hw, d_howo, d_W, d_Wo, d_sv, d_sh;  // run-time integer division is ~40 instructions
  // stride-2 backward: 2x2 blocks of padded coordinates (rows 2a, 2a+1) that meet the plane
  int a0, b0, NA, NB;
  MnvFastDiv d_nab, d_nb;
};

__device__ __forceinline__ int ceil_div_pos(int a, int b) {  // b > 0, any a
  return a >= 0 ? (a + b - 1) / b : -((-a) / b);
}

// Products of small indices (LDS offsets, plane coordinates: far below 2^23) on the
// full-rate 24-bit multiplier; the 32-bit integer multiply runs at a quarter of that.
__device__ __forceinline__ int m24(int a, int b) { return __mul24(a, b); }

// a / stride for a >= 0; ST = the compile-time stride, or 0 for a run-time one
template <int ST>
__device__ __forceinline__ int div_stride(int a, const MnvFastDiv& d) {
  return ST == 1 ? a : ST == 2 ? (a >> 1) : mnv_fastdiv(a, d);
}

// A run of `count` floats starting `first` floats into a 16-byte aligned tensor of `total`
// floats, moved HBM -> registers -> LDS in aligned 16-byte pieces.  The run is widened down
// to the previous 16-byte boundary (element e of the run lands at lds[(first & 3) + e]) and
// read through a buffer resource that ends with the tensor, so the last piece may hang over
// the end and reads zeros there.  issue() and commit() are separate so that the loads of
// the next group stay in flight while the current one is being worked on.
// NT: non-temporal loads, for tensors of 256 MB and more (5.65 -> 5.97 TB/s on the pool1
// forward pass with operands cycled so that none is cached).
template <int NV, bool NT>
struct PoolStage {
  mnv_f4 r[NV];
  int nvec;
  __device__ __forceinline__ void issue(const float* base, size_t total, size_t first, int count) {
    const size_t a0 = first & ~(size_t)3;
    nvec = (int)((first + count - a0 + 3) >> 2);
    size_t left = (total - a0) * sizeof(float);
    if (left > 0x7fffffffu) left = 0x7fffffffu;
    mnv_rsrc rs = mnv_make_rsrc(base + a0, (unsigned)left);
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int v = threadIdx.x + u * MNV_POOL_THREADS;
      if (v < nvec)
        r[u] = __builtin_bit_cast(mnv_f4, __builtin_amdgcn_raw_buffer_load_b128(rs, v * 16, 0, NT ? 2 : 0));
    }
  }
  __device__ __forceinline__ void commit(float* lds) const {
#pragma unroll
    for (int u = 0; u < NV; ++u) {
      const int v = threadIdx.x + u * MNV_POOL_THREADS;
      if (v < nvec) *reinterpret_cast<mnv_f4*>(lds + 4 * v) = r[u];
    }
  }
};

// Writes the `cnt` floats of a plane group from LDS to global memory.  In `lx` the group's
// first float sits at index `shift` = its global float index modulo 4, so LDS vector v is
// global vector v of the 16-byte aligned address just below the group.  Stores are 16 bytes,
// non-temporal, and lane t of a pass takes the vector whose absolute index is congruent
// to t modulo 8: every eight lanes then write one whole 128-byte line.  (A copy whose
// 16-byte stores start off a 64-byte boundary loses 12% of its rate on this part, at any
// offset that is not a multiple of 64 bytes; plane groups of odd planes start anywhere.)
// The first and the last vector may be shared with the neighbouring groups and are written
// float by float.
__device__ __forceinline__ void pool_write_group(const float* lx, float* group_dst, int shift, int cnt) {
  float* gout = group_dst - shift;
  const int lead = (int)((reinterpret_cast<uintptr_t>(gout) >> 4) & 7);
  const int nv = (shift + cnt + 3) >> 2;
  for (int v = (int)threadIdx.x - lead; v < nv; v += MNV_POOL_THREADS) {
    if (v < 0) continue;
    const int e0 = 4 * v - shift;  // position of the vector's first float in the group
    if (e0 >= 0 && e0 + 4 <= cnt) {
      __builtin_nontemporal_store(*reinterpret_cast<const mnv_f4*>(lx + 4 * v),
                                  reinterpret_cast<mnv_f4*>(gout) + v);
    } else {
      for (int k = 0; k < 4; ++k)
        if (e0 + k >= 0 && e0 + k < cnt) gout[4 * v + k] = lx[4 * v + k];
    }
  }
}

// Value (and position) of window (i, j) of the plane at b.  KS / ST are the compile-time
// square window and stride, or 0 for the run-time ones in g.  Maximum: strict '<' from
// -inf in scan order, so the first maximum wins and a NaN never does; `arg` starts at the
// first in-range position.  Average: scan-order sum over the in-range part / full area.
template <bool MAX, int KS, int ST>
__device__ __forceinline__ float pool_window(const float* b, const PoolGeom& g, int i, int j,
                                            int* arg) {
  const int sv = ST ? ST : g.sv, sh = ST ? ST : g.sh;
  const int kh = KS ? KS : g.kh, kw = KS ? KS : g.kw;
  const int y0 = i * sv - g.ph, x0 = j * sh - g.pw;
  float r = MAX ? -INFINITY : 0.f;
  int at = m24(max(y0, 0), g.W) + max(x0, 0);
  if (KS && y0 >= 0 && x0 >= 0 && y0 + KS <= g.H && x0 + KS <= g.W) {
    // window inside the plane (all of them when nothing is padded or clipped): no checks
    const int base = m24(y0, g.W) + x0;
#pragma unroll
    for (int dy = 0; dy < KS; ++dy)
#pragma unroll
      for (int dx = 0; dx < KS; ++dx) {
        const float v = b[base + dy * g.W + dx];
        if (MAX) {
          if (r < v) {
            r = v;
            at = base + dy * g.W + dx;
          }
        } else {
          r += v;
        }
      }
  } else if (KS) {
#pragma unroll
    for (int dy = 0; dy < KS; ++dy)
#pragma unroll
      for (int dx = 0; dx < KS; ++dx) {
        const int y = y0 + dy, x = x0 + dx;
        const bool ok = ((unsigned)y < (unsigned)g.H) & ((unsigned)x < (unsigned)g.W);
        const float v = ok ? b[y * g.W + x] : (MAX ? -INFINITY : 0.f);
        if (MAX) {
          if (r < v) {
            r = v;
            at = y * g.W + x;
          }
        } else {
          r += v;
        }
      }
  } else {
    const int ys = max(y0, 0), xs = max(x0, 0);
    const int ye = min(y0 + kh, g.H), xe = min(x0 + kw, g.W);
    for (int y = ys; y < ye; ++y)
      for (int x = xs; x < xe; ++x) {
        const float v = b[y * g.W + x];
        if (MAX) {
          if (r < v) {
            r = v;
            at = y * g.W + x;
          }
        } else {
          r += v;
        }
      }
  }
  if (arg) *arg = at;
  return MAX ? r : r / (float)(kh * kw);
}

// ---- LDS-staged kernels: groups of `ppb` planes per workgroup, software pipelined ------
template <bool MAX, int KS, int ST, bool NT>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_fwd_lds_kernel(
    const float* __restrict__ bottom, float* __restrict__ top, int planes, int ppb, PoolGeom g) {
  extern __shared__ float lds[];
  const int hw = g.H * g.W, howo = g.Ho * g.Wo;
  const size_t total = (size_t)planes * hw;
  const int groups = (planes + ppb - 1) / ppb;
  PoolStage<MNV_POOL_XV, NT> sx;
  int grp = blockIdx.x;
  if (grp < groups) {
    const int p0 = grp * ppb;
    sx.issue(bottom, total, (size_t)p0 * hw, min(ppb, planes - p0) * hw);
  }
  for (; grp < groups; grp += gridDim.x) {
    const int p0 = grp * ppb, np = min(ppb, planes - p0);
    const int shift = (int)(((size_t)p0 * hw) & 3);
    __syncthreads();  // the previous group's windows have been read
    sx.commit(lds);
    const int nxt = grp + gridDim.x;
    if (nxt < groups) {
      const int q0 = nxt * ppb;
      sx.issue(bottom, total, (size_t)q0 * hw, min(ppb, planes - q0) * hw);
    }
    __syncthreads();
    float* topg = top + (size_t)p0 * howo;  // uniform base, 32-bit per-thread offsets
    // lane t writes the float whose global index is congruent to t modulo 32: every 32
    // lanes fill one 128-byte line
    const int lead = (int)((reinterpret_cast<uintptr_t>(topg) >> 2) & 31);
    for (int q = (int)threadIdx.x - lead; q < np * howo; q += MNV_POOL_THREADS) {
      if (q < 0) continue;
      const int pl = mnv_fastdiv(q, g.d_howo), o = q - m24(pl, howo);
      const int i = mnv_fastdiv(o, g.d_Wo), j = o - m24(i, g.Wo);
      __builtin_nontemporal_store(pool_window<MAX, KS, ST>(lds + shift + m24(pl, hw), g, i, j, nullptr),
                                  &topg[(unsigned)q]);
    }
  }
}

// LDS: plane data [ppb*hw + 8], top_diff [ppb*howo + 8], arg-max positions [ppb*howo].
template <bool MAX, int KS, int ST, bool NT>
__global__ __launch_bounds__(MNV_POOL_THREADS) void mnv_pool_bwd_lds_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, int planes, int ppb, PoolGeom g, int relu) {
  extern __shared__ float lds[];
  const int hw = g.H * g.W, howo = g.Ho * g.Wo;
  const size_t total_x = (size_t)planes * hw, total_d = (size_t)planes * howo;
  const int groups = (planes + ppb - 1) / ppb;
  float* lx = lds;
  float* ld = lds + ((ppb * hw + 8 + 3) & ~3);
  int* sarg = reinterpret_cast<int*>(ld + ((ppb * howo + 8 + 3) & ~3));
  const int sv = ST ? ST : g.sv, sh = ST ? ST : g.sh;
  const int kh = KS ? KS : g.kh, kw = KS ? KS : g.kw;
  PoolStage<MAX ? MNV_POOL_XV : 1, NT> sx;
  PoolStage<MNV_POOL_DV, NT> sd;
  int grp = blockIdx.x;
  if (grp < groups) {
    const int p0 = grp * ppb, np = min(ppb, planes - p0);
    if (MAX) sx.issue(bottom, total_x, (size_t)p0 * hw, np * hw);
    sd.issue(top_diff, total_d, (size_t)p0 * howo, np * howo);
  }
  for (; grp < groups; grp += gridDim.x) {
    const int p0 = grp * ppb, np = min(ppb, planes - p0);
    const int shift_x = (int)(((size_t)p0 * hw) & 3);
    const float* bx = lx + shift_x;
    const float* bd = ld + (int)(((size_t)p0 * howo) & 3);
    __syncthreads();  // the previous group has been read
    if (MAX) sx.commit(lx);
    sd.commit(ld);
    const int nxt = grp + gridDim.x;
    if (nxt < groups) {
      const int q0 = nxt * ppb, nq = min(ppb, planes - q0);
      if (MAX) sx.issue(bottom, total_x, (size_t)q0 * hw, nq * hw);
      sd.issue(top_diff, total_d, (size_t)q0 * howo, nq * howo);
    }
    __syncthreads();
    if (MAX) {
      // first maximum of every window in scan order, as a flat position in its plane
      for (int q = threadIdx.x; q < np * howo; q += MNV_POOL_THREADS) {
        const int pl = mnv_fastdiv(q, g.d_howo), o = q - m24(pl, howo);
        const int i = mnv_fastdiv(o, g.d_Wo), j = o - m24(i, g.Wo);
        int arg;
        pool_window<true, KS, ST>(bx + m24(pl, hw), g, i, j, &arg);
        sarg[q] = arg;
      }
      __syncthreads();
    }
    // The gradients go to LDS first, over the plane data (dead once the arg-max positions
    // are known), and leave as dense 16-byte stores: written straight from the loop below
    // they would be 4-byte stores at a stride of two.
    float* lout = lx + shift_x;
    if constexpr (ST == 2 && (KS == 2 || KS == 3)) {
      // A thread owns a 2x2 block of padded coordinates (rows 2a, 2a+1; columns 2b, 2b+1).
      // Row 2a lies in windows a-1 (3-wide only) and a, row 2a+1 in window a alone, so the
      // block's four positions draw on the same four windows: their arg-max positions and
      // gradients are read once, and each position adds the ones it wins in ascending
      // window order, like a sequential scatter.
      const int nblk = g.NA * g.NB;
      for (int q = threadIdx.x; q < np * nblk; q += MNV_POOL_THREADS) {
        const int pl = mnv_fastdiv(q, g.d_nab), r = q - m24(pl, nblk);
        const int ai = mnv_fastdiv(r, g.d_nb), bi = r - m24(ai, g.NB);
        const int a = g.a0 + ai, b = g.b0 + bi;
        const int y = 2 * a - g.ph, x = 2 * b - g.pw;
        const float* d = bd + m24(pl, howo);
        const int* sa = sarg + m24(pl, howo);
        const bool vi0 = KS == 3 && a >= 1 && a - 1 < g.Ho, vi1 = a < g.Ho;
        const bool vj0 = KS == 3 && b >= 1 && b - 1 < g.Wo, vj1 = b < g.Wo;
        const int o11 = m24(a, g.Wo) + b, o10 = o11 - 1, o01 = o11 - g.Wo, o00 = o01 - 1;
        // a window that does not exist contributes +0.0f, which changes no sum
        float d00 = (vi0 && vj0) ? d[o00] : 0.f, d01 = (vi0 && vj1) ? d[o01] : 0.f;
        float d10 = (vi1 && vj0) ? d[o10] : 0.f, d11 = (vi1 && vj1) ? d[o11] : 0.f;
        const int p00 = m24(y, g.W) + x, p01 = p00 + 1, p10 = p00 + g.W, p11 = p10 + 1;
        float g00, g01, g10, g11;
        if (MAX) {
          const int s00 = (vi0 && vj0) ? sa[o00] : -1, s01 = (vi0 && vj1) ? sa[o01] : -1;
          const int s10 = (vi1 && vj0) ? sa[o10] : -1, s11 = (vi1 && vj1) ? sa[o11] : -1;
          g00 = (((0.f + (s00 == p00 ? d00 : 0.f)) + (s01 == p00 ? d01 : 0.f)) +
                 (s10 == p00 ? d10 : 0.f)) + (s11 == p00 ? d11 : 0.f);
          g01 = (0.f + (s01 == p01 ? d01 : 0.f)) + (s11 == p01 ? d11 : 0.f);
          g10 = (0.f + (s10 == p10 ? d10 : 0.f)) + (s11 == p10 ? d11 : 0.f);
          g11 = 0.f + (s11 == p11 ? d11 : 0.f);
        } else {
          const float area = (float)(KS * KS);
          d00 = d00 / area; d01 = d01 / area; d10 = d10 / area; d11 = d11 / area;
          g00 = (((0.f + d00) + d01) + d10) + d11;
          g01 = (0.f + d01) + d11;
          g10 = (0.f + d10) + d11;
          g11 = 0.f + d11;
        }
        const bool y0ok = (unsigned)y < (unsigned)g.H, y1ok = (unsigned)(y + 1) < (unsigned)g.H;
        const bool x0ok = (unsigned)x < (unsigned)g.W, x1ok = (unsigned)(x + 1) < (unsigned)g.W;
        const int po = m24(pl, hw);
        if (MAX && relu) {  // lout lies over the plane data: a position's own value is still there
          if (y0ok && x0ok) g00 = lout[po + p00] > 0.f ? g00 : 0.f;
          if (y0ok && x1ok) g01 = lout[po + p01] > 0.f ? g01 : 0.f;
          if (y1ok && x0ok) g10 = lout[po + p10] > 0.f ? g10 : 0.f;
          if (y1ok && x1ok) g11 = lout[po + p11] > 0.f ? g11 : 0.f;
        }
        if (y0ok && x0ok) lout[po + p00] = g00;
        if (y0ok && x1ok) lout[po + p01] = g01;
        if (y1ok && x0ok) lout[po + p10] = g10;
        if (y1ok && x1ok) lout[po + p11] = g11;
      }
    } else {
      for (int q = threadIdx.x; q < np * hw; q += MNV_POOL_THREADS) {
        const int pl = mnv_fastdiv(q, g.d_hw), pos = q - pl * hw;
        const int y = mnv_fastdiv(pos, g.d_W), x = pos - y * g.W;
        // windows i with i*sv - ph <= y < i*sv - ph + kh, clipped to [0, Ho); likewise j
        const int ay = y + g.ph - kh + sv, ax = x + g.pw - kw + sh;  // ceil((y+ph-kh+1)/sv)
        const int i_lo = ay > 0 ? div_stride<ST>(ay, g.d_sv) : 0;
        const int i_hi = min(div_stride<ST>(y + g.ph, g.d_sv), g.Ho - 1);
        const int j_lo = ax > 0 ? div_stride<ST>(ax, g.d_sh) : 0;
        const int j_hi = min(div_stride<ST>(x + g.pw, g.d_sh), g.Wo - 1);
        const float* d = bd + pl * howo;
        const int* sa = sarg + pl * howo;
        float acc = 0.f;
        // gradients are added in ascending window order, like a sequential scatter
        if (KS && ST) {
          constexpr int CNT = (KS && ST) ? (KS + ST - 1) / (ST ? ST : 1) : 1;
  #pragma unroll
          for (int a = 0; a < CNT; ++a)
  #pragma unroll
            for (int c = 0; c < CNT; ++c) {
              const int i = i_lo + a, j = j_lo + c;
              if ((i <= i_hi) & (j <= j_hi)) {
                const int o = i * g.Wo + j;
                if (MAX) {
                  if (sa[o] == pos) acc += d[o];
                } else {
                  acc += d[o] / (float)(kh * kw);
                }
              }
            }
        } else {
          for (int i = i_lo; i <= i_hi; ++i)
            for (int j = j_lo; j <= j_hi; ++j) {
              const int o = i * g.Wo + j;
              if (MAX) {
                if (sa[o] == pos) acc += d[o];
              } else {
                acc += d[o] / (float)(kh * kw);
              }
            }
        }
        if (MAX && relu) acc = lout[q] > 0.f ? acc : 0.f;
        lout[q] = acc;
      }
    }
    __syncthreads();
    pool_write_group(lx, bottom_diff + (size_t)p0 * hw, shift_x, np * hw);
  }
}

// ---- max-pooling gradient of 3x3/2 and 2x2/2 windows: an ordered scatter in LDS --------
// Every window's first maximum is found once and noted in LDS (position and pass); the
// plane data is then cleared and the gradients are added to it window by window.  No
// atomics and still the sums of a sequential scatter, bit for bit:
//  * 2x2/2 windows do not overlap: one pass.
//  * 3x3/2: a position with an odd (padded) coordinate lies in at most two windows, and a
//    two-term sum does not depend on its order.  A position with both coordinates even
//    lies in four windows, whose scan order is: the one that has it at its corner (2,2),
//    then (2,0), then (0,2), then (0,0).  So the additions are made in four passes keyed by
//    where in its window the maximum sits -- pass = 2*[row 0] + [column 0] -- with a
//    barrier between passes.  Within a pass no two windows write the same position (equal
//    row parity within a pass means equal row offset, hence the same window row; likewise
//    for columns), so plain read-add-write is safe.
// Against the gather kernel above this halves the integer work per element, which is what
// bounds the gradient (the bytes moved are the same).
// XV / DV: 16-byte vectors of plane data / top_diff a thread stages for the next group;
// WPT: windows per thread and group.  The small configuration (4, 1, 4) keeps the kernel
// under 64 registers so that eight workgroups share a CU: the phases of a group are
// separated by barriers and bound by LDS latency, and more resident workgroups hide that.
template <int KS, int ST, int XV, int DV, int WPT, bool NT>
__global__ __launch_bounds__(MNV_POOL_THREADS, XV <= 4 ? 7 : 4) void mnv_maxpool_bwd_scatter_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, int planes, int ppb, PoolGeom g, int relu) {
  extern __shared__ float lds[];
  const int hw = g.H * g.W, howo = g.Ho * g.Wo;
  const size_t total_x = (size_t)planes * hw, total_d = (size_t)planes * howo;
  const int groups = (planes + ppb - 1) / ppb;
  // LDS: plane data [ppb*hw + 8], top_diff [ppb*howo + 8], window codes [ppb*howo]
  float* lx = lds;
  float* ld = lds + ((ppb * hw + 8 + 3) & ~3);
  int* code = reinterpret_cast<int*>(ld + ((ppb * howo + 8 + 3) & ~3));
  PoolStage<XV, NT> sx;
  PoolStage<DV, NT> sd;
  int grp = blockIdx.x;
  if (grp < groups) {
    const int p0 = grp * ppb, np = min(ppb, planes - p0);
    sx.issue(bottom, total_x, (size_t)p0 * hw, np * hw);
    sd.issue(top_diff, total_d, (size_t)p0 * howo, np * howo);
  }
  for (; grp < groups; grp += gridDim.x) {
    const int p0 = grp * ppb, np = min(ppb, planes - p0);
    const int shift_x = (int)(((size_t)p0 * hw) & 3);
    const float* bd = ld + (int)(((size_t)p0 * howo) & 3);
    __syncthreads();  // the previous group's gradients have left LDS
    sx.commit(lx);
    sd.commit(ld);
    const int nxt = grp + gridDim.x;
    if (nxt < groups) {
      const int q0 = nxt * ppb, nq = min(ppb, planes - q0);
      sx.issue(bottom, total_x, (size_t)q0 * hw, nq * hw);
      sd.issue(top_diff, total_d, (size_t)q0 * howo, nq * howo);
    }
    __syncthreads();
    // first maximum of every window: (LDS index of the position) * 4 + pass.  Two windows
    // per thread and iteration, so that the LDS reads of one overlap the compares of the
    // other; when every window of the wavefront lies inside its plane (all of them when
    // nothing is padded or clipped) the two scans are straight-line code.
    const int nwin = np * howo;
    for (int q0 = 0; q0 < nwin; q0 += 2 * MNV_POOL_THREADS) {
      int q[2], base[2], i[2], j[2], po[2];
      bool inside = true;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        q[u] = q0 + threadIdx.x + u * MNV_POOL_THREADS;
        const int qq = min(q[u], nwin - 1);  // a window past the end repeats the last one
        const int pl = mnv_fastdiv(qq, g.d_howo), o = qq - m24(pl, howo);
        i[u] = mnv_fastdiv(o, g.d_Wo);
        j[u] = o - m24(i[u], g.Wo);
        po[u] = shift_x + m24(pl, hw);
        const int y0 = i[u] * ST - g.ph, x0 = j[u] * ST - g.pw;
        base[u] = m24(y0, g.W) + x0;
        inside = inside && y0 >= 0 && x0 >= 0 && y0 + KS <= g.H && x0 + KS <= g.W;
      }
      int arg[2], pass[2];
      if (__all(inside)) {
        float v[2][KS * KS];
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int dy = 0; dy < KS; ++dy)
#pragma unroll
            for (int dx = 0; dx < KS; ++dx) v[u][dy * KS + dx] = lx[po[u] + base[u] + dy * g.W + dx];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          float r = -INFINITY;
          int rel = 0, ps = 3;  // offset of the maximum from the window's corner, its pass
#pragma unroll
          for (int dy = 0; dy < KS; ++dy)
#pragma unroll
            for (int dx = 0; dx < KS; ++dx)
              if (r < v[u][dy * KS + dx]) {
                r = v[u][dy * KS + dx];
                rel = dy * g.W + dx;
                ps = (dy == 0 ? 2 : 0) + (dx == 0 ? 1 : 0);
              }
          arg[u] = base[u] + rel;
          pass[u] = KS == 3 ? ps : 0;
        }
      } else {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          pool_window<true, KS, ST>(lx + po[u], g, i[u], j[u], &arg[u]);
          pass[u] = 0;
          if (KS == 3) {
            const int y = mnv_fastdiv(arg[u], g.d_W), x = arg[u] - m24(y, g.W);
            pass[u] = (y == i[u] * ST - g.ph ? 2 : 0) + (x == j[u] * ST - g.pw ? 1 : 0);
          }
        }
      }
      // Fused ReLU gradient: a position receives gradients only from windows whose maximum
      // it is, and the gate tests that same value, so a window whose maximum is not positive
      // is dropped here and its position keeps the +0 it was cleared to -- what the gate
      // would have selected.
#pragma unroll
      for (int u = 0; u < 2; ++u)
        if (q[u] < nwin) {
          int c = ((po[u] + arg[u]) << 2) | pass[u];
          if (relu && !(lx[po[u] + arg[u]] > 0.f)) c = -1;
          code[q[u]] = c;
        }
    }
    __syncthreads();  // every window has read the plane data: the planes become the gradient
    // this thread's windows, read once for all passes (at most WPT of them)
    int wc[WPT];
    float wd[WPT];
#pragma unroll
    for (int k = 0; k < WPT; ++k) {
      const int q = threadIdx.x + k * MNV_POOL_THREADS;
      const bool in = q < np * howo;
      wc[k] = in ? code[q] : -1;
      wd[k] = in ? bd[q] : 0.f;
    }
    const int nv = (shift_x + np * hw + 3) >> 2;
    for (int v = threadIdx.x; v < nv; v += MNV_POOL_THREADS)
      reinterpret_cast<mnv_f4*>(lx)[v] = mnv_f4{0.f, 0.f, 0.f, 0.f};
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < (KS == 3 ? 4 : 1); ++pass) {
#pragma unroll
      for (int k = 0; k < WPT; ++k)
        if (wc[k] >= 0 && (wc[k] & 3) == pass) lx[wc[k] >> 2] += wd[k];
      __syncthreads();
    }
    pool_write_group(lx, bottom_diff + (size_t)p0 * hw, shift_x, np * hw);
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
    float* __restrict__ bottom_diff, size_t planes, PoolGeom g, int relu) {
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
    if (MAX && relu) acc = b[pos] > 0.f ? acc : 0.f;
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
  g->a0 = ph >> 1;
  g->b0 = pw >> 1;
  g->NA = ((ph + h - 1) >> 1) - g->a0 + 1;
  g->NB = ((pw + w - 1) >> 1) - g->b0 + 1;
  g->d_nab = mnv_fastdiv_make(g->NA * g->NB);
  g->d_nb = mnv_fastdiv_make(g->NB);
  return MNV_OK;
}

unsigned pool_grid(size_t total) {
  size_t blocks = mnv_ceil_div(total, MNV_POOL_THREADS);
  if (blocks > 4 * MNV_MAX_STREAM_BLOCKS) blocks = 4 * MNV_MAX_STREAM_BLOCKS;
  return (unsigned)blocks;
}

// Planes per workgroup for the LDS path: as many as fit the register staging and 48 KiB of
// LDS, but few enough that every workgroup gets several groups to pipeline.  0 = a plane is
// too large (or a pointer not 16-byte aligned): use the direct kernels.
int planes_per_block(const PoolGeom& g, long long planes, bool bwd) {
  const long long hw = (long long)g.H * g.W, howo = (long long)g.Ho * g.Wo;
  long long ppb = (MNV_POOL_X_FLOATS - 6) / hw;
  if (bwd) {
    ppb = std::min(ppb, (MNV_POOL_D_FLOATS - 6) / howo);
    ppb = std::min(ppb, (12288 - 24) / (hw + 2 * howo));
  }
  if (ppb < 1) return 0;
  long long cap = planes / 4096;
  if (cap < 1) cap = 1;
  if (ppb > cap) ppb = cap;
  if (ppb > 64) ppb = 64;
  return (int)ppb;
}

// Workgroups of a pipelined launch: `rounds` times what fits on the chip at once, each
// looping over its share of the groups.  One round keeps every workgroup resident for the
// whole kernel; several rounds let the dispatcher hand the slots of workgroups that
// finish early to new ones, which evens out the spread between CUs (the forward kernel
// gains 7% from six rounds, the gradient kernels nothing).
unsigned lds_grid(long long groups, size_t lds_bytes, int rounds = 1) {
  long long per_cu = (160 * 1024) / (long long)(lds_bytes + 512);
  if (per_cu > 8) per_cu = 8;
  if (per_cu < 1) per_cu = 1;
  long long blocks = 256 * per_cu * rounds;
  return (unsigned)(groups < blocks ? groups : blocks);
}

template <bool MAX>
int pool_fwd(const float* bottom, float* top, int n, int c, int h, int w, int sv, int sh, int kh,
             int kw, int ph, int pw, mnv_stream_t stream) {
  PoolGeom g;
  if (!bottom || !top) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  long long planes = (long long)n * c;
  int ppb = mnv_aligned16(bottom) ? planes_per_block(g, planes, false) : 0;
  if (ppb > 0) {
    size_t lds = ((size_t)ppb * h * w + 8) * sizeof(float);
    long long groups = (planes + ppb - 1) / ppb;
    const bool sq = kh == kw && sv == sh;
    const bool nt = (size_t)planes * h * w * sizeof(float) >= MNV_PAST_CACHE_BYTES;
    auto kernel = (sq && kh == 3 && sv == 2)
                      ? (nt ? mnv_pool_fwd_lds_kernel<MAX, 3, 2, true> : mnv_pool_fwd_lds_kernel<MAX, 3, 2, false>)
                  : (sq && kh == 2 && sv == 2)
                      ? (nt ? mnv_pool_fwd_lds_kernel<MAX, 2, 2, true> : mnv_pool_fwd_lds_kernel<MAX, 2, 2, false>)
                      : (nt ? mnv_pool_fwd_lds_kernel<MAX, 0, 0, true> : mnv_pool_fwd_lds_kernel<MAX, 0, 0, false>);
    hipLaunchKernelGGL(kernel, dim3(lds_grid(groups, lds, 6)), dim3(MNV_POOL_THREADS), lds,
                       mnv_stream(stream), bottom, top, (int)planes, ppb, g);
  } else {
    hipLaunchKernelGGL((mnv_pool_fwd_kernel<MAX>), dim3(pool_grid((size_t)planes * g.Ho * g.Wo)),
                       dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top, (size_t)planes,
                       g);
  }
  return MNV_LAUNCH_STATUS();
}

template <bool MAX>
int pool_bwd(const float* bottom, const float* top_diff, float* bottom_diff, int n, int c, int h,
             int w, int sv, int sh, int kh, int kw, int ph, int pw, mnv_stream_t stream,
             int relu = 0) {
  PoolGeom g;
  if (!bottom || !top_diff || !bottom_diff) return MNV_ERR_INVALID;
  int rc = make_geom(&g, n, c, h, w, sv, sh, kh, kw, ph, pw);
  if (rc) return rc;
  long long planes = (long long)n * c;
  const bool aligned = mnv_aligned16(bottom) && mnv_aligned16(top_diff) && mnv_aligned16(bottom_diff);
  if (MAX && aligned && kh == kw && sv == sh && sv == 2 && (kh == 2 || kh == 3)) {
    const long long hw = (long long)h * w, howo = (long long)g.Ho * g.Wo;
    // small configuration first: planes that fit 4 staged vectors and 4 windows per thread
    long long small = std::min((long long)(MNV_POOL_THREADS * 4 * 4 - 6) / hw,
                               std::min((long long)(MNV_POOL_THREADS * 4 * 1 - 6) / howo,
                                        (long long)(4 * MNV_POOL_THREADS) / howo));
    long long big = std::min((long long)planes_per_block(g, planes, true),
                             (long long)(8 * MNV_POOL_THREADS) / howo);
    const long long cap = std::max(1LL, planes / 4096);
    small = std::min(small, cap);
    // one large plane per group leaves the small configuration's window slots a quarter
    // empty: such planes go two to a group in the large one
    const bool use_small = small >= 2 || (small == 1 && big <= 1);
    const int spb = (int)(use_small ? small : big);
    if (spb > 0) {
      const size_t lds = ((((size_t)spb * hw + 8 + 3) & ~(size_t)3) + (((size_t)spb * howo + 8 + 3) & ~(size_t)3) +
                          (size_t)spb * howo) * sizeof(float);
      const long long groups = (planes + spb - 1) / spb;
      const bool nt = (size_t)planes * hw * sizeof(float) >= MNV_PAST_CACHE_BYTES;
      auto kernel =
          kh == 3 ? (use_small ? (nt ? mnv_maxpool_bwd_scatter_kernel<3, 2, 4, 1, 4, true>
                                     : mnv_maxpool_bwd_scatter_kernel<3, 2, 4, 1, 4, false>)
                               : (nt ? mnv_maxpool_bwd_scatter_kernel<3, 2, 8, 4, 8, true>
                                     : mnv_maxpool_bwd_scatter_kernel<3, 2, 8, 4, 8, false>))
                  : (use_small ? (nt ? mnv_maxpool_bwd_scatter_kernel<2, 2, 4, 1, 4, true>
                                     : mnv_maxpool_bwd_scatter_kernel<2, 2, 4, 1, 4, false>)
                               : (nt ? mnv_maxpool_bwd_scatter_kernel<2, 2, 8, 4, 8, true>
                                     : mnv_maxpool_bwd_scatter_kernel<2, 2, 8, 4, 8, false>));
      hipLaunchKernelGGL(kernel, dim3(lds_grid(groups, lds)), dim3(MNV_POOL_THREADS), lds,
                         mnv_stream(stream), bottom, top_diff, bottom_diff, (int)planes, spb, g,
                         relu);
      return MNV_LAUNCH_STATUS();
    }
  }
  int ppb = aligned ? planes_per_block(g, planes, true) : 0;
  if (ppb > 0) {
    const size_t hw = (size_t)h * w, howo = (size_t)g.Ho * g.Wo;
    size_t lds = (((ppb * hw + 8 + 3) & ~(size_t)3) + ((ppb * howo + 8 + 3) & ~(size_t)3) +
                  ppb * howo) * sizeof(float);
    long long groups = (planes + ppb - 1) / ppb;
    const bool sq = kh == kw && sv == sh;
    const bool nt = (size_t)planes * hw * sizeof(float) >= MNV_PAST_CACHE_BYTES;
    auto kernel = (sq && kh == 3 && sv == 2)
                      ? (nt ? mnv_pool_bwd_lds_kernel<MAX, 3, 2, true> : mnv_pool_bwd_lds_kernel<MAX, 3, 2, false>)
                  : (sq && kh == 2 && sv == 2)
                      ? (nt ? mnv_pool_bwd_lds_kernel<MAX, 2, 2, true> : mnv_pool_bwd_lds_kernel<MAX, 2, 2, false>)
                      : (nt ? mnv_pool_bwd_lds_kernel<MAX, 0, 0, true> : mnv_pool_bwd_lds_kernel<MAX, 0, 0, false>);
    hipLaunchKernelGGL(kernel, dim3(lds_grid(groups, lds)), dim3(MNV_POOL_THREADS), lds,
                       mnv_stream(stream), bottom, top_diff, bottom_diff, (int)planes, ppb, g, relu);
  } else {
    hipLaunchKernelGGL((mnv_pool_bwd_kernel<MAX>), dim3(pool_grid((size_t)planes * h * w)),
                       dim3(MNV_POOL_THREADS), 0, mnv_stream(stream), bottom, top_diff,
                       bottom_diff, (size_t)planes, g, relu);
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
int mnv_maxpool_bwd_relu(const float* bottom, const float* top, const float* top_diff,
                         float* bottom_diff, int n, int c, int h, int w, int sv, int sh, int kh,
                         int kw, int ph, int pw, mnv_stream_t s) {
  (void)top;
  return pool_bwd<true>(bottom, top_diff, bottom_diff, n, c, h, w, sv, sh, kh, kw, ph, pw, s, 1);
}
int mnv_avgpool_bwd(const float* bottom, const float* top, const float* top_diff,
                    float* bottom_diff, int n, int c, int h, int w, int sv, int sh, int kh,
                    int kw, int ph, int pw, mnv_stream_t s) {
  (void)top;
  if (!bottom) return MNV_ERR_INVALID;
  return pool_bwd<false>(bottom, top_diff, bottom_diff, n, c, h, w, sv, sh, kh, kw, ph, pw, s);
}

}  // extern "C"
