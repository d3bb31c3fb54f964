// Softmax forward / backward over an image batch {W,H,C,N}
// (reference CPU forward minerva/op/impl/basic.cpp:219-261; cuDNN modes selected at
// minerva/op/impl/cuda/cuda_perform.cu:339-397).
//   instance: one softmax over the C*H*W contiguous values of each image;
//   channel : one softmax over the C values (stride H*W) at each (n,h,w).
// forward : y_i = exp(x_i - max) / sum_j exp(x_j - max)
// backward: dx_i = y_i * (dy_i - sum_j dy_j*y_j)
// Roofline: HBM bandwidth, 8 bytes per element forward and 12 backward: a line of
// up to 8192 values is held in registers between the passes, so it is read once.
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_SM_THREADS 256
#define MNV_SM_CACHE 8  // 16-byte vectors cached per thread

template <int GROUP>
__device__ __forceinline__ float group_max(float v, float* lds) {
  v = mnv_wave_max(v);
  v = __shfl(v, 0, MNV_WAVE);
  if (GROUP > MNV_WAVE) {
    const int w = threadIdx.x / MNV_WAVE;
    __syncthreads();
    if ((threadIdx.x % MNV_WAVE) == 0) lds[w] = v;
    __syncthreads();
    v = lds[0];
#pragma unroll
    for (int q = 1; q < GROUP / MNV_WAVE; ++q) v = fmaxf(v, lds[q]);
  }
  return v;
}

template <int GROUP>
__device__ __forceinline__ float group_sum(float v, float* lds) {
  v = mnv_wave_sum(v);
  v = __shfl(v, 0, MNV_WAVE);
  if (GROUP > MNV_WAVE) {
    const int w = threadIdx.x / MNV_WAVE;
    __syncthreads();
    if ((threadIdx.x % MNV_WAVE) == 0) lds[w] = v;
    __syncthreads();
    v = lds[0];
#pragma unroll
    for (int q = 1; q < GROUP / MNV_WAVE; ++q) v += lds[q];
  }
  return v;
}

// Keeps a per-thread pointer in a pair of vector registers and hides its value from the
// compiler, which otherwise addresses the line as (scalar base + 32-bit lane offset).
// Measured on 8192 lines of 8192 floats: forward 5.8 -> 6.1 TB/s, backward 5.9 -> 6.1 TB/s.
// A plain copy written in both forms runs at the same rate, so the form of the address is
// not what costs: what changes is where the compiler puts the address arithmetic and the
// waits between the guarded loads and stores.
template <class T>
__device__ __forceinline__ T* lane_pointer(T* p) {
  asm volatile("" : "+v"(p));
  return p;
}

// One line per GROUP threads of an NTH-thread workgroup (GROUP = one wavefront or the whole
// workgroup); the line (len % 4 == 0, len <= GROUP*4*CACHE) is cached in registers.
// Stores are non-temporal; NT: so are the loads (inputs of 256 MB and more, which no cache
// holds until the next operator).  Lines of up to 8192 values take 512 threads with four
// vectors each rather than 256 with eight (more wavefronts, shorter per-thread chains): on
// 8192 lines of 8192, operands cycled through four sets, 6.3 TB/s against 5.8 TB/s (a plain
// copy of the same operands: 6.3 TB/s).
template <int GROUP, int CACHE, int NTH, bool NT>
__global__ __launch_bounds__(NTH) void mnv_softmax_fwd_cached_kernel(
    const float* __restrict__ in, float* __restrict__ out, int len, int lines) {
  __shared__ float lds[NTH / MNV_WAVE];
  constexpr int LPB = NTH / GROUP;
  const int t = threadIdx.x % GROUP;
  const int len4 = len >> 2;
  // the trip count is block-uniform when GROUP spans the block (and the line index then a
  // scalar: the compiler cannot tell that threadIdx.x / GROUP is 0); with one wavefront per
  // line no barrier is used
  for (int line = blockIdx.x * LPB + (LPB > 1 ? threadIdx.x / GROUP : 0); line < lines; line += gridDim.x * LPB) {
    const mnv_f4* x4 = lane_pointer(reinterpret_cast<const mnv_f4*>(in + (size_t)line * len) + t);
    mnv_f4* y4 = lane_pointer(reinterpret_cast<mnv_f4*>(out + (size_t)line * len) + t);
    mnv_f4 v[CACHE];
    // all loads first, in a loop of their own: a use inside the same guarded block would
    // make each load wait for the one before it
#pragma unroll
    for (int u = 0; u < CACHE; ++u)
      if (t + u * GROUP < len4) v[u] = mnv_ldx4<NT>(x4 + u * GROUP);
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < CACHE; ++u)
      if (t + u * GROUP < len4) mx = fmaxf(mx, fmaxf(fmaxf(v[u].x, v[u].y), fmaxf(v[u].z, v[u].w)));
    mx = group_max<GROUP>(mx, lds);
    float s = 0.f;
#pragma unroll
    for (int u = 0; u < CACHE; ++u) {
      if (t + u * GROUP < len4) {
        // exp through the hardware exp2: relative error ~1e-6 for the arguments <= 0 here
        v[u].x = __expf(v[u].x - mx);
        v[u].y = __expf(v[u].y - mx);
        v[u].z = __expf(v[u].z - mx);
        v[u].w = __expf(v[u].w - mx);
        s += (v[u].x + v[u].y) + (v[u].z + v[u].w);
      }
    }
    s = group_sum<GROUP>(s, lds);
    const float inv = 1.0f / s;  // one reciprocal per thread instead of a division per element
#pragma unroll
    for (int u = 0; u < CACHE; ++u) {
      if (t + u * GROUP < len4) {
        mnv_f4 o;
        o.x = v[u].x * inv;
        o.y = v[u].y * inv;
        o.z = v[u].z * inv;
        o.w = v[u].w * inv;
        __builtin_nontemporal_store(o, y4 + u * GROUP);
      }
    }
  }
}

// Any length / alignment / stride: three passes over the line.  Element i of line
// (a, b) lives at in[a*outer + b + i*stride]; `inner` = number of b values.
template <int GROUP>
__global__ __launch_bounds__(MNV_SM_THREADS) void mnv_softmax_fwd_generic_kernel(
    const float* __restrict__ in, float* __restrict__ out, int len, int lines, int inner,
    size_t outer, size_t stride) {
  __shared__ float lds[MNV_SM_THREADS / MNV_WAVE];
  constexpr int LPB = MNV_SM_THREADS / GROUP;
  const int t = threadIdx.x % GROUP;
  for (int line = blockIdx.x * LPB + (LPB > 1 ? threadIdx.x / GROUP : 0); line < lines; line += gridDim.x * LPB) {
    size_t base = (size_t)(line / inner) * outer + (size_t)(line % inner);
    const float* x = in + base;
    float* y = out + base;
    float mx = -INFINITY;
    for (int i = t; i < len; i += GROUP) mx = fmaxf(mx, x[i * stride]);
    mx = group_max<GROUP>(mx, lds);
    float s = 0.f;
    for (int i = t; i < len; i += GROUP) {
      float e = expf(x[i * stride] - mx);
      y[i * stride] = e;
      s += e;
    }
    s = group_sum<GROUP>(s, lds);
    for (int i = t; i < len; i += GROUP) y[i * stride] = y[i * stride] / s;
  }
}

template <int GROUP, int CACHE, int NTH>
__global__ __launch_bounds__(NTH) void mnv_softmax_bwd_cached_kernel(
    const float* __restrict__ dy, const float* __restrict__ y, float* __restrict__ dx, int len,
    int lines) {
  __shared__ float lds[NTH / MNV_WAVE];
  constexpr int LPB = NTH / GROUP;
  const int t = threadIdx.x % GROUP;
  const int len4 = len >> 2;
  for (int line = blockIdx.x * LPB + (LPB > 1 ? threadIdx.x / GROUP : 0); line < lines; line += gridDim.x * LPB) {
    const mnv_f4* d4 = lane_pointer(reinterpret_cast<const mnv_f4*>(dy + (size_t)line * len) + t);
    const mnv_f4* t4 = lane_pointer(reinterpret_cast<const mnv_f4*>(y + (size_t)line * len) + t);
    mnv_f4* o4 = lane_pointer(reinterpret_cast<mnv_f4*>(dx + (size_t)line * len) + t);
    mnv_f4 d[CACHE], p[CACHE];
#pragma unroll
    for (int u = 0; u < CACHE; ++u) {  // loads only, so that none waits for another
      if (t + u * GROUP < len4) {
        d[u] = d4[u * GROUP];
        p[u] = __builtin_nontemporal_load(t4 + u * GROUP);
      }
    }
    float dot = 0.f;
#pragma unroll
    for (int u = 0; u < CACHE; ++u)
      if (t + u * GROUP < len4)
        dot += (d[u].x * p[u].x + d[u].y * p[u].y) + (d[u].z * p[u].z + d[u].w * p[u].w);
    dot = group_sum<GROUP>(dot, lds);
#pragma unroll
    for (int u = 0; u < CACHE; ++u) {
      if (t + u * GROUP < len4) {
        mnv_f4 o;
        o.x = p[u].x * (d[u].x - dot);
        o.y = p[u].y * (d[u].y - dot);
        o.z = p[u].z * (d[u].z - dot);
        o.w = p[u].w * (d[u].w - dot);
        __builtin_nontemporal_store(o, o4 + u * GROUP);
      }
    }
  }
}

template <int GROUP>
__global__ __launch_bounds__(MNV_SM_THREADS) void mnv_softmax_bwd_generic_kernel(
    const float* __restrict__ dy, const float* __restrict__ y, float* __restrict__ dx, int len,
    int lines, int inner, size_t outer, size_t stride) {
  __shared__ float lds[MNV_SM_THREADS / MNV_WAVE];
  constexpr int LPB = MNV_SM_THREADS / GROUP;
  const int t = threadIdx.x % GROUP;
  for (int line = blockIdx.x * LPB + (LPB > 1 ? threadIdx.x / GROUP : 0); line < lines; line += gridDim.x * LPB) {
    size_t base = (size_t)(line / inner) * outer + (size_t)(line % inner);
    float dot = 0.f;
    for (int i = t; i < len; i += GROUP) dot += dy[base + i * stride] * y[base + i * stride];
    dot = group_sum<GROUP>(dot, lds);
    for (int i = t; i < len; i += GROUP)
      dx[base + i * stride] = y[base + i * stride] * (dy[base + i * stride] - dot);
  }
}

// Channel mode with H*W > 1.  A workgroup owns POS neighbouring (h,w) positions of one image
// (POS * 4 contiguous bytes of every channel plane: a full 128-byte line for POS = 32) and
// splits the channels over G thread groups, thread (p, g) taking channels g, g + G, ...; the
// groups' maxima and sums meet in LDS.  A thread keeps its up to CACHE values in registers
// between the passes, so a position's channels are read once and written once (8 bytes per
// element forward, 12 backward); with more than G * CACHE channels the passes re-read memory.
// (One thread per position walking all channels, the first version, left a chip with 65536
// positions to 256 workgroups with one load in flight per thread: 0.4 TB/s.)
// Workgroups are dealt round-robin to the 8 XCDs: workgroup b of `total` takes block
// (b % 8) * (total / 8) + b / 8, so each XCD walks a contiguous run of blocks.
__device__ __forceinline__ int channel_block(unsigned b, unsigned total) {
  const unsigned per = total / 8;
  return (int)(b < per * 8 ? (b % 8) * per + b / 8 : b);
}

template <int POS, int G, int CACHE>
__global__ __launch_bounds__(POS* G, POS* G >= 1024 ? 8 : 1) void mnv_softmax_channel_fwd_kernel(
    const float* __restrict__ in, float* __restrict__ out, int c, int hw, int blocks_per_image) {
  __shared__ float red[G][POS];
  const int p = threadIdx.x % POS, g = threadIdx.x / POS;
  // a plane size off the 128-byte grid makes neighbouring runs of positions share a line at
  // either end: such runs go to one XCD, whose L2 then sees both halves of the line (planes of
  // 181 x 181: 0.24 -> 0.30 of the HBM peak; aligned planes lose 5% that way and keep the
  // plain order)
  const int blk = hw % 32 ? channel_block(blockIdx.x, gridDim.x) : (int)blockIdx.x;
  const int img = blk / blocks_per_image;
  const int pos = (blk - img * blocks_per_image) * POS + p;
  const bool live = pos < hw;
  const size_t base = (size_t)img * c * hw + (live ? pos : 0);
  const bool cached = c <= G * CACHE;
  float v[CACHE];
  float mx = -INFINITY;
  if (cached) {
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      const int k = g + i * G;
      v[i] = (live && k < c) ? in[base + (size_t)k * hw] : -INFINITY;
    }
#pragma unroll
    for (int i = 0; i < CACHE; ++i) mx = fmaxf(mx, v[i]);
  } else if (live) {
    for (int k = g; k < c; k += G) mx = fmaxf(mx, in[base + (size_t)k * hw]);
  }
  red[g][p] = mx;
  __syncthreads();
#pragma unroll
  for (int q = 0; q < G; ++q) mx = fmaxf(mx, red[q][p]);
  __syncthreads();
  float sum = 0.f;
  if (cached) {
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      v[i] = __expf(v[i] - mx);  // hardware exp2, as in the line kernels; exp(-inf) = 0 past the last channel
      sum += v[i];
    }
  } else if (live) {
    for (int k = g; k < c; k += G) sum += __expf(in[base + (size_t)k * hw] - mx);
  }
  red[g][p] = sum;
  __syncthreads();
  sum = 0.f;
#pragma unroll
  for (int q = 0; q < G; ++q) sum += red[q][p];   // the same order in every thread of a position
  if (!live) return;
  const float inv = 1.0f / sum;  // one reciprocal per thread instead of a division per element
  if (cached) {
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      const int k = g + i * G;
      if (k < c) __builtin_nontemporal_store(v[i] * inv, out + base + (size_t)k * hw);
    }
  } else {
    for (int k = g; k < c; k += G) out[base + (size_t)k * hw] = __expf(in[base + (size_t)k * hw] - mx) * inv;
  }
}

template <int POS, int G, int CACHE>
__global__ __launch_bounds__(POS* G) void mnv_softmax_channel_bwd_kernel(
    const float* __restrict__ dy, const float* __restrict__ y, float* __restrict__ dx, int c, int hw,
    int blocks_per_image) {
  __shared__ float red[G][POS];
  const int p = threadIdx.x % POS, g = threadIdx.x / POS;
  // a plane size off the 128-byte grid makes neighbouring runs of positions share a line at
  // either end: such runs go to one XCD, whose L2 then sees both halves of the line (planes of
  // 181 x 181: 0.24 -> 0.30 of the HBM peak; aligned planes lose 5% that way and keep the
  // plain order)
  const int blk = hw % 32 ? channel_block(blockIdx.x, gridDim.x) : (int)blockIdx.x;
  const int img = blk / blocks_per_image;
  const int pos = (blk - img * blocks_per_image) * POS + p;
  const bool live = pos < hw;
  const size_t base = (size_t)img * c * hw + (live ? pos : 0);
  const bool cached = c <= G * CACHE;
  float vy[CACHE], vd[CACHE];
  float dot = 0.f;
  if (cached) {
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      const int k = g + i * G;
      const bool ok = live && k < c;
      vy[i] = ok ? y[base + (size_t)k * hw] : 0.f;
      vd[i] = ok ? dy[base + (size_t)k * hw] : 0.f;
    }
#pragma unroll
    for (int i = 0; i < CACHE; ++i) dot += vd[i] * vy[i];
  } else if (live) {
    for (int k = g; k < c; k += G) dot += dy[base + (size_t)k * hw] * y[base + (size_t)k * hw];
  }
  red[g][p] = dot;
  __syncthreads();
  dot = 0.f;
#pragma unroll
  for (int q = 0; q < G; ++q) dot += red[q][p];
  if (!live) return;
  if (cached) {
#pragma unroll
    for (int i = 0; i < CACHE; ++i) {
      const int k = g + i * G;
      if (k < c) __builtin_nontemporal_store(vy[i] * (vd[i] - dot), dx + base + (size_t)k * hw);
    }
  } else {
    for (int k = g; k < c; k += G)
      dx[base + (size_t)k * hw] = y[base + (size_t)k * hw] * (dy[base + (size_t)k * hw] - dot);
  }
}

// Few channels: 64 positions x 4 channel groups; otherwise 32 positions x 32 groups
// (up to 1024 channels in registers).
#define MNV_SMC_SMALL_C 64

bool dims_ok(int n, int c, int h, int w, long long* len) {
  if (n <= 0 || c <= 0 || h <= 0 || w <= 0) return false;
  long long l = (long long)c * h * w;
  if (l > 0x7fffffffLL) return false;
  *len = l;
  return true;
}

unsigned line_grid(int lines, int lpb) {
  size_t b = mnv_ceil_div((size_t)lines, lpb);
  return (unsigned)(b < 65536 ? b : 65536);
}

// Contiguous lines of `len` floats (instance mode, or channel mode with H*W == 1).
#define MNV_SM_WIDE 512      // threads per line for lines of more than 4096 values
#define MNV_SM_WIDE_CACHE 4  // 16-byte vectors cached per thread in that configuration
template <int GROUP, int CACHE, int NTH>
void launch_fwd_cached(const float* in, float* out, int len, int lines, bool nt, hipStream_t s) {
  const dim3 grid(line_grid(lines, NTH / GROUP)), block(NTH);
  if (nt)
    hipLaunchKernelGGL((mnv_softmax_fwd_cached_kernel<GROUP, CACHE, NTH, true>), grid, block, 0, s, in,
                       out, len, lines);
  else
    hipLaunchKernelGGL((mnv_softmax_fwd_cached_kernel<GROUP, CACHE, NTH, false>), grid, block, 0, s, in,
                       out, len, lines);
}

int softmax_lines_fwd(const float* in, float* out, int len, int lines, hipStream_t s) {
  bool vec = (len % 4 == 0) && mnv_aligned16(in) && mnv_aligned16(out);
  const bool big = (size_t)len * lines * sizeof(float) >= MNV_PAST_CACHE_BYTES;
  if (vec && len <= MNV_WAVE * 4 * MNV_SM_CACHE)
    launch_fwd_cached<MNV_WAVE, MNV_SM_CACHE, MNV_SM_THREADS>(in, out, len, lines, big, s);
  else if (vec && len <= MNV_SM_THREADS * 4 * MNV_SM_WIDE_CACHE)
    launch_fwd_cached<MNV_SM_THREADS, MNV_SM_WIDE_CACHE, MNV_SM_THREADS>(in, out, len, lines, big, s);
  else if (vec && len <= MNV_SM_WIDE * 4 * MNV_SM_WIDE_CACHE)
    launch_fwd_cached<MNV_SM_WIDE, MNV_SM_WIDE_CACHE, MNV_SM_WIDE>(in, out, len, lines, big, s);
  else if (len <= 1024)
    hipLaunchKernelGGL((mnv_softmax_fwd_generic_kernel<MNV_WAVE>), dim3(line_grid(lines, 4)),
                       dim3(MNV_SM_THREADS), 0, s, in, out, len, lines, 1, (size_t)len, (size_t)1);
  else
    hipLaunchKernelGGL((mnv_softmax_fwd_generic_kernel<MNV_SM_THREADS>), dim3(line_grid(lines, 1)),
                       dim3(MNV_SM_THREADS), 0, s, in, out, len, lines, 1, (size_t)len, (size_t)1);
  return MNV_LAUNCH_STATUS();
}

int softmax_lines_bwd(const float* dy, const float* y, float* dx, int len, int lines,
                      hipStream_t s) {
  bool vec = (len % 4 == 0) && mnv_aligned16(dy) && mnv_aligned16(y) && mnv_aligned16(dx);
  if (vec && len <= MNV_WAVE * 4 * MNV_SM_CACHE)
    hipLaunchKernelGGL((mnv_softmax_bwd_cached_kernel<MNV_WAVE, MNV_SM_CACHE, MNV_SM_THREADS>),
                       dim3(line_grid(lines, 4)), dim3(MNV_SM_THREADS), 0, s, dy, y, dx, len, lines);
  else if (vec && len <= MNV_SM_THREADS * 4 * MNV_SM_WIDE_CACHE)
    hipLaunchKernelGGL((mnv_softmax_bwd_cached_kernel<MNV_SM_THREADS, MNV_SM_WIDE_CACHE, MNV_SM_THREADS>),
                       dim3(line_grid(lines, 1)), dim3(MNV_SM_THREADS), 0, s, dy, y, dx, len, lines);
  else if (vec && len <= MNV_SM_WIDE * 4 * MNV_SM_WIDE_CACHE)
    hipLaunchKernelGGL((mnv_softmax_bwd_cached_kernel<MNV_SM_WIDE, MNV_SM_WIDE_CACHE, MNV_SM_WIDE>),
                       dim3(line_grid(lines, 1)), dim3(MNV_SM_WIDE), 0, s, dy, y, dx, len, lines);
  else if (len <= 1024)
    hipLaunchKernelGGL((mnv_softmax_bwd_generic_kernel<MNV_WAVE>), dim3(line_grid(lines, 4)),
                       dim3(MNV_SM_THREADS), 0, s, dy, y, dx, len, lines, 1, (size_t)len, (size_t)1);
  else
    hipLaunchKernelGGL((mnv_softmax_bwd_generic_kernel<MNV_SM_THREADS>), dim3(line_grid(lines, 1)),
                       dim3(MNV_SM_THREADS), 0, s, dy, y, dx, len, lines, 1, (size_t)len, (size_t)1);
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" {

int mnv_softmax_instance_fwd(const float* bottom, float* top, int num_images, int num_channels,
                             int height, int width, mnv_stream_t stream) {
  long long len;
  if (!bottom || !top || !dims_ok(num_images, num_channels, height, width, &len))
    return MNV_ERR_INVALID;
  return softmax_lines_fwd(bottom, top, (int)len, num_images, mnv_stream(stream));
}

int mnv_softmax_channel_fwd(const float* bottom, float* top, int num_images, int num_channels,
                            int height, int width, mnv_stream_t stream) {
  long long len;
  if (!bottom || !top || !dims_ok(num_images, num_channels, height, width, &len))
    return MNV_ERR_INVALID;
  long long hw = (long long)height * width;
  if (hw == 1) return softmax_lines_fwd(bottom, top, num_channels, num_images, mnv_stream(stream));
  const bool small = num_channels <= MNV_SMC_SMALL_C;
  const long long per_image = (hw + (small ? 63 : 31)) / (small ? 64 : 32);
  if (per_image * num_images > 0x7fffffffLL) return MNV_ERR_INVALID;
  const dim3 grid((unsigned)(per_image * num_images));
  if (small)
    hipLaunchKernelGGL((mnv_softmax_channel_fwd_kernel<64, 4, 16>), grid, dim3(256), 0,
                       mnv_stream(stream), bottom, top, num_channels, (int)hw, (int)per_image);
  else
    hipLaunchKernelGGL((mnv_softmax_channel_fwd_kernel<32, 32, 32>), grid, dim3(1024), 0,
                       mnv_stream(stream), bottom, top, num_channels, (int)hw, (int)per_image);
  return MNV_LAUNCH_STATUS();
}

int mnv_softmax_instance_bwd(const float* top_diff, const float* top, float* bottom_diff,
                             int num_images, int num_channels, int height, int width,
                             mnv_stream_t stream) {
  long long len;
  if (!top_diff || !top || !bottom_diff ||
      !dims_ok(num_images, num_channels, height, width, &len))
    return MNV_ERR_INVALID;
  return softmax_lines_bwd(top_diff, top, bottom_diff, (int)len, num_images, mnv_stream(stream));
}

int mnv_softmax_channel_bwd(const float* top_diff, const float* top, float* bottom_diff,
                            int num_images, int num_channels, int height, int width,
                            mnv_stream_t stream) {
  long long len;
  if (!top_diff || !top || !bottom_diff ||
      !dims_ok(num_images, num_channels, height, width, &len))
    return MNV_ERR_INVALID;
  long long hw = (long long)height * width;
  if (hw == 1)
    return softmax_lines_bwd(top_diff, top, bottom_diff, num_channels, num_images,
                             mnv_stream(stream));
  const bool small = num_channels <= MNV_SMC_SMALL_C;
  const long long per_image = (hw + (small ? 63 : 31)) / (small ? 64 : 32);
  if (per_image * num_images > 0x7fffffffLL) return MNV_ERR_INVALID;
  const dim3 grid((unsigned)(per_image * num_images));
  if (small)
    hipLaunchKernelGGL((mnv_softmax_channel_bwd_kernel<64, 4, 16>), grid, dim3(256), 0,
                       mnv_stream(stream), top_diff, top, bottom_diff, num_channels, (int)hw,
                       (int)per_image);
  else if (num_channels <= 512)
    hipLaunchKernelGGL((mnv_softmax_channel_bwd_kernel<32, 32, 16>), grid, dim3(1024), 0,
                       mnv_stream(stream), top_diff, top, bottom_diff, num_channels, (int)hw,
                       (int)per_image);
  else
    hipLaunchKernelGGL((mnv_softmax_channel_bwd_kernel<32, 32, 32>), grid, dim3(1024), 0,
                       mnv_stream(stream), top_diff, top, bottom_diff, num_channels, (int)hw,
                       (int)per_image);
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
