// Local response normalisation across channels, forward and backward, on an image batch
// {W,H,C,N} (reference kernels minerva/op/impl/cuda/cuda_kernel.h:223-331, launchers
// minerva/op/impl/cuda/cuda_perform.cu:643-667):
//   scale[n,c,p] = 1 + alpha/size * sum_{c' in window(c)} bottom[n,c',p]^2
//   top          = bottom * scale^(-beta)
//   bottom_diff  = top_diff * scale^(-beta)
//                  - 2*alpha*beta/size * bottom * sum_{c' in window'(c)} top_diff*top/scale
// window(c) = [c - pre_pad, c + post_pad] clipped to the channels, pre_pad = (size-1)/2 forward
// and size - (size+1)/2 backward (the adjoint window; the same for odd sizes).
// Roofline: HBM bandwidth; forward moves 12 bytes per element (bottom in, scale and top
// out), backward 20 (bottom, top, scale, top_diff in, bottom_diff out).
//
// A thread owns one (image, position) and walks its channels, which are H*W floats apart, so
// every access of a wavefront is 256 contiguous bytes.  The window sum is the reference's
// running sum (add the entering channel, then subtract the leaving one, in fp32), kept in
// a register.  For the common window sizes (3, 5, 7) the walk is unrolled by the window size:
// the last `size` values then sit in a register ring with compile-time indices, so nothing is
// read twice, and the loads of the next `size` channels are issued before the current ones
// are consumed.  Other sizes take the generic kernels, which re-read the value that leaves
// the window and the one needed for the output (cache hits).  All accesses are ordinary:
// non-temporal 4-byte stores measured 35% slower here.
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_LRN_THREADS 256

// s^e for s >= 1 through the hardware log2 / exp2: relative error ~1e-6
__device__ __forceinline__ float pow_ge1(float s, float e) { return __expf(e * __logf(s)); }

__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_fwd_kernel(
    const float* __restrict__ bottom, float* __restrict__ scale, float* __restrict__ top,
    int size, float alpha_over_size, float negative_beta, int channels, int hw, size_t positions,
    MnvFastDiv d_hw) {
  const int pre_pad = (size - 1) / 2, post_pad = size - pre_pad - 1;
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < positions;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int n = mnv_fastdiv((int)q, d_hw), p = (int)q - n * hw;
    const size_t base = (size_t)n * channels * hw + p;
    const float* in = bottom + base;
    float accum = 0.f;
    for (int head = 0; head < channels + post_pad; ++head) {
      if (head < channels) {
        const float v = in[(size_t)head * hw];
        accum += v * v;
      }
      if (head >= size) {
        const float u = in[(size_t)(head - size) * hw];
        accum -= u * u;
      }
      const int c = head - post_pad;
      if (c >= 0) {
        const float s = 1.f + accum * alpha_over_size;
        scale[base + (size_t)c * hw] = s;
        top[base + (size_t)c * hw] = in[(size_t)c * hw] * pow_ge1(s, negative_beta);
      }
    }
  }
}

__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_bwd_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top,
    const float* __restrict__ scale, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, int size, float negative_beta, float cache_ratio,
    int channels, int hw, size_t positions, MnvFastDiv d_hw) {
  const int pre_pad = size - (size + 1) / 2, post_pad = size - pre_pad - 1;
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < positions;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int n = mnv_fastdiv((int)q, d_hw), p = (int)q - n * hw;
    const size_t base = (size_t)n * channels * hw + p;
    const float* x = bottom + base;
    const float* y = top + base;
    const float* sc = scale + base;
    const float* dy = top_diff + base;
    float accum = 0.f;
    for (int head = 0; head < channels + post_pad; ++head) {
      if (head < channels) {
        const size_t o = (size_t)head * hw;
        accum += dy[o] * y[o] / sc[o];
      }
      if (head >= size) {
        const size_t o = (size_t)(head - size) * hw;
        accum -= dy[o] * y[o] / sc[o];
      }
      const int c = head - post_pad;
      if (c >= 0) {
        const size_t o = (size_t)c * hw;
        bottom_diff[base + o] = dy[o] * pow_ge1(sc[o], negative_beta) - cache_ratio * x[o] * accum;
      }
    }
  }
}

// ---- window size known at compile time ---------------------------------------------
// Slot u of a ring holds the value of channel head with head % SIZE == u; the value that
// leaves the window when channel `head` enters is the one already in slot head % SIZE.
// Slots start at zero, and channels past the end enter as zero: adding or subtracting
// 0*0 leaves the running sum bit-for-bit unchanged, so the partial windows at both ends
// need no special case.
// G = a multiple of SIZE channels are handled per iteration and the next G loaded ahead: a
// thread keeps G 4-byte loads in flight, which is what it takes to cover the memory latency.
template <int SIZE, int G>
__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_fwd_ring_kernel(
    const float* __restrict__ bottom, float* __restrict__ scale, float* __restrict__ top,
    float alpha_over_size, float negative_beta, int channels, int hw, size_t positions,
    MnvFastDiv d_hw) {
  constexpr int pre_pad = (SIZE - 1) / 2, post_pad = SIZE - pre_pad - 1;
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < positions;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int n = mnv_fastdiv((int)q, d_hw), p = (int)q - n * hw;
    const size_t base = (size_t)n * channels * hw + p;
    const float* in = bottom + base;
    static_assert(G % SIZE == 0, "group must be whole windows");
    float win[SIZE], nxt[G];
#pragma unroll
    for (int u = 0; u < SIZE; ++u) win[u] = 0.f;
#pragma unroll
    for (int u = 0; u < G; ++u) nxt[u] = u < channels ? in[(size_t)u * hw] : 0.f;
    float accum = 0.f;
    for (int h0 = 0; h0 < channels + post_pad; h0 += G) {
      float cur[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        cur[u] = nxt[u];
        const int h = h0 + G + u;
        nxt[u] = h < channels ? in[(size_t)h * hw] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int head = h0 + u;
        accum += cur[u] * cur[u];
        accum -= win[u % SIZE] * win[u % SIZE];
        win[u % SIZE] = cur[u];
        const int c = head - post_pad;
        if (c >= 0 && c < channels) {
          const float s = 1.f + accum * alpha_over_size;
          const float self = win[(u - post_pad + SIZE) % SIZE];
          scale[base + (size_t)c * hw] = s;
          top[base + (size_t)c * hw] = self * pow_ge1(s, negative_beta);
        }
      }
    }
  }
}

template <int SIZE, int G>
__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_bwd_ring_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top,
    const float* __restrict__ scale, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, float negative_beta, float cache_ratio, int channels, int hw,
    size_t positions, MnvFastDiv d_hw) {
  constexpr int pre_pad = SIZE - (SIZE + 1) / 2, post_pad = SIZE - pre_pad - 1;
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < positions;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int n = mnv_fastdiv((int)q, d_hw), p = (int)q - n * hw;
    const size_t base = (size_t)n * channels * hw + p;
    const float* x = bottom + base;
    const float* y = top + base;
    const float* sc = scale + base;
    const float* dy = top_diff + base;
    // rings: ratio = dy*y/scale (the summed quantity), and dy, scale for the output term
    static_assert(G % SIZE == 0, "group must be whole windows");
    float rwin[SIZE], dwin[SIZE], swin[SIZE];
    float ndy[G], ny[G], nsc[G], nx[G];  // next group; nx is bottom at the output channel
#pragma unroll
    for (int u = 0; u < SIZE; ++u) {
      rwin[u] = 0.f; dwin[u] = 0.f; swin[u] = 1.f;
    }
#pragma unroll
    for (int u = 0; u < G; ++u) {
      const bool in_range = u < channels;
      ndy[u] = in_range ? dy[(size_t)u * hw] : 0.f;
      ny[u] = in_range ? y[(size_t)u * hw] : 0.f;
      nsc[u] = in_range ? sc[(size_t)u * hw] : 1.f;
      const int c = u - post_pad;
      nx[u] = (c >= 0 && c < channels) ? x[(size_t)c * hw] : 0.f;
    }
    float accum = 0.f;
    for (int h0 = 0; h0 < channels + post_pad; h0 += G) {
      float cdy[G], cy[G], csc[G], cx[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        cdy[u] = ndy[u]; cy[u] = ny[u]; csc[u] = nsc[u]; cx[u] = nx[u];
        const int h = h0 + G + u;
        const bool in_range = h < channels;
        ndy[u] = in_range ? dy[(size_t)h * hw] : 0.f;
        ny[u] = in_range ? y[(size_t)h * hw] : 0.f;
        nsc[u] = in_range ? sc[(size_t)h * hw] : 1.f;
        const int c = h - post_pad;
        nx[u] = (c >= 0 && c < channels) ? x[(size_t)c * hw] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int head = h0 + u;
        const float r = cdy[u] * cy[u] / csc[u];  // 0 past the last channel
        accum += r;
        accum -= rwin[u % SIZE];
        rwin[u % SIZE] = r; dwin[u % SIZE] = cdy[u]; swin[u % SIZE] = csc[u];
        const int c = head - post_pad;
        if (c >= 0 && c < channels) {
          const int slot = (u - post_pad + SIZE) % SIZE;
          const float out = dwin[slot] * pow_ge1(swin[slot], negative_beta) - cache_ratio * cx[u] * accum;
          bottom_diff[base + (size_t)c * hw] = out;
        }
      }
    }
  }
}

int check_dims(int size, int n, int c, int h, int w, size_t* positions, int* hw) {
  if (size <= 0 || n <= 0 || c <= 0 || h <= 0 || w <= 0) return MNV_ERR_INVALID;
  long long plane = (long long)h * w, pos = plane * n;
  if (plane > 0x7fffffffLL || pos > 0x7fffffffLL || pos * c > 0x7fffffffLL) return MNV_ERR_INVALID;
  *positions = (size_t)pos;
  *hw = (int)plane;
  return MNV_OK;
}

unsigned lrn_grid(size_t positions) {
  size_t blocks = mnv_ceil_div(positions, MNV_LRN_THREADS);
  if (blocks > 4 * MNV_MAX_STREAM_BLOCKS) blocks = 4 * MNV_MAX_STREAM_BLOCKS;
  return (unsigned)blocks;
}

}  // namespace

extern "C" {

int mnv_lrn_fwd(const float* bottom, float* scale, float* top, int local_size, float alpha,
                float beta, int num_images, int channels, int height, int width,
                mnv_stream_t stream) {
  if (!bottom || !scale || !top) return MNV_ERR_INVALID;
  size_t positions;
  int hw;
  int rc = check_dims(local_size, num_images, channels, height, width, &positions, &hw);
  if (rc) return rc;
  const dim3 grid(lrn_grid(positions)), block(MNV_LRN_THREADS);
  hipStream_t s = mnv_stream(stream);
  const float aos = alpha / local_size;
  const MnvFastDiv d = mnv_fastdiv_make(hw);
  switch (local_size) {
    case 3:
      hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<3, 18>), grid, block, 0, s, bottom, scale, top, aos,
                         -beta, channels, hw, positions, d);
      break;
    case 5:
      hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<5, 20>), grid, block, 0, s, bottom, scale, top, aos,
                         -beta, channels, hw, positions, d);
      break;
    case 7:
      hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<7, 21>), grid, block, 0, s, bottom, scale, top, aos,
                         -beta, channels, hw, positions, d);
      break;
    default:
      hipLaunchKernelGGL(mnv_lrn_fwd_kernel, grid, block, 0, s, bottom, scale, top, local_size,
                         aos, -beta, channels, hw, positions, d);
  }
  return MNV_LAUNCH_STATUS();
}

int mnv_lrn_bwd(const float* bottom, const float* top, const float* scale, const float* top_diff,
                float* bottom_diff, int local_size, float alpha, float beta, int num_images,
                int channels, int height, int width, mnv_stream_t stream) {
  if (!bottom || !top || !scale || !top_diff || !bottom_diff) return MNV_ERR_INVALID;
  size_t positions;
  int hw;
  int rc = check_dims(local_size, num_images, channels, height, width, &positions, &hw);
  if (rc) return rc;
  const dim3 grid(lrn_grid(positions)), block(MNV_LRN_THREADS);
  hipStream_t s = mnv_stream(stream);
  const float ratio = (float)(2. * alpha * beta / local_size);
  const MnvFastDiv d = mnv_fastdiv_make(hw);
  switch (local_size) {
    case 3:
      hipLaunchKernelGGL((mnv_lrn_bwd_ring_kernel<3, 9>), grid, block, 0, s, bottom, top, scale,
                         top_diff, bottom_diff, -beta, ratio, channels, hw, positions, d);
      break;
    case 5:
      hipLaunchKernelGGL((mnv_lrn_bwd_ring_kernel<5, 10>), grid, block, 0, s, bottom, top, scale,
                         top_diff, bottom_diff, -beta, ratio, channels, hw, positions, d);
      break;
    case 7:
      hipLaunchKernelGGL((mnv_lrn_bwd_ring_kernel<7, 14>), grid, block, 0, s, bottom, top, scale,
                         top_diff, bottom_diff, -beta, ratio, channels, hw, positions, d);
      break;
    default:
      hipLaunchKernelGGL(mnv_lrn_bwd_kernel, grid, block, 0, s, bottom, top, scale, top_diff,
                         bottom_diff, local_size, -beta, ratio, channels, hw, positions, d);
  }
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
