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
// read twice, the loads of the next channels are issued before the current ones are
// consumed, and a thread handles several neighbouring positions per access.  Other sizes
// (and tensors of 2 GiB or more) take the generic kernels, which re-read the value that
// leaves the window and the one needed for the output (cache hits).  All accesses are
// ordinary: non-temporal 4-byte stores measured 35% slower here.
#include <math.h>

#include <algorithm>

#include "mnv_common.h"

namespace {

// Threads the ring kernels aim for: four rounds of the 256 x 1024 threads the chip holds.
// Measured on 256 x 96 x 55 x 55, 256 x 96 x 27 x 27 and 256 x 256 x 13 x 13: from 2^17
// threads on, the small shapes are at their rate (13 x 13 planes: 4x faster than one thread
// per position column); the largest gains another 5% up to 2^20.
#define MNV_LRN_WANT_THREADS ((size_t)1 << 20)


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
// A thread owns V consecutive positions of one image (V = 4 forward, 2 backward: the
// backward pass keeps four tensors in flight) and reads / writes them with one buffer
// access of 4*V bytes per channel; buffer accesses need only 4-byte alignment, which is
// all an odd plane size leaves.  Its byte offset is fixed and the channel advances through
// the wavefront-uniform scalar offset, so the walk costs no address arithmetic.  A group
// that hangs over the end of its plane reads a few floats of the next channel into lanes
// whose results are dropped, and stores its valid elements one by one.
//
// Slot u of a ring holds the value of channel head with head % SIZE == u; the value that
// leaves the window when channel `head` enters is the one already in slot head % SIZE.
// Slots start at zero, and channels past the end enter as zero: adding or subtracting
// 0*0 leaves the running sum bit-for-bit unchanged, so the partial windows at both ends
// need no special case.  G (a multiple of SIZE) channels are handled per iteration and the
// next G loaded ahead.
template <int V>
struct LrnVec {
  float v[V];
};
template <int V>
__device__ __forceinline__ LrnVec<V> lrn_load(mnv_rsrc r, unsigned voff, unsigned soff);
template <>
__device__ __forceinline__ LrnVec<4> lrn_load<4>(mnv_rsrc r, unsigned voff, unsigned soff) {
  mnv_f4 t = __builtin_bit_cast(mnv_f4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0));
  return LrnVec<4>{{t.x, t.y, t.z, t.w}};
}
template <>
__device__ __forceinline__ LrnVec<2> lrn_load<2>(mnv_rsrc r, unsigned voff, unsigned soff) {
  typedef float f2 __attribute__((ext_vector_type(2)));
  f2 t = __builtin_bit_cast(f2, __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)soff, 0));
  return LrnVec<2>{{t.x, t.y}};
}
// NT: the 16-byte stores bypass the caches (for tensors that cannot stay in the 256 MB
// last-level cache anyway; smaller ones are written through it: 51% -> 66% of HBM peak on
// the norm1 shape, while 256 x 96 x 55 x 55 is 4% faster the other way).
template <int V, bool NT>
__device__ __forceinline__ void lrn_store(mnv_rsrc r, unsigned voff, unsigned soff, const float (&o)[V],
                                          int valid) {
  if (valid == V) {
    if (V == 4) {
      mnv_f4 t = {o[0], o[1], o[2], o[3 % V]};
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, t),
                                             r, (int)voff, (int)soff, NT ? 2 : 0);
    } else {
      typedef float f2 __attribute__((ext_vector_type(2)));
      f2 t = {o[0], o[1]};
      __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(__attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned, t),
                                            r, (int)voff, (int)soff, 0);
    }
  } else {
#pragma unroll
    for (int t = 0; t < V; ++t)
      if (t < valid)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, o[t]), r, (int)(voff + 4u * t),
                                              (int)soff, 0);
  }
}

template <int SIZE, int G, int V, bool NT>
__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_fwd_ring_kernel(
    const float* __restrict__ bottom, float* __restrict__ scale, float* __restrict__ top,
    float alpha_over_size, float negative_beta, int channels, int hw, int groups_per_image,
    size_t groups, unsigned bytes, MnvFastDiv d_gpi, int seg_len, int nseg, MnvFastDiv d_groups) {
  static_assert(G % SIZE == 0, "group must be whole windows");
  constexpr int pre_pad = (SIZE - 1) / 2, post_pad = SIZE - pre_pad - 1;
  const mnv_rsrc rin = mnv_make_rsrc(bottom, bytes), rsc = mnv_make_rsrc(scale, bytes),
                 rtop = mnv_make_rsrc(top, bytes);
  const unsigned cstep = (unsigned)hw * 4u;  // bytes from one channel to the next
  // A thread walks the channels [c0, c1) of one segment for V neighbouring positions: the
  // channel range is cut into nseg segments when the positions alone do not fill the chip
  // (13 x 13 planes with 256 channels); a segment starts its window sum afresh pre_pad
  // channels early.
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < groups * nseg;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int seg = mnv_fastdiv((int)q, d_groups), qq = (int)q - seg * (int)groups;
    const int n = mnv_fastdiv(qq, d_gpi), p0 = (qq - n * groups_per_image) * V;
    const int valid = min(V, hw - p0);
    const unsigned voff = ((unsigned)n * (unsigned)channels * (unsigned)hw + (unsigned)p0) * 4u;
    const int c0 = seg * seg_len, c1 = min(channels, c0 + seg_len);
    const int h_start = c0 - pre_pad, h_end = min(channels, c1 + post_pad);
    LrnVec<V> win[SIZE], nxt[G];
#pragma unroll
    for (int u = 0; u < SIZE; ++u)
#pragma unroll
      for (int t = 0; t < V; ++t) win[u].v[t] = 0.f;
    auto fetch = [&](int h, int u) {
      if (h >= 0 && h < h_end) {
        nxt[u] = lrn_load<V>(rin, voff, (unsigned)h * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) nxt[u].v[t] = 0.f;
      }
    };
#pragma unroll
    for (int u = 0; u < G; ++u) fetch(h_start + u, u);
    float accum[V];
#pragma unroll
    for (int t = 0; t < V; ++t) accum[t] = 0.f;
    for (int h0 = h_start; h0 < c1 + post_pad; h0 += G) {
      LrnVec<V> cur[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        cur[u] = nxt[u];
        fetch(h0 + G + u, u);
      }
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int c = h0 + u - post_pad;
#pragma unroll
        for (int t = 0; t < V; ++t) {
          accum[t] += cur[u].v[t] * cur[u].v[t];
          accum[t] -= win[u % SIZE].v[t] * win[u % SIZE].v[t];
        }
        win[u % SIZE] = cur[u];
        if (c >= c0 && c < c1) {
          float s[V], o[V];
#pragma unroll
          for (int t = 0; t < V; ++t) {
            s[t] = 1.f + accum[t] * alpha_over_size;
            o[t] = win[(u - post_pad + SIZE) % SIZE].v[t] * pow_ge1(s[t], negative_beta);
          }
          lrn_store<V, NT>(rsc, voff, (unsigned)c * cstep, s, valid);
          lrn_store<V, NT>(rtop, voff, (unsigned)c * cstep, o, valid);
        }
      }
    }
  }
}

template <int SIZE, int G, int V>
__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_bwd_ring_kernel(
    const float* __restrict__ bottom, const float* __restrict__ top,
    const float* __restrict__ scale, const float* __restrict__ top_diff,
    float* __restrict__ bottom_diff, float negative_beta, float cache_ratio, int channels, int hw,
    int groups_per_image, size_t groups, unsigned bytes, MnvFastDiv d_gpi, int seg_len, int nseg,
    MnvFastDiv d_groups) {
  static_assert(G % SIZE == 0, "group must be whole windows");
  constexpr int pre_pad = SIZE - (SIZE + 1) / 2, post_pad = SIZE - pre_pad - 1;
  const mnv_rsrc rx = mnv_make_rsrc(bottom, bytes), ry = mnv_make_rsrc(top, bytes),
                 rs = mnv_make_rsrc(scale, bytes), rdy = mnv_make_rsrc(top_diff, bytes),
                 rdx = mnv_make_rsrc(bottom_diff, bytes);
  const unsigned cstep = (unsigned)hw * 4u;
  for (size_t q = (size_t)blockIdx.x * MNV_LRN_THREADS + threadIdx.x; q < groups * nseg;
       q += (size_t)gridDim.x * MNV_LRN_THREADS) {
    const int seg = mnv_fastdiv((int)q, d_groups), qq = (int)q - seg * (int)groups;
    const int n = mnv_fastdiv(qq, d_gpi), p0 = (qq - n * groups_per_image) * V;
    const int valid = min(V, hw - p0);
    const unsigned voff = ((unsigned)n * (unsigned)channels * (unsigned)hw + (unsigned)p0) * 4u;
    const int c0 = seg * seg_len, c1 = min(channels, c0 + seg_len);  // this thread's outputs
    const int h_start = c0 - pre_pad, h_end = min(channels, c1 + post_pad);
    // rings: ratio = dy*y/scale (the summed quantity), and dy, scale for the output term
    LrnVec<V> rwin[SIZE], dwin[SIZE], swin[SIZE];
    LrnVec<V> ndy[G], ny[G], nsc[G], nx[G];  // next group; nx is bottom at the output channel
#pragma unroll
    for (int u = 0; u < SIZE; ++u)
#pragma unroll
      for (int t = 0; t < V; ++t) {
        rwin[u].v[t] = 0.f; dwin[u].v[t] = 0.f; swin[u].v[t] = 1.f;
      }
    auto fetch = [&](int h, int u) {
      if (h >= 0 && h < h_end) {
        ndy[u] = lrn_load<V>(rdy, voff, (unsigned)h * cstep);
        ny[u] = lrn_load<V>(ry, voff, (unsigned)h * cstep);
        nsc[u] = lrn_load<V>(rs, voff, (unsigned)h * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) {
          ndy[u].v[t] = 0.f; ny[u].v[t] = 0.f; nsc[u].v[t] = 1.f;
        }
      }
      const int c = h - post_pad;
      if (c >= c0 && c < c1) {
        nx[u] = lrn_load<V>(rx, voff, (unsigned)c * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) nx[u].v[t] = 0.f;
      }
    };
#pragma unroll
    for (int u = 0; u < G; ++u) fetch(h_start + u, u);
    float accum[V];
#pragma unroll
    for (int t = 0; t < V; ++t) accum[t] = 0.f;
    for (int h0 = h_start; h0 < c1 + post_pad; h0 += G) {
      LrnVec<V> cdy[G], cy[G], csc[G], cx[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        cdy[u] = ndy[u]; cy[u] = ny[u]; csc[u] = nsc[u]; cx[u] = nx[u];
        fetch(h0 + G + u, u);
      }
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int c = h0 + u - post_pad;
        LrnVec<V> r;
#pragma unroll
        for (int t = 0; t < V; ++t) {
          r.v[t] = cdy[u].v[t] * cy[u].v[t] / csc[u].v[t];  // 0 past the last channel
          accum[t] += r.v[t];
          accum[t] -= rwin[u % SIZE].v[t];
        }
        rwin[u % SIZE] = r; dwin[u % SIZE] = cdy[u]; swin[u % SIZE] = csc[u];
        if (c >= c0 && c < c1) {
          const int slot = (u - post_pad + SIZE) % SIZE;
          float o[V];
#pragma unroll
          for (int t = 0; t < V; ++t)
            o[t] = dwin[slot].v[t] * pow_ge1(swin[slot].v[t], negative_beta) -
                   cache_ratio * cx[u].v[t] * accum[t];
          lrn_store<V, false>(rdx, voff, (unsigned)c * cstep, o, valid);
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

// Channel segments per thread column: enough threads for every SIMD to hold several
// wavefronts, segments no shorter than four windows (a segment re-reads size - 1
// channels of its neighbours).
void lrn_segments(size_t groups, int channels, int size, int* seg_len, int* nseg) {
  const size_t want_threads = MNV_LRN_WANT_THREADS;
  size_t n = groups >= want_threads ? 1 : (want_threads + groups - 1) / groups;
  const size_t max_n = (size_t)std::max(1, channels / (4 * size));
  if (n > max_n) n = max_n;
  *seg_len = (int)((channels + n - 1) / n);
  *nseg = (channels + *seg_len - 1) / *seg_len;
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
  const dim3 block(MNV_LRN_THREADS);
  hipStream_t s = mnv_stream(stream);
  const float aos = alpha / local_size;
  const size_t bytes = positions * channels * sizeof(float);
  constexpr int V = 4;
  const int gpi = (hw + V - 1) / V;
  const size_t groups = (size_t)gpi * num_images;
  const bool ring = bytes < 0x80000000ull && (local_size == 3 || local_size == 5 || local_size == 7);
  if (ring) {
    int seg_len, nseg;
    lrn_segments(groups, channels, local_size, &seg_len, &nseg);
    const dim3 grid(lrn_grid(groups * nseg));
    const MnvFastDiv d = mnv_fastdiv_make(gpi), dg = mnv_fastdiv_make((int)groups);
    const bool nt = 3 * bytes >= ((size_t)512 << 20);
#define MNV_LRN_FWD(SIZE, G)                                                                        \
  if (nt)                                                                                           \
    hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<SIZE, G, V, true>), grid, block, 0, s, bottom,      \
                       scale, top, aos, -beta, channels, hw, gpi, groups, (unsigned)bytes, d,       \
                       seg_len, nseg, dg);                                                          \
  else                                                                                              \
    hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<SIZE, G, V, false>), grid, block, 0, s, bottom,     \
                       scale, top, aos, -beta, channels, hw, gpi, groups, (unsigned)bytes, d,       \
                       seg_len, nseg, dg)
    if (local_size == 3) {
      MNV_LRN_FWD(3, 6);
    } else if (local_size == 5) {
      MNV_LRN_FWD(5, 5);
    } else {
      MNV_LRN_FWD(7, 7);
    }
#undef MNV_LRN_FWD
  } else {
    hipLaunchKernelGGL(mnv_lrn_fwd_kernel, dim3(lrn_grid(positions)), block, 0, s, bottom, scale, top,
                       local_size, aos, -beta, channels, hw, positions, mnv_fastdiv_make(hw));
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
  const dim3 block(MNV_LRN_THREADS);
  hipStream_t s = mnv_stream(stream);
  const float ratio = (float)(2. * alpha * beta / local_size);
  const size_t bytes = positions * channels * sizeof(float);
  constexpr int V = 2;
  const int gpi = (hw + V - 1) / V;
  const size_t groups = (size_t)gpi * num_images;
  const bool ring = bytes < 0x80000000ull && (local_size == 3 || local_size == 5 || local_size == 7);
  if (ring) {
    int seg_len, nseg;
    lrn_segments(groups, channels, local_size, &seg_len, &nseg);
    const dim3 grid(lrn_grid(groups * nseg));
    const MnvFastDiv d = mnv_fastdiv_make(gpi), dg = mnv_fastdiv_make((int)groups);
#define MNV_LRN_BWD(SIZE, G)                                                                     \
  hipLaunchKernelGGL((mnv_lrn_bwd_ring_kernel<SIZE, G, V>), grid, block, 0, s, bottom, top, scale, \
                     top_diff, bottom_diff, -beta, ratio, channels, hw, gpi, groups,             \
                     (unsigned)bytes, d, seg_len, nseg, dg)
    if (local_size == 3) MNV_LRN_BWD(3, 6);
    else if (local_size == 5) MNV_LRN_BWD(5, 5);
    else MNV_LRN_BWD(7, 7);
#undef MNV_LRN_BWD
  } else {
    hipLaunchKernelGGL(mnv_lrn_bwd_kernel, dim3(lrn_grid(positions)), block, 0, s, bottom, top, scale,
                       top_diff, bottom_diff, local_size, -beta, ratio, channels, hw, positions,
                       mnv_fastdiv_make(hw));
  }
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
