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
// leaves the window and the one needed for the output (cache hits).  Planes of 512 positions
// and more that do not lie on 64-byte boundaries take variants of the ring kernels whose
// stores are re-cut on those boundaries (lrn_store_recut below).
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

// s^e for s >= 1 through the hardware log2 / exp2 instructions themselves (v_log_f32,
// v_exp_f32: 1 ulp each; relative error of the power ~1e-6).  The library wrappers add range
// fix-ups for denormal arguments and results (five more instructions per value), which
// cannot occur here: s >= 1, and s^e underflows only for |e| log2 s > 126.
__device__ __forceinline__ float pow_ge1(float s, float e) {
  return __builtin_amdgcn_exp2f(e * __builtin_amdgcn_logf(s));
}

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

// ---- stores re-cut on 64-byte boundaries ------------------------------------------------
// An odd plane size (55 x 55) leaves every channel at a different offset from a 64-byte
// boundary, and a wavefront's run of 64 * V floats then begins and ends inside a 64-byte
// sector that a neighbouring wavefront completes later: both write that sector in part, and
// the memory side pays a read-modify-write for each.  Re-cutting the run inside the
// wavefront does not help by itself (the partial sectors at its two ends stay).  What helps
// is ownership by sector: the runs of neighbouring wavefronts overlap by 16 positions
// (a wavefront covers 64 * V positions and advances by 64 * V - 16; the 16 shared positions
// are computed twice), and in every channel a wavefront writes exactly the sectors that
// BEGIN inside the first 64 * V - 16 positions of its run, whole, wherever the sector grid
// falls in that channel.  Measured on 256 x 96 x 55 x 55 with the arithmetic taken out:
// 213 -> 178 us for one tensor read and two written.
// The values travel through a strip of LDS that belongs to the wavefront (a wavefront's LDS
// accesses are executed in order, so no workgroup barrier is needed).  Only the sector that
// holds the first floats of a plane and the one that holds its last floats are written
// element by element.
#define MNV_LRN_STRIP (64 * 4 + 16)  // floats per wavefront and stream
#define MNV_LRN_RECUT_MIN_PLANE 512   // positions per plane from which the re-cut kernels run
template <int V>
struct LrnRecut {
  static constexpr int RUN = 64 * V;        // positions a wavefront covers
  static constexpr int OWN = RUN - 16;      // positions it advances by
  static constexpr int LANES = OWN / 4;     // lanes that store one 16-byte vector
};
// r: floats from the wavefront's first position to the first sector boundary at or after it in
// this channel (wavefront-uniform); pw: first position of the wavefront in its plane;
// voff: the lane's own byte offset (image, position pw + V * lane); soff: channel byte offset.
template <int V, bool NT>
__device__ __forceinline__ void lrn_store_recut(float* strip, int r, mnv_rsrc rs, unsigned voff,
                                                unsigned soff, const float (&val)[V], int lane,
                                                int pw, int hw) {
#pragma unroll
  for (int t = 0; t < V; ++t) strip[V * lane + t] = val[t];
  __builtin_amdgcn_wave_barrier();
  const unsigned vbase = voff - (unsigned)(4 * V * lane);  // byte offset of position pw
  if (lane < LrnRecut<V>::LANES) {
    const int e = r + 4 * lane, t = pw + e;
    if (t < hw) {
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = strip[e + j];
      if (t + 4 <= hw) {
        mnv_f4 v = {o[0], o[1], o[2], o[3]};
        __builtin_amdgcn_raw_buffer_store_b128(
            __builtin_bit_cast(__attribute__((__vector_size__(4 * sizeof(unsigned)))) unsigned, v), rs,
            (int)(vbase + 4u * e), (int)soff, NT ? 2 : 0);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (t + j < hw)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, o[j]), rs,
                                                  (int)(vbase + 4u * (e + j)), (int)soff, 0);
      }
    }
  } else if (pw == 0) {
    // the floats of the plane in front of its first sector boundary
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int e = 4 * (lane - LrnRecut<V>::LANES) + j;
      if (e < r && e < hw)
        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, strip[e]), rs,
                                              (int)(vbase + 4u * e), (int)soff, 0);
    }
  }
  __builtin_amdgcn_wave_barrier();
}

template <int SIZE, int G, int V, bool NT, bool RECUT>
__global__ __launch_bounds__(MNV_LRN_THREADS) void mnv_lrn_fwd_ring_kernel(
    const float* __restrict__ bottom, float* __restrict__ scale, float* __restrict__ top,
    float alpha_over_size, float negative_beta, int channels, int hw, int groups_per_image,
    size_t groups, unsigned bytes, MnvFastDiv d_gpi, int seg_len, int nseg, MnvFastDiv d_groups) {
  static_assert(G % SIZE == 0, "group must be whole windows");
  constexpr int pre_pad = (SIZE - 1) / 2, post_pad = SIZE - pre_pad - 1;
  const mnv_rsrc rin = mnv_make_rsrc(bottom, bytes), rsc = mnv_make_rsrc(scale, bytes),
                 rtop = mnv_make_rsrc(top, bytes);
  const unsigned cstep = (unsigned)hw * 4u;  // bytes from one channel to the next
  __shared__ float strips[RECUT ? 2 * (MNV_LRN_THREADS / 64) * MNV_LRN_STRIP : 1];
  const int lane = threadIdx.x % 64;
  float* const strip_s = strips + (RECUT ? (threadIdx.x / 64) * 2 * MNV_LRN_STRIP : 0);
  float* const strip_t = strip_s + (RECUT ? MNV_LRN_STRIP : 0);
  // floats from a 64-byte boundary to the first element of each output tensor
  const int phase_s = (int)((reinterpret_cast<uintptr_t>(scale) >> 2) & 15u);
  const int phase_t = (int)((reinterpret_cast<uintptr_t>(top) >> 2) & 15u);
  // A thread walks the channels [c0, c1) of one segment for V neighbouring positions: the
  // channel range is cut into nseg segments when the positions alone do not fill the chip
  // (13 x 13 planes with 256 channels); a segment starts its window sum afresh pre_pad
  // channels early.
  // Workgroups never straddle channel segments (the thread columns of a segment are padded to
  // whole workgroups), so the segment, and with it every channel offset, is a scalar: a
  // channel offset that the compiler cannot prove uniform costs a readfirstlane loop around
  // every buffer access.  RECUT: the workgroups of one run of positions (one per segment) are
  // neighbours in launch order; otherwise segments are the slow index.  d_groups divides by
  // nseg (RECUT) or by the workgroups of a segment.
  const int bps = (int)((groups + MNV_LRN_THREADS - 1) / MNV_LRN_THREADS);
  for (int vb = blockIdx.x; vb < bps * nseg; vb += gridDim.x) {
    int seg, blk;
    if (RECUT) {
      blk = mnv_fastdiv(vb, d_groups);
      seg = vb - blk * nseg;
    } else {
      seg = mnv_fastdiv(vb, d_groups);
      blk = vb - seg * bps;
    }
    // RECUT: a "group" is a lane of a wavefront of its plane (groups_per_image = 64 x the
    // wavefronts of a plane), wavefronts advance by OWN positions, image and wavefront are
    // scalars
    const int wave0 = blk * MNV_LRN_THREADS + __builtin_amdgcn_readfirstlane((int)threadIdx.x / 64) * 64;
    const int qq = RECUT ? wave0 + lane : blk * MNV_LRN_THREADS + (int)threadIdx.x;
    if (RECUT ? wave0 >= (int)groups : qq >= (int)groups) continue;
    const int n = RECUT ? mnv_fastdiv(wave0, d_gpi) : mnv_fastdiv(qq, d_gpi);
    const int gi = qq - n * groups_per_image;
    const int pw = RECUT ? (wave0 - n * groups_per_image) / 64 * LrnRecut<V>::OWN : 0;
    const int p0 = RECUT ? pw + V * lane : gi * V;
    const int valid = min(V, hw - p0);
    const unsigned voff = ((unsigned)n * (unsigned)channels * (unsigned)hw + (unsigned)p0) * 4u;
    // float index of the wavefront's first position in channel 0 of its image
    const int wave_first = RECUT ? n * channels * hw + pw : 0;
    const int c0 = seg * seg_len, c1 = min(channels, c0 + seg_len);
    const int h_start = c0 - pre_pad, h_end = min(channels, c1 + post_pad);
    // Two register sets take turns as "current group" and "group being loaded" (the loop is
    // unrolled by two), so that no value is copied from one to the other.
    LrnVec<V> win[SIZE], set_a[G], set_b[G];
#pragma unroll
    for (int u = 0; u < SIZE; ++u)
#pragma unroll
      for (int t = 0; t < V; ++t) win[u].v[t] = 0.f;
    auto fetch = [&](LrnVec<V>(&dst)[G], int h, int u) {
      if (h >= 0 && h < h_end) {
        dst[u] = lrn_load<V>(rin, voff, (unsigned)h * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) dst[u].v[t] = 0.f;
      }
    };
#pragma unroll
    for (int u = 0; u < G; ++u) fetch(set_a, h_start + u, u);
    float accum[V];
#pragma unroll
    for (int t = 0; t < V; ++t) accum[t] = 0.f;
    auto group = [&](LrnVec<V>(&cur)[G], LrnVec<V>(&nxt)[G], int h0) {
#pragma unroll
      for (int u = 0; u < G; ++u) fetch(nxt, h0 + G + u, u);
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
          if (RECUT) {
            const int first = wave_first + c * hw;
            lrn_store_recut<V, NT>(strip_s, (16 - ((first + phase_s) & 15)) & 15, rsc, voff,
                                   (unsigned)c * cstep, s, lane, pw, hw);
            lrn_store_recut<V, NT>(strip_t, (16 - ((first + phase_t) & 15)) & 15, rtop, voff,
                                   (unsigned)c * cstep, o, lane, pw, hw);
          } else {
            lrn_store<V, NT>(rsc, voff, (unsigned)c * cstep, s, valid);
            lrn_store<V, NT>(rtop, voff, (unsigned)c * cstep, o, valid);
          }
        }
      }
    };
    const int h_last = c1 + post_pad;
    for (int h0 = h_start; h0 < h_last; h0 += 2 * G) {
      group(set_a, set_b, h0);
      if (h0 + G < h_last) group(set_b, set_a, h0 + G);
    }
  }
}

template <int SIZE, int G, int V, bool NT, bool RECUT>
__global__ __launch_bounds__(MNV_LRN_THREADS, (SIZE <= 5 && !RECUT) ? 4 : 1) void mnv_lrn_bwd_ring_kernel(
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
  __shared__ float strips[RECUT ? (MNV_LRN_THREADS / 64) * MNV_LRN_STRIP : 1];
  const int lane = threadIdx.x % 64;
  float* const strip = strips + (RECUT ? (threadIdx.x / 64) * MNV_LRN_STRIP : 0);
  const int phase = (int)((reinterpret_cast<uintptr_t>(bottom_diff) >> 2) & 15u);
  // Workgroups never straddle channel segments (the thread columns of a segment are padded to
  // whole workgroups), so the segment, and with it every channel offset, is a scalar: a
  // channel offset that the compiler cannot prove uniform costs a readfirstlane loop around
  // every buffer access.  RECUT: the workgroups of one run of positions (one per segment) are
  // neighbours in launch order; otherwise segments are the slow index.  d_groups divides by
  // nseg (RECUT) or by the workgroups of a segment.
  const int bps = (int)((groups + MNV_LRN_THREADS - 1) / MNV_LRN_THREADS);
  for (int vb = blockIdx.x; vb < bps * nseg; vb += gridDim.x) {
    int seg, blk;
    if (RECUT) {
      blk = mnv_fastdiv(vb, d_groups);
      seg = vb - blk * nseg;
    } else {
      seg = mnv_fastdiv(vb, d_groups);
      blk = vb - seg * bps;
    }
    // RECUT: a "group" is a lane of a wavefront of its plane (groups_per_image = 64 x the
    // wavefronts of a plane), wavefronts advance by OWN positions, image and wavefront are
    // scalars
    const int wave0 = blk * MNV_LRN_THREADS + __builtin_amdgcn_readfirstlane((int)threadIdx.x / 64) * 64;
    const int qq = RECUT ? wave0 + lane : blk * MNV_LRN_THREADS + (int)threadIdx.x;
    if (RECUT ? wave0 >= (int)groups : qq >= (int)groups) continue;
    const int n = RECUT ? mnv_fastdiv(wave0, d_gpi) : mnv_fastdiv(qq, d_gpi);
    const int gi = qq - n * groups_per_image;
    const int pw = RECUT ? (wave0 - n * groups_per_image) / 64 * LrnRecut<V>::OWN : 0;
    const int p0 = RECUT ? pw + V * lane : gi * V;
    const int valid = min(V, hw - p0);
    const unsigned voff = ((unsigned)n * (unsigned)channels * (unsigned)hw + (unsigned)p0) * 4u;
    const int wave_first = RECUT ? n * channels * hw + pw : 0;
    const int c0 = seg * seg_len, c1 = min(channels, c0 + seg_len);  // this thread's outputs
    const int h_start = c0 - pre_pad, h_end = min(channels, c1 + post_pad);
    // rings: ratio = dy*y/scale (the summed quantity), and dy, scale for the output term
    LrnVec<V> rwin[SIZE], dwin[SIZE], swin[SIZE];
    // the next group of channels and the current one, in two register sets that take turns
    // (loop unrolled by two); x is bottom at the output channel
    struct Group {
      LrnVec<V> dy[G], y[G], sc[G], x[G];
    } set_a, set_b;
#pragma unroll
    for (int u = 0; u < SIZE; ++u)
#pragma unroll
      for (int t = 0; t < V; ++t) {
        rwin[u].v[t] = 0.f; dwin[u].v[t] = 0.f; swin[u].v[t] = 1.f;
      }
    auto fetch = [&](Group& g, int h, int u) {
      if (h >= 0 && h < h_end) {
        g.dy[u] = lrn_load<V>(rdy, voff, (unsigned)h * cstep);
        g.y[u] = lrn_load<V>(ry, voff, (unsigned)h * cstep);
        g.sc[u] = lrn_load<V>(rs, voff, (unsigned)h * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) {
          g.dy[u].v[t] = 0.f; g.y[u].v[t] = 0.f; g.sc[u].v[t] = 1.f;
        }
      }
      const int c = h - post_pad;
      if (c >= c0 && c < c1) {
        g.x[u] = lrn_load<V>(rx, voff, (unsigned)c * cstep);
      } else {
#pragma unroll
        for (int t = 0; t < V; ++t) g.x[u].v[t] = 0.f;
      }
    };
#pragma unroll
    for (int u = 0; u < G; ++u) fetch(set_a, h_start + u, u);
    float accum[V];
#pragma unroll
    for (int t = 0; t < V; ++t) accum[t] = 0.f;
    auto group = [&](Group& cur, Group& nxt, int h0) {
#pragma unroll
      for (int u = 0; u < G; ++u) fetch(nxt, h0 + G + u, u);
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int c = h0 + u - post_pad;
        LrnVec<V> r;
#pragma unroll
        for (int t = 0; t < V; ++t) {
          // 0 past the last channel; scale >= 1, and the hardware reciprocal is good to 1 ulp
          r.v[t] = cur.dy[u].v[t] * cur.y[u].v[t] * __builtin_amdgcn_rcpf(cur.sc[u].v[t]);
          accum[t] += r.v[t];
          accum[t] -= rwin[u % SIZE].v[t];
        }
        rwin[u % SIZE] = r; dwin[u % SIZE] = cur.dy[u]; swin[u % SIZE] = cur.sc[u];
        if (c >= c0 && c < c1) {
          const int slot = (u - post_pad + SIZE) % SIZE;
          float o[V];
#pragma unroll
          for (int t = 0; t < V; ++t)
            o[t] = dwin[slot].v[t] * pow_ge1(swin[slot].v[t], negative_beta) -
                   cache_ratio * cur.x[u].v[t] * accum[t];
          if (RECUT)
            lrn_store_recut<V, NT>(strip, (16 - ((wave_first + c * hw + phase) & 15)) & 15, rdx, voff,
                                   (unsigned)c * cstep, o, lane, pw, hw);
          else
            lrn_store<V, false>(rdx, voff, (unsigned)c * cstep, o, valid);
        }
      }
    };
    const int h_last = c1 + post_pad;
    for (int h0 = h_start; h0 < h_last; h0 += 2 * G) {
      group(set_a, set_b, h0);
      if (h0 + G < h_last) group(set_b, set_a, h0 + G);
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

// The re-cut kernels run best on short segments, whose workgroups are neighbours in launch
// order: the workgroups in residence then stream through a compact part of the tensors
// (a few dozen images), much as a plain copy does, and the halo channels a segment re-reads
// were fetched by its neighbour a moment ago.  Measured on 256 x 96 x 55 x 55 (forward, 4 / 8 /
// 16 / 24 segments: 191 / 175 / 157 / 166 us) and 256 x 256 x 27 x 27 (16 / 32 / 43: 125 / 111 /
// 109 us); the backward pass re-reads three tensors per halo channel and pays for the ratio
// of every halo value, so its segments stay longer (4 / 6 / 8 / 16 segments of the first
// shape: 288 / 278 / 287 / 302 us).
void lrn_short_segments(int channels, int len, int* seg_len, int* nseg) {
  *seg_len = std::min(channels, len);
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
  // Planes of 512 positions and more have their stores re-cut on 64-byte boundaries (see
  // lrn_store_recut) unless they lie on such boundaries already; on smaller planes the
  // wavefronts that hang over the end of a plane would idle too many lanes.
  const bool recut = hw >= MNV_LRN_RECUT_MIN_PLANE && (hw % 16 != 0 || ((reinterpret_cast<uintptr_t>(scale) |
                                                     reinterpret_cast<uintptr_t>(top)) & 63u));
  const int gpi = recut ? 64 * ((hw + LrnRecut<V>::OWN - 1) / LrnRecut<V>::OWN) : (hw + V - 1) / V;
  const size_t groups = (size_t)gpi * num_images;
  const bool ring = bytes < 0x80000000ull && (local_size == 3 || local_size == 5 || local_size == 7) &&
                    groups * (size_t)channels < 0x7fffffffull;
  if (ring) {
    int seg_len, nseg;
    lrn_segments(groups, channels, local_size, &seg_len, &nseg);
    if (recut) lrn_short_segments(channels, std::max(6, local_size + 1), &seg_len, &nseg);
    const size_t bps = mnv_ceil_div(groups, MNV_LRN_THREADS);
    const dim3 grid((unsigned)std::min<size_t>(bps * nseg, 4 * MNV_MAX_STREAM_BLOCKS));
    const MnvFastDiv d = mnv_fastdiv_make(gpi), dg = mnv_fastdiv_make(recut ? nseg : (int)bps);
    const bool nt = 3 * bytes >= ((size_t)512 << 20);
#define MNV_LRN_FWD_(SIZE, G, NT, RECUT)                                                           \
  hipLaunchKernelGGL((mnv_lrn_fwd_ring_kernel<SIZE, G, V, NT, RECUT>), grid, block, 0, s, bottom,  \
                     scale, top, aos, -beta, channels, hw, gpi, groups, (unsigned)bytes, d,        \
                     seg_len, nseg, dg)
#define MNV_LRN_FWD(SIZE, G)                                                                        \
  if (recut) {                                                                                      \
    if (nt) MNV_LRN_FWD_(SIZE, G, true, true); else MNV_LRN_FWD_(SIZE, G, false, true);             \
  } else if (nt)                                                                                    \
    MNV_LRN_FWD_(SIZE, G, true, false);                                                             \
  else                                                                                              \
    MNV_LRN_FWD_(SIZE, G, false, false)
    if (local_size == 3) {
      MNV_LRN_FWD(3, 6);
    } else if (local_size == 5) {
      MNV_LRN_FWD(5, 5);
    } else {
      MNV_LRN_FWD(7, 7);
    }
#undef MNV_LRN_FWD
#undef MNV_LRN_FWD_
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
  const bool recut = hw >= MNV_LRN_RECUT_MIN_PLANE && (hw % 16 != 0 || (reinterpret_cast<uintptr_t>(bottom_diff) & 63u));
  const int gpi = recut ? 64 * ((hw + LrnRecut<V>::OWN - 1) / LrnRecut<V>::OWN) : (hw + V - 1) / V;
  const size_t groups = (size_t)gpi * num_images;
  const bool ring = bytes < 0x80000000ull && (local_size == 3 || local_size == 5 || local_size == 7) &&
                    groups * (size_t)channels < 0x7fffffffull;
  if (ring) {
    int seg_len, nseg;
    lrn_segments(groups, channels, local_size, &seg_len, &nseg);
    if (recut) lrn_short_segments(channels, 16, &seg_len, &nseg);
    const size_t bps = mnv_ceil_div(groups, MNV_LRN_THREADS);
    const dim3 grid((unsigned)std::min<size_t>(bps * nseg, 4 * MNV_MAX_STREAM_BLOCKS));
    const MnvFastDiv d = mnv_fastdiv_make(gpi), dg = mnv_fastdiv_make(recut ? nseg : (int)bps);
    const bool nt = 5 * bytes >= ((size_t)512 << 20);
#define MNV_LRN_BWD_(SIZE, G, NT, RECUT)                                                         \
  hipLaunchKernelGGL((mnv_lrn_bwd_ring_kernel<SIZE, G, V, NT, RECUT>), grid, block, 0, s, bottom, \
                     top, scale, top_diff, bottom_diff, -beta, ratio, channels, hw, gpi, groups, \
                     (unsigned)bytes, d, seg_len, nseg, dg)
#define MNV_LRN_BWD(SIZE, G)                                                                     \
  if (recut) {                                                                                   \
    if (nt) MNV_LRN_BWD_(SIZE, G, true, true); else MNV_LRN_BWD_(SIZE, G, false, true);          \
  } else                                                                                         \
    MNV_LRN_BWD_(SIZE, G, false, false)
    if (local_size == 3) {
      MNV_LRN_BWD(3, 6);
    } else if (local_size == 5) {
      MNV_LRN_BWD(5, 5);
    } else {
      MNV_LRN_BWD(7, 7);
    }
#undef MNV_LRN_BWD
#undef MNV_LRN_BWD_
  } else {
    hipLaunchKernelGGL(mnv_lrn_bwd_kernel, dim3(lrn_grid(positions)), block, 0, s, bottom, top, scale,
                       top_diff, bottom_diff, local_size, -beta, ratio, channels, hw, positions,
                       mnv_fastdiv_make(hw));
  }
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
