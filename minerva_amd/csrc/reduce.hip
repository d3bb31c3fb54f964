// Reductions of a column-major {m,n} matrix: sum / max along either dimension,
// arg-max along either dimension, and the convolution bias gradient.
// Roofline: HBM bandwidth, 4 algorithmic bytes per input element.
//
// Reference semantics (minerva/op/impl/basic.cpp:189-217, 369-398): a left fold in
// ascending index order that starts from the first element; max / arg-max use a
// strict '<', so the first occurrence of the maximum wins and a NaN is never
// selected unless it is the first element.  Max and arg-max reproduce that
// exactly under any parallel order by reducing (value, index) pairs: the larger
// value wins, equal values keep the lower index (so the bits of a +0 / -0 tie are
// the reference's), NaNs are skipped, and a NaN in position 0 is restored at the
// end.  Sums are tree-ordered (fp32), which differs from the sequential fold only
// in rounding.
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_NONE 0x7fffffff

struct SumAcc {
  static constexpr int ROW_UNROLL = 2;  // columns in flight per thread in the row reducer
  float s;
  __device__ void init() { s = 0.f; }
  __device__ void push(float v, int) { s += v; }
  __device__ void merge(const SumAcc& o) { s += o.s; }
  __device__ SumAcc shfl_down(int off) const {
    SumAcc r;
    r.s = __shfl_down(s, off, MNV_WAVE);
    return r;
  }
  // first = element 0 of the reduced line (only the pair reducers need it)
  __device__ float result_value(float) const { return s; }
};

struct ArgAcc {
  static constexpr int ROW_UNROLL = 4;
  float v;
  int idx;
  __device__ void init() {
    v = -INFINITY;
    idx = MNV_NONE;
  }
  // Elements reach one accumulator in ascending index order.
  __device__ void push(float x, int i) {
    bool take = (idx == MNV_NONE) ? (x == x) : (x > v);
    if (take) {
      v = x;
      idx = i;
    }
  }
  __device__ void merge(const ArgAcc& o) {
    bool take = (o.idx != MNV_NONE) &&
                (idx == MNV_NONE || o.v > v || (o.v == v && o.idx < idx));
    if (take) {
      v = o.v;
      idx = o.idx;
    }
  }
  __device__ ArgAcc shfl_down(int off) const {
    ArgAcc r;
    r.v = __shfl_down(v, off, MNV_WAVE);
    r.idx = __shfl_down(idx, off, MNV_WAVE);
    return r;
  }
  __device__ float result_value(float first) const { return (first != first) ? first : v; }
  __device__ float result_index(float first) const {
    return (first != first || idx == MNV_NONE) ? 0.f : (float)idx;
  }
};

// What a reducer writes.
struct EmitValue {
  template <class Acc>
  __device__ static float get(const Acc& a, float first) { return a.result_value(first); }
};
struct EmitIndex {
  __device__ static float get(const ArgAcc& a, float first) { return a.result_index(first); }
};

// ---------------------------------------------------------------------------
// Along dimension 0: each of the n columns is m contiguous floats.
// GROUP threads (one wavefront, or the whole 256-thread workgroup) share a column.
// ---------------------------------------------------------------------------
#define MNV_RC_THREADS 256

template <class Acc, class Emit, int GROUP, bool VEC4, bool NT>
__global__ __launch_bounds__(MNV_RC_THREADS) void mnv_reduce_col_kernel(
    const float* __restrict__ in, float* __restrict__ out, int m, int n) {
  constexpr int COLS = MNV_RC_THREADS / GROUP;
  __shared__ Acc part[MNV_RC_THREADS / MNV_WAVE];
  const int g = threadIdx.x / GROUP;
  const int t = threadIdx.x % GROUP;
  for (int c = blockIdx.x * COLS + g; c < n; c += gridDim.x * COLS) {
    const float* col = in + (size_t)c * m;
    Acc acc;
    acc.init();
    if (VEC4) {
      const mnv_f4* col4 = reinterpret_cast<const mnv_f4*>(col);
      const int m4 = m >> 2;
      int i = t;
      // two independent 16-byte loads in flight per thread
      for (; i + GROUP < m4; i += 2 * GROUP) {
        mnv_f4 a = mnv_ldx4<NT>(col4 + i), b = mnv_ldx4<NT>(col4 + i + GROUP);
        acc.push(a.x, 4 * i); acc.push(a.y, 4 * i + 1); acc.push(a.z, 4 * i + 2); acc.push(a.w, 4 * i + 3);
        int j = i + GROUP;
        acc.push(b.x, 4 * j); acc.push(b.y, 4 * j + 1); acc.push(b.z, 4 * j + 2); acc.push(b.w, 4 * j + 3);
      }
      if (i < m4) {
        mnv_f4 a = mnv_ldx4<NT>(col4 + i);
        acc.push(a.x, 4 * i); acc.push(a.y, 4 * i + 1); acc.push(a.z, 4 * i + 2); acc.push(a.w, 4 * i + 3);
      }
    } else {
      for (int i = t; i < m; i += GROUP) acc.push(col[i], i);
    }
#pragma unroll
    for (int off = MNV_WAVE / 2; off > 0; off >>= 1) acc.merge(acc.shfl_down(off));
    if (GROUP > MNV_WAVE) {
      const int w = threadIdx.x / MNV_WAVE;
      if ((threadIdx.x % MNV_WAVE) == 0) part[w] = acc;
      __syncthreads();
      if (threadIdx.x == 0) {
        for (int q = 1; q < MNV_RC_THREADS / MNV_WAVE; ++q) acc.merge(part[q]);
        out[c] = Emit::get(acc, col[0]);
      }
      __syncthreads();
    } else if (t == 0) {
      out[c] = Emit::get(acc, col[0]);
    }
  }
}

template <class Acc, class Emit>
int launch_reduce_col(const float* in, float* out, int m, int n, mnv_stream_t stream) {
  if (n == 0) return MNV_OK;
  if (!in || !out || m <= 0 || n < 0) return MNV_ERR_INVALID;
  hipStream_t s = mnv_stream(stream);
  bool vec4 = (m % 4 == 0) && mnv_aligned16(in);
  const bool big = (size_t)m * n * sizeof(float) >= MNV_PAST_CACHE_BYTES;
  if (m > 2048) {
    unsigned grid = (unsigned)(n < 65536 ? n : 65536);
    if (vec4 && big)
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_RC_THREADS, true, true>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
    else if (vec4)
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_RC_THREADS, true, false>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
    else
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_RC_THREADS, false, false>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
  } else {
    size_t blocks = mnv_ceil_div((size_t)n, MNV_RC_THREADS / MNV_WAVE);
    unsigned grid = (unsigned)(blocks < 65536 ? blocks : 65536);
    if (vec4 && big)
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_WAVE, true, true>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
    else if (vec4)
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_WAVE, true, false>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
    else
      hipLaunchKernelGGL((mnv_reduce_col_kernel<Acc, Emit, MNV_WAVE, false, false>), dim3(grid),
                         dim3(MNV_RC_THREADS), 0, s, in, out, m, n);
  }
  return MNV_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------
// Along dimension 1: out[r] = reduce_c in[r + c*m] (stride m between elements).
// A workgroup owns RL*W consecutive rows (128 contiguous bytes per column) and
// splits the columns over CG thread groups; partial results meet in LDS.
// ---------------------------------------------------------------------------
template <class Acc, class Emit, int RL, int CG, bool VEC4, bool NT>
__global__ __launch_bounds__(RL* CG) void mnv_reduce_row_kernel(const float* __restrict__ in,
                                                                float* __restrict__ out, int m,
                                                                int n) {
  constexpr int W = VEC4 ? 4 : 1;
  constexpr int ROWS = RL * W;
  __shared__ Acc part[CG][ROWS + 1];
  const int rl = threadIdx.x % RL;
  const int cg = threadIdx.x / RL;
  const int r0 = blockIdx.x * ROWS + rl * W;
  Acc acc[W];
#pragma unroll
  for (int q = 0; q < W; ++q) acc[q].init();
  if (r0 < m) {
    if (VEC4) {
      // several columns in flight per thread: with one workgroup per 32 rows there are few
      // wavefronts per SIMD, and the loads of a thread are what keeps HBM busy (measured:
      // four for the (value, index) pairs, 4.9 -> 6.0 TB/s; two for sums, where four lose 7%)
      constexpr int U = Acc::ROW_UNROLL;
      int c = cg;
      for (; c + (U - 1) * CG < n; c += U * CG) {
        mnv_f4 v[U];
#pragma unroll
        for (int u = 0; u < U; ++u)
          v[u] = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(in + (size_t)(c + u * CG) * m + r0));
#pragma unroll
        for (int u = 0; u < U; ++u) {
          acc[0].push(v[u].x, c + u * CG); acc[1 % W].push(v[u].y, c + u * CG);
          acc[2 % W].push(v[u].z, c + u * CG); acc[3 % W].push(v[u].w, c + u * CG);
        }
      }
      for (; c < n; c += CG) {
        mnv_f4 a = mnv_ldx4<NT>(reinterpret_cast<const mnv_f4*>(in + (size_t)c * m + r0));
        acc[0].push(a.x, c); acc[1 % W].push(a.y, c); acc[2 % W].push(a.z, c); acc[3 % W].push(a.w, c);
      }
    } else {
      for (int c = cg; c < n; c += CG) acc[0].push(in[(size_t)c * m + r0], c);
    }
  }
#pragma unroll
  for (int q = 0; q < W; ++q) part[cg][rl * W + q] = acc[q];
  __syncthreads();
  for (int sft = CG / 2; sft > 0; sft >>= 1) {
    if (cg < sft) {
#pragma unroll
      for (int q = 0; q < W; ++q) {
        Acc a = part[cg][rl * W + q];
        a.merge(part[cg + sft][rl * W + q]);
        part[cg][rl * W + q] = a;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < ROWS) {
    int r = blockIdx.x * ROWS + threadIdx.x;
    if (r < m) out[r] = Emit::get(part[0][threadIdx.x], in[r]);
  }
}

template <class Acc, class Emit>
int launch_reduce_row(const float* in, float* out, int m, int n, mnv_stream_t stream) {
  if (m == 0) return MNV_OK;
  if (!in || !out || m < 0 || n <= 0) return MNV_ERR_INVALID;
  hipStream_t s = mnv_stream(stream);
  bool vec4 = (m % 4 == 0) && mnv_aligned16(in);
  if (vec4) {
    constexpr int RL = 8, CG = 64;
    unsigned grid = (unsigned)mnv_ceil_div((size_t)m, RL * 4);
    if ((size_t)m * n * sizeof(float) >= MNV_PAST_CACHE_BYTES)
      hipLaunchKernelGGL((mnv_reduce_row_kernel<Acc, Emit, RL, CG, true, true>), dim3(grid),
                         dim3(RL * CG), 0, s, in, out, m, n);
    else
      hipLaunchKernelGGL((mnv_reduce_row_kernel<Acc, Emit, RL, CG, true, false>), dim3(grid),
                         dim3(RL * CG), 0, s, in, out, m, n);
  } else {
    constexpr int RL = 32, CG = 16;
    unsigned grid = (unsigned)mnv_ceil_div((size_t)m, RL);
    hipLaunchKernelGGL((mnv_reduce_row_kernel<Acc, Emit, RL, CG, false, false>), dim3(grid),
                       dim3(RL * CG), 0, s, in, out, m, n);
  }
  return MNV_LAUNCH_STATUS();
}

// ---------------------------------------------------------------------------
// Convolution bias gradient: db[k] = sum over images and positions of dY[n,k,:,:]
// (reference cuda_perform.cu:320-337).  A channel's data is N runs of hw contiguous
// floats, one per image.  Workgroup (k, g) sums channel k over image group g: its four
// wavefronts take the group's images round-robin and read each run with 16-byte loads
// from its first aligned address (at most three single floats on either side).  With
// several groups per channel the group sums go to a scratch area and a second, tiny
// kernel adds them in group order, so the result does not depend on scheduling.
// ---------------------------------------------------------------------------
#define MNV_BIAS_THREADS 256

template <bool NT>
__global__ __launch_bounds__(MNV_BIAS_THREADS) void mnv_conv_bwd_bias_kernel(
    const float* __restrict__ top_diff, float* __restrict__ out, int N, int K, int hw,
    int images_per_group) {
  constexpr int NW = MNV_BIAS_THREADS / MNV_WAVE;
  __shared__ float part[NW];
  const int k = blockIdx.x, g = blockIdx.y;
  const int wave = threadIdx.x / MNV_WAVE, lane = threadIdx.x % MNV_WAVE;
  const int img_end = min(N, (g + 1) * images_per_group);
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int img = g * images_per_group + wave; img < img_end; img += NW) {
    const float* p = top_diff + ((size_t)img * K + k) * hw;
    int head = (int)((4 - ((reinterpret_cast<uintptr_t>(p) >> 2) & 3)) & 3);
    if (head > hw) head = hw;
    const int n4 = (hw - head) >> 2, tail = (hw - head) & 3;
    const mnv_f4* p4 = reinterpret_cast<const mnv_f4*>(p + head);
    float edge0 = 0.f, edge1 = 0.f;  // used after the vectors so that they do not wait for these
    if (lane < head) edge0 = p[lane];
    if (lane < tail) edge1 = p[head + 4 * n4 + lane];
    // Four loads in flight per lane in every iteration, the last one included: a vector
    // past the end of the run is read from the run's last vector instead (a cache hit) and
    // counted as 0, so there is no one-load-at-a-time remainder loop (a run of 55 x 55
    // floats would spend four of its six trips to memory in it).
    if (n4 > 0) {
      const int last = n4 - 1;
      for (int i = lane; i < n4; i += 4 * MNV_WAVE) {
        const int i1 = i + MNV_WAVE, i2 = i + 2 * MNV_WAVE, i3 = i + 3 * MNV_WAVE;
        mnv_f4 a = mnv_ldx4<NT>(p4 + i), b = mnv_ldx4<NT>(p4 + min(i1, last)),
               c = mnv_ldx4<NT>(p4 + min(i2, last)), d = mnv_ldx4<NT>(p4 + min(i3, last));
        s0 += (a.x + a.y) + (a.z + a.w);
        s1 += i1 < n4 ? (b.x + b.y) + (b.z + b.w) : 0.f;
        s2 += i2 < n4 ? (c.x + c.y) + (c.z + c.w) : 0.f;
        s3 += i3 < n4 ? (d.x + d.y) + (d.z + d.w) : 0.f;
      }
    }
    s0 += edge0;
    s1 += edge1;
  }
  float s = mnv_wave_sum((s0 + s1) + (s2 + s3));
  if (lane == 0) part[wave] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int q = 0; q < NW; ++q) t += part[q];
    out[(size_t)k * gridDim.y + g] = t;
  }
}

__global__ __launch_bounds__(256) void mnv_conv_bwd_bias_finish_kernel(
    const float* __restrict__ partial, float* __restrict__ bias_diff, int K, int groups) {
  const int k = blockIdx.x * 256 + threadIdx.x;
  if (k >= K) return;
  float t = 0.f;
  for (int g = 0; g < groups; ++g) t += partial[(size_t)k * groups + g];
  bias_diff[k] = t;
}

// Image groups per channel: enough workgroups to fill the chip, at least four images
// per wavefront's worth of work in each.
int bias_groups(int num_images, int channels) {
  int want = (2048 + channels - 1) / channels;
  int max_groups = (num_images + 3) / 4;
  if (want > max_groups) want = max_groups;
  if (want < 1) want = 1;
  int per = (num_images + want - 1) / want;
  return (num_images + per - 1) / per;
}

}  // namespace

extern "C" {

int mnv_reduce_sum_col(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_col<SumAcc, EmitValue>(in, out, m, n, s);
}
int mnv_reduce_max_col(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_col<ArgAcc, EmitValue>(in, out, m, n, s);
}
int mnv_reduce_sum_row(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_row<SumAcc, EmitValue>(in, out, m, n, s);
}
int mnv_reduce_max_row(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_row<ArgAcc, EmitValue>(in, out, m, n, s);
}
int mnv_maxindex_col(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_col<ArgAcc, EmitIndex>(in, out, m, n, s);
}
int mnv_maxindex_row(const float* in, float* out, int m, int n, mnv_stream_t s) {
  return launch_reduce_row<ArgAcc, EmitIndex>(in, out, m, n, s);
}

size_t mnv_conv_bwd_bias_workspace_bytes(int num_images, int top_num_channels) {
  if (num_images <= 0 || top_num_channels <= 0) return 0;
  int groups = bias_groups(num_images, top_num_channels);
  return groups > 1 ? (size_t)groups * top_num_channels * sizeof(float) : 0;
}

int mnv_conv_bwd_bias(const float* top_diff, float* bias_diff, int num_images,
                      int top_num_channels, int top_height, int top_width, void* workspace,
                      size_t workspace_bytes, mnv_stream_t stream) {
  if (top_num_channels == 0) return MNV_OK;
  if (!top_diff || !bias_diff || num_images <= 0 || top_num_channels < 0 || top_height <= 0 ||
      top_width <= 0)
    return MNV_ERR_INVALID;
  long long hw = (long long)top_height * top_width;
  if (hw > 0x7fffffffLL || top_num_channels > 0x7fffffff / 2) return MNV_ERR_INVALID;
  int groups = bias_groups(num_images, top_num_channels);
  if (groups > 65535) groups = 65535;
  if (!workspace || workspace_bytes < (size_t)groups * top_num_channels * sizeof(float)) groups = 1;
  int per = (num_images + groups - 1) / groups;
  hipStream_t s = mnv_stream(stream);
  float* out = groups > 1 ? reinterpret_cast<float*>(workspace) : bias_diff;
  if ((size_t)num_images * top_num_channels * hw * sizeof(float) >= MNV_PAST_CACHE_BYTES)
    hipLaunchKernelGGL(mnv_conv_bwd_bias_kernel<true>, dim3(top_num_channels, groups),
                       dim3(MNV_BIAS_THREADS), 0, s, top_diff, out, num_images, top_num_channels,
                       (int)hw, per);
  else
    hipLaunchKernelGGL(mnv_conv_bwd_bias_kernel<false>, dim3(top_num_channels, groups),
                       dim3(MNV_BIAS_THREADS), 0, s, top_diff, out, num_images, top_num_channels,
                       (int)hw, per);
  int rc = MNV_LAUNCH_STATUS();
  if (rc || groups == 1) return rc;
  hipLaunchKernelGGL(mnv_conv_bwd_bias_finish_kernel, dim3((top_num_channels + 255) / 256),
                     dim3(256), 0, s, reinterpret_cast<const float*>(workspace), bias_diff,
                     top_num_channels, groups);
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
