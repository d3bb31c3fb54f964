// HBM-streaming kernel templates: out[i] = op(in0[i] [, in1[i]]) over flat fp32
// buffers.  Roofline: HBM bandwidth; algorithmic bytes = 4*(NIN+1) per element
// (4 per element for the fill).  Each thread keeps UNROLL independent 16-byte
// loads per input in flight before it touches any of them, every wavefront
// load/store covers 1 KiB of contiguous memory, and the grid is sized so that
// all 256 CUs hold several workgroups.
#pragma once
#include "mnv_common.h"

#define MNV_STREAM_THREADS 256
#define MNV_STREAM_UNROLL 4

template <bool NT>
__device__ __forceinline__ mnv_f4 mnv_ld4(const mnv_f4* p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}
template <bool NT>
__device__ __forceinline__ void mnv_st4(mnv_f4* p, mnv_f4 v) {
  if (NT) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// NIN = 0 (fill), 1 (unary / scalar) or 2 (binary).  n4 = n / 4 full vectors,
// the n % 4 trailing floats are handled by the first threads of block 0.
template <class Op, int NIN, bool NT>
__global__ __launch_bounds__(MNV_STREAM_THREADS) void mnv_stream_vec4_kernel(
    const float* __restrict__ in0, const float* __restrict__ in1, float* __restrict__ out,
    size_t n, Op op) {
  const size_t n4 = n >> 2;
  const mnv_f4* a4 = reinterpret_cast<const mnv_f4*>(in0);
  const mnv_f4* b4 = reinterpret_cast<const mnv_f4*>(in1);
  mnv_f4* o4 = reinterpret_cast<mnv_f4*>(out);
  const size_t chunk = (size_t)MNV_STREAM_THREADS * MNV_STREAM_UNROLL;
  for (size_t base = (size_t)blockIdx.x * chunk + threadIdx.x; base < n4;
       base += (size_t)gridDim.x * chunk) {
    mnv_f4 a[MNV_STREAM_UNROLL], b[MNV_STREAM_UNROLL];
#pragma unroll
    for (int u = 0; u < MNV_STREAM_UNROLL; ++u) {
      size_t i = base + (size_t)u * MNV_STREAM_THREADS;
      if (i < n4) {
        if (NIN >= 1) a[u] = mnv_ld4<NT>(a4 + i);
        if (NIN >= 2) b[u] = mnv_ld4<NT>(b4 + i);
      }
    }
#pragma unroll
    for (int u = 0; u < MNV_STREAM_UNROLL; ++u) {
      size_t i = base + (size_t)u * MNV_STREAM_THREADS;
      if (i < n4) {
        mnv_f4 r;
        r.x = op(NIN >= 1 ? a[u].x : 0.f, NIN >= 2 ? b[u].x : 0.f);
        r.y = op(NIN >= 1 ? a[u].y : 0.f, NIN >= 2 ? b[u].y : 0.f);
        r.z = op(NIN >= 1 ? a[u].z : 0.f, NIN >= 2 ? b[u].z : 0.f);
        r.w = op(NIN >= 1 ? a[u].w : 0.f, NIN >= 2 ? b[u].w : 0.f);
        mnv_st4<NT>(o4 + i, r);
      }
    }
  }
  if (blockIdx.x == 0) {
    size_t i = (n4 << 2) + threadIdx.x;
    if (i < n) out[i] = op(NIN >= 1 ? in0[i] : 0.f, NIN >= 2 ? in1[i] : 0.f);
  }
}

// Fallback for buffers that are not 16-byte aligned.
template <class Op, int NIN>
__global__ __launch_bounds__(MNV_STREAM_THREADS) void mnv_stream_scalar_kernel(
    const float* __restrict__ in0, const float* __restrict__ in1, float* __restrict__ out,
    size_t n, Op op) {
  for (size_t i = (size_t)blockIdx.x * MNV_STREAM_THREADS + threadIdx.x; i < n;
       i += (size_t)gridDim.x * MNV_STREAM_THREADS)
    out[i] = op(NIN >= 1 ? in0[i] : 0.f, NIN >= 2 ? in1[i] : 0.f);
}

// Buffers above this many bytes of traffic cannot stay in the 256 MB last-level
// cache between kernels, so they stream past it with non-temporal loads and stores.
// Measured on 8192^2 operands, cycling through four sets of them so that no pass finds its
// operands cached: everything non-temporal moves 6.3 TB/s (one input) / 6.5 TB/s (two
// inputs); first input ordinary 6.0 / 6.4; everything ordinary 5.8 / 5.8.  (When one set
// is reused, a third of it is still cached on the next pass and the ordinary first input
// looks best: 7.0 / 7.3 TB/s.)
#define MNV_STREAM_NT_BYTES ((size_t)512 << 20)

template <class Op, int NIN>
static int mnv_stream_launch(const float* in0, const float* in1, float* out, size_t n, Op op,
                             mnv_stream_t stream) {
  if (n == 0) return MNV_OK;
  if (!out || (NIN >= 1 && !in0) || (NIN >= 2 && !in1)) return MNV_ERR_INVALID;
  hipStream_t s = mnv_stream(stream);
  bool vec = mnv_aligned16(out) && (NIN < 1 || mnv_aligned16(in0)) && (NIN < 2 || mnv_aligned16(in1));
  if (vec) {
    size_t n4 = n >> 2;
    size_t blocks = mnv_ceil_div(n4 ? n4 : 1, (size_t)MNV_STREAM_THREADS * MNV_STREAM_UNROLL);
    if (blocks > MNV_MAX_STREAM_BLOCKS) blocks = MNV_MAX_STREAM_BLOCKS;
    bool nt = n * 4 * (NIN + 1) >= MNV_STREAM_NT_BYTES;
    if (nt)
      hipLaunchKernelGGL((mnv_stream_vec4_kernel<Op, NIN, true>), dim3((unsigned)blocks),
                         dim3(MNV_STREAM_THREADS), 0, s, in0, in1, out, n, op);
    else
      hipLaunchKernelGGL((mnv_stream_vec4_kernel<Op, NIN, false>), dim3((unsigned)blocks),
                         dim3(MNV_STREAM_THREADS), 0, s, in0, in1, out, n, op);
  } else {
    size_t blocks = mnv_ceil_div(n, MNV_STREAM_THREADS);
    if (blocks > MNV_MAX_STREAM_BLOCKS) blocks = MNV_MAX_STREAM_BLOCKS;
    hipLaunchKernelGGL((mnv_stream_scalar_kernel<Op, NIN>), dim3((unsigned)blocks),
                       dim3(MNV_STREAM_THREADS), 0, s, in0, in1, out, n, op);
  }
  return MNV_LAUNCH_STATUS();
}
