// Random tensor generators behind Randn and RandBernoulli (reference
// minerva/op/impl/cuda.cpp:599-607; cuRAND / kernel launchers
// minerva/op/impl/cuda/cuda_perform.cu:617-633).  The reference seeds cuRAND's default
// generator from the wall clock on every call, so its values cannot be reproduced; here
// the generator is counter based (Philox4x32-10, Salmon et al., "Parallel random numbers:
// as easy as 1, 2, 3", SC'11) and the seed is an argument: the same seed gives the same
// tensor on any launch geometry, and the host layer draws one seed per call.
//   element block b = i / 4 uses counter (lo32(b), hi32(b), 0, 0) and key (lo32(seed), hi32(seed))
//   normal:    x0,x1 -> Box-Muller pair for elements 4b, 4b+1; x2,x3 -> 4b+2, 4b+3
//              u1 = (x >> 8 + 1) * 2^-24 in (0, 1], u2 = (x >> 8) * 2^-24 in [0, 1)
//              z = sqrt(-2 ln u1) * (cos, sin)(2 pi u2);   out = mean + stddev * z
//   bernoulli: out = ((x >> 8) * 2^-24 < p) ? 1 : 0
// Roofline: HBM bandwidth, 4 bytes per element (write only).
#include <math.h>

#include "mnv_common.h"

namespace {

#define MNV_RNG_THREADS 256

struct Philox4 {
  unsigned x[4];
};

__device__ __forceinline__ Philox4 philox4x32_10(unsigned c0, unsigned c1, unsigned c2, unsigned c3,
                                                unsigned k0, unsigned k1) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const unsigned hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const unsigned hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const unsigned n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  Philox4 r;
  r.x[0] = c0; r.x[1] = c1; r.x[2] = c2; r.x[3] = c3;
  return r;
}

__device__ __forceinline__ void box_muller(unsigned a, unsigned b, float* z0, float* z1) {
  const float u1 = (float)((a >> 8) + 1u) * 5.9604644775390625e-8f;  // 2^-24, in (0, 1]
  const float u2 = (float)(b >> 8) * 5.9604644775390625e-8f;         // in [0, 1)
  const float r = sqrtf(-2.0f * __logf(u1));
  float s, c;
  __sincosf(6.283185307179586f * u2, &s, &c);
  *z0 = r * c;
  *z1 = r * s;
}

template <bool NORMAL>
__global__ __launch_bounds__(MNV_RNG_THREADS) void mnv_random_kernel(float* __restrict__ dst, size_t n,
                                                                   unsigned k0, unsigned k1, float a,
                                                                   float b, bool vec) {
  const size_t blocks4 = (n + 3) >> 2;
  for (size_t q = (size_t)blockIdx.x * MNV_RNG_THREADS + threadIdx.x; q < blocks4;
       q += (size_t)gridDim.x * MNV_RNG_THREADS) {
    const Philox4 r = philox4x32_10((unsigned)q, (unsigned)(q >> 32), 0u, 0u, k0, k1);
    float v[4];
    if (NORMAL) {  // a = mean, b = stddev
      box_muller(r.x[0], r.x[1], &v[0], &v[1]);
      box_muller(r.x[2], r.x[3], &v[2], &v[3]);
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] = a + b * v[t];
    } else {  // a = p
#pragma unroll
      for (int t = 0; t < 4; ++t)
        v[t] = ((float)(r.x[t] >> 8) * 5.9604644775390625e-8f < a) ? 1.f : 0.f;
    }
    const size_t i = q << 2;
    if (vec && i + 4 <= n) {
      mnv_f4 o = {v[0], v[1], v[2], v[3]};
      *reinterpret_cast<mnv_f4*>(dst + i) = o;
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        if (i + t < n) dst[i + t] = v[t];
    }
  }
}

template <bool NORMAL>
int launch(float* dst, size_t n, unsigned long long seed, float a, float b, mnv_stream_t stream) {
  if (n == 0) return MNV_OK;
  if (!dst) return MNV_ERR_INVALID;
  size_t blocks = mnv_ceil_div((n + 3) >> 2, MNV_RNG_THREADS);
  if (blocks > MNV_MAX_STREAM_BLOCKS) blocks = MNV_MAX_STREAM_BLOCKS;
  hipLaunchKernelGGL(mnv_random_kernel<NORMAL>, dim3((unsigned)blocks), dim3(MNV_RNG_THREADS), 0,
                     mnv_stream(stream), dst, n, (unsigned)seed, (unsigned)(seed >> 32), a, b,
                     mnv_aligned16(dst));
  return MNV_LAUNCH_STATUS();
}

}  // namespace

extern "C" {

int mnv_randn(float* dst, size_t n, unsigned long long seed, float mean, float stddev,
              mnv_stream_t stream) {
  return launch<true>(dst, n, seed, mean, stddev, stream);
}

int mnv_rand_bernoulli(float* dst, size_t n, unsigned long long seed, float p, mnv_stream_t stream) {
  if (!(p >= 0.f && p <= 1.f)) return MNV_ERR_INVALID;
  return launch<false>(dst, n, seed, p, 0.f, stream);
}

}  // extern "C"
