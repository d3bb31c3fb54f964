// Shared helpers of the gfx950 operator library (host + device side).
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "mnv_hip.h"

#define MNV_WAVE 64

// Propagate a HIP runtime error as the C-ABI status.
#define MNV_HIP_TRY(expr)                      \
  do {                                         \
    hipError_t mnv_e_ = (expr);                \
    if (mnv_e_ != hipSuccess) return (int)mnv_e_; \
  } while (0)

// Status of the launch that was just issued (does not synchronise).
#define MNV_LAUNCH_STATUS() ((int)hipGetLastError())

static inline hipStream_t mnv_stream(mnv_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

static inline bool mnv_aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static inline size_t mnv_ceil_div(size_t a, size_t b) { return (a + b - 1) / b; }

// Compute units of the current device (cached per device; 256, the MI355X's count, when no
// device can be asked, so that size queries work on a machine without a GPU).
int mnv_cu_count();

// Upper bound on grid.x for grid-stride kernels: enough resident work for
// 256 CUs without paying launch cost for millions of tiny blocks.
#define MNV_MAX_STREAM_BLOCKS 16384u

// Division by a run-time constant d >= 1, prepared on the host; valid for 0 <= n < 2^31
// and branch-free (d == 1 gives mul == 0, shift == 0):  n / d == (mulhi(n, mul) + n) >> shift.
struct MnvFastDiv {
  unsigned mul, shift;
};

static inline MnvFastDiv mnv_fastdiv_make(int d) {
  MnvFastDiv f;
  unsigned s = 0;
  while ((1ull << s) < (unsigned long long)d) ++s;  // ceil(log2 d)
  f.shift = s;
  f.mul = (unsigned)((((1ull << s) - (unsigned long long)d) << 32) / (unsigned long long)d + 1);
  if (d <= 1) f.mul = 0;
  return f;
}

#ifdef __HIPCC__
__device__ __forceinline__ int mnv_fastdiv(int n, const MnvFastDiv& f) {
  return (int)((__umulhi((unsigned)n, f.mul) + (unsigned)n) >> f.shift);
}

typedef float mnv_f4 __attribute__((ext_vector_type(4)));
// the same four floats where only their 4-byte alignment is known
typedef float mnv_f4u __attribute__((ext_vector_type(4), aligned(4)));
#ifdef __HIPCC__
// A 16-byte load of data that is read once.  NT: non-temporal, for tensors of 256 MB and
// more, which cannot stay in the last-level cache anyway (measured with operands cycled so
// that none is cached: column sums 5.95 -> 6.66 TB/s, broadcast 6.16 -> 6.36, transpose
// 5.53 -> 5.68); smaller tensors are read through the caches for the operator that follows.
template <bool NT>
__device__ __forceinline__ mnv_f4 mnv_ldx4(const mnv_f4* p) {
  if (NT) return __builtin_nontemporal_load(p);
  return *p;
}
#endif
#define MNV_PAST_CACHE_BYTES ((size_t)256 << 20)



// Buffer addressing: every operand is read through a raw buffer resource whose extent is
// the tensor's byte size, so a masked-off element is fetched with an offset past the end
// and the hardware returns 0 for it: no divergent branch, no address clamp, no fault.
// Operands are therefore limited to 2^31 - 1 bytes.
#define MNV_OOB 0x80000000u
typedef __amdgpu_buffer_rsrc_t mnv_rsrc;

__device__ __forceinline__ mnv_rsrc mnv_make_rsrc(const float* p, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(p), 0, bytes, 0x00020000);
}
__device__ __forceinline__ float mnv_buf_load(mnv_rsrc r, unsigned byte_off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, (int)byte_off, 0, 0));
}
__device__ __forceinline__ void mnv_buf_load4(mnv_rsrc r, unsigned byte_off, float (&v)[4]) {
  mnv_f4 t = __builtin_bit_cast(mnv_f4, __builtin_amdgcn_raw_buffer_load_b128(r, (int)byte_off, 0, 0));
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}


__device__ __forceinline__ float mnv_wave_sum(float v) {
#pragma unroll
  for (int off = MNV_WAVE / 2; off > 0; off >>= 1) v += __shfl_down(v, off, MNV_WAVE);
  return v;
}

__device__ __forceinline__ float mnv_wave_max(float v) {
#pragma unroll
  for (int off = MNV_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_down(v, off, MNV_WAVE));
  return v;
}
#endif
