// Data movement behind Concat, Slice and Select (reference minerva/op/impl/cuda.cpp:80-155
// and :644-655; SelectKernel minerva/op/impl/cuda/cuda_kernel.h:333-342).
//
// Concat and Slice along dimension d of a column-major tensor move, for every index of the
// dimensions above d, one contiguous run of (extent along d) * (product of the dimensions
// below d) floats: a 2-D copy with different row pitches on the two sides.  The reference
// issues one cublasScopy per image for this; here it is one launch per input.  Select
// gathers whole columns of a matrix.  Roofline: HBM bandwidth, 8 bytes per element moved;
// everything is a pure copy, hence bit-exact.
#include "mnv_common.h"

namespace {

#define MNV_GATHER_THREADS 256

// rows of `row_elems` floats; row r is read at src + r*src_pitch and written at
// dst + r*dst_pitch.  VEC: row_elems, both pitches and both pointers are multiples of four
// floats, so a thread moves 16 bytes at a time.
template <bool VEC>
__global__ __launch_bounds__(MNV_GATHER_THREADS) void mnv_copy_2d_kernel(
    const float* __restrict__ src, float* __restrict__ dst, size_t row_elems, size_t rows,
    size_t src_pitch, size_t dst_pitch) {
  const size_t per_row = VEC ? row_elems >> 2 : row_elems;
  for (size_t r = blockIdx.y; r < rows; r += gridDim.y) {
    const float* s = src + r * src_pitch;
    float* d = dst + r * dst_pitch;
    for (size_t i = (size_t)blockIdx.x * MNV_GATHER_THREADS + threadIdx.x; i < per_row;
         i += (size_t)gridDim.x * MNV_GATHER_THREADS) {
      if (VEC)
        reinterpret_cast<mnv_f4*>(d)[i] = reinterpret_cast<const mnv_f4*>(s)[i];
      else
        d[i] = s[i];
    }
  }
}

// dst[:, j] = src[:, indices[j]] for a column-major {rows, cols} matrix
__global__ __launch_bounds__(MNV_GATHER_THREADS) void mnv_select_kernel(
    const float* __restrict__ src, float* __restrict__ dst, const int* __restrict__ indices,
    int rows, int count) {
  for (int j = blockIdx.y; j < count; j += gridDim.y) {
    const float* s = src + (size_t)indices[j] * rows;
    float* d = dst + (size_t)j * rows;
    for (int i = blockIdx.x * MNV_GATHER_THREADS + threadIdx.x; i < rows;
         i += gridDim.x * MNV_GATHER_THREADS)
      d[i] = s[i];
  }
}

}  // namespace

extern "C" {

int mnv_copy_2d(const float* src, float* dst, size_t row_elems, size_t rows, size_t src_pitch,
                size_t dst_pitch, mnv_stream_t stream) {
  if (row_elems == 0 || rows == 0) return MNV_OK;
  if (!src || !dst || src_pitch < row_elems || dst_pitch < row_elems) return MNV_ERR_INVALID;
  const bool vec = ((row_elems | src_pitch | dst_pitch) & 3) == 0 && mnv_aligned16(src) &&
                   mnv_aligned16(dst);
  const size_t per_row = vec ? row_elems >> 2 : row_elems;
  size_t gx = mnv_ceil_div(per_row, MNV_GATHER_THREADS);
  size_t gy = rows < 65535 ? rows : 65535;
  // enough workgroups to fill the chip, not one per 256 elements of a huge tensor
  const size_t want = 8 * MNV_MAX_STREAM_BLOCKS;
  if (gx * gy > want) gx = mnv_ceil_div(want, gy);
  if (gx < 1) gx = 1;
  const dim3 grid((unsigned)gx, (unsigned)gy);
  if (vec)
    hipLaunchKernelGGL(mnv_copy_2d_kernel<true>, grid, dim3(MNV_GATHER_THREADS), 0,
                       mnv_stream(stream), src, dst, row_elems, rows, src_pitch, dst_pitch);
  else
    hipLaunchKernelGGL(mnv_copy_2d_kernel<false>, grid, dim3(MNV_GATHER_THREADS), 0,
                       mnv_stream(stream), src, dst, row_elems, rows, src_pitch, dst_pitch);
  return MNV_LAUNCH_STATUS();
}

size_t mnv_select_workspace_bytes(int num_indices) {
  return num_indices > 0 ? (size_t)num_indices * sizeof(int) : 0;
}

int mnv_select(const float* src, float* dst, const int* indices_host, int num_indices, int rows,
               int cols, void* workspace, size_t workspace_bytes, mnv_stream_t stream) {
  if (num_indices == 0 || rows == 0) return MNV_OK;
  if (!src || !dst || !indices_host || num_indices < 0 || rows < 0 || cols <= 0)
    return MNV_ERR_INVALID;
  for (int j = 0; j < num_indices; ++j)
    if (indices_host[j] < 0 || indices_host[j] >= cols) return MNV_ERR_INVALID;
  if (!workspace || workspace_bytes < (size_t)num_indices * sizeof(int)) return MNV_ERR_WORKSPACE;
  hipStream_t s = mnv_stream(stream);
  // pageable host memory: the runtime stages the indices before this call returns
  MNV_HIP_TRY(hipMemcpyAsync(workspace, indices_host, (size_t)num_indices * sizeof(int),
                             hipMemcpyHostToDevice, s));
  unsigned gx = (unsigned)mnv_ceil_div((size_t)rows, MNV_GATHER_THREADS);
  if (gx > 1024) gx = 1024;
  const dim3 grid(gx, (unsigned)(num_indices < 65535 ? num_indices : 65535));
  hipLaunchKernelGGL(mnv_select_kernel, grid, dim3(MNV_GATHER_THREADS), 0, s, src, dst,
                     reinterpret_cast<const int*>(workspace), rows, num_indices);
  return MNV_LAUNCH_STATUS();
}

}  // extern "C"
