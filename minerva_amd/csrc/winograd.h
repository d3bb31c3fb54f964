// 3 x 3 unit-stride convolutions by F(2 x 2, 3 x 3) minimal filtering (winograd.hip), as the
// convolution entry points of conv.hip call it.
#pragma once
#include "mnv_common.h"

// Images per launch group that the pass would run with under this workspace, 0 when it does
// not run this way: other filter extents or strides, a source channel count that is not a
// multiple of 16, the mode switched off (mnv_conv_winograd_mode), a workspace too small for
// one image, or (mode 1) a geometry where the direct kernels are expected to be as fast.
// (Cin, Hs, Ws): the tensor that is read; Cout: channels of the tensor that is written;
// (pad_h, pad_w): padding of the correlation (the data gradient passes 2 - pad).
int mnv_wino_images(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R, int S,
                    int sv, int sh, size_t workspace_bytes);

// Bytes the pass wants to run all N images as one group.
size_t mnv_wino_workspace_bytes(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w);

// dst {N, Cout, Hs + 2 pad_h - 2, Ws + 2 pad_w - 2} = correlation of src {N, Cin, Hs, Ws} with
// the 3 x 3 filters.  `filter` is the caller's {K, C, 3, 3} tensor: forward (transposed = 0)
// K = Cout, C = Cin, taps flipped; data gradient (transposed = 1) K = Cin, C = Cout, taps as
// stored.  Epilogue in this order, each optional: + bias[co]; max(., 0); kept where gate > 0.
// `images`: what mnv_wino_images returned for this workspace.
int mnv_wino_conv(const float* src, const float* filter, const float* bias, const float* gate,
                  float* dst, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w,
                  int transposed, int relu, int images, void* workspace, size_t workspace_bytes,
                  hipStream_t s);
