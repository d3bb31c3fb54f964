// 3 x 3 and 5 x 5 unit-stride convolutions by minimal filtering, F(m x m, r x r) with r = 3 or 5
// (winograd.hip), as the convolution entry points of conv.hip call it.
#pragma once
#include "mnv_common.h"

// Images per launch group that the pass would run with under this workspace, 0 when it does
// not run this way: other filter extents or strides, a source channel count that is not a
// multiple of 16, the mode switched off (mnv_conv_winograd_mode), a workspace too small for
// one image, or (mode 1) a geometry where the direct kernels are expected to be as fast.
// (Cin, Hs, Ws): the tensor that is read; Cout: channels of the tensor that is written;
// (pad_h, pad_w): padding of the correlation (the data gradient passes R - 1 - pad).
int mnv_wino_images(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R, int S,
                    int sv, int sh, size_t workspace_bytes);

// Bytes the pass wants to run all N images as one group.
size_t mnv_wino_workspace_bytes(int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R);

// dst {N, Cout, Hs + 2 pad_h - (R - 1), Ws + 2 pad_w - (R - 1)} = correlation of src {N, Cin, Hs, Ws} with
// the R x R filters.  `filter` is the caller's {K, C, R, R} tensor: forward (transposed = 0)
// K = Cout, C = Cin, taps flipped; data gradient (transposed = 1) K = Cin, C = Cout, taps as
// stored.  Epilogue in this order, each optional: + bias[co]; max(., 0); kept where gate > 0.
// `images`: what mnv_wino_images returned for this workspace.
int mnv_wino_conv(const float* src, const float* filter, const float* bias, const float* gate,
                  float* dst, int N, int Cin, int Cout, int Hs, int Ws, int pad_h, int pad_w, int R,
                  int transposed, int relu, int images, void* workspace, size_t workspace_bytes,
                  hipStream_t s);

// The filter gradient of the same layers by F(r x r, m x m): the sum over images and tiles is the
// reduction dimension of the products, which run as one equal-shares launch of the MFMA
// core.  (C, H, W): bottom; K: channels of top_diff; (ph, pw): the layer's padding.
// mnv_wino_grad_images as mnv_wino_images (no condition on the channel counts' divisors);
// with more than one group the products accumulate group by group.
int mnv_wino_grad_images(int N, int C, int K, int H, int W, int ph, int pw, int R, int S, int sv,
                         int sh, size_t workspace_bytes);
size_t mnv_wino_grad_workspace_bytes(int N, int C, int K, int H, int W, int ph, int pw, int R);
// filter_diff {K, C, R, R} = the gradient; `accumulate`: added to what is there; `sgd_w`: the value
// stored is sgd_w - sgd_scale * gradient.  `plan` (optional): nothing is launched, plan[0] =
// rows of the tile, plan[1] = 1, plan[2] = workgroups of the equal-shares launch (0: the product
// is too small for it and runs one workgroup per tile).
int mnv_wino_filter_grad(const float* bottom, const float* top_diff, float* filter_diff, int N, int C,
                         int K, int H, int W, int ph, int pw, int R, int images, int accumulate,
                         const float* sgd_w, float sgd_scale, void* workspace,
                         size_t workspace_bytes, hipStream_t s, int* plan);
