// Geometry of one Conv2d call and the entry points of the specialised convolution kernels.
#pragma once

#include "common.h"

namespace lten_hip {

struct ConvGeo {
	int N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo;
};

// Kernels for stride 1, dilation 1 that stage the input patch of an output tile in LDS (conv_patch.hip).
// *_takes: whether the kernel family covers this geometry and these pointers.
bool conv_patch_forward_takes(const ConvGeo& g, const float* x, const float* y);
int conv_patch_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y);
bool conv_patch_wgrad_takes(const ConvGeo& g);
int conv_patch_wgrad_parts(const ConvGeo& g);  // partial [Cout x Cin*kh*kw] matrices the kernel writes
int conv_patch_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts);

// Sums `parts` partial matrices of `count` floats in a fixed order.
int conv_reduce_partials(const float* partial, int parts, int64_t count, float* out);

}  // namespace lten_hip
