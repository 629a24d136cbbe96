// Geometry of one Conv2d call and the entry points of the specialised convolution kernels.
#pragma once

#include "common.h"

#include <hip/hip_runtime.h>

namespace lten_hip {

struct ConvGeo {
	int N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, dh, dw, Ho, Wo;
};

// Kernels for stride 1, dilation 1 that stage the input patch of an output tile in LDS (conv_patch.hip).
// *_takes: whether the kernel family covers this geometry and these pointers.
bool conv_patch_forward_takes(const ConvGeo& g, const float* x, const float* y);
int conv_patch_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y);
// the same tile with the LDS patch filled by direct global->LDS loads (conv_patch_fast.hip)
bool conv_patch_fast_forward_takes(const ConvGeo& g, const float* x, const float* w);
int conv_patch_fast_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y);
bool conv_patch_wgrad_takes(const ConvGeo& g);
int conv_patch_wgrad_parts(const ConvGeo& g, bool upper_bound = false);  // partial [Cout x Cin*kh*kw] matrices the kernel writes
int conv_patch_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts);
// the same product with both LDS tiles filled by direct global->LDS loads (padding 1, W % 64 == 0, 16-byte aligned x and dy)
bool conv_patch_fast_wgrad_takes(const ConvGeo& g, const float* x, const float* dy);
int conv_patch_fast_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts);

// 3x3, stride 1, at most four output channels: a stream over x on the vector ALUs (conv_fewout.hip).  dgrad: w is the
// weight array of the convolution whose data gradient is computed, read transposed and flipped in place.
bool conv_fewout_takes(const ConvGeo& g, const float* x, const float* y);
int conv_fewout_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y, bool dgrad);

// 3x3, stride 1, one or two input channels: a stream of y from registers, no LDS (conv_fewin.hip).
bool conv_fewin_takes(const ConvGeo& g, const float* x, const float* y);
int conv_fewin_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y);

// Kernels for stride 1, dilation 1 and Cin*kh*kw <= 32 (first layers): the whole reduction fits one MFMA tile
// dimension, the work is bound by the HBM traffic of y / dy (conv_smallk.hip).
bool conv_smallk_takes(const ConvGeo& g);
int conv_smallk_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y);
int conv_smallk_wgrad_parts(const ConvGeo& g);
int conv_smallk_wgrad(const ConvGeo& g, const float* x, const float* dy, float* partial, int parts);

// Sums `parts` partial matrices of `count` floats in a fixed order.
int conv_reduce_partials(const float* partial, int parts, int64_t count, float* out);

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

#if defined(__HIPCC__)
// Four consecutive floats of a row starting at column gx; columns outside [0, limit) read as 0.  With VEC
// (limit % 4 == 0, gx % 4 == 0, 16-byte aligned row) the four are inside or outside together.
template <bool VEC>
__device__ __forceinline__ float4 load_row4(const float* row, int gx, int limit)
{
	float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
	if (VEC) {
		if (gx >= 0 && gx + 3 < limit) v = *reinterpret_cast<const float4*>(row + gx);
	} else {
		if (gx >= 0 && gx < limit) v.x = row[gx];
		if (gx + 1 >= 0 && gx + 1 < limit) v.y = row[gx + 1];
		if (gx + 2 >= 0 && gx + 2 < limit) v.z = row[gx + 2];
		if (gx + 3 >= 0 && gx + 3 < limit) v.w = row[gx + 3];
	}
	return v;
}
#endif

}  // namespace lten_hip
