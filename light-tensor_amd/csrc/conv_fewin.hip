// Conv2d forward, 3x3, stride 1, column padding 1, with one or two input channels (a first layer).
//
// The work is a stream of y to HBM (Cout planes written for every plane read): 9 * Cin multiply-adds per output
// value, far below what the vector ALUs do in the time the store takes, and no reuse that would call for LDS.  A
// workgroup computes 8 rows x 128 columns of one image for all or a share of the output channels; a thread owns four
// consecutive pixels of one row.  It loads the 3 x 4 input values above, at and below its pixels as three 16-byte loads per
// input channel (x is small and stays in the caches), takes the columns left and right of them from the adjacent
// lanes (at the ends of a tile row from memory, or zero outside the image), and keeps these 18 * Cin values in
// registers.  Output channels are then walked in groups of eight: the group's 72 * Cin weights are wave-uniform
// (scalar loads), each thread does 288 * Cin multiply-adds and stores eight float4, so that a wave-wide store covers
// 1 KB of one output row — a quarter of the store instructions of the MFMA kernel for the same bytes.
//
// Needs W % 4 == 0 and 16-byte aligned x and y.
#include "conv_common.h"

namespace lten_hip {

// v[ci][i][0..5] = input columns wo - 1 .. wo + 4 of input row ho - ph + i of image n (zero outside the image, all
// zero for a thread that is not `inside` the output).  To be called by all 64 lanes of a wavefront: the columns
// beside a thread's own four come from the adjacent lanes.
template <int CIN>
__device__ __forceinline__ void load_window(const ConvGeo& g, const float* __restrict__ x, int n, int ho, int wo, int tq, bool inside, float (&v)[CIN][3][6])
{
#pragma unroll
	for (int ci = 0; ci < CIN; ci++) {
		const float* xc = x + ((int64_t)n * g.Cin + ci) * g.H * g.W;
#pragma unroll
		for (int i = 0; i < 3; i++) {
			const int gy = ho - g.ph + i;
			const bool row_ok = inside && gy >= 0 && gy < g.H;
			float4 mid = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
			if (row_ok) mid = *reinterpret_cast<const float4*>(xc + (int64_t)gy * g.W + wo);
			// every lane takes part in the exchange; lanes outside the image pass zeros
			float left = __shfl_up(mid.w, 1, 64), right = __shfl_down(mid.x, 1, 64);
			if (tq == 0) left = (row_ok && wo > 0) ? xc[(int64_t)gy * g.W + wo - 1] : 0.0f;
			if (tq == 31 || wo + 4 >= g.W) right = (row_ok && wo + 4 < g.W) ? xc[(int64_t)gy * g.W + wo + 4] : 0.0f;
			v[ci][i][0] = left; v[ci][i][1] = mid.x; v[ci][i][2] = mid.y; v[ci][i][3] = mid.z; v[ci][i][4] = mid.w; v[ci][i][5] = right;
		}
	}
}

template <int CIN>
__global__ __launch_bounds__(256) void conv2d_fewin_forward_kernel(ConvGeo g, const float* __restrict__ x, const float* __restrict__ w,
                                                                   const float* __restrict__ bias, float* __restrict__ y)
{
	constexpr int TH = 8, TW = 128, CG = 8;
	const int tid = threadIdx.x;
	const int trow = tid >> 5, tq = tid & 31;
	const int tiles_w = (g.Wo + TW - 1) / TW;
	const int w0 = (int)(blockIdx.x % tiles_w) * TW, h0 = (int)(blockIdx.x / tiles_w) * TH;
	const int n = blockIdx.y;
	const int ho = h0 + trow, wo = w0 + 4 * tq;  // Wo == W: the pixel columns are the input columns
	const bool inside = ho < g.Ho && wo < g.W;

	float v[CIN][3][6];
	load_window<CIN>(g, x, n, ho, wo, tq, inside, v);
	if (!inside) return;

	const int64_t plane = (int64_t)g.Ho * g.Wo;
	float* yp = y + ((int64_t)n * g.Cout * g.Ho + ho) * g.Wo + wo;
	// blockIdx.z picks this workgroup's share of the output channels (groups c0 = CG z, CG (z + gridDim.z), ...)
	for (int c0 = CG * blockIdx.z; c0 < g.Cout; c0 += CG * gridDim.z) {
#pragma unroll
		for (int cc = 0; cc < CG; cc++) {
			const int co = c0 + cc;
			if (co >= g.Cout) break;  // the same for every thread
			const float b = bias ? bias[co] : 0.0f;
			float acc[4] = { b, b, b, b };
#pragma unroll
			for (int ci = 0; ci < CIN; ci++) {
				const float* wr = w + ((int64_t)co * g.Cin + ci) * 9;
#pragma unroll
				for (int i = 0; i < 3; i++)
#pragma unroll
					for (int j = 0; j < 3; j++) {
						const float wv = wr[3 * i + j];
#pragma unroll
						for (int p = 0; p < 4; p++) acc[p] = fmaf(v[ci][i][p + j], wv, acc[p]);
					}
			}
			*reinterpret_cast<float4*>(yp + co * plane) = make_float4(acc[0], acc[1], acc[2], acc[3]);
		}
	}
}

bool conv_fewin_takes(const ConvGeo& g, const float* x, const float* y)
{
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.kh == 3 && g.kw == 3 && g.pw == 1 && g.ph <= 2 && g.Cin >= 1 && g.Cin <= 2 &&
	       g.Cout >= 1 && g.W % 4 == 0 && aligned16(x) && aligned16(y) && g.N < 65536;
}

int conv_fewin_forward(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	// More wavefronts per CU keep more stores in flight: while the tiles alone give fewer than eight workgroups per
	// CU, the groups of eight output channels are dealt to up to four workgroups per tile (32 output channels on
	// 32 x 128 x 128: 15.4 us with one workgroup per tile, 12.6 with two, 12.2 with four; a kernel that only
	// writes the 67 MB takes 11.1-11.5).
	const uint64_t tiles = ceil_div((uint64_t)g.Wo, 128) * ceil_div((uint64_t)g.Ho, 8);
	unsigned split = 1;
	while (split < 4 && tiles * g.N * split < 2048 && 8 * 2 * split <= (unsigned)g.Cout) split *= 2;
	const dim3 grid((unsigned)tiles, (unsigned)g.N, split), block(256);
	set_kernel_name("conv2d_fewin_forward_3x3_8x128");
	if (g.Cin == 1) conv2d_fewin_forward_kernel<1><<<grid, block, 0, stream()>>>(g, x, w, bias, y);
	else conv2d_fewin_forward_kernel<2><<<grid, block, 0, stream()>>>(g, x, w, bias, y);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
