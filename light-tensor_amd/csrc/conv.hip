// im2col / col2im and the fused (implicit-GEMM) Conv2d forward and weight gradient for gfx950.
//
// l-ten lowers Conv2d to one im2col + one GEMM per image (l-ten/conv2d.cpp:164-171 forward,
// l-ten/backprop.cpp:1949-1953 weight gradient), writing and re-reading a [Cin*kh*kw, Hout*Wout] column
// buffer each time.  Here the column matrix is not stored as a rule: the GEMM operand fetch computes the im2col
// address on the fly (col[k][hw] = x[ci][ho*sh - ph + i][wo*sw - pw + j], zero outside the image), and one
// launch covers the whole batch (deep layers on small images are the exception: conv_forward_by_columns).
// The standalone im2col / col2im kernels keep the semantics of l-ten's
// CUDA ones (l-ten/im_col.cu:65-96, 123-162) for callers that still want the buffer.
#include "conv_common.h"
#include "gemm_f32_core.h"
#include "sgemm_common.h"

#include <algorithm>

namespace lten_hip {

template <typename T>
__global__ __launch_bounds__(256) void im2col_kernel(const T* im, ConvGeo g, T* col)
{
	// one thread per element of col, consecutive threads along Hout*Wout
	const int64_t total = (int64_t)g.Cin * g.kh * g.kw * g.Ho * g.Wo;
	for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
		const int wo = (int)(idx % g.Wo);
		const int ho = (int)((idx / g.Wo) % g.Ho);
		const int r = (int)(idx / ((int64_t)g.Wo * g.Ho));
		const int j = r % g.kw, i = (r / g.kw) % g.kh, c = r / (g.kw * g.kh);
		const int y = ho * g.sh - g.ph + i * g.dh, x = wo * g.sw - g.pw + j * g.dw;
		col[idx] = (y >= 0 && y < g.H && x >= 0 && x < g.W) ? im[((int64_t)c * g.H + y) * g.W + x] : (T)0;
	}
}

template <typename T>
__global__ __launch_bounds__(256) void col2im_kernel(const T* col, ConvGeo g, T* im)
{
	// one thread per image element gathers every column entry that maps to it, kernel taps in increasing
	// (i, j) order — the order in which l-ten's CPU scatter-add reaches that element (l-ten/im_col.h:41-55)
	const int64_t total = (int64_t)g.Cin * g.H * g.W;
	for (int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x; idx < total; idx += (int64_t)gridDim.x * 256) {
		const int x = (int)(idx % g.W), y = (int)((idx / g.W) % g.H), c = (int)(idx / ((int64_t)g.W * g.H));
		T s = (T)0;  // integer types wrap as l-ten's `+=` on T does
		for (int i = 0; i < g.kh; i++) {
			const int yy = y + g.ph - i * g.dh;
			if (yy < 0 || yy % g.sh != 0 || yy / g.sh >= g.Ho) continue;
			for (int j = 0; j < g.kw; j++) {
				const int xx = x + g.pw - j * g.dw;
				if (xx < 0 || xx % g.sw != 0 || xx / g.sw >= g.Wo) continue;
				s += col[(((int64_t)c * g.kh + i) * g.kw + j) * g.Ho * g.Wo + (int64_t)(yy / g.sh) * g.Wo + xx / g.sw];
			}
		}
		im[idx] = s;
	}
}

// Per reduction index k = (ci, i, j): where the tap lies relative to the top left tap of channel 0, and which tap it is.
struct KTap {
	int off;  // (ci*H + i*dh)*W + j*dw
	int ij;   // i*dh | (j*dw) << 16
};
constexpr int MAX_KTAB = 4608;  // Cin*kh*kw up to 4608 (e.g. 512 channels of 3x3) use the LDS table

__device__ __forceinline__ KTap make_tap(const ConvGeo& g, int k)
{
	const int j = k % g.kw, i = (k / g.kw) % g.kh, ci = k / (g.kw * g.kh);
	KTap t;
	t.off = (ci * g.H + i * g.dh) * g.W + j * g.dw;
	t.ij = (i * g.dh) | ((j * g.dw) << 16);
	return t;
}

// Forward: y[n][co][hw] = sum_k w[co][k] * col_n[k][hw]  (+ bias[co]).  GEMM rows = co, columns = the pixels of the
// whole batch (n, hw) in one run, so that small images fill the column tiles together.  A thread stages the same
// column in every k-step (the tile's columns divide the workgroup's threads), so its pixel is decomposed once; every
// load is issued whatever the position, from an address that lies inside the operand (see GemmCore::run).
template <int BM, int BN, int BK, int WM, int WN, bool TAB>
__global__ __launch_bounds__(WM* WN * 64) void conv2d_forward_kernel(ConvGeo g, const float* x, const float* w, const float* bias, float* y)
{
	typedef GemmCore<BM, BN, BK, WM, WN, false, true> Core;
	static_assert(Core::T % BN == 0 && (BM * BK) % Core::T == 0 && (BN * BK) % Core::T == 0, "a thread's column is the same in every fetch");
	__shared__ float lds[Core::LDS_FLOATS];
	__shared__ KTap ktab[TAB ? MAX_KTAB : 1];  // TAB: Cin*kh*kw <= MAX_KTAB (the host picks the instantiation)
	__shared__ int col_img[BN], col_hw[BN];  // for the stores: image and pixel of every column of the tile (-1: none)

	const int Kc = g.Cin * g.kh * g.kw, HW = g.Ho * g.Wo;
	const int cols = g.N * HW;  // below 2^31 (checked by the host)
	const int tiles_n = (int)(((int64_t)cols + BN - 1) / BN);
	const int m0 = (blockIdx.x / tiles_n) * BM;
	const int n0 = (blockIdx.x % tiles_n) * BN;
	if (TAB) {
		for (int k = threadIdx.x; k < Kc; k += Core::T) ktab[k] = make_tap(g, k);
	}
	// this thread's column
	const unsigned col = (unsigned)n0 + threadIdx.x % BN;
	const bool col_ok = col < (unsigned)cols;
	const int img = (int)(min(col, (unsigned)cols - 1) / (unsigned)HW), hw = (int)(min(col, (unsigned)cols - 1) - (unsigned)img * HW);
	const int ho = hw / g.Wo, wo = hw - ho * g.Wo;
	const int yy = ho * g.sh - g.ph, xx = wo * g.sw - g.pw;
	const float* xi = x + (int64_t)img * g.Cin * g.H * g.W;
	const int pix = yy * g.W + xx;  // the top left tap of channel 0 (may lie outside the image)
	if (threadIdx.x < BN) {
		col_img[threadIdx.x] = col_ok ? img : -1;
		col_hw[threadIdx.x] = hw;
	}
	__syncthreads();

	// (conditions joined with & rather than &&: no branches between the loads)
	auto fetch_a = [&](int row, int k, bool& inside) -> float {
		inside = (m0 + row < g.Cout) & (k < Kc);
		return w[(int64_t)min(m0 + row, g.Cout - 1) * Kc + min(k, Kc - 1)];
	};
	auto fetch_b = [&](int, int k, bool& inside) -> float {
		const KTap t = TAB ? ktab[min(k, Kc - 1)] : make_tap(g, min(k, Kc - 1));
		const int ty = yy + (t.ij & 0xFFFF), tx = xx + (t.ij >> 16);
		inside = col_ok & (k < Kc) & ((unsigned)ty < (unsigned)g.H) & ((unsigned)tx < (unsigned)g.W);
		return xi[(pix + t.off) & -(int)inside];  // offset 0 for what lies outside; a mask, not a choice: a choice becomes a branch around the table read
	};

	v16f acc[Core::FM][Core::FN];
	Core::run(lds, 0, Kc, fetch_a, fetch_b, acc);
	Core::for_each(acc, [&](int row, int c, float v) {
		const int co = m0 + row, im = col_img[c];
		if (co < g.Cout && im >= 0) y[((int64_t)im * g.Cout + co) * HW + col_hw[c]] = bias ? v + bias[co] : v;
	});
}

// Weight gradient: dw[co][k] = sum_n sum_hw dy[n][co][hw] * col_n[k][hw].  GEMM rows = co, columns = k, reduction
// over the pixels of the whole batch (n, hw) in one run.  Workgroup (tile, slice) reduces one slice of that run and
// writes a partial [Cout x Kc] matrix; conv_reduce_partials adds the partials in a fixed order.  A thread stages the
// same pixel offset of every k-step, so the pixel is decomposed once per step; loads are unconditional as in the
// forward kernel.
template <int BM, int BN, int BK, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void conv2d_wgrad_kernel(ConvGeo g, const float* x, const float* dy, float* partial, int64_t slice_len)
{
	typedef GemmCore<BM, BN, BK, WM, WN, false, false> Core;
	static_assert(Core::T % BK == 0 && (BM * BK) % Core::T == 0 && (BN * BK) % Core::T == 0, "a thread's pixel offset is the same in every fetch of a step");
	__shared__ float lds[Core::LDS_FLOATS];
	__shared__ KTap ktab[BN];

	const int Kc = g.Cin * g.kh * g.kw, HW = g.Ho * g.Wo;
	const int R = g.N * HW;  // below 2^31 (checked by the host)
	const int tiles_n = (Kc + BN - 1) / BN;
	const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;
	const int r0 = (int)(blockIdx.y * slice_len), r1 = (int)min((int64_t)R, r0 + slice_len);
	float* out = partial + (int64_t)blockIdx.y * g.Cout * Kc;
	if (threadIdx.x < BN) ktab[threadIdx.x] = make_tap(g, min(n0 + (int)threadIdx.x, Kc - 1));
	__syncthreads();
	const int64_t in_image = (int64_t)g.Cin * g.H * g.W;

	auto fetch_a = [&](int row, int rr, bool& inside) -> float {
		const int r = min(rr, r1 - 1);
		const int img = r / HW, hw = r - img * HW;
		inside = (m0 + row < g.Cout) & (rr < r1);
		return dy[((int64_t)img * g.Cout + min(m0 + row, g.Cout - 1)) * HW + hw];
	};
	auto fetch_b = [&](int row, int rr, bool& inside) -> float {
		const int r = min(rr, r1 - 1);
		const int img = r / HW, hw = r - img * HW;
		const int ho = hw / g.Wo, wo = hw - ho * g.Wo;
		const KTap t = ktab[row];
		const int yy = ho * g.sh - g.ph, xx = wo * g.sw - g.pw;
		const int ty = yy + (t.ij & 0xFFFF), tx = xx + (t.ij >> 16);
		inside = (n0 + row < Kc) & (rr < r1) & ((unsigned)ty < (unsigned)g.H) & ((unsigned)tx < (unsigned)g.W);
		return x[img * in_image + ((yy * g.W + xx + t.off) & -(int)inside)];
	};

	v16f acc[Core::FM][Core::FN];
	Core::run(lds, r0, r1, fetch_a, fetch_b, acc);
	Core::for_each(acc, [&](int row, int col, float v) {
		const int co = m0 + row, k = n0 + col;
		if (co < g.Cout && k < Kc) out[(int64_t)co * Kc + k] = v;
	});
}

// Data gradient for any stride: dx[n][ci][y][x] = sum over (co, i, j) of dy[n][co][oy][ox] * w[co][ci][i][j] with
// oy = (y + ph - i) / sh, ox = (x + pw - j) / sw where those divide and lie inside dy.  GEMM rows = ci, columns = input
// pixels, reduction over (co, i, j).  A pixel is reached only through the tap rows i = (y + ph) mod sh (+ sh, + 2 sh ...)
// and the tap columns alike, so the pixels are taken class by class (blockIdx.y = (y mod sh, x mod sw)): the columns of
// a tile are pixels of one class from the whole batch, and the reduction runs over that class's taps only, a quarter of
// the window at stride 2.  Which output row a tap row reaches from input row y (or none) is tabulated per column of
// the tile in LDS, likewise for the columns, so a gather costs three table reads and no division.  A class without
// taps (a 1 x 1 window at stride 2 reaches one pixel in four) stores zeros.
constexpr int DG_MAXW = 16;    // window rows and columns the per-column tables hold
constexpr int DG_MAXK = 2304;  // reduction length of a class the LDS tables hold (Cout * taps of the class)
template <int BM, int BN, int BK, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void conv2d_dgrad_kernel(ConvGeo g, const float* w, const float* dy, float* dx, int max_tiles_n)
{
	typedef GemmCore<BM, BN, BK, WM, WN, false, true> Core;
	static_assert(Core::T % BN == 0 && (BM * BK) % Core::T == 0 && (BN * BK) % Core::T == 0, "a thread's column is the same in every fetch");
	__shared__ float lds[Core::LDS_FLOATS];
	__shared__ KTap ktab[DG_MAXK];             // per k = (co, tap of the class): co * Ho * Wo, and i | j << 16
	__shared__ int wtab[DG_MAXK];              // (co * Cin * kh + i) * kw + j: the weight of channel 0 for that k
	__shared__ int col_img[BN], col_hw[BN];    // for the stores: image and pixel of every column of the tile (-1: none)
	__shared__ int row_of[BN][DG_MAXW], column_of[BN][DG_MAXW];  // output row reached through tap row i (-1: none), likewise columns

	const int taps = g.kh * g.kw, HWi = g.H * g.W, HWo = g.Ho * g.Wo;
	// this workgroup's class of pixels and its taps
	const int cy = blockIdx.y / g.sw, cx = blockIdx.y % g.sw;
	const int Hc = cy < g.H ? (g.H - cy + g.sh - 1) / g.sh : 0, Wc = cx < g.W ? (g.W - cx + g.sw - 1) / g.sw : 0;
	const int i0 = (cy + g.ph) % g.sh, j0 = (cx + g.pw) % g.sw;
	const int Na = i0 < g.kh ? (g.kh - i0 + g.sh - 1) / g.sh : 0, Nb = j0 < g.kw ? (g.kw - j0 + g.sw - 1) / g.sw : 0;
	const int Kd = g.Cout * Na * Nb;
	const int cols = g.N * Hc * Wc;  // below 2^31 (checked by the host)
	const int tiles_n = (int)(((int64_t)cols + BN - 1) / BN);
	const int tn = blockIdx.x % max_tiles_n, m0 = (blockIdx.x / max_tiles_n) * BM, n0 = tn * BN;
	if (tn >= tiles_n) return;  // the classes differ in size by a row or a column
	for (int k = threadIdx.x; k < Kd; k += Core::T) {
		const int co = k / (Na * Nb), t = k - co * (Na * Nb), a = t / Nb;
		const int i = i0 + g.sh * a, j = j0 + g.sw * (t - a * Nb);
		ktab[k].off = co * HWo;
		ktab[k].ij = i | (j << 16);
		wtab[k] = (co * g.Cin * g.kh + i) * g.kw + j;
	}
	const unsigned col = (unsigned)n0 + threadIdx.x % BN;
	const bool col_ok = col < (unsigned)cols;
	const unsigned per_image = (unsigned)(Hc * Wc);
	const unsigned colc = min(col, (unsigned)cols - 1);
	const int img = (int)(colc / per_image), rem = (int)(colc - (unsigned)img * per_image);
	const int yy = cy + g.sh * (rem / Wc), xx = cx + g.sw * (rem % Wc);
	const int c = threadIdx.x % BN;
	if (threadIdx.x < BN) {
		col_img[c] = col_ok ? img : -1;
		col_hw[c] = yy * g.W + xx;
		for (int i = 0; i < g.kh; i++) {
			const int num = yy + g.ph - i, q = num / g.sh;
			row_of[c][i] = (num >= 0 && q * g.sh == num && q < g.Ho) ? q : -1;
		}
		for (int j = 0; j < g.kw; j++) {
			const int num = xx + g.pw - j, q = num / g.sw;
			column_of[c][j] = (num >= 0 && q * g.sw == num && q < g.Wo) ? q : -1;
		}
	}
	__syncthreads();
	const float* dyi = dy + (int64_t)img * g.Cout * HWo;

	auto fetch_a = [&](int row, int k, bool& inside) -> float {
		inside = (m0 + row < g.Cin) & (k < Kd);
		return w[wtab[min(k, max(Kd - 1, 0))] + min(m0 + row, g.Cin - 1) * taps];
	};
	auto fetch_b = [&](int, int k, bool& inside) -> float {
		const KTap t = ktab[min(k, max(Kd - 1, 0))];
		const int oy = row_of[c][t.ij & 0xFFFF], ox = column_of[c][t.ij >> 16];
		inside = col_ok & (k < Kd) & ((oy | ox) >= 0);
		return dyi[(t.off + oy * g.Wo + ox) & -(int)inside];
	};

	v16f acc[Core::FM][Core::FN];
	Core::run(lds, 0, Kd, fetch_a, fetch_b, acc);
	Core::for_each(acc, [&](int row, int cc, float v) {
		const int ci = m0 + row, im = col_img[cc];
		if (ci < g.Cin && im >= 0) dx[((int64_t)im * g.Cin + ci) * HWi + col_hw[cc]] = v;
	});
}

static bool dgrad_gemm_takes(const ConvGeo& g)
{
	const uint64_t class_taps = ceil_div((uint64_t)g.kh, g.sh) * ceil_div((uint64_t)g.kw, g.sw);
	return g.dh == 1 && g.dw == 1 && g.kh <= DG_MAXW && g.kw <= DG_MAXW && (uint64_t)g.Cout * class_taps <= DG_MAXK &&
	       g.sh * g.sw <= 64 && (uint64_t)g.N * g.H * g.W < (1ull << 31) && (uint64_t)g.Cout * g.Ho * g.Wo < (1ull << 31) &&
	       (uint64_t)g.Cout * g.Cin * g.kh * g.kw < (1ull << 31);
}

static int make_geo(ConvGeo& g, uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph,
                    int pw, int sh, int sw, int dh, int dw)
{
	LTEN_HIP_REQUIRE(kh > 0 && kw > 0 && sh > 0 && sw > 0 && dh > 0 && dw > 0 && ph >= 0 && pw >= 0, "conv: bad kernel geometry");
	LTEN_HIP_REQUIRE(N < 65536 && Cin < (1u << 20) && Cout < (1u << 20) && H < (1u << 15) && W < (1u << 15), "conv: dimension too large");
	LTEN_HIP_REQUIRE(Cin * H * W < (1ull << 31) && Cout * H * W < (1ull << 31), "conv: one image must stay below 2^31 elements");
	const int64_t eh = (int64_t)H + 2 * ph - ((int64_t)dh * (kh - 1) + 1), ew = (int64_t)W + 2 * pw - ((int64_t)dw * (kw - 1) + 1);
	LTEN_HIP_REQUIRE(eh >= 0 && ew >= 0, "conv: kernel larger than the padded image");
	g.N = (int)N; g.Cin = (int)Cin; g.H = (int)H; g.W = (int)W; g.Cout = (int)Cout;
	g.kh = kh; g.kw = kw; g.ph = ph; g.pw = pw; g.sh = sh; g.sw = sw; g.dh = dh; g.dw = dw;
	// l-ten/conv2d.cpp:102-103 (dilation 1) and l-ten/im_col.cu:104-107
	g.Ho = (int)(eh / sh + 1);
	g.Wo = (int)(ew / sw + 1);
	return 0;
}

// The implicit-GEMM weight gradient cuts the batch's run of pixels into slices: enough (tile, slice) pairs to fill 256
// CUs four times over, slices a multiple of the k-step and at least 256 pixels long.
static void wgrad_split(const ConvGeo& g, int& slices, int64_t& slice_len)
{
	const uint64_t R = (uint64_t)g.N * g.Ho * g.Wo, Kc = (uint64_t)g.Cin * g.kh * g.kw;
	const uint64_t tiles = ceil_div((uint64_t)g.Cout, 64) * ceil_div(Kc, 64);
	const uint64_t want = std::max<uint64_t>(1, 1024 / tiles);
	slice_len = (int64_t)(ceil_div(ceil_div(R, want), 64) * 64);
	if (slice_len < 256) slice_len = 256;
	slices = (int)ceil_div(R, (uint64_t)slice_len);
}

// The column matrices of the whole batch, col[n][k][hw] with k = (ci, i, j): a thread writes four consecutive pixels of
// one row (n, k) per step, the threads of a row side by side, several short rows to a workgroup.  The pixel count of an
// image is rounded up to a multiple of 4 in the rows of col (`pitch`, the tail zero), so every store is one of 16 bytes.
// Row (n, k) starts at col + n * image_stride + k * k_stride: [n][k][pitch] for a batch of products, or [k][all pixels of
// the batch] (image_stride = HW, pitch = HW: no padding between images) for one product over the whole batch; `vec`: the
// rows start on 16-byte boundaries.
__global__ __launch_bounds__(256) void im2col_batch_kernel(const float* __restrict__ x, ConvGeo g, float* __restrict__ col, int row_threads, int block_rows, unsigned pitch,
                                                           int64_t image_stride, int64_t k_stride, bool vec)
{
	const unsigned Kc = (unsigned)(g.Cin * g.kh * g.kw), HW = (unsigned)(g.Ho * g.Wo), taps = (unsigned)(g.kh * g.kw);
	const unsigned r = threadIdx.x / (unsigned)row_threads, q = threadIdx.x - r * row_threads;
	const unsigned n = blockIdx.y, k = blockIdx.x * block_rows + r;
	if (r >= (unsigned)block_rows || k >= Kc) return;
	const unsigned ci = k / taps, ij = k - ci * taps;
	const int i = (int)(ij / (unsigned)g.kw), j = (int)ij - i * g.kw;
	const float* xc = x + ((int64_t)n * g.Cin + ci) * g.H * g.W;
	float* out = col + (int64_t)n * image_stride + (int64_t)k * k_stride;
	for (unsigned hw = q * 4; hw < pitch; hw += row_threads * 4) {
		int ho = (int)(hw / (unsigned)g.Wo), wo = (int)hw - ho * g.Wo;
		float v[4];
#pragma unroll
		for (int e = 0; e < 4; e++) {
			const int yy = ho * g.sh - g.ph + i * g.dh, xx = wo * g.sw - g.pw + j * g.dw;
			const bool inside = ((unsigned)yy < (unsigned)g.H) & ((unsigned)xx < (unsigned)g.W) & (hw + e < HW);
			const float t = xc[(yy * g.W + xx) & -(int)inside];
			v[e] = inside ? t : 0.0f;
			if (++wo == g.Wo) { wo = 0; ho++; }
		}
		if (vec) *reinterpret_cast<float4*>(out + hw) = make_float4(v[0], v[1], v[2], v[3]);
		else {
#pragma unroll
			for (int e = 0; e < 4; e++)
				if (hw + e < pitch) out[hw + e] = v[e];
		}
	}
}

// y[n][co][hw] += bias[co], four pixels per thread
__global__ __launch_bounds__(256) void conv_add_bias_kernel(float* __restrict__ y, const float* __restrict__ bias, int Cout, int hw4, int64_t total4)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= total4) return;
	const float b = bias[(int)((idx / hw4) % Cout)];
	float4 v = reinterpret_cast<float4*>(y)[idx];
	v.x += b; v.y += b; v.z += b; v.w += b;
	reinterpret_cast<float4*>(y)[idx] = v;
}

// the same, one pixel per thread (pixel counts that are no multiple of 4)
__global__ __launch_bounds__(256) void conv_add_bias_each_kernel(float* __restrict__ y, const float* __restrict__ bias, int Cout, int hw, int64_t total)
{
	const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
	if (idx >= total) return;
	y[idx] += bias[(int)((idx / hw) % Cout)];
}

static void conv_add_bias(float* y, const float* bias, uint64_t N, uint64_t Cout, uint64_t HW)
{
	if (HW % 4 == 0 && aligned16(y)) {
		const int64_t total4 = (int64_t)(N * Cout * HW / 4);
		conv_add_bias_kernel<<<dim3((unsigned)ceil_div((uint64_t)total4, 256)), dim3(256), 0, stream()>>>(y, bias, (int)Cout, (int)(HW / 4), total4);
	} else {
		const int64_t total = (int64_t)(N * Cout * HW);
		conv_add_bias_each_kernel<<<dim3((unsigned)ceil_div((uint64_t)total, 256)), dim3(256), 0, stream()>>>(y, bias, (int)Cout, (int)HW, total);
	}
}

// Deep layers on small images that the patch kernels do not take (a stride, a window other than 3 x 3, images that fill
// less than half of a patch tile): the implicit GEMM below gathers its operand element by element and runs at 45
// TFLOP/s, the direct-to-LDS GEMM tiles at 85-90 on a column matrix that is already laid out.  With enough output
// channels to pay for writing and reading that matrix (4 bytes per 2 x Cout flops), l-ten's own scheme is ahead: the
// column matrices of the batch into library memory in one launch, one strided batch of products W x col_n straight into
// y, the bias in a pass over y (32 x 256 x 14 x 14 -> 256 channels 3 x 3: 156 us on the implicit GEMM).
// Returns -1 when the layer does not qualify or the library memory cannot be had.
static int conv_forward_by_columns(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const uint64_t Kc = (uint64_t)g.Cin * g.kh * g.kw, HW = (uint64_t)g.Ho * g.Wo, N = g.N;
	const uint64_t pitch = (HW + 3) & ~3ull;  // rows of the column matrices start on 16-byte boundaries
	const uint64_t elems = N * Kc * pitch;
	// (few output channels or pixels only under a long reduction, where the implicit GEMM's handful of tiles walk it one after
	// another: 4 x 256 x 8 x 8 -> 512 channels 5 x 5 at stride 2, 16 pixels an image, took 519 us)
	const bool long_k = Kc >= 2048 && g.Cout >= 8 && HW >= 4;
	if (!(((g.Cout >= 32 && HW >= 32) || long_k) && Kc >= 256 && (Kc % 32 == 0 || (Kc % 4 == 0 && Kc >= 512)) && aligned16(w) &&
	      elems <= (1ull << 27) && (uint64_t)g.Cin * g.H * g.W < (1ull << 30) && N * g.Cout * HW < (1ull << 40))) return -1;
	// Measured rates, on the work of whole tiles.  The implicit GEMM: 46 TFLOP/s once its 64 x 64 tiles give every CU a
	// workgroup.  The batch of products: 110 TFLOP/s on the 64 x 64 direct-to-LDS tiles and 92 on the 128 x 128 ones, which
	// sgemm_run picks when they fill the chip (a K that is no multiple of their k-step costs a second pass); 45 on the
	// 32 x 32 tiles that take a batch too small for those, again in proportion to the CUs they fill.  The column matrix is written and read at 2.5 TB/s, and the two extra launches cost 8 us.
	auto whole = [](uint64_t n, uint64_t t) { return (double)(ceil_div(n, t) * t); };
	const double implicit_us = 2.0 * whole((uint64_t)g.Cout, 64) * whole(N * HW, 64) * (double)Kc /
	                           (46e6 * std::min(1.0, (double)(ceil_div((uint64_t)g.Cout, 64) * ceil_div(N * HW, 64)) / 256.0));
	const uint64_t tiles128 = ceil_div((uint64_t)g.Cout, 128) * ceil_div(HW, 128) * N, tiles64 = ceil_div((uint64_t)g.Cout, 64) * ceil_div(HW, 64) * N;
	double gemm_us;
	if (tiles128 >= 256) gemm_us = 2.0 * whole((uint64_t)g.Cout, 128) * whole(HW, 128) * (double)(N * Kc) / 92e6;
	else if (tiles64 >= 128) gemm_us = 2.0 * whole((uint64_t)g.Cout, 64) * whole(HW, 64) * (double)(N * Kc) / (110e6 * std::min(1.0, (double)tiles64 / 256.0));
	else gemm_us = 2.0 * whole((uint64_t)g.Cout, 32) * whole(HW, 32) * (double)(N * Kc) / (45e6 * std::min(1.0, (double)(ceil_div((uint64_t)g.Cout, 32) * ceil_div(HW, 32) * N) / 256.0));
	if (Kc % 32 != 0) gemm_us *= 1.15;
	// Several images and a K in whole k-steps: one product over the pixels of the whole batch, col[k][(n, hw)], whose tiles
	// the GEMM stores image by image into y.  No tile is padded per image (196 pixels fill 3.06 tiles of 64 columns, 49
	// pixels 0.77 of one), and the images need no padding between them.
	const uint64_t P = N * HW, ppitch = (P + 3) & ~3ull;
	bool whole_batch = N >= 2 && Kc % 32 == 0 && N * g.Cout * HW < (1ull << 31) && Kc * ppitch <= (1ull << 27) && Kc * ppitch < (1ull << 30);
	if (whole_batch) {
		const double whole_us = sgemm_grouped_columns_estimate((uint64_t)g.Cout, P, Kc, nullptr);
		if (whole_us < gemm_us) gemm_us = whole_us;
		else whole_batch = false;  // (few images: a product per image on the 32 x 32 tiles fills more CUs)
	}
	if (implicit_us < 1.05 * (gemm_us + 4.0 * (double)elems / 2.5e6 + 8.0)) return -1;
	if (whole_batch) {
		float* col = static_cast<float*>(library_scratch(Kc * ppitch * sizeof(float)));
		if (col == nullptr) return -1;
		const int row_threads = (int)std::min<uint64_t>(256, pitch / 4), block_rows = 256 / row_threads;
		im2col_batch_kernel<<<dim3((unsigned)ceil_div(Kc, (uint64_t)block_rows), (unsigned)N), dim3(256), 0, stream()>>>(x, g, col, row_threads, block_rows, (unsigned)HW,
		                                                                                                             (int64_t)HW, (int64_t)ppitch, HW % 4 == 0);
		LTEN_HIP_LAUNCH_CHECK();
		int rc;
		{
			RowsReadableToPitch promise;  // (the rows of the columns are ppitch long)
			rc = sgemm_grouped_columns((uint64_t)g.Cout, P, Kc, w, Kc, col, ppitch, y, HW, (int64_t)((uint64_t)g.Cout * HW), bias);
		}
		if (rc == 0) {
			set_kernel_name("conv2d_im2col_gemm");
			return 0;
		}
		// (the tiles did not take the shape: the batch of products below)
	}
	// (behind the columns: room for the partial sums of a reduction that the GEMM entry splits, one image on a long K)
	const uint64_t behind = g.N == 1 ? 65 * (uint64_t)g.Cout * HW * sizeof(float) + 4096 : 0;
	float* col = static_cast<float*>(library_scratch(elems * sizeof(float) + behind));
	if (col == nullptr) return -1;
	const int row_threads = (int)std::min<uint64_t>(256, pitch / 4), block_rows = 256 / row_threads;
	im2col_batch_kernel<<<dim3((unsigned)ceil_div(Kc, (uint64_t)block_rows), (unsigned)N), dim3(256), 0, stream()>>>(x, g, col, row_threads, block_rows, (unsigned)pitch,
	                                                                                                             (int64_t)(Kc * pitch), (int64_t)pitch, true);
	LTEN_HIP_LAUNCH_CHECK();
	int rc;
	{
		LibraryScratchHold hold(elems * sizeof(float));  // the GEMM entry must not hand the columns' memory to a split reduction
		RowsReadableToPitch promise;                     // (the columns' rows are `pitch` long, the weights' rows whole)
		rc = lten_hip_sgemm_strided_batched(0, 0, (uint64_t)g.Cout, HW, Kc, 1.0f, w, Kc, 0, col, pitch, (int64_t)(Kc * pitch), 0.0f, y, HW,
		                                    (int64_t)((uint64_t)g.Cout * HW), N);
	}
	if (rc != 0) return rc;
	if (bias != nullptr) {
		conv_add_bias(y, bias, N, (uint64_t)g.Cout, HW);
		LTEN_HIP_LAUNCH_CHECK();
	}
	set_kernel_name("conv2d_im2col_batched_gemm");
	return 0;
}

// dx[n][c][y][x] = sum over the taps (i, j) that reach the pixel of col[n][(c, i, j)][(y + ph - i) / sh][(x + pw - j) / sw],
// taps in increasing (i, j) order as in col2im_kernel; one thread per pixel, the taps of its stride class only.
__global__ __launch_bounds__(256) void col2im_batch_kernel(const float* __restrict__ col, ConvGeo g, float* __restrict__ dx, unsigned HW)
{
	// (HW: the length of a row of col, the output pixels rounded up to a multiple of 4)
	const unsigned pix = blockIdx.x * 256 + threadIdx.x, HWi = (unsigned)(g.H * g.W);
	if (pix >= HWi) return;
	const unsigned c = blockIdx.y, n = blockIdx.z;
	const int y = (int)(pix / (unsigned)g.W), x = (int)pix - y * g.W;
	const int qy = (y + g.ph) / g.sh, ry = (y + g.ph) - qy * g.sh, qx = (x + g.pw) / g.sw, rx = (x + g.pw) - qx * g.sw;
	const float* cc = col + ((int64_t)n * g.Cin + c) * (g.kh * g.kw) * HW;
	float s = 0.0f;
	for (int i = ry, yy = qy; i < g.kh && yy >= 0; i += g.sh, yy--) {
		if (yy >= g.Ho) continue;
		for (int j = rx, xx = qx; j < g.kw && xx >= 0; j += g.sw, xx--) {
			if (xx >= g.Wo) continue;
			s += cc[(unsigned)(i * g.kw + j) * HW + (unsigned)(yy * g.Wo + xx)];
		}
	}
	dx[((int64_t)n * g.Cin + c) * HWi + pix] = s;
}

// rows of `cols` floats copied into rows of `pitch` floats, the tail of every row zero
__global__ __launch_bounds__(256) void pad_rows_f32_kernel(const float* __restrict__ src, float* __restrict__ dst, int rows, int cols, int pitch)
{
	const unsigned idx = blockIdx.x * 256 + threadIdx.x;  // (rows * pitch below 2^30: checked by the host)
	if (idx >= (unsigned)rows * (unsigned)pitch) return;
	const unsigned r = idx / (unsigned)pitch, c = idx - r * pitch;
	dst[idx] = c < (unsigned)cols ? src[r * (unsigned)cols + c] : 0.0f;
}

// The data gradient with a stride, l-ten's decomposition (l-ten/backprop.cpp:2022-2028: col = W^T dy_n, then col2im) done
// once for the batch: one strided batch of TN products into column matrices in library memory, one col2im launch.
// Returns -1 when the layer does not qualify or the memory cannot be had.
static int conv_dgrad_by_columns(const ConvGeo& g, const float* w, const float* dy, float* dx)
{
	const uint64_t Kc = (uint64_t)g.Cin * g.kh * g.kw, HW = (uint64_t)g.Ho * g.Wo, N = g.N;
	// rows of both operands and of the columns on 16-byte boundaries: what is not so already is copied into padded rows
	const uint64_t kpitch = (Kc + 3) & ~3ull, hpitch = (HW + 3) & ~3ull;
	const uint64_t elems = N * Kc * hpitch;
	if (!(g.Cout >= 4 && aligned16(w) && aligned16(dy) && elems <= (1ull << 27) && (uint64_t)g.H * g.W < (1ull << 30) && g.Cin < 65536 &&
	      (uint64_t)g.Cout * kpitch < (1ull << 30) && N * g.Cout * hpitch < (1ull << 30))) return -1;
	const uint64_t w_elems = kpitch != Kc ? (uint64_t)g.Cout * kpitch : 0, dy_elems = hpitch != HW ? N * g.Cout * hpitch : 0;
	float* col = static_cast<float*>(library_scratch((elems + w_elems + dy_elems) * sizeof(float)));
	if (col == nullptr) return -1;
	const float* wp = w;
	const float* dyp = dy;
	if (w_elems != 0) {
		float* padded = col + elems;
		pad_rows_f32_kernel<<<dim3((unsigned)ceil_div(w_elems, 256)), dim3(256), 0, stream()>>>(w, padded, g.Cout, (int)Kc, (int)kpitch);
		LTEN_HIP_LAUNCH_CHECK();
		wp = padded;
	}
	if (dy_elems != 0) {
		float* padded = col + elems + w_elems;
		pad_rows_f32_kernel<<<dim3((unsigned)ceil_div(dy_elems, 256)), dim3(256), 0, stream()>>>(dy, padded, (int)(N * g.Cout), (int)HW, (int)hpitch);
		LTEN_HIP_LAUNCH_CHECK();
		dyp = padded;
	}
	int rc;
	{
		LibraryScratchHold hold((elems + w_elems + dy_elems) * sizeof(float));
		RowsReadableToPitch promise;  // (padded copies, or rows that are whole multiples of four floats as they are)
		rc = lten_hip_sgemm_strided_batched(1, 0, Kc, HW, (uint64_t)g.Cout, 1.0f, wp, kpitch, 0, dyp, hpitch, (int64_t)((uint64_t)g.Cout * hpitch), 0.0f, col,
		                                    hpitch, (int64_t)(Kc * hpitch), N);
	}
	if (rc != 0) return rc;
	col2im_batch_kernel<<<dim3((unsigned)ceil_div((uint64_t)g.H * g.W, 256), (unsigned)g.Cin, (unsigned)N), dim3(256), 0, stream()>>>(col, g, dx, (unsigned)hpitch);
	LTEN_HIP_LAUNCH_CHECK();
	set_kernel_name("conv2d_dgrad_batched_gemm_col2im");
	return 0;
}

// The column matrix of the whole batch with a row per output pixel, colT[(n, hw)][k], k = (ci, i, j), rows `pitch` floats
// long (a multiple of 4, the tail zero): a thread writes four consecutive k of one pixel.
__global__ __launch_bounds__(256) void im2col_rows_kernel(const float* __restrict__ x, ConvGeo g, float* __restrict__ colT, unsigned pitch, unsigned total4)
{
	const unsigned t = blockIdx.x * 256 + threadIdx.x;
	if (t >= total4) return;
	const unsigned kq = pitch / 4, p = t / kq, k0 = (t - p * kq) * 4;
	const unsigned HW = (unsigned)(g.Ho * g.Wo), taps = (unsigned)(g.kh * g.kw), Kc = (unsigned)g.Cin * taps;
	const unsigned n = p / HW, hw = p - n * HW, ho = hw / (unsigned)g.Wo, wo = hw - ho * g.Wo;
	int ci = (int)(k0 / taps), r = (int)(k0 - ci * taps), i = r / g.kw, j = r - i * g.kw;
	const int y0 = (int)ho * g.sh - g.ph, x0 = (int)wo * g.sw - g.pw;
	const float* xn = x + (int64_t)n * g.Cin * g.H * g.W;
	float v[4];
#pragma unroll
	for (int e = 0; e < 4; e++) {
		const bool inside = (k0 + e < Kc) & ((unsigned)(y0 + i) < (unsigned)g.H) & ((unsigned)(x0 + j) < (unsigned)g.W);
		const float f = xn[((ci * g.H + y0 + i) * g.W + x0 + j) & -(int)inside];
		v[e] = inside ? f : 0.0f;
		if (++j == g.kw) {
			j = 0;
			if (++i == g.kh) { i = 0; ci++; }
		}
	}
	*reinterpret_cast<float4*>(colT + (int64_t)p * pitch + k0) = make_float4(v[0], v[1], v[2], v[3]);
}

// out[(n * HW + hw) * pitch + co] = in[(n * Cout + co) * HW + hw] (0 for co >= Cout): 32 x 32 tiles through LDS
__global__ __launch_bounds__(256) void pixels_major_kernel(const float* __restrict__ in, float* __restrict__ out, int Cout, int HW, int pitch)
{
	__shared__ float tile[32][33];
	const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5, n = blockIdx.z;
#pragma unroll
	for (int r = 0; r < 4; r++) {
		const int co = blockIdx.y * 32 + ty + 8 * r, hw = blockIdx.x * 32 + tx;
		tile[ty + 8 * r][tx] = (co < Cout && hw < HW) ? in[((int64_t)n * Cout + co) * HW + hw] : 0.0f;
	}
	__syncthreads();
#pragma unroll
	for (int r = 0; r < 4; r++) {
		const int hw = blockIdx.x * 32 + ty + 8 * r, co = blockIdx.y * 32 + tx;
		if (hw < HW && co < pitch) out[((int64_t)n * HW + hw) * pitch + co] = tile[tx][ty + 8 * r];
	}
}

// The weight gradient over few output pixels in all (small maps, small batches): the implicit GEMM's tiles each walk a
// reduction of a few k-steps, most of their time is prologue and epilogue (32 x 512 x 7 x 7 -> 512 channels 3 x 3: 36
// TFLOP/s; one image: 4).  With the batch's columns and dy both laid out with a row per pixel, dw = dyT^T colT is one
// plain TN product over all pixels, which the GEMM entry places as it does any other (the direct-to-LDS tiles, a split
// reduction when the output is small).  `current_us`: the estimate for the kernel that would run otherwise.
// Returns -1 when the layer does not qualify or the library memory cannot be had.
static int conv_wgrad_by_columns(const ConvGeo& g, const float* x, const float* dy, float* dw, double current_us)
{
	const uint64_t Kc = (uint64_t)g.Cin * g.kh * g.kw, HW = (uint64_t)g.Ho * g.Wo, N = g.N, Cout = g.Cout;
	const uint64_t P = N * HW, kp = (Kc + 3) & ~3ull, cp = (Cout + 3) & ~3ull;
	if (!(P <= 8192 && Cout >= 32 && Kc >= 64 && P * kp <= (1ull << 27) && (uint64_t)g.Cin * g.H * g.W < (1ull << 30) && aligned16(dw))) return -1;
	auto whole = [](uint64_t n, uint64_t t) { return (double)(ceil_div(n, t) * t); };
	const double flops = 2.0 * (double)(Cout * Kc) * (double)P;
	if (flops < 1e8) return -1;  // (a handful of launches either way)
	const uint64_t tiles128 = ceil_div(Cout, 128) * ceil_div(Kc, 128), tiles64 = ceil_div(Cout, 64) * ceil_div(Kc, 64), tiles32 = ceil_div(Cout, 32) * ceil_div(Kc, 32);
	const bool splits = tiles32 <= 256 && P >= 1536;
	double gemm_us;
	// (sgemm_run: the direct-to-LDS tiles from K = 256 in whole k-steps of 32, or from 512 with a second pass for the rest)
	if (tiles64 >= 65 && tiles64 < 256 && P >= 4096 && Cout >= 128 && Kc >= 128)  // (a long reduction into a mid-size output: slices of K on the same tiles)
		gemm_us = flops / 95e6 + 8.0;
	else if ((tiles128 >= 128 || tiles64 >= 128) && P >= 256 && (P % 32 == 0 || P >= 512))
		gemm_us = 2.0 * whole(Cout, tiles128 >= 128 ? 128 : 64) * whole(Kc, tiles128 >= 128 ? 128 : 64) * (double)P / 85e6 * (P % 32 == 0 ? 1.0 : 1.15) + 8.0;
	else
		gemm_us = flops / (45e6 * (splits ? 1.0 : std::min(1.0, (double)tiles32 / 256.0))) + (splits ? 8.0 : 4.0);
	// (the two copies: 4 bytes per column element at 2.5 TB/s and 12 us for the launches; a margin of 15 %)
	if (current_us < 1.15 * (gemm_us + 4.0 * (double)(P * kp) / 2.5e6 + 12.0)) return -1;
	const uint64_t behind = splits ? 65 * Cout * Kc * sizeof(float) + 4096 : 0;
	const uint64_t held = (P * kp + P * cp) * sizeof(float);
	float* colT = static_cast<float*>(library_scratch(held + behind));
	if (colT == nullptr) return -1;
	float* dyT = colT + P * kp;
	const unsigned total4 = (unsigned)(P * (kp / 4));
	im2col_rows_kernel<<<dim3((unsigned)ceil_div((uint64_t)total4, 256)), dim3(256), 0, stream()>>>(x, g, colT, (unsigned)kp, total4);
	LTEN_HIP_LAUNCH_CHECK();
	pixels_major_kernel<<<dim3((unsigned)ceil_div(HW, 32), (unsigned)ceil_div(cp, 32), (unsigned)N), dim3(256), 0, stream()>>>(dy, dyT, (int)Cout, (int)HW, (int)cp);
	LTEN_HIP_LAUNCH_CHECK();
	int rc;
	{
		LibraryScratchHold hold(held);
		RowsReadableToPitch promise;  // (both copies have rows of whole multiples of four floats)
		rc = lten_hip_sgemm(1, 0, Cout, Kc, P, 1.0f, dyT, cp, colT, kp, 0.0f, dw, Kc);
	}
	if (rc == 0) set_kernel_name("conv2d_wgrad_columns_gemm");
	return rc;
}

// Picks the forward kernel for a geometry (x, w, y non-null, non-empty problem).
static int conv_forward_dispatch(const ConvGeo& g, const float* x, const float* w, const float* bias, float* y)
{
	const uint64_t Cout = g.Cout, N = g.N;
	const int HW = g.Ho * g.Wo;
	const int variant = get_option(OPT_CONV_VARIANT);  // 0 automatic, 1 implicit GEMM for every shape
	if (variant == 0 && conv_fewin_takes(g, x, y)) return conv_fewin_forward(g, x, w, bias, y);
	if (variant != 1 && conv_smallk_takes(g)) return conv_smallk_forward(g, x, w, bias, y);
	if (variant == 0 && conv_fewout_takes(g, x, y)) return conv_fewout_forward(g, x, w, bias, y, false);
	// A 1 x 1 layer (stride 1, no padding) is a product per image of the weights with the image as it lies in memory,
	// y[n] = W[Cout x Cin] x[n][Cin x HW]: a strided batch of plain GEMMs with the weights as the operand all share
	// (32 x 256 x 56 x 56 -> 64 channels: 44 us there, 70 us on the implicit GEMM below; 32 x 512 x 14 x 14 -> 512: 38
	// against 73 us; the stride-1 data gradient of such a layer comes the same way).  The GEMM has no per-row bias: a
	// bias is added in a pass over y, which pays while y is small beside the work (estimates: 75 TFLOP/s here, 48 on the
	// implicit GEMM, the pass at 4 TB/s + 3 us; 256 -> 64 channels yes, 64 -> 256 no).
	if (variant == 0 && g.kh == 1 && g.kw == 1 && g.sh == 1 && g.sw == 1 && g.ph == 0 && g.pw == 0 && g.dh == 1 && g.dw == 1 &&
	    g.Cin >= 16 && N < 65536 && (HW % 4 == 0 || g.Cin < 256)) {  // (channel images off 16-byte boundaries: by columns, below)
		const double flops = 2.0 * (double)N * (double)Cout * HW * g.Cin, y_bytes = 4.0 * (double)N * (double)Cout * HW;
		const bool pass_pays = HW % 4 == 0 && aligned16(y) && flops / 48e6 > flops / 75e6 + 2.0 * y_bytes / 4e6 + 3.0;
		if (bias == nullptr || pass_pays) {
			int rc = lten_hip_sgemm_strided_batched(0, 0, Cout, (uint64_t)HW, (uint64_t)g.Cin, 1.0f, w, (uint64_t)g.Cin, 0, x, (uint64_t)HW,
			                                        (int64_t)g.Cin * HW, 0.0f, y, (uint64_t)HW, (int64_t)Cout * HW, N);
			if (rc == 0 && bias != nullptr) {
				conv_add_bias(y, bias, N, Cout, (uint64_t)HW);
				LTEN_HIP_LAUNCH_CHECK();
			}
			if (rc == 0) set_kernel_name("conv2d_1x1_batched_gemm");
			return rc;
		}
	}
	// variant 2: the register-staged patch kernel even where the direct-to-LDS one would run; 5: the direct-to-LDS
	// one with its four-row tile also where the two-row tile would be picked
	// (6: the direct-to-LDS one with its narrow-image tiles however few workgroups that gives)
	if ((variant == 0 || variant == 5 || variant == 6) && conv_patch_forward_takes(g, x, y) && conv_patch_fast_forward_takes(g, x, w)) return conv_patch_fast_forward(g, x, w, bias, y);
	// The register-staged patch kernel's tiles are 128 columns wide (the direct-to-LDS one above has 16 x 32 tiles for
	// narrow images): on images of at most 56 columns more than half of a tile is padding, and with fewer than 256 tiles
	// CUs stay idle; the implicit GEMM over the batch's flattened pixels is ahead there (32 x 48 x 50 x 50 -> 96
	// channels: 154 against 178 us, 4 x 64 x 126 x 126 -> 64: 82 against 90 us, 64 x 16 x 30 x 30 -> 32: 18 against 27 us).
	const uint64_t patch_tiles = ceil_div((uint64_t)g.Wo, 128) * ceil_div((uint64_t)g.Ho, 4) * ceil_div(Cout, 64) * N;
	const bool narrow = variant == 0 && (g.Wo <= 56 || patch_tiles < 256);
	if (!narrow && variant != 1 && conv_patch_forward_takes(g, x, y)) return conv_patch_forward(g, x, w, bias, y);
	if (variant == 0) {
		const int rc = conv_forward_by_columns(g, x, w, bias, y);
		if (rc >= 0) return rc;
	}
	LTEN_HIP_REQUIRE(N * HW < (1ull << 31), "conv2d_forward: the batch's output pixels must number less than 2^31 on this route");
	// at most 32 output channels: 32 x 128 tiles, unless those are fewer than the CUs (then half-empty 64 x 64 tiles,
	// twice as many: 64 x 10 x 12 x 12 -> 20 channels 5 x 5: 14.7 against 18.7 us)
	if (Cout > 32 || ceil_div(N * HW, 128) < 256) {
		set_kernel_name("conv2d_forward_64x64x32");
		const dim3 grid((unsigned)(ceil_div(Cout, 64) * ceil_div(N * HW, 64)));
		if (g.Cin * g.kh * g.kw <= MAX_KTAB) conv2d_forward_kernel<64, 64, 32, 2, 2, true><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
		else conv2d_forward_kernel<64, 64, 32, 2, 2, false><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
	} else {
		set_kernel_name("conv2d_forward_32x128x32");
		const dim3 grid((unsigned)(ceil_div(Cout, 32) * ceil_div(N * HW, 128)));
		if (g.Cin * g.kh * g.kw <= MAX_KTAB) conv2d_forward_kernel<32, 128, 32, 1, 4, true><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
		else conv2d_forward_kernel<32, 128, 32, 1, 4, false><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, y);
	}
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// dw2[ci][co][i][j] = w[co][ci][kh-1-i][kw-1-j]: the weights of the stride-1 convolution that maps dy to dx.
__global__ __launch_bounds__(256) void flip_weights_kernel(const float* __restrict__ w, float* __restrict__ w2, int Cout, int Cin, int kh, int kw)
{
	const int total = Cout * Cin * kh * kw;
	for (int idx = blockIdx.x * 256 + threadIdx.x; idx < total; idx += gridDim.x * 256) {
		const int j = idx % kw, i = (idx / kw) % kh, co = (idx / (kw * kh)) % Cout, ci = idx / (kw * kh * Cout);
		w2[idx] = w[((co * Cin + ci) * kh + (kh - 1 - i)) * kw + (kw - 1 - j)];
	}
}

// Data gradient of a first layer (at most four input channels) with a short reduction, any window, stride 1: P
// threads per element of dx share its Cout * kh * kw products (product r of an element goes to thread r % P; a table
// in LDS turns r into channel and tap), every load is issued whatever the position (clamped into the image, the weight
// replaced by zero outside), eight products a thread are in flight, and the P sums are added by lane exchanges.
// Weights sit in LDS, dy comes through the caches (neighbouring elements read neighbouring values); one load
// instruction per product is what bounds it.  The transposed problem has one to four output channels, which leaves
// the MFMA tiles of the forward kernels almost empty (l-ten's MNIST layer, 64 x 1 x 28 x 28 <- 10 channels 5 x 5:
// 41 us there, 13 us here).
template <int P>
__global__ __launch_bounds__(256) void conv2d_dgrad_direct_kernel(ConvGeo g, const float* __restrict__ w, const float* __restrict__ dy, float* __restrict__ dx)
{
	extern __shared__ float s_w[];  // [Cout][Cin][kh][kw] as in memory, then the table
	constexpr int U = 8;  // products in flight per thread
	const int taps = g.kh * g.kw, wcount = g.Cout * g.Cin * taps, R = g.Cout * taps, Rp = (R + P * U - 1) / (P * U) * (P * U);
	int* s_tab = reinterpret_cast<int*>(s_w + wcount);
	for (int i = threadIdx.x; i < wcount; i += 256) s_w[i] = w[i];
	for (int r = threadIdx.x; r < Rp; r += 256) {  // entries past R pad the last round: sign bit set, counted as outside
		const int co = r / taps, t = r - co * taps, i = t / g.kw;
		s_tab[r] = r < R ? (co << 16) | (i << 8) | (t - i * g.kw) : (int)0x80000000;
	}
	__syncthreads();
	const uint32_t gid = blockIdx.x * 256u + threadIdx.x, total = (uint32_t)g.N * g.Cin * g.H * g.W;
	const int p = (int)(gid % P);
	const bool live = gid / P < total;  // every lane stays for the exchange below
	const uint32_t idx = live ? gid / P : 0;
	const int xw = (int)(idx % (uint32_t)g.W), t1 = (int)(idx / (uint32_t)g.W);
	const int yh = t1 % g.H, t2 = t1 / g.H;
	const int ci = t2 % g.Cin, n = t2 / g.Cin;
	const int plane = g.Ho * g.Wo;
	const float* dyn = dy + (int64_t)n * g.Cout * plane;
	const float* wci = s_w + ci * taps;
	float acc = 0.0f;
	for (int r0 = p; r0 < Rp; r0 += P * U) {
#pragma unroll
		for (int u = 0; u < U; ++u) {
			const int e = s_tab[r0 + u * P];
			const int co = (e >> 16) & 0x7fff, i = (e >> 8) & 255, j = e & 255;
			const int oy = yh + g.ph - i, ox = xw + g.pw - j;  // the output position whose tap (i, j) lies on this input position
			const bool inside = e >= 0 && (unsigned)oy < (unsigned)g.Ho && (unsigned)ox < (unsigned)g.Wo;
			const float v = dyn[co * plane + min(max(oy, 0), g.Ho - 1) * g.Wo + min(max(ox, 0), g.Wo - 1)];
			const float wv = wci[co * g.Cin * taps + i * g.kw + j];
			acc += v * (inside ? wv : 0.0f);
		}
	}
#pragma unroll
	for (int d = 1; d < P; d *= 2) acc += __shfl_xor(acc, d, 64);
	if (live && p == 0) dx[idx] = acc;
}

static bool dgrad_direct_takes(const ConvGeo& g)
{
	const uint64_t taps = (uint64_t)g.kh * g.kw, wcount = (uint64_t)g.Cout * g.Cin * taps;
	return g.sh == 1 && g.sw == 1 && g.dh == 1 && g.dw == 1 && g.Cin <= 4 && g.kh <= 255 && g.kw <= 255 && g.Cout <= 1024 &&
	       (wcount + g.Cout * taps + 64) * 4 <= 48 * 1024 && g.Cout * taps <= 1024 &&
	       (uint64_t)g.N * g.Cin * g.H * g.W < (1ull << 28) && (uint64_t)g.Cout * g.Ho * g.Wo < (1ull << 31);
}

// The data gradient of a stride-1 convolution is a stride-1 convolution of dy with the flipped, channel-transposed
// weights and pads k - 1 - p; it then runs on the forward kernels.
static bool dgrad_as_forward(const ConvGeo& g)
{
	return g.sh == 1 && g.sw == 1 && g.ph <= g.kh - 1 && g.pw <= g.kw - 1 && (uint64_t)g.Cout * g.Cin * g.kh * g.kw < (1ull << 31);
}

}  // namespace lten_hip

using namespace lten_hip;

template <typename T>
static int im2col_run(const T* im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, T* col)
{
	ConvGeo g;
	if (int rc = make_geo(g, 1, C, H, W, 1, kh, kw, ph, pw, sh, sw, dh, dw)) return rc;
	const int64_t total = (int64_t)C * kh * kw * g.Ho * g.Wo;
	if (total == 0) return 0;
	LTEN_HIP_REQUIRE(im && col, "im2col: null pointer");
	im2col_kernel<T><<<dim3((unsigned)std::min<uint64_t>(ceil_div(total, 256), 65536)), dim3(256), 0, stream()>>>(im, g, col);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

template <typename T>
static int col2im_run(const T* col, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, T* im)
{
	ConvGeo g;
	if (int rc = make_geo(g, 1, C, H, W, 1, kh, kw, ph, pw, sh, sw, dh, dw)) return rc;
	const int64_t total = (int64_t)C * H * W;
	if (total == 0) return 0;
	LTEN_HIP_REQUIRE(im && col, "col2im: null pointer");
	col2im_kernel<T><<<dim3((unsigned)std::min<uint64_t>(ceil_div(total, 256), 65536)), dim3(256), 0, stream()>>>(col, g, im);
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

extern "C" {

// the three instantiations of l-ten/im_col.cu:199-218 each
int lten_hip_im2col_f32(const float* im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, float* col)
{
	return im2col_run<float>(im, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, col);
}
int lten_hip_im2col_i32(const int32_t* im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, int32_t* col)
{
	return im2col_run<int32_t>(im, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, col);
}
int lten_hip_im2col_u8(const uint8_t* im, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, uint8_t* col)
{
	return im2col_run<uint8_t>(im, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, col);
}
int lten_hip_col2im_f32(const float* col, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, float* im)
{
	return col2im_run<float>(col, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, im);
}
int lten_hip_col2im_i32(const int32_t* col, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, int32_t* im)
{
	return col2im_run<int32_t>(col, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, im);
}
int lten_hip_col2im_u8(const uint8_t* col, int C, int H, int W, int kh, int kw, int ph, int pw, int sh, int sw, int dh, int dw, uint8_t* im)
{
	return col2im_run<uint8_t>(col, C, H, W, kh, kw, ph, pw, sh, sw, dh, dw, im);
}

int lten_hip_conv2d_forward_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph,
                                int pw, int sh, int sw, const float* x, const float* w, const float* bias, float* y)
{
	ConvGeo g;
	if (int rc = make_geo(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, 1, 1)) return rc;
	if (N == 0 || Cout == 0 || g.Ho * g.Wo == 0) return 0;
	LTEN_HIP_REQUIRE(x && w && y, "conv2d_forward: null pointer");
	return conv_forward_dispatch(g, x, w, bias, y);
}

uint64_t lten_hip_conv2d_dgrad_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh,
                                               int kw, int ph, int pw, int sh, int sw)
{
	ConvGeo g;
	if (make_geo(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, 1, 1)) return 0;
	const uint64_t Kc = Cin * kh * kw;
	return sizeof(float) * std::max<uint64_t>(Cout * Kc, Kc * (uint64_t)g.Ho * g.Wo) + 16;
}

int lten_hip_conv2d_dgrad_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph,
                              int pw, int sh, int sw, const float* w, const float* dy, float* dx, void* workspace)
{
	ConvGeo g;
	if (int rc = make_geo(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, 1, 1)) return rc;
	const uint64_t HW = (uint64_t)g.Ho * g.Wo, Kc = Cin * kh * kw;
	if (N == 0 || Cin * H * W == 0) return 0;
	LTEN_HIP_REQUIRE(dx != nullptr, "conv2d_dgrad: dx is null");
	if (Cout == 0 || HW == 0) return lten_hip_zero(dx, N * Cin * H * W * sizeof(float));
	LTEN_HIP_REQUIRE(w && dy && workspace, "conv2d_dgrad: null pointer");
	float* work = static_cast<float*>(workspace);
	// Few images of at most 16 columns: l-ten's decomposition (GEMM + col2im per image) is ahead of a convolution with so
	// few columns that its workgroups walk a long reduction one after another (8 x 256 x 14 x 14 <- 512 channels: 166
	// against 237 us; at 16 images the two launches per image cost more: 16 x 64 x 8 x 8 <- 64: 160 against 41 us, and
	// so they do when the reduction is short: 8 x 64 x 8 x 8 <- 64 channels 89 us)
	const bool few_narrow = get_option(OPT_CONV_VARIANT) == 0 && W <= 16 && N <= 8 && Cin > 32 && Cout * kh * kw >= 2048;
	if (dgrad_as_forward(g) && few_narrow) {
		// ... unless the transposed problem is one for the column matrices of the whole batch (8 x 256 x 14 x 14 <- 256: 60 us)
		ConvGeo g2;
		if (int rc = make_geo(g2, N, Cout, g.Ho, g.Wo, Cin, kh, kw, kh - 1 - ph, kw - 1 - pw, 1, 1, 1, 1)) return rc;
		if (g2.Ho == (int)H && g2.Wo == (int)W) {
			flip_weights_kernel<<<dim3((unsigned)std::min<uint64_t>(ceil_div(Cout * Kc, 256), 1024)), dim3(256), 0, stream()>>>(w, work, (int)Cout, (int)Cin, kh, kw);
			LTEN_HIP_LAUNCH_CHECK();
			const int rc = conv_forward_by_columns(g2, dy, work, nullptr, dx);
			if (rc >= 0) return rc;
		}
	}
	if (dgrad_as_forward(g) && get_option(OPT_CONV_VARIANT) != 1 && !few_narrow) {
		ConvGeo gt;  // the transposed problem: dy is the input, dx the output
		if (int rc = make_geo(gt, N, Cout, g.Ho, g.Wo, Cin, kh, kw, kh - 1 - ph, kw - 1 - pw, 1, 1, 1, 1)) return rc;
		// (the vector-ALU stream wants pixels to spread over the chip: one image of 56 x 56 <- 384 channels took 239 us on it)
		if (get_option(OPT_CONV_VARIANT) == 0 && gt.Ho == (int)H && gt.Wo == (int)W && !conv_smallk_takes(gt) && conv_fewout_takes(gt, dy, dx) &&
		    (N * H * W >= 32768 || Cout <= 64))
			return conv_fewout_forward(gt, dy, w, nullptr, dx, true);  // reads w transposed and flipped in place
		// Few input channels, or few tiles of the transposed problem under a long reduction: as a convolution of dy the
		// gradient fills a fraction of its tiles' rows (10 channels of 32) or leaves most CUs idle, and l-ten's decomposition
		// done once for the batch is ahead while its columns stay below 100 MB (l-ten's own MNIST network, 1024 x 10 x 12 x 12
		// <- 20 channels 5 x 5: 115 -> 93 us; its first layer 1024 x 1 x 28 x 28 <- 10: 105 -> 77 us on the element-wise
		// kernel below, which keeps the small batches; 64 x 20 x 8 x 8 <- 50 channels 5 x 5: 61 -> 17 us).
		// With few input channels an estimate of both decides: the columns are written and read at about 1.2 TB/s; as a
		// convolution of dy the gradient runs on the 3 x 3 patch kernels at about 20 TFLOP/s where they take it, else on
		// the implicit GEMM at 45 TFLOP/s of tile rows, 32 or 64 of them for the few channels (16 x 16 x 64 x 64 <- 16
		// channels 3 x 3: columns 44, patch kernel 18 us; 64 x 16 x 32 x 32 <- 32: 46 against 30 us, <- 64: 44 against 55 us;
		// 128 x 3 x 32 x 32 <- 64 channels 5 x 5: 48 against 272 us).
		bool few_channels = false;
		if (Cin <= 16 && (N * Cin * H * W >= (1u << 16) || 2.0 * (double)(N * HW) * (double)(Cout * Kc) >= 2e7) && gt.Ho == (int)H && gt.Wo == (int)W) {
			const double macs = 2.0 * (double)(N * H * W) * Cout * kh * kw;  // per output channel of the convolution of dy
			const uint64_t patch_tiles = ceil_div(W, 128) * ceil_div(H, 4) * ceil_div(Cin, 64) * N;
			const bool on_patches = conv_patch_forward_takes(gt, dy, dx) && (conv_patch_fast_forward_takes(gt, dy, work) || (W > 56 && patch_tiles >= 256));
			const double tile_rows = ceil_div(N * H * W, 128) >= 256 ? 32.0 : 64.0;
			const double as_convolution_us = on_patches ? 10.0 + macs * Cin / 20e6 : 14.0 + macs * tile_rows / 45e6;
			few_channels = 15.0 + 4.0 * (double)(Kc * HW * N) / 1.2e6 < as_convolution_us;
		}
		// (small inputs only where the work is large all the same: 4 x 3 x 14 x 14 <- 1024 channels 7 x 7 took 3.8 ms as a convolution of dy)
		if (get_option(OPT_CONV_VARIANT) == 0 && kh * kw > 1 && Kc * HW * N * sizeof(float) <= (100ull << 20) &&
		    (N * Cin * H * W >= (1u << 18) / 4 || 2.0 * (double)(N * HW) * (double)(Cout * Kc) >= 2e7) &&
		    (few_channels || (ceil_div(Cin, 64) * ceil_div(N * H * W, 64) < 128 && Cout * kh * kw >= 1024))) {
			const int rc = conv_dgrad_by_columns(g, w, dy, dx);
			if (rc >= 0) return rc;
		}
		if (get_option(OPT_CONV_VARIANT) == 0 && dgrad_direct_takes(g)) {
			const uint64_t total = N * Cin * H * W;
			set_kernel_name("conv2d_dgrad_direct");
			const size_t lds = (size_t)((Cout * Kc + Cout * kh * kw + 64) * sizeof(float));
			// eight threads an element while that fills the chip (the loads of one thread wait on each other less), one
			// beyond (every load instruction of a wavefront costs the same 16 clocks, and one thread an element issues
			// the fewest of the rest): 32 x 2 x 64 x 64 <- 24 channels 4 x 4: 61 against 74 us
			if (total < 131072) conv2d_dgrad_direct_kernel<8><<<dim3((unsigned)ceil_div(total * 8, 256)), dim3(256), lds, stream()>>>(g, w, dy, dx);
			else conv2d_dgrad_direct_kernel<1><<<dim3((unsigned)ceil_div(total, 256)), dim3(256), lds, stream()>>>(g, w, dy, dx);
			LTEN_HIP_LAUNCH_CHECK();
			return 0;
		}
		flip_weights_kernel<<<dim3((unsigned)std::min<uint64_t>(ceil_div(Cout * Kc, 256), 1024)), dim3(256), 0, stream()>>>(w, work, (int)Cout, (int)Cin, kh, kw);
		LTEN_HIP_LAUNCH_CHECK();
		ConvGeo g2;
		if (int rc = make_geo(g2, N, Cout, g.Ho, g.Wo, Cin, kh, kw, kh - 1 - ph, kw - 1 - pw, 1, 1, 1, 1)) return rc;
		LTEN_HIP_REQUIRE(g2.Ho == (int)H && g2.Wo == (int)W, "conv2d_dgrad: internal geometry mismatch");
		return conv_forward_dispatch(g2, dy, work, nullptr, dx);
	}
	// A strided first layer: the rows of the implicit GEMM below are the input channels, a handful in a tile of 64, and
	// with a large window the padding costs more than l-ten's decomposition image by image does (32 x 3 x 224 x 224 <- 64
	// channels 7 x 7 stride 2: 3.8 ms below, 1.0 ms image by image; 3 x 3 and 5 x 5 windows stay below: 32 x 4 x 56 x 56
	// <- 64 channels 3 x 3 stride 2 64 against 332 us).  Estimates: the tile loop at 45 TFLOP/s of padded work; 16 us +
	// 9 us per million elements of the column buffer per image.
	const double padded_us = 2.0 * 64 * ceil_div(Cin, 64) * (double)(N * H * W) * Cout * kh * kw / ((double)sh * sw) / 45e6;
	const double by_image_us = (double)N * (16.0 + 9e-6 * (double)Kc * HW);
	const bool padded_rows = get_option(OPT_CONV_VARIANT) == 0 && Cin <= 8 && padded_us > 1.5 * by_image_us;
	// With a stride, l-ten's decomposition done once for the batch is ahead of the implicit GEMM below from about a
	// megabyte of columns on (32 x 64 x 56 x 56 <- 128 channels 3 x 3 stride 2: 130 -> 101 us; 32 x 128 x 28 x 28 <- 256:
	// 174 -> 86 us; 32 x 4 x 56 x 56 <- 64: 65 -> 15 us; the first layer above: 333 us), except for 1 x 1 windows, whose
	// columns are dy itself (32 x 64 x 56 x 56 <- 128 at stride 2: 24 against 36 us), while the layers are small: the
	// implicit GEMM runs them at 29 TFLOP/s (only the pixels that a 1 x 1 window reaches do any work, and with few of
	// them few of its tiles), the GEMM of the decomposition at 88, and the pass that spreads its result over dx takes
	// the rest (32 x 256 x 56 x 56 <- 512 at stride 2: 222 -> 148 us; 32 x 1024 x 14 x 14 <- 2048: 231 -> 97 us;
	// 4 x 512 x 28 x 28 <- 1024: 84 -> 32 us; 32 x 128 x 56 x 56 <- 256 level at 65 us and left below).
	bool one_by_one_pays = false;
	if (kh * kw == 1) {
		const double flops = 2.0 * (double)N * HW * Cout * Cin;
		const double tiles = (double)(ceil_div(Cin, 64) * ceil_div(N * HW, 64));
		const double implicit_us = std::max(20.0, flops / (29e6 * std::min(1.0, tiles / 256.0)));
		const double columns_us = 10.0 + flops / 88e6 + 4.0 * (double)(N * Cin * H * W + 2 * N * Cin * HW) / 2.5e6;
		one_by_one_pays = columns_us * 1.1 < implicit_us;
	}
	if (get_option(OPT_CONV_VARIANT) == 0 && !dgrad_as_forward(g) && (kh * kw > 1 || padded_rows || one_by_one_pays) &&
	    (N * Kc * HW >= (1u << 18) || 2.0 * (double)(N * HW) * (double)(Cout * Kc) >= 2e7)) {  // (or few columns under many channels: 64 x 8 x 8 x 8 <- 1024 at stride 2 ran image by image, 1.3 ms)
		const int rc = conv_dgrad_by_columns(g, w, dy, dx);
		if (rc >= 0) return rc;
	}
	// any stride: one implicit-GEMM launch for the batch (64 x 64 x 28 x 28 <- 128 channels at stride 2: 722 us image by image)
	if (get_option(OPT_CONV_VARIANT) == 0 && (!few_narrow || !dgrad_as_forward(g)) && !padded_rows && dgrad_gemm_takes(g)) {
		set_kernel_name("conv2d_dgrad_64x64x32");
		// one grid row per class of pixels (y mod sh, x mod sw); class (0, 0) has the most
		const uint64_t max_tiles_n = ceil_div(N * ceil_div(H, (uint64_t)sh) * ceil_div(W, (uint64_t)sw), 64);
		conv2d_dgrad_kernel<64, 64, 32, 2, 2><<<dim3((unsigned)(ceil_div(Cin, 64) * max_tiles_n), (unsigned)(sh * sw)), dim3(256), 0, stream()>>>(g, w, dy, dx, (int)max_tiles_n);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}
	// l-ten/backprop.cpp:2022-2028 per image: col = W^T dy_n (TN GEMM), then col2im
	for (uint64_t n = 0; n < N; n++) {
		if (int rc = lten_hip_sgemm(1, 0, Kc, HW, Cout, 1.0f, w, Kc, dy + n * Cout * HW, HW, 0.0f, work, HW)) return rc;
		if (int rc = lten_hip_col2im_f32(work, (int)Cin, (int)H, (int)W, kh, kw, ph, pw, sh, sw, 1, 1, dx + n * Cin * H * W)) return rc;
	}
	set_kernel_name("conv2d_dgrad_sgemm_col2im");
	return 0;
}

uint64_t lten_hip_conv2d_wgrad_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh,
                                               int kw, int ph, int pw, int sh, int sw)
{
	ConvGeo g;
	if (make_geo(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, 1, 1)) return 0;
	int slices;
	int64_t slice_len;
	wgrad_split(g, slices, slice_len);
	// enough for whichever kernel the call picks
	uint64_t parts = (uint64_t)slices;
	if (conv_smallk_takes(g)) parts = std::max<uint64_t>(parts, conv_smallk_wgrad_parts(g));
	if (conv_patch_wgrad_takes(g)) parts = std::max<uint64_t>(parts, conv_patch_wgrad_parts(g, true));
	return parts * Cout * Cin * kh * kw * sizeof(float);
}

int lten_hip_conv2d_wgrad_f32(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph,
                              int pw, int sh, int sw, const float* x, const float* dy, float* dw, void* workspace)
{
	ConvGeo g;
	if (int rc = make_geo(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, 1, 1)) return rc;
	const int64_t Kc = (int64_t)Cin * kh * kw, count = (int64_t)Cout * Kc;
	if (count == 0) return 0;
	LTEN_HIP_REQUIRE(dw != nullptr, "conv2d_wgrad: dw is null");
	if (N == 0 || g.Ho * g.Wo == 0) return lten_hip_zero(dw, count * sizeof(float));
	LTEN_HIP_REQUIRE(x && dy && workspace, "conv2d_wgrad: null pointer");
	if (get_option(OPT_CONV_VARIANT) != 1 && conv_smallk_takes(g)) {
		const int parts = conv_smallk_wgrad_parts(g);
		if (int rc = conv_smallk_wgrad(g, x, dy, static_cast<float*>(workspace), parts)) return rc;
		return conv_reduce_partials(static_cast<const float*>(workspace), parts, count, dw);
	}
	// images of at most 16 columns: an eighth of the patch kernel's 128-column tile (8 x 256 x 14 x 14 -> 512: 129 against 199 us);
	// rows that do not allow 16-byte loads, of at most 56 columns (the kernel's chunks are 64 pixels of one row):
	// 32 x 32 x 30 x 30 -> 64: 33 against 47 us, 32 x 48 x 50 x 50 -> 96: 151 against 177 us
	const bool narrow = get_option(OPT_CONV_VARIANT) == 0 && (g.Wo <= 16 || ((g.W % 4 != 0 || g.Wo % 4 != 0) && g.Wo <= 56));
	if (get_option(OPT_CONV_VARIANT) == 0) {
		// few output pixels in all: one plain product on pixel-major copies, when the estimate favours it.  What would run
		// otherwise, measured up to the 8192 output pixels P of a batch that this route takes: the patch kernel 28 us + the
		// work at 80 TFLOP/s; the implicit GEMM at 60 TFLOP/s x P / (P + 1100), 17 us or more (two launches).
		const double P = (double)N * g.Ho * g.Wo, flops = 2.0 * (double)count * P;
		const double current_us = (!narrow && conv_patch_wgrad_takes(g)) ? 28.0 + flops / 80e6 : std::max(17.0, flops / (60e6 * P / (P + 1100.0)));
		const int rc = conv_wgrad_by_columns(g, x, dy, dw, current_us);
		if (rc >= 0) return rc;
	}
	if (!narrow && get_option(OPT_CONV_VARIANT) != 1 && conv_patch_wgrad_takes(g)) {
		const int parts = conv_patch_wgrad_parts(g);
		if (int rc = conv_patch_wgrad(g, x, dy, static_cast<float*>(workspace), parts)) return rc;
		return conv_reduce_partials(static_cast<const float*>(workspace), parts, count, dw);
	}
	int parts;
	int64_t slice_len;
	wgrad_split(g, parts, slice_len);
	LTEN_HIP_REQUIRE(parts < 65536 && (uint64_t)N * g.Ho * g.Wo < (1ull << 31), "conv2d_wgrad: the batch's output pixels must number less than 2^31 on this route");
	float* partial = static_cast<float*>(workspace);
	// (also for at most 32 output channels: half-empty 64 x 64 tiles with four wavefronts are ahead of 32 x 32 tiles with
	// one: 64 x 10 x 12 x 12 -> 20 channels 5 x 5: 17.5 against 29.3 us)
	set_kernel_name("conv2d_wgrad_64x64x32");
	const dim3 grid((unsigned)(ceil_div(Cout, 64) * ceil_div(Kc, 64)), (unsigned)parts);
	conv2d_wgrad_kernel<64, 64, 32, 2, 2><<<grid, dim3(256), 0, stream()>>>(g, x, dy, partial, slice_len);
	LTEN_HIP_LAUNCH_CHECK();
	return conv_reduce_partials(partial, parts, count, dw);
}

}  // extern "C"
