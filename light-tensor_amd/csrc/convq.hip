// Conv2d_q forward: uint8 input (NCHW) x uint8 weights -> int32 -> requantized uint8, for the whole batch.
//
// l-ten does this per image as a u8 im2col followed by quantized_matmul(false, false, Cout, Ho*Wo, Cin*kh*kw)
// with the weights as the left operand (l-ten/conv2d.cpp:355-372): element = sum_k w[co][k] * col[k][p]
//   - zpW * sum_k col[k][p] - zpIn * sum_k w[co][k] + K * zpW * zpIn (+ bias[p]), then the requantize of
// l-ten/math_fns.cpp:1474.  Positions outside the image hold the byte 0 in the column buffer (not the zero point).
//
// Windows of at most 64 taps for fewer than 48 output channels (the 1 -> 10 channel 5x5 layer of l-ten's quantized
// MNIST network has 25 taps) run in one launch without a column buffer: a thread owns one output position, gathers its window into 16 packed dwords,
// and takes the products with unsigned dot4 instructions against the weights of up to 64 output channels held in
// LDS; consecutive lanes are consecutive positions of a row, so loads and the byte stores of y run along rows.
// Longer windows also run in one launch where the weights fit LDS beside the image (small images, at most 64 output
// channels) or, a block of output channels at a time, beside the input rows of a band of output rows (any image):
// convq_image.hip.  Other longer
// windows run as three launches for the whole batch (the first also pads the weights): the patches of all output
// positions as rows of a
// [N * Ho * Wo][K] matrix (K padded to a multiple of 16 with the input zero point, the weights padded alike with
// theirs, so the padding multiplies to nothing), one int8 GEMM of qgemm.hip with the positions as rows (NT: both
// operands contiguous in K, the shape its MFMA tiles are built for) into int32 sums, and a pass that adds l-ten's
// per-position bias, requantizes and stores in NCHW order.  When the workspace that needs would exceed 2 GiB the
// call follows l-ten's own decomposition image by image: im2col_u8, then the GEMM with the weights on the left.
#include <algorithm>
#include "conv_common.h"
#include "qgemm_common.h"

namespace lten_hip {

constexpr int CQ_MAXK = 64, CQ_CO = 64;

// one launch for small images with windows above 64 taps (convq_image.hip); -1 = not a shape for it
int conv2dq_image_dispatch(const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in, int zp_w, float mult,
                           float zp_out, void* y, bool out_acc);
// one launch for larger images, a band of output rows per workgroup (convq_image.hip); -1 = not a shape for it
int conv2dq_band_dispatch(const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in, int zp_w, float mult,
                          float zp_out, void* y, bool out_acc);

double conv2dq_band_estimate_us(const ConvGeo& g);

// ND = dwords of packed taps a thread holds (4 taps each): 4, 8, 12 or 16, the smallest that covers K.
template <int OUT, int ND>
__global__ __launch_bounds__(256) void conv2dq_direct_kernel(ConvGeo g, const uint8_t* __restrict__ x, const uint8_t* __restrict__ w,
                                                             const int32_t* __restrict__ bias, int zp_in, int zp_w, float mult, float zp_out,
                                                             void* __restrict__ y)
{
	__shared__ __attribute__((aligned(16))) uint32_t s_w[CQ_CO][ND];
	const int tid = threadIdx.x;
	const int K = g.Cin * g.kh * g.kw, HW = g.Ho * g.Wo;
	const int co0 = blockIdx.y * CQ_CO, nco = min(CQ_CO, g.Cout - co0);

	// N * HW < 2^31 (checked by the host): 32-bit divisions
	const uint32_t gid = blockIdx.x * 256u + tid;
	const bool live = gid < (uint32_t)g.N * (uint32_t)HW;
	const int n = live ? (int)(gid / (uint32_t)HW) : 0, pos = live ? (int)(gid - (uint32_t)n * (uint32_t)HW) : 0;
	const int ho = (int)((uint32_t)pos / (uint32_t)g.Wo), wo = pos - ho * g.Wo;
	const int y0 = ho * g.sh - g.ph, x0 = wo * g.sw - g.pw;
	const uint8_t* xn = x + (int64_t)n * g.Cin * g.H * g.W + (int64_t)y0 * g.W + x0;  // tap (0, 0, 0) of this position's window

	// The window, tap k in byte k % 4 of dword k / 4; (ci, i, j) of tap k is the same for every thread and is stepped,
	// not divided out.  The loads are issued before the weights are staged, so that the two latencies overlap.
	uint8_t tap[4 * ND];
	{
		int i = 0, j = 0, plane_row = 0;  // plane_row = ci * H + i
#pragma unroll
		for (int k = 0; k < 4 * ND; k++) {
			tap[k] = 0;
			if (k < K) {
				const int yy = y0 + i, xx = x0 + j;
				if (live && yy >= 0 && yy < g.H && xx >= 0 && xx < g.W) tap[k] = xn[(int64_t)plane_row * g.W + j];
				if (++j == g.kw) {
					j = 0;
					plane_row++;
					if (++i == g.kh) {
						i = 0;
						plane_row += g.H - g.kh;
					}
				}
			}
		}
	}

	// weights of this block's output channels, four taps per dword, taps past K as zero bytes (every load issued, the
	// byte of a tap past K discarded)
	for (int idx = tid; idx < CQ_CO * ND; idx += 256) {
		const int co = idx / ND, d = idx % ND;
		uint32_t v = 0;
		if (co < nco && K > 0) {
			const uint8_t* wr = w + (int64_t)(co0 + co) * K;
#pragma unroll
			for (int b = 0; b < 4; b++) {
				const int k = 4 * d + b;
				const uint32_t byte = wr[min(k, K - 1)];
				v |= (k < K ? byte : 0u) << (8 * b);
			}
		}
		s_w[co][d] = v;
	}
	__syncthreads();
	if (!live) return;

	uint32_t xk[ND];
#pragma unroll
	for (int d = 0; d < ND; d++)
		xk[d] = (uint32_t)tap[4 * d] | (uint32_t)tap[4 * d + 1] << 8 | (uint32_t)tap[4 * d + 2] << 16 | (uint32_t)tap[4 * d + 3] << 24;
	uint32_t xsum = 0;
#pragma unroll
	for (int d = 0; d < ND; d++) xsum = __builtin_amdgcn_udot4(xk[d], 0x01010101u, xsum, false);
	// l-ten/math_fns.cpp:1362-1380,1433: row_vector[p] = -zpA * sum_k B[k][p] with A = weights; broadcast = K zpA zpB
	const int base = -zp_w * (int)xsum + K * zp_w * zp_in + (bias ? bias[pos] : 0);

	for (int co = 0; co < nco; co++) {
		// the byte sum of the channel's weights rides along: the dwords are in registers anyway
		uint32_t dot = 0, wsum = 0;
#pragma unroll
		for (int d = 0; d < ND; d++) {
			const uint32_t wd = s_w[co][d];
			dot = __builtin_amdgcn_udot4(wd, xk[d], dot, false);
			wsum = __builtin_amdgcn_udot4(wd, 0x01010101u, wsum, false);
		}
		const int v = (int)dot + base - zp_in * (int)wsum;
		const int64_t o = ((int64_t)n * g.Cout + co0 + co) * HW + pos;
		if (OUT == Q_OUT_ACC) static_cast<int*>(y)[o] = v;
		else static_cast<uint8_t*>(y)[o] = (uint8_t)requant<OUT>(v, mult, zp_out);
	}
}

template <int OUT>
static void launch_conv2dq_direct(const dim3& grid, int K, const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in,
                                  int zp_w, float mult, float zp_out, void* y)
{
	if (K <= 16) conv2dq_direct_kernel<OUT, 4><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
	else if (K <= 32) conv2dq_direct_kernel<OUT, 8><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
	else if (K <= 48) conv2dq_direct_kernel<OUT, 12><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
	else conv2dq_direct_kernel<OUT, 16><<<grid, dim3(256), 0, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
}

// Row r = n * Ho * Wo + p of the patch matrix: the window of output position p of image n in l-ten's column order
// (ci, i, j).  Bytes outside the image are 0, as in l-ten's im2col (not the zero point); bytes from K on hold the input
// zero point.  A thread builds sixteen consecutive bytes of a row; the tap table (offset of the tap inside an image and
// its (i, j)) of the workgroup's 64 bytes of a row is built once per workgroup in LDS.  (Sixteen bytes and one 16-byte
// store per thread.)
__global__ __launch_bounds__(256) void conv2dq_rows_kernel(ConvGeo g, const uint8_t* __restrict__ x, uint8_t* __restrict__ rows, int Kp, int zp_in,
                                                           unsigned row_blocks, const uint8_t* __restrict__ w, uint8_t* __restrict__ wp, int Cp, int zp_w)
{
	__shared__ int s_tap[128];  // [64] offsets, then [64] i | j << 16
	const int K = g.Cin * g.kh * g.kw, HW = g.Ho * g.Wo;
	if (blockIdx.x >= row_blocks) {
		// the workgroups behind the rows pad the weights: wp[co][k] for co < Cp, k < Kp, with the weight zero point past K
		// and in the rows past Cout
		const int idx = (int)(blockIdx.x - row_blocks) * 256 + (int)threadIdx.x;
		if (idx < Cp * Kp) {
			const int co = idx / Kp, k = idx - co * Kp;
			wp[idx] = (co < g.Cout && k < K) ? w[(int64_t)co * K + k] : (uint8_t)zp_w;
		}
		return;
	}
	// A workgroup builds 64 consecutive rows x 64 bytes: a wavefront's lanes are 64 consecutive positions at one chunk, so
	// that each of its loads reads neighbouring bytes of the image (consecutive chunks of one row would read 64 channel
	// planes at once); the four wavefronts write the four chunks of the same 64 bytes of every row.
	const uint32_t chunks_per_row = (uint32_t)Kp / 16, groups = (chunks_per_row + 3) / 4;
	const uint32_t tile = blockIdx.x / groups, grp = blockIdx.x - tile * groups;
	const uint32_t r = tile * 64 + (threadIdx.x & 63), kc = grp * 4 + (threadIdx.x >> 6);
	if (threadIdx.x < 64) {  // the taps of this workgroup's 64 bytes of a row
		const int kt = min((int)grp * 64 + (int)threadIdx.x, K - 1);
		const int j = kt % g.kw, i = (kt / g.kw) % g.kh, ci = kt / (g.kw * g.kh);
		s_tap[threadIdx.x] = (ci * g.H + i) * g.W + j;
		s_tap[64 + threadIdx.x] = i | (j << 16);
	}
	__syncthreads();
	if (r >= (uint32_t)g.N * (uint32_t)HW || kc >= chunks_per_row) return;
	const int n = (int)(r / (uint32_t)HW), pos = (int)(r - (uint32_t)n * (uint32_t)HW);
	const int ho = pos / g.Wo, wo = pos - ho * g.Wo;
	const int y0 = ho * g.sh - g.ph, x0 = wo * g.sw - g.pw;
	const uint8_t* xn = x + (int64_t)n * g.Cin * g.H * g.W;
	const int base = y0 * g.W + x0;
	uint32_t bytes[16];
#pragma unroll
	for (int b = 0; b < 16; b++) {  // all sixteen loads first
		const int k = 16 * (int)kc + b, kl = 16 * (int)(threadIdx.x >> 6) + b;
		const int ij = s_tap[64 + kl];
		const int yy = y0 + (ij & 0xFFFF), xx = x0 + (ij >> 16);
		const bool inside = ((unsigned)yy < (unsigned)g.H) & ((unsigned)xx < (unsigned)g.W);
		const uint32_t byte = xn[(s_tap[kl] + base) & -(int)inside];  // offset 0 for taps outside: always a valid address
		bytes[b] = k < K ? (inside ? byte : 0u) : (uint32_t)zp_in;
	}
	uint4 out;
	out.x = bytes[0] | bytes[1] << 8 | bytes[2] << 16 | bytes[3] << 24;
	out.y = bytes[4] | bytes[5] << 8 | bytes[6] << 16 | bytes[7] << 24;
	out.z = bytes[8] | bytes[9] << 8 | bytes[10] << 16 | bytes[11] << 24;
	out.w = bytes[12] | bytes[13] << 8 | bytes[14] << 16 | bytes[15] << 24;
	reinterpret_cast<uint4*>(rows)[(uint64_t)r * chunks_per_row + kc] = out;
}

// y[n][co][p] = requantize(acc[n * HW + p][co] + bias[p]) (or the int32 sum itself): a workgroup takes 64 positions x 64
// channels, reads the sums along the channels and stores along the positions, through LDS.
template <int OUT>
__global__ __launch_bounds__(256) void conv2dq_finish_kernel(const int32_t* __restrict__ acc, const int32_t* __restrict__ bias, void* __restrict__ y,
                                                             int rows, int HW, int Cout, int Cp, float mult, float zp_out)
{
	__shared__ int s[64][65];
	const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
	const int ncp = min(64, Cp - c0), nco = min(64, Cout - c0);  // columns of the sums to read, channels to store
	for (int e = threadIdx.x; e < 64 * ncp; e += 256) {
		const int rr = e / ncp, cc = e - rr * ncp;
		s[rr][cc] = acc[(int64_t)min(r0 + rr, rows - 1) * Cp + c0 + cc];
	}
	__syncthreads();
	// a thread keeps its position and walks the channels: the position is decomposed once
	const int rr = threadIdx.x & 63, r = r0 + rr;
	if (r >= rows) return;
	const int n = r / HW, pos = r - n * HW;
	const int b = bias ? bias[pos] : 0;
	for (int cc = threadIdx.x >> 6; cc < nco; cc += 4) {
		const int v = s[rr][cc] + b;
		const int64_t o = ((int64_t)n * Cout + c0 + cc) * HW + pos;
		if (OUT == Q_OUT_ACC) static_cast<int*>(y)[o] = v;
		else static_cast<uint8_t*>(y)[o] = (uint8_t)requant<OUT>(v, mult, zp_out);
	}
}

static int make_geo_q(ConvGeo& g, uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw, int sh, int sw)
{
	LTEN_HIP_REQUIRE(kh > 0 && kw > 0 && sh > 0 && sw > 0 && ph >= 0 && pw >= 0, "conv2dq: bad kernel geometry");
	LTEN_HIP_REQUIRE(N < 65536 && Cin < (1u << 20) && Cout < (1u << 20) && H < (1u << 15) && W < (1u << 15), "conv2dq: dimension too large");
	LTEN_HIP_REQUIRE(Cin * H * W < (1ull << 31) && Cout * H * W < (1ull << 31), "conv2dq: one image must stay below 2^31 elements");
	const int64_t eh = (int64_t)H + 2 * ph - kh, ew = (int64_t)W + 2 * pw - kw;
	LTEN_HIP_REQUIRE(eh >= 0 && ew >= 0, "conv2dq: kernel larger than the padded image");
	LTEN_HIP_REQUIRE(Cin * (uint64_t)kh * kw * 255 * 255 < (1ull << 31), "conv2dq: Cin*kh*kw too large for an int32 accumulator");
	g.N = (int)N; g.Cin = (int)Cin; g.H = (int)H; g.W = (int)W; g.Cout = (int)Cout;
	g.kh = kh; g.kw = kw; g.ph = ph; g.pw = pw; g.sh = sh; g.sw = sw; g.dh = 1; g.dw = 1;
	g.Ho = (int)(eh / sh + 1);  // l-ten/conv2d.cpp:322-323
	g.Wo = (int)(ew / sw + 1);
	return 0;
}

static uint64_t align16(uint64_t v) { return (v + 15) & ~15ull; }
static uint64_t align256(uint64_t v) { return (v + 255) & ~255ull; }

// Workspace of the whole-batch route: patch rows, padded weights, int32 sums, the GEMM's zero-point terms.
struct BatchedPlan {
	bool ok;
	uint64_t rows, Kp, Cp, off_wp, off_acc, off_terms, bytes;
};

static BatchedPlan batched_plan(const ConvGeo& g)
{
	BatchedPlan b;
	const uint64_t K = (uint64_t)g.Cin * g.kh * g.kw;
	b.rows = (uint64_t)g.N * g.Ho * g.Wo;
	b.Kp = (K + 15) & ~15ull;
	b.Cp = ((uint64_t)g.Cout + 3) & ~3ull;
	b.off_wp = align256(b.rows * b.Kp);
	b.off_acc = b.off_wp + align256(b.Cp * b.Kp);
	b.off_terms = b.off_acc + align256(b.rows * b.Cp * 4);
	b.bytes = b.off_terms + 4 * (b.rows + b.Cp) + 16;
	b.ok = b.bytes <= (2ull << 30) && b.rows < (1ull << 31) && b.rows * b.Kp < (1ull << 32) && b.Cp * b.Kp < (1ull << 31);
	return b;
}

static int conv2dq_run(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw, int sh, int sw,
                       const uint8_t* x, const uint8_t* w, const int32_t* bias, const lten_hip_qparams* qp, void* y, bool out_acc,
                       void* workspace)
{
	ConvGeo g;
	if (int rc = make_geo_q(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)) return rc;
	LTEN_HIP_REQUIRE(qp != nullptr, "conv2dq: qparams is null");
	const int64_t HW = (int64_t)g.Ho * g.Wo, K = (int64_t)Cin * kh * kw;
	if (N == 0 || Cout == 0 || HW == 0) return 0;
	LTEN_HIP_REQUIRE(x && w && y, "conv2dq: null pointer");
	const int zp_in = qp[0].zero_point, zp_w = qp[1].zero_point;
	// l-ten/math_fns.cpp:1436 with qparams[0] = weights, [1] = input (l-ten/conv2d.cpp:347-349), left to right in fp32
	volatile float ab = qp[1].scale * qp[0].scale;
	const float mult = ab / qp[2].scale, zp_out = (float)qp[2].zero_point;

	// Windows of at most 64 taps for 48 output channels and more: the band kernel's matrix cores are ahead of the dot
	// products below, which issue at a quarter of the vector rate (8 x 16 x 56 x 56 -> 64 channels 2 x 2, stride 2: 26.5
	// -> 6.9 us; 8 x 64 x 56 x 56 -> 256 channels 1 x 1: 30.0 -> 16.6 us; 64 x 3 x 224 x 224 -> 64 channels 3 x 3: 181 ->
	// 130 us), not for fewer (256 x 3 x 32 x 32 -> 32: 14.5 us below, 19.0 there; l-ten's MNIST conv1, 10 channels: 6.6
	// and 7.3).  Option "conv_variant" 2 keeps the kernel below.
	if (K <= CQ_MAXK && Cout >= 48 && (get_option(OPT_CONV_VARIANT) == 0 || get_option(OPT_CONV_VARIANT) == 3)) {
		const int rc = conv2dq_band_dispatch(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, out_acc);
		if (rc >= 0) return rc;
	}
	if (K <= CQ_MAXK && (uint64_t)N * HW < (1ull << 31) && get_option(OPT_CONV_VARIANT) != 1) {
		const dim3 grid((unsigned)ceil_div((uint64_t)N * HW, 256), (unsigned)ceil_div(Cout, CQ_CO));
		set_kernel_name("conv2dq_direct");
		if (out_acc) launch_conv2dq_direct<Q_OUT_ACC>(grid, (int)K, g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
		else if (mult == mult && (mult < 0 ? -mult : mult) <= 0.99f)
			launch_conv2dq_direct<Q_OUT_U8_FAST>(grid, (int)K, g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
		else launch_conv2dq_direct<Q_OUT_U8_EXACT>(grid, (int)K, g, x, w, bias, zp_in, zp_w, mult, zp_out, y);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}

	// small images with a longer window (l-ten's quantized MNIST conv2): still one launch, no workspace (convq_image.hip;
	// option "conv_variant" 2 keeps such shapes on the three launches below, 3 skips the small-image kernel)
	const BatchedPlan bp = batched_plan(g);
	if (get_option(OPT_CONV_VARIANT) == 0 || get_option(OPT_CONV_VARIANT) == 3) {
		int rc = get_option(OPT_CONV_VARIANT) == 3 ? -1 : conv2dq_image_dispatch(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, out_acc);
		if (rc >= 0) return rc;
		// larger images or more channels: a band of output rows and a block of output channels per workgroup, the input rows
		// it needs in LDS -- unless long windows leave a workgroup so few pixels and channels that it stages more than it
		// computes and the three launches below are ahead, which take 30 us + 1.3 us per MB of patch rows (32 x 1024 x 14
		// x 14 -> 256 channels 1 x 1: 132 us on bands, 43 below; 32 x 128 x 28 x 28 -> 256 channels 3 x 3 stride 2: 55 and 44)
		const bool rows_ahead = get_option(OPT_CONV_VARIANT) == 0 && bp.ok && workspace != nullptr &&
		                        conv2dq_band_estimate_us(g) > 30.0 + 1.3e-6 * (double)bp.rows * (double)bp.Kp;
		if (!rows_ahead) rc = conv2dq_band_dispatch(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, out_acc);
		if (rc >= 0) return rc;
	}

	LTEN_HIP_REQUIRE(workspace != nullptr, "conv2dq: workspace is null");
	if (bp.ok && get_option(OPT_CONV_VARIANT) != 1) {
		uint8_t* base = static_cast<uint8_t*>(workspace);
		uint8_t* rows = base;
		uint8_t* wp = base + bp.off_wp;
		int32_t* sums = reinterpret_cast<int32_t*>(base + bp.off_acc);
		int32_t* terms = reinterpret_cast<int32_t*>(base + bp.off_terms);
		const unsigned row_blocks = (unsigned)(ceil_div(bp.rows, 64) * ceil_div(bp.Kp / 16, 4)), weight_blocks = (unsigned)ceil_div(bp.Cp * bp.Kp, 256);
		conv2dq_rows_kernel<<<dim3(row_blocks + weight_blocks), dim3(256), 0, stream()>>>(g, x, rows, (int)bp.Kp, zp_in, row_blocks, w, wp,
		                                                                                                (int)bp.Cp, zp_w);
		LTEN_HIP_LAUNCH_CHECK();
		if (int rc = lten_hip_quantized_matmul_acc(0, 1, bp.rows, bp.Cp, bp.Kp, rows, wp, sums, qp, nullptr, terms)) return rc;
		const dim3 grid((unsigned)ceil_div(bp.rows, 64), (unsigned)ceil_div(Cout, 64));
		set_kernel_name("conv2dq_rows_gemm_finish");
		if (out_acc) conv2dq_finish_kernel<Q_OUT_ACC><<<grid, dim3(256), 0, stream()>>>(sums, bias, y, (int)bp.rows, (int)HW, (int)Cout, (int)bp.Cp, mult, zp_out);
		else if (mult == mult && (mult < 0 ? -mult : mult) <= 0.99f)
			conv2dq_finish_kernel<Q_OUT_U8_FAST><<<grid, dim3(256), 0, stream()>>>(sums, bias, y, (int)bp.rows, (int)HW, (int)Cout, (int)bp.Cp, mult, zp_out);
		else conv2dq_finish_kernel<Q_OUT_U8_EXACT><<<grid, dim3(256), 0, stream()>>>(sums, bias, y, (int)bp.rows, (int)HW, (int)Cout, (int)bp.Cp, mult, zp_out);
		LTEN_HIP_LAUNCH_CHECK();
		return 0;
	}

	// l-ten's own decomposition, image by image: column buffer, then C[Cout x HW] = W[Cout x K] * col[K x HW]
	uint8_t* col = static_cast<uint8_t*>(workspace);
	int32_t* terms = reinterpret_cast<int32_t*>(col + align16((uint64_t)K * HW));
	const lten_hip_qparams q3[3] = { qp[1], qp[0], qp[2] };
	for (uint64_t n = 0; n < N; n++) {
		if (int rc = lten_hip_im2col_u8(x + n * Cin * H * W, (int)Cin, (int)H, (int)W, kh, kw, ph, pw, sh, sw, 1, 1, col)) return rc;
		int rc;
		if (out_acc) rc = lten_hip_quantized_matmul_acc(0, 0, Cout, (uint64_t)HW, (uint64_t)K, w, col, static_cast<int32_t*>(y) + n * Cout * HW, q3, bias, terms);
		else rc = lten_hip_quantized_matmul(0, 0, Cout, (uint64_t)HW, (uint64_t)K, 1, w, col, 0, static_cast<uint8_t*>(y) + n * Cout * HW, q3, bias, terms);
		if (rc) return rc;
	}
	return 0;
}

}  // namespace lten_hip

using namespace lten_hip;

extern "C" {

uint64_t lten_hip_conv2dq_workspace_bytes(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph,
                                          int pw, int sh, int sw)
{
	ConvGeo g;
	if (make_geo_q(g, N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw)) return 0;
	const uint64_t HW = (uint64_t)g.Ho * g.Wo, K = Cin * kh * kw;
	const uint64_t per_image = align16(K * HW) + 4 * (Cout + HW) + 16;
	const BatchedPlan bp = batched_plan(g);
	return bp.ok ? std::max(per_image, bp.bytes) : per_image;
}

int lten_hip_conv2dq_forward(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw, int sh,
                             int sw, const uint8_t* x, const uint8_t* w, const int32_t* bias, const lten_hip_qparams* qparams_in_wt_out,
                             uint8_t* y, void* workspace)
{
	return conv2dq_run(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, x, w, bias, qparams_in_wt_out, y, false, workspace);
}

int lten_hip_conv2dq_forward_acc(uint64_t N, uint64_t Cin, uint64_t H, uint64_t W, uint64_t Cout, int kh, int kw, int ph, int pw,
                                 int sh, int sw, const uint8_t* x, const uint8_t* w, const int32_t* bias,
                                 const lten_hip_qparams* qparams_in_wt_out, int32_t* acc, void* workspace)
{
	return conv2dq_run(N, Cin, H, W, Cout, kh, kw, ph, pw, sh, sw, x, w, bias, qparams_in_wt_out, acc, true, workspace);
}

}  // extern "C"
