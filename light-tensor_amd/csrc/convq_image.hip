// Conv2d_q forward for small images and windows above 64 taps, in one launch (l-ten/conv2d.cpp:265-387; the second
// convolution of l-ten's quantized MNIST network, 10 -> 20 channels 5 x 5 on 12 x 12, is the shape it is for).
//
// A workgroup takes 16 output positions of one image.  The image (at most 32 KB) and the weights of all output
// channels are staged in LDS once; the patch matrix is never written anywhere: the four wavefronts take the k-steps of
// 64 taps in turn, and every lane builds the 16 bytes the 16x16x64 int8 MFMA wants from it (position lane % 16, taps
// 16 (lane / 16) .. + 15 of the k-step) straight from the image in LDS through a tap table, flips them into the signed
// domain and multiplies them with the weight fragments of up to four blocks of 16 channels; the wavefronts' sums meet
// in LDS.  Positions are the MFMA's rows and channels its columns, so a lane ends with four consecutive positions of
// one channel, which are consecutive bytes of y.
//
// Arithmetic as in convq.hip: element = sum_k (x - zpIn)(w - zpW) (+ bias[position]) with positions outside the image
// counting as the byte 0, obtained from the signed products by the identity of qgemm.hip,
//   sum (a - zpA)(b - zpB) = sum a'b' + (128 - zpB) SA + (128 - zpA) SB + K (zpA zpB - 16384),
// a' = a - 128, SA / SB the byte sums of a position's window and of a channel's weights.  Taps past K hold 0x80 in the
// window (a' = 0) and signed zeros in the weights.
#include "conv_common.h"
#include "qgemm_common.h"

namespace lten_hip {

constexpr int CQI_POS = 16;           // positions per workgroup: one block of MFMA rows; its four wavefronts split the k-steps
constexpr int CQI_MAX_IMAGE = 32768;  // bytes of one image: tap offsets fit 16 bits
constexpr int CQI_PAD = 16;           // bytes behind a weight row in LDS: rows 16 apart land on different banks
constexpr int CQI_RED = 4 * 64 * (4 * 4 + 1 + 4) * 4;  // bytes of the wavefronts' partial results when they meet in LDS

struct ImagePlan {
	int Kp, ncb, img16, wpitch;
	unsigned off_w, off_tap, bytes;
};

// tap table entry: offset of the tap inside the image (16 bits) | i << 16 (7 bits) | j << 23 (7 bits) | bit 30: past K
constexpr uint32_t TAP_PAST_K = 1u << 30;

// CHECK: windows may reach outside the image (padding); without it every tap of every position lies inside.
template <int OUT, bool CHECK>
__global__ __launch_bounds__(256) void conv2dq_image_kernel(ConvGeo g, const uint8_t* __restrict__ x, const uint8_t* __restrict__ w,
                                                            const int32_t* __restrict__ bias, int zp_in, int zp_w, float mult, float zp_out,
                                                            void* __restrict__ y, ImagePlan pl, int blocks_per_image)
{
	extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
	uint8_t* const s_img = smem;
	uint8_t* const s_w = smem + pl.off_w;
	uint32_t* const s_tap = reinterpret_cast<uint32_t*>(smem + pl.off_tap);

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int lrow = lane & 15, lgrp = lane >> 4;
	const int K = g.Cin * g.kh * g.kw, HW = g.Ho * g.Wo, Kp = pl.Kp;
	const int n = (int)blockIdx.x / blocks_per_image, blk = (int)blockIdx.x % blocks_per_image;
	const int img_bytes = g.Cin * g.H * g.W;
	const uint8_t* xn = x + (int64_t)n * img_bytes;

	// ---- the image: 16 bytes per thread and round where the image starts on a 16-byte boundary, bytes otherwise
	if ((reinterpret_cast<uintptr_t>(xn) & 15) == 0) {
		for (int i = tid * 16; i < img_bytes; i += 256 * 16) {
			if (i + 16 <= img_bytes) *reinterpret_cast<v4i*>(s_img + i) = *reinterpret_cast<const v4i*>(xn + i);
			else
				for (int b = i; b < img_bytes; b++) s_img[b] = xn[b];
		}
	} else {
		for (int i = tid; i < img_bytes; i += 256) s_img[i] = xn[i];
	}
	// ---- tap table
	for (int k = tid; k < Kp; k += 256) {
		const int kc = min(k, K - 1);
		const int j = kc % g.kw, i = (kc / g.kw) % g.kh, ci = kc / (g.kw * g.kh);
		s_tap[k] = (uint32_t)((ci * g.H + i) * g.W + j) | (uint32_t)i << 16 | (uint32_t)j << 23 | (k < K ? 0u : TAP_PAST_K);
	}
	// ---- weights: 16 bytes of a row per thread and round, into the signed domain; rows past Cout and taps past K are zeros
	const int chunks = Kp / 16;
	for (int idx = tid; idx < pl.ncb * 16 * chunks; idx += 256) {
		const int co = idx / chunks, k0 = (idx - co * chunks) * 16;
		uint32_t d[4] = { 0, 0, 0, 0 };
		if (co < g.Cout) {
			const uint8_t* wr = w + (int64_t)co * K;
#pragma unroll
			for (int b = 0; b < 16; b++) {
				const int k = k0 + b;
				const uint32_t raw = wr[min(k, K - 1)];
				const uint32_t byte = k < K ? raw : 0x80u;  // 0x80 is the signed domain's zero
				d[b >> 2] |= (byte ^ 0x80u) << (8 * (b & 3));
			}
		}
		*reinterpret_cast<v4i*>(s_w + co * pl.wpitch + k0) = v4i{ (int)d[0], (int)d[1], (int)d[2], (int)d[3] };
	}
	// ---- the bias of this lane's four output positions is asked for now, so that it is there when the sums are
	const int p0 = blk * CQI_POS + lgrp * 4;  // first of this lane's four positions
	int bv[4];
#pragma unroll
	for (int e = 0; e < 4; e++) bv[e] = (bias != nullptr && p0 + e < HW) ? bias[p0 + e] : 0;
	__syncthreads();

	// ---- this lane's position (row of the MFMA) and its window's corner
	const int pos = blk * CQI_POS + lrow;
	const bool live = pos < HW;
	const int ho = live ? pos / g.Wo : 0, wo = live ? pos - ho * g.Wo : 0;
	const int y0 = ho * g.sh - g.ph, x0 = wo * g.sw - g.pw;
	const int base = y0 * g.W + x0;

	v4i acc[4];
	uint32_t sw[4];  // byte sums of the weights this lane feeds: channel 16 cb + lrow, its k-groups
#pragma unroll
	for (int cb = 0; cb < 4; cb++) {
		acc[cb] = v4i{ 0, 0, 0, 0 };
		sw[cb] = 0;
	}
	uint32_t sa = 0;
	for (int ks = wave * 64; ks < Kp; ks += 4 * 64) {  // the wavefronts take the k-steps in turn
		uint32_t d[4] = { 0, 0, 0, 0 };
#pragma unroll
		for (int b = 0; b < 16; b++) {
			const uint32_t t = s_tap[ks + lgrp * 16 + b];
			uint32_t raw;
			if (CHECK) {
				const int yy = y0 + (int)((t >> 16) & 127), xx = x0 + (int)((t >> 23) & 127);
				const bool inside = ((unsigned)yy < (unsigned)g.H) & ((unsigned)xx < (unsigned)g.W) & ((t & TAP_PAST_K) == 0) & live;
				const uint32_t byte = s_img[((int)(t & 0xFFFF) + base) & -(int)inside];  // offset 0 for taps outside: a valid address
				// outside the image: the byte 0; past K: 0x80, which the flip below turns into nothing
				raw = inside ? byte : ((t & TAP_PAST_K) ? 0x80u : 0u);
			} else {
				const bool real = ((t & TAP_PAST_K) == 0) & live;
				const uint32_t byte = s_img[((int)(t & 0xFFFF) + base) & -(int)real];
				raw = real ? byte : 0x80u;  // (a position past the image's last one is never stored)
			}
			d[b >> 2] |= raw << (8 * (b & 3));
		}
#pragma unroll
		for (int q = 0; q < 4; q++) sa = __builtin_amdgcn_sad_u8(d[q], 0u, sa);
		const v4i a = flip_sign_bits(v4i{ (int)d[0], (int)d[1], (int)d[2], (int)d[3] });
#pragma unroll
		for (int cb = 0; cb < 4; cb++) {
			if (cb < pl.ncb) {
				const v4i b = *reinterpret_cast<const v4i*>(s_w + (cb * 16 + lrow) * pl.wpitch + ks + lgrp * 16);
				const v4i braw = flip_sign_bits(b);  // back to l-ten's bytes for the sum (taps past K then hold 0x80)
#pragma unroll
				for (int q = 0; q < 4; q++) sw[cb] = __builtin_amdgcn_sad_u8((unsigned)braw[q], 0u, sw[cb]);
				// lane (lrow, lgrp), register e holds out[position 4 lgrp + e][channel lrow]
				acc[cb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[cb], 0, 0, 0);
			}
		}
	}
	// ---- the wavefronts' shares meet in LDS (the image and the weights are no longer needed); wavefront 0 finishes
	__syncthreads();
	int* const red = reinterpret_cast<int*>(smem);
	constexpr int PER = 4 * 4 + 1 + 4;  // values per lane
	if (wave != 0) {
		int* mine = red + (wave * PER) * 64 + lane;
#pragma unroll
		for (int cb = 0; cb < 4; cb++) {
#pragma unroll
			for (int e = 0; e < 4; e++) mine[(cb * 4 + e) * 64] = acc[cb][e];
			mine[(17 + cb) * 64] = (int)sw[cb];
		}
		mine[16 * 64] = (int)sa;
	}
	__syncthreads();
	if (wave != 0) return;
	for (int ow = 1; ow < 4; ow++) {
		const int* other = red + (ow * PER) * 64 + lane;
#pragma unroll
		for (int cb = 0; cb < 4; cb++) {
#pragma unroll
			for (int e = 0; e < 4; e++) acc[cb][e] += other[(cb * 4 + e) * 64];
			sw[cb] += (uint32_t)other[(17 + cb) * 64];
		}
		sa += (uint32_t)other[16 * 64];
	}
	// a lane holds the byte sum of its k-groups only; after the fold lanes 0..15 (and their copies) hold the rows' sums,
	// less the 0x80 bytes of the taps past K
	sa += __shfl_xor(sa, 16, 64);
	sa += __shfl_xor(sa, 32, 64);
	const int row_sum = (int)sa - 128 * (Kp - K);

	const int coef_a = 128 - zp_w, coef_b = 128 - zp_in;
	const int konst = K * (zp_in * zp_w - 16384);
	int rt[4];
#pragma unroll
	for (int e = 0; e < 4; e++) {
		const int rs = __shfl(row_sum, lgrp * 4 + e, 64);
		rt[e] = coef_a * rs + konst + bv[e];
	}
#pragma unroll
	for (int cb = 0; cb < 4; cb++) {
		const int co = cb * 16 + lrow;
		// the channel's byte sum: its four k-groups sit in lanes lrow, lrow + 16, + 32, + 48
		uint32_t wsum = sw[cb];
		wsum += __shfl_xor(wsum, 16, 64);
		wsum += __shfl_xor(wsum, 32, 64);
		if (cb >= pl.ncb || co >= g.Cout) continue;
		const int ct = coef_b * ((int)wsum - 128 * (Kp - K));
		const int64_t o = ((int64_t)n * g.Cout + co) * HW + p0;
#pragma unroll
		for (int e = 0; e < 4; e++) {
			if (p0 + e >= HW) continue;
			const int v = acc[cb][e] + rt[e] + ct;
			if (OUT == Q_OUT_ACC) static_cast<int*>(y)[o + e] = v;
			else static_cast<uint8_t*>(y)[o + e] = (uint8_t)requant<OUT>(v, mult, zp_out);
		}
	}
}

// Whether the one-launch route takes the call, and its LDS layout.  Few workgroups per image and few in all: every
// workgroup stages the whole image and all weights, which pays while the call is bound by launch latency (three
// launches otherwise) and not beyond.
static bool image_plan(const ConvGeo& g, ImagePlan& pl)
{
	const int64_t K = (int64_t)g.Cin * g.kh * g.kw, HW = (int64_t)g.Ho * g.Wo, img = (int64_t)g.Cin * g.H * g.W;
	if (K <= 64 || K > 1024 || img > CQI_MAX_IMAGE || g.Cout > 64 || g.kh > 127 || g.kw > 127 || HW > 1024) return false;
	const int64_t blocks = (int64_t)g.N * ((HW + CQI_POS - 1) / CQI_POS);
	if (blocks > 4096) return false;
	pl.Kp = (int)((K + 63) & ~63ll);
	pl.ncb = (g.Cout + 15) / 16;
	pl.img16 = (int)((img + 15) & ~15ll);
	pl.wpitch = pl.Kp + CQI_PAD;
	pl.off_w = (unsigned)pl.img16;
	pl.off_tap = pl.off_w + (unsigned)(pl.ncb * 16 * pl.wpitch);
	pl.bytes = pl.off_tap + (unsigned)pl.Kp * 4;
	if (pl.bytes < (unsigned)CQI_RED) pl.bytes = CQI_RED;
	return pl.bytes <= 64 * 1024;
}

// 0 = launched; -1 = not a shape for this route
int conv2dq_image_dispatch(const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in, int zp_w, float mult,
                           float zp_out, void* y, bool out_acc)
{
	ImagePlan pl;
	if (!image_plan(g, pl)) return -1;
	const int per_image = (g.Ho * g.Wo + CQI_POS - 1) / CQI_POS;
	const dim3 grid((unsigned)(g.N * per_image));
	// windows that cannot reach outside the image need no bounds checks on the way
	const bool check = g.ph > 0 || g.pw > 0;
	set_kernel_name("conv2dq_image");
#define LTEN_LAUNCH(OUTV)                                                                                                                              \
	if (check) conv2dq_image_kernel<OUTV, true><<<grid, dim3(256), pl.bytes, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, pl, per_image); \
	else conv2dq_image_kernel<OUTV, false><<<grid, dim3(256), pl.bytes, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, pl, per_image);
	if (out_acc) { LTEN_LAUNCH(Q_OUT_ACC) }
	else if (mult == mult && (mult < 0 ? -mult : mult) <= 0.99f) { LTEN_LAUNCH(Q_OUT_U8_FAST) }
	else { LTEN_LAUNCH(Q_OUT_U8_EXACT) }
#undef LTEN_LAUNCH
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

}  // namespace lten_hip
