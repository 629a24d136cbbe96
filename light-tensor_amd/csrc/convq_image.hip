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

// The same idea for images of any size and any number of output channels: a workgroup takes a band of TB output rows of
// one image and a block of up to 64 output channels (the grid's second axis) and stages the input rows the band's
// windows reach, pixel-major with the channels innermost: [RH rows][RW columns][PP bytes], byte ci of a
// pixel its channel ci, channels padded with zeros to a multiple of CP (4, 8 or 16 by the channel count), the padding
// written out as zero pixels (PL zero columns on the left, rows above and below the image as zero rows).  The
// reduction runs in the order (tap, channel) instead of l-ten's (channel, tap), the weights being staged in the same
// order, so that the 16 bytes a lane feeds to a 16x16x64 MFMA are 16 / CP aligned pieces of CP consecutive channels of
// a pixel: one to four LDS reads and no arithmetic per fragment, no bounds checks (the byte-wise gather of the
// small-image kernel above, an addition, a byte read and a shift-or per byte, made this kernel take 73.7 us on 32 x 64 x
// 56 x 56 -> 64 channels 3 x 3; the patch-row route with its workspace 157 us; this kernel 28.9 us, of which about 7 are
// the loads of the region, 3.7 the weights, 9.5 the k-steps and 3.8 the stores: all 448 workgroups are resident at
// once and pass through these phases together).  A wavefront owns up to four blocks of 16 positions at a time and
// walks the k-steps once for all of them.
struct BandPlan {
	int CP, CPtot, PP, UC, Kp, ncb, wpitch, TB, RH, RW, PL;
	unsigned off_w, off_unit, off_kmap, bytes;
	unsigned inv_rw4, inv_rh, inv_cq;  // reciprocals for small_div: RW / 4, RH, Cin / 4
};

// n / d for n d < 2^32 by one multiplication, inv = small_div_inverse(d): a thread of the band kernel's staging loops
// splits its item number three ways per item, 30-odd instructions per 32-bit division otherwise.
static inline unsigned small_div_inverse(unsigned d) { return d <= 1 ? 0u : (unsigned)((0x100000000ull + d - 1) / d); }
__device__ __forceinline__ int small_div(int n, unsigned inv) { return inv == 0 ? n : (int)__umulhi((unsigned)n, inv); }

// Weights of a window of T taps into the band kernel's order, for rows that keep dword alignment and channel counts
// that are multiples of four: four channels of a row are 4 T consecutive bytes, T dwords, and become T dwords of the
// new order (one per tap, its four bytes the four channels), permuted in registers: T dword loads along memory and T
// dword writes to LDS per thread, where scattering the bytes of every loaded dword took four byte writes that met on a
// few LDS banks (8 of 20 us on 4 x 64 x 56 x 56 -> 64 channels 3 x 3).
template <int T>
__device__ __forceinline__ void band_stage_weights(const uint8_t* __restrict__ w, uint8_t* s_w, int Cout, int Cin, int CPtot, int wpitch, int tid,
                                                   unsigned inv_cq)
{
	const int cq = Cin / 4, K = Cin * T;
	for (int u = tid; u < Cout * cq; u += 256) {
		const int co = small_div(u, inv_cq), q = u - co * cq;
		const uint32_t* src = reinterpret_cast<const uint32_t*>(w + (int64_t)co * K) + q * T;
		uint32_t in[T];
#pragma unroll
		for (int i = 0; i < T; i++) in[i] = src[i];
		uint8_t* dst = s_w + co * wpitch + 4 * q;
#pragma unroll
		for (int t = 0; t < T; t++) {
			uint32_t v = 0;
#pragma unroll
			for (int b = 0; b < 4; b++) {
				const int pos = b * T + t;  // byte of the 4 T that holds (channel b, tap t)
				v |= ((in[pos >> 2] >> (8 * (pos & 3))) & 0xFFu) << (8 * b);
			}
			*reinterpret_cast<uint32_t*>(dst + t * CPtot) = v ^ 0x80808080u;
		}
	}
}

template <int OUT, int CP>
__global__ __launch_bounds__(256, 2) void conv2dq_band_kernel(ConvGeo g, const uint8_t* __restrict__ x, const uint8_t* __restrict__ w,
                                                           const int32_t* __restrict__ bias, int zp_in, int zp_w, float mult, float zp_out,
                                                           void* __restrict__ y, BandPlan pl, int bands_per_image)
{
	extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
	uint8_t* const s_rgn = smem;
	uint8_t* const s_w = smem + pl.off_w;
	uint32_t* const s_unit = reinterpret_cast<uint32_t*>(smem + pl.off_unit);

	const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
	const int lrow = lane & 15, lgrp = lane >> 4;
	const int T = g.kh * g.kw, K = g.Cin * T, HW = g.Ho * g.Wo, Kp = pl.Kp, RH = pl.RH, RW = pl.RW, PP = pl.PP, CPtot = pl.CPtot;
	// workgroups go to the eight XCDs in turn: number b works on band (b % 8) * (bands / 8) + b / 8 (the first bands % 8
	// XCDs one more), so that neighbouring bands of an image, which share the input rows under their windows, find
	// them in the same L2
	const int nb = (int)gridDim.x, xcd = (int)blockIdx.x & 7;
	const int bid = xcd * (nb >> 3) + min(xcd, nb & 7) + ((int)blockIdx.x >> 3);
	const int n = bid / bands_per_image, hb = (bid % bands_per_image) * pl.TB;
	const int rows_here = min(pl.TB, g.Ho - hb);
	// grid row: this workgroup's block of 16 ncb output channels
	const int co0 = (int)blockIdx.y * pl.ncb * 16, cout_here = min(g.Cout - co0, pl.ncb * 16);
	w += (int64_t)co0 * (g.Cin * g.kh * g.kw);
	const int rgn_y0 = hb * g.sh - g.ph;  // image row of region row 0
	const uint8_t* xn = x + (int64_t)n * g.Cin * g.H * g.W;

	// ---- the region: four columns of four channels at a time (four dword loads where the image's rows keep dword
	// alignment, W % 4 == 0 and an aligned image: such a dword lies inside the image or outside as a whole), transposed
	// in registers into four dwords of four channels each
	const int rw4 = RW / 4, cg_n = CPtot / 4, items = cg_n * RH * rw4;
	const bool fast = (g.W & 3) == 0 && (reinterpret_cast<uintptr_t>(xn) & 3) == 0;
	// Every load comes from an address clamped into the image and its value is dropped afterwards where the dword lies
	// outside: no branch stands between the four loads of an item.  The split of the item number is by multiplication.
	// (Several items in flight per thread are no faster, 32.9 us with three and 33.7 with six against 31.3 with one on
	// 32 x 64 x 56 x 56 -> 64 channels 3 x 3: the loads of all workgroups start together on caches that hold nothing
	// yet, and what they wait for is the memory behind them, 7 us in all, not one another.)
	for (int idx = tid; idx < items; idx += 256) {
		const int q1 = small_div(idx, pl.inv_rw4), c4 = idx - q1 * rw4, cg = small_div(q1, pl.inv_rh), r = q1 - cg * RH;
		const int yy = rgn_y0 + r, col0 = c4 * 4 - pl.PL;
		const int yc = min(max(yy, 0), g.H - 1);
		uint32_t d[4];
		if (fast) {
			const bool inside = yy == yc && col0 >= 0 && col0 + 4 <= g.W;
			const int cc = min(max(col0, 0), g.W - 4);
#pragma unroll
			for (int c = 0; c < 4; c++) {
				const int ci = cg * 4 + c;
				const uint32_t v = *reinterpret_cast<const uint32_t*>(xn + ((int64_t)min(ci, g.Cin - 1) * g.H + yc) * g.W + cc);
				d[c] = inside && ci < g.Cin ? v : 0u;
			}
		} else {
#pragma unroll
			for (int c = 0; c < 4; c++) {
				const int ci = cg * 4 + c;
				const uint8_t* row = xn + ((int64_t)min(ci, g.Cin - 1) * g.H + yc) * g.W;
				d[c] = 0;
#pragma unroll
				for (int b = 0; b < 4; b++) {
					const int col = col0 + b;
					const uint32_t v = row[min(max(col, 0), g.W - 1)];
					d[c] |= (yy == yc && col >= 0 && col < g.W && ci < g.Cin ? v : 0u) << (8 * b);
				}
			}
		}
		// byte b of d[c] is (column b, channel c): out[b] = the four channels of column b
		const uint32_t lo01 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u), hi01 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);
		const uint32_t lo23 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u), hi23 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
		uint32_t out[4];
		out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
		out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
		out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
		out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
		uint8_t* dst = s_rgn + (r * RW + c4 * 4) * PP + cg * 4;
#pragma unroll
		for (int b = 0; b < 4; b++) *reinterpret_cast<uint32_t*>(dst + b * PP) = out[b];
	}
	// ---- unit table: a unit is CP consecutive channels of one tap; entry = its byte offset inside the region for the
	// position (hb, 0), bit 30 for units past the last tap
	for (int u = tid; u < Kp / CP; u += 256) {
		const int t = u / pl.UC, cc = u - t * pl.UC;
		const int tc = min(t, T - 1), i = tc / g.kw, j = tc - i * g.kw;
		s_unit[u] = (uint32_t)((i * RW + j + pl.PL - g.pw) * PP + cc * CP) | (t < T ? 0u : TAP_PAST_K);
	}
	// ---- weights in the order (tap, channel), into the signed domain; rows past Cout, channels past Cin and units past
	// the last tap hold signed zeros.  Three ways, by what the shape allows: permuted in registers (band_stage_weights:
	// 1 x 1, 3 x 3, 5 x 5 and 7 x 7 windows of a multiple of four channels); else, where the weight rows keep dword alignment,
	// read along memory, a dword of four consecutive (channel, tap) bytes per thread, and scattered byte by byte into
	// the new order; else a thread builds a dword of the new order from four bytes it gathers.  On 4 x 64 x 56 x 56 ->
	// 64 channels 3 x 3 the three take 3.7, 8 and 10.8 us of the kernel's time.
	const bool w_fast = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(w) & 3) == 0;
	const bool w_taps = w_fast && (g.Cin & 3) == 0 && (T == 1 || T == 9 || T == 25 || T == 49);
	if (w_taps) {
		for (int idx = tid; idx < pl.ncb * pl.wpitch; idx += 256) reinterpret_cast<v4i*>(s_w)[idx] = v4i{ 0, 0, 0, 0 };
		__syncthreads();
		if (T == 1) band_stage_weights<1>(w, s_w, cout_here, g.Cin, CPtot, pl.wpitch, tid, pl.inv_cq);  // a plain copy: one tap, the orders agree
		else if (T == 9) band_stage_weights<9>(w, s_w, cout_here, g.Cin, CPtot, pl.wpitch, tid, pl.inv_cq);
		else if (T == 25) band_stage_weights<25>(w, s_w, cout_here, g.Cin, CPtot, pl.wpitch, tid, pl.inv_cq);
		else band_stage_weights<49>(w, s_w, cout_here, g.Cin, CPtot, pl.wpitch, tid, pl.inv_cq);
	} else if (w_fast) {
		// where byte k of a weight row (l-ten's order: channel k / T, tap k % T) goes in the new order: worked out once, the
		// divisions by T for every byte had been most of the staging time
		uint16_t* const s_kmap = reinterpret_cast<uint16_t*>(smem + pl.off_kmap);
		for (int k = tid; k < K; k += 256) {
			const int ci = k / T;
			s_kmap[k] = (uint16_t)((k - ci * T) * CPtot + ci);
		}
		for (int idx = tid; idx < pl.ncb * pl.wpitch; idx += 256) reinterpret_cast<v4i*>(s_w)[idx] = v4i{ 0, 0, 0, 0 };
		__syncthreads();
		// (eight loads in flight per thread: one load, then its four byte writes, made a chain of round trips to the L2)
		const int total = cout_here * (K / 4);   // the block's weights are one run of cout_here * K bytes: dword number idx holds bytes 4 idx .. + 3
		constexpr int U = 8;
		// this thread's dwords are 256 apart: (row, byte in the row) advance by (1024 / K, 1024 % K), no division per dword
		const int step_co = 1024 / K, step_k = 1024 - step_co * K;
		int co = (4 * tid) / K, k = 4 * tid - co * K;
		for (int idx0 = tid; idx0 < total; idx0 += 256 * U) {
			uint32_t v[U];
#pragma unroll
			for (int u = 0; u < U; u++) v[u] = reinterpret_cast<const uint32_t*>(w)[min(idx0 + u * 256, total - 1)] ^ 0x80808080u;
#pragma unroll
			for (int u = 0; u < U; u++) {
				if (idx0 + u * 256 < total) {
					uint8_t* row = s_w + co * pl.wpitch;
#pragma unroll
					for (int b = 0; b < 4; b++) row[s_kmap[k + b]] = (uint8_t)(v[u] >> (8 * b));  // K % 4 == 0: the four bytes lie in one row
				}
				co += step_co;
				k += step_k;
				if (k >= K) {
					k -= K;
					co++;
				}
			}
		}
	} else {
		const int kd = Kp / 4;
		for (int idx = tid; idx < pl.ncb * 16 * kd; idx += 256) {
			const int co = idx / kd, k0 = (idx - co * kd) * 4;
			const int t = k0 / CPtot, c0 = k0 - t * CPtot;
			uint32_t v = 0;
			if (co < cout_here && t < T) {
				const uint8_t* wr = w + (int64_t)co * K + t;
#pragma unroll
				for (int b = 0; b < 4; b++) {
					const uint32_t raw = wr[min(c0 + b, g.Cin - 1) * T];
					v |= ((c0 + b < g.Cin ? raw : 0x80u) ^ 0x80u) << (8 * b);
				}
			}
			*reinterpret_cast<uint32_t*>(s_w + co * pl.wpitch + k0) = v;
		}
	}
	__syncthreads();

	const int coef_a = 128 - zp_w, coef_b = 128 - zp_in;
	const int konst = K * (zp_in * zp_w - 16384);
	const int band_pos = rows_here * g.Wo;            // positions of this band
	const int nblocks = (band_pos + 15) / 16;
	constexpr int BW = 4;                             // blocks a wavefront holds at a time
	constexpr int UPG = 16 / CP;                      // units per k-group of 16 bytes
	for (int pass0 = 0; pass0 < nblocks; pass0 += 4 * BW) {
		// this wavefront's blocks of the pass: pass0 + wave + 4 u
		int base[BW];
#pragma unroll
		for (int u = 0; u < BW; u++) {
			const int p = min((pass0 + wave + 4 * u) * 16 + lrow, band_pos - 1);  // positions past the band repeat its last one and are not stored
			const int dh = p / g.Wo, wo = p - dh * g.Wo;
			base[u] = (dh * g.sh * RW + wo * g.sw) * PP;
		}
		v4i acc[BW][4];
		uint32_t sa[BW], sw[4];
#pragma unroll
		for (int u = 0; u < BW; u++) {
			sa[u] = 0;
#pragma unroll
			for (int cb = 0; cb < 4; cb++) acc[u][cb] = v4i{ 0, 0, 0, 0 };
		}
#pragma unroll
		for (int cb = 0; cb < 4; cb++) sw[cb] = 0;
		// operands of a k-step: the weights' fragments and, per block, the 16 bytes of this lane's position and k-group.
		// The next step's are read from LDS while this step's MFMAs run (two sets of registers in turn): with two
		// wavefronts per SIMD, reading and then multiplying left the matrix pipe idle for the length of the reads.
		struct Operands {
			v4i bf[4];
			uint32_t d[BW][4];
		};
		auto read_step = [&](int ks, Operands& f) {
			uint32_t uoff[UPG];
#pragma unroll
			for (int q = 0; q < UPG; q++) uoff[q] = s_unit[(ks + lgrp * 16) / CP + q];
#pragma unroll
			for (int cb = 0; cb < 4; cb++) {
				f.bf[cb] = v4i{ 0, 0, 0, 0 };
				if (cb < pl.ncb) f.bf[cb] = *reinterpret_cast<const v4i*>(s_w + (cb * 16 + lrow) * pl.wpitch + ks + lgrp * 16);
			}
#pragma unroll
			for (int u = 0; u < BW; u++) {
#pragma unroll
				for (int q = 0; q < UPG; q++) {
					// a unit past the last tap reads the region's first bytes and counts as nothing
					const bool real = (uoff[q] & TAP_PAST_K) == 0;
					const uint8_t* src = s_rgn + (real ? uoff[q] + (uint32_t)base[u] : 0u);
					if (CP == 16) {
						const v4i v = *reinterpret_cast<const v4i*>(src);
						f.d[u][0] = real ? (uint32_t)v.x : 0u; f.d[u][1] = real ? (uint32_t)v.y : 0u;
						f.d[u][2] = real ? (uint32_t)v.z : 0u; f.d[u][3] = real ? (uint32_t)v.w : 0u;
					} else if (CP == 8) {
						const uint2 v = *reinterpret_cast<const uint2*>(src);
						f.d[u][2 * q] = real ? v.x : 0u; f.d[u][2 * q + 1] = real ? v.y : 0u;
					} else {
						const uint32_t v = *reinterpret_cast<const uint32_t*>(src);
						f.d[u][q] = real ? v : 0u;
					}
				}
			}
		};
		auto multiply = [&](const Operands& f) {
#pragma unroll
			for (int cb = 0; cb < 4; cb++) {
				if (cb < pl.ncb) {
					const v4i braw = flip_sign_bits(f.bf[cb]);  // back to l-ten's bytes for the sum (padding then holds 0x80)
#pragma unroll
					for (int q = 0; q < 4; q++) sw[cb] = __builtin_amdgcn_sad_u8((unsigned)braw[q], 0u, sw[cb]);
				}
			}
#pragma unroll
			for (int u = 0; u < BW; u++) {
				if (pass0 + wave + 4 * u >= nblocks) break;  // the same for the whole wavefront
#pragma unroll
				for (int q = 0; q < 4; q++) sa[u] = __builtin_amdgcn_sad_u8(f.d[u][q], 0u, sa[u]);
				const v4i a = flip_sign_bits(v4i{ (int)f.d[u][0], (int)f.d[u][1], (int)f.d[u][2], (int)f.d[u][3] });
#pragma unroll
				for (int cb = 0; cb < 4; cb++)
					if (cb < pl.ncb) acc[u][cb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, f.bf[cb], acc[u][cb], 0, 0, 0);
			}
		};
		Operands f0, f1;
		{
			read_step(0, f0);
			for (int ks = 0; ks < Kp; ks += 128) {
				if (ks + 64 < Kp) read_step(ks + 64, f1);
				multiply(f0);
				if (ks + 64 < Kp) {
					if (ks + 128 < Kp) read_step(ks + 128, f0);
					multiply(f1);
				}
			}
		}
		// channel sums: the four k-groups of channel 16 cb + lrow sit in lanes lrow, + 16, + 32, + 48; every byte of
		// padding in a weight row held 0x80
		int ct[4];
#pragma unroll
		for (int cb = 0; cb < 4; cb++) {
			uint32_t s4 = sw[cb];
			s4 += __shfl_xor(s4, 16, 64);
			s4 += __shfl_xor(s4, 32, 64);
			ct[cb] = coef_b * ((int)s4 - 128 * (Kp - K));
		}
#pragma unroll
		for (int u = 0; u < BW; u++) {
			const int blk = pass0 + wave + 4 * u;
			if (blk >= nblocks) break;
			uint32_t rs = sa[u];
			rs += __shfl_xor(rs, 16, 64);
			rs += __shfl_xor(rs, 32, 64);
			const int p0 = blk * 16 + lgrp * 4;  // first of this lane's four positions in the band
			int rt[4];
#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int row_sum = __shfl((int)rs, lgrp * 4 + e, 64);
				const int pos = min(hb * g.Wo + p0 + e, HW - 1);
				rt[e] = coef_a * row_sum + konst + (bias != nullptr ? bias[pos] : 0);
			}
			// the four positions are four consecutive bytes of y: one dword store where they all exist and the dword is aligned
			const bool whole = OUT != Q_OUT_ACC && p0 + 4 <= band_pos && ((HW | (hb * g.Wo)) & 3) == 0 && (reinterpret_cast<uintptr_t>(y) & 3) == 0;
#pragma unroll
			for (int cb = 0; cb < 4; cb++) {
				const int co = cb * 16 + lrow;
				if (cb >= pl.ncb || co >= cout_here) continue;
				const int64_t o = ((int64_t)n * g.Cout + co0 + co) * HW + hb * g.Wo + p0;
				if (OUT == Q_OUT_ACC) {
#pragma unroll
					for (int e = 0; e < 4; e++)
						if (p0 + e < band_pos) static_cast<int*>(y)[o + e] = acc[u][cb][e] + rt[e] + ct[cb];
				} else {
					uint32_t word = 0;
#pragma unroll
					for (int e = 0; e < 4; e++) word |= (requant<OUT>(acc[u][cb][e] + rt[e] + ct[cb], mult, zp_out) & 0xFFu) << (8 * e);
					if (whole) *reinterpret_cast<uint32_t*>(static_cast<uint8_t*>(y) + o) = word;
					else {
#pragma unroll
						for (int e = 0; e < 4; e++)
							if (p0 + e < band_pos) static_cast<uint8_t*>(y)[o + e] = (uint8_t)(word >> (8 * e));
					}
				}
			}
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

// The band kernel's plan: blocks of 64 output channels per workgroup (32 or 16 where the weights of 64 would not leave
// room for one window's height of input rows), the tallest band whose region fits 64 KB of LDS beside the weights
// and the tables, shortened while that leaves the chip with fewer than two workgroups per CU.
static bool band_plan(const ConvGeo& g, BandPlan& pl)
{
	const int64_t T = (int64_t)g.kh * g.kw, K = (int64_t)g.Cin * T;
	if (g.pw > 64 || g.Cin > 1024 || g.Cout > 16 * 65535) return false;
	pl.CP = g.Cin <= 4 ? 4 : g.Cin <= 8 ? 8 : 16;
	pl.CPtot = (g.Cin + pl.CP - 1) / pl.CP * pl.CP;
	pl.PP = pl.CPtot + (pl.CPtot % 32 == 0 ? 16 : 0);  // pixels 32 or 64 bytes apart would meet on the same LDS banks
	pl.UC = pl.CPtot / pl.CP;
	const int64_t kprime = T * pl.CPtot;
	if (kprime > 4096) return false;
	pl.Kp = (int)((kprime + 63) & ~63ll);
	pl.wpitch = pl.Kp + CQI_PAD;
	pl.PL = (g.pw + 3) & ~3;
	// the rightmost byte a window reaches is column (Wo - 1) sw + kw - 1 - pw of the image
	const int reach = (g.Wo - 1) * g.sw + g.kw - g.pw;   // image columns 0 .. reach - 1 (beyond W: padding)
	pl.RW = (pl.PL + (reach > g.W ? reach : g.W) + 3) & ~3;
	const int all_cb = (g.Cout + 15) / 16;
	int tb = 0;
	int64_t fixed = 0;
	for (int ncb = all_cb < 4 ? all_cb : 4; ncb >= 1 && tb == 0; ncb = ncb == 3 ? 2 : ncb / 2) {
		pl.ncb = ncb;
		fixed = (int64_t)ncb * 16 * pl.wpitch + (int64_t)(pl.Kp / pl.CP) * 4 + 2 * K + 32;
		for (int t = 1; t <= g.Ho && t <= 64; t++) {
			const int64_t rh = (int64_t)(t - 1) * g.sh + g.kh;
			if (rh * pl.RW * pl.PP + fixed > 64 * 1024) break;
			tb = t;
		}
	}
	if (tb == 0) return false;
	// 16 channels per workgroup against many blocks of them: every block stages the region again and an operand read
	// from it feeds one MFMA; the patch-row route with its GEMM is level there (8 x 256 x 14 x 14 -> 256 channels: 42 us
	// both ways) and ahead beyond
	if (pl.ncb == 1 && all_cb > 2) return false;
	const int64_t cblocks = (all_cb + pl.ncb - 1) / pl.ncb;
	while (tb > 1 && (int64_t)g.N * ((g.Ho + tb - 1) / tb) * cblocks < 512) tb--;
	pl.TB = tb;
	pl.RH = (tb - 1) * g.sh + g.kh;
	pl.inv_rw4 = small_div_inverse((unsigned)pl.RW / 4);
	pl.inv_rh = small_div_inverse((unsigned)pl.RH);
	pl.inv_cq = small_div_inverse((unsigned)g.Cin / 4);
	pl.off_w = (unsigned)((pl.RH * pl.RW * pl.PP + 15) & ~15);
	pl.off_unit = pl.off_w + (unsigned)(pl.ncb * 16 * pl.wpitch);
	pl.off_kmap = pl.off_unit + (unsigned)(pl.Kp / pl.CP) * 4;
	pl.bytes = pl.off_kmap + (unsigned)((2 * K + 15) & ~15ll);
	return (int64_t)g.N * ((g.Ho + tb - 1) / tb) < (1ll << 31);
}

// What the band kernel is expected to take, in us (negative: no plan for the shape).  Its workgroups stage their rows of
// the input and their block of the weights before every band, and that staging is where the time goes: the bytes all
// workgroups stage, at the 1.3 TB/s measured over shapes from 30 to 190 MB of it (32 x 64 x 56 x 56 -> 64 channels 3 x 3:
// 38 MB, 29 us; 32 x 1024 x 14 x 14 -> 256 channels 1 x 1, one output row and 32 channels per workgroup: 186 MB, 132 us).
double conv2dq_band_estimate_us(const ConvGeo& g)
{
	BandPlan pl;
	if (!band_plan(g, pl)) return -1.0;
	const double wgs = (double)g.N * ((g.Ho + pl.TB - 1) / pl.TB) * ((((g.Cout + 15) / 16) + pl.ncb - 1) / pl.ncb);
	return wgs * ((double)pl.RH * pl.RW * pl.PP + (double)pl.ncb * 16 * pl.wpitch) / 1.3e6;
}

// 0 = launched; -1 = not a shape for this route
int conv2dq_band_dispatch(const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in, int zp_w, float mult,
                          float zp_out, void* y, bool out_acc)
{
	BandPlan pl;
	if (!band_plan(g, pl)) return -1;
	const int per_image = (g.Ho + pl.TB - 1) / pl.TB;
	const int all_cb = (g.Cout + 15) / 16;
	const dim3 grid((unsigned)(g.N * per_image), (unsigned)((all_cb + pl.ncb - 1) / pl.ncb));
	set_kernel_name("conv2dq_band");
	const int out = out_acc ? Q_OUT_ACC : (mult == mult && (mult < 0 ? -mult : mult) <= 0.99f) ? Q_OUT_U8_FAST : Q_OUT_U8_EXACT;
#define LTEN_LAUNCH(OUTV, CPV) conv2dq_band_kernel<OUTV, CPV><<<grid, dim3(256), pl.bytes, stream()>>>(g, x, w, bias, zp_in, zp_w, mult, zp_out, y, pl, per_image)
#define LTEN_LAUNCH_CP(OUTV)                                  \
	if (pl.CP == 16) LTEN_LAUNCH(OUTV, 16);                   \
	else if (pl.CP == 8) LTEN_LAUNCH(OUTV, 8);                \
	else LTEN_LAUNCH(OUTV, 4);
	if (out == Q_OUT_ACC) { LTEN_LAUNCH_CP(Q_OUT_ACC) }
	else if (out == Q_OUT_U8_FAST) { LTEN_LAUNCH_CP(Q_OUT_U8_FAST) }
	else { LTEN_LAUNCH_CP(Q_OUT_U8_EXACT) }
#undef LTEN_LAUNCH_CP
#undef LTEN_LAUNCH
	LTEN_HIP_LAUNCH_CHECK();
	return 0;
}

// 0 = launched; -1 = not a shape for this route
int conv2dq_image_dispatch(const ConvGeo& g, const uint8_t* x, const uint8_t* w, const int32_t* bias, int zp_in, int zp_w, float mult,
                           float zp_out, void* y, bool out_acc)
{
	ImagePlan pl;
	if (!image_plan(g, pl)) return -1;
	// The band kernel, where it applies, is ahead whenever it can permute the weights in registers (1 x 1, 3 x 3, 5 x 5 or
	// 7 x 7 windows of a multiple of four channels: 16 x 64 x 14 x 14 -> 64 channels 3 x 3 takes 19.4 us here and 10.0 there,
	// 1 x 16 x 32 x 32 -> 32 7.0 and 5.4) and otherwise once the workgroups of this kernel, each of which stages the
	// image and all weights again, would stage more than 16 MB in all (l-ten's quantized MNIST conv2, 10 channels and
	// 5 x 5: 5.5 us here and 9.7 there for one image, 9.5 and 11.7 for 256, 9.4 MB staged; 512 images go there, 11.6 us)
	const int64_t staged = (int64_t)g.N * ((g.Ho * g.Wo + CQI_POS - 1) / CQI_POS) * ((int64_t)pl.img16 + (int64_t)pl.ncb * 16 * pl.Kp);
	const int taps = g.kh * g.kw;
	const bool permuted = (g.Cin & 3) == 0 && (taps == 1 || taps == 9 || taps == 25 || taps == 49) && (reinterpret_cast<uintptr_t>(w) & 3) == 0;
	BandPlan other;
	if ((permuted || staged > (16ll << 20)) && band_plan(g, other)) return -1;
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
